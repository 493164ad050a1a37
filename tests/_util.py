"""Shared helpers of the GPU parity tests: seeded inputs and the tolerance check."""
import torch

REL = 2e-3
REL_BY_DTYPE = {torch.float16: 2e-3, torch.bfloat16: 3e-3, torch.float32: 2e-3, None: 2e-3}


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _randn(shape, seed, dtype):
    return torch.randn(shape, generator=_gen(seed)).to(dtype)


def assert_close(got, ref, what, out_dtype=None):
    got = got.detach().double().cpu()
    ref = ref.detach().double().cpu()
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    tol = REL_BY_DTYPE[out_dtype]
    rel = (got - ref).norm() / ref.norm().clamp(min=1e-30)
    assert rel <= tol, f"{what}: norm-wise relative error {rel:.3e} > {tol}"
    ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7, None: 0.0, torch.float32: 0.0}[out_dtype]
    bound = tol * ref.abs().max() + ulp * ref.abs()
    worst = ((got - ref).abs() - bound).max()
    assert worst <= 0, f"{what}: element-wise error exceeds bound by {worst:.3e}"
