"""Shared helpers of the GPU parity tests: seeded inputs and the tolerance check.

Bars.  Bucket ids, permutations and gathers are compared bit for bit elsewhere.  Attention outputs and
log-sum-exps are held to 2e-3 (norm-wise, and element-wise up to the rounding of the output type) against
the float64 oracle: that is the stated tolerance, and fp16 outputs and every log-sum-exp meet it.

bf16 outputs cannot: the reference's own arithmetic (P rounded to bf16 before P.V, the output stored in
bf16) sits 2.3e-3 from the exact result on N(0,1) data, two faithful implementations of that arithmetic
that differ only in the exponent their P is scaled by sit 3.1e-3 from each other, and the reference's
PyTorch path (scores, soft-max and output all rounded to bf16) 4.4e-3 from the exact result and 5e-3 from
its own kernels (tests/test_oracle.py::test_bf16_arithmetic_floor measures all of these on the CPU).
A bf16 result is therefore held to
  - the distance from the exact result of the SAME computation done by the oracle in the reference's
    arithmetic (``reference_arithmetic=``, oracle functions called with round_dtype=torch.bfloat16), times
    1.05, or 2e-3 if that is larger: the HIP result must be as close to the exact one as the reference's
    kernels are; and, where a test has no such result at hand,
  - 3e-3 against the float64 oracle.
"""
import torch

REL = 2e-3
REL_BY_DTYPE = {torch.float16: 2e-3, torch.bfloat16: 3e-3, torch.float32: 2e-3, None: 2e-3}


def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _randn(shape, seed, dtype):
    return torch.randn(shape, generator=_gen(seed)).to(dtype)


def rel_err(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return ((a - b).norm() / b.norm().clamp(min=1e-30)).item()


def assert_close(got, ref, what, out_dtype=None, reference_arithmetic=None):
    got = got.detach().double().cpu()
    ref = ref.detach().double().cpu()
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    tol = REL_BY_DTYPE[out_dtype]
    if reference_arithmetic is not None:
        floor = rel_err(reference_arithmetic, ref)
        tol = max(REL, 1.05 * floor)
    rel = (got - ref).norm() / ref.norm().clamp(min=1e-30)
    assert rel <= tol, f"{what}: norm-wise relative error {rel:.3e} > {tol:.3e}"
    ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7, None: 0.0, torch.float32: 0.0}[out_dtype]
    bound = max(tol, REL_BY_DTYPE[out_dtype]) * ref.abs().max() + ulp * ref.abs()
    worst = ((got - ref).abs() - bound).max()
    assert worst <= 0, f"{what}: element-wise error exceeds bound by {worst:.3e}"
