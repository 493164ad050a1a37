"""GPU parity tests of the individual operators (through the C ABI) against the CPU oracle.

Tolerances.  Bucket ids, permutations and gathers are compared bit for bit.  Attention outputs and
log-sum-exps (fp32) are compared with the oracle evaluated in float64 on the same fp16/bf16 inputs:
norm-wise  ||x - ref|| <= tol ||ref||  per tensor, and element-wise
|x - ref| <= tol * max(|ref|) + one unit in the last place of the output type.
tol = 2e-3 for fp16 outputs and for every log-sum-exp.  For bf16 outputs tol = 3e-3: the reference's
own arithmetic (P rounded to bf16 before P.V, src/hyper_attn_triton.py:135, and the output stored in
bf16, both round-to-nearest) is 2.3e-3 away from float64 on N(0,1) inputs, 1.7e-3 of it from storing
the output alone, so no bf16 implementation can sit inside 2e-3 of a float64 oracle.
"""
import math

import numpy as np
import pytest
import torch

from oracle import hyper_oracle as O

pytestmark = pytest.mark.gpu

from _util import _gen, _randn, assert_close


@pytest.fixture(scope="module")
def ha():
    import hyperattention_amd
    from hyperattention_amd import _lib
    _lib.lib()  # fails loudly when the HIP library is missing
    return hyperattention_amd


# ------------------------------------------------------------------------------------- hash
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("b,h,n,d,r", [(1, 2, 2048, 64, 8), (2, 3, 1000, 128, 8), (1, 1, 777, 64, 5),
                                       (1, 2, 513, 32, 12), (1, 1, 300, 256, 16),
                                       # rows shorter than the width the kernel is built for
                                       (1, 2, 700, 96, 8), (2, 1, 300, 40, 7), (1, 1, 515, 8, 3), (1, 1, 257, 200, 9)])
def test_hash_bit_exact(ha, dtype, b, h, n, d, r):
    x = _randn((b, h, n, d), 1, dtype)
    proj = _randn((1, 1, d, r), 2, dtype)
    want = O.lsh_hash(x, proj[0, 0])
    got = ha.lsh_hash(x.cuda(), proj.cuda())
    assert got.dtype == torch.int32 and got.shape == (b, h, n)
    assert np.array_equal(got.cpu().numpy(), want)


def test_hash_reference_test_shape(ha):
    # unit_tests/test_lsh.py:25-31: fp16, (4, 32, 2048, 128), 8 projections
    x = _randn((4, 32, 2048, 128), 3, torch.float16)
    lsh = ha.AngularLSH(num_projs=8, dim=(1, 1, 128), rng=_gen(4)).to(device="cuda", dtype=torch.float16)
    got = lsh.hash_triton(x.cuda())
    want = O.lsh_hash(x, lsh.proj_dir[0, 0].cpu())
    assert np.array_equal(got.cpu().numpy(), want)


def test_hash_per_head_projection_strided_and_special_rows(ha):
    b, h, n, d, r = 2, 2, 300, 64, 8
    big = _randn((b, n, h, d), 5, torch.float16)
    x = big.transpose(1, 2)  # (b,h,n,d) view with a non-trivial row stride
    x[0, 0, 7] = 0  # zero row -> bucket 0
    x[1, 1, 9] = -x[1, 1, 8]
    proj = _randn((b, h, d, r), 6, torch.float16)
    want = O.lsh_hash(x, proj)
    got = ha.lsh_hash(big.cuda().transpose(1, 2), proj.cuda())
    assert np.array_equal(got.cpu().numpy(), want)
    assert got[0, 0, 7].item() == 0


def test_hash_golden_vectors(ha):
    data = np.load(__file__.rsplit("/", 1)[0] + "/golden/lsh_hash_fp16.npz")
    x = torch.from_numpy(data["x"]).view(torch.float16)
    proj = torch.from_numpy(data["proj"]).view(torch.float16)
    got = ha.lsh_hash(x.cuda(), proj.cuda().view(1, 1, *proj.shape))
    assert np.array_equal(got.cpu().numpy(), data["buckets"])


# ------------------------------------------------------------------------------------- sort
@pytest.mark.parametrize("segs,n,num_keys,kind", [
    (6, 100, 256, "uniform"), (4, 2048, 256, "uniform"), (3, 4096, 256, "skew"), (2, 5000, 64, "uniform"),
    (64, 32768, 256, "uniform"), (2, 65536 + 17, 256, "skew"), (3, 4097, 256, "same"), (2, 3000, 4096, "uniform"),
    (1, 20000, 65536, "uniform"),
    # 64 chunks per segment: every scatter workgroup adds up its segment's histograms; 65: the scan launch does
    (2, 64 * 4096, 256, "uniform"), (1, 64 * 4096 + 5, 256, "skew"), (1, 300000, 4096, "uniform"),
    # beyond 2^24 keys per segment a row number no longer fits beside its digit in the word a chunk is staged
    # in: the scatter writes each row where it belongs instead
    (1, (1 << 24) + 3, 256, "uniform"),
])
def test_sort_bit_exact(ha, segs, n, num_keys, kind):
    g = np.random.default_rng(7)
    if kind == "uniform":
        keys = g.integers(0, num_keys, size=(1, segs, n))
    elif kind == "skew":
        keys = np.minimum(g.geometric(0.05, size=(1, segs, n)) - 1, num_keys - 1)
        keys[0, 0, : n // 2] = num_keys - 1
    else:
        keys = np.full((1, segs, n), 3)
    keys = keys.astype(np.int32)
    want = O.stable_bucket_argsort(keys)
    for out_dtype in (torch.int64, torch.int32):
        got = ha.bucket_argsort(torch.from_numpy(keys).cuda(), num_keys, out_dtype)
        assert got.dtype == out_dtype
        assert np.array_equal(got.cpu().numpy().astype(np.int64), want)


def test_sort_matches_torch_sort_on_device(ha):
    keys = torch.randint(0, 256, (2, 8, 8192), generator=_gen(8), dtype=torch.int32).cuda()
    got = ha.bucket_argsort(keys)
    want = torch.sort(keys, dim=2, stable=True)[1]
    assert torch.equal(got, want)


# ----------------------------------------------------------------------------------- gather
@pytest.mark.parametrize("dtype,d", [(torch.float16, 64), (torch.bfloat16, 128), (torch.float32, 16)])
def test_gather_rows(ha, dtype, d):
    x = _randn((2, 3, 500, d), 9, dtype)
    idx = torch.randint(0, 500, (2, 3, 300), generator=_gen(10))
    got = ha.indexing(x.cuda(), idx.cuda())
    assert torch.equal(got.cpu(), O.gather_rows(x, idx))
    padded = ha.indexing(x.cuda(), idx.cuda().int(), chunk_size=128)  # 500 % 128 != 0 -> rows 300 -> 384
    want = O.gather_rows(x, idx, 128)
    assert padded.shape == want.shape and torch.equal(padded.cpu(), want)


def _reference_arithmetic(dtype, oracle_call):
    """The oracle's result in the reference's own arithmetic for a bf16 case (None otherwise): what a bf16
    output is measured against, see _util."""
    if dtype != torch.bfloat16:
        return None
    return oracle_call(round_dtype=torch.bfloat16)[0]


# ------------------------------------------------------------------------------------ flash
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("b,h,n,d", [(1, 2, 2048, 64), (2, 2, 1000, 128), (1, 3, 200, 64), (1, 1, 1, 64), (1, 2, 321, 128)])
def test_flash_attention(ha, dtype, causal, b, h, n, d):
    q, k, v = (_randn((b, n, h, d), s, dtype) for s in (11, 12, 13))
    o, lse = ha.flash_attn_func(q.cuda(), k.cuda(), v.cuda(), None, causal, None)
    assert o.shape == (b, n, h, d) and o.dtype == dtype
    assert lse.shape == (b, h, math.ceil(n / 128) * 128) and lse.dtype == torch.float32
    ro, rl = O.exact_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), None, causal)
    assert_close(o.transpose(1, 2), ro, "flash out", dtype, _reference_arithmetic(
        dtype, lambda **kw: O.exact_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), None, causal, **kw)))
    assert_close(lse[:, :, :n], rl, "flash lse")


def test_flash_attention_different_lengths_and_scale(ha):
    q = _randn((1, 300, 2, 64), 14, torch.float16)
    k, v = (_randn((1, 700, 2, 64), s, torch.float16) for s in (15, 16))
    o, lse = ha.flash_attn_func(q.cuda(), k.cuda(), v.cuda(), None, False, 0.2)
    ro, rl = O.exact_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), 0.2, False)
    assert_close(o.transpose(1, 2), ro, "flash out", torch.float16)
    assert_close(lse[:, :, :300], rl, "flash lse")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("causal", [False, True])
def test_flash_attention_wide_logit_range(ha, dtype, causal):
    """Scores spanning ~100 log2 units whose row maxima keep growing along the key sequence: the
    kernel's reference exponent has to be raised again and again (its rare path), late keys dominate."""
    b, h, n, d = 1, 2, 1536, 64
    q, k, v = (_randn((b, n, h, d), s, dtype) for s in (61, 62, 63))
    direction = torch.nn.functional.normalize(_randn((d,), 64, torch.float32), dim=0)
    ramp = torch.linspace(-4.0, 4.0, n).view(1, n, 1, 1)           # keys drift along `direction`
    k = (k.float() + ramp * direction * 16.0).to(dtype)
    q = (q.float() * 0.5 + direction * 4.0 * torch.sign(_randn((b, n, h, 1), 65, torch.float32))).to(dtype)
    o, lse = ha.flash_attn_func(q.cuda(), k.cuda(), v.cuda(), None, causal, None)
    ro, rl = O.exact_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), None, causal)
    spread = (q.float().transpose(1, 2) @ k.float().transpose(1, 2).transpose(-1, -2) / 8.0)
    assert (spread.max() - spread.min()) * 1.4427 > 60, "the case must span many powers of two"
    assert_close(o.transpose(1, 2), ro, "flash out", dtype, _reference_arithmetic(
        dtype, lambda **kw: O.exact_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), None, causal, **kw)))
    assert_close(lse[:, :, :n], rl, "flash lse")


@pytest.mark.parametrize("d", [32, 96, 40])
def test_flash_attention_other_head_dims(ha, d):
    """Head dims other than the built 64 / 128 (the reference takes any d <= 128,
    src/flash_attn_triton.py:801) run zero-padded; the default scale is that of the original d."""
    b, h, n = 1, 2, 640
    q, k, v = (_randn((b, n, h, d), s, torch.float16) for s in (66, 67, 68))
    o, lse = ha.flash_attn_func(q.cuda(), k.cuda(), v.cuda(), None, True, None)
    assert o.shape == (b, n, h, d)
    ro, rl = O.exact_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), None, True)
    assert_close(o.transpose(1, 2), ro, "flash out", torch.float16)
    assert_close(lse[:, :, :n], rl, "flash lse")


def test_flash_rejects_bias_and_bad_types(ha):
    q = torch.zeros((1, 128, 1, 64), dtype=torch.float16, device="cuda")
    with pytest.raises(NotImplementedError):
        ha.flash_attn_func(q, q, q, torch.zeros(1, 1, 1, 128, device="cuda"))
    with pytest.raises(AssertionError):
        ha.flash_attn_func(q.float(), q.float(), q.float())
    with pytest.raises(AssertionError):
        ha.flash_attn_func(q.cpu(), q.cpu(), q.cpu())


# --------------------------------------------------------------- block + sampled attention
def _sorted_inputs(b, h, n, d, dtype, seed, nbuckets=64):
    q, k, v = (_randn((b, h, n, d), seed + i, dtype) for i in range(3))
    g = _gen(seed + 3)
    qb = torch.randint(0, nbuckets, (b, h, n), generator=g)
    kb = torch.randint(0, nbuckets, (b, h, n), generator=g)
    qi = torch.sort(qb, dim=2, stable=True)[1]
    ki = torch.sort(kb, dim=2, stable=True)[1]
    return q, k, v, qi, ki


def _run_hyper(ha, q, k, v, qi, ki, block, sample, scale, smooth, sampled_idx=None, idx_dtype=torch.int64):
    c = lambda t: t.cuda()
    o, lse = ha.hyper_attn_func(c(q).transpose(1, 2), c(k).transpose(1, 2), c(v).transpose(1, 2),
                                c(qi).to(idx_dtype).transpose(1, 2), c(ki).to(idx_dtype).transpose(1, 2),
                                block, sample, scale, smooth,
                                sampled_idx=None if sampled_idx is None else c(sampled_idx))
    return o.transpose(1, 2), lse


@pytest.mark.parametrize("dtype,d,block,sample", [
    (torch.bfloat16, 128, 512, 128),   # unit_tests/test_hyper_attention.py:31-37 (batch, heads reduced)
    (torch.bfloat16, 64, 256, 128),    # unit_tests/test_hyper_attention.py:139-146
    (torch.float16, 64, 256, 256),
    (torch.float16, 128, 128, 0),
    (torch.float16, 64, 384, 128),
])
@pytest.mark.parametrize("smooth", [False, True])
def test_block_sampled_attention(ha, dtype, d, block, sample, smooth):
    b, h, n = 1, 2, 2048
    q, k, v, qi, ki = _sorted_inputs(b, h, n, d, dtype, 20)
    k[:, :, :128] *= 4.0  # unit_tests/test_hyper_attention.py:43: makes the sampled columns matter
    o, lse = _run_hyper(ha, q, k, v, qi, ki, block, sample, None, smooth)
    assert o.shape == (b, h, n, d) and o.dtype == dtype and lse.shape == (b, h, n) and lse.dtype == torch.float32
    ro, rl = O.block_sampled_attention(q, k, v, qi, ki, block, sample, None, smooth)
    assert_close(o, ro, "hyper out", dtype, _reference_arithmetic(
        dtype, lambda **kw: O.block_sampled_attention(q, k, v, qi, ki, block, sample, None, smooth, **kw)))
    assert_close(lse, rl, "hyper lse")


def test_block_sampled_explicit_samples_int32_idx_and_ragged_tail(ha):
    # n = 1920 is a multiple of 128 but not of 256 (half-filled last workgroup) nor of the block size
    b, h, n, d = 2, 2, 1920, 64
    q, k, v, qi, ki = _sorted_inputs(b, h, n, d, torch.float16, 30)
    sampled = torch.randint(0, n, (256,), generator=_gen(31))
    for smooth in (False, True):
        o, lse = _run_hyper(ha, q, k, v, qi, ki, 512, 256, 0.11, smooth, sampled, torch.int32)
        ro, rl = O.block_sampled_attention(q, k, v, qi, ki, 512, 256, 0.11, smooth, sampled)
        assert_close(o, ro, "hyper out", torch.float16)
        assert_close(lse, rl, "hyper lse")


@pytest.mark.parametrize("per_batch", [False, True])
def test_block_sampled_one_sample_list_per_head(ha, per_batch):
    """A different explicit sample list for every head (and batch entry): checked head by head against the
    oracle, which takes one list."""
    b, h, n, d = 2, 3, 1024, 64
    q, k, v, qi, ki = _sorted_inputs(b, h, n, d, torch.bfloat16, 35)
    sampled = torch.randint(0, n, (b, h, 128), generator=_gen(36))
    if not per_batch:
        sampled = sampled[0]
    o, lse = _run_hyper(ha, q, k, v, qi, ki, 256, 128, None, False, sampled, torch.int32)
    for bi in range(b):
        for hi in range(h):
            sl = (slice(bi, bi + 1), slice(hi, hi + 1))
            s_list = sampled[bi, hi] if per_batch else sampled[hi]
            ro, rl = O.block_sampled_attention(q[sl], k[sl], v[sl], qi[sl], ki[sl], 256, 128, None, False, s_list)
            assert_close(o[sl], ro, f"hyper out b{bi} h{hi}", torch.bfloat16, _reference_arithmetic(
                torch.bfloat16, lambda **kw: O.block_sampled_attention(q[sl], k[sl], v[sl], qi[sl], ki[sl], 256, 128, None,
                                                                        False, s_list, **kw)))
            assert_close(lse[sl], rl, f"hyper lse b{bi} h{hi}")


@pytest.mark.parametrize("n,block", [(128, 512), (256, 1024), (384, 512)])
def test_block_attention_smooth_block_longer_than_sequence(ha, n, block):
    """smooth_block with a block much longer than the sequence: the window offset
    (src/hyper_attn_triton.py:101,105-106) is negative before the modulo; every key is visited once."""
    q, k, v, qi, ki = _sorted_inputs(1, 2, n, 64, torch.float16, 90)
    o, lse = _run_hyper(ha, q, k, v, qi, ki, block, 0, None, True, idx_dtype=torch.int32)
    ro, rl = O.block_sampled_attention(q, k, v, qi, ki, block, 0, None, True)
    assert_close(o, ro, "hyper out", torch.float16)
    assert_close(lse, rl, "hyper lse")


def test_block_attention_full_block_is_exact_attention(ha):
    b, h, n, d = 1, 2, 512, 64
    q, k, v, qi, ki = _sorted_inputs(b, h, n, d, torch.float16, 40)
    o, lse = _run_hyper(ha, q, k, v, qi, ki, n, 0, None, False)
    ro, rl = O.exact_attention(q, k, v)
    assert_close(o, ro, "hyper out", torch.float16)
    assert_close(lse, rl, "hyper lse")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shift", [-30.0, 0.0, 30.0])
def test_block_attention_resumes_partial_result(ha, dtype, shift):
    """resume=(o, lse): the kernel continues a partial attention over other keys (add_self_attentions,
    src/attn_utils.py:6-50, folded into the kernel).  `shift` moves the previous part's scores far below
    / above the new ones; some rows have an empty previous part (lse = -inf)."""
    b, h, n, d = 1, 2, 512, 64
    q, k, v, qi, ki = _sorted_inputs(b, h, n, d, dtype, 70)
    k_prev, v_prev = (_randn((b, h, 256, d), s, dtype) for s in (74, 75))
    scale = d ** -0.5
    s_prev = q.double() @ k_prev.double().transpose(-1, -2) * scale + shift
    s_new = q.double() @ k.double().transpose(-1, -2) * scale
    l_prev = torch.logsumexp(s_prev, dim=-1)
    o_prev = torch.softmax(s_prev, dim=-1) @ v_prev.double()
    l_prev[:, :, ::7] = float("-inf")          # rows without a previous part
    o_prev[:, :, ::7] = 0.0
    o_dev = o_prev.to(dtype).cuda().transpose(1, 2).contiguous()       # (b, n, h, d)
    l_dev = l_prev.float().cuda().contiguous()
    c = lambda t: t.cuda()
    o, lse = ha.hyper_attn_func(c(q).transpose(1, 2), c(k).transpose(1, 2), c(v).transpose(1, 2),
                                c(qi).transpose(1, 2), c(ki).transpose(1, 2), n, 0, None, False,
                                resume=(o_dev, l_dev))
    assert o.data_ptr() == o_dev.data_ptr() and lse.data_ptr() == l_dev.data_ptr()
    # expected: exact attention over the union, the previous part entering through its ROUNDED rows
    w_prev = torch.exp(l_prev.float().double() - torch.logaddexp(l_prev.float().double(), torch.logsumexp(s_new, -1)))
    want = w_prev.unsqueeze(-1) * o_prev.to(dtype).double() + (1 - w_prev).unsqueeze(-1) * (torch.softmax(s_new, -1) @ v.double())
    want_lse = torch.logaddexp(l_prev.float().double(), torch.logsumexp(s_new, -1))
    assert_close(o.transpose(1, 2), want, "resumed out", dtype)
    assert_close(lse, want_lse, "resumed lse")


@pytest.mark.parametrize("run", [2, 3, 8])
@pytest.mark.parametrize("dtype,d,block,sample,smooth,resume", [
    (torch.bfloat16, 128, 256, 256, False, True),    # the shape the library streams by default (plain, d = 128)
    (torch.bfloat16, 128, 256, 128, True, False),    # smooth windows: the general instance
    (torch.float16, 64, 256, 128, False, True),
    (torch.float16, 64, 128, 256, False, False),     # one 128-key block per 128 queries
    (torch.float16, 128, 384, 0, True, True),        # no samples, a block that is not a power of two
])
def test_streaming_kernel_equals_the_one_tile_kernel(ha, monkeypatch, run, dtype, d, block, sample, smooth, resume):
    """A workgroup that takes a run of query tiles (the library's choice for large d = 128 launches; forced here
    by the library's measurement switch) computes bit for bit what one workgroup per tile computes: output and
    log-sum-exp, with and without a partial result to resume, whole runs and a last run that is shorter."""
    b, h, n = 1, 2, 2304                       # 9 tiles of 256: runs of 2, 3 and 8 all leave a shorter last run or none
    q, k, v, qi, ki = _sorted_inputs(b, h, n, d, dtype, 90)
    c = lambda t: t.cuda()

    def call(tiles):
        monkeypatch.setenv("HA_STREAM_TILES", str(tiles))
        kw = {}
        if resume:
            g = _gen(95)
            o_prev = torch.randn((b, n, h, d), generator=g).to(dtype).cuda()
            l_prev = torch.randn((b, h, n), generator=g).cuda()
            l_prev[:, :, ::5] = float("-inf")
            o_prev[:, ::5] = 0
            kw["resume"] = (o_prev, l_prev)
        o, lse = ha.hyper_attn_func(c(q).transpose(1, 2), c(k).transpose(1, 2), c(v).transpose(1, 2),
                                    c(qi).transpose(1, 2), c(ki).transpose(1, 2), block, sample, None, smooth, **kw)
        torch.cuda.synchronize()
        return o.clone(), lse.clone()

    o1, l1 = call(1)
    o2, l2 = call(run)
    assert torch.isfinite(o1.float()).all()
    assert torch.equal(o1, o2), f"out differs, max {float((o1.float() - o2.float()).abs().max()):.3e}"
    assert torch.equal(l1, l2), f"lse differs, max {float((l1 - l2).abs().max()):.3e}"


@pytest.mark.parametrize("dtype,d,smooth,block,per_head", [
    (torch.float16, 64, False, 256, False),
    (torch.bfloat16, 128, True, 256, True),
    (torch.float16, 64, True, 128, False),
])
def test_residual_estimator_option(ha, dtype, d, smooth, block, per_head):
    """sample_bias + mask_sampled_in_block (the HyperAttention paper's residual estimator; not in the reference)
    against the oracle option, which tests/test_oracle.py pins by the per-row definition.  The sample list
    has repeats and entries inside and outside every tile's key window."""
    b, h, n, samples = 2, 2, 1024, 128
    q, k, v, qi, ki = _sorted_inputs(b, h, n, d, dtype, 90)
    g = _gen(91)
    sampled = torch.randint(0, n, (h, samples) if per_head else (samples,), generator=g)
    bias = float(np.log(n / samples))
    kw = dict(sampled_idx=sampled.cuda(), sample_bias=bias, mask_sampled_in_block=True)
    o, lse = ha.hyper_attn_func(q.transpose(1, 2).cuda(), k.transpose(1, 2).cuda(), v.transpose(1, 2).cuda(),
                                qi.transpose(1, 2).cuda(), ki.transpose(1, 2).cuda(), block, samples, None, smooth, **kw)
    s_full = sampled.view(1, h, samples).expand(b, h, samples) if per_head else sampled
    ro, rl = O.block_sampled_attention(q, k, v, qi, ki, block, samples, None, smooth, s_full, sample_bias=bias,
                                       mask_sampled_in_block=True)
    # (bf16: the secondary bar of _util; the option has no reference arithmetic to be measured against)
    assert_close(o.transpose(1, 2), ro, "estimator out", dtype)
    assert_close(lse, rl, "estimator lse")
    # the option changes the result (the plain operator counts the samples un-weighted and twice)
    plain, _ = ha.hyper_attn_func(q.transpose(1, 2).cuda(), k.transpose(1, 2).cuda(), v.transpose(1, 2).cuda(),
                                  qi.transpose(1, 2).cuda(), ki.transpose(1, 2).cuda(), block, samples, None, smooth,
                                  sampled_idx=sampled.cuda())
    assert float((plain.float() - o.float()).abs().max()) > 1e-3
    # default sample list (rows 0 .. samples-1) with the mask, bias alone, and the error paths
    o2, lse2 = ha.hyper_attn_func(q.transpose(1, 2).cuda(), k.transpose(1, 2).cuda(), v.transpose(1, 2).cuda(),
                                  qi.transpose(1, 2).cuda(), ki.transpose(1, 2).cuda(), block, samples, None, smooth,
                                  mask_sampled_in_block=True)
    ro2, rl2 = O.block_sampled_attention(q, k, v, qi, ki, block, samples, None, smooth, None, mask_sampled_in_block=True)
    assert_close(lse2, rl2, "default samples, masked: lse")
    o3, lse3 = ha.hyper_attn_func(q.transpose(1, 2).cuda(), k.transpose(1, 2).cuda(), v.transpose(1, 2).cuda(),
                                  qi.transpose(1, 2).cuda(), ki.transpose(1, 2).cuda(), block, samples, None, smooth,
                                  sample_bias=bias)
    ro3, rl3 = O.block_sampled_attention(q, k, v, qi, ki, block, samples, None, smooth, None, sample_bias=bias)
    assert_close(lse3, rl3, "bias alone: lse")
    with pytest.raises(NotImplementedError):
        ha.hyper_attn_func(q.transpose(1, 2).cuda().requires_grad_(), k.transpose(1, 2).cuda(), v.transpose(1, 2).cuda(),
                           qi.transpose(1, 2).cuda(), ki.transpose(1, 2).cuda(), block, samples, None, smooth, sample_bias=bias)


@pytest.mark.parametrize("smooth", [False, True])
def test_operators_take_grouped_query_heads(ha, smooth):
    """Fewer k/v heads than q heads (not in the reference, which wants them equal): the same bits as with the
    k/v heads, their sort order and their per-head sample lists repeated for every query head of a group."""
    b, h, hk, n, d = 2, 4, 2, 1024, 64
    q, _, _, qi, _ = _sorted_inputs(b, h, n, d, torch.float16, 95)
    _, k, v, _, ki = _sorted_inputs(b, hk, n, d, torch.float16, 96)
    sampled = torch.randint(0, n, (hk, 128), generator=_gen(97))
    c = lambda t: t.cuda().transpose(1, 2)
    rep = lambda t: t.repeat_interleave(h // hk, dim=1)
    got, got_lse = ha.hyper_attn_func(c(q), c(k), c(v), c(qi), c(ki), 256, 128, None, smooth, sampled_idx=sampled.cuda())
    want, want_lse = ha.hyper_attn_func(c(q), c(rep(k)), c(rep(v)), c(qi), c(rep(ki)), 256, 128, None, smooth,
                                        sampled_idx=rep(sampled.view(1, hk, 128)).view(h, 128).cuda())
    assert torch.equal(got, want) and torch.equal(got_lse, want_lse)
    fo, fl = ha.flash_attn_func(c(q), c(k), c(v), None, True)
    wo, wl = ha.flash_attn_func(c(q), c(rep(k)), c(rep(v)), None, True)
    assert torch.equal(fo, wo) and torch.equal(fl, wl)


def test_block_attention_value_dim_differs(ha):
    """unit_tests/test_hyper_attention.py:120-133: V narrower than Q and K gives the matching columns
    of the full-width result; the other way round (wider V) follows from the same definition."""
    b, h, n, d = 1, 2, 1024, 128
    q, k, v, qi, ki = _sorted_inputs(b, h, n, d, torch.bfloat16, 80)
    full, lse_full = _run_hyper(ha, q, k, v, qi, ki, 256, 128, None, False)
    small, lse_small = _run_hyper(ha, q, k, v[..., :d // 2].clone(), qi, ki, 256, 128, None, False)
    assert small.shape == (b, h, n, d // 2)
    assert torch.equal(small, full[..., :d // 2]) and torch.equal(lse_small, lse_full)
    wide, lse_wide = _run_hyper(ha, q[..., :64].clone(), k[..., :64].clone(), v, qi, ki, 256, 128, None, False)
    ro, rl = O.block_sampled_attention(q[..., :64], k[..., :64], v, qi, ki, 256, 128, None, False)
    assert wide.shape == (b, h, n, d)
    assert_close(wide, ro, "wide-v out", torch.bfloat16)
    assert_close(lse_wide, rl, "wide-v lse")


def test_block_attention_argument_errors(ha):
    z = torch.zeros((1, 256, 1, 64), dtype=torch.float16, device="cuda")
    idx = torch.arange(256, device="cuda").view(1, 256, 1)
    with pytest.raises(AssertionError):
        ha.hyper_attn_func(z, z, z, idx, idx, 128, 100)       # sample_size % 128
    with pytest.raises(AssertionError):
        ha.hyper_attn_func(z.float(), z.float(), z.float(), idx, idx, 128, 0)
    z2 = torch.zeros((1, 192, 1, 64), dtype=torch.float16, device="cuda")
    idx2 = torch.arange(192, device="cuda").view(1, 192, 1)
    with pytest.raises(AssertionError):
        ha.hyper_attn_func(z2, z2, z2, idx2, idx2, 128, 0)    # seqlen_k % 128
    z3 = torch.zeros((1, 256, 1, 256), dtype=torch.float16, device="cuda")
    with pytest.raises(AssertionError):
        ha.hyper_attn_func(z3, z3, z3, idx, idx, 128, 0)      # head dim > 128


# ------------------------------------------------------------------------------------ merge
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_add_self_attentions(ha, dtype):
    b, h, n, d = 2, 2, 300, 64
    q, k, v = (_randn((b, h, n, d), s, dtype) for s in (50, 51, 52))
    a1, l1 = O.exact_attention(q, k[:, :, :100], v[:, :, :100])
    a2, l2 = O.exact_attention(q, k[:, :, 100:], v[:, :, 100:])
    got, glse = ha.add_self_attentions(a1.to(dtype).cuda(), l1.float().unsqueeze(-1).cuda(),
                                       a2.to(dtype).cuda(), l2.float().unsqueeze(-1).cuda())
    want, wlse = O.add_self_attentions(a1.to(dtype).double(), l1.float().double().unsqueeze(-1),
                                       a2.to(dtype).double(), l2.float().double().unsqueeze(-1))
    assert got.dtype == dtype and glse.shape == (b, h, n, 1)
    assert_close(got, want, "merge out", dtype)
    assert_close(glse, wlse, "merge lse")
    # and against the exact attention over the union of the two key sets
    ro, rl = O.exact_attention(q, k, v)
    assert_close(got, ro, "merge vs union", dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_add_self_attentions_is_the_same_with_and_without_grad(ha, dtype):
    """The weight is rounded to the attention's type on both routes (src/attn_utils.py:21): the kernel and
    the differentiable tensor arithmetic give the same merge up to the last rounding of the output."""
    b, h, n, d = 1, 2, 200, 64
    a1, a2 = (_randn((b, h, n, d), s, dtype).cuda() for s in (70, 71))
    l1, l2 = (_randn((b, h, n, 1), s, torch.float32).cuda() * 3 for s in (72, 73))
    plain, plain_lse = ha.add_self_attentions(a1, l1, a2, l2)
    g1 = a1.clone().requires_grad_()
    grad, grad_lse = ha.add_self_attentions(g1, l1, a2, l2)
    # torch rounds c*a1 and (1-c)*a2 to the type before adding them, the kernel rounds once: one ulp apart
    ulp = 2.0 ** (-10 if dtype == torch.float16 else -7)
    assert float((plain.float() - grad.detach().float()).abs().max()) <= 2 * ulp * float(plain.float().abs().max())
    assert torch.allclose(plain_lse, grad_lse.detach(), rtol=0, atol=1e-5)
    # the weight itself: with a1 = 1, a2 = 0 the merged rows ARE the rounded weight
    ones, zeros = torch.ones_like(a1), torch.zeros_like(a2)
    c_kernel, _ = ha.add_self_attentions(ones, l1, zeros, l2)
    c_ref = torch.sigmoid(l1 - l2).to(dtype)
    assert torch.equal(c_kernel, c_ref.expand_as(c_kernel))


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("dtype,levels", [(torch.float16, 3), (torch.bfloat16, 2), (torch.float16, 0)])
def test_merge_levels_equals_the_chain_of_segment_merges(ha, dtype, levels, packed):
    """ha_lse_merge_levels against the per-level in-place merges it stands for (bit for bit), and its shifted
    log-sum-exps against lse - log(weight) from the weights those merges write.  packed: the level arrays hold
    only the second halves of the level's segments, one after the other."""
    import ctypes
    from hyperattention_amd import _lib
    b, h, d, leaf = 2, 3, 64, 40
    n = leaf << levels
    dev = dict(device="cuda")
    o_leaf = _randn((b, h, n, d), 80, dtype).cuda()
    lse_leaf = _randn((b, h, n), 81, torch.float32).cuda() * 4
    o_un = _randn((max(levels, 1), b, h, n, d), 82, dtype).cuda()
    lse_un = _randn((max(levels, 1), b, h, n), 83, torch.float32).cuda() * 4
    if levels:
        lse_un[0, :, :, -5:] += 200.0   # weight of what was there rounds to 0
        lse_un[levels - 1, :, :, n - leaf:n - leaf + 5] -= 200.0   # weight of the level's call is 0
    lib, code = _lib.lib(), 0 if dtype == torch.float16 else 1
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # the chain, deepest level first
    out, lse = o_leaf.clone(), lse_leaf.clone()
    cs = {}
    for j in reversed(range(levels)):
        H, half = (b * h) << j, n >> (j + 1)
        out2, lse2 = out.view(H, 2, half, d)[:, 1], lse.view(H, 2, half)[:, 1]
        o2 = o_un[j].view(H, 2, half, d)[:, 1].contiguous()
        l2 = lse_un[j].view(H, 2, half)[:, 1].contiguous()
        c = torch.empty((H, half), dtype=torch.float32, **dev)
        _lib.check(lib.ha_lse_merge_segments(
            out2.data_ptr(), lse2.data_ptr(), o2.data_ptr(), l2.data_ptr(), out2.data_ptr(), lse2.data_ptr(),
            c.data_ptr(), H, half, d, 2 * half * d, d, half * d, d, 2 * half * d, d, 2 * half, half, 2 * half, half,
            code, stream))
        cs[j] = c
    got, got_lse = torch.empty_like(o_leaf), torch.empty_like(lse_leaf)
    shifted = torch.full((max(levels, 1), b, h, n), float("nan"), dtype=torch.float32, **dev)
    leaf_shifted = torch.empty_like(lse_leaf)
    ptrs = lambda x: (ctypes.c_void_p * max(levels, 1))(*[x[j].data_ptr() for j in range(levels)])
    if packed:
        # (levels, b, h, n/2[, d]): the second halves of the segments of n >> j rows, one after the other
        second = lambda x, j, tail: x[j].reshape(b, h, 1 << j, 2, n >> (j + 1), *tail)[:, :, :, 1].reshape(b, h, n // 2, *tail)
        o_pk = torch.stack([second(o_un, j, (d,)) for j in range(levels)]) if levels else o_un[:, :, :, : n // 2]
        l_pk = torch.stack([second(lse_un, j, ()) for j in range(levels)]) if levels else lse_un[:, :, :, : n // 2]
        o_pk, l_pk = o_pk.contiguous(), l_pk.contiguous()
        s_pk = torch.full((max(levels, 1), b, h, n // 2), float("nan"), dtype=torch.float32, **dev)
        _lib.check(lib.ha_lse_merge_levels(o_leaf.data_ptr(), lse_leaf.data_ptr(), ptrs(o_pk), ptrs(l_pk), ptrs(s_pk),
                                           leaf_shifted.data_ptr(), got.data_ptr(), got_lse.data_ptr(), levels, b * h, n, d,
                                           code, 1, stream))
        for j in range(levels):
            shifted[j].view(b, h, 1 << j, 2, n >> (j + 1))[:, :, :, 1] = s_pk[j].view(b, h, 1 << j, n >> (j + 1))
    else:
        _lib.check(lib.ha_lse_merge_levels(o_leaf.data_ptr(), lse_leaf.data_ptr(), ptrs(o_un), ptrs(lse_un), ptrs(shifted),
                                           leaf_shifted.data_ptr(), got.data_ptr(), got_lse.data_ptr(), levels, b * h, n, d,
                                           code, 0, stream))
    torch.cuda.synchronize()
    assert torch.equal(got, out) and torch.equal(got_lse, lse)
    log_w = torch.zeros((b, h, n), dtype=torch.float64, **dev)
    for j in range(levels):
        H, half = (b * h) << j, n >> (j + 1)
        c = cs[j].double()
        log_w2 = log_w.view(H, 2, half)[:, 1]
        want = lse_un[j].view(H, 2, half)[:, 1].double() - torch.log1p(-c) - log_w2
        have = shifted[j].view(H, 2, half)
        assert torch.isnan(have[:, 0]).all(), "first halves are not written"
        have = have[:, 1].double()
        both_inf = torch.isinf(want) & torch.isinf(have) & (want > 0) & (have > 0)
        assert (both_inf | ((want - have).abs() <= 1e-4 * (1 + want.abs()))).all(), f"shifted lse of level {j}"
        log_w2 += torch.log(c)
    want = lse_leaf.double() - log_w
    have = leaf_shifted.double()
    both_inf = torch.isinf(want) & torch.isinf(have) & (want > 0) & (have > 0)
    assert (both_inf | ((want - have).abs() <= 1e-4 * (1 + want.abs()))).all(), "shifted lse of the leaves"
    if levels:
        assert torch.isinf(leaf_shifted).any() and torch.isinf(shifted[levels - 1][~torch.isnan(shifted[levels - 1])]).any()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_merge_segments_in_place(ha, dtype):
    """ha_lse_merge_segments on the second halves of every head, in place, with the weight written out:
    the merge of one level of the causal recursion (hyper_attention.py:86-89)."""
    import ctypes
    from hyperattention_amd import _lib
    b, h, n, d = 2, 3, 256, 64
    half = n // 2
    q, k, v = (_randn((b, h, n, d), s, dtype) for s in (60, 61, 62))
    q2 = q[:, :, half:]
    a1, l1 = O.exact_attention(q2, k[:, :, half:], v[:, :, half:])          # what the second halves hold
    a2, l2 = O.exact_attention(q2, k[:, :, :half], v[:, :, :half])          # the un-masked call of the level
    out = torch.zeros((b, h, n, d), dtype=dtype).cuda()
    lse = torch.zeros((b, h, n), dtype=torch.float32).cuda()
    out[:, :, half:] = a1.to(dtype).cuda()
    lse[:, :, half:] = l1.float().cuda()
    o_un, lse_un = a2.to(dtype).cuda().contiguous(), l2.float().cuda().contiguous()
    w = torch.empty((b, h, half), dtype=torch.float32, device="cuda")
    out2, lse2 = out[:, :, half:], lse[:, :, half:]
    lib = _lib.lib()
    _lib.check(lib.ha_lse_merge_segments(
        out2.data_ptr(), lse2.data_ptr(), o_un.data_ptr(), lse_un.data_ptr(), out2.data_ptr(), lse2.data_ptr(),
        w.data_ptr(), b * h, half, d, n * d, d, half * d, d, n * d, d, n, half, n, half,
        0 if dtype == torch.float16 else 1, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    want, wlse = O.add_self_attentions(a1.to(dtype).double(), l1.float().double().unsqueeze(-1),
                                       a2.to(dtype).double(), l2.float().double().unsqueeze(-1))
    assert_close(out[:, :, half:], want, "segment merge out", dtype)
    assert_close(lse[:, :, half:], wlse.squeeze(-1), "segment merge lse")
    ro, rl = O.exact_attention(q2, k, v)
    assert_close(out[:, :, half:], ro, "segment merge vs union", dtype)
    assert float(out[:, :, :half].abs().max()) == 0 and float(lse[:, :, :half].abs().max()) == 0  # first halves untouched
    c = torch.sigmoid(l1.float() - l2.float()).to(dtype).float()
    assert float((w.cpu() - c).abs().max()) <= 2 * torch.finfo(dtype).eps
