"""GPU parity tests of the attention backward (through the C ABI, driven by torch autograd) against
gradients of the CPU oracle.

The oracle's forward functions are plain torch arithmetic in float64, so torch autograd differentiates
them as they stand; tests/test_oracle.py checks those gradients against finite differences and against
the closed formulas.  A gradient arriving for the log-sum-exp output is ignored by the operators, as
in the reference (src/hyper_attn_triton.py:922-945, src/flash_attn_triton.py:1014-1040): the loss used
here depends on the attention output only.

Tolerances: norm-wise ||g - ref|| <= tol ||ref|| per gradient tensor, tol = 3e-3 for fp16 and 8e-3 for
bf16.  They are wider than the forward's because P and dS are rounded to the input type before the
products, as the reference does (src/hyper_attn_triton.py:345,367), and dS has twice the relative
error of P, and gradients that several calls add to are rounded once per call.  500 random
configurations with the default soft-max scale stay below 1.6e-3 in fp16 and 5.4e-3 in bf16; with
scales up to 0.2 (peaked soft-max: dP - D cancels, and D comes from the rounded output) fp16 reaches
3.0e-3.
"""
import numpy as np
import pytest
import torch

from oracle import hyper_oracle as O

pytestmark = pytest.mark.gpu

from _util import _gen, _randn

TOL = {torch.float16: 3e-3, torch.bfloat16: 8e-3}


@pytest.fixture(scope="module")
def ha():
    import hyperattention_amd
    from hyperattention_amd import _lib
    _lib.lib()  # fails loudly when the HIP library is missing
    return hyperattention_amd


def _check(got, ref, what, dtype):
    got = got.detach().double().cpu()
    ref = ref.detach().double().cpu()
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got).all(), f"{what}: non-finite values"
    # a gradient that is exactly zero (a single key: the soft-max is constant) is compared absolutely
    rel = ((got - ref).norm() / ref.norm().clamp(min=1e-3)).item()
    assert rel <= TOL[dtype], f"{what}: norm-wise relative error {rel:.3e} > {TOL[dtype]}"
    # no element far off: a wrong row or a dropped tile shows here even when the norm hides it
    worst = ((got - ref).abs().max() / ref.abs().max().clamp(min=1e-3)).item()
    assert worst <= 10 * TOL[dtype], f"{what}: worst element error {worst:.3e} of the largest gradient"


def _oracle_grads(fn, q, k, v, do):
    q64, k64, v64 = (x.double().requires_grad_() for x in (q, k, v))
    out, _ = fn(q64, k64, v64)
    out.backward(do.double())
    return q64.grad, k64.grad, v64.grad


def _gpu_grads(fn, q, k, v, do):
    """fn takes (b,n,h,d) CUDA tensors and returns (o (b,n,h,d), lse); inputs here are (b,h,n,d) CPU."""
    qg, kg, vg = (x.cuda().transpose(1, 2).contiguous().requires_grad_() for x in (q, k, v))
    o, lse = fn(qg, kg, vg)
    o.backward(do.cuda().transpose(1, 2).contiguous())
    torch.cuda.synchronize()
    return o, lse, qg.grad.transpose(1, 2), kg.grad.transpose(1, 2), vg.grad.transpose(1, 2)


# ------------------------------------------------------------------------------- exact attention
@pytest.mark.parametrize("dtype,b,h,nq,nk,d,causal", [
    (torch.float16, 1, 2, 256, 256, 64, False),
    (torch.float16, 1, 2, 256, 256, 64, True),
    (torch.float16, 2, 3, 300, 300, 64, True),       # ragged: last tiles are partial
    (torch.bfloat16, 1, 2, 333, 333, 128, True),
    (torch.bfloat16, 1, 2, 200, 517, 128, False),    # more keys than queries
    (torch.float16, 1, 1, 640, 130, 64, False),      # more queries than keys
    (torch.float16, 1, 2, 1, 1, 64, True),           # a single row
    (torch.float16, 1, 2, 300, 130, 64, True),       # causal with fewer keys than queries (mask row >= col)
    (torch.bfloat16, 1, 2, 200, 517, 128, True),     # causal with more keys: the last keys get no gradient
])
def test_flash_backward(ha, dtype, b, h, nq, nk, d, causal):
    q = _randn((b, h, nq, d), 11, dtype)
    k = _randn((b, h, nk, d), 12, dtype)
    v = _randn((b, h, nk, d), 13, dtype)
    do = _randn((b, h, nq, d), 14, dtype)
    ref = _oracle_grads(lambda a, b_, c: O.exact_attention(a, b_, c, None, causal), q, k, v, do)
    o, lse, dq, dk, dv = _gpu_grads(lambda a, b_, c: ha.flash_attn_func(a, b_, c, None, causal), q, k, v, do)
    with torch.no_grad():
        o_plain, _ = ha.flash_attn_func(q.cuda().transpose(1, 2), k.cuda().transpose(1, 2), v.cuda().transpose(1, 2),
                                        None, causal)
    assert torch.equal(o.detach(), o_plain), "the forward under autograd differs from the plain forward"
    for got, want, name in zip((dq, dk, dv), ref, ("dq", "dk", "dv")):
        _check(got, want, f"flash {name}", dtype)


# ------------------------------------------------------------------- sorted blocks + sampled keys
def _perms(b, h, n, seed):
    g = _gen(seed)
    return torch.stack([torch.stack([torch.randperm(n, generator=g) for _ in range(h)]) for _ in range(b)])


@pytest.mark.parametrize("dtype,b,h,n,d,block,sample,smooth", [
    (torch.float16, 1, 2, 1024, 64, 256, 256, False),
    (torch.float16, 1, 2, 1024, 64, 256, 256, True),
    (torch.float16, 2, 2, 768, 64, 256, 0, False),      # no samples; the last block is shorter
    (torch.float16, 1, 1, 768, 64, 512, 128, True),     # smoothed, block does not divide the length
    (torch.bfloat16, 1, 2, 2048, 128, 512, 512, True),
    (torch.bfloat16, 1, 3, 1024, 128, 256, 128, False),
    (torch.float16, 1, 2, 512, 64, 512, 128, False),    # one block = exact attention plus the samples
    (torch.float16, 1, 1, 384, 64, 128, 128, False),
])
def test_block_backward(ha, dtype, b, h, n, d, block, sample, smooth):
    q = _randn((b, h, n, d), 21, dtype)
    k = _randn((b, h, n, d), 22, dtype)
    v = _randn((b, h, n, d), 23, dtype)
    do = _randn((b, h, n, d), 24, dtype)
    qi, ki = _perms(b, h, n, 25), _perms(b, h, n, 26)
    ref = _oracle_grads(lambda a, b_, c: O.block_sampled_attention(a, b_, c, qi, ki, block, sample, None, smooth),
                        q, k, v, do)
    qi_g, ki_g = qi.cuda().transpose(1, 2), ki.cuda().transpose(1, 2)
    o, lse, dq, dk, dv = _gpu_grads(lambda a, b_, c: ha.hyper_attn_func(a, b_, c, qi_g, ki_g, block, sample, None, smooth),
                                    q, k, v, do)
    for got, want, name in zip((dq, dk, dv), ref, ("dq", "dk", "dv")):
        _check(got, want, f"block {name}", dtype)


@pytest.mark.parametrize("per_head", [False, True])
def test_block_backward_explicit_samples_with_repeats(ha, per_head):
    # sampled rows given explicitly, some of them twice: each occurrence is one more column of the
    # soft-max, and the key's gradient adds them up
    dtype, b, h, n, d, block, sample = torch.float16, 1, 2, 1024, 64, 256, 128
    q = _randn((b, h, n, d), 31, dtype)
    k = _randn((b, h, n, d), 32, dtype)
    v = _randn((b, h, n, d), 33, dtype)
    do = _randn((b, h, n, d), 34, dtype)
    qi, ki = _perms(b, h, n, 35), _perms(b, h, n, 36)
    g = _gen(37)
    if per_head:
        si = torch.randint(0, n, (b, h, sample), generator=g)
        si[:, :, 5] = si[:, :, 4]
        si_gpu = si[0]
    else:
        si = torch.randint(0, n, (sample,), generator=g)
        si[5] = si[4]
        si[100] = si[4]
        si_gpu = si
    ref = _oracle_grads(lambda a, b_, c: O.block_sampled_attention(a, b_, c, qi, ki, block, sample, None, False,
                                                                   sampled_idx=si), q, k, v, do)
    qi_g, ki_g = qi.cuda().transpose(1, 2), ki.cuda().transpose(1, 2)
    o, lse, dq, dk, dv = _gpu_grads(
        lambda a, b_, c: ha.hyper_attn_func(a, b_, c, qi_g, ki_g, block, sample, None, False, sampled_idx=si_gpu),
        q, k, v, do)
    for got, want, name in zip((dq, dk, dv), ref, ("dq", "dk", "dv")):
        _check(got, want, f"block {name}", dtype)


def test_block_backward_int32_indices_and_sorted_buckets(ha):
    # permutations as the module makes them: stable argsort of LSH buckets, int32
    dtype, b, h, n, d = torch.float16, 1, 2, 2048, 64
    q = _randn((b, h, n, d), 41, dtype)
    k = _randn((b, h, n, d), 42, dtype)
    v = _randn((b, h, n, d), 43, dtype)
    do = _randn((b, h, n, d), 44, dtype)
    proj = _randn((d, 8), 45, dtype)
    qi = torch.from_numpy(O.stable_bucket_argsort(O.lsh_hash(q, proj)))
    ki = torch.from_numpy(O.stable_bucket_argsort(O.lsh_hash(k, proj)))
    ref = _oracle_grads(lambda a, b_, c: O.block_sampled_attention(a, b_, c, qi, ki, 256, 256), q, k, v, do)
    qi_g, ki_g = qi.int().cuda().transpose(1, 2), ki.int().cuda().transpose(1, 2)
    o, lse, dq, dk, dv = _gpu_grads(lambda a, b_, c: ha.hyper_attn_func(a, b_, c, qi_g, ki_g, 256, 256), q, k, v, do)
    for got, want, name in zip((dq, dk, dv), ref, ("dq", "dk", "dv")):
        _check(got, want, f"block {name}", dtype)


# ------------------------------------------------------------------------- adding to gradients that are there
@pytest.mark.parametrize("kind,dtype,d", [("block", torch.bfloat16, 64), ("block", torch.float16, 128),
                                          ("block_smooth", torch.float16, 64), ("flash_causal", torch.bfloat16, 64),
                                          ("flash", torch.float16, 128)])
def test_backward_accumulate_adds_to_what_is_there(ha, kind, dtype, d):
    # ha_attn_grads.accumulate: dq, dk, dv hold values when the call starts and hold value + gradient when it
    # ends (one rounding of the fp32 sum), through the C ABI, against the same call without the flag
    import ctypes
    from hyperattention_amd import _lib, ops
    b, h, n, block, sample = 2, 3, 768, 256, 128
    q, k, v, do = (_randn((b, h, n, d), 170 + i, dtype).cuda().transpose(1, 2).contiguous() for i in range(4))
    o = torch.empty_like(q)
    lse = torch.empty((b, h, n), device="cuda", dtype=torch.float32)
    lib = _lib.lib()
    stream = ops._stream(q)
    if kind.startswith("block"):
        qi, ki = (_perms(b, h, n, 175 + i).cuda().transpose(1, 2) for i in range(2))
        a, keep = ops._block_attn_args(q, k, v, o, lse, qi, ki, block, sample, d ** -0.5, kind == "block_smooth", None)
        _lib.check(lib.ha_block_attn_fwd(ctypes.byref(a), stream))
        run = lambda g: _lib.check(lib.ha_block_attn_bwd(ctypes.byref(a), ctypes.byref(g), stream))
        t = a.t
    else:
        t = ops._operands(q, k, v, o, lse, d ** -0.5, layout_bnhd=True, lse_row_stride=n)
        causal = int(kind == "flash_causal")
        _lib.check(lib.ha_flash_attn_fwd(ctypes.byref(t), causal, stream))
        run = lambda g: _lib.check(lib.ha_flash_attn_bwd(ctypes.byref(t), causal, ctypes.byref(g), stream))
    sample_size = sample if kind.startswith("block") else 0
    plain = [torch.empty_like(x) for x in (q, k, v)]
    g0, ws0 = ops._attn_grads(t, do, *plain, sample_size=sample_size)
    run(g0)
    base = [_randn((b, h, n, d), 180 + i, dtype).cuda().transpose(1, 2).contiguous() for i in range(3)]
    added = [x.clone() for x in base]
    g1, ws1 = ops._attn_grads(t, do, *added, accumulate=True, sample_size=sample_size)
    run(g1)
    torch.cuda.synchronize()
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    for got, grad, start, name in zip(added, plain, base, ("dq", "dk", "dv")):
        # the kernel adds its fp32 sum to the stored value and rounds once, where `grad` is that sum rounded
        # (the sampled keys' share is added by a second kernel, with a rounding of its own): a few roundings
        # of values of the result's size, so the distance is of the order of one unit in the last place
        want = grad.float() + start.float()
        rel = float((got.float() - want).norm() / want.norm())
        assert rel <= 1.5 * ulp, f"{kind} {name}: relative distance {rel:.3e}"
        assert not torch.equal(got, start)


# ------------------------------------------------------------------------- grouped-query heads
@pytest.mark.parametrize("kind", ["flash", "flash_causal", "block"])
def test_backward_grouped_query_heads_through_the_c_abi(ha, kind):
    # 4 query heads on 2 key/value heads, handed to the C entry points as they are (kv_group = 2): the
    # gradient of a key head is the sum over the query heads of its group
    import ctypes
    from hyperattention_amd import _lib, ops
    dtype, b, h, hk, n, d, block, sample = torch.float16, 1, 4, 2, 512, 64, 256, 128
    q = _randn((b, h, n, d), 61, dtype)
    k = _randn((b, hk, n, d), 62, dtype)
    v = _randn((b, hk, n, d), 63, dtype)
    do = _randn((b, h, n, d), 64, dtype)
    qi, ki = _perms(b, h, n, 65), _perms(b, hk, n, 66)
    expand = lambda x: x.repeat_interleave(h // hk, dim=1)
    if kind == "block":
        fn = lambda a, b_, c: O.block_sampled_attention(a, expand(b_), expand(c), qi, expand(ki), block, sample)
    else:
        fn = lambda a, b_, c: O.exact_attention(a, expand(b_), expand(c), None, kind == "flash_causal")
    ref = _oracle_grads(fn, q, k, v, do)

    qg, kg, vg, dog = (x.cuda().transpose(1, 2).contiguous() for x in (q, k, v, do))  # (b,n,heads,d)
    o = torch.empty_like(qg)
    lse = torch.empty((b, h, n), device="cuda", dtype=torch.float32)
    dq, dk, dv = torch.empty_like(qg), torch.empty_like(kg), torch.empty_like(vg)
    lib = _lib.lib()
    stream = ops._stream(qg)
    if kind == "block":
        qi_g, ki_g = qi.cuda().transpose(1, 2), ki.cuda().transpose(1, 2)
        a, keep = ops._block_attn_args(qg, kg, vg, o, lse, qi_g, ki_g, block, sample, d ** -0.5, False, None)
        assert a.t.kv_group == 2
        _lib.check(lib.ha_block_attn_fwd(ctypes.byref(a), stream))
        g, ws = ops._attn_grads(a.t, dog, dq, dk, dv, sample_size=sample)
        _lib.check(lib.ha_block_attn_bwd(ctypes.byref(a), ctypes.byref(g), stream))
    else:
        t = ops._operands(qg, kg, vg, o, lse, d ** -0.5, layout_bnhd=True, lse_row_stride=n)
        assert t.kv_group == 2
        causal = int(kind == "flash_causal")
        _lib.check(lib.ha_flash_attn_fwd(ctypes.byref(t), causal, stream))
        g, ws = ops._attn_grads(t, dog, dq, dk, dv)
        _lib.check(lib.ha_flash_attn_bwd(ctypes.byref(t), causal, ctypes.byref(g), stream))
    torch.cuda.synchronize()
    for got, want, name in zip((dq, dk, dv), ref, ("dq", "dk", "dv")):
        _check(got.transpose(1, 2), want, f"{kind} {name}", dtype)


# ------------------------------------------------------------------------------- the module
@pytest.mark.parametrize("causal,n,min_seq_len,block,sample,smooth,kv_heads", [
    (False, 1024, 256, 128, 128, False, 2),
    (True, 1024, 256, 128, 128, False, 2),    # two hashed levels, on views with accumulated gradients
    (True, 1025, 600, 128, 128, False, 2),    # odd length: the operator-by-operator recursion, padded
    (True, 2048, 512, 256, 256, True, 2),     # smoothed blocks
    (True, 1024, 600, 128, 128, False, 2),    # the off-diagonal call is exact (min_seq_len > n/2)
    (True, 2048, 256, 128, 128, False, 1),    # three levels; two query heads on one key/value head
    (False, 1024, 256, 128, 128, True, 1),    # one un-masked call with grouped heads taken as they are
])
def test_module_backward(ha, causal, n, min_seq_len, block, sample, smooth, kv_heads):
    # the module under autograd: operators with their own backward, merges as tensor arithmetic;
    # log-sum-exps carry no gradient (detach_lse), as the reference's operators return none for them
    dtype, b, h, d = torch.float16, 1, 2, 64
    q = _randn((b, h, n, d), 51, dtype)
    k = _randn((b, kv_heads, n, d), 52, dtype)
    v = _randn((b, kv_heads, n, d), 53, dtype)
    do = _randn((b, h, n, d), 54, dtype)
    m = ha.HyperAttention(input_dim=d, block_size=block, sample_size=sample, min_seq_len=min_seq_len, smooth_block=smooth,
                          rng=_gen(55))
    m = m.to(device="cuda", dtype=dtype)
    proj = m.lsh.proj_dir[0, 0].cpu()
    expand = lambda x: x.repeat_interleave(h // kv_heads, dim=1)
    ref = _oracle_grads(lambda a, b_, c: O.hyper_forward(a, expand(b_), expand(c), proj, causal=causal, block_size=block,
                                                         sample_size=sample, min_seq_len=min_seq_len, smooth_block=smooth,
                                                         detach_lse=True), q, k, v, do)
    qg, kg, vg = (x.cuda().requires_grad_() for x in (q, k, v))
    out = m(qg, kg, vg, causal=causal)
    with torch.no_grad():
        out_plain = m(q.cuda(), k.cuda(), v.cuda(), causal=causal)
    rel = ((out.detach().double() - out_plain.double()).norm() / out_plain.double().norm()).item()
    assert rel < 2e-3, f"forward under autograd vs one-call forward: {rel:.3e}"
    out.backward(do.cuda())
    torch.cuda.synchronize()
    for got, want, name in zip((qg.grad, kg.grad, vg.grad), ref, ("dq", "dk", "dv")):
        _check(got, want, f"module {name}", dtype)


def test_module_backward_random_configurations(ha):
    """Seeded random constructor arguments and shapes for the module under autograd (causal recursion on
    segments with grouped heads, smoothed blocks, odd tile counts per block, no samples, more than 8
    projections): gradients against torch autograd on the oracle, the reference's constant-log-sum-exp convention."""
    rng = np.random.default_rng(21)
    for case in range(6):
        d = int(rng.choice([64, 128]))
        dtype = [torch.float16, torch.bfloat16][int(rng.integers(0, 2))]
        causal = case % 3 != 2
        block = 128 * int(rng.integers(1, 4))
        sample = 128 * int(rng.integers(0, 3))
        smooth = bool(rng.integers(0, 2))
        r = int(rng.integers(2, 13))
        hk = int(rng.integers(1, 3))
        h = hk * int(rng.integers(1, 3))
        levels = int(rng.integers(1, 3)) if causal else 0
        leaf = 128 * int(rng.integers(2, 4))
        n = (leaf << levels) if causal else 128 * int(rng.integers(4, 9))
        msl = leaf if causal else 128
        sample = min(sample, leaf)
        what = (f"case {case}: d {d} {dtype} causal {causal} n {n} min_seq_len {msl} block {block} sample {sample} "
                f"smooth {smooth} r {r} heads {h}/{hk}")
        q = _randn((1, h, n, d), 1200 + case, dtype)
        k, v = (_randn((1, hk, n, d), s + case, dtype) for s in (1300, 1400))
        do = _randn((1, h, n, d), 1500 + case, dtype)
        m = ha.HyperAttention(input_dim=d, lsh_num_projs=r, block_size=block, sample_size=sample, min_seq_len=msl,
                              smooth_block=smooth, rng=_gen(1600 + case)).to(device="cuda", dtype=dtype)
        proj = m.lsh.proj_dir[0, 0].cpu()
        expand = lambda x: x.repeat_interleave(h // hk, dim=1)
        ref = _oracle_grads(lambda a, b_, c: O.hyper_forward(a, expand(b_), expand(c), proj, causal=causal,
                                                             lsh_num_projs=r, block_size=block, sample_size=sample,
                                                             min_seq_len=msl, smooth_block=smooth, detach_lse=True),
                            q, k, v, do)
        qg, kg, vg = (x.cuda().requires_grad_() for x in (q, k, v))
        m(qg, kg, vg, causal=causal).backward(do.cuda())
        torch.cuda.synchronize()
        for got, want, name in zip((qg.grad, kg.grad, vg.grad), ref, ("dq", "dk", "dv")):
            _check(got, want, f"{what}: {name}", dtype)


def test_module_backward_twice_and_retain_graph(ha):
    # the backward neither consumes nor disturbs what it saved: two passes over one graph agree
    dtype, b, h, n, d = torch.bfloat16, 1, 2, 1024, 64
    q, k, v, do = (_randn((b, h, n, d), 70 + i, dtype).cuda() for i in range(4))
    m = ha.HyperAttention(input_dim=d, block_size=128, sample_size=128, min_seq_len=256, rng=_gen(75)).to(device="cuda", dtype=dtype)
    qg, kg, vg = (x.clone().requires_grad_() for x in (q, k, v))
    out = m(qg, kg, vg, causal=True)
    out.backward(do, retain_graph=True)
    first = [x.grad.clone() for x in (qg, kg, vg)]
    for x in (qg, kg, vg):
        x.grad = None
    out.backward(do)
    for a, b_ in zip(first, (qg.grad, kg.grad, vg.grad)):
        # the sampled keys' sums are accumulated with atomics, in an order that can differ between runs
        assert ((a.double() - b_.double()).norm() / a.double().norm()).item() < 1e-3


def test_gradients_of_heads_far_into_large_tensors_equal_those_of_the_heads_alone(ha):
    """2^20 rows, 24 heads: the last heads start more than 2^31 bytes into q, k, v and the gradients.  A head's
    gradients inside the big call equal those of the same head in a call of its own (the sampled keys' sums are
    accumulated with atomics, so to rounding)."""
    dtype, h, n, d = torch.bfloat16, 24, 1 << 20, 64
    g = torch.Generator(device="cuda").manual_seed(240)
    q, k, v = (torch.randn((1, h, n, d), generator=g, device="cuda", dtype=dtype).requires_grad_() for _ in range(3))
    dout = torch.randn((1, h, n, d), generator=g, device="cuda", dtype=dtype)
    assert q[0, h - 1].data_ptr() - q.data_ptr() > 1 << 31
    m = ha.HyperAttention(input_dim=d, block_size=256, sample_size=256, min_seq_len=4096,
                          rng=torch.Generator().manual_seed(241)).to(device="cuda", dtype=dtype)
    for causal in (True, False):
        grads = torch.autograd.grad(m(q, k, v, causal=causal), (q, k, v), dout)
        for head in (0, h - 1):
            sl = slice(head, head + 1)
            q1, k1, v1 = (x[:, sl].detach().clone().requires_grad_() for x in (q, k, v))
            alone = torch.autograd.grad(m(q1, k1, v1, causal=causal), (q1, k1, v1), dout[:, sl].contiguous())
            for big, one, what in zip(grads, alone, ("dq", "dk", "dv")):
                assert torch.isfinite(one.float()).all()
                rel = (big[:, sl].double() - one.double()).norm() / one.double().norm()
                assert float(rel) < 1e-3, (causal, head, what, float(rel))


def test_module_backward_on_views_agrees_with_operator_by_operator_at_length_32768(ha):
    # two routes to the same gradient at a length the CPU oracle does not reach: the recursion on views
    # with accumulated gradients, and the reference's recursion operator by operator under torch autograd
    dtype, b, h, n, d = torch.bfloat16, 1, 4, 32768, 64
    q, k, v, do = (_randn((b, h, n, d), 80 + i, dtype).cuda() for i in range(4))
    m = ha.HyperAttention(input_dim=d, block_size=256, sample_size=256, min_seq_len=2048, rng=_gen(85)).to(device="cuda", dtype=dtype)
    grads = []
    for route in ("views", "operators"):
        qg, kg, vg = (x.clone().requires_grad_() for x in (q, k, v))
        if route == "views":
            out = m(qg, kg, vg, causal=True)
        else:
            out, _ = m._forward_composed(qg, kg, vg, d ** -0.5, True)
        out.backward(do)
        grads.append((out.detach(), qg.grad, kg.grad, vg.grad))
    torch.cuda.synchronize()
    for a, b_, name in zip(grads[0], grads[1], ("out", "dq", "dk", "dv")):
        rel = ((a.double() - b_.double()).norm() / b_.double().norm()).item()
        # both round to bf16, the operator route once per level more (its gradients are added by torch)
        assert rel < 8e-3, f"{name}: {rel:.3e}"


def test_full_size_causal_backward_properties(ha):
    """Benchmark shape (batch 1, 32 heads, seq 131072, d 64, fp16, causal), too long for the oracle's
    autograd: what the mathematics fixes at any size.

    Every call of the recursion is soft-max attention over some set of keys, merged with weights that sum
    to one per query, and the scores enter as q.k only.  So per head
      sum_i <q_i, dq_i> = sum_ij S_ij dS_ij = sum_j <k_j, dk_j>,
      sum_j dv_j = sum_i dout_i                        (every query's weights over all its keys sum to one),
    the gradients are linear in dout, and a query of the first leaf only ever meets exact causal
    attention, so its dq is the exact attention's on that leaf (checked against the oracle)."""
    b, h, n, d = 1, 32, 131072, 64
    g = torch.Generator(device="cuda").manual_seed(190)
    q, k, v = (torch.randn((b, h, n, d), generator=g, device="cuda", dtype=torch.float16).requires_grad_()
               for _ in range(3))
    dout = torch.randn((b, h, n, d), generator=g, device="cuda", dtype=torch.float16)
    m = ha.HyperAttention(input_dim=d, block_size=256, sample_size=256, min_seq_len=2048,
                          rng=torch.Generator().manual_seed(191)).to(device="cuda", dtype=torch.float16)
    out = m(q, k, v, causal=True)
    dq, dk, dv = torch.autograd.grad(out, (q, k, v), dout, retain_graph=True)
    assert all(torch.isfinite(x).all() for x in (dq, dk, dv))

    qdq, kdk = (q.detach().float() * dq.float()), (k.detach().float() * dk.float())
    a, c = qdq.double().sum((0, 2, 3)), kdk.double().sum((0, 2, 3))
    noise = qdq.double().pow(2).sum((0, 2, 3)).sqrt() + kdk.double().pow(2).sum((0, 2, 3)).sqrt()
    assert float(((a - c).abs() / noise).max()) < 3e-3, ((a - c).abs() / noise).max()  # measured 6e-4

    sv, so = dv.double().sum(2), dout.double().sum(2)
    rel = (sv - so).norm() / so.norm()
    assert float(rel) < 2e-4, rel  # measured 2e-5

    dq2, dk2, dv2 = torch.autograd.grad(out, (q, k, v), 2 * dout, retain_graph=True)
    for x2, x, what in ((dq2, dq, "dq"), (dk2, dk, "dk"), (dv2, dv, "dv")):
        rel = (x2.double() - 2 * x.double()).norm() / x.double().norm()
        assert float(rel) < 1e-3, (what, rel)  # measured 3e-4: P and dS are rounded, small values lose bits

    # queries of the first leaf: exact causal attention only
    leaf = slice(0, 2048)
    ql, kl, vl = (x[:, :2, leaf].detach().double().cpu().requires_grad_() for x in (q, k, v))
    ro, _ = O.exact_attention(ql, kl, vl, None, True)
    (rdq,) = torch.autograd.grad(ro, (ql,), dout[:, :2, leaf].double().cpu())
    _check(dq[:, :2, leaf], rdq, "dq of the first leaf", torch.float16)
