"""GPU parity tests of the HyperAttention module (whole forward pass) against the CPU oracle, plus
size-independent properties at the full benchmark shapes.  Tolerances as in test_gpu_ops.py."""
import numpy as np
import pytest
import torch

from _util import _gen, _randn, assert_close
from oracle import hyper_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ha():
    import hyperattention_amd
    from hyperattention_amd import _lib
    _lib.lib()
    return hyperattention_amd


def _module(ha, d, dtype, seed, **kw):
    m = ha.HyperAttention(input_dim=d, rng=_gen(seed), **kw).to(device="cuda", dtype=dtype)
    return m, m.lsh.proj_dir[0, 0].cpu()


def _oracle(q, k, v, proj, m, causal, scale=None, sampled_idx=None, round_dtype=None):
    return O.hyper_forward(q, k, v, proj, scale=scale, causal=causal, lsh_num_projs=m.lsh_num_projs,
                           block_size=m.block_size, sample_size=m.sample_size, min_seq_len=m.min_seq_len,
                           smooth_block=m.smooth_block, sampled_idx=sampled_idx, round_dtype=round_dtype)


def _reference_arithmetic(dtype, *args, **kw):
    """The oracle's output in the reference's own arithmetic for a bf16 case (None otherwise): what a bf16
    output is measured against, see _util."""
    if dtype != torch.bfloat16:
        return None
    return _oracle(*args, round_dtype=torch.bfloat16, **kw)[0]


# --------------------------------------------------------------------------- non-causal
def test_non_causal_config1(ha):
    """benchmark configuration c1: batch 1, 4 heads, seq 4096, d 64, r 8, block 256, sample 256, min_seq_len 2048
    (inputs cast to fp16 for the GPU; both the default and an explicit seeded sample set)."""
    g = _gen(100)
    q, k, v = (torch.randn((1, 4, 4096, 64), generator=g).half() for _ in range(3))
    proj = torch.randn((64, 8), generator=g).half()
    sampled = torch.randint(0, 4096, (256,), generator=g)
    for s_idx in (None, sampled):
        m = ha.HyperAttention(input_dim=64, proj_dir=proj, sampled_idx=s_idx).to(device="cuda", dtype=torch.float16)
        attn, lse = m(q.cuda(), k.cuda(), v.cuda(), causal=False, return_lse=True)
        assert attn.shape == (1, 4, 4096, 64) and lse.shape == (1, 4, 4096, 1) and lse.dtype == torch.float32
        ro, rl = _oracle(q, k, v, proj, m, False, sampled_idx=s_idx)
        assert_close(attn, ro, "attn", torch.float16)
        assert_close(lse, rl, "lse")
    only = m(q.cuda(), k.cuda(), v.cuda())
    assert torch.equal(only, attn)


@pytest.mark.parametrize("dtype,d,block,sample,smooth", [
    (torch.bfloat16, 128, 512, 512, True),    # benchmark configuration c4 at reduced batch/heads/length
    (torch.float16, 64, 256, 256, True),
    (torch.bfloat16, 64, 128, 128, False),
])
def test_non_causal_variants(ha, dtype, d, block, sample, smooth):
    q, k, v = (_randn((2, 2, 2048, d), s, dtype) for s in (110, 111, 112))
    m, proj = _module(ha, d, dtype, 113, block_size=block, sample_size=sample, smooth_block=smooth)
    attn, lse = m(q.cuda(), k.cuda(), v.cuda(), scale=0.1, return_lse=True)
    ro, rl = _oracle(q, k, v, proj, m, False, scale=0.1)
    assert_close(attn, ro, "attn", dtype, _reference_arithmetic(dtype, q, k, v, proj, m, False, scale=0.1))
    assert_close(lse, rl, "lse")


def test_non_causal_short_sequence_is_exact(ha):
    q, k, v = (_randn((1, 2, 1000, 64), s, torch.float16) for s in (120, 121, 122))
    m, proj = _module(ha, 64, torch.float16, 123)  # min_seq_len 2048 > 1000
    attn, lse = m(q.cuda(), k.cuda(), v.cuda(), return_lse=True)
    ro, rl = O.exact_attention(q, k, v)
    assert_close(attn, ro, "attn", torch.float16)
    assert_close(lse.squeeze(-1), rl, "lse")


# ------------------------------------------------------------------------------- causal
@pytest.mark.parametrize("dtype,d,n,msl,block,sample", [
    (torch.float16, 64, 4096, 512, 256, 256),    # three levels (2048, 1024, 512 halves) + leaves of 512
    (torch.bfloat16, 128, 2048, 256, 256, 128),
    (torch.float16, 64, 2048, 2048, 256, 256),   # top-level leaf: exact causal
    (torch.float16, 64, 3000, 2048, 256, 256),   # one level whose off-diagonal is the exact kernel
])
def test_causal_forward(ha, dtype, d, n, msl, block, sample):
    q, k, v = (_randn((1, 2, n, d), s, dtype) for s in (130, 131, 132))
    m, proj = _module(ha, d, dtype, 133, block_size=block, sample_size=sample, min_seq_len=msl)
    attn, lse = m(q.cuda(), k.cuda(), v.cuda(), causal=True, return_lse=True)
    ro, rl = _oracle(q, k, v, proj, m, True)
    assert attn.shape == (1, 2, n, d)
    assert_close(attn, ro, "attn", dtype, _reference_arithmetic(dtype, q, k, v, proj, m, True))
    if n <= msl:  # the reference returns the exact kernel's padded (b, h, n_rounded) lse here
        assert lse.shape == (1, 2, -(-n // 128) * 128)
        assert_close(lse[:, :, :n], rl.squeeze(-1), "lse")
    else:
        assert lse.shape == (1, 2, n, 1)
        assert_close(lse, rl, "lse")


def _no_composed_path(m, monkeypatch):
    """the module may not fall back to the operator-by-operator recursion"""
    def refuse(*a, **k):
        raise AssertionError("the operator-by-operator recursion ran")
    monkeypatch.setattr(m, "_forward_composed", refuse)


@pytest.mark.parametrize("n,msl,block", [
    (2047, 1024, 256),   # appended row -> 2048 -> halves of 1024: hashed off-diagonal part, exact leaves
    (1001, 600, 256),    # -> 1002 -> halves of 501 < 600: exact off-diagonal part (any length), exact leaves
    (4095, 512, 128),    # three hashed levels (2048, 1024, 512): the appended row is in the last segment of each
    (1537, 1024, 128),   # -> 1538 -> halves of 769: exact, leaves of 769 and 768 rows
])
def test_causal_odd_lengths(ha, monkeypatch, n, msl, block):
    """An odd length runs in the one-call forward (hyper_attention.py:61-64, 94-96): the zero row the reference
    appends is hashed and placed like any other query of the hashed levels (its bucket shifts the blocks of
    the rows behind it) and its result is dropped; the exact parts work on ragged segments."""
    q, k, v = (_randn((1, 2, n, 64), s, torch.float16) for s in (140, 141, 142))
    m, proj = _module(ha, 64, torch.float16, 143, block_size=block, sample_size=128, min_seq_len=msl)
    _no_composed_path(m, monkeypatch)
    attn, lse = m(q.cuda(), k.cuda(), v.cuda(), causal=True, return_lse=True)
    ro, rl = _oracle(q, k, v, proj, m, True)
    assert attn.shape == (1, 2, n, 64) and lse.shape == (1, 2, n, 1)
    assert_close(attn, ro, "attn", torch.float16)
    assert_close(lse, rl, "lse")


@pytest.mark.parametrize("d,dtype,kv_heads", [(128, torch.bfloat16, 1), (64, torch.float16, 2), (128, torch.float16, 2)])
def test_one_call_forward_is_the_same_with_streaming_workgroups(ha, monkeypatch, d, dtype, kv_heads):
    """The whole causal forward with the gathered levels run by workgroups that stream runs of query tiles
    (forced by the library's measurement switch) equals the forward with one tile per workgroup bit for bit:
    an odd length (the last query of the last segment of every hashed level is the appended row, which the
    stream kernel has to drop), resumed partial results at every level, grouped-query heads."""
    n, msl = 9215, 2304   # -> 9216 -> halves of 4608 and 2304: two hashed levels of 18 and 9 tiles per segment
    q = _randn((1, 2, n, d), 160, dtype).cuda()
    k, v = (_randn((1, kv_heads, n, d), s, dtype).cuda() for s in (161, 162))
    m, _ = _module(ha, d, dtype, 163, block_size=256, sample_size=256, min_seq_len=msl)
    _no_composed_path(m, monkeypatch)
    out = {}
    for tiles in (1, 4):
        monkeypatch.setenv("HA_STREAM_TILES", str(tiles))
        attn, lse = m(q, k, v, causal=True, return_lse=True)
        torch.cuda.synchronize()
        out[tiles] = (attn.clone(), lse.clone())
    assert torch.isfinite(out[1][0].float()).all()
    assert torch.equal(out[1][0], out[4][0]) and torch.equal(out[1][1], out[4][1])


def test_causal_odd_length_sort_places_the_appended_row(ha):
    """The query order of every hashed level of an odd length is the stable bucket sort of the segment's rows
    with the appended zero row (bucket of the zero vector: 0) as its last row."""
    from hyperattention_amd import ops
    n, msl = 4095, 512
    q, k = (_randn((1, 2, n, 64), s, torch.float16).cuda() for s in (144, 145))
    m, proj = _module(ha, 64, torch.float16, 146, min_seq_len=msl)
    q_idx, k_idx = ops.forward_sort(q, k, m.lsh.proj_dir, causal=True, lsh_num_projs=8, min_seq_len=msl)
    pad = lambda x: torch.nn.functional.pad(x, (0, 0, 0, 1))
    bq = torch.from_numpy(np.asarray(O.lsh_hash(pad(q.cpu()).double(), proj.double()))).reshape(1, 2, n + 1)
    bk = torch.from_numpy(np.asarray(O.lsh_hash(pad(k.cpu()).double(), proj.double()))).reshape(1, 2, n + 1)
    assert int(bq[0, 0, n]) == 0
    assert len(q_idx) == 3
    for j, half in enumerate((2048, 1024, 512)):
        segs = 1 << j
        want_q = torch.sort(bq.reshape(1, 2 * segs, 2 * half)[:, :, half:], dim=2, stable=True)[1]
        want_k = torch.sort(bk.reshape(1, 2 * segs, 2 * half)[:, :, :half], dim=2, stable=True)[1]
        assert torch.equal(q_idx[j].cpu().long(), want_q), f"level {j} queries"
        assert torch.equal(k_idx[j].cpu().long(), want_k), f"level {j} keys"


def test_causal_composed_path_equals_fused_path(ha):
    q, k, v = (_randn((1, 2, 2048, 64), s, torch.float16).cuda() for s in (150, 151, 152))
    m, _ = _module(ha, 64, torch.float16, 153, min_seq_len=512)
    fused, lse_f = m(q, k, v, causal=True, return_lse=True)
    comp, lse_c = m._forward_composed(q, k, v, 64 ** -0.5, True)
    assert_close(comp, fused, "composed vs fused", torch.float16)
    assert_close(lse_c, lse_f, "composed vs fused lse")


@pytest.mark.parametrize("causal", [False, True])
def test_permuted_views_are_read_in_place(ha, causal):
    """(sq, b, np, hn) tensors seen as (b, np, sq, hn), the layout of the reference's ChatGLM caller
    (chatglm_fast_attention.py:42-58), and grouped-query k/v: same bits as from contiguous copies."""
    n, b, h, hk, d = 2048, 2, 4, 2, 64
    q_s = _randn((n, b, h, d), 170, torch.float16).cuda()
    k_s, v_s = (_randn((n, b, hk, d), s, torch.float16).cuda() for s in (171, 172))
    q, k, v = (x.permute(1, 2, 0, 3) for x in (q_s, k_s, v_s))
    assert not q.is_contiguous()
    m, _ = _module(ha, d, torch.float16, 173, min_seq_len=512)
    got, lse = m(q, k, v, causal=causal, return_lse=True)
    want, wlse = m(q.contiguous(), k.contiguous(), v.contiguous(), causal=causal, return_lse=True)
    assert got.is_contiguous() and torch.equal(got, want) and torch.equal(lse, wlse)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("d,dv", [(96, 96), (32, 32), (40, 72), (64, 128), (128, 64), (100, 100)])
def test_module_other_head_dim(ha, causal, d, dv):
    """Head dims other than 64 and 128, and a value dim apart from the q/k dim: hashed with the module's own
    (d, r) projection; multiples of 8 are read by the kernels as they are, 100 runs zero-padded."""
    q, k = (_randn((1, 2, 2048, d), s, torch.float16) for s in (180, 181))
    v = _randn((1, 2, 2048, dv), 182, torch.float16)
    m, proj = _module(ha, d, torch.float16, 183, min_seq_len=512)
    attn, lse = m(q.cuda(), k.cuda(), v.cuda(), causal=causal, return_lse=True)
    assert attn.shape == (1, 2, 2048, dv) and m.lsh.proj_dir.shape[-2] == d
    ro, rl = _oracle(q, k, v, proj, m, causal)
    assert_close(attn, ro, "attn", torch.float16)
    assert_close(lse, rl, "lse")


@pytest.mark.parametrize("n,msl", [(1001, 600), (2047, 512)])
def test_grouped_query_with_an_odd_length(ha, monkeypatch, n, msl):
    """Grouped-query k/v with an odd length: taken as they are by the one-call forward (the reference needs as
    many k/v heads as q heads, hyper_attention.py:43,67-68: the oracle gets them expanded)."""
    h, hk = 4, 2
    q = _randn((1, h, n, 64), 190, torch.float16)
    k, v = (_randn((1, hk, n, 64), s, torch.float16) for s in (191, 192))
    m, proj = _module(ha, 64, torch.float16, 193, block_size=256, sample_size=128, min_seq_len=msl)
    _no_composed_path(m, monkeypatch)
    attn, lse = m(q.cuda(), k.cuda(), v.cuda(), causal=True, return_lse=True)
    ro, rl = _oracle(q, k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1), proj, m, True)
    assert_close(attn, ro, "attn", torch.float16)
    assert_close(lse, rl, "lse")


def test_top_level_leaf_returns_the_same_lse_shape_with_and_without_grad(ha):
    """n <= min_seq_len under a causal mask: one exact call whose padded 3-d log-sum-exp the reference returns as
    it is (hyper_attention.py:52-58); the shape must not depend on whether gradients are wanted."""
    q, k, v = (_randn((1, 2, 1000, 64), s, torch.float16).cuda() for s in (150, 151, 152))
    m, _ = _module(ha, 64, torch.float16, 153)
    attn, lse = m(q, k, v, causal=True, return_lse=True)
    attn_g, lse_g = m(q.clone().requires_grad_(), k, v, causal=True, return_lse=True)
    assert lse.shape == lse_g.shape == (1, 2, 1024)
    assert torch.equal(attn, attn_g.detach()) and torch.equal(lse[..., :1000], lse_g.detach()[..., :1000])


@pytest.mark.parametrize("causal", [False, True])
def test_more_than_eight_projections_in_one_call(ha, causal):
    """4096 buckets: the one-call forward sorts in two digit passes; against the oracle and the composed path."""
    dtype, n = torch.float16, 4096
    q, k, v = (_randn((1, 2, n, 64), s, dtype) for s in (160, 161, 162))
    m, proj = _module(ha, 64, dtype, 163, lsh_num_projs=12, block_size=128, sample_size=128, min_seq_len=1024)
    attn, lse = m(q.cuda(), k.cuda(), v.cuda(), causal=causal, return_lse=True)
    ro, rl = _oracle(q, k, v, proj, m, causal)
    assert_close(attn, ro, "attn", dtype)
    assert_close(lse, rl, "lse")
    co, cl = m._forward_composed(q.cuda(), k.cuda(), v.cuda(), 64 ** -0.5, causal)
    assert_close(attn, co.double().cpu(), "one call vs composed", dtype)


def test_other_head_dims_leave_the_module_as_it_is(ha):
    q, k, v = (_randn((1, 2, 2048, 32), s, torch.float16).cuda() for s in (170, 171, 172))
    m, _ = _module(ha, 32, torch.float16, 173, min_seq_len=512)
    before = m.lsh.proj_dir.clone()
    m(q, k, v, causal=True)
    assert m.lsh.proj_dir.shape == before.shape and torch.equal(m.lsh.proj_dir, before)


@pytest.mark.parametrize("causal", [False, True])
def test_module_residual_estimator(ha, causal):
    """residual_estimator=True (not in the reference): samples weighted by n_key / sample_size, block keys left out
    of them, in every hashed call of the recursion; against the oracle's option."""
    dtype, n = torch.float16, 2048
    q, k, v = (_randn((1, 2, n, 64), s, dtype) for s in (190, 191, 192))
    m, proj = _module(ha, 64, dtype, 193, block_size=128, sample_size=128, min_seq_len=512, residual_estimator=True)
    attn, lse = m(q.cuda(), k.cuda(), v.cuda(), causal=causal, return_lse=True)
    ro, rl = O.hyper_forward(q, k, v, proj, causal=causal, block_size=128, sample_size=128, min_seq_len=512,
                             residual_estimator=True)
    assert_close(attn, ro, "attn", dtype)
    assert_close(lse, rl, "lse")
    plain, _ = _module(ha, 64, dtype, 193, block_size=128, sample_size=128, min_seq_len=512)
    assert float((plain(q.cuda(), k.cuda(), v.cuda(), causal=causal).float() - attn.float()).abs().max()) > 1e-3
    with pytest.raises(NotImplementedError):
        m(q.cuda().requires_grad_(), k.cuda(), v.cuda(), causal=causal)


def test_random_configurations_against_the_oracle(ha):
    """Seeded random constructor arguments and shapes (block sizes with an odd number of 128-key tiles, no
    samples, smoothed blocks, grouped heads, both head dims and types, 1..10 projections, with and without the
    causal recursion): the module against the oracle, output and log-sum-exp."""
    rng = np.random.default_rng(11)
    for case in range(12):
        d = int(rng.choice([64, 128]))
        dtype = [torch.float16, torch.bfloat16][int(rng.integers(0, 2))]
        causal = bool(rng.integers(0, 2))
        block = 128 * int(rng.integers(1, 5))
        sample = 128 * int(rng.integers(0, 3))
        smooth = bool(rng.integers(0, 2))
        r = int(rng.integers(1, 11))
        hk = int(rng.integers(1, 3))
        h = hk * int(rng.integers(1, 3))
        levels = int(rng.integers(1, 3)) if causal else 0
        leaf = 128 * int(rng.integers(2, 6))
        n = (leaf << levels) if causal else 128 * int(rng.integers(4, 17))
        msl = leaf if causal else int(rng.integers(1, n + 1))
        if causal:
            sample = min(sample, leaf)      # the default sample list must fit the shortest hashed level
        what = (f"case {case}: d {d} {dtype} causal {causal} n {n} min_seq_len {msl} block {block} sample {sample} "
                f"smooth {smooth} r {r} heads {h}/{hk}")
        q = _randn((1, h, n, d), 800 + case, dtype)
        k, v = (_randn((1, hk, n, d), s + case, dtype) for s in (900, 1000))
        m, proj = _module(ha, d, dtype, 1100 + case, lsh_num_projs=r, block_size=block, sample_size=sample,
                          min_seq_len=msl, smooth_block=smooth)
        attn, lse = m(q.cuda(), k.cuda(), v.cuda(), causal=causal, return_lse=True)
        expand = lambda x: x.repeat_interleave(h // hk, dim=1)
        args = (q, expand(k), expand(v), proj, m, causal)
        ro, rl = _oracle(*args)
        assert_close(attn, ro, what + ": attn", dtype, _reference_arithmetic(dtype, *args))
        assert_close(lse, rl, what + ": lse")


def test_module_argument_errors(ha):
    m, _ = _module(ha, 64, torch.float16, 160)
    q = torch.zeros((1, 1, 256, 64), dtype=torch.float16, device="cuda")
    with pytest.raises(AssertionError):
        m(q, q[:, :, :128], q[:, :, :128])            # n_query != n_key
    with pytest.raises(AssertionError):
        m(q.float(), q.float(), q.float())            # fp32 on the GPU path
    with pytest.raises(ValueError):
        ha.HyperAttention(lsh_num_projs=0)
    m2 = ha.HyperAttention(input_dim=64, min_seq_len=128, bogus_keyword=1).to("cuda", torch.float16)
    bad = torch.zeros((1, 1, 192, 64), dtype=torch.float16, device="cuda")
    with pytest.raises(AssertionError):
        m2(bad, bad, bad)                             # hashed path needs n % 128 == 0


# ----------------------------------------------- full-size shapes: size-independent properties
def test_full_size_non_causal_properties(ha):
    """benchmark configuration c2 (batch 1, 32 heads, seq 32768, d 64, fp16): permutations are valid and stable,
    the fused forward equals the operator-by-operator composition, and a sampled head slice matches
    the oracle."""
    b, h, n, d = 1, 32, 32768, 64
    g = torch.Generator(device="cuda").manual_seed(170)
    q, k, v = (torch.randn((b, h, n, d), generator=g, device="cuda", dtype=torch.float16) for _ in range(3))
    m, proj = _module(ha, d, torch.float16, 171)
    attn, lse = m(q, k, v, return_lse=True)
    buckets = m.lsh.hash(q)
    perm = ha.bucket_argsort(buckets)
    sorted_b = torch.gather(buckets.long(), 2, perm)
    assert (sorted_b[:, :, 1:] >= sorted_b[:, :, :-1]).all()
    ties = sorted_b[:, :, 1:] == sorted_b[:, :, :-1]
    assert (perm[:, :, 1:][ties] > perm[:, :, :-1][ties]).all()
    assert torch.equal(torch.sort(perm, dim=2)[0], torch.arange(n, device="cuda").expand(b, h, n))
    comp, lse_c = m.forward_no_causal_mask(q, k, v, d ** -0.5)
    assert torch.equal(comp, attn) and torch.equal(lse_c, lse)
    for head in (0, 17, 31):
        sl = slice(head, head + 1)
        ro, rl = _oracle(q[:, sl].cpu(), k[:, sl].cpu(), v[:, sl].cpu(), proj, m, False)
        assert_close(attn[:, sl], ro, f"attn head {head}", torch.float16)
        assert_close(lse[:, sl], rl, f"lse head {head}")


def test_full_size_causal_properties(ha):
    """benchmark configuration c3 (batch 1, 32 heads, seq 131072, d 64, fp16, causal): the first leaf is exact
    causal attention, lse is finite, heads are independent, and one head matches the oracle."""
    b, h, n, d = 1, 32, 131072, 64
    g = torch.Generator(device="cuda").manual_seed(180)
    q, k, v = (torch.randn((b, h, n, d), generator=g, device="cuda", dtype=torch.float16) for _ in range(3))
    m, proj = _module(ha, d, torch.float16, 181)
    attn, lse = m(q, k, v, causal=True, return_lse=True)
    assert attn.shape == (b, h, n, d) and lse.shape == (b, h, n, 1)
    assert torch.isfinite(attn).all() and torch.isfinite(lse).all()
    # rows of the first leaf (2048) only ever see exact causal attention
    leaf = slice(0, 2048)
    ro, rl = O.exact_attention(q[:, :4, leaf].cpu(), k[:, :4, leaf].cpu(), v[:, :4, leaf].cpu(), None, True)
    assert_close(attn[:, :4, leaf], ro, "first leaf", torch.float16)
    assert_close(lse[:, :4, leaf, 0], rl, "first leaf lse")
    # the result for one head does not depend on the other heads being there
    one, lse_one = m(q[:, 5:6].contiguous(), k[:, 5:6].contiguous(), v[:, 5:6].contiguous(), causal=True,
                     return_lse=True)
    assert torch.equal(one, attn[:, 5:6]) and torch.equal(lse_one, lse[:, 5:6])
    # whole-head parity on a slice of the sequence (the oracle recursion at full length, one head)
    ro, rl = _oracle(q[:, 5:6].cpu(), k[:, 5:6].cpu(), v[:, 5:6].cpu(), proj, m, True)
    assert_close(one, ro, "attn head 5", torch.float16)
    assert_close(lse_one, rl, "lse head 5")
    # the kernels sum a row's P after rounding it to fp16 (the reference sums the fp32 values,
    # src/hyper_attn_triton.py:121-135): the log-sum-exp stays within 1e-3 of the float64 one in absolute terms
    worst = float((lse_one.double().cpu() - rl).abs().max())
    assert worst <= 1e-3, f"|lse - float64 lse| = {worst:.2e}"


@pytest.mark.parametrize("b,h,hk,n,d,msl,causal,r,dtype", [
    (1, 4, 4, 8192, 64, 1024, True, 8, torch.float16),      # leaves of 1024 rows: a unit per leaf
    (2, 4, 2, 16384, 128, 2048, True, 7, torch.bfloat16),   # grouped-query, 7 projections
    (1, 2, 2, 40960, 64, 6000, True, 8, torch.float16),     # leaves of 5120 rows: units of 4096 and 1024
    (1, 2, 1, 12800, 64, 2048, False, 8, torch.float16),    # one segment of units 4096, 4096, 4096, 512
    (1, 2, 2, 8192, 64, 1024, True, 12, torch.float16),     # 4096 buckets: two-digit sort per level
    (1, 1, 1, 262144, 64, 128, True, 4, torch.float16),     # more units per segment than one ranking serves
    (1, 2, 2, 8192, 64, 128, True, 8, torch.float16),       # 32 units of 128 rows in the longest segment
    (1, 2, 2, 16384, 64, 9000, True, 8, torch.float16),     # top level exact, none hashed
])
def test_forward_sort_is_the_stable_sort_of_every_level(ha, b, h, hk, n, d, msl, causal, r, dtype):
    """The orders that the one-call forward works with are, bit for bit, the stable sorts of the bucket ids of
    every level's query and key segment (hyper_attention.py:112-117 inside :51-96)."""
    from hyperattention_amd import ops
    q = _randn((b, h, n, d), 300, dtype).cuda()
    k = _randn((b, hk, n, d), 301, dtype).cuda()
    proj = _randn((1, 1, d, r), 302, dtype).cuda()
    q_idx, k_idx = ops.forward_sort(q, k, proj, causal=causal, lsh_num_projs=r, min_seq_len=msl)
    bq, bk = ops.lsh_hash(q, proj), ops.lsh_hash(k, proj)
    assert len(q_idx) == len(k_idx) and len(q_idx) >= 1
    for level in range(len(q_idx)):
        half = (n >> (level + 1)) if causal else n
        hashed = not (msl > half)
        assert (q_idx[level] is not None) == hashed and (k_idx[level] is not None) == hashed
        if not hashed:
            continue
        if causal:
            want_q = bq.view(b, h << level, 2, half)[:, :, 1].sort(dim=-1, stable=True).indices
            want_k = bk.view(b, hk << level, 2, half)[:, :, 0].sort(dim=-1, stable=True).indices
        else:
            want_q = bq.sort(dim=-1, stable=True).indices
            want_k = bk.sort(dim=-1, stable=True).indices
        assert torch.equal(q_idx[level].long(), want_q), f"query order of level {level}"
        assert torch.equal(k_idx[level].long(), want_k), f"key order of level {level}"
    if causal:
        assert (n >> len(q_idx)) <= msl < (n >> (len(q_idx) - 1))


def test_forward_sort_random_shapes(ha):
    """Seeded random shapes (leaf lengths that are not powers of two, ragged units, skewed buckets from
    clustered rows, 1 to 16 projections): every level's orders equal the stable sort of the library's own ids."""
    from hyperattention_amd import ops
    rng = np.random.default_rng(7)
    for case in range(10):
        levels = int(rng.integers(0, 4))
        leaf = 128 * int(rng.integers(1, 41))            # 128 .. 5120 rows
        n = leaf << levels
        causal = bool(rng.integers(0, 2)) or levels > 0
        r = int(rng.integers(1, 17))
        hk = int(rng.integers(1, 3))
        h = hk * int(rng.integers(1, 3))
        d = int(rng.choice([32, 64, 96, 128]))
        msl = leaf if causal else int(rng.integers(1, n + 1))
        q = _randn((1, h, n, d), 400 + case, torch.float16).cuda()
        k = _randn((1, hk, n, d), 500 + case, torch.float16).cuda()
        if case % 2:   # clustered rows: a few directions plus noise, so that buckets are very uneven
            centres = _randn((1, 1, 4, d), 600 + case, torch.float16).cuda()
            q = (centres[:, :, torch.arange(n, device="cuda") % 4] + 0.05 * q).contiguous()
        proj = _randn((1, 1, d, r), 700 + case, torch.float16).cuda()
        q_idx, k_idx = ops.forward_sort(q, k, proj, causal=causal, lsh_num_projs=r, min_seq_len=msl)
        bq, bk = ops.lsh_hash(q, proj), ops.lsh_hash(k, proj)
        what = f"case {case}: n {n} leaf {leaf} levels {levels} causal {causal} r {r} heads {h}/{hk} d {d}"
        assert len(q_idx) == (levels if causal else 1), what
        for level in range(len(q_idx)):
            half = (n >> (level + 1)) if causal else n
            if msl > half:
                assert q_idx[level] is None, what
                continue
            if causal:
                want_q = bq.view(1, h << level, 2, half)[:, :, 1].sort(dim=-1, stable=True).indices
                want_k = bk.view(1, hk << level, 2, half)[:, :, 0].sort(dim=-1, stable=True).indices
            else:
                want_q, want_k = bq.sort(dim=-1, stable=True).indices, bk.sort(dim=-1, stable=True).indices
            assert torch.equal(q_idx[level].long(), want_q) and torch.equal(k_idx[level].long(), want_k), \
                f"{what}, level {level}"


def _check_sort_properties(ha, buckets):
    """the permutation of every head is a permutation, sorts its keys, and keeps equal keys in row order"""
    b, h, n = buckets.shape
    perm = ha.bucket_argsort(buckets)
    sorted_b = torch.gather(buckets.long(), 2, perm)
    assert (sorted_b[:, :, 1:] >= sorted_b[:, :, :-1]).all()
    ties = sorted_b[:, :, 1:] == sorted_b[:, :, :-1]
    assert (perm[:, :, 1:][ties] > perm[:, :, :-1][ties]).all()
    assert torch.equal(torch.sort(perm, dim=2)[0], torch.arange(n, device="cuda").expand(b, h, n))


def test_full_size_c4_properties(ha):
    """benchmark configuration c4 at full size (batch 2, 32 heads, seq 65536, d 128, bf16, block 512, sample
    512, smooth_block: windows of four 128-key tiles that wrap around at 65536): permutations valid and
    stable on every head, the fused forward equals the operator-by-operator composition bit for bit, and
    one head matches the oracle."""
    b, h, n, d = 2, 32, 65536, 128
    g = torch.Generator(device="cuda").manual_seed(270)
    q, k, v = (torch.randn((b, h, n, d), generator=g, device="cuda", dtype=torch.bfloat16) for _ in range(3))
    m, proj = _module(ha, d, torch.bfloat16, 271, block_size=512, sample_size=512, smooth_block=True)
    attn, lse = m(q, k, v, return_lse=True)
    assert attn.shape == (b, h, n, d) and lse.shape == (b, h, n, 1)
    assert torch.isfinite(attn).all() and torch.isfinite(lse).all()
    _check_sort_properties(ha, m.lsh.hash(q))
    _check_sort_properties(ha, m.lsh.hash(k))
    comp, lse_c = m.forward_no_causal_mask(q, k, v, d ** -0.5)
    assert torch.equal(comp, attn) and torch.equal(lse_c, lse)
    del comp, lse_c
    bi, head = 1, 7
    sl = (slice(bi, bi + 1), slice(head, head + 1))
    qc, kc, vc = q[sl].cpu(), k[sl].cpu(), v[sl].cpu()
    ro, rl = _oracle(qc, kc, vc, proj, m, False)
    assert_close(attn[sl], ro, "attn batch 1 head 7", torch.bfloat16,
                 _reference_arithmetic(torch.bfloat16, qc, kc, vc, proj, m, False))
    assert_close(lse[sl], rl, "lse batch 1 head 7")


def _clustered(b, hq, hkv, n, d, seed):
    """benchmark configuration c5 inputs: keys = 4 x one of 64 unit-norm centroids + N(0, 0.5^2) noise, queries
    from the same centroids with their own noise, values N(0,1); bf16"""
    g = _gen(seed)
    cent = torch.nn.functional.normalize(torch.randn((64, d), generator=g), dim=-1)
    kc = torch.randint(0, 64, (b, hkv, n), generator=g)
    qc = torch.randint(0, 64, (b, hq, n), generator=g)
    k = (4 * cent[kc] + 0.5 * torch.randn((b, hkv, n, d), generator=g)).bfloat16()
    q = (4 * cent[qc] + 0.5 * torch.randn((b, hq, n, d), generator=g)).bfloat16()
    v = torch.randn((b, hkv, n, d), generator=g).bfloat16()
    return q, k, v


def test_full_size_c5_properties(ha):
    """benchmark configuration c5 at full size (32 query heads on 2 KV heads, seq 32768, d 128, bf16, causal,
    min_seq_len 2048: four levels + leaves; clustered keys, so the buckets are filled unevenly):
    the native grouped call equals the call on expanded K/V bit for bit, permutations are valid under the
    skew, and two query heads of different groups match the oracle."""
    from hyperattention_amd import ops
    b, hq, hkv, n, d = 1, 32, 2, 32768, 128
    q, k, v = _clustered(b, hq, hkv, n, d, 290)
    m, proj = _module(ha, d, torch.bfloat16, 291)
    qg, kg, vg = q.cuda(), k.cuda(), v.cuda()
    native, lse_n = ops.hyper_forward(qg, kg, vg, m.lsh.proj_dir, scale=d ** -0.5, causal=True, lsh_num_projs=8,
                                      block_size=256, sample_size=256, min_seq_len=2048, smooth_block=False)
    group = hq // hkv
    attn, lse = m(qg, kg.repeat_interleave(group, dim=1), vg.repeat_interleave(group, dim=1), causal=True,
                  return_lse=True)
    assert torch.equal(native, attn) and torch.equal(lse_n.unsqueeze(-1), lse)
    assert torch.isfinite(attn).all() and torch.isfinite(lse).all()
    buckets = m.lsh.hash(kg)
    counts = torch.bincount(buckets[0, 0].long(), minlength=256)
    assert counts.max() > 1.5 * n / 256, "clustered keys fill the buckets unevenly"
    _check_sort_properties(ha, buckets)
    _check_sort_properties(ha, m.lsh.hash(qg))
    for head in (3, 20):  # query heads of KV group 0 and 1
        sl = slice(head, head + 1)
        kv = slice(head // group, head // group + 1)
        ro, rl = _oracle(q[:, sl], k[:, kv], v[:, kv], proj, m, True)
        assert_close(attn[:, sl], ro, f"attn head {head}", torch.bfloat16,
                     _reference_arithmetic(torch.bfloat16, q[:, sl], k[:, kv], v[:, kv], proj, m, True))
        assert_close(lse[:, sl], rl, f"lse head {head}")


@pytest.mark.parametrize("n,h,d,causal,dtype", [(1 << 20, 24, 64, True, torch.bfloat16),
                                                (1 << 19, 20, 128, False, torch.float16)])
def test_heads_far_into_large_tensors_equal_the_heads_computed_alone(ha, n, h, d, causal, dtype):
    """Sequences of 2^20 and 2^19 rows: the last heads of q, k, v start more than 2^31 bytes into their tensors
    (row numbers and byte offsets beyond 32 bits).  A head's result inside the big call equals, bit for bit, the
    result of the same head in a call of its own."""
    g = torch.Generator(device="cuda").manual_seed(230)
    q, k, v = (torch.randn((1, h, n, d), generator=g, device="cuda", dtype=dtype) for _ in range(3))
    assert q[0, h - 1].data_ptr() - q.data_ptr() > 1 << 31
    m, _ = _module(ha, d, dtype, 231, min_seq_len=4096)
    out, lse = m(q, k, v, causal=causal, return_lse=True)
    for head in (0, h // 2, h - 1):
        sl = slice(head, head + 1)
        o1, l1 = m(q[:, sl].contiguous(), k[:, sl].contiguous(), v[:, sl].contiguous(), causal=causal, return_lse=True)
        assert torch.isfinite(o1.float()).all()
        assert torch.equal(out[:, sl], o1) and torch.equal(lse[:, sl], l1), head


def test_grouped_query_heads(ha):
    """benchmark configuration c5 shape family (32 query heads on 2 KV heads, d 128, bf16, causal, clustered
    keys) at reduced length: the expanded-KV module call matches the oracle, and the native grouped
    call (K/V not expanded) gives bit-identical results."""
    from hyperattention_amd import ops
    b, hq, hkv, n, d = 1, 8, 2, 4096, 128
    g = _gen(190)
    cent = torch.nn.functional.normalize(torch.randn((64, d), generator=g), dim=-1)
    kc = torch.randint(0, 64, (b, hkv, n), generator=g)
    qc = torch.randint(0, 64, (b, hq, n), generator=g)
    k = (4 * cent[kc] + 0.5 * torch.randn((b, hkv, n, d), generator=g)).bfloat16()
    q = (4 * cent[qc] + 0.5 * torch.randn((b, hq, n, d), generator=g)).bfloat16()
    v = torch.randn((b, hkv, n, d), generator=g).bfloat16()
    k_exp = k.repeat_interleave(hq // hkv, dim=1)
    v_exp = v.repeat_interleave(hq // hkv, dim=1)
    m, proj = _module(ha, d, torch.bfloat16, 191, min_seq_len=1024)
    attn, lse = m(q.cuda(), k_exp.cuda(), v_exp.cuda(), causal=True, return_lse=True)
    ro, rl = _oracle(q, k_exp, v_exp, proj, m, True)
    assert_close(attn, ro, "attn", torch.bfloat16, _reference_arithmetic(torch.bfloat16, q, k_exp, v_exp, proj, m, True))
    assert_close(lse, rl, "lse")
    native, lse_n = ops.hyper_forward(q.cuda(), k.cuda(), v.cuda(), m.lsh.proj_dir, scale=d ** -0.5, causal=True,
                                      lsh_num_projs=8, block_size=256, sample_size=256, min_seq_len=1024,
                                      smooth_block=False)
    assert torch.equal(native, attn) and torch.equal(lse_n.unsqueeze(-1), lse)


def test_forward_is_capturable_in_a_hip_graph(ha):
    # The library neither allocates, nor synchronises, nor records memsets: one forward (hash, sorts,
    # leaves, levels) can be captured into a HIP graph and replayed on new data.  Every replay is
    # compared with the eager result, with eager work and synchronisations between the replays.
    dtype, b, h, n, d = torch.float16, 1, 4, 4096, 64
    m = ha.HyperAttention(input_dim=d, block_size=256, sample_size=256, min_seq_len=1024, rng=_gen(90)).to(
        device="cuda", dtype=dtype)
    q, k, v = (_randn((b, h, n, d), 91 + i, dtype).cuda() for i in range(3))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up on a side stream, as graph capture asks for
        for _ in range(2):
            m(q, k, v, causal=True)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = m(q, k, v, causal=True)
    for it in range(3):
        fresh = [_randn((b, h, n, d), 100 + 3 * it + i, dtype).cuda() for i in range(3)]
        for dst, src in zip((q, k, v), fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        want = m(*fresh, causal=True)
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {it} differs from the eager forward"
