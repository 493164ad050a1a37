"""CPU oracle for the HyperAttention forward path.

TEST INFRASTRUCTURE ONLY.  This module restates, on the CPU, the algorithm of the
reference's forward path so that the HIP kernels can be checked against it.  Only the
test-suite, the smoke check and the benchmark's ``cpu_baseline`` leg may import it; the
product package never does.

Every function cites the reference lines it follows (paths relative to the reference
checkout).  How each function is pinned (none of them by re-typing its own formula):

==========================  =====================================================================
function                    pinned by (tests/test_oracle_*.py)
==========================  =====================================================================
gray_lut                    closed form ``i ^ (i >> 1)``; neighbours differ in exactly one bit
lsh_hash                    exact rational arithmetic (fractions) on small inputs; scale and
                            negation invariants; committed golden vectors
stable_bucket_argsort       brute-force O(n^2) stable ranking; permutation/sortedness invariants
gather_rows                 per-element python loop
exact_attention             torch.nn.functional.scaled_dot_product_attention; per-row python loop
block_sampled_attention     reduces to exact_attention for block_size = n, sample 0; equals
                            lse-merge of (block only, sampled only); brute-force per-row python
                            loop on tiny sizes, incl. smooth_block windows
add_self_attentions         merging attention over two disjoint key sets == attention over union
hyper_forward               min_seq_len >= n -> exact causal; one-level split with block = n/2
                            -> exact causal; brute-force row-by-row definition on tiny sizes
round_dtype (reference      equals the un-rounded result exactly for float64, converges to it as the
arithmetic mode)            type widens (bf16 > fp16 > fp32), error within the type's rounding bound
gradients (torch autograd   central finite differences of the same functions in float64; the
of the functions above)     closed formulas dV = P^T dO, dS = P (dP - D) scale, dQ = dS K,
                            dK = dS^T Q written out per (query, key) pair on tiny sizes
==========================  =====================================================================

Parity unpinned (no reference test or fixture fixes it, tolerance comes from the stated
2e-3 bound): the exact rounding of the reference's Triton ``tl.dot``/``tl.exp`` and of
``torch.sort`` as a third-party routine (pinned here by the definition of a stable sort).
"""
from __future__ import annotations

import math
from fractions import Fraction

import numpy as np
import torch

TILE = 128  # query/key tile edge of the reference kernels (src/hyper_attn_triton.py:694)


# ----------------------------------------------------------------------------- hashing
def gray_lut(num_projs: int) -> np.ndarray:
    """Reflected Gray-code table ``perm`` of length 2**num_projs (int32).

    Follows src/angular_lsh_triton.py:168-173: a(1) = [0, 1];
    a(n) = a(n-1) ++ (reverse(a(n-1)) + 2**(n-1)).
    """
    if num_projs <= 0:
        raise ValueError("Invalid value for num_projs")  # src/angular_lsh_triton.py:166
    table = [0, 1]
    for bit in range(1, num_projs):
        table = table + [x + (1 << bit) for x in reversed(table)]
    return np.asarray(table, dtype=np.int32)


def _exact_sign_positive(x_row: np.ndarray, p_col: np.ndarray) -> bool:
    """Sign of the exact (rational) dot product; used only when fp64 cannot decide."""
    acc = Fraction(0)
    for a, b in zip(x_row.tolist(), p_col.tolist()):
        acc += Fraction(a) * Fraction(b)
    return acc > 0


def lsh_projection_bits(x: np.ndarray, proj: np.ndarray) -> np.ndarray:
    """Boolean (..., n, r): ``x @ proj > 0`` with the sign of the *exact* dot product.

    Follows src/angular_lsh_triton.py:76-78 (kernel) and :176-177 (torch form).  Inputs are
    fp16/bf16/fp32 values held in float64, so every product is exact in float64; the sum is
    accumulated in float64 and any entry too close to zero for float64 to decide is re-done
    in rational arithmetic.
    """
    x64 = np.asarray(x, dtype=np.float64)
    p64 = np.asarray(proj, dtype=np.float64)
    d = x64.shape[-1]
    acc = x64 @ p64
    # bound on the float64 summation error, any order: d * 2^-53 * sum |x_k p_kj|
    mag = np.abs(x64) @ np.abs(p64)
    unsure = np.abs(acc) <= (2.0 * d * 2.0 ** -53) * mag
    bits = acc > 0
    if unsure.any():
        flat_x = x64.reshape(-1, d)
        flat_bits = bits.reshape(-1, bits.shape[-1])
        # broadcast projections: support a shared (d, r) matrix only on this slow path
        rows, cols = np.nonzero(unsure.reshape(-1, unsure.shape[-1]))
        p2 = p64.reshape(-1, d, p64.shape[-1])
        for i, j in zip(rows.tolist(), cols.tolist()):
            pm = p2[0] if p2.shape[0] == 1 else p2[i // (flat_x.shape[0] // p2.shape[0])]
            flat_bits[i, j] = _exact_sign_positive(flat_x[i], pm[:, j])
    return bits


def lsh_hash(x, proj) -> np.ndarray:
    """Angular-LSH bucket ids, int32, shape ``x.shape[:-1]``.

    Follows src/angular_lsh_triton.py:175-179 (``hash_torch``) and :76-88 (kernel):
    bit_j = [x . P[:, j] > 0]; bin = sum_j bit_j * 2**j; bucket = perm[bin].
    ``proj`` has shape (d, r) or broadcastable (..., d, r) as at :103.
    """
    x = _to_numpy64(x)
    proj = _to_numpy64(proj)
    r = proj.shape[-1]
    bits = lsh_projection_bits(x, proj)
    enc = (1 << np.arange(r, dtype=np.int64))  # enc_vec, src/angular_lsh_triton.py:164
    bin_ids = (bits.astype(np.int64) * enc).sum(-1)
    return gray_lut(r)[bin_ids]


# ------------------------------------------------------------------------ sort / gather
def stable_bucket_argsort(buckets) -> np.ndarray:
    """Stable argsort along the last axis (ties keep ascending index), int64.

    Follows the call sites hyper_attention.py:116-117 (``torch.sort(..., dim=2, stable=True)``).
    """
    b = np.asarray(_to_numpy(buckets))
    return np.argsort(b, axis=-1, kind="stable").astype(np.int64)


def gather_rows(x, idx, chunk_size: int = -1):
    """out[b, h, s, :] = x[b, h, idx[b, h, s], :], optionally zero-padded to a chunk multiple.

    Follows src/attn_utils.py:27-50 (``indexing``).
    """
    xt = torch.as_tensor(x)
    it = torch.as_tensor(np.asarray(_to_numpy(idx))).long()
    out = torch.gather(xt, 2, it.unsqueeze(-1).expand(-1, -1, -1, xt.shape[-1]))
    if chunk_size > 0 and xt.shape[-2] % chunk_size != 0:
        new_n = math.ceil(out.shape[2] / chunk_size) * chunk_size
        out = torch.nn.functional.pad(out, (0, 0, 0, new_n - out.shape[2]))
    return out


# --------------------------------------------------------------------------- attention
def _lse_dtype(round_dtype):
    """The reference's kernels store their log-sum-exps in float32 (src/hyper_attn_triton.py:688,
    src/flash_attn_triton.py:826); float64 stays float64 so that the mode can be checked against the
    un-rounded functions."""
    return torch.float64 if round_dtype == torch.float64 else torch.float32


def _round_p(p, round_dtype, dtype):
    """P as the reference's kernels hand it to the P.V product: rounded to the value type
    (src/hyper_attn_triton.py:135,167 and src/flash_attn_triton.py:233: ``p.to(v.dtype)``)."""
    return p if round_dtype is None else p.to(round_dtype).to(dtype)


def exact_attention(q, k, v, scale=None, causal=False, dtype=torch.float64, q_chunk=1024, round_dtype=None):
    """Exact softmax attention and log-sum-exp.  (b,h,n,d) layout.

    Follows src/flash_attn_triton.py:149 (causal loop bound), :171-177 (scores, mask
    ``row >= col``), :236-241 (lse) — the same function without tiling.
    Returns out (b,h,nq,dv) and lse (b,h,nq), both in ``dtype``.

    ``round_dtype`` (torch.float16 / torch.bfloat16) switches on the reference kernels' own
    roundings: the un-normalised P = exp(s - row max) is rounded to that type before P.V (:233), the
    row sum is taken over the un-rounded P (:222), and the output is stored in that type (:259-267);
    out is then returned as a tensor of ``round_dtype`` and lse as float32 (:826).  The reference's
    running maximum differs from the row maximum by a factor that is not a power of two, so its
    roundings are these only in distribution, not value by value.
    """
    q = torch.as_tensor(q).to(dtype)
    k = torch.as_tensor(k).to(dtype)
    v = torch.as_tensor(v).to(dtype)
    d = q.shape[-1]
    scale = scale or 1.0 / math.sqrt(d)  # src/flash_attn_triton.py:805
    nq, nk = q.shape[2], k.shape[2]
    out = torch.empty(q.shape[:3] + (v.shape[-1],), dtype=dtype)
    lse = torch.empty(q.shape[:3], dtype=dtype)
    cols = torch.arange(nk)
    for s in range(0, nq, q_chunk):
        e = min(s + q_chunk, nq)
        ke = min(e, nk) if causal else nk
        scores = torch.matmul(q[:, :, s:e], k[:, :, :ke].transpose(-1, -2)) * scale
        if causal:
            rows = torch.arange(s, e)
            scores = scores.masked_fill(rows[:, None] < cols[None, :ke], float("-inf"))
        l = torch.logsumexp(scores, dim=-1)
        lse[:, :, s:e] = l
        if round_dtype is None:
            out[:, :, s:e] = torch.matmul(torch.exp(scores - l.unsqueeze(-1)), v[:, :, :ke])
        else:
            m = scores.max(dim=-1, keepdim=True).values
            p = torch.exp(scores - m)
            out[:, :, s:e] = torch.matmul(_round_p(p, round_dtype, dtype), v[:, :, :ke]) / p.sum(-1, keepdim=True)
    if round_dtype is not None:
        return out.to(round_dtype), lse.to(_lse_dtype(round_dtype))
    return out, lse


def block_key_positions(n_q: int, n_k: int, block_size: int, smooth_block: bool):
    """Sorted-key positions visited by each 128-row tile of sorted queries.

    Follows src/hyper_attn_triton.py:99-109 with ``block_size`` already divided by 128 as at
    :726.  Returns (pos, valid): int64 (tiles, T*128) and bool mask of the same shape.
    When the block is so much longer than the sequence that (T-1)*64 > n_k the reference's offset
    goes negative before its remainder (outside what it was written for); the mathematical modulo is
    used here, and by the HIP kernel.
    """
    T = -(-block_size // TILE)
    tiles = -(-n_q // TILE)
    pos = np.zeros((tiles, T * TILE), dtype=np.int64)
    valid = np.zeros((tiles, T * TILE), dtype=bool)
    offs = np.arange(TILE, dtype=np.int64)
    for t in range(tiles):
        block_id = t // T
        block_offs = n_k + (t % T) * TILE - ((T - 1) * TILE) // 2
        end_n = min((block_id + 1) * TILE * T, n_k)
        for i, start_n in enumerate(range(block_id * TILE * T, end_n, TILE)):
            if smooth_block:
                p = (start_n + block_offs + offs) % n_k
            else:
                p = start_n + offs
            pos[t, i * TILE:(i + 1) * TILE] = p
            valid[t, i * TILE:(i + 1) * TILE] = True
    return pos, valid


def block_sampled_attention(q, k, v, q_sort_idx, k_sort_idx, block_size, sample_size=0,
                            scale=None, smooth_block=False, sampled_idx=None,
                            dtype=torch.float64, round_dtype=None, sample_bias=0.0,
                            mask_sampled_in_block=False):
    """Sorted block-diagonal + fixed-column attention, (b,h,n,d) layout.

    Follows src/hyper_attn_triton.py:70-192 (``_fwd_hyper_kernel``): tile ``t`` of 128 sorted
    queries attends to the sorted keys of its block (:99-141) and then to the sampled key
    rows (:142-173) under one running soft-max; results are scattered to the queries'
    original rows (:176-192).  The sampled rows are the explicit list ``sampled_idx`` (key
    rows in original order, shared by all queries; shape (s,) or (b,h,s)); the default
    ``arange(sample_size)`` is what the backward kernel (:576-581) and
    unit_tests/test_hyper_attention.py:65-67,200-201 use.  No n/s weighting, no removal of
    columns already in the block.
    Returns out (b,h,nq,dv) and lse (b,h,nq) in ``dtype``.  ``round_dtype``: the kernel's own
    roundings as in exact_attention (P to the value type before both P.V products, :135 and :167;
    out stored in that type, :189-192; lse float32, :688).
    ``sample_bias`` / ``mask_sampled_in_block`` (NOT in the reference; the residual estimator of the
    HyperAttention paper): the bias is added to the scaled score of every sampled key (log of the weight a
    sample carries in the soft-max sums), and with the mask a sampled key that is among the valid block
    keys of the query's tile is left out of the sampled part.  Pinned by the per-row definition in
    tests/test_oracle.py.
    """
    q = torch.as_tensor(q).to(dtype)
    k = torch.as_tensor(k).to(dtype)
    v = torch.as_tensor(v).to(dtype)
    b, h, nq, d = q.shape
    nk = k.shape[2]
    dv = v.shape[-1]
    scale = scale or 1.0 / math.sqrt(d)  # src/hyper_attn_triton.py:686
    assert sample_size % TILE == 0  # src/hyper_attn_triton.py:911
    assert nk % TILE == 0 and nq % TILE == 0  # :695 and the comment at :24
    qi = torch.as_tensor(np.asarray(_to_numpy(q_sort_idx))).long()
    ki = torch.as_tensor(np.asarray(_to_numpy(k_sort_idx))).long()
    if sampled_idx is None:
        sampled_idx = np.arange(sample_size)
    si = torch.as_tensor(np.asarray(_to_numpy(sampled_idx))).long()
    if si.dim() == 1:
        si = si.view(1, 1, -1).expand(b, h, -1)
    assert si.shape[-1] == sample_size

    pos_np, valid_np = block_key_positions(nq, nk, block_size, smooth_block)
    pos = torch.from_numpy(pos_np)
    valid = torch.from_numpy(valid_np)
    tiles, width = pos.shape

    out = torch.empty((b, h, nq, dv), dtype=dtype)
    lse = torch.empty((b, h, nq), dtype=dtype)
    for ib in range(b):
        for ih in range(h):
            qs = q[ib, ih][qi[ib, ih]].view(tiles, TILE, d)
            krow = ki[ib, ih][pos]                      # (tiles, width) original key rows
            kg = k[ib, ih][krow]                        # (tiles, width, d)
            vg = v[ib, ih][krow]
            s_blk = torch.matmul(qs, kg.transpose(-1, -2)) * scale
            s_blk = s_blk.masked_fill(~valid[:, None, :], float("-inf"))
            if sample_size > 0:
                ks = k[ib, ih][si[ib, ih]]
                vs = v[ib, ih][si[ib, ih]]
                s_smp = torch.matmul(qs, ks.t()) * scale + sample_bias
                if mask_sampled_in_block:
                    # (tiles, width, s): sampled row j equals valid block key w of tile t
                    same = (krow[:, :, None] == si[ib, ih][None, None, :]) & valid[:, :, None]
                    s_smp = s_smp.masked_fill(same.any(dim=1)[:, None, :], float("-inf"))
                scores = torch.cat([s_blk, s_smp], dim=-1)
            else:
                scores = s_blk
            l = torch.logsumexp(scores, dim=-1)
            if round_dtype is None:
                p = torch.exp(scores - l.unsqueeze(-1))
                norm = 1.0
            else:
                p_full = torch.exp(scores - scores.max(dim=-1, keepdim=True).values)
                norm = p_full.sum(-1, keepdim=True)
                p = _round_p(p_full, round_dtype, dtype)
            o = torch.matmul(p[..., :width], vg)
            if sample_size > 0:
                o = o + torch.matmul(p[..., width:], vs)
            o = o / norm
            out[ib, ih][qi[ib, ih]] = o.view(nq, dv)
            lse[ib, ih][qi[ib, ih]] = l.view(nq)
    if round_dtype is not None:
        return out.to(round_dtype), lse.to(_lse_dtype(round_dtype))
    return out, lse


def add_self_attentions(attn1, lse1, attn2, lse2):
    """Merge two partial attentions over disjoint key sets.

    Follows src/attn_utils.py:21-23 line by line, including the cast of ``c`` to the dtype of
    ``attn1`` and the ``+ eps`` inside the log.  Shapes: attn (b,h,n,d), lse (b,h,n,1).
    """
    c = (1 / (1 + (lse2 - lse1).exp())).to(dtype=attn1.dtype)
    attn = c * attn1 + (1 - c) * attn2
    lse = lse1 - (c + torch.finfo(lse1.dtype).eps).log()
    return attn, lse


def forward_no_causal_mask(q, k, v, scale, proj, lsh_num_projs, block_size, sample_size,
                           min_seq_len, smooth_block, sampled_idx=None, dtype=torch.float64,
                           detach_lse=False, round_dtype=None, residual_estimator=False):
    """Follows hyper_attention.py:103-132.  Returns attn (b,h,n,dv), lse (b,h,n,1).
    ``residual_estimator`` (not in the reference): the hashed call weights its samples by
    n_key / sample_size and leaves out those that lie in the query's block (block_sampled_attention)."""
    n_query = q.shape[2]
    if min_seq_len > n_query:  # :109
        attn, lse = exact_attention(q, k, v, scale, False, dtype, round_dtype=round_dtype)
    else:
        q_idx = stable_bucket_argsort(lsh_hash(q, proj))  # :116
        k_idx = stable_bucket_argsort(lsh_hash(k, proj))  # :117
        est = dict(sample_bias=math.log(k.shape[2] / sample_size), mask_sampled_in_block=True) \
            if residual_estimator and sample_size > 0 else {}
        attn, lse = block_sampled_attention(q, k, v, q_idx, k_idx, block_size, sample_size,
                                            scale, smooth_block, sampled_idx, dtype, round_dtype=round_dtype, **est)
    if detach_lse:
        lse = lse.detach()
    return attn, lse.unsqueeze(-1)


def hyper_forward(q, k, v, proj, scale=None, causal=False, lsh_num_projs=8, block_size=256,
                  sample_size=256, min_seq_len=2048, smooth_block=False, sampled_idx=None,
                  dtype=torch.float64, detach_lse=False, round_dtype=None, residual_estimator=False):
    """HyperAttention.forward with return_lse=True, (b,h,n,d) layout.

    Follows hyper_attention.py:25-101: non-causal dispatch (:48-49), causal leaf (:52-57),
    pad-if-odd (:61-64), halves-as-heads (:67-69), recursion (:71), un-masked off-diagonal
    call on (second-half queries, first-half keys/values) (:82-84), merge of the lower half
    (:86-89), concatenation and un-padding (:91-96).  ``proj`` is the (d, r) projection
    matrix (already rounded to the input precision); ``sampled_idx`` indexes rows *within the
    key tensor handed to each un-masked call*.  lse is always returned as (b,h,n,1).

    Gradients (torch autograd differentiates this function as it stands).  ``detach_lse=True``
    gives the gradient the reference's autograd computes: its attention operators return no
    gradient for their log-sum-exp output (src/hyper_attn_triton.py:922-945,
    src/flash_attn_triton.py:1014-1040), so every log-sum-exp entering a merge is a constant there.

    ``round_dtype`` (torch.float16 / torch.bfloat16): the reference's own arithmetic instead of
    ``dtype`` throughout: the attention operators round P and their outputs to that type (see
    exact_attention), their log-sum-exps are float32, and the merges then run on tensors of that type,
    so that add_self_attentions rounds the weight c and every product and sum (src/attn_utils.py:21-23).
    """
    q = torch.as_tensor(q).to(dtype)
    k = torch.as_tensor(k).to(dtype)
    v = torch.as_tensor(v).to(dtype)
    n_query = q.shape[2]
    b, h, n_key, dim = k.shape
    scale = scale or dim ** (-0.5)  # :44
    assert n_query == n_key  # :45
    kw = dict(proj=proj, lsh_num_projs=lsh_num_projs, block_size=block_size,
              sample_size=sample_size, min_seq_len=min_seq_len, smooth_block=smooth_block,
              sampled_idx=sampled_idx, dtype=dtype, detach_lse=detach_lse, round_dtype=round_dtype,
              residual_estimator=residual_estimator)
    if causal is False:
        return forward_no_causal_mask(q, k, v, scale, **kw)
    if n_key <= min_seq_len:  # :52
        attn, lse = exact_attention(q, k, v, scale, True, dtype, round_dtype=round_dtype)
        if detach_lse:
            lse = lse.detach()
        return attn, lse.unsqueeze(-1)
    if n_query % 2:  # :61-64
        q = torch.nn.functional.pad(q, (0, 0, 0, 1))
        k = torch.nn.functional.pad(k, (0, 0, 0, 1))
        v = torch.nn.functional.pad(v, (0, 0, 0, 1))
    n = q.shape[2]
    half = n // 2
    q_bd = q.reshape(b, 2 * h, half, q.shape[-1])
    k_bd = k.reshape(b, 2 * h, half, k.shape[-1])
    v_bd = v.reshape(b, 2 * h, half, v.shape[-1])
    attn_bd, lse_bd = hyper_forward(q_bd, k_bd, v_bd, scale=scale, causal=True, **kw)
    attn_bd = attn_bd.reshape(b, h, n, -1)
    lse_bd = lse_bd.reshape(b, h, n, 1)
    attn_un, lse_un = forward_no_causal_mask(q[:, :, half:], k[:, :, :half], v[:, :, :half],
                                             scale, **kw)  # :82-84
    attn_dn, lse_dn = add_self_attentions(attn_bd[:, :, half:], lse_bd[:, :, half:],
                                          attn_un, lse_un)  # :87-89
    attn = torch.cat((attn_bd[:, :, :half], attn_dn), dim=-2)
    lse = torch.cat((lse_bd[:, :, :half], lse_dn), dim=-2)
    if n_query % 2:
        attn = attn[:, :, :-1]
        lse = lse[:, :, :-1]
    return attn, lse


# ------------------------------------------------------------------------------ helpers
def _to_numpy(a):
    if isinstance(a, torch.Tensor):
        return a.detach().cpu().numpy() if a.dtype != torch.bfloat16 else a.detach().cpu().float().numpy()
    return a


def _to_numpy64(a) -> np.ndarray:
    if isinstance(a, torch.Tensor):
        return a.detach().cpu().to(torch.float64).numpy()
    return np.asarray(a, dtype=np.float64)
