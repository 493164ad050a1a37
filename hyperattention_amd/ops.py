"""Operator layer: the reference's L2 functions (same names, argument order and layouts), each a thin
shim that checks its tensors and hands raw device pointers to one C symbol of libhyperattn.so.

Reference interfaces mirrored here:
  hash            <- AngularLSHTriton.hash_triton           src/angular_lsh_triton.py:99-145,181-182
  bucket_argsort  <- torch.sort(..., dim=2, stable=True)[1] hyper_attention.py:116-117
  indexing        <- indexing                               src/attn_utils.py:27-50
  hyper_attn_func <- hyper_attn_func                        src/hyper_attn_triton.py:668-742,895-945
  flash_attn_func <- flash_attn_func (no bias)              src/flash_attn_triton.py:795-872,995-1040
  add_self_attentions <- add_self_attentions                src/attn_utils.py:6-24
The two attention operators are differentiable in q, k, v (HyperAttnFunc, FlashAttnFunc below: torch
autograd functions over ha_block_attn_bwd / ha_flash_attn_bwd), as the reference's are.
"""
from __future__ import annotations

import ctypes
import math

import torch

from . import _lib
from ._lib import AttnGrads, HA_BF16, HA_F16, HA_IDX_I32, HA_IDX_I64, AttnOperands, BlockAttnArgs, ForwardArgs


def _dtype_code(t: torch.Tensor) -> int:
    assert t.dtype in (torch.float16, torch.bfloat16), "Only support fp16 and bf16"
    return HA_F16 if t.dtype == torch.float16 else HA_BF16


def _idx_code(t: torch.Tensor) -> int:
    assert t.dtype in (torch.int32, torch.int64), "index tensors must be int32 or int64"
    return HA_IDX_I32 if t.dtype == torch.int32 else HA_IDX_I64


def _stream(t: torch.Tensor):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


# ------------------------------------------------------------------------------------- hash
def lsh_hash(mat: torch.Tensor, proj_dir: torch.Tensor) -> torch.Tensor:
    """int32 bucket ids (b,h,n) of mat (b,h,n,d); proj_dir is (b,h,d,r) or (1,1,d,r)."""
    batch, nheads, seqlen, d = mat.shape
    num_projs = proj_dir.shape[-1]
    assert proj_dir.shape == (batch, nheads, d, num_projs) or proj_dir.shape == (1, 1, d, num_projs)
    assert mat.dtype == proj_dir.dtype, "All three tensors must have the same type"
    assert mat.dtype in (torch.float16, torch.bfloat16), "Only support fp16 and bf16"
    assert mat.is_cuda and proj_dir.is_cuda
    if mat.stride(-1) != 1:
        mat = mat.contiguous()
    proj_dir = proj_dir.contiguous()
    if proj_dir.shape[:2] == (1, 1):
        psb, psh = 0, 0
    else:
        psb, psh = proj_dir.stride(0), proj_dir.stride(1)
    buckets = torch.empty((batch, nheads, seqlen), device=mat.device, dtype=torch.int32)
    with torch.cuda.device(mat.device):
        _lib.check(_lib.lib().ha_lsh_hash(
            _ptr(mat), _ptr(proj_dir), _ptr(buckets), batch, nheads, seqlen, d, num_projs,
            mat.stride(0), mat.stride(1), mat.stride(2), psb, psh, _dtype_code(mat), _stream(mat)))
    return buckets


# ------------------------------------------------------------------------------------- sort
def bucket_argsort(buckets: torch.Tensor, num_keys: int = 256, out_dtype=torch.int64) -> torch.Tensor:
    """Stable argsort along the last dim of int32 keys in [0, num_keys); (b,h,n) -> (b,h,n)."""
    assert buckets.is_cuda and buckets.dtype == torch.int32
    buckets = buckets.contiguous()
    n = buckets.shape[-1]
    segs = buckets.numel() // n
    out = torch.empty(buckets.shape, device=buckets.device, dtype=out_dtype)
    L = _lib.lib()
    ws_bytes = L.ha_bucket_argsort_workspace_bytes(segs, n, num_keys)
    ws = torch.empty(max(int(ws_bytes), 256), device=buckets.device, dtype=torch.uint8)
    with torch.cuda.device(buckets.device):
        _lib.check(L.ha_bucket_argsort(_ptr(buckets), _ptr(out), _idx_code(out), segs, n, n, 0, num_keys,
                                       _ptr(ws), ws.numel(), _stream(buckets)))
    return out


# ----------------------------------------------------------------------------------- gather
def indexing(x: torch.Tensor, indices: torch.Tensor, chunk_size: int = -1) -> torch.Tensor:
    """out[b,h,s] = x[b,h,indices[b,h,s]]; rows zero-padded up to a multiple of chunk_size when
    x.shape[2] is not one (the reference's padding branch)."""
    assert x.is_cuda and indices.is_cuda and x.dim() == 4 and indices.dim() == 3
    b, h, n, d = x.shape
    s = indices.shape[2]
    if x.stride(-1) != 1:
        x = x.contiguous()
    indices = indices.contiguous()
    n_out = s
    if not (chunk_size < 0 or (chunk_size > 0 and n % chunk_size == 0)):
        n_out = math.ceil(s / chunk_size) * chunk_size
    out = torch.empty((b, h, n_out, d), device=x.device, dtype=x.dtype)
    with torch.cuda.device(x.device):
        _lib.check(_lib.lib().ha_gather_rows(
            _ptr(x), _ptr(indices), _idx_code(indices), _ptr(out), b, h, n, s, n_out, d,
            x.stride(0), x.stride(1), x.stride(2), x.element_size(), _stream(x)))
    return out


# -------------------------------------------------------------------------------- attention
def _operands(q, k, v, out, lse, scale, *, layout_bnhd: bool, lse_row_stride: int):
    """Fill AttnOperands from tensors laid out (b,n,h,d) [layout_bnhd] or (b,h,n,d)."""
    t = AttnOperands()
    t.q, t.k, t.v, t.out, t.lse = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr()
    if layout_bnhd:
        b, nq, h, d = q.shape
        nk = k.shape[1]
        hk = k.shape[2]
        sn, sh = 1, 2
    else:
        b, h, nq, d = q.shape
        nk = k.shape[2]
        hk = k.shape[1]
        sn, sh = 2, 1
    t.batch, t.heads, t.n_q, t.n_k, t.d, t.dv = b, h, nq, nk, d, v.shape[-1]
    t.q_stride_b, t.q_stride_h, t.q_stride_n = q.stride(0), q.stride(sh), q.stride(sn)
    t.k_stride_b, t.k_stride_h, t.k_stride_n = k.stride(0), k.stride(sh), k.stride(sn)
    t.v_stride_b, t.v_stride_h, t.v_stride_n = v.stride(0), v.stride(sh), v.stride(sn)
    t.o_stride_b, t.o_stride_h, t.o_stride_n = out.stride(0), out.stride(sh), out.stride(sn)
    t.lse_stride_b, t.lse_stride_h = h * lse_row_stride, lse_row_stride
    t.segs, t.seg_stride_rows, t.q_seg_offset, t.k_seg_offset = 1, 0, 0, 0
    t.kv_group = h // hk
    t.scale = scale
    t.dtype = _dtype_code(q)
    return t


KERNEL_HEAD_DIMS = (64, 128)  # head dims the attention kernels are built for


def padded_head_dim(d):
    """The built head dim that a head dim d <= 128 is zero-padded to."""
    return 64 if d <= 64 else 128


_SAMPLED_BOUNDS = {}  # bounds of explicit sample lists already looked at


def check_sampled_idx(sampled_idx, n_k: int):
    """An explicit sample list names key rows of the call it is used in: every entry must lie in
    [0, n_k).  Inside the causal recursion the same list serves every level, so n_k is the key length of
    the smallest hashed level; a larger entry would read keys of the second half there (future tokens)
    or past the tensor.  The bounds of a list are computed once per tensor version (a host read of a device
    tensor: pass the list once before capturing a graph)."""
    if sampled_idx is None:
        return
    # keyed by the tensor's identity, storage and version; an inference tensor has no version counter and is
    # checked on every call
    version = None if sampled_idx.is_inference() else sampled_idx._version
    key = (id(sampled_idx), sampled_idx.data_ptr(), tuple(sampled_idx.shape), version)
    cached = _SAMPLED_BOUNDS.get(key) if version is not None else None
    if cached is None:
        lo, hi = (int(sampled_idx.min()), int(sampled_idx.max())) if sampled_idx.numel() else (0, -1)
        cached = (version, lo, hi)
        if version is not None:
            if len(_SAMPLED_BOUNDS) > 64:
                _SAMPLED_BOUNDS.clear()
            _SAMPLED_BOUNDS[key] = cached
    assert cached[1] >= 0 and cached[2] < n_k, \
        f"sampled_idx must lie in [0, {n_k}) (the key length of the shortest hashed call); got [{cached[1]}, {cached[2]}]"


def smallest_hashed_key_length(n: int, min_seq_len: int, causal: bool):
    """Key length of the shortest call that uses the hashed kernel (hyper_attention.py:52,109), or None."""
    if not causal:
        return None if min_seq_len > n else n
    smallest = None
    while n > min_seq_len:
        n = (n + 1) // 2
        if not min_seq_len > n:
            smallest = n
    return smallest


def _block_attn_args(q, k, v, o, lse, q_sort_idx, k_sort_idx, block_size, sample_size, softmax_scale,
                     smooth_block, sampled_idx, accumulate=False, layout_bnhd=True):
    """BlockAttnArgs for (b,n,h,d) tensors with (b,n,h) index tensors [layout_bnhd] or (b,h,n,d) tensors
    with (b,h,n) index tensors; the second result keeps the device copy of sampled_idx alive."""
    if layout_bnhd:
        batch, seqlen_q, nheads, _ = q.shape
        sn, sh = 1, 2
    else:
        batch, nheads, seqlen_q, _ = q.shape
        sn, sh = 2, 1
    a = BlockAttnArgs()
    a.t = _operands(q, k, v, o, lse, softmax_scale, layout_bnhd=layout_bnhd, lse_row_stride=seqlen_q)
    a.q_idx, a.k_idx = q_sort_idx.data_ptr(), k_sort_idx.data_ptr()
    a.idx_type = _idx_code(q_sort_idx)
    a.q_idx_stride_b, a.q_idx_stride_h, a.q_idx_stride_n = q_sort_idx.stride(0), q_sort_idx.stride(sh), q_sort_idx.stride(sn)
    a.k_idx_stride_b, a.k_idx_stride_h, a.k_idx_stride_n = k_sort_idx.stride(0), k_sort_idx.stride(sh), k_sort_idx.stride(sn)
    keep = None
    a.sampled_stride_b = a.sampled_stride_h = 0
    if sampled_idx is not None:
        check_sampled_idx(sampled_idx, k.shape[sn])
        keep = sampled_idx.to(device=q.device, dtype=q_sort_idx.dtype).contiguous()
        k_heads = k.shape[sh]
        assert keep.shape in ((sample_size,), (k_heads, sample_size), (batch, k_heads, sample_size)), \
            "sampled_idx must be (sample_size,), (nheads, sample_size) or (batch, nheads, sample_size) (k/v heads)"
        a.sampled_idx = keep.data_ptr()
        if keep.dim() >= 2:
            a.sampled_stride_h = sample_size
        if keep.dim() == 3:
            a.sampled_stride_b = k_heads * sample_size
    a.block_size, a.sample_size = block_size, sample_size
    a.smooth_block, a.accumulate = int(bool(smooth_block)), int(bool(accumulate))
    return a, keep


def _sampled_positions(k_sort_idx, sampled_idx, sample_size):
    """Position of every sampled key row in its head's sorted key order, int32 (batch, nheads, sample_size),
    plus the sample list expanded to that shape (None for the default rows 0..sample_size-1).
    k_sort_idx: (batch, seqlen, nheads) permutations."""
    batch, n, nheads = k_sort_idx.shape
    order = k_sort_idx.transpose(1, 2).long()                                    # (b, h, n): row at each position
    inverse = torch.empty_like(order)
    inverse.scatter_(2, order, torch.arange(n, device=order.device).expand_as(order))  # position of each row
    if sampled_idx is None:
        rows, expanded = torch.arange(sample_size, device=order.device).expand(batch, nheads, -1), None
    else:
        rows = sampled_idx.to(device=order.device, dtype=torch.long)
        rows = rows.expand(batch, nheads, sample_size) if rows.dim() < 3 else rows
        expanded = rows.to(k_sort_idx.dtype).contiguous()
    return inverse.gather(2, rows).to(torch.int32).contiguous(), expanded


def hyper_attn_func(q, k, v, q_sort_idx, k_sort_idx, block_size, sample_size=0, softmax_scale=None,
                    smooth_block=False, *, sampled_idx=None, resume=None, sample_bias=0.0,
                    mask_sampled_in_block=False):
    """q, k: (batch, seqlen, nheads, headdim); v: (batch, seqlen, nheads, v_headdim);
    q_sort_idx, k_sort_idx: (batch, seqlen, nheads) permutations; returns o (batch, seqlen, nheads,
    v_headdim) and lse (batch, nheads, seqlen) fp32.  `sampled_idx` (keyword only, not in the
    reference) lists the sampled key rows: shape (sample_size,) for one list shared by every head, or
    (nheads, sample_size) / (batch, nheads, sample_size) for a list per head; default 0..sample_size-1.
    `resume` (keyword only, not in the reference) is a pair (o, lse) of a previous partial attention
    over other keys, shaped like the results: the kernel continues from it and updates both in place,
    which equals add_self_attentions(previous, this call) in fp32.
    `sample_bias`, `mask_sampled_in_block` (keyword only, not in the reference): the residual estimator of
    the HyperAttention paper.  The bias (e.g. log(seqlen_k / sample_size)) is added to the scaled score of
    every sampled key; with the mask a sampled key that is also among the block keys of the query's tile is
    left out of the sampled part.  Forward only, head dims 64 and 128."""
    q, k, v = [x if x.stride(-1) == 1 else x.contiguous() for x in [q, k, v]]
    assert sample_size % 128 == 0
    reweight = bool(sample_bias) or bool(mask_sampled_in_block)
    if reweight:
        if _wants_grad(q, k, v):
            raise NotImplementedError("the residual estimator (sample_bias, mask_sampled_in_block) has no backward")
        assert v.shape[-1] == q.shape[-1] and q.shape[-1] in KERNEL_HEAD_DIMS, \
            "the residual estimator is built for head dims 64 and 128"
        assert sample_size > 0, "the residual estimator needs sampled keys"
    built = v.shape[-1] == q.shape[-1] and q.shape[-1] in KERNEL_HEAD_DIMS
    if _wants_grad(q, k, v) and built:
        assert resume is None, "resume has no backward"
        return HyperAttnFunc.apply(q, k, v, q_sort_idx, k_sort_idx, block_size, sample_size, softmax_scale,
                                   smooth_block, sampled_idx)
    if not built and (_wants_grad(q, k, v) or q.shape[-1] % 8 or v.shape[-1] % 8):
        # A value head dim different from the q/k head dim (src/hyper_attn_triton.py:679,692-693;
        # unit_tests/test_hyper_attention.py:120-133) or a head dim other than 64 and 128: the forward
        # kernels take any multiples of 8 as they are (the missing pieces of a row are read as zeros).
        # The backward, and head dims that are not multiples of 8, go through zero-padded copies: zero
        # columns change neither q.k nor the wanted columns of the output, so this is exact.
        assert resume is None, "resume needs head dims that are multiples of 8"
        d_qk, d_v = q.shape[-1], v.shape[-1]
        assert d_qk <= 128 and d_v <= 128, "FlashAttention only support head dimensions up to 128"
        wide = padded_head_dim(max(d_qk, d_v))
        pad = lambda x: torch.nn.functional.pad(x, (0, wide - x.shape[-1]))
        o, lse = hyper_attn_func(pad(q), pad(k), pad(v), q_sort_idx, k_sort_idx, block_size, sample_size,
                                 softmax_scale or 1.0 / math.sqrt(d_qk), smooth_block, sampled_idx=sampled_idx)
        return o[..., :d_v], lse
    batch, seqlen_q, nheads, d = q.shape
    _, seqlen_k, _, _ = k.shape
    # (the reference wants as many k/v heads as q heads; fewer, dividing them, are grouped-query heads: q head
    # h reads k/v head h // (nheads // k_heads), and k_sort_idx, per-head sample lists and dk, dv go by k/v heads)
    k_heads = k.shape[2]
    assert k.shape == (batch, seqlen_k, k_heads, d) and nheads % k_heads == 0
    assert v.shape[:3] == (batch, seqlen_k, k_heads)
    assert q_sort_idx.shape == q.shape[:3]
    assert k_sort_idx.shape == k.shape[:3]
    assert d <= 128, "FlashAttention only support head dimensions up to 128"
    assert q.dtype == k.dtype == v.dtype, "All tensors must have the same type"
    assert q.dtype in [torch.float16, torch.bfloat16], "Only support fp16 and bf16"
    assert q.is_cuda and k.is_cuda and v.is_cuda and q_sort_idx.is_cuda and k_sort_idx.is_cuda
    assert q_sort_idx.dtype == k_sort_idx.dtype
    softmax_scale = softmax_scale or 1.0 / math.sqrt(d)
    if resume is None:
        lse = torch.empty((batch, nheads, seqlen_q), device=q.device, dtype=torch.float32)
        o = torch.empty((batch, seqlen_q, nheads, v.shape[-1]), device=q.device, dtype=q.dtype)
    else:
        o, lse = resume
        assert o.shape == (batch, seqlen_q, nheads, v.shape[-1]) and o.dtype == q.dtype and o.is_cuda
        assert lse.shape == (batch, nheads, seqlen_q) and lse.dtype == torch.float32 and lse.is_contiguous()
        assert o.stride(-1) == 1
    assert seqlen_k % 128 == 0, "keys sequence length must be divisible by 128"

    pos = None
    if mask_sampled_in_block:
        # a position per (batch, head, slot): the sample list goes in that shape too (one set of strides)
        if sampled_idx is not None:
            check_sampled_idx(sampled_idx, seqlen_k)
        pos, sampled_idx = _sampled_positions(k_sort_idx, sampled_idx, sample_size)
    a, keep = _block_attn_args(q, k, v, o, lse, q_sort_idx, k_sort_idx, block_size, sample_size, softmax_scale,
                               smooth_block, sampled_idx, accumulate=resume is not None)
    if reweight:
        a.sample_bias = float(sample_bias)
        if pos is not None:
            a.sampled_pos, a.mask_sampled_in_block = pos.data_ptr(), 1
            a.sampled_stride_b, a.sampled_stride_h = pos.shape[1] * sample_size, sample_size
    with torch.cuda.device(q.device):
        _lib.check(_lib.lib().ha_block_attn_fwd(ctypes.byref(a), _stream(q)))
    return o, lse


def flash_attn_func(q, k, v, bias=None, causal=False, softmax_scale=None):
    """q: (batch, seqlen_q, nheads, headdim); k, v: (batch, seqlen_k, nheads, headdim).
    Returns o like q and lse (batch, nheads, ceil(seqlen_q/128)*128) fp32 (padding rows undefined)."""
    if bias is not None:
        raise NotImplementedError("attention bias is not part of the HyperAttention forward path")
    q, k, v = [x if x.stride(-1) == 1 else x.contiguous() for x in [q, k, v]]
    batch, seqlen_q, nheads, d = q.shape
    _, seqlen_k, _, _ = k.shape
    k_heads = k.shape[2]   # fewer than nheads, dividing them: grouped-query heads (not in the reference)
    assert k.shape == (batch, seqlen_k, k_heads, d) and nheads % k_heads == 0
    assert v.shape == (batch, seqlen_k, k_heads, d)
    assert d <= 128, "FlashAttention only support head dimensions up to 128"
    if _wants_grad(q, k, v) and d in KERNEL_HEAD_DIMS:
        return FlashAttnFunc.apply(q, k, v, bias, causal, softmax_scale)
    if d not in KERNEL_HEAD_DIMS and (_wants_grad(q, k, v) or d % 8):
        # the forward kernels take any multiple of 8; the backward and other head dims run zero-padded to a
        # built width (exact; costs the padded copies)
        pad = lambda x: torch.nn.functional.pad(x, (0, padded_head_dim(d) - d))
        o, lse = flash_attn_func(pad(q), pad(k), pad(v), None, causal, softmax_scale or 1.0 / math.sqrt(d))
        return o[..., :d], lse
    assert q.dtype == k.dtype == v.dtype, "All tensors must have the same type"
    assert q.dtype in [torch.float16, torch.bfloat16], "Only support fp16 and bf16"
    assert q.is_cuda and k.is_cuda and v.is_cuda
    softmax_scale = softmax_scale or 1.0 / math.sqrt(d)
    seqlen_q_rounded = math.ceil(seqlen_q / 128) * 128
    lse = torch.empty((batch, nheads, seqlen_q_rounded), device=q.device, dtype=torch.float32)
    o = torch.empty_like(q)
    t = _operands(q, k, v, o, lse, softmax_scale, layout_bnhd=True, lse_row_stride=seqlen_q_rounded)
    with torch.cuda.device(q.device):
        _lib.check(_lib.lib().ha_flash_attn_fwd(ctypes.byref(t), int(bool(causal)), _stream(q)))
    return o, lse


def add_self_attentions(attn1, lse1, attn2, lse2):
    """attn1, attn2: [b, h, n, d]; lse1, lse2: [b, h, n, 1] fp32.  Returns (attn, lse)."""
    assert attn1.is_cuda and attn1.shape == attn2.shape and attn1.dtype == attn2.dtype
    if _wants_grad(attn1, attn2, lse1, lse2):
        # differentiable form, in the reference's own arithmetic (src/attn_utils.py:21-23): the weight is
        # rounded to the attention's type before it is used
        # (the logarithm is taken in fp32, as the kernel does; the reference takes it in the attention's type)
        c = torch.sigmoid(lse1 - lse2).to(attn1.dtype)
        return c * attn1 + (1 - c) * attn2, lse1 - (c.float() + torch.finfo(lse1.dtype).eps).log()
    b, h, n, d = attn1.shape
    a1 = attn1.contiguous()
    a2 = attn2.contiguous()
    l1 = lse1.to(torch.float32).contiguous().view(-1)
    l2 = lse2.to(torch.float32).contiguous().view(-1)
    assert l1.numel() == b * h * n and l2.numel() == b * h * n
    out = torch.empty_like(a1)
    lse = torch.empty((b, h, n, 1), device=attn1.device, dtype=torch.float32)
    with torch.cuda.device(attn1.device):
        _lib.check(_lib.lib().ha_lse_merge(_ptr(a1), _ptr(l1), _ptr(a2), _ptr(l2), _ptr(out), _ptr(lse),
                                           b * h * n, d, d, d, d, 1, 1, 1, _dtype_code(a1), _stream(a1)))
    return out, lse


# ------------------------------------------------------------------------------- backward
def _wants_grad(*tensors):
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


def _attn_grads(t, dout, dq, dk, dv, layout_bnhd=True, accumulate=False, sample_size=0):
    """AttnGrads for (b,n,h,d) [layout_bnhd] or (b,h,n,d) gradient tensors plus the workspace the C side asks for."""
    sn, sh = (1, 2) if layout_bnhd else (2, 1)
    g = AttnGrads()
    g.dout, g.dq, g.dk, g.dv = dout.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr()
    g.do_stride_b, g.do_stride_h, g.do_stride_n = dout.stride(0), dout.stride(sh), dout.stride(sn)
    g.dq_stride_b, g.dq_stride_h, g.dq_stride_n = dq.stride(0), dq.stride(sh), dq.stride(sn)
    g.dk_stride_b, g.dk_stride_h, g.dk_stride_n = dk.stride(0), dk.stride(sh), dk.stride(sn)
    g.dv_stride_b, g.dv_stride_h, g.dv_stride_n = dv.stride(0), dv.stride(sh), dv.stride(sn)
    g.accumulate = int(bool(accumulate))
    nbytes = _lib.lib().ha_attn_bwd_workspace_bytes(ctypes.byref(t), sample_size)
    if nbytes <= 0:
        _lib.check(int(nbytes) if nbytes < 0 else -3)
    ws = torch.empty((nbytes,), device=dout.device, dtype=torch.uint8)
    g.workspace, g.workspace_bytes = ws.data_ptr(), nbytes
    return g, ws


class HyperAttnFunc(torch.autograd.Function):
    """hyper_attn_func with its backward (HyperAttnFunc, src/hyper_attn_triton.py:895-945): gradients for
    q, k, v; a gradient arriving for lse is ignored, as there."""

    @staticmethod
    def forward(ctx, q, k, v, q_sort_idx, k_sort_idx, block_size, sample_size, softmax_scale, smooth_block,
                sampled_idx):
        o, lse = hyper_attn_func(q, k, v, q_sort_idx, k_sort_idx, block_size, sample_size, softmax_scale,
                                 smooth_block, sampled_idx=sampled_idx)
        ctx.save_for_backward(q, k, v, q_sort_idx, k_sort_idx, o, lse)
        # no gradient is returned for lse: saying so up front keeps autograd from computing one
        ctx.mark_non_differentiable(lse)
        ctx.sampled_idx = sampled_idx
        ctx.conf = (block_size, sample_size, softmax_scale or 1.0 / math.sqrt(q.shape[-1]), smooth_block)
        return o, lse

    @staticmethod
    def backward(ctx, do, dlse=None):
        q, k, v, q_sort_idx, k_sort_idx, o, lse = ctx.saved_tensors
        block_size, sample_size, softmax_scale, smooth_block = ctx.conf
        do = do.contiguous()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        a, keep = _block_attn_args(q, k, v, o, lse, q_sort_idx, k_sort_idx, block_size, sample_size, softmax_scale,
                                   smooth_block, ctx.sampled_idx)
        g, ws = _attn_grads(a.t, do, dq, dk, dv, sample_size=sample_size)
        with torch.cuda.device(q.device):
            _lib.check(_lib.lib().ha_block_attn_bwd(ctypes.byref(a), ctypes.byref(g), _stream(q)))
        return dq, dk, dv, None, None, None, None, None, None, None


class FlashAttnFunc(torch.autograd.Function):
    """flash_attn_func with its backward (FlashAttnFunc, src/flash_attn_triton.py:995-1040)."""

    @staticmethod
    def forward(ctx, q, k, v, bias, causal, softmax_scale):
        o, lse = flash_attn_func(q, k, v, bias, causal, softmax_scale)
        ctx.save_for_backward(q, k, v, o, lse)
        ctx.mark_non_differentiable(lse)
        ctx.conf = (bool(causal), softmax_scale or 1.0 / math.sqrt(q.shape[-1]))
        return o, lse

    @staticmethod
    def backward(ctx, do, dlse=None):
        q, k, v, o, lse = ctx.saved_tensors
        causal, softmax_scale = ctx.conf
        do = do.contiguous()
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        t = _operands(q, k, v, o, lse, softmax_scale, layout_bnhd=True, lse_row_stride=lse.shape[-1])
        g, ws = _attn_grads(t, do, dq, dk, dv)
        with torch.cuda.device(q.device):
            _lib.check(_lib.lib().ha_flash_attn_bwd(ctypes.byref(t), int(causal), ctypes.byref(g), _stream(q)))
        return dq, dk, dv, None, None, None


# ------------------------------------------------------------------------- whole forward pass
class WorkspaceCache:
    """Workspaces of the one-call forward kept between calls: one tensor per (device, stream), grown when a
    larger shape arrives, and the sizes the library asked for per shape.

    Under stream capture the cache is bypassed: a captured call gets a fresh tensor from the capturing graph's
    own memory pool (two graphs captured on one stream must not share a workspace: their replays may overlap).
    A tensor that is replaced by a larger one is kept alive in `retired`, because a graph captured earlier, or
    work still queued on the stream, may point at it.  The cache is not part of a module's state: copies and
    pickles of it start empty."""

    def __init__(self):
        self.sizes = {}
        self.slots = {}
        self.retired = []

    def tensor(self, device, stream, nbytes, capturing=False):
        if capturing:
            return torch.empty(int(nbytes), device=device, dtype=torch.uint8)
        slot = (device.index, stream)
        ws = self.slots.get(slot)
        if ws is None or ws.numel() < int(nbytes):
            if ws is not None:
                self.retired.append(ws)
            ws = torch.empty(int(nbytes), device=device, dtype=torch.uint8)
            self.slots[slot] = ws
        return ws

    def __deepcopy__(self, memo):
        return WorkspaceCache()

    def __reduce__(self):
        return (WorkspaceCache, ())


def causal_plan(n: int, min_seq_len: int):
    """Lengths of the causal recursion (hyper_attention.py:51-96): (halves, leaf).  halves[j] is the length of
    the two halves a level-j virtual head is cut into, after the zero row an odd length gets appended
    (:61-64); leaf the length the recursion stops at.  Only n itself can be odd in a shape the kernels take:
    hashed halves are multiples of 128, and a level with shorter halves is the last."""
    halves = []
    while n > min_seq_len:
        n = (n + 1) // 2
        halves.append(n)
    return halves, n


def forward_plan_supported(n: int, min_seq_len: int, causal: bool, lsh_num_projs: int) -> bool:
    """True when ha_forward covers this shape: any length, up to 16 projections."""
    return lsh_num_projs <= 16


def forward_plan_even(n: int, min_seq_len: int) -> bool:
    """True when every level of the causal recursion has an even length (what the recursion under autograd,
    which works on equal segments of the whole tensors, takes)."""
    while n > min_seq_len:
        if n % 2:
            return False
        n //= 2
    return True


def _forward_args(q, k, v, out, lse, proj, *, scale, causal, lsh_num_projs, block_size, sample_size, min_seq_len,
                  smooth_block, sampled_idx=None, workspace=None, stream=None):
    """ForwardArgs for (b,h,n,d) q and (b,h_kv,n,d) k, v with its workspace attached; the second result keeps
    the tensors alive that the struct only points to (the workspace last).  `workspace`: a WorkspaceCache the
    caller owns; the workspace tensor of the current (device, stream) and the sizes the library asked for are
    kept there and reused, so that a caller that runs many forwards neither allocates nor asks per call.
    `stream`: the raw handle of the current stream, if the caller has it already."""
    assert q.is_cuda and k.is_cuda
    assert q.stride(-1) == 1 and k.stride(-1) == 1 and (v is None or v.stride(-1) == 1)
    assert q.dtype == k.dtype and (v is None or v.dtype == q.dtype), "All tensors must have the same type"
    b, h, n, d = q.shape
    hk = k.shape[1]
    a = ForwardArgs()
    a.q, a.k = q.data_ptr(), k.data_ptr()
    if v is not None:
        a.v, a.out, a.lse = v.data_ptr(), out.data_ptr(), lse.data_ptr()
    keep = []
    if proj is not None:
        assert proj.dtype == q.dtype, "All three tensors must have the same type"
        p = proj.reshape(d, lsh_num_projs).contiguous()
        keep.append(p)
        a.proj = p.data_ptr()
    if sampled_idx is not None:
        shortest = smallest_hashed_key_length(n, min_seq_len, bool(causal))
        if shortest is not None:
            check_sampled_idx(sampled_idx, shortest)
        s = sampled_idx.to(device=q.device, dtype=torch.int32).contiguous()
        assert s.shape == (sample_size,)
        keep.append(s)
        a.sampled_idx = s.data_ptr()
    a.batch, a.heads, a.kv_heads, a.n, a.d = b, h, hk, n, d
    a.dv = v.shape[-1] if v is not None else d
    a.lsh_num_projs, a.block_size, a.sample_size, a.min_seq_len = lsh_num_projs, block_size, sample_size, min_seq_len
    a.smooth_block, a.causal = int(bool(smooth_block)), int(bool(causal))
    a.scale = scale
    a.dtype = _dtype_code(q)
    a.q_stride_b, a.q_stride_h, a.q_stride_n = q.stride(0), q.stride(1), q.stride(2)
    a.k_stride_b, a.k_stride_h, a.k_stride_n = k.stride(0), k.stride(1), k.stride(2)
    if v is not None:
        a.v_stride_b, a.v_stride_h, a.v_stride_n = v.stride(0), v.stride(1), v.stride(2)
    shape_key = (b, h, hk, n, d, a.dv, lsh_num_projs, min_seq_len, a.causal)
    ws_bytes = workspace.sizes.get(shape_key) if workspace is not None else None
    if ws_bytes is None:
        ws_bytes = _lib.lib().ha_forward_workspace_bytes(ctypes.byref(a))
        if ws_bytes < 0:
            _lib.check(int(ws_bytes))
        if workspace is not None:
            workspace.sizes[shape_key] = ws_bytes
    if workspace is not None:
        if stream is None:
            stream = torch.cuda.current_stream(q.device).cuda_stream
        ws = workspace.tensor(q.device, stream, ws_bytes, capturing=torch.cuda.is_current_stream_capturing())
    else:
        ws = torch.empty(int(ws_bytes), device=q.device, dtype=torch.uint8)
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    keep.append(ws)
    return a, keep


def hyper_forward(q, k, v, proj, *, scale, causal, lsh_num_projs, block_size, sample_size, min_seq_len,
                  smooth_block, sampled_idx=None, workspace=None):
    """One-call forward for (b,h,n,d) q and (b,h_kv,n,d) k, v of any strides with a contiguous last
    dimension (permuted views are read in place).  Returns contiguous out (b,h,n,dv) and lse (b,h,n) fp32.
    `workspace`: see _forward_args."""
    assert v.is_cuda
    b, h, n, d = q.shape
    out = torch.empty((b, h, n, v.shape[-1]), device=q.device, dtype=q.dtype)
    lse = torch.empty((b, h, n), device=q.device, dtype=torch.float32)
    stream = torch.cuda.current_stream(q.device).cuda_stream
    a, keep = _forward_args(q, k, v, out, lse, proj, scale=scale, causal=causal, lsh_num_projs=lsh_num_projs,
                            block_size=block_size, sample_size=sample_size, min_seq_len=min_seq_len,
                            smooth_block=smooth_block, sampled_idx=sampled_idx, workspace=workspace, stream=stream)
    if q.device.index == torch.cuda.current_device():
        _lib.check(_lib.lib().ha_forward(ctypes.byref(a), ctypes.c_void_p(stream)))
    else:
        with torch.cuda.device(q.device):
            _lib.check(_lib.lib().ha_forward(ctypes.byref(a), ctypes.c_void_p(stream)))
    return out, lse


def forward_sort(q, k, proj, *, causal, lsh_num_projs, min_seq_len):
    """Bucket orders of every hashed level of the forward pass (ha_forward_sort): one hash launch for q and
    k, one ranking, one placement.  Returns (q_idx, k_idx): per level (0 = whole sequence) an int32 tensor
    (b, h * 2^level, half) / (b, h_kv * 2^level, half) of rows local to the level's query segment (second
    halves) / key segment (first halves), or None where the level is exact.  With an odd n the last query of
    the last segment of every head is the zero row the recursion appends (it has no row in q).  The tensors are views of one
    workspace."""
    b, h, n, d = q.shape
    hk = k.shape[1]
    a, keep = _forward_args(q, k, None, None, None, proj, scale=1.0, causal=causal, lsh_num_projs=lsh_num_projs,
                            block_size=128, sample_size=0, min_seq_len=min_seq_len, smooth_block=False)
    ws = keep[-1]
    q_off = (ctypes.c_int64 * 48)()
    k_off = (ctypes.c_int64 * 48)()
    levels = ctypes.c_int(0)
    with torch.cuda.device(q.device):
        _lib.check(_lib.lib().ha_forward_sort(ctypes.byref(a), q_off, k_off, ctypes.byref(levels), _stream(q)))
    q_idx, k_idx = [], []
    halves = causal_plan(n, min_seq_len)[0] if causal else [n]
    for j in range(levels.value):
        if q_off[j] < 0:
            q_idx.append(None)
            k_idx.append(None)
            continue
        segs = (1 << j) if causal else 1
        half = halves[j] if causal else n
        q_idx.append(ws[q_off[j]:q_off[j] + 4 * b * h * segs * half].view(torch.int32).view(b, h * segs, half))
        k_idx.append(ws[k_off[j]:k_off[j] + 4 * b * hk * segs * half].view(torch.int32).view(b, hk * segs, half))
    return q_idx, k_idx
