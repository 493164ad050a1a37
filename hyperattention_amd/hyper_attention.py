"""HyperAttention module: same constructor and forward signature as the reference
(hyper_attention.py:9-132), computed by the HIP library.

Inputs whose causal recursion only meets even lengths take one library call (ha_forward: q and k
hashed in one launch, the rows ranked once for all levels, leaves, then each level merged in place).
Other shapes (an odd length somewhere in the recursion) are composed here from the same HIP operators,
following the reference's recursion step by step.

With inputs that require grad the forward keeps what the backward needs: the non-causal case is one
differentiable operator call, the causal recursion with even lengths runs on segments of the whole
tensors with the calls' gradients accumulated by the kernels (_CausalRecursionFunc), anything else
operator by operator under torch autograd.
"""
from __future__ import annotations

import ctypes
import math

import torch

from . import _lib, ops
from .angular_lsh import AngularLSH


class _CausalRecursionFunc(torch.autograd.Function):
    """The causal divide-and-conquer (hyper_attention.py:51-96) with its gradient, for lengths that stay
    even down to the leaves; key and value may have fewer heads than the query (grouped queries).

    Same arithmetic as the reference's recursion under autograd: exact causal attention on the leaves,
    one un-masked call per level on (second-half queries, first-half keys/values), merges with the
    weight rounded to the attention's type (src/attn_utils.py:21-23), and log-sum-exps that carry no
    gradient (src/hyper_attn_triton.py:922-945).  What differs is the bookkeeping.  All rows are hashed
    in one launch and ranked once for all levels (ha_forward_sort).  Every call reads and writes its
    segments of the whole (batch, heads, n, d) tensors through the C entry points; the result of level j
    (the second halves of its segments: n/2 rows per head) is kept packed in o_un[j], (batch, heads, n/2, d).  One pass merges the leaf and level
    results of every row (ha_lse_merge_levels) and, on the way, turns the merge weights into the shifted
    log-sum-exps that the backward hands to each call in place of a weighted copy of the output gradient.
    In the backward the gradients of the calls are accumulated by the kernels (`accumulate`), so there
    are no concatenations, zero-padded slice gradients or gradient additions.
    """

    @staticmethod
    def _segments(t, lens, j, leaves=False):
        """Point the operands at the segments of level j: the un-masked call on (second-half queries,
        first-half keys) of every segment of lens[j] rows, or the leaves."""
        if leaves:
            t.n_q = t.n_k = lens[j]
            t.segs, t.seg_stride_rows, t.q_seg_offset, t.k_seg_offset = 1 << j, lens[j], 0, 0
        else:
            half = lens[j + 1]
            t.n_q = t.n_k = half
            t.segs, t.seg_stride_rows, t.q_seg_offset, t.k_seg_offset = 1 << j, lens[j], half, 0
            # out and lse hold the rows the call writes and nothing else: segment after segment
            t.o_seg_stride_rows, t.o_seg_offset = half, 0
        return t

    @staticmethod
    def _level_args(module, query, key, value, out, lse, scale, lens, j, q_idx, k_idx, sampled):
        """BlockAttnArgs of the hashed un-masked call of level j on the whole tensors."""
        b, h, n, d = query.shape
        hk, half, segs = key.shape[1], lens[j + 1], 1 << j
        a = _lib.BlockAttnArgs()
        a.t = _CausalRecursionFunc._segments(
            ops._operands(query, key, value, out, lse, scale, layout_bnhd=False, lse_row_stride=n // 2), lens, j)
        a.q_idx, a.k_idx, a.idx_type = q_idx.data_ptr(), k_idx.data_ptr(), ops._idx_code(q_idx)
        a.q_idx_stride_b, a.q_idx_stride_h, a.q_idx_stride_n = h * segs * half, segs * half, 1
        a.k_idx_stride_b, a.k_idx_stride_h, a.k_idx_stride_n = hk * segs * half, segs * half, 1
        a.sampled_stride_b = a.sampled_stride_h = 0
        if sampled is not None:
            a.sampled_idx = sampled.data_ptr()
        a.block_size, a.sample_size = module.block_size, module.sample_size
        a.smooth_block, a.accumulate = int(bool(module.smooth_block)), 0
        return a

    @staticmethod
    def _sampled(module, query, lens, hashed):
        """The module's explicit sample list as an int32 device tensor, checked against the shortest hashed
        level (the list serves every level)."""
        if module.sampled_idx is None or not any(hashed):
            return None
        ops.check_sampled_idx(module.sampled_idx, min(lens[j + 1] for j in range(len(hashed)) if hashed[j]))
        sampled = module.sampled_idx.to(device=query.device, dtype=torch.int32).contiguous()
        assert sampled.shape == (module.sample_size,), "inside the causal recursion sampled_idx is one (sample_size,) list"
        return sampled

    @staticmethod
    def forward(ctx, module, scale, query, key, value, proj):
        b, h, n, d = query.shape
        lens = [n]
        while lens[-1] > module.min_seq_len:
            lens.append(lens[-1] // 2)
        levels = len(lens) - 1
        lib, stream = _lib.lib(), ops._stream(query)
        dev = query.device
        f32 = dict(device=dev, dtype=torch.float32)
        hashed = [not module.min_seq_len > lens[j + 1] for j in range(levels)]  # hyper_attention.py:109
        segments = _CausalRecursionFunc._segments
        operands = lambda out, lse, rows=n: ops._operands(query, key, value, out, lse, scale, layout_bnhd=False,
                                                           lse_row_stride=rows)

        q_idx = k_idx = [None] * levels
        if any(hashed):
            q_idx, k_idx = ops.forward_sort(query, key, proj, causal=True,
                                            lsh_num_projs=module.lsh_num_projs, min_seq_len=module.min_seq_len)
        sampled = _CausalRecursionFunc._sampled(module, query, lens, hashed)
        o_leaf, lse_leaf = torch.empty_like(query), torch.empty((b, h, n), **f32)
        # level results, packed: a level writes the second halves of its segments, n/2 rows per head
        o_un = torch.empty((levels, b, h, n // 2, d), device=dev, dtype=query.dtype)
        lse_un = torch.empty((levels, b, h, n // 2), **f32)
        lse_shifted, leaf_shifted = torch.empty((levels, b, h, n // 2), **f32), torch.empty((b, h, n), **f32)
        out, lse = torch.empty_like(query), torch.empty((b, h, n), **f32)
        with torch.cuda.device(dev):
            # leaves: exact causal attention on every segment of lens[levels] rows
            t = segments(operands(o_leaf, lse_leaf), lens, levels, leaves=True)
            _lib.check(lib.ha_flash_attn_fwd(ctypes.byref(t), 1, stream))
            for j in range(levels):
                if hashed[j]:
                    a = _CausalRecursionFunc._level_args(module, query, key, value, o_un[j], lse_un[j], scale, lens, j,
                                                         q_idx[j], k_idx[j], sampled)
                    _lib.check(lib.ha_block_attn_fwd(ctypes.byref(a), stream))
                else:
                    t = segments(operands(o_un[j], lse_un[j], n // 2), lens, j)
                    _lib.check(lib.ha_flash_attn_fwd(ctypes.byref(t), 0, stream))
            ptrs = lambda x: (ctypes.c_void_p * max(levels, 1))(*[x[j].data_ptr() for j in range(levels)])
            _lib.check(lib.ha_lse_merge_levels(
                o_leaf.data_ptr(), lse_leaf.data_ptr(), ptrs(o_un), ptrs(lse_un), ptrs(lse_shifted),
                leaf_shifted.data_ptr(), out.data_ptr(), lse.data_ptr(), levels, b * h, n, d, ops._dtype_code(query),
                1, stream))

        tensors = [query, key, value, o_leaf, leaf_shifted, o_un, lse_shifted]
        if sampled is not None:
            tensors.append(sampled)
        for j in range(levels):
            if hashed[j]:
                tensors += [q_idx[j], k_idx[j]]
        ctx.save_for_backward(*tensors)
        ctx.hashed, ctx.lens, ctx.module, ctx.scale, ctx.has_sampled = hashed, lens, module, scale, sampled is not None
        lse = lse.unsqueeze(-1)
        ctx.mark_non_differentiable(lse)
        return out, lse

    @staticmethod
    def backward(ctx, dout, dlse=None):
        saved = list(ctx.saved_tensors)
        query, key, value, o_leaf, leaf_shifted, o_un, lse_shifted = saved[:7]
        rest = saved[7:]
        sampled = rest.pop(0) if ctx.has_sampled else None
        module, scale, lens, hashed = ctx.module, ctx.scale, ctx.lens, ctx.hashed
        b, h, n, d = query.shape
        levels = len(lens) - 1
        lib, stream = _lib.lib(), ops._stream(query)
        segments = _CausalRecursionFunc._segments

        with torch.cuda.device(query.device):
            # The gradient of the output splits at every merge, from the top level down: (1 - c) of it goes
            # to the un-masked call of the level, c of it further down.  A call's gradients are linear in
            # the output gradient it is given, and that enters only through P = exp(s - lse): weighting a
            # row's output gradient by w equals giving the call the log-sum-exp lse - log(w) for that row
            # (w = 0: lse = +inf, P = 0).  So every call gets the output gradient as it is and the shifted
            # log-sum-exps that the forward's merge pass wrote, and no weighted copy of the gradient is made.
            dout = dout.contiguous()
            dq, dk, dv = torch.empty_like(query), torch.empty_like(key), torch.empty_like(value)
            # leaves first: they write every row of dq, dk, dv; the levels then add to their segments
            t = segments(ops._operands(query, key, value, o_leaf, leaf_shifted, scale, layout_bnhd=False,
                                       lse_row_stride=n), lens, levels, leaves=True)
            g, ws = ops._attn_grads(t, dout, dq, dk, dv, layout_bnhd=False)
            _lib.check(lib.ha_flash_attn_bwd(ctypes.byref(t), 1, ctypes.byref(g), stream))
            for j in range(levels):
                if hashed[j]:
                    q_idx, k_idx = rest.pop(0), rest.pop(0)
                    a = _CausalRecursionFunc._level_args(module, query, key, value, o_un[j], lse_shifted[j], scale,
                                                         lens, j, q_idx, k_idx, sampled)
                    g, ws = ops._attn_grads(a.t, dout, dq, dk, dv, layout_bnhd=False, accumulate=True,
                                            sample_size=module.sample_size)
                    _lib.check(lib.ha_block_attn_bwd(ctypes.byref(a), ctypes.byref(g), stream))
                else:
                    t = segments(ops._operands(query, key, value, o_un[j], lse_shifted[j], scale, layout_bnhd=False,
                                               lse_row_stride=n // 2), lens, j)
                    g, ws = ops._attn_grads(t, dout, dq, dk, dv, layout_bnhd=False, accumulate=True)
                    _lib.check(lib.ha_flash_attn_bwd(ctypes.byref(t), 0, ctypes.byref(g), stream))
        return None, None, dq, dk, dv, None


class HyperAttention(torch.nn.Module):

    def __init__(self, input_dim=64, lsh_num_projs=8, block_size=256, sample_size=256, min_seq_len=2048,
                 smooth_block=False, **kwargs):
        """
        - block_size and sample_size must be divisible by 128
        Optional keyword hooks (not in the reference, for reproducible runs): `rng` (torch.Generator
        for the projection), `proj_dir` (explicit (input_dim, lsh_num_projs) projection) and
        `sampled_idx` (explicit sampled key rows, shape (sample_size,)).
        `residual_estimator=True` (not in the reference either; the estimator of the HyperAttention paper):
        every hashed call weights its sampled keys by n_key / sample_size and leaves out those that are
        already among the block keys of the query.  Forward only, head dims 64 and 128.
        """
        super().__init__()
        self.input_dim = input_dim
        self.lsh_num_projs = lsh_num_projs
        self.block_size = block_size
        self.sample_size = sample_size
        self.min_seq_len = min_seq_len
        self.smooth_block = smooth_block
        self.lsh = AngularLSH(num_projs=self.lsh_num_projs, dim=(1, 1, input_dim), rng=kwargs.get('rng'))
        if kwargs.get('proj_dir') is not None:
            proj = torch.as_tensor(kwargs['proj_dir']).reshape(1, 1, input_dim, lsh_num_projs)
            self.lsh.proj_dir = proj.to(self.lsh.proj_dir.dtype).clone()
        self.sampled_idx = kwargs.get('sampled_idx')
        self.residual_estimator = bool(kwargs.get('residual_estimator', False))
        # workspace of the one-call forward, one per (device, stream), kept between calls
        self._workspace = ops.WorkspaceCache()

    def forward(self, query: torch.tensor, key: torch.tensor, value: torch.tensor, scale=None, causal=False,
                return_lse=False):
        """
        inputs:
            - query, key, value: (batch, heads, seq_len, dim); same sequence lengths
            - sequence lengths must be divisible by block_size
        output:
            - attn: (approximation of) the attention output (batch, heads, seq_len, dim_v)
            - lse: (approximation of) log-sum-exp of the scaled qk matrix, (batch, heads, seq_len, 1)
        """
        # permuted views (e.g. (sq, b, np, hn) tensors seen as (b, np, sq, hn)) are read in place
        query, key, value = [x if x.stride(-1) == 1 else x.contiguous() for x in (query, key, value)]

        n_query = query.shape[2]
        batch_size, n_heads, n_key, dim = key.shape
        scale = scale or dim ** (-0.5)
        assert n_query == n_key

        dim_v = value.shape[-1]
        proj = self.lsh.proj_dir
        built = dim in ops.KERNEL_HEAD_DIMS and dim_v == dim
        if not built and (dim % 8 or dim_v % 8 or ops._wants_grad(query, key, value)):
            # The forward kernels take head dims that are multiples of 8 as they are, the value dim apart
            # from the q/k dim.  Other head dims, and the backward for anything but 64 and 128 with equal
            # dims, run zero-padded: zero columns change neither the projections, nor q.k, nor the wanted
            # outputs
            assert dim <= 128 and dim_v <= 128, "FlashAttention only support head dimensions up to 128"
            wide = ops.padded_head_dim(max(dim, dim_v))
            pad = lambda x: torch.nn.functional.pad(x, (0, wide - x.shape[-1]))
            attn, lse = self._forward_built(pad(query), pad(key), pad(value), scale, causal,
                                            torch.nn.functional.pad(proj, (0, 0, 0, wide - dim)))
            attn = attn[..., :dim_v]
        else:
            attn, lse = self._forward_built(query, key, value, scale, causal, proj)
        return (attn, lse) if return_lse else attn

    def _forward_built(self, query, key, value, scale, causal, proj):
        """forward() for a head dim the kernels are built for, value dim equal to it; proj: the
        (1, 1, dim, lsh_num_projs) projection to hash with.  Returns (attn, lse)."""
        n_key = key.shape[2]
        # gradients are taken operator by operator, as in the reference (each attention operator has its own
        # backward and the merges are differentiable tensor arithmetic); the one-call forward has none
        if self.residual_estimator and ops._wants_grad(query, key, value):
            raise NotImplementedError("residual_estimator has no backward")
        if (ops.forward_plan_supported(n_key, self.min_seq_len, causal is not False, self.lsh_num_projs)
                and not ops._wants_grad(query, key, value) and not self.residual_estimator):
            attn, lse = ops.hyper_forward(
                query, key, value, proj, scale=scale, causal=causal is not False,
                lsh_num_projs=self.lsh_num_projs, block_size=self.block_size, sample_size=self.sample_size,
                min_seq_len=self.min_seq_len, smooth_block=self.smooth_block, sampled_idx=self.sampled_idx,
                workspace=self._workspace)
            if causal is not False and n_key <= self.min_seq_len:
                # the reference returns the exact kernel's padded 3-d lse for a top-level leaf
                n_rounded = -(-n_key // 128) * 128
                if n_rounded != n_key:
                    lse = torch.nn.functional.pad(lse, (0, n_rounded - n_key))
            else:
                lse = lse.unsqueeze(-1)
        elif (causal is not False and n_key > self.min_seq_len and not self.residual_estimator
              and self.lsh_num_projs <= 16 and ops.forward_plan_even(n_key, self.min_seq_len)):
            # gradients wanted and every level has an even length: the recursion and its gradient on
            # segments of the whole tensors, grouped-query heads as they are
            attn, lse = _CausalRecursionFunc.apply(self, scale, query.contiguous(), key.contiguous(), value.contiguous(),
                                                   proj)
        else:
            if key.shape[1] != query.shape[1] and causal is not False:
                # grouped-query inputs on the operator-by-operator recursion: it follows the reference, which
                # folds halves into heads (hyper_attention.py:67-68), and that needs as many k/v heads as q
                # heads; a single un-masked call takes the groups as they are
                group = query.shape[1] // key.shape[1]
                key, value = key.repeat_interleave(group, dim=1), value.repeat_interleave(group, dim=1)
            query, key, value = query.contiguous(), key.contiguous(), value.contiguous()
            attn, lse = self._forward_composed(query, key, value, scale, causal, proj)

        if causal is not False and n_key <= self.min_seq_len and lse.dim() == 4:
            # a top-level leaf: the exact kernel's padded 3-d lse, whichever path computed it
            n_rounded = -(-n_key // 128) * 128
            lse = torch.nn.functional.pad(lse.squeeze(-1), (0, n_rounded - n_key))
        return attn, lse

    # ---- the reference's recursion, operator by operator (shapes ha_forward does not take) --------
    def _forward_composed(self, query, key, value, scale, causal, proj=None):
        batch_size, n_heads, n_key, dim = key.shape
        n_query = query.shape[2]
        if causal is False:
            return self.forward_no_causal_mask(query, key, value, scale, proj)
        if n_key <= self.min_seq_len:
            attn, lse = ops.flash_attn_func(query.transpose(1, 2), key.transpose(1, 2), value.transpose(1, 2),
                                            None, True, scale)
            return attn.transpose(1, 2), lse[:, :, :n_query].unsqueeze(-1)
        if n_query % 2:
            query = torch.nn.functional.pad(query, (0, 0, 0, 1), mode='constant', value=0.)
            key = torch.nn.functional.pad(key, (0, 0, 0, 1), mode='constant', value=0.)
            value = torch.nn.functional.pad(value, (0, 0, 0, 1), mode='constant', value=0.)
        half = key.shape[2] // 2
        q_bd = query.view(batch_size, 2 * n_heads, half, query.shape[-1])
        k_bd = key.view(batch_size, 2 * n_heads, half, key.shape[-1])
        v_bd = value.view(batch_size, 2 * n_heads, half, value.shape[-1])
        attn_bd, lse_bd = self._forward_composed(q_bd, k_bd, v_bd, scale, True, proj)
        attn_bd = attn_bd.contiguous().view(batch_size, n_heads, -1, value.shape[-1])
        lse_bd = lse_bd.contiguous().view(batch_size, n_heads, -1, 1)
        attn_unmasked, lse_unmasked = self.forward_no_causal_mask(
            query[:, :, half:, :], key[:, :, :half, :], value[:, :, :half, :], scale, proj)
        attn_down, lse_down = ops.add_self_attentions(attn_bd[:, :, half:, :], lse_bd[:, :, half:, :],
                                                      attn_unmasked, lse_unmasked)
        attn = torch.cat((attn_bd[:, :, :half, :], attn_down), dim=-2)
        lse = torch.cat((lse_bd[:, :, :half, :], lse_down), dim=-2)
        if n_query % 2:
            attn = attn[:, :, :-1, :]
            lse = lse[:, :, :-1, :]
        return attn, lse

    def forward_no_causal_mask(self, query, key, value, scale, proj=None):
        """
            - sequence lengths must be divisible by block_size
            - proj (not in the reference): projection to hash with instead of the module's own
        """
        batch_size, head_size, n_query, dim = query.shape

        if self.min_seq_len > n_query:
            attn, lse = ops.flash_attn_func(query.transpose(1, 2), key.transpose(1, 2), value.transpose(1, 2),
                                            None, False, scale)
            lse = lse[:, :, :n_query]
        else:
            num_keys = 1 << self.lsh_num_projs
            query_sort_idx = ops.bucket_argsort(self.lsh.hash(query, proj), num_keys)
            key_sort_idx = ops.bucket_argsort(self.lsh.hash(key, proj), num_keys)
            estimator = {}
            if self.residual_estimator and self.sample_size > 0:
                estimator = dict(sample_bias=math.log(key.shape[2] / self.sample_size), mask_sampled_in_block=True)
            attn, lse = ops.hyper_attn_func(query.transpose(1, 2), key.transpose(1, 2), value.transpose(1, 2),
                                            query_sort_idx.transpose(1, 2), key_sort_idx.transpose(1, 2),
                                            self.block_size, self.sample_size, scale, self.smooth_block,
                                            sampled_idx=self.sampled_idx, **estimator)
        attn = attn.transpose(1, 2)
        return attn, lse.unsqueeze(-1)
