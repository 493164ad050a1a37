"""HyperAttention module: same constructor and forward signature as the reference
(hyper_attention.py:9-132), computed by the HIP library.

Contiguous inputs whose causal recursion only meets even lengths take one library call
(ha_forward: hash once, all sorts in one batch, leaves, then each level merged in place).  Other
shapes (an odd length somewhere in the recursion, more than 8 projections) are composed here from
the same HIP operators, following the reference's recursion step by step.

With inputs that require grad the forward keeps what the backward needs: the non-causal case is one
differentiable operator call, the causal recursion with even lengths runs on views of the tensors
with the calls' gradients accumulated by the kernels (_CausalRecursionFunc), anything else operator
by operator under torch autograd.
"""
from __future__ import annotations

import ctypes

import torch

from . import _lib, ops
from .angular_lsh import AngularLSH


class _CausalRecursionFunc(torch.autograd.Function):
    """The causal divide-and-conquer (hyper_attention.py:51-96) with its gradient, for lengths that stay
    even down to the leaves.

    Same arithmetic as the reference's recursion under autograd: exact causal attention on the leaves,
    one un-masked call per level on (second-half queries, first-half keys/values), merges with the
    weight rounded to the attention's type (src/attn_utils.py:21-23), and log-sum-exps that carry no
    gradient (src/hyper_attn_triton.py:922-945).  What differs is the bookkeeping: every call reads and
    writes strided views of the (batch, heads, n, d) tensors through the C entry points, the merges
    run in place, and in the backward the gradients of the calls are accumulated by the kernels
    (`accumulate`), so there are no concatenations, zero-padded slice gradients or gradient additions.
    """

    @staticmethod
    def forward(ctx, module, scale, query, key, value):
        b, h, n, d = query.shape
        lens = [n]
        while lens[-1] > module.min_seq_len:
            lens.append(lens[-1] // 2)
        levels = len(lens) - 1
        lib, stream = _lib.lib(), ops._stream(query)
        f32 = dict(device=query.device, dtype=torch.float32)
        heads = lambda x, j: x.view(b, h << j, lens[j], x.shape[-1])

        with torch.cuda.device(query.device):
            # leaves: exact causal attention on every segment of lens[levels] rows
            o_leaf, lse_leaf = torch.empty_like(query), torch.empty((b, h, n), **f32)
            t = ops._operands(heads(query, levels), heads(key, levels), heads(value, levels), heads(o_leaf, levels),
                              lse_leaf.view(b, h << levels, lens[levels]), scale, layout_bnhd=False,
                              lse_row_stride=lens[levels])
            _lib.check(lib.ha_flash_attn_fwd(ctypes.byref(t), 1, stream))
            out, lse = o_leaf.clone(), lse_leaf.clone()

            # a row's bucket does not depend on the level: hash once, sort per level
            hashed = [j for j in range(levels) if not module.min_seq_len > lens[j + 1]]
            if hashed:
                buckets_q, buckets_k = module.lsh.hash(query), module.lsh.hash(key)
            per_level = []
            for j in reversed(range(levels)):  # deepest level first, as the recursion returns
                H, half = h << j, lens[j + 1]
                q2 = query.view(b, H, 2, half, d)[:, :, 1]
                k1 = key.view(b, H, 2, half, d)[:, :, 0]
                v1 = value.view(b, H, 2, half, d)[:, :, 0]
                o_un, lse_un = torch.empty((b, H, half, d), device=query.device, dtype=query.dtype), torch.empty((b, H, half), **f32)
                if module.min_seq_len > half:  # hyper_attention.py:109
                    q_idx = k_idx = None
                    t = ops._operands(q2, k1, v1, o_un, lse_un, scale, layout_bnhd=False, lse_row_stride=half)
                    _lib.check(lib.ha_flash_attn_fwd(ctypes.byref(t), 0, stream))
                else:
                    num_keys = 1 << module.lsh_num_projs
                    q_idx = ops.bucket_argsort(buckets_q.view(b, H, 2, half)[:, :, 1], num_keys, torch.int32)
                    k_idx = ops.bucket_argsort(buckets_k.view(b, H, 2, half)[:, :, 0], num_keys, torch.int32)
                    a, keep = ops._block_attn_args(q2, k1, v1, o_un, lse_un, q_idx, k_idx, module.block_size,
                                                   module.sample_size, scale, module.smooth_block, module.sampled_idx,
                                                   layout_bnhd=False)
                    _lib.check(lib.ha_block_attn_fwd(ctypes.byref(a), stream))
                # merge into the second halves, in place; c: the weight of what was there (fp32 copy of the
                # weight rounded to the attention's type)
                out2 = out.view(b, H, 2, half, d)[:, :, 1]
                lse2 = lse.view(b, H, 2, half)[:, :, 1]
                c = torch.empty((b, H, half), **f32)
                _lib.check(lib.ha_lse_merge_segments(
                    out2.data_ptr(), lse2.data_ptr(), o_un.data_ptr(), lse_un.data_ptr(), out2.data_ptr(),
                    lse2.data_ptr(), c.data_ptr(), b * H, half, d, 2 * half * d, d, half * d, d, 2 * half * d, d,
                    2 * half, half, 2 * half, half, ops._dtype_code(query), stream))
                per_level.append((j, o_un, lse_un, c, q_idx, k_idx))

        tensors = [query, key, value, o_leaf, lse_leaf]
        layout = []
        for j, o_un, lse_un, c, q_idx, k_idx in per_level:
            layout.append((j, q_idx is not None))
            tensors += [o_un, lse_un, c] + ([q_idx, k_idx] if q_idx is not None else [])
        ctx.save_for_backward(*tensors)
        ctx.layout, ctx.lens, ctx.module, ctx.scale = layout, lens, module, scale
        lse = lse.unsqueeze(-1)
        ctx.mark_non_differentiable(lse)
        return out, lse

    @staticmethod
    def backward(ctx, dout, dlse=None):
        saved = list(ctx.saved_tensors)
        query, key, value, o_leaf, lse_leaf = saved[:5]
        rest = saved[5:]
        module, scale, lens = ctx.module, ctx.scale, ctx.lens
        b, h, n, d = query.shape
        levels = len(lens) - 1
        lib, stream = _lib.lib(), ops._stream(query)
        heads = lambda x, j: x.view(b, h << j, lens[j], x.shape[-1])

        per_level = {}
        for j, hashed in ctx.layout:
            o_un, lse_un, c = rest[:3]
            q_idx, k_idx = (rest[3], rest[4]) if hashed else (None, None)
            rest = rest[5:] if hashed else rest[3:]
            per_level[j] = (o_un, lse_un, c, q_idx, k_idx)

        with torch.cuda.device(query.device):
            # The gradient of the output splits at every merge, from the top level down: (1 - c) of it goes
            # to the un-masked call of the level, c of it further down.  A call's gradients are linear in
            # the output gradient it is given, and that enters only through P = exp(s - lse): weighting a
            # row's output gradient by w equals giving the call the log-sum-exp lse - log(w) for that row
            # (w = 0: lse = +inf, P = 0).  So every call gets the output gradient as it is and a shifted
            # copy of its small log-sum-exp array, and no weighted copy of the gradient is ever made.
            dout = dout.contiguous()
            log_w = torch.zeros((b, h, n), device=query.device, dtype=torch.float32)
            lse_shifted = {}
            for j in range(levels):
                H, half = h << j, lens[j + 1]
                lse_un, c = per_level[j][1], per_level[j][2]
                log_w2 = log_w.view(b, H, 2, half)[:, :, 1]
                lse_shifted[j] = lse_un - torch.log1p(-c) - log_w2
                log_w2.add_(torch.log(c))
            lse_leaf = lse_leaf - log_w

            dq, dk, dv = torch.empty_like(query), torch.empty_like(key), torch.empty_like(value)
            # leaves first: they write every row of dq, dk, dv; the levels then add to their views
            t = ops._operands(heads(query, levels), heads(key, levels), heads(value, levels), heads(o_leaf, levels),
                              lse_leaf.view(b, h << levels, lens[levels]), scale, layout_bnhd=False,
                              lse_row_stride=lens[levels])
            g, ws = ops._attn_grads(t, heads(dout, levels), heads(dq, levels), heads(dk, levels), heads(dv, levels),
                                    layout_bnhd=False)
            _lib.check(lib.ha_flash_attn_bwd(ctypes.byref(t), 1, ctypes.byref(g), stream))
            for j in range(levels):
                H, half = h << j, lens[j + 1]
                o_un, _, _, q_idx, k_idx = per_level[j]
                lse_un = lse_shifted[j]
                do2 = dout.view(b, H, 2, half, d)[:, :, 1]
                q2 = query.view(b, H, 2, half, d)[:, :, 1]
                k1 = key.view(b, H, 2, half, d)[:, :, 0]
                v1 = value.view(b, H, 2, half, d)[:, :, 0]
                dq2 = dq.view(b, H, 2, half, d)[:, :, 1]
                dk1 = dk.view(b, H, 2, half, d)[:, :, 0]
                dv1 = dv.view(b, H, 2, half, d)[:, :, 0]
                if q_idx is None:
                    t = ops._operands(q2, k1, v1, o_un, lse_un, scale, layout_bnhd=False, lse_row_stride=half)
                    g, ws = ops._attn_grads(t, do2, dq2, dk1, dv1, layout_bnhd=False, accumulate=True)
                    _lib.check(lib.ha_flash_attn_bwd(ctypes.byref(t), 0, ctypes.byref(g), stream))
                else:
                    a, keep = ops._block_attn_args(q2, k1, v1, o_un, lse_un, q_idx, k_idx, module.block_size,
                                                   module.sample_size, scale, module.smooth_block, module.sampled_idx,
                                                   layout_bnhd=False)
                    g, ws = ops._attn_grads(a.t, do2, dq2, dk1, dv1, layout_bnhd=False, accumulate=True,
                                            sample_size=module.sample_size)
                    _lib.check(lib.ha_block_attn_bwd(ctypes.byref(a), ctypes.byref(g), stream))
        return None, None, dq, dk, dv


class HyperAttention(torch.nn.Module):

    def __init__(self, input_dim=64, lsh_num_projs=8, block_size=256, sample_size=256, min_seq_len=2048,
                 smooth_block=False, **kwargs):
        """
        - block_size and sample_size must be divisible by 128
        Optional keyword hooks (not in the reference, for reproducible runs): `rng` (torch.Generator
        for the projection), `proj_dir` (explicit (input_dim, lsh_num_projs) projection) and
        `sampled_idx` (explicit sampled key rows, shape (sample_size,)).
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
        if dim not in ops.KERNEL_HEAD_DIMS or dim_v != dim:
            # head dims the kernels are not built for (and a value dim different from the q/k dim) run
            # zero-padded: zero columns change neither the projections, nor q.k, nor the wanted outputs
            assert dim <= 128 and dim_v <= 128, "FlashAttention only support head dimensions up to 128"
            wide = ops.padded_head_dim(max(dim, dim_v))
            pad = lambda x: torch.nn.functional.pad(x, (0, wide - x.shape[-1]))
            proj = self.lsh.proj_dir
            self.lsh.proj_dir = torch.nn.functional.pad(proj, (0, 0, 0, wide - dim))
            try:
                res = self.forward(pad(query), pad(key), pad(value), scale, causal, True)
            finally:
                self.lsh.proj_dir = proj
            attn, lse = res[0][..., :dim_v], res[1]
            return (attn, lse) if return_lse else attn

        # gradients are taken operator by operator, as in the reference (each attention operator has its own
        # backward and the merges are differentiable tensor arithmetic); the one-call forward has none
        if (ops.forward_plan_supported(n_key, self.min_seq_len, causal is not False, self.lsh_num_projs)
                and not ops._wants_grad(query, key, value)):
            attn, lse = ops.hyper_forward(
                query, key, value, self.lsh.proj_dir, scale=scale, causal=causal is not False,
                lsh_num_projs=self.lsh_num_projs, block_size=self.block_size, sample_size=self.sample_size,
                min_seq_len=self.min_seq_len, smooth_block=self.smooth_block, sampled_idx=self.sampled_idx)
            if causal is not False and n_key <= self.min_seq_len:
                # the reference returns the exact kernel's padded 3-d lse for a top-level leaf
                n_rounded = -(-n_key // 128) * 128
                lse = torch.nn.functional.pad(lse, (0, n_rounded - n_key))
            else:
                lse = lse.unsqueeze(-1)
        else:
            if key.shape[1] != query.shape[1]:
                # grouped-query inputs on the operator-by-operator path: it follows the reference, which
                # wants as many k/v heads as q heads (hyper_attention.py:43,67-68)
                group = query.shape[1] // key.shape[1]
                key, value = key.repeat_interleave(group, dim=1), value.repeat_interleave(group, dim=1)
            query, key, value = query.contiguous(), key.contiguous(), value.contiguous()
            if (causal is not False and n_key > self.min_seq_len and ops._wants_grad(query, key, value)
                    and ops.forward_plan_supported(n_key, self.min_seq_len, True, 8)):
                # every level has an even length: the recursion and its gradient on views, in place
                attn, lse = _CausalRecursionFunc.apply(self, scale, query, key, value)
            else:
                attn, lse = self._forward_composed(query, key, value, scale, causal)

        if not return_lse:
            return attn
        else:
            return attn, lse

    # ---- the reference's recursion, operator by operator (shapes ha_forward does not take) --------
    def _forward_composed(self, query, key, value, scale, causal):
        batch_size, n_heads, n_key, dim = key.shape
        n_query = query.shape[2]
        if causal is False:
            return self.forward_no_causal_mask(query, key, value, scale)
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
        attn_bd, lse_bd = self._forward_composed(q_bd, k_bd, v_bd, scale, True)
        attn_bd = attn_bd.contiguous().view(batch_size, n_heads, -1, value.shape[-1])
        lse_bd = lse_bd.contiguous().view(batch_size, n_heads, -1, 1)
        attn_unmasked, lse_unmasked = self.forward_no_causal_mask(
            query[:, :, half:, :], key[:, :, :half, :], value[:, :, :half, :], scale)
        attn_down, lse_down = ops.add_self_attentions(attn_bd[:, :, half:, :], lse_bd[:, :, half:, :],
                                                      attn_unmasked, lse_unmasked)
        attn = torch.cat((attn_bd[:, :, :half, :], attn_down), dim=-2)
        lse = torch.cat((lse_bd[:, :, :half, :], lse_down), dim=-2)
        if n_query % 2:
            attn = attn[:, :, :-1, :]
            lse = lse[:, :, :-1, :]
        return attn, lse

    def forward_no_causal_mask(self, query, key, value, scale):
        """
            - sequence lengths must be divisible by block_size
        """
        batch_size, head_size, n_query, dim = query.shape

        if self.min_seq_len > n_query:
            attn, lse = ops.flash_attn_func(query.transpose(1, 2), key.transpose(1, 2), value.transpose(1, 2),
                                            None, False, scale)
            lse = lse[:, :, :n_query]
        else:
            num_keys = 1 << self.lsh_num_projs
            query_sort_idx = ops.bucket_argsort(self.lsh.hash(query), num_keys)
            key_sort_idx = ops.bucket_argsort(self.lsh.hash(key), num_keys)
            attn, lse = ops.hyper_attn_func(query.transpose(1, 2), key.transpose(1, 2), value.transpose(1, 2),
                                            query_sort_idx.transpose(1, 2), key_sort_idx.transpose(1, 2),
                                            self.block_size, self.sample_size, scale, self.smooth_block,
                                            sampled_idx=self.sampled_idx)
        attn = attn.transpose(1, 2)
        return attn, lse.unsqueeze(-1)
