"""HyperAttention module: same constructor and forward signature as the reference
(hyper_attention.py:9-132), computed by the HIP library.

Contiguous inputs whose causal recursion only meets even lengths take one library call
(ha_forward: hash once, all sorts in one batch, leaves, then each level merged in place).  Other
shapes (an odd length somewhere in the recursion, more than 8 projections) are composed here from
the same HIP operators, following the reference's recursion step by step.
"""
from __future__ import annotations

import torch

from . import ops
from .angular_lsh import AngularLSH


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
            attn, lse = self._forward_composed(query.contiguous(), key.contiguous(), value.contiguous(), scale, causal)

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
