"""Angular LSH module with the reference's constructor, buffers and method names
(AngularLSHTriton, src/angular_lsh_triton.py:148-185); hashing runs in the HIP kernel."""
from __future__ import annotations

import torch

from . import ops


class AngularLSH(torch.nn.Module):
    """
    inputs:
        - num_projs: positive number of random projections of the hash function
        - dim: tuple whose last entry is the dimension of the hashed vectors, e.g. (1, 1, 64)
        - mat: a tensor whose last dimension equals dim[-1]
    output:
        - buckets: int32 tensor of shape mat.shape[:-1] with entries in [0, 2^num_projs - 1]
    """

    def __init__(self, num_projs, dim, rng=None):
        super().__init__()
        self.num_projs = num_projs
        if num_projs > 0:
            self.register_buffer('perm', self._unit_hamming_distance_array(self.num_projs), persistent=False)
            self.register_buffer('proj_dir', torch.randn(dim + (num_projs,), generator=rng), persistent=False)
            self.register_buffer('enc_vec', 2 ** torch.arange(self.num_projs).view(1, 1, 1, -1), persistent=False)
        else:
            raise ValueError("Invalid value for num_projs")

    @staticmethod
    def _unit_hamming_distance_array(size_n):
        # reflected Gray code: entry i is i ^ (i >> 1)
        i = torch.arange(1 << size_n, dtype=torch.int32)
        return i ^ (i >> 1)

    def hash(self, mat, proj=None):
        """Bucket ids from the HIP kernel; mat is (b, h, n, d) fp16/bf16 on the GPU.  proj (not in the
        reference): a projection to use instead of the module's own, e.g. one with zero rows added for
        zero-padded inputs."""
        proj = self.proj_dir if proj is None else proj
        if proj.dim() == 3:
            proj = proj.unsqueeze(0)
        return ops.lsh_hash(mat, proj)

    # the reference's method name for the device kernel
    hash_triton = hash

    def hash_torch(self, mat):
        """The same function written with torch operators (an API of the reference; the
        attention module never calls it)."""
        mask = torch.einsum('...nd,...dr -> ...nr', mat, self.proj_dir)
        mask = mask > 0
        bin_ids = (mask * self.enc_vec).sum(-1)
        return self.perm[bin_ids]

    def __repr__(self):
        return f"AngularLSH(num_proj={self.num_projs}, proj_dir.shape={self.proj_dir.shape})"


AngularLSHTriton = AngularLSH
