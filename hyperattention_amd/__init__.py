"""MI355X-native HyperAttention (HIP kernels behind the reference's module API): the forward path and
the backward of its attention operators."""
from .hyper_attention import HyperAttention
from .angular_lsh import AngularLSH, AngularLSHTriton
from .ops import (add_self_attentions, bucket_argsort, flash_attn_func, hyper_attn_func, indexing, lsh_hash)

__all__ = ["HyperAttention", "AngularLSH", "AngularLSHTriton", "add_self_attentions", "bucket_argsort",
           "flash_attn_func", "hyper_attn_func", "indexing", "lsh_hash"]
