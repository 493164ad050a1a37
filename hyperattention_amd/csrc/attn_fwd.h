// Device-side parameter block of the attention kernels (validated and filled by the C entry points).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// x / y for 0 <= x < 2^31 as (x * magic) >> shift, with shift = 31 + ceil(log2 y) and
// magic = floor(2^shift / y) + 1 < 2^32 (exact for every such x)
struct ha_divisor {
  uint32_t magic;
  int shift;
};

constexpr int HA_MAX_RAGGED_LEVELS = 30;

struct ha_attn_kernel_params {
  const void* q;
  const void* k;
  const void* v;
  void* out;
  float* lse;
  const void* q_idx;        // gather mode only
  const void* k_idx;
  const void* sampled_idx;  // may be null: rows 0..sample-1
  int64_t q_sb, q_sh, q_sn;
  int64_t k_sb, k_sh, k_sn;
  int64_t v_sb, v_sh, v_sn;
  int64_t o_sb, o_sh, o_sn;
  int64_t lse_sb, lse_sh;
  int64_t qi_sb, qi_sh, qi_sn;
  int64_t ki_sb, ki_sh, ki_sn;
  int64_t si_sb, si_sh;
  int64_t seg_stride, q_seg_off, k_seg_off;
  int batch, heads, segs, kv_group;
  int n_q, n_k;
  int block_tiles;    // ceil(block_size / 128)
  int sample_chunks;  // sample_size / 64
  int smooth, accumulate, idx64;
  int qk_pieces, v_pieces;  // 16-byte pieces in a row of q/k and of v/out (filled by ha_attn_launch)
  // residual estimator (gathered kernel, REWEIGHT instances only)
  const int32_t* sampled_pos;  // sorted-order position of every sampled key; null: nothing is masked
  float sample_bias_raw;       // added to the raw q.k of a sampled key: bias / softmax scale
  float scale_log2;   // softmax scale * log2(e)
  // Queries of the last segment of every head that exist (gathered kernel): an entry of its query order at or
  // past this number names a row that is not there (the zero row the causal recursion appends to an odd
  // length, hyper_attention.py:61-64); it is placed like any other row and its result is dropped.
  int n_q_last;
  // first row of segment g in the out / lse tensors: o_seg_off + g * o_seg_stride (= the query side's unless
  // the caller packs the rows a call writes)
  int64_t o_seg_off, o_seg_stride;
  // Streaming gathered kernel: consecutive query tiles of one (virtual) head per workgroup (the last
  // workgroup of a head may have fewer); 1: the one-tile kernels
  int tiles_per_wg;
  // Ragged segments (exact kernels; rag_levels < 0: regular).  Inside a causal recursion with odd lengths the
  // segments of a level neither start at multiples of one stride nor hold the same number of rows: level i
  // cuts a segment of (padded) length 2*rag_half[i] into two, and the rows that exist are the first rag_n of
  // the whole sequence.  Segment number `seg` has rag_levels bits, most significant first: bit i says which
  // half of its level-i ancestor it lies in.  rag_split: the launch is the off-diagonal part of the level
  // below (queries = second half, keys = first half of the segment, halves of rag_half[rag_levels] rows).
  int rag_levels, rag_split, rag_n;
  int rag_half[HA_MAX_RAGGED_LEVELS + 1];
  // the divisors of the workgroup -> (head, segment, tile) decomposition as multiply-and-shift
  // constants (filled by ha_attn_launch): the kernel never divides
  ha_divisor div_qtiles, div_segs, div_heads, div_kv_heads, div_kv_group, div_block_tiles;
};

int ha_attn_launch(const ha_attn_kernel_params& p, int d, int dv, int dtype, bool gather, bool causal, bool reweight,
                   hipStream_t stream);

// argument checks shared by the forward and backward entry points (defined in api.hip); `who` names
// the entry point in the error message
int ha_check_operands(const ha_attn_operands& t, const char* who);
int ha_check_block_attn_args(const ha_block_attn_args& a, const char* who);
