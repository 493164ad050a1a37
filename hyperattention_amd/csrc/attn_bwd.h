// Kernel-level parameters of the attention backward passes (internal; the C ABI is in
// include/hyperattn.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ha_common.h"

// which gradient a launch computes, and over which (query, key) pairs
enum ha_bwd_pass {
  HA_BWD_DQ_EXACT = 0,     // dq of exact attention
  HA_BWD_DQ_BLOCK = 1,     // dq of the sorted blocks and the sampled keys
  HA_BWD_DKV_EXACT = 2,    // dk, dv of exact attention
  HA_BWD_DKV_BLOCK = 3,    // dk, dv: what the sorted blocks contribute
  HA_BWD_DKV_SAMPLED = 4,  // dk, dv: what the sampled keys receive from every query
};

struct ha_attn_bwd_params {
  const void *q, *k, *v, *dout;
  const void* out;   // the forward's output and log-sum-exp: read by the dq passes, which write `stats`
  const float* lse;
  f32x2* stats;  // per query {log-sum-exp * log2(e), -sum_c dO*O}, contiguous (batch, heads, n_q): written
                 // by the dq pass of a call for the dk/dv passes that follow it
  void* dq;
  void *dk, *dv;       // written directly by the exact and the block passes
  float *dk32, *dv32;  // fp32 (batch, heads / kv_group, sample_size, d): sums of the sampled keys, by slot
  int64_t q_sb, q_sh, q_sn;
  int64_t k_sb, k_sh, k_sn;
  int64_t v_sb, v_sh, v_sn;
  int64_t do_sb, do_sh, do_sn;
  int64_t o_sb, o_sh, o_sn;
  int64_t lse_sb, lse_sh;
  int64_t dq_sb, dq_sh, dq_sn;
  int64_t dk_sb, dk_sh, dk_sn;
  int64_t dv_sb, dv_sh, dv_sn;
  const void *q_idx, *k_idx, *sampled_idx;
  int64_t qi_sb, qi_sh, qi_sn;
  int64_t ki_sb, ki_sh, ki_sn;
  int64_t si_sb, si_sh;
  int batch, heads, kv_group;
  int segs;                                // segments per head, as in the forward
  int64_t seg_stride, q_seg_off, k_seg_off;  // rows
  int64_t o_seg_stride, o_seg_off;           // the forward's out / lse (the query side's unless packed)
  int n_q, n_k;
  int block_tiles;  // ceil(block_size / 128)
  int sample_size;
  int smooth, idx64;
  int accumulate;  // add to dq / dk / dv instead of overwriting them
  int q_split;  // sampled-key pass: queries per workgroup
  float scale, scale_log2;
};
