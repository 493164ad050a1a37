// Merge of two partial attentions computed over disjoint key sets.
// Stands in for add_self_attentions (src/attn_utils.py:6-24 of the reference):
//   c = 1 / (1 + exp(lse2 - lse1)); attn = c*attn1 + (1-c)*attn2; lse = lse1 - log(c + eps).
// The arithmetic here is fp32 throughout (the reference rounds c to fp16/bf16 first), with the
// same eps = 2^-23 inside the log.  One 8-element piece (16 bytes) per lane.
#include "ha_common.h"

namespace {

template <typename T>
__global__ __launch_bounds__(256) void lse_merge_kernel(const T* a1, const float* l1, const T* a2, const float* l2,
                                                        T* ao, float* lo, int64_t rows,
                                                        int pieces, int64_t s1, int64_t s2, int64_t so,
                                                        int64_t ls1, int64_t ls2, int64_t lso) {
  typedef typename ElemTraits<T>::vec8 vec8;
  const int64_t item = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t row = item / pieces;
  const int piece = (int)(item % pieces);
  if (row >= rows) return;
  const float x1 = l1[row * ls1], x2 = l2[row * ls2];
  const float c = 1.0f / (1.0f + __expf(x2 - x1));
  const vec8 v1 = *reinterpret_cast<const vec8*>(a1 + row * s1 + piece * 8);
  const vec8 v2 = *reinterpret_cast<const vec8*>(a2 + row * s2 + piece * 8);
  vec8 r;
#pragma unroll
  for (int e = 0; e < 8; ++e) r[e] = (T)(c * (float)v1[e] + (1.0f - c) * (float)v2[e]);
  *reinterpret_cast<vec8*>(ao + row * so + piece * 8) = r;
  if (piece == 0) lo[row * lso] = x1 - __logf(c + 1.1920929e-07f);
}

}  // namespace

extern "C" int ha_lse_merge(const void* attn1, const float* lse1, const void* attn2, const float* lse2,
                            void* attn_out, float* lse_out, int64_t rows, int64_t d, int64_t attn1_stride,
                            int64_t attn2_stride, int64_t out_stride, int64_t lse1_stride, int64_t lse2_stride,
                            int64_t lse_out_stride, int dtype, void* stream) {
  HA_REQUIRE(attn1 && lse1 && attn2 && lse2 && attn_out && lse_out, HA_ERR_NULL, "ha_lse_merge: null pointer");
  HA_REQUIRE(dtype == HA_F16 || dtype == HA_BF16, HA_ERR_DTYPE, "ha_lse_merge: Only support fp16 and bf16");
  HA_REQUIRE(rows > 0 && d > 0 && d % 8 == 0, HA_ERR_SHAPE, "ha_lse_merge: rows > 0 and d % 8 == 0 required");
  HA_REQUIRE(attn1_stride % 8 == 0 && attn2_stride % 8 == 0 && out_stride % 8 == 0 &&
                 ((uintptr_t)attn1 % 16) == 0 && ((uintptr_t)attn2 % 16) == 0 && ((uintptr_t)attn_out % 16) == 0,
             HA_ERR_SHAPE, "ha_lse_merge: rows must be 16-byte aligned");
  const int pieces = (int)(d / 8);
  const int64_t items = rows * pieces;
  // In place, the lanes of a row read its log-sum-exps before one of them writes the merged one: that
  // holds inside a wave, so a row's d/8 lanes must not straddle two waves.
  const bool in_place = lse_out == lse1 || lse_out == lse2 || attn_out == attn1 || attn_out == attn2;
  HA_REQUIRE(!in_place || 64 % pieces == 0, HA_ERR_UNSUPPORTED,
             "ha_lse_merge: in place needs a head dimension of 8, 16, 32, 64, 128, 256 or 512");
  HA_REQUIRE((items + 255) / 256 < (1ll << 31), HA_ERR_SHAPE, "ha_lse_merge: too many rows");
  dim3 grid((unsigned)((items + 255) / 256));
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HA_F16)
    hipLaunchKernelGGL((lse_merge_kernel<f16_t>), grid, dim3(256), 0, s, (const f16_t*)attn1, lse1,
                       (const f16_t*)attn2, lse2, (f16_t*)attn_out, lse_out, rows, pieces, attn1_stride,
                       attn2_stride, out_stride, lse1_stride, lse2_stride, lse_out_stride);
  else
    hipLaunchKernelGGL((lse_merge_kernel<bf16_t>), grid, dim3(256), 0, s, (const bf16_t*)attn1, lse1,
                       (const bf16_t*)attn2, lse2, (bf16_t*)attn_out, lse_out, rows, pieces, attn1_stride,
                       attn2_stride, out_stride, lse1_stride, lse2_stride, lse_out_stride);
  return ha_launch_status("ha_lse_merge");
}

// The same merge for rows that come in equal segments with their own strides (the second halves of
// the heads of a (batch, heads, n, d) tensor, say), in place if wanted, with the weight c of the first
// input written out as well: what the causal recursion needs per level, in one pass.  c is rounded to
// the attention's type before it is used, as the reference does (src/attn_utils.py:21).
namespace {

template <typename T>
__global__ __launch_bounds__(256) void lse_merge_segments_kernel(const T* a1, const float* l1, const T* a2,
                                                                 const float* l2, T* ao, float* lo,
                                                                 float* __restrict__ wo, int64_t rows,
                                                                 int64_t seg_len, int pieces, int64_t a1_ss, int64_t a1_rs,
                                                                 int64_t a2_ss, int64_t a2_rs, int64_t ao_ss, int64_t ao_rs,
                                                                 int64_t l1_ss, int64_t l2_ss, int64_t lo_ss, int64_t wo_ss) {
  typedef typename ElemTraits<T>::vec8 vec8;
  const int64_t item = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t row = item / pieces;
  const int piece = (int)(item % pieces);
  if (row >= rows) return;
  const int64_t seg = row / seg_len, i = row - seg * seg_len;
  const float x1 = l1[seg * l1_ss + i], x2 = l2[seg * l2_ss + i];
  const float c = (float)(T)(1.0f / (1.0f + __expf(x2 - x1)));
  const vec8 v1 = *reinterpret_cast<const vec8*>(a1 + seg * a1_ss + i * a1_rs + piece * 8);
  const vec8 v2 = *reinterpret_cast<const vec8*>(a2 + seg * a2_ss + i * a2_rs + piece * 8);
  vec8 r;
#pragma unroll
  for (int e = 0; e < 8; ++e) r[e] = (T)(c * (float)v1[e] + (1.0f - c) * (float)v2[e]);
  *reinterpret_cast<vec8*>(ao + seg * ao_ss + i * ao_rs + piece * 8) = r;
  if (piece == 0) {
    lo[seg * lo_ss + i] = x1 - __logf(c + 1.1920929e-07f);
    if (wo) wo[seg * wo_ss + i] = c;
  }
}

}  // namespace

extern "C" int ha_lse_merge_segments(const void* attn1, const float* lse1, const void* attn2, const float* lse2,
                                     void* attn_out, float* lse_out, float* weight_out, int64_t segs, int64_t seg_len,
                                     int64_t d, int64_t attn1_seg_stride, int64_t attn1_row_stride,
                                     int64_t attn2_seg_stride, int64_t attn2_row_stride, int64_t out_seg_stride,
                                     int64_t out_row_stride, int64_t lse1_seg_stride, int64_t lse2_seg_stride,
                                     int64_t lse_out_seg_stride, int64_t weight_seg_stride, int dtype, void* stream) {
  HA_REQUIRE(attn1 && lse1 && attn2 && lse2 && attn_out && lse_out, HA_ERR_NULL, "ha_lse_merge_segments: null pointer");
  HA_REQUIRE(dtype == HA_F16 || dtype == HA_BF16, HA_ERR_DTYPE, "ha_lse_merge_segments: Only support fp16 and bf16");
  HA_REQUIRE(segs > 0 && seg_len > 0 && d > 0 && d % 8 == 0, HA_ERR_SHAPE,
             "ha_lse_merge_segments: segs, seg_len > 0 and d % 8 == 0 required");
  const int64_t strides[] = {attn1_seg_stride, attn1_row_stride, attn2_seg_stride, attn2_row_stride, out_seg_stride, out_row_stride};
  for (int64_t s : strides) HA_REQUIRE(s % 8 == 0, HA_ERR_SHAPE, "ha_lse_merge_segments: rows must be 16-byte aligned");
  HA_REQUIRE(((uintptr_t)attn1 % 16) == 0 && ((uintptr_t)attn2 % 16) == 0 && ((uintptr_t)attn_out % 16) == 0, HA_ERR_SHAPE,
             "ha_lse_merge_segments: tensors must be 16-byte aligned");
  const int pieces = (int)(d / 8);
  const int64_t rows = segs * seg_len, items = rows * pieces;
  HA_REQUIRE((items + 255) / 256 < (1ll << 31), HA_ERR_SHAPE, "ha_lse_merge_segments: too many rows");
  // In place, the lanes of a row read its log-sum-exps before one of them writes the merged one: that
  // holds inside a wave, so a row's d/8 lanes must not straddle two waves.
  const bool in_place = lse_out == lse1 || lse_out == lse2 || attn_out == attn1 || attn_out == attn2;
  HA_REQUIRE(!in_place || 64 % pieces == 0, HA_ERR_UNSUPPORTED,
             "ha_lse_merge_segments: in place needs a head dimension of 8, 16, 32, 64, 128, 256 or 512");
  dim3 grid((unsigned)((items + 255) / 256));
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HA_F16)
    hipLaunchKernelGGL((lse_merge_segments_kernel<f16_t>), grid, dim3(256), 0, s, (const f16_t*)attn1, lse1,
                       (const f16_t*)attn2, lse2, (f16_t*)attn_out, lse_out, weight_out, rows, seg_len, pieces,
                       attn1_seg_stride, attn1_row_stride, attn2_seg_stride, attn2_row_stride, out_seg_stride,
                       out_row_stride, lse1_seg_stride, lse2_seg_stride, lse_out_seg_stride, weight_seg_stride);
  else
    hipLaunchKernelGGL((lse_merge_segments_kernel<bf16_t>), grid, dim3(256), 0, s, (const bf16_t*)attn1, lse1,
                       (const bf16_t*)attn2, lse2, (bf16_t*)attn_out, lse_out, weight_out, rows, seg_len, pieces,
                       attn1_seg_stride, attn1_row_stride, attn2_seg_stride, attn2_row_stride, out_seg_stride,
                       out_row_stride, lse1_seg_stride, lse2_seg_stride, lse_out_seg_stride, weight_seg_stride);
  return ha_launch_status("ha_lse_merge_segments");
}
