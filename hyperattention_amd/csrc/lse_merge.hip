// Merge of two partial attentions computed over disjoint key sets.
// Stands in for add_self_attentions (src/attn_utils.py:6-24 of the reference):
//   c = 1 / (1 + exp(lse2 - lse1)); attn = c*attn1 + (1-c)*attn2; lse = lse1 - log(c + eps).
// c is rounded to the attention's type before it is used, as the reference does (src/attn_utils.py:21);
// the rest is fp32, with the same eps = 2^-23 inside the log.  One 8-element piece (16 bytes) per lane.
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
  const float c = (float)(T)(1.0f / (1.0f + __expf(x2 - x1)));
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

// All merges of the causal recursion in one pass over the rows.
// A row of a (batch, heads, n, d) tensor takes part in the un-masked call of level j (segments of n / 2^j
// rows) iff it lies in the second half of its segment.  Deepest level first, as the recursion returns
// (hyper_attention.py:86-89), its leaf result is merged with the results of those calls, each merge with the
// arithmetic of lse_merge_segments_kernel (weight rounded to the attention's type, merged rows rounded
// after every level).  All per-level arrays have the layout of the whole tensors; rows outside a level's
// second halves are neither read nor written.
//
// For a backward pass the row's weights are turned into shifted log-sum-exps on the way: the gradient of the
// output reaches the call of level j scaled by w_j = (1 - c_j) * prod of c_i over the shallower levels i the
// row takes part in, and the leaf by the product of all its c_i.  A call's gradients depend on its output
// gradient only through P = exp(s - lse) times that gradient, so scaling the gradient by w equals handing the
// call lse - log(w): those are written to shifted[j] and leaf_shifted (w = 0 gives +inf: P = 0).
namespace {

constexpr int MERGE_MAX_LEVELS = 24;

struct MergeLevels {
  const void* o_un[MERGE_MAX_LEVELS];
  const float* lse_un[MERGE_MAX_LEVELS];
  float* shifted[MERGE_MAX_LEVELS];
  int levels;
};

// MAXL: levels the instance is unrolled for (the recursion rarely goes deeper than 8)
template <typename T, int MAXL>
__global__ __launch_bounds__(256) void lse_merge_levels_kernel(const T* __restrict__ o_leaf, const float* __restrict__ lse_leaf,
                                                               T* __restrict__ out, float* __restrict__ lse_out,
                                                               float* __restrict__ leaf_shifted, MergeLevels lv,
                                                               int64_t rows, int64_t n, int pieces, int packed) {
  typedef typename ElemTraits<T>::vec8 vec8;
  const int64_t item = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t row = item / pieces;
  const int piece = (int)(item % pieces);
  if (row >= rows) return;
  // leaf number of the row inside its sequence: its bit (levels - 1 - j) says which half of its level-j
  // segment the row is in (such a half is 2^(levels - 1 - j) leaves long)
  const uint32_t leaf_no = (uint32_t)(row % n) / (uint32_t)(n >> lv.levels);
  const int64_t at = row * pieces * 8 + piece * 8;
  float x = lse_leaf[row];
  const float x_leaf = x;
  vec8 r = *reinterpret_cast<const vec8*>(o_leaf + at);
  float c_of[MAXL], x_of[MAXL];
  vec8 v_of[MAXL];
  // Row of the level-j arrays that holds this row's result.  Packed arrays keep only the rows a level writes,
  // the second halves of its segments of n >> j rows one after the other: (batch * heads, n / 2) rows.
  const int64_t seq = row / n;
  const uint32_t r_in = (uint32_t)(row - seq * n);
  auto level_row = [&](int j) -> int64_t {
    if (!packed) return row;
    // the segment number from the leaf number: shifts only (the leaf length need not be a power of two)
    const uint32_t len = (uint32_t)(n >> j), half = len >> 1, sg = leaf_no >> (lv.levels - j);
    return seq * (n >> 1) + (int64_t)sg * half + (r_in - sg * len - half);
  };
  // every load first, so that they are all in flight before the chain of weights (each level's weight needs
  // the log-sum-exp the deeper levels left) starts
#pragma unroll
  for (int j = MAXL - 1; j >= 0; --j) {
    c_of[j] = 1.0f;
    x_of[j] = 0.0f;
    if (j < lv.levels && ((leaf_no >> (lv.levels - 1 - j)) & 1u)) {
      const int64_t lr = level_row(j);
      x_of[j] = lv.lse_un[j][lr];
      v_of[j] = *reinterpret_cast<const vec8*>((const T*)lv.o_un[j] + lr * pieces * 8 + piece * 8);
    }
  }
#pragma unroll
  for (int j = MAXL - 1; j >= 0; --j) {
    if (j < lv.levels && ((leaf_no >> (lv.levels - 1 - j)) & 1u)) {
      const float c = (float)(T)(1.0f / (1.0f + __expf(x_of[j] - x)));
#pragma unroll
      for (int e = 0; e < 8; ++e) r[e] = (T)(c * (float)r[e] + (1.0f - c) * (float)v_of[j][e]);
      x = x - __logf(c + 1.1920929e-07f);
      c_of[j] = c;
    }
  }
  *reinterpret_cast<vec8*>(out + at) = r;
  if (piece != 0) return;
  lse_out[row] = x;
  if (!leaf_shifted) return;
  float log_w = 0.0f;  // log of the product of the weights c of the shallower levels
#pragma unroll
  for (int j = 0; j < MAXL; ++j) {
    if (j < lv.levels && ((leaf_no >> (lv.levels - 1 - j)) & 1u)) {
      lv.shifted[j][level_row(j)] = x_of[j] - log1pf(-c_of[j]) - log_w;
      log_w += logf(c_of[j]);
    }
  }
  leaf_shifted[row] = x_leaf - log_w;
}

}  // namespace

extern "C" int ha_lse_merge_levels(const void* o_leaf, const float* lse_leaf, const void* const* o_un,
                                   const float* const* lse_un, float* const* lse_shifted, float* leaf_shifted,
                                   void* out, float* lse_out, int levels, int64_t batch_heads, int64_t n, int64_t d,
                                   int dtype, int packed, void* stream) {
  HA_REQUIRE(o_leaf && lse_leaf && out && lse_out && (levels == 0 || (o_un && lse_un)), HA_ERR_NULL,
             "ha_lse_merge_levels: null pointer");
  HA_REQUIRE(dtype == HA_F16 || dtype == HA_BF16, HA_ERR_DTYPE, "ha_lse_merge_levels: Only support fp16 and bf16");
  HA_REQUIRE(levels >= 0 && levels <= MERGE_MAX_LEVELS, HA_ERR_UNSUPPORTED, "ha_lse_merge_levels: at most %d levels",
             MERGE_MAX_LEVELS);
  HA_REQUIRE(batch_heads > 0 && n > 0 && d > 0 && d % 8 == 0, HA_ERR_SHAPE,
             "ha_lse_merge_levels: sizes must be positive and d % 8 == 0");
  HA_REQUIRE((n >> levels) << levels == n, HA_ERR_SHAPE, "ha_lse_merge_levels: n must be divisible by 2^levels");
  HA_REQUIRE((leaf_shifted != nullptr) == (lse_shifted != nullptr) || levels == 0, HA_ERR_NULL,
             "ha_lse_merge_levels: leaf_shifted and lse_shifted go together");
  HA_REQUIRE(((uintptr_t)o_leaf % 16) == 0 && ((uintptr_t)out % 16) == 0, HA_ERR_SHAPE,
             "ha_lse_merge_levels: tensors must be 16-byte aligned");
  HA_REQUIRE(out != o_leaf && lse_out != lse_leaf, HA_ERR_UNSUPPORTED, "ha_lse_merge_levels: not in place");
  MergeLevels lv;
  lv.levels = levels;
  for (int j = 0; j < MERGE_MAX_LEVELS; ++j) {
    lv.o_un[j] = nullptr; lv.lse_un[j] = nullptr; lv.shifted[j] = nullptr;
  }
  for (int j = 0; j < levels; ++j) {
    HA_REQUIRE(o_un[j] && lse_un[j] && (!leaf_shifted || lse_shifted[j]), HA_ERR_NULL,
               "ha_lse_merge_levels: null pointer for level %d", j);
    HA_REQUIRE(((uintptr_t)o_un[j] % 16) == 0, HA_ERR_SHAPE, "ha_lse_merge_levels: tensors must be 16-byte aligned");
    lv.o_un[j] = o_un[j];
    lv.lse_un[j] = lse_un[j];
    lv.shifted[j] = leaf_shifted ? lse_shifted[j] : nullptr;
  }
  const int pieces = (int)(d / 8);
  const int64_t rows = batch_heads * n, items = rows * pieces;
  HA_REQUIRE((items + 255) / 256 < (1ll << 31), HA_ERR_SHAPE, "ha_lse_merge_levels: too many rows");
  dim3 grid((unsigned)((items + 255) / 256));
  hipStream_t s = (hipStream_t)stream;
#define HA_MERGE_LEVELS(TT, LL)                                                                                  \
  hipLaunchKernelGGL((lse_merge_levels_kernel<TT, LL>), grid, dim3(256), 0, s, (const TT*)o_leaf, lse_leaf, (TT*)out, \
                     lse_out, leaf_shifted, lv, rows, n, pieces, packed)
  if (dtype == HA_F16) {
    if (levels <= 8) HA_MERGE_LEVELS(f16_t, 8); else HA_MERGE_LEVELS(f16_t, MERGE_MAX_LEVELS);
  } else {
    if (levels <= 8) HA_MERGE_LEVELS(bf16_t, 8); else HA_MERGE_LEVELS(bf16_t, MERGE_MAX_LEVELS);
  }
#undef HA_MERGE_LEVELS
  return ha_launch_status("ha_lse_merge_levels");
}
