// Angular LSH bucket ids: sign bits of r random projections, Gray-coded.
// Follows the definition in src/angular_lsh_triton.py:76-88 and :175-179 of the reference
// (bit_j = [x . P[:, j] > 0], bin = sum_j bit_j << j, bucket = perm[bin], perm[i] = i ^ (i >> 1)).
//
// lsh_hash_mfma_kernel: a wave projects 16 rows at a time with v_mfma_f32_16x16x32 (rows x 16 projection
// slots, fp32 accumulation), reading the rows straight from HBM as MFMA operands, so the kernel is purely
// bandwidth bound.  Built for rows of 32, 64, 128 and 256 elements; a row of any other multiple of 8
// elements runs in the next width with its missing elements (and the missing rows of the projection) read
// as zeros.  fp32 accumulation cannot decide the
// sign of a projection that nearly cancels, so a second MFMA on |x| and |P| gives sum |x_k P_kj|, which
// bounds the accumulation error of any summation order (d * 2^-23 * sum, used with a factor 2 margin;
// fp16/bf16 products are exact in fp32 and subnormal inputs are not flushed).  Whenever some
// |projection| is inside that bound, the 16-row tile is recomputed in fp64 (products exact, sum exact
// to 2^-53), which happens for well under 1 % of the tiles on random data.
#include "ha_common.h"
#include "bucket_sort.h"

namespace {

template <typename T>
struct HashMfma;
template <>
struct HashMfma<f16_t> {
  static __device__ __forceinline__ f32x4 run(f16x8 a, f16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};
template <>
struct HashMfma<bf16_t> {
  static __device__ __forceinline__ f32x4 run(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};

constexpr int HASH_TILES_PER_WAVE = 32;  // tiles of 512 elements (16 MFMA rows of 32 elements)
constexpr int HASH_UNROLL = 8;           // tiles in flight per wave

// A data row of D elements is cut into PARTS = D/32 MFMA rows of 32 elements, so that one load
// instruction of the wave (16 bytes per lane) covers whole rows: 16/PARTS data rows of D*2 bytes.
// MFMA row m = (data row)*PARTS + part; lane (m = lane%16, kg = lane/16) holds elements
// part*32 + 8*kg .. +7 of its data row.  The C registers i = 0..3 of a lane are MFMA rows 4*kg + i
// of projection slot lane%16; the partial projections of one data row are summed afterwards.
// Up to two tensors per launch (queries and keys of one forward): blockIdx.y + blockIdx.z * gridDim.y counts
// the (batch, head) sequences of the first tensor, then those of the second (a grid dimension holds 65535).
struct HashTensors {
  const void* x[2];
  void* out[2];        // bucket ids, (batch, heads, n) contiguous, int32 or (OUT8) one byte each
  int64_t sb[2], sh[2], sn[2];
  int heads[2];
  int seqs0;           // batch * heads of the first tensor
  int seqs;            // sequences of both tensors together
  int64_t n_read;      // rows of a sequence that exist; rows from there up to n hash as zero rows
};

template <typename T, int D, bool OUT8>
__global__ __launch_bounds__(256) void lsh_hash_mfma_kernel(const HashTensors ten, const T* __restrict__ proj, int64_t n,
                                                            int r, int64_t psb, int64_t psh, int d_real) {
  typedef typename ElemTraits<T>::vec8 vec8;
  constexpr int PARTS = D / 32;
  constexpr int ROWS = 16 / PARTS;            // data rows per tile
  constexpr int NS = PARTS >= 4 ? 1 : 4 / PARTS;  // data rows per lane (sums of C registers)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int seq = (int)(blockIdx.y + blockIdx.z * gridDim.y);
  if (seq >= ten.seqs) return;  // the last layer of the grid may be partly empty
  const int which = seq >= ten.seqs0 ? 1 : 0;
  const int bh = seq - (which ? ten.seqs0 : 0);
  const int heads = ten.heads[which];
  const int b = bh / heads, h = bh % heads;
  const T* xbase = (const T*)ten.x[which] + b * ten.sb[which] + h * ten.sh[which];
  const int64_t sn = ten.sn[which];
  const T* pbase = proj + b * psb + h * psh;
  int32_t* obase = OUT8 ? nullptr : (int32_t*)ten.out[which] + (int64_t)bh * n;
  uint8_t* obase8 = OUT8 ? (uint8_t*)ten.out[which] + (int64_t)bh * n : nullptr;
  const int m = lane & 15, kg = lane >> 4;
  const int my_row = m / PARTS, my_part = m % PARTS;  // data row inside a tile, 32-element part of it
  const int j = m;                                    // projection slot of this lane's C registers

  // the projection matrix goes through LDS once per block (one coalesced pass instead of a chain of
  // dependent 2-byte loads per lane)
  __shared__ T lds_p[D * 16];
  // rows of d_real <= D elements: the missing elements of a row and the missing rows of the projection are
  // zeros (they add nothing to a dot product)
  for (int i = threadIdx.x; i < D * r; i += blockDim.x) lds_p[i] = i < d_real * r ? pbase[i] : (T)0.f;
  __syncthreads();
  // B operands: P and |P| for every part: slot j, group kg holds P[part*32 + 8*kg + e][j]; slots >= r are zero
  vec8 pf[PARTS], pa[PARTS];
  const int jc = j < r ? j : 0;
#pragma unroll
  for (int pt = 0; pt < PARTS; ++pt)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float v = j < r ? ha_to_float(lds_p[(pt * 32 + 8 * kg + e) * r + jc]) : 0.f;
      pf[pt][e] = (T)v;
      pa[pt][e] = (T)__builtin_fabsf(v);
    }
  const float tol = (float)(D + 8) * 4.76837158203125e-07f;  // 2 * (d + 8) * 2^-23

  // A row's parts meet different B operands, but an MFMA has one B operand per lane column, not per
  // row: so the tile is multiplied once per part with the rows of the other parts zeroed.  (For
  // PARTS == 1 this is a single MFMA.)
  const int64_t wave_row0 = ((int64_t)blockIdx.x * 4 + wave) * HASH_TILES_PER_WAVE * ROWS;
  for (int t0 = 0; t0 < HASH_TILES_PER_WAVE; t0 += HASH_UNROLL) {
    if (wave_row0 + (int64_t)t0 * ROWS >= n) break;
    vec8 xf[HASH_UNROLL];
#pragma unroll
    for (int u = 0; u < HASH_UNROLL; ++u) {
      const int64_t row = wave_row0 + (int64_t)(t0 + u) * ROWS + my_row;
      vec8 z = {};
      if (row < ten.n_read && my_part * 32 + 8 * kg < d_real) z = *reinterpret_cast<const vec8*>(xbase + row * sn + my_part * 32 + 8 * kg);
      xf[u] = z;
    }
#pragma unroll
    for (int u = 0; u < HASH_UNROLL; ++u) {
      const int64_t tile_row0 = wave_row0 + (int64_t)(t0 + u) * ROWS;
      if (tile_row0 >= n) break;
      f32x4 c = {0.f, 0.f, 0.f, 0.f}, ca = {0.f, 0.f, 0.f, 0.f};
      const u32x4 raw = __builtin_bit_cast(u32x4, xf[u]);
#pragma unroll
      for (int pt = 0; pt < PARTS; ++pt) {
        const u32x4 sel = (PARTS == 1 || my_part == pt) ? raw : u32x4{0u, 0u, 0u, 0u};
        c = HashMfma<T>::run(__builtin_bit_cast(vec8, sel), pf[pt], c);
        ca = HashMfma<T>::run(__builtin_bit_cast(vec8, sel & 0x7fff7fffu), pa[pt], ca);
      }
      // sum the parts of each data row: C register i of this lane is MFMA row 4*kg + i
      float s[NS], sa[NS];
      if (PARTS <= 4) {
#pragma unroll
        for (int q = 0; q < NS; ++q) {
          s[q] = 0.f;
          sa[q] = 0.f;
#pragma unroll
          for (int i = 0; i < 4 / NS; ++i) {
            s[q] += c[q * (4 / NS) + i];
            sa[q] += ca[q * (4 / NS) + i];
          }
        }
      } else {  // PARTS == 8: a data row spans the C registers of lanes kg and kg^1
        s[0] = c[0] + c[1] + c[2] + c[3];
        sa[0] = ca[0] + ca[1] + ca[2] + ca[3];
        s[0] += __shfl_xor(s[0], 16);
        sa[0] += __shfl_xor(sa[0], 16);
      }
      uint64_t pos[NS];
      bool unsure = false;
#pragma unroll
      for (int q = 0; q < NS; ++q) {
        pos[q] = __ballot(s[q] > 0.f);
        unsure = unsure || (j < r && __builtin_fabsf(s[q]) <= tol * sa[q]);
      }
      int bin;
      if (__any(unsure)) {
        // exact recomputation of the tile in fp64: this lane's 8 elements, then a sum over the lanes
        // that share the data row (parts: lane bits 0..log2(PARTS)-1, groups kg: lane bits 4, 5)
        const int64_t row = tile_row0 + my_row;
        bin = 0;
        for (int jj = 0; jj < r; ++jj) {
          double part = 0.0;
          if (row < n)
#pragma unroll
            for (int e = 0; e < 8; ++e)
              part = __builtin_fma((double)ha_to_float(xf[u][e]),
                                   (double)ha_to_float(lds_p[(my_part * 32 + 8 * kg + e) * r + jj]), part);
          for (int off = 1; off < PARTS; off <<= 1) part += __shfl_xor(part, off);
          part += __shfl_xor(part, 16);
          part += __shfl_xor(part, 32);
          bin |= (part > 0.0 ? 1 : 0) << jj;
        }
        // every lane of a data row now holds its bin; lane L < ROWS must hold the bin of row L
        bin = __shfl(bin, (lane % ROWS) * PARTS);
      } else {
        // data row L of the tile sits in sum q = L % NS of the lanes with kg = L / NS (PARTS <= 4),
        // or in the lanes with kg = 2*L (PARTS == 8); its bits are 16 consecutive ballot bits
        const int L = lane % ROWS;
        const int q = PARTS <= 4 ? L % NS : 0;
        const int g = PARTS <= 4 ? L / NS : 2 * L;
        uint64_t sel = pos[0];
#pragma unroll
        for (int qq = 1; qq < NS; ++qq) sel = q == qq ? pos[qq] : sel;
        bin = (int)((sel >> (16 * g)) & ((1u << r) - 1u));
      }
      if (lane < ROWS && tile_row0 + lane < n) {
        if (OUT8)
          obase8[tile_row0 + lane] = (uint8_t)(bin ^ (bin >> 1));
        else
          obase[tile_row0 + lane] = bin ^ (bin >> 1);
      }
    }
  }
}

template <typename T, int D, bool OUT8>
int launch_hash_mfma(HashTensors ten, int64_t seqs, const void* proj, int64_t n, int64_t r, int64_t psb, int64_t psh,
                     int64_t d_real, hipStream_t stream) {
  const int64_t rows_per_block = 4 * HASH_TILES_PER_WAVE * (16 / (D / 32));
  ten.seqs = (int)seqs;
  if (ten.n_read <= 0 || ten.n_read > n) ten.n_read = n;
  const int64_t gy = seqs < 32768 ? seqs : 32768, gz = (seqs + gy - 1) / gy;
  dim3 grid((unsigned)((n + rows_per_block - 1) / rows_per_block), (unsigned)gy, (unsigned)gz);
  hipLaunchKernelGGL((lsh_hash_mfma_kernel<T, D, OUT8>), grid, dim3(256), 0, stream, ten, (const T*)proj, n, (int)r, psb, psh,
                     (int)d_real);
  return ha_launch_status("ha_lsh_hash");
}

}  // namespace

extern "C" int ha_lsh_hash(const void* x, const void* proj, int32_t* buckets, int64_t batch,
                           int64_t heads, int64_t n, int64_t d, int64_t r, int64_t x_stride_b,
                           int64_t x_stride_h, int64_t x_stride_n, int64_t proj_stride_b,
                           int64_t proj_stride_h, int dtype, void* stream) {
  return ha_hash_i32(x, proj, buckets, batch, heads, n, n, d, r, x_stride_b, x_stride_h, x_stride_n, proj_stride_b,
                     proj_stride_h, dtype, (hipStream_t)stream);
}

// ha_lsh_hash for sequences of which only the first n_read rows exist: the ids of rows n_read .. n-1 are those
// of zero rows (the rows the causal recursion appends to odd lengths)
int ha_hash_i32(const void* x, const void* proj, int32_t* buckets, int64_t batch, int64_t heads, int64_t n,
                int64_t n_read, int64_t d, int64_t r, int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_n,
                int64_t proj_stride_b, int64_t proj_stride_h, int dtype, hipStream_t stream) {
  HA_REQUIRE(x && proj && buckets, HA_ERR_NULL, "ha_lsh_hash: null pointer");
  HA_REQUIRE(dtype == HA_F16 || dtype == HA_BF16, HA_ERR_DTYPE, "ha_lsh_hash: Only support fp16 and bf16");
  HA_REQUIRE(batch > 0 && heads > 0 && n > 0, HA_ERR_SHAPE, "ha_lsh_hash: batch, heads, n must be positive");
  HA_REQUIRE(batch * heads < (1ll << 30), HA_ERR_SHAPE, "ha_lsh_hash: batch*heads must be below 2^30");
  HA_REQUIRE(r >= 1, HA_ERR_SHAPE, "ha_lsh_hash: Invalid value for num_projs");
  HA_REQUIRE(r <= 16, HA_ERR_UNSUPPORTED, "ha_lsh_hash: num_projs > 16 is not supported");
  HA_REQUIRE(d >= 8 && d <= 256 && d % 8 == 0, HA_ERR_HEADDIM, "ha_lsh_hash: d must be a multiple of 8 in [8, 256]");
  HA_REQUIRE(x_stride_n % 8 == 0 && x_stride_h % 8 == 0 && x_stride_b % 8 == 0 && ((uintptr_t)x % 16) == 0,
             HA_ERR_SHAPE, "ha_lsh_hash: rows must be 16-byte aligned");
  hipStream_t s = stream;
  HashTensors ten = {};
  ten.x[0] = x; ten.out[0] = buckets;
  ten.sb[0] = x_stride_b; ten.sh[0] = x_stride_h; ten.sn[0] = x_stride_n;
  ten.heads[0] = ten.heads[1] = (int)heads;
  ten.seqs0 = (int)(batch * heads);
  ten.n_read = n_read;
  // built for rows of 32, 64, 128 and 256 elements; a shorter row runs in the next width
#define HA_HASH_MFMA(DD)                                                                                              \
  if (d <= DD) {                                                                                                      \
    if (dtype == HA_F16)                                                                                              \
      return launch_hash_mfma<f16_t, DD, false>(ten, batch * heads, proj, n, r, proj_stride_b, proj_stride_h, d, s);  \
    return launch_hash_mfma<bf16_t, DD, false>(ten, batch * heads, proj, n, r, proj_stride_b, proj_stride_h, d, s);   \
  }
  HA_HASH_MFMA(32) HA_HASH_MFMA(64) HA_HASH_MFMA(128) HA_HASH_MFMA(256)
#undef HA_HASH_MFMA
  return ha_fail(HA_ERR_HEADDIM, "ha_lsh_hash: d must be a multiple of 8 in [8, 256]");
}

// Bucket ids of the queries and keys of one forward pass as one byte each (r <= 8 projections, one shared
// projection matrix), in one launch.  q: (batch, heads, n_read, d), k: (batch, kv_heads, n_read, d), d in {64, 128};
// ids: n >= n_read per sequence, the ids past n_read being those of zero rows.
int ha_hash_pair_u8(const void* q, const void* k, const void* proj, uint8_t* ids_q, uint8_t* ids_k, int64_t batch,
                    int64_t heads, int64_t kv_heads, int64_t n, int64_t n_read, int64_t d, int64_t r,
                    const int64_t (&q_strides)[3], const int64_t (&k_strides)[3], int dtype, hipStream_t stream) {
  HA_REQUIRE(r >= 1 && r <= 8, HA_ERR_UNSUPPORTED, "ha_forward: byte-sized bucket ids need at most 8 projections");
  HA_REQUIRE(batch * (heads + kv_heads) < (1ll << 30), HA_ERR_SHAPE, "ha_forward: batch*(heads + kv_heads) must be below 2^30");
  HashTensors ten = {};
  ten.x[0] = q; ten.x[1] = k; ten.out[0] = ids_q; ten.out[1] = ids_k;
  ten.sb[0] = q_strides[0]; ten.sh[0] = q_strides[1]; ten.sn[0] = q_strides[2];
  ten.sb[1] = k_strides[0]; ten.sh[1] = k_strides[1]; ten.sn[1] = k_strides[2];
  ten.heads[0] = (int)heads; ten.heads[1] = (int)kv_heads;
  ten.seqs0 = (int)(batch * heads);
  ten.n_read = n_read;
  const int64_t seqs = batch * (heads + kv_heads);
#define HA_HASH_PAIR(DD)                                                                                  \
  if (d <= DD) {                                                                                          \
    if (dtype == HA_F16) return launch_hash_mfma<f16_t, DD, true>(ten, seqs, proj, n, r, 0, 0, d, stream); \
    return launch_hash_mfma<bf16_t, DD, true>(ten, seqs, proj, n, r, 0, 0, d, stream);                    \
  }
  HA_HASH_PAIR(32) HA_HASH_PAIR(64) HA_HASH_PAIR(128)
#undef HA_HASH_PAIR
  return ha_fail(HA_ERR_UNSUPPORTED, "ha_forward: paired hash not built for head dim %lld", (long long)d);
}
