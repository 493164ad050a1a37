// Angular LSH bucket ids: sign bits of r random projections, Gray-coded.
// Follows the definition in src/angular_lsh_triton.py:76-88 and :175-179 of the reference
// (bit_j = [x . P[:, j] > 0], bin = sum_j bit_j << j, bucket = perm[bin], perm[i] = i ^ (i >> 1)).
//
// One thread owns one row.  A block first copies its rows from HBM into LDS with fully
// coalesced 16-byte loads (XOR-swizzled so the per-row reads that follow are bank-conflict
// free), then every thread walks its row and accumulates the r dot products in fp64:
// products of fp16/bf16 values are exact in fp64, so the sign equals that of the exact dot
// product, independent of accumulation order.  fp64 FMA runs at the same rate as unpacked fp32
// FMA on CDNA4, so exactness costs nothing extra.  The projection matrix is converted to fp64
// once per block and read from LDS as wave-wide broadcasts.
#include "ha_common.h"

namespace {

template <typename T, int RMAX>
__global__ void lsh_hash_kernel(const T* __restrict__ x, const T* __restrict__ proj,
                                int32_t* __restrict__ buckets, int heads, int64_t n, int d, int r,
                                int64_t sb, int64_t sh, int64_t sn, int64_t psb, int64_t psh) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  double* P = reinterpret_cast<double*>(smem);                         // [d][RMAX]
  u32x4* rows = reinterpret_cast<u32x4*>(smem + (size_t)d * RMAX * 8);  // [blockDim.x][d/8] 16-byte chunks

  const int tid = threadIdx.x;
  const int nthreads = blockDim.x;
  const int bh = blockIdx.y;
  const int b = bh / heads, h = bh % heads;
  const int64_t row0 = (int64_t)blockIdx.x * nthreads;
  const int cpr = d >> 3;  // 16-byte chunks per row
  // XOR swizzle of the chunk index by the row: only when it stays inside the row
  const int swz = (cpr % 8 == 0) ? 7 : (((cpr & (cpr - 1)) == 0) ? cpr - 1 : 0);

  const T* pbase = proj + b * psb + h * psh;
  for (int i = tid; i < d * RMAX; i += nthreads) {
    const int k = i / RMAX, j = i % RMAX;
    P[i] = j < r ? (double)ha_to_float(pbase[(int64_t)k * r + j]) : 0.0;
  }

  const T* xbase = x + b * sb + h * sh;
  const int total_chunks = nthreads * cpr;
  for (int i = tid; i < total_chunks; i += nthreads) {
    const int lr = i / cpr, c = i % cpr;
    const int64_t grow = row0 + lr;
    u32x4 val = {0u, 0u, 0u, 0u};
    if (grow < n) val = *reinterpret_cast<const u32x4*>(xbase + grow * sn + c * 8);
    rows[lr * cpr + (c ^ (lr & swz))] = val;
  }
  __syncthreads();

  double acc[RMAX];
#pragma unroll
  for (int j = 0; j < RMAX; ++j) acc[j] = 0.0;

  typedef typename ElemTraits<T>::vec8 vec8;
  for (int c = 0; c < cpr; ++c) {
    u32x4 raw = rows[tid * cpr + (c ^ (tid & swz))];
    vec8 xv = __builtin_bit_cast(vec8, raw);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const double xe = (double)(float)xv[e];
      const double* pk = P + (c * 8 + e) * RMAX;
#pragma unroll
      for (int j = 0; j < RMAX; ++j) acc[j] = __builtin_fma(xe, pk[j], acc[j]);
    }
  }

  int bin = 0;
#pragma unroll
  for (int j = 0; j < RMAX; ++j) bin |= (acc[j] > 0.0 ? 1 : 0) << j;
  const int64_t grow = row0 + tid;
  if (grow < n) buckets[(int64_t)bh * n + grow] = bin ^ (bin >> 1);
}

template <typename T>
int launch_hash(const void* x, const void* proj, int32_t* buckets, int64_t batch, int64_t heads,
                int64_t n, int64_t d, int64_t r, int64_t sb, int64_t sh, int64_t sn, int64_t psb,
                int64_t psh, hipStream_t stream) {
  const int threads = d <= 64 ? 256 : (d <= 128 ? 128 : 64);
  const int rmax = r <= 8 ? 8 : 16;
  const size_t lds = (size_t)d * rmax * 8 + (size_t)threads * d * 2;
  dim3 grid((unsigned)((n + threads - 1) / threads), (unsigned)(batch * heads));
  if (rmax == 8)
    hipLaunchKernelGGL((lsh_hash_kernel<T, 8>), grid, dim3(threads), lds, stream, (const T*)x,
                       (const T*)proj, buckets, (int)heads, n, (int)d, (int)r, sb, sh, sn, psb, psh);
  else
    hipLaunchKernelGGL((lsh_hash_kernel<T, 16>), grid, dim3(threads), lds, stream, (const T*)x,
                       (const T*)proj, buckets, (int)heads, n, (int)d, (int)r, sb, sh, sn, psb, psh);
  return ha_launch_status("ha_lsh_hash");
}

}  // namespace

extern "C" int ha_lsh_hash(const void* x, const void* proj, int32_t* buckets, int64_t batch,
                           int64_t heads, int64_t n, int64_t d, int64_t r, int64_t x_stride_b,
                           int64_t x_stride_h, int64_t x_stride_n, int64_t proj_stride_b,
                           int64_t proj_stride_h, int dtype, void* stream) {
  HA_REQUIRE(x && proj && buckets, HA_ERR_NULL, "ha_lsh_hash: null pointer");
  HA_REQUIRE(dtype == HA_F16 || dtype == HA_BF16, HA_ERR_DTYPE, "ha_lsh_hash: Only support fp16 and bf16");
  HA_REQUIRE(batch > 0 && heads > 0 && n > 0, HA_ERR_SHAPE, "ha_lsh_hash: batch, heads, n must be positive");
  HA_REQUIRE(batch * heads <= 65535, HA_ERR_SHAPE, "ha_lsh_hash: batch*heads must be <= 65535");
  HA_REQUIRE(r >= 1, HA_ERR_SHAPE, "ha_lsh_hash: Invalid value for num_projs");
  HA_REQUIRE(r <= 16, HA_ERR_UNSUPPORTED, "ha_lsh_hash: num_projs > 16 is not supported");
  HA_REQUIRE(d >= 8 && d <= 256 && d % 8 == 0, HA_ERR_HEADDIM, "ha_lsh_hash: d must be a multiple of 8 in [8, 256]");
  HA_REQUIRE(x_stride_n % 8 == 0 && x_stride_h % 8 == 0 && x_stride_b % 8 == 0 && ((uintptr_t)x % 16) == 0,
             HA_ERR_SHAPE, "ha_lsh_hash: rows must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  if (dtype == HA_F16)
    return launch_hash<f16_t>(x, proj, buckets, batch, heads, n, d, r, x_stride_b, x_stride_h, x_stride_n,
                              proj_stride_b, proj_stride_h, s);
  return launch_hash<bf16_t>(x, proj, buckets, batch, heads, n, d, r, x_stride_b, x_stride_h, x_stride_n,
                             proj_stride_b, proj_stride_h, s);
}
