// Single-purpose loops for pricing the board's power limit (a measurement aid; nothing on the forward path
// calls them).  Each loop does one thing with finite, changing operands for a given number of trips, two
// workgroups of four waves per CU like the d = 64 attention kernels:
//   HA_PROBE_MFMA          v_mfma_f32_32x32x16 on register operands only
//   HA_PROBE_LDS_MFMA      the same MFMAs fed from LDS by the attention kernels' K (ds_read_b128) and V^T
//                          (ds_read_b64_tr_b16) read pattern: 2 + 4 reads per 8 MFMAs
//   HA_PROBE_SOFTMAX       the soft-max arithmetic of a 16-key half-step alone: 16 multiply-adds, 16 exponentials,
//                          8 packed conversions
//   HA_PROBE_BLOCK         all three together in the order of the attention kernels' half-step block
//   HA_PROBE_BLOCK_WIDE    the same with sixteen large MFMAs per block, the ratio of the d = 128 kernels
// With the board's power and clock sampled around them (bench.py) they separate the energy of a matrix flop,
// of an LDS operand byte and of the soft-max from the idle draw and from each other.
#include "ha_common.h"
#include "attn_tiles.h"

namespace {

constexpr int PROBE_THREADS = 256;

template <int KIND, int WIDE = 1>
__global__ __launch_bounds__(PROBE_THREADS, 2) void ha_power_probe_kernel(long long trips, float* sink) {
  typedef f16_t T;
  typedef ElemTraits<T>::vec8 vec8;
  constexpr int D = 64;
  __shared__ __attribute__((aligned(1024))) unsigned char lds_k[64 * D * 2];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_v[64 * D * 2];
  const int lane = threadIdx.x & 63, hi = lane >> 5, col = lane & 31;

  // finite operands of mixed sign, different per lane and per register
  auto value = [&](int i) -> T {
    const unsigned h = (unsigned)(threadIdx.x * 8 + i) * 2654435761u;
    return (T)(((int)(h >> 24) - 128) * (1.0f / 1024.0f));
  };
  for (int i = threadIdx.x; i < 64 * D; i += PROBE_THREADS) {
    reinterpret_cast<T*>(lds_k)[i] = value(i & 7);
    reinterpret_cast<T*>(lds_v)[i] = value((i >> 3) & 7);
  }
  __syncthreads();
  vec8 a[4], b[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      a[j][e] = value(j * 8 + e);
      b[j][e] = value(32 + j * 8 + e);
    }
  f32x16 acc[4], sa[2], s[2];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[j][i] = 0.f;
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s[j][i] = (float)value(i + 16 * j) * 4.f;
      sa[j][i] = 0.f;
    }

  // per-lane LDS offsets of the operand reads, as in the attention kernels
  int off_k[4], off_v[2];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) off_k[ks] = tile_offset<D>(col, ks * 2 + hi);
  {
    const int g = lane >> 4, sl = lane & 15;
    const int key = (g >> 1) * 4 + (sl >> 2), w = sl & 3;
#pragma unroll
    for (int db = 0; db < 2; ++db) off_v[db] = v_tile_offset<D>(key, db * 4 + (g & 1) * 2 + (w >> 1)) + (w & 1) * 8;
  }
  float m = 3.0f, l = 0.f;
  vec8 pb[2] = {b[0], b[1]};

  for (long long t = 0; t < trips; ++t) {
#pragma unroll
    for (int h = 0; h < 4; ++h) {  // one half-step block: 8 large MFMAs
      vec8 kf[2], vf[2];
      if (KIND == HA_PROBE_LDS_MFMA || KIND == HA_PROBE_BLOCK) {
#pragma unroll
        for (int k2 = 0; k2 < 2; ++k2) kf[k2] = lds_read_k<T>(lds_k, off_k[(h & 1) * 2 + k2] + (h >> 1) * 32 * D * 2);
#pragma unroll
        for (int db = 0; db < 2; ++db) vf[db] = lds_read_vt<T>(lds_v, off_v[db] + h * 16 * D * 2, D * 2);
      } else {
        kf[0] = a[h & 3]; kf[1] = a[(h + 1) & 3];
        vf[0] = a[(h + 2) & 3]; vf[1] = a[(h + 3) & 3];
      }
      if (KIND != HA_PROBE_SOFTMAX) {
#pragma unroll
        for (int rep = 0; rep < WIDE; ++rep) {
#pragma unroll
        for (int db = 0; db < 2; ++db)
#pragma unroll
          for (int nb = 0; nb < 2; ++nb) acc[db * 2 + nb] = Mfma<T>::run(vf[db], pb[nb], acc[db * 2 + nb]);
#pragma unroll
        for (int k2 = 0; k2 < 2; ++k2)
#pragma unroll
          for (int nb = 0; nb < 2; ++nb) sa[nb] = Mfma<T>::run(kf[k2], b[(h + k2 + nb) & 3], sa[nb]);
        }
      }
      if (KIND == HA_PROBE_SOFTMAX || KIND == HA_PROBE_BLOCK) {
        vec8 pn[2];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
          for (int e = 0; e < 8; ++e)
            pn[nb][e] = (T)__builtin_amdgcn_exp2f(__builtin_fmaf(s[nb][(h & 1) * 8 + e], 0.18f, -m));
        m += 1e-6f;  // the reference exponent drifts, so that no exponential is invariant over the trips
        typedef ElemTraits<T>::vec4 vec4;
        f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
          sum = Mfma<T>::quad_sum(__builtin_shufflevector(pn[nb], pn[nb], 0, 1, 2, 3), sum);
          sum = Mfma<T>::quad_sum(__builtin_shufflevector(pn[nb], pn[nb], 4, 5, 6, 7), sum);
        }
        l += sum[0];
        pb[0] = pn[0];
        pb[1] = pn[1];
      }
      if (KIND == HA_PROBE_BLOCK) {
#pragma unroll
        for (int g = 0; g < 8 * WIDE; ++g) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, WIDE == 1 ? 3 : 2, 0);
          __builtin_amdgcn_sched_group_barrier(0x400, WIDE == 1 ? 2 : 1, 0);
        }
      }
    }
    if ((t & 1023) == 1023) {
      // keep the accumulators finite over long runs
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[j][i] *= 1e-3f;
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i) sa[j][i] *= 1e-3f;
      l *= 1e-3f;
    }
  }
  float r = l;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) r += acc[j][i];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) r += sa[j][i];
  if (r == 12345.678f) sink[threadIdx.x] = r;  // never true in practice: keeps the loop alive
}

}  // namespace

extern "C" int ha_power_probe(int kind, int64_t trips, int workgroups, void* sink, void* stream_) {
  HA_REQUIRE(sink, HA_ERR_NULL, "ha_power_probe: null sink (256 floats of device memory)");
  HA_REQUIRE(trips > 0 && trips <= (1ll << 32) && workgroups > 0 && workgroups <= 65536, HA_ERR_SHAPE,
             "ha_power_probe: trips and workgroups must be positive");
  hipStream_t stream = (hipStream_t)stream_;
  switch (kind) {
    case HA_PROBE_MFMA:
      hipLaunchKernelGGL(ha_power_probe_kernel<HA_PROBE_MFMA>, dim3(workgroups), dim3(PROBE_THREADS), 0, stream, (long long)trips, (float*)sink);
      break;
    case HA_PROBE_LDS_MFMA:
      hipLaunchKernelGGL(ha_power_probe_kernel<HA_PROBE_LDS_MFMA>, dim3(workgroups), dim3(PROBE_THREADS), 0, stream, (long long)trips, (float*)sink);
      break;
    case HA_PROBE_SOFTMAX:
      hipLaunchKernelGGL(ha_power_probe_kernel<HA_PROBE_SOFTMAX>, dim3(workgroups), dim3(PROBE_THREADS), 0, stream, (long long)trips, (float*)sink);
      break;
    case HA_PROBE_BLOCK:
      hipLaunchKernelGGL(ha_power_probe_kernel<HA_PROBE_BLOCK>, dim3(workgroups), dim3(PROBE_THREADS), 0, stream, (long long)trips, (float*)sink);
      break;
    case HA_PROBE_BLOCK_WIDE:
      hipLaunchKernelGGL((ha_power_probe_kernel<HA_PROBE_BLOCK, 2>), dim3(workgroups), dim3(PROBE_THREADS), 0, stream, (long long)trips, (float*)sink);
      break;
    default:
      return ha_fail(HA_ERR_UNSUPPORTED, "ha_power_probe: unknown kind %d", kind);
  }
  return ha_launch_status("ha_power_probe");
}
