// MFMA attention forward kernels for gfx950: the sorted block-diagonal + sampled-column kernel and
// the exact (flash) kernel share one body.
//
// Reference semantics: _fwd_hyper_kernel (src/hyper_attn_triton.py:26-192) and _fwd_kernel with
// bias "none" (src/flash_attn_triton.py:57-267).
//
// Work decomposition.  A workgroup of 4 waves owns 256 consecutive (sorted) query positions of one
// (virtual) head; wave w owns 64 of them as two 32-wide MFMA column blocks.  Keys are streamed in
// chunks of 64 rows through double-buffered LDS: K row-major, V transposed so that both MFMA
// operands are read as 16-byte ds_reads.  16-byte pieces are XOR-swizzled instead of padded.
//
// MFMA formulation (v_mfma_f32_32x32x16_{f16,bf16}; A: lane -> row lane%32, k = 8*(lane/32)..+7;
// B: lane -> column lane%32, same k; C: lane -> column lane%32, rows 8*(i/4) + 4*(lane/32) + i%4):
//   S^T = K  Q^T   (M = keys,  N = queries, K = head dim)   -> a lane holds 16 keys of ONE query
//   O^T = V^T P^T  (M = dv,    N = queries, K = keys)       -> P^T comes straight from the S^T registers
// so the soft-max statistics (running max, running sum) are per-lane scalars; only one exchange
// with lane^32 per chunk is needed for the row maximum.  The key order inside every group of 16 is
// permuted in the transposed V tile to match the C-register -> B-operand reuse.
//
// The soft-max runs in base 2 (scale*log2(e) folded into one FMA, v_exp_f32 is 2^x); P is rounded
// to the input type before P.V as the reference does (src/hyper_attn_triton.py:135).
#include "ha_common.h"
#include "attn_fwd.h"

namespace {

constexpr int WG_THREADS = 256;
constexpr int WG_QUERIES = 256;  // sorted query positions per workgroup
constexpr int KC = 64;           // keys per LDS chunk
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;
constexpr float RESCALE_SLACK = 8.0f;  // log2 units

template <typename T>
struct Mfma;
template <>
struct Mfma<f16_t> {
  static __device__ __forceinline__ f32x16 run(f16x8 a, f16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  // c + a[0] + a[1]
  static __device__ __forceinline__ float pair_sum(f16x2 a, float c) {
    const f16x2 ones = {(f16_t)1.0f, (f16_t)1.0f};
    return __builtin_amdgcn_fdot2(a, ones, c, false);
  }
};
template <>
struct Mfma<bf16_t> {
  static __device__ __forceinline__ f32x16 run(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float pair_sum(bf16x2 a, float c) {
    const bf16x2 ones = {(bf16_t)1.0f, (bf16_t)1.0f};
    return __builtin_amdgcn_fdot2_f32_bf16(a, ones, c, false);
  }
};

// position of key k (0..63) inside the transposed V tile: within each group of 16 keys the order is
// 0-3, 8-11, 4-7, 12-15, so that lane half `hi` of the MFMA reads its 8 keys contiguously
__device__ __forceinline__ int vt_key_pos(int k) {
  const int k16 = k & 15;
  return (k & ~15) + ((k16 >> 2) & 1) * 8 + (k16 >> 3) * 4 + (k16 & 3);
}
__device__ __forceinline__ int vt_swizzle(int dvrow) { return (dvrow & 7) ^ ((dvrow >> 3) & 7); }

constexpr int NUM_XCD = 8;
__device__ __forceinline__ int xcd_contiguous_id(int linear, int total) {
  const int xcd = linear % NUM_XCD, k = linear / NUM_XCD;
  const int q = total / NUM_XCD, r = total % NUM_XCD;
  return xcd * q + (xcd < r ? xcd : r) + k;
}

template <typename T, int D, bool GATHER, bool CAUSAL>
__global__ __launch_bounds__(WG_THREADS, (D <= 64 ? 2 : 1)) void attn_fwd_kernel(const ha_attn_kernel_params p) {
  typedef typename ElemTraits<T>::vec8 vec8;
  typedef typename ElemTraits<T>::vec4 vec4;
  typedef typename ElemTraits<T>::vec2 vec2;
  constexpr int DV = D;
  constexpr int KSTEPS = D / 16;      // MFMA k-steps of Q.K^T
  constexpr int DB = DV / 32;         // 32-row blocks of O^T
  constexpr int PR = D / 8;           // 16-byte pieces per K row
  constexpr int PV = DV / 8;          // 16-byte pieces per V row

  __shared__ __attribute__((aligned(16))) T lds_k[2][KC * D];
  __shared__ __attribute__((aligned(16))) T lds_vt[2][DV * KC];

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int hi = lane >> 5, col = lane & 31;

  // ---- which (virtual) head and query tile -----------------------------------------------------
  // Workgroups are handed to the 8 XCDs round-robin by their linear id, and each XCD has its own
  // L2.  Re-number them so that every XCD works through one contiguous range of (head, query tile):
  // the query tiles that share a head's K/V then meet in the same L2.
  const int wg = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int qtiles = (p.n_q + WG_QUERIES - 1) / WG_QUERIES;
  const int vhead = wg / qtiles;
  const int qt = wg % qtiles;
  const int seg = vhead % p.segs;
  const int bh = vhead / p.segs;
  const int b = bh / p.heads, h = bh % p.heads;
  const int hk = h / p.kv_group;

  const T* qb = (const T*)p.q + b * p.q_sb + h * p.q_sh + (p.q_seg_off + (int64_t)seg * p.seg_stride) * p.q_sn;
  const T* kb = (const T*)p.k + b * p.k_sb + hk * p.k_sh + (p.k_seg_off + (int64_t)seg * p.seg_stride) * p.k_sn;
  const T* vb = (const T*)p.v + b * p.v_sb + hk * p.v_sh + (p.k_seg_off + (int64_t)seg * p.seg_stride) * p.v_sn;
  T* ob = (T*)p.out + b * p.o_sb + h * p.o_sh + (p.q_seg_off + (int64_t)seg * p.seg_stride) * p.o_sn;
  float* lb = p.lse + b * p.lse_sb + h * p.lse_sh + p.q_seg_off + (int64_t)seg * p.seg_stride;
  const int64_t qidx_off = b * p.qi_sb + h * p.qi_sh + (int64_t)seg * p.n_q * p.qi_sn;
  const int64_t kidx_off = b * p.ki_sb + hk * p.ki_sh + (int64_t)seg * p.n_k * p.ki_sn;
  const int64_t sidx_off = b * p.si_sb + hk * p.si_sh;

  // original row of sorted query position pq of this head, or -1 past the end
  auto query_row = [&](int pq) -> int {
    if (pq >= p.n_q) return -1;
    return GATHER ? ha_load_idx(p.q_idx, qidx_off + (int64_t)pq * p.qi_sn, p.idx64) : pq;
  };

  // ---- Q fragments (B operand), soft-max state, accumulators ------------------------------------
  vec8 qf[2][KSTEPS];
  float m_run[2], l_run[2];
  f32x16 acc[DB][2];
  int qrow[2];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    qrow[nb] = query_row(qt * WG_QUERIES + wave * 64 + nb * 32 + col);
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      vec8 z = {};
      if (qrow[nb] >= 0) z = *reinterpret_cast<const vec8*>(qb + (int64_t)qrow[nb] * p.q_sn + ks * 16 + hi * 8);
      qf[nb][ks] = z;
    }
    m_run[nb] = -INFINITY;
    l_run[nb] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[db][nb][i] = 0.f;
    if (p.accumulate && qrow[nb] >= 0) {
      // resume from a previous partial attention: weight exp(lse_prev) with normalised output
      m_run[nb] = lb[qrow[nb]] * LOG2E;
      l_run[nb] = hi == 0 ? 1.f : 0.f;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int q4 = 0; q4 < 4; ++q4) {
          const vec4 o = *reinterpret_cast<const vec4*>(ob + (int64_t)qrow[nb] * p.o_sn + db * 32 + q4 * 8 + hi * 4);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[db][nb][q4 * 4 + e] = (float)o[e];
        }
    }
  }

  // ---- key-chunk schedule -------------------------------------------------------------------
  // chunk positions are in units of KC sorted keys, "unwrapped" (taken modulo n_k/KC when used)
  const int nk_chunks = p.n_k / KC;  // GATHER only (n_k % 128 == 0)
  int uni_start = 0, n_blk_chunks = 0, my_lo = 0, my_hi = 0, n_chunks = 0;
  if (GATHER) {
    int start[2], end[2];
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      const int t = qt * 2 + t2;  // reference query tile of 128
      const int block_id = t / p.block_tiles;
      const int first = block_id * p.block_tiles * 128;
      int last = (block_id + 1) * p.block_tiles * 128;
      last = last < p.n_k ? last : p.n_k;
      int cnt = last > first ? (last - first) / KC : 0;
      if (t * 128 >= p.n_q) cnt = 0;
      int s = first / KC;
      if (p.smooth) s = (first + p.n_k + (t % p.block_tiles) * 128 - ((p.block_tiles - 1) * 128) / 2) / KC;
      start[t2] = s;
      end[t2] = s + cnt;
    }
    if (end[1] == start[1]) { start[1] = end[0]; end[1] = end[0]; }
    uni_start = start[0];
    const int uni_end = end[1] > end[0] ? end[1] : end[0];
    n_blk_chunks = uni_end - uni_start;
    my_lo = start[wave >> 1];
    my_hi = end[wave >> 1];
    n_chunks = n_blk_chunks + p.sample_chunks;
  } else {
    int kend = p.n_k;
    if (CAUSAL) {
      const int qend = (qt + 1) * WG_QUERIES;
      kend = kend < qend ? kend : qend;
    }
    n_chunks = (kend + KC - 1) / KC;
  }
  const int wave_q_first = qt * WG_QUERIES + wave * 64;

  // ---- staging: global -> registers -> LDS ------------------------------------------------------
  // Every thread owns the same 16-byte piece `pc` of two adjacent key rows (pair `pr`) of the chunk,
  // for K and for V (NP passes when a row has more than 8 pieces).  The original row numbers of the
  // chunk after next are fetched while the current one is computed, so the row loads never wait for
  // an index load.
  constexpr int NP = (KC / 2) * PR / WG_THREADS;  // 1 for d = 64, 2 for d = 128
  constexpr int PAIRS_PER_PASS = WG_THREADS / PR;
  vec8 stage_k[NP][2];
  vec8 stage_v[NP][2];
  int rows[NP][2];
  const int my_pc = tid % PR;
  const int my_pr = tid / PR;

  auto key_row = [&](int ci, int r) -> int {  // original row of key r of chunk ci, or -1
    if (GATHER) {
      if (ci < n_blk_chunks) {
        const int pos = ((uni_start + ci) % nk_chunks) * KC + r;
        return ha_load_idx(p.k_idx, kidx_off + (int64_t)pos * p.ki_sn, p.idx64);
      }
      const int s = (ci - n_blk_chunks) * KC + r;
      return p.sampled_idx ? ha_load_idx(p.sampled_idx, sidx_off + s, p.idx64) : s;
    }
    const int row = ci * KC + r;
    return row < p.n_k ? row : -1;
  };

  auto fetch_rows = [&](int ci) {
#pragma unroll
    for (int j = 0; j < NP; ++j)
#pragma unroll
      for (int u = 0; u < 2; ++u) rows[j][u] = key_row(ci, (my_pr + j * PAIRS_PER_PASS) * 2 + u);
  };

  auto load_chunk = [&]() {
#pragma unroll
    for (int j = 0; j < NP; ++j)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        vec8 zk = {}, zv = {};
        if (rows[j][u] >= 0) {
          zk = *reinterpret_cast<const vec8*>(kb + (int64_t)rows[j][u] * p.k_sn + my_pc * 8);
          zv = *reinterpret_cast<const vec8*>(vb + (int64_t)rows[j][u] * p.v_sn + my_pc * 8);
        }
        stage_k[j][u] = zk;
        stage_v[j][u] = zv;
      }
  };

  auto store_chunk = [&](int buf) {
#pragma unroll
    for (int j = 0; j < NP; ++j) {
      const int r0 = (my_pr + j * PAIRS_PER_PASS) * 2;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int r = r0 + u;
        *reinterpret_cast<vec8*>(&lds_k[buf][r * D + ((my_pc ^ (r & 7)) * 8)]) = stage_k[j][u];
      }
      const int pos = vt_key_pos(r0);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int dvrow = my_pc * 8 + e;
        vec2 pair;
        pair[0] = stage_v[j][0][e];
        pair[1] = stage_v[j][1][e];
        *reinterpret_cast<vec2*>(&lds_vt[buf][dvrow * KC + (((pos >> 3) ^ vt_swizzle(dvrow)) * 8) + (pos & 7)]) = pair;
      }
    }
  };

  if (n_chunks > 0) {
    fetch_rows(0);
    load_chunk();
    if (n_chunks > 1) fetch_rows(1);
    store_chunk(0);
  }
  __syncthreads();

  for (int ci = 0; ci < n_chunks; ++ci) {
    const int buf = ci & 1;
    const bool more = ci + 1 < n_chunks;
    if (more) {
      load_chunk();                            // rows of chunk ci+1 (fetched one iteration ago)
      if (ci + 2 < n_chunks) fetch_rows(ci + 2);  // in flight during this chunk's compute
    }

    bool active = true;
    bool need_mask = false;
    if (GATHER) {
      if (ci < n_blk_chunks) {
        const int u = uni_start + ci;
        active = u >= my_lo && u < my_hi;
      }
    } else {
      const int k_first = ci * KC;
      if (CAUSAL) {
        active = k_first <= wave_q_first + 63;
        need_mask = k_first + KC - 1 > wave_q_first;
      }
      need_mask = need_mask || (k_first + KC > p.n_k);
    }

    if (active) {
      // ---- S^T = K Q^T ---------------------------------------------------------------------
      f32x16 s[2][2];
#pragma unroll
      for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
          for (int i = 0; i < 16; ++i) s[mb][nb][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks) {
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
          const int key = mb * 32 + col;
          const vec8 a = *reinterpret_cast<const vec8*>(&lds_k[buf][key * D + (((ks * 2 + hi) ^ (key & 7)) * 8)]);
#pragma unroll
          for (int nb = 0; nb < 2; ++nb) s[mb][nb] = Mfma<T>::run(a, qf[nb][ks], s[mb][nb]);
        }
      }

      if (need_mask) {
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
          for (int nb = 0; nb < 2; ++nb) {
            const int qpos = wave_q_first + nb * 32 + col;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const int key = ci * KC + mb * 32 + 8 * (i >> 2) + 4 * hi + (i & 3);
              const bool dead = key >= p.n_k || (CAUSAL && key > qpos);
              if (dead) s[mb][nb][i] = -INFINITY;
            }
          }
      }

      // ---- online soft-max (base 2) with a lazily updated reference maximum ---------------------
      // m_run is only raised when some row's maximum exceeds it by more than RESCALE_SLACK (in log2
      // units), so the accumulator rescale is skipped in most chunks; until then p may grow up to
      // 2^RESCALE_SLACK, which fp16/bf16 and the fp32 sums hold comfortably.
      float mx[2];
      bool grow = false;
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        float v = s[0][nb][0];
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
          for (int i = 0; i < 16; ++i) v = fmaxf(v, s[mb][nb][i]);
        v = fmaxf(v, __shfl_xor(v, 32)) * p.scale_log2;
        mx[nb] = v;
        grow = grow || (v > m_run[nb] + RESCALE_SLACK);
      }
      if (__any(grow)) {
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
          const float m_new = fmaxf(m_run[nb], mx[nb]);
          const float alpha = __builtin_amdgcn_exp2f(m_run[nb] - m_new);
          m_run[nb] = m_new;
          l_run[nb] *= alpha;
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[db][nb][i] *= alpha;
        }
      }

      // p = 2^(s*scale - m), rounded to the input type; row sums are taken over the rounded values
      vec8 pb[KC / 16][2];
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        const float m_use = m_run[nb];
        float sum = l_run[nb];
#pragma unroll
        for (int ks = 0; ks < KC / 16; ++ks) {
#pragma unroll
          for (int e = 0; e < 8; e += 2) {
            const int i = (ks & 1) * 8 + e;
            vec2 pp;
            pp[0] = (T)__builtin_amdgcn_exp2f(__builtin_fmaf(s[ks >> 1][nb][i], p.scale_log2, -m_use));
            pp[1] = (T)__builtin_amdgcn_exp2f(__builtin_fmaf(s[ks >> 1][nb][i + 1], p.scale_log2, -m_use));
            sum = Mfma<T>::pair_sum(pp, sum);
            pb[ks][nb][e] = pp[0];
            pb[ks][nb][e + 1] = pp[1];
          }
        }
        l_run[nb] = sum;
      }

      // ---- O^T += V^T P^T ---------------------------------------------------------------------
#pragma unroll
      for (int ks = 0; ks < KC / 16; ++ks) {
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const int dvrow = db * 32 + col;
          const vec8 a = *reinterpret_cast<const vec8*>(&lds_vt[buf][dvrow * KC + (((ks * 2 + hi) ^ vt_swizzle(dvrow)) * 8)]);
#pragma unroll
          for (int nb = 0; nb < 2; ++nb) acc[db][nb] = Mfma<T>::run(a, pb[ks][nb], acc[db][nb]);
        }
      }
    }

    if (more) store_chunk(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: normalise, stage O through LDS, write whole rows ---------------------------------
  // two halves of 128 queries each: the K buffers hold exactly 2*KC*D = 128*DV elements
  T* lds_o = &lds_k[0][0];
  static_assert(sizeof(lds_k) == (size_t)128 * DV * sizeof(T), "O staging tile");
#pragma unroll 1
  for (int half = 0; half < 2; ++half) {
    if ((wave >> 1) == half) {
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        const float l_tot = l_run[nb] + __shfl_xor(l_run[nb], 32);
        const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
        const int lrow = (wave & 1) * 64 + nb * 32 + col;  // row inside this half
        if (hi == 0 && qrow[nb] >= 0)
          lb[qrow[nb]] = l_tot > 0.f ? (m_run[nb] + __builtin_amdgcn_logf(l_tot)) * LN2 : -INFINITY;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int q4 = 0; q4 < 4; ++q4) {
            vec4 o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = (T)(acc[db][nb][q4 * 4 + e] * inv);
            const int piece = db * 4 + q4;
            *reinterpret_cast<vec4*>(&lds_o[lrow * DV + ((piece ^ (lrow & 7)) * 8) + hi * 4]) = o;
          }
      }
    }
    __syncthreads();
    // 128 rows x PV pieces, all 256 threads
#pragma unroll
    for (int j = 0; j < 128 * PV / WG_THREADS; ++j) {
      const int i = tid + j * WG_THREADS;
      const int lrow = i / PV, pc = i % PV;
      const int row = query_row(qt * WG_QUERIES + half * 128 + lrow);
      if (row >= 0) {
        const vec8 o = *reinterpret_cast<const vec8*>(&lds_o[lrow * DV + ((pc ^ (lrow & 7)) * 8)]);
        *reinterpret_cast<vec8*>(ob + (int64_t)row * p.o_sn + pc * 8) = o;
      }
    }
    __syncthreads();
  }
}

template <typename T, int D>
int launch_variant(const ha_attn_kernel_params& p, int grid, bool gather, bool causal, hipStream_t stream) {
  if (gather)
    hipLaunchKernelGGL((attn_fwd_kernel<T, D, true, false>), dim3(grid), dim3(WG_THREADS), 0, stream, p);
  else if (causal)
    hipLaunchKernelGGL((attn_fwd_kernel<T, D, false, true>), dim3(grid), dim3(WG_THREADS), 0, stream, p);
  else
    hipLaunchKernelGGL((attn_fwd_kernel<T, D, false, false>), dim3(grid), dim3(WG_THREADS), 0, stream, p);
  return ha_launch_status(gather ? "ha_block_attn_fwd" : "ha_flash_attn_fwd");
}

}  // namespace

int ha_attn_launch(const ha_attn_kernel_params& p, int d, int dtype, bool gather, bool causal, hipStream_t stream) {
  const int64_t qtiles = (p.n_q + WG_QUERIES - 1) / WG_QUERIES;
  const int64_t grid = qtiles * p.batch * p.heads * p.segs;
  if (grid <= 0 || grid >= (1ll << 31)) return ha_fail(HA_ERR_SHAPE, "attention: grid of %lld workgroups", (long long)grid);
  if (dtype == HA_F16) {
    if (d == 64) return launch_variant<f16_t, 64>(p, (int)grid, gather, causal, stream);
    return launch_variant<f16_t, 128>(p, (int)grid, gather, causal, stream);
  }
  if (d == 64) return launch_variant<bf16_t, 64>(p, (int)grid, gather, causal, stream);
  return launch_variant<bf16_t, 128>(p, (int)grid, gather, causal, stream);
}
