// MFMA attention forward kernels for gfx950: the sorted block-diagonal + sampled-column kernel and
// the exact (flash) kernel share one body.
//
// Reference semantics: _fwd_hyper_kernel (src/hyper_attn_triton.py:26-192) and _fwd_kernel with
// bias "none" (src/flash_attn_triton.py:57-267); the resume-from-a-previous-partial-result mode
// folds add_self_attentions (src/attn_utils.py:6-50) into the kernel.
//
// Work decomposition.  A workgroup owns 256 consecutive (sorted) query positions of one (virtual) head:
// 4 waves of 64 queries (two 32-wide MFMA column blocks) at head dim 64, 8 waves of 32 queries at head
// dim 128 (WaveShape below).  Query rows and key
// rows go from HBM straight into LDS (global_load_lds, 16 bytes per lane, whole rows per
// instruction, no staging registers), row-major with their 16-byte pieces XOR-swizzled by the row
// number (the swizzle is applied on the source side: a lane fetches the piece that belongs in its
// LDS slot).  Q and K operands are read with ds_read_b128, the V^T operand with the transposing
// ds_read_b64_tr_b16.
//
// MFMA formulation (v_mfma_f32_32x32x16_{f16,bf16}; A: lane -> row lane%32, k = 8*(lane/32)..+7;
// B: lane -> column lane%32, same k; C: lane -> column lane%32, rows 8*(i/4) + 4*(lane/32) + i%4):
//   S^T = K  Q^T   (M = keys,  N = queries, K = head dim)   -> a lane holds 16 keys of ONE query
//   O^T = V^T P^T  (M = dv,    N = queries, K = keys)       -> P^T comes straight from the S^T registers
// so the soft-max statistics are per-lane scalars.  ds_read_b64_tr_b16 gives lane i of a 16-lane
// group element i%4 of the 8-byte words addressed by lanes 4j + i/4 (j = 0..3), so a group that
// points its lanes at (key j, dv word w) receives V[key 0..3][dv base + i]: the V^T operand in
// exactly the key order of the C registers.
//
// Software pipeline.  The loop body is a chain of straight-line blocks, one per half-step of 16 keys, and
// each block mixes three independent things: the exponentials of half-step u, the P.V MFMAs of
// half-step u-1 and half of the S^T MFMAs of the next 32-key step, issued one MFMA and its share of the
// vector work at a time (clustering the MFMAs of a block, with or without a raised wave priority, measured
// 4 to 6 % slower); two waves per SIMD fill each other's gaps.  Keys are streamed in tiles of 64
// rows; the K tiles are shifted by 32 keys against the V tiles (K tile c holds keys 64c-32..64c+31),
// so the K rows read during an iteration all sit in one tile, which is read in that iteration only
// and can be refilled in the next, and the V^T operands of a half-step are fetched one block ahead.
//
// Soft-max without a running maximum.  The exponentials use the current reference exponent m of
// the row as is (base 2, scale*log2(e) folded into one FMA; v_exp_f32 is 2^x); P is rounded to the
// input type before P.V as the reference does (src/hyper_attn_triton.py:135) and the row sums are
// taken over the rounded values.  Only when the sum of a lane's 8 values of a half-step reaches 2^14
// (or is not a number: nothing seen yet) is the row maximum computed, m raised, the accumulators
// rescaled and the half-step redone; below that bound every value is finite in fp16 and the result
// does not depend on m beyond rounding.  m only ever grows, and starts from the true maximum of the
// first keys or from the log-sum-exp of the partial result that is being resumed.
#include "ha_common.h"
#include "attn_tiles.h"
#include "attn_fwd.h"

#include <stdlib.h>

namespace {

constexpr int WG_QUERIES = 256;  // sorted query positions per workgroup
constexpr int KC = 64;           // keys per LDS tile
constexpr float HALF_SUM_LIMIT = 16384.f;  // 2^14: a lane's half-step sum below this has no fp16 overflow
// Reference exponent (log2 units) of a row that has seen no key yet.  Finite on purpose: a masked score
// (-inf) then gives P = 2^(-inf) = 0 without any special case, where -inf - (-inf) would be a NaN that
// sends every half-step of a masked chunk through the rescaling path; a real score gives 2^(+huge) = inf,
// which takes that path once and sets the row's true exponent.
constexpr float M_FLOOR = -1e30f;

// How a workgroup's 256 queries are split over its waves.  A wave's registers hold the output accumulators
// of its queries (queries x head dim floats over 64 lanes), their query fragments and two S^T buffers: 64
// queries per wave fit 256 registers at head dim 64, at head dim 128 only 32 do.  256 registers is what lets
// two waves share a SIMD, and a wave on its own leaves the matrix pipe idle through every stretch of vector
// work and every wait (one wave per SIMD with 64 queries and 512 registers ran the d = 128 loop at 1170
// cycles per 16 keys where its MFMAs alone take 512).  So: 4 waves x 64 queries at d = 64 (two workgroups per
// CU), 8 waves x 32 queries at d = 128 (one workgroup per CU, LDS-bound), two waves per SIMD either way.
template <int D>
struct WaveShape {
  static constexpr int NB = D <= 64 ? 2 : 1;        // 32-query MFMA column blocks per wave
  static constexpr int QW = 32 * NB;                // queries per wave
  static constexpr int WAVES = WG_QUERIES / QW;     // waves per workgroup
  static constexpr int THREADS = 64 * WAVES;
};

// x / y for 0 <= x < 2^31 by the divisor's multiply-and-shift constants
__device__ __forceinline__ int fast_div(int x, ha_divisor y) { return (int)(((uint64_t)(uint32_t)x * y.magic) >> y.shift); }

// LDS byte offsets of one lane's operand reads, relative to a tile base (fixed for the whole kernel).
template <int D>
struct LaneOffsets {
  int k[D / 16];  // Q / K operand piece of k-step ks for tile row lane%32 (add 32 rows for the upper half)
  int v[D / 32];  // V^T operand word for dv block db, keys 0..3 (+4 for the upper lane half) of a 16-key half-step
};

// P of the 8 values of half-step H a lane holds per query block (elements 8H..8H+7 of its S^T
// registers), rounded to T, and their sums.  m is the reference exponent (log2 units).
// sums of the 8 values per query block of a half-step's P.  They go through the matrix pipe: v_dot2
// does not overlap with the big MFMAs at all.
template <typename T, int NB>
__device__ __forceinline__ void half_step_sums(const typename ElemTraits<T>::vec8 (&pn)[NB], float (&sum)[NB]) {
  typedef typename ElemTraits<T>::vec4 vec4;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const vec4 lo = __builtin_shufflevector(pn[nb], pn[nb], 0, 1, 2, 3);
    const vec4 hi = __builtin_shufflevector(pn[nb], pn[nb], 4, 5, 6, 7);
    f32x4 acc_sum = {0.f, 0.f, 0.f, 0.f};
    acc_sum = Mfma<T>::quad_sum(lo, acc_sum);
    acc_sum = Mfma<T>::quad_sum(hi, acc_sum);
    sum[nb] = acc_sum[0];
  }
}
template <typename T, int NB, int H>
__device__ __forceinline__ void half_step_p(const f32x16 (&s_use)[NB], const float (&m)[NB], float scale_log2,
                                            typename ElemTraits<T>::vec8 (&pn)[NB], float (&sum)[NB]) {
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
#pragma unroll
    for (int e = 0; e < 8; ++e)
      pn[nb][e] = (T)__builtin_amdgcn_exp2f(__builtin_fmaf(s_use[nb][H * 8 + e], scale_log2, -m[nb]));
  half_step_sums<T, NB>(pn, sum);
}

// The rare path of a half-step: raise the reference exponents to the row maxima of the half-step,
// rescale the row sums and redo the half-step's P.  alpha is what everything accumulated under the old
// exponents has to be multiplied by.
template <typename T, int NB, int H>
__device__ __forceinline__ void half_step_rescale(const f32x16 (&s_use)[NB], float scale_log2,
                                                  float (&alpha)[NB], float (&m_run)[NB], float (&l_run)[NB],
                                                  typename ElemTraits<T>::vec8 (&pn)[NB], float (&sum)[NB]) {
  float m_use[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    // only this half-step's values: the other half of the step raises the exponents itself if it has
    // to, and the two rare paths of a step then share no work the compiler would compute up front
    float v = s_use[nb][H * 8];
#pragma unroll
    for (int e = 1; e < 8; ++e) v = fmaxf(v, s_use[nb][H * 8 + e]);
    v = ha_max_xor32(v) * scale_log2;
    const float m_new = fmaxf(m_run[nb], v);
    // 2^(old - new) <= 1; nothing is accumulated yet under the floor exponent of a fresh row
    alpha[nb] = __builtin_amdgcn_exp2f(m_run[nb] - m_new);
    m_run[nb] = m_new;
    l_run[nb] *= alpha[nb];
    // rows that have seen no key yet (all masked) keep the floor; their P is 2^(-inf) = 0
    m_use[nb] = m_new;
  }
  half_step_p<T, NB, H>(s_use, m_use, scale_log2, pn, sum);
}

// One block of the pipeline: half-step H (16 keys) of the 32-key step whose S^T is s_use.
//   MFMAs : P.V of the previous half-step (operands vf, pb, both in registers) and this half's share
//           (k-steps H*KSTEPS/2 ..) of the next step's S^T, K rows k_row_off.. of k_tile
//   VALU  : P of this half-step from s_use -> pb (for the next block) and the row sums
//   LDS   : V^T of this half-step's keys (v_key_off.. of v_tile) -> vf (for the next block)
template <typename T, int D, int H>
__device__ __forceinline__ void half_step(const f32x16 (&s_use)[WaveShape<D>::NB], f32x16 (&s_fill)[WaveShape<D>::NB],
                                          const unsigned char* k_tile, int k_row_off,
                                          const unsigned char* v_tile, int v_key_off, const LaneOffsets<D>& lo,
                                          const typename ElemTraits<T>::vec8 (&qf)[WaveShape<D>::NB][D / 16],
                                          f32x16 (&acc)[D / 32][WaveShape<D>::NB], float (&m_run)[WaveShape<D>::NB],
                                          float (&l_run)[WaveShape<D>::NB],
                                          typename ElemTraits<T>::vec8 (&pb)[WaveShape<D>::NB],
                                          typename ElemTraits<T>::vec8 (&vf)[D / 32], float scale_log2) {
  typedef typename ElemTraits<T>::vec8 vec8;
  constexpr int NB = WaveShape<D>::NB;
  constexpr int KH = D / 32;  // k-steps of this half
  constexpr int DB = D / 32;

  vec8 kf[KH];
#pragma unroll
  for (int k2 = 0; k2 < KH; ++k2) kf[k2] = lds_read_k<T>(k_tile, lo.k[H * KH + k2] + k_row_off);
  vec8 vf_next[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) vf_next[db] = lds_read_vt<T>(v_tile, lo.v[db] + v_key_off, D * 2);
  // the LDS reads stay at the head of the block: their latency hides behind the P.V MFMAs and the
  // exponentials instead of being waited for where the compiler would sink them to
  __builtin_amdgcn_sched_barrier(0);

#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[db][nb] = Mfma<T>::run(vf[db], pb[nb], acc[db][nb]);
  if (H == 0) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) s_fill[nb][i] = 0.f;
  }
#pragma unroll
  for (int k2 = 0; k2 < KH; ++k2)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) s_fill[nb] = Mfma<T>::run(kf[k2], qf[nb][H * KH + k2], s_fill[nb]);

  vec8 pn[NB];
  float sum[NB];
  half_step_p<T, NB, H>(s_use, m_run, scale_log2, pn, sum);
  // Issue order of the block: each of its NB*D/16 large MFMAs is followed by a share of the P arithmetic (8 NB
  // multiply-adds, 4 NB conversions, 8 NB exponentials in all), so the soft-max fills the issue slots behind
  // every MFMA instead of running as one burst after the last of them.  Measured 3 % faster than the
  // scheduler's own order.
  constexpr int MFMAS = NB * D / 16;
#pragma unroll
  for (int g = 0; g < MFMAS; ++g) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                          // one MFMA
    __builtin_amdgcn_sched_group_barrier(0x002, (12 * NB + MFMAS - 1) / MFMAS, 0);  // its share of plain VALU
    __builtin_amdgcn_sched_group_barrier(0x400, 8 * NB / MFMAS, 0);             // and of the transcendentals
  }
  // One compare for all query blocks: their sums are >= 0 or NaN, so the total is below the limit
  // only if every one is.  Not "total >= limit": a NaN (row that has seen nothing yet) must take the rare
  // path too.
  float total = sum[0];
#pragma unroll
  for (int nb = 1; nb < NB; ++nb) total += sum[nb];
  const bool redo = !(total < HALF_SUM_LIMIT);
  if (__builtin_expect(__builtin_amdgcn_ballot_w64(redo) != 0, false)) {
    float alpha[NB];
    half_step_rescale<T, NB, H>(s_use, scale_log2, alpha, m_run, l_run, pn, sum);
    // the accumulators hold everything up to the previous half-step (its P.V was issued above; the
    // P.V of this half-step is added by the next block, under the new exponents)
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[db][nb][i] *= alpha[nb];
  }
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    l_run[nb] += sum[nb];
    pb[nb] = pn[nb];
  }
#pragma unroll
  for (int db = 0; db < DB; ++db) vf[db] = vf_next[db];
}

}  // namespace

// PLAIN (gathered kernel only): the common configuration, for which the per-iteration bookkeeping of the
// general one is compiled out: no smoothing, default samples (rows 0 .. sample_size-1), and both
// 128-query tiles of the workgroup inside one key block, so no chunk is ever masked for half of it.
// Head dims below the built width D (NARROW kernels): a row holds fewer 16-byte pieces than its LDS slot.
// A lane whose piece lies past the end of the row fetches these zeros instead, so the tiles hold the rows
// zero-padded to D: zero columns change neither q.k nor the other columns of the output.
__device__ __attribute__((aligned(16))) const unsigned char ha_zero_piece[16] = {0};

template <bool NARROW>
__device__ __forceinline__ const unsigned char* piece_address(const unsigned char* base, int row, uint32_t stride_bytes,
                                                              uint32_t piece, int pieces_in_row) {
  const unsigned char* a = row_address(base, row, stride_bytes, piece << 4);
  if (NARROW && (int)piece >= pieces_in_row) a = ha_zero_piece;
  return a;
}

template <typename T, int D, bool GATHER, bool CAUSAL, bool PLAIN = false, bool NARROW = false, bool REWEIGHT = false>
__global__ __launch_bounds__(WaveShape<D>::THREADS, 2) void ha_attn_fwd_kernel(const ha_attn_kernel_params p) {
  typedef typename ElemTraits<T>::vec8 vec8;
  typedef typename ElemTraits<T>::vec4 vec4;
  constexpr int NB = WaveShape<D>::NB;        // 32-query column blocks per wave
  constexpr int QW = WaveShape<D>::QW;        // queries per wave
  constexpr int WAVES = WaveShape<D>::WAVES;  // waves per workgroup
  constexpr int DV = D;
  constexpr int KSTEPS = D / 16;  // MFMA k-steps of Q.K^T
  constexpr int DB = DV / 32;     // 32-row blocks of O^T
  constexpr int PR = D / 8;       // 16-byte pieces per row

  // Separate LDS objects (two K tiles, two V tiles of KC rows, the query rows): the compiler then
  // knows that a tile being filled from HBM and a tile being read do not alias, and does not
  // serialise them.  The query region (QW rows per wave) is reused for the output rows at the end.
  constexpr int TILE_BYTES = KC * D * 2;
  // The key tiles ask for the larger alignment only to be placed first: LDS offsets below 64 KB fit
  // the immediate field of the LDS reads, which matters at d = 128 where the workgroup uses 130 KB.
  constexpr int Q_WAVE_BYTES = QW * D * 2;  // a wave's part of the query region
  __shared__ __attribute__((aligned(1024))) unsigned char lds_k0[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_k1[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_v0[TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_v1[TILE_BYTES];
  __shared__ __attribute__((aligned(16))) unsigned char lds_q[4 * TILE_BYTES];
  __shared__ int lds_qrow[WG_QUERIES];   // original row of every query position (-1: past the end)
  __shared__ float lds_w[WG_QUERIES];    // weight of the resumed partial result per query position

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  // the same number, known to the compiler to be wave-uniform: what the tile loads derive from it
  // (chunk numbers, index array addresses, LDS destinations) then stays in scalar registers
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);
  const int hi = lane >> 5, col = lane & 31;

  // ---- which (virtual) head and query tile -----------------------------------------------------
  // Workgroup number = (((batch, kv head), segment), tile, query head inside the kv group), the last one
  // fastest: the query heads that share a kv head work on the same tile side by side, on one XCD, so that the
  // K and V rows of the tile (the same for all of them) come from HBM once and from L2 after that.
  const int wg = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int qtiles = (p.n_q + WG_QUERIES - 1) / WG_QUERIES;
  // Exact causal attention: a workgroup takes the tile pair (qtiles-1-s, s), so that every workgroup of the
  // launch has the same number of key chunks to go through.  The hardware hands out workgroups in order and
  // a slot freed by a short one stays empty until the ones queued before it are placed: with one tile per
  // workgroup (4 to 32 chunks in a 2048-row leaf) the slots of a CU stood empty for 8 us at a time.
  constexpr bool PAIRED = CAUSAL && !GATHER;
  const int wg_per_seq = PAIRED ? (qtiles + 1) / 2 : qtiles;  // what p.div_qtiles divides by
  const int wg_tile = fast_div(wg, p.div_kv_group);
  const int hg = wg - wg_tile * p.kv_group;
  const int vseq = fast_div(wg_tile, p.div_qtiles);
  const int slot = wg_tile - vseq * wg_per_seq;
  const int bhk = fast_div(vseq, p.div_segs);
  const int seg = vseq - bhk * p.segs;
  const int b = fast_div(bhk, p.div_kv_heads), hk = bhk - b * fast_div(p.heads, p.div_kv_group);
  const int h = hk * p.kv_group + hg;

  // ---- rows of this segment -----------------------------------------------------------------------
  int n_q = p.n_q, n_k = p.n_k;
  int64_t seg_q_row = p.q_seg_off + (int64_t)seg * p.seg_stride, seg_k_row = p.k_seg_off + (int64_t)seg * p.seg_stride;
  int64_t seg_o_row = p.o_seg_off + (int64_t)seg * p.o_seg_stride;  // first row of the segment in out / lse
  if (!GATHER && p.rag_levels >= 0) {
    // walk down from the whole sequence: where the segment starts and how many of its rows exist
    int start = 0, real = p.rag_n;
    for (int i = 0; i < p.rag_levels; ++i) {
      const int c = p.rag_half[i];
      if ((seg >> (p.rag_levels - 1 - i)) & 1) {
        start += c;
        real = max(real - c, 0);
      } else {
        real = min(real, c);
      }
    }
    if (p.rag_split) {
      const int c = p.rag_half[p.rag_levels];
      seg_q_row = start + c;
      seg_k_row = start;
      n_q = min(max(real - c, 0), c);
      n_k = min(real, c);
    } else {
      seg_q_row = seg_k_row = start;
      n_q = n_k = real;
    }
    seg_o_row = seg_q_row;
  }
  // gathered kernel: entries of the query order from this number on name a row that does not exist
  const int q_rows_exist = (GATHER && seg == p.segs - 1) ? p.n_q_last : n_q;

  if constexpr (!PAIRED) {
    const int qt = slot;
    if (qt * WG_QUERIES >= n_q) return;  // ragged launches: the grid is sized for the longest segment
#include "attn_fwd_tile.inc"
  } else {
    // the long tile first.  No barrier between the two: the last iteration of a tile ends with one, and after
    // it a wave touches only its own part of the query region.
    const int t_long = qtiles - 1 - slot;
    if (t_long * WG_QUERIES < n_q) {  // ragged launches: the grid is sized for the longest segment
      const int qt = t_long;
#include "attn_fwd_tile.inc"
    }
    if (slot != t_long && slot * WG_QUERIES < n_q) {  // an odd number of tiles: the middle one has no partner
      const int qt = slot;
#include "attn_fwd_tile.inc"
    }
  }
}

#include "attn_fwd_stream.inc"

namespace {

template <typename T, int D, bool GATHER, bool CAUSAL, bool PLAIN = false, bool NARROW = false, bool REWEIGHT = false>
int launch_one(const ha_attn_kernel_params& p, int grid, hipStream_t stream, const char* what) {
  hipLaunchKernelGGL((ha_attn_fwd_kernel<T, D, GATHER, CAUSAL, PLAIN, NARROW, REWEIGHT>), dim3(grid), dim3(WaveShape<D>::THREADS), 0,
                     stream, p);
  return ha_launch_status(what);
}

template <typename T, int D>
int launch_variant(const ha_attn_kernel_params& p, int grid, bool gather, bool causal, bool reweight, hipStream_t stream) {
  const bool narrow = p.qk_pieces != D / 8 || p.v_pieces != D / 8;
  if (gather && reweight)  // the entry point has checked that the head dims are the built ones
    return launch_one<T, D, true, false, false, false, true>(p, grid, stream, "ha_block_attn_fwd");
  if (gather) {
    const bool plain = !p.smooth && !p.sampled_idx && p.block_tiles % 2 == 0 && p.n_q % WG_QUERIES == 0;
    if (p.tiles_per_wg > 1) {  // set by ha_attn_launch for the instances built below
      if (plain) hipLaunchKernelGGL((ha_attn_fwd_stream_kernel<T, D, true>), dim3(grid), dim3(WaveShape<D>::THREADS), 0, stream, p);
      else hipLaunchKernelGGL((ha_attn_fwd_stream_kernel<T, D, false>), dim3(grid), dim3(WaveShape<D>::THREADS), 0, stream, p);
      return ha_launch_status("ha_block_attn_fwd");
    }
    if (narrow) return launch_one<T, D, true, false, false, true>(p, grid, stream, "ha_block_attn_fwd");
    if (plain) return launch_one<T, D, true, false, true>(p, grid, stream, "ha_block_attn_fwd");
    return launch_one<T, D, true, false>(p, grid, stream, "ha_block_attn_fwd");
  }
  if (narrow) {
    if (causal) return launch_one<T, D, false, true, false, true>(p, grid, stream, "ha_flash_attn_fwd");
    return launch_one<T, D, false, false, false, true>(p, grid, stream, "ha_flash_attn_fwd");
  }
  if (causal) return launch_one<T, D, false, true>(p, grid, stream, "ha_flash_attn_fwd");
  return launch_one<T, D, false, false>(p, grid, stream, "ha_flash_attn_fwd");
}

}  // namespace

static ha_divisor make_divisor(int64_t y) {
  if (y < 1) y = 1;
  int s = 0;
  while ((int64_t(1) << s) < y) ++s;
  ha_divisor d;
  d.shift = 31 + s;
  d.magic = (uint32_t)((uint64_t(1) << d.shift) / (uint64_t)y + 1);
  return d;
}

int ha_attn_launch(const ha_attn_kernel_params& params, int d, int dv, int dtype, bool gather, bool causal,
                   bool reweight, hipStream_t stream) {
  ha_attn_kernel_params p = params;
  // the kernels are built for rows of 64 and 128 elements; other head dims (multiples of 8) run in the
  // next width with the missing pieces of every row read as zeros
  const int width = d <= 64 && dv <= 64 ? 64 : 128;
  p.qk_pieces = d / 8;
  p.v_pieces = dv / 8;
  int64_t qtiles = (p.n_q + WG_QUERIES - 1) / WG_QUERIES;
  if (causal && !gather) qtiles = (qtiles + 1) / 2;  // exact causal attention: one workgroup per pair of tiles
  // Gathered attention with whole 256-query tiles, whole key blocks and an even number of at least four key
  // chunks per tile can run as a stream: a workgroup takes a run of tiles of its head
  // (ha_attn_fwd_stream_kernel), as long a run as still leaves every CU its full set of resident workgroups.
  // It is the default where it measured faster: head dim 128 (one workgroup per CU, nothing else covers a
  // workgroup's set-up and output stage) in the plain configuration, 4 to 7 % on a level of 64 tiles per head
  // at 8 chunks per tile.  At head dim 64 the second workgroup of the CU covers them already and the stream
  // measured 2 to 5 % slower; with smooth windows (18 chunks per tile) it measured the same.
  p.tiles_per_wg = 1;
  const char* stream_env = getenv("HA_STREAM_TILES");  // measurement aid: force the run length (1: off)
  const bool plain = !p.smooth && !p.sampled_idx && p.block_tiles % 2 == 0;
  if (gather && !reweight && p.qk_pieces == width / 8 && p.v_pieces == width / 8 && p.n_q % WG_QUERIES == 0 && qtiles >= 2 &&
      p.sample_chunks % 2 == 0 && p.n_k % (p.block_tiles * 128) == 0 && 2 * p.block_tiles + p.sample_chunks >= 4 &&
      (stream_env || (width == 128 && plain))) {
    const int64_t slots = 256 * (width == 64 ? 2 : 1);  // workgroups the chip holds at once
    int r = 16;
    while (r > 1 && (r > qtiles || (qtiles / r) * p.batch * p.heads * p.segs < slots)) r /= 2;
    if (stream_env) r = atoi(stream_env) < 1 ? 1 : (atoi(stream_env) > qtiles ? (int)qtiles : atoi(stream_env));
    p.tiles_per_wg = r;
    qtiles = (qtiles + r - 1) / r;
  }
  p.div_qtiles = make_divisor(qtiles);
  p.div_segs = make_divisor(p.segs);
  p.div_heads = make_divisor(p.heads);
  p.div_kv_heads = make_divisor(p.heads / p.kv_group);
  p.div_kv_group = make_divisor(p.kv_group);
  p.div_block_tiles = make_divisor(p.block_tiles);
  const int64_t grid = qtiles * p.batch * p.heads * p.segs;
  if (grid <= 0 || grid >= (1ll << 31)) return ha_fail(HA_ERR_SHAPE, "attention: grid of %lld workgroups", (long long)grid);
  if (dtype == HA_F16) {
    if (width == 64) return launch_variant<f16_t, 64>(p, (int)grid, gather, causal, reweight, stream);
    return launch_variant<f16_t, 128>(p, (int)grid, gather, causal, reweight, stream);
  }
  if (width == 64) return launch_variant<bf16_t, 64>(p, (int)grid, gather, causal, reweight, stream);
  return launch_variant<bf16_t, 128>(p, (int)grid, gather, causal, reweight, stream);
}
