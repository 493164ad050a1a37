// MFMA attention forward kernels for gfx950: the sorted block-diagonal + sampled-column kernel and
// the exact (flash) kernel share one body.
//
// Reference semantics: _fwd_hyper_kernel (src/hyper_attn_triton.py:26-192) and _fwd_kernel with
// bias "none" (src/flash_attn_triton.py:57-267); the resume-from-a-previous-partial-result mode
// folds add_self_attentions (src/attn_utils.py:6-50) into the kernel.
//
// Work decomposition.  A workgroup of 4 waves owns 256 consecutive (sorted) query positions of one
// (virtual) head; wave w owns 64 of them as two 32-wide MFMA column blocks.  Query rows and key
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
// Software pipeline.  On this hardware a wave's MFMAs overlap only with vector instructions of the
// SAME wave, so the loop body is a chain of straight-line blocks, one per half-step of 16 keys, and
// each block mixes three independent things: the exponentials of half-step u, the P.V MFMAs of
// half-step u-1 and half of the S^T MFMAs of the next 32-key step.  Keys are streamed in tiles of 64
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

namespace {

constexpr int WG_THREADS = 256;
constexpr int WG_QUERIES = 256;  // sorted query positions per workgroup
constexpr int KC = 64;           // keys per LDS tile
constexpr float HALF_SUM_LIMIT = 16384.f;  // 2^14: a lane's half-step sum below this has no fp16 overflow
// Reference exponent (log2 units) of a row that has seen no key yet.  Finite on purpose: a masked score
// (-inf) then gives P = 2^(-inf) = 0 without any special case, where -inf - (-inf) would be a NaN that
// sends every half-step of a masked chunk through the rescaling path; a real score gives 2^(+huge) = inf,
// which takes that path once and sets the row's true exponent.
constexpr float M_FLOOR = -1e30f;

// Head dims whose kernel needs more than 256 registers keep the S^T accumulators in VGPRs by hand.
template <int D>
struct S_IN_VGPR {
  static constexpr bool value = D > 64;
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
template <typename T>
__device__ __forceinline__ void half_step_sums(const typename ElemTraits<T>::vec8 (&pn)[2], float (&sum)[2]) {
  typedef typename ElemTraits<T>::vec4 vec4;
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const vec4 lo = __builtin_shufflevector(pn[nb], pn[nb], 0, 1, 2, 3);
    const vec4 hi = __builtin_shufflevector(pn[nb], pn[nb], 4, 5, 6, 7);
    f32x4 acc_sum = {0.f, 0.f, 0.f, 0.f};
    acc_sum = Mfma<T>::quad_sum(lo, acc_sum);
    acc_sum = Mfma<T>::quad_sum(hi, acc_sum);
    sum[nb] = acc_sum[0];
  }
}
template <typename T, int H, bool SUMS = true>
__device__ __forceinline__ void half_step_p(const f32x16 (&s_use)[2], const float (&m)[2], float scale_log2,
                                            typename ElemTraits<T>::vec8 (&pn)[2], float (&sum)[2]) {
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int e = 0; e < 8; ++e)
      pn[nb][e] = (T)__builtin_amdgcn_exp2f(__builtin_fmaf(s_use[nb][H * 8 + e], scale_log2, -m[nb]));
  if (SUMS) half_step_sums<T>(pn, sum);
}

// The rare path of a half-step: raise the reference exponents to the row maxima of the half-step,
// rescale the row sums and redo the half-step's P.  alpha is what everything accumulated under the old
// exponents has to be multiplied by.
template <typename T, int D, int H>
__device__ __forceinline__ void half_step_rescale(const f32x16 (&s_use)[2], float scale_log2,
                                                  float (&alpha)[2], float (&m_run)[2], float (&l_run)[2],
                                                  typename ElemTraits<T>::vec8 (&pn)[2], float (&sum)[2]) {
  float m_use[2];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
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
  half_step_p<T, H>(s_use, m_use, scale_log2, pn, sum);
}

// One block of the pipeline: half-step H (16 keys) of the 32-key step whose S^T is s_use.
//   MFMAs : P.V of the previous half-step (operands vf, pb, both in registers) and this half's share
//           (k-steps H*KSTEPS/2 ..) of the next step's S^T, K rows k_row_off.. of k_tile
//   VALU  : P of this half-step from s_use -> pb (for the next block) and the row sums
//   LDS   : V^T of this half-step's keys (v_key_off.. of v_tile) -> vf (for the next block)
template <typename T, int D, int H>
__device__ __forceinline__ void half_step(const f32x16 (&s_use)[2], f32x16 (&s_fill)[2],
                                          const unsigned char* k_tile, int k_row_off,
                                          const unsigned char* v_tile, int v_key_off, const LaneOffsets<D>& lo,
                                          const typename ElemTraits<T>::vec8 (&qf)[2][D / 16],
                                          f32x16 (&acc)[D / 32][2], float (&m_run)[2], float (&l_run)[2],
                                          typename ElemTraits<T>::vec8 (&pb)[2],
                                          typename ElemTraits<T>::vec8 (&vf)[D / 32], float scale_log2) {
  typedef typename ElemTraits<T>::vec8 vec8;
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
    for (int nb = 0; nb < 2; ++nb) acc[db][nb] = Mfma<T>::run(vf[db], pb[nb], acc[db][nb]);
  if (S_IN_VGPR<D>::value) {
#pragma unroll
    for (int k2 = 0; k2 < KH; ++k2)
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) Mfma<T>::run_vgpr_acc(kf[k2], qf[nb][H * KH + k2], s_fill[nb], H == 0 && k2 == 0);
  } else {
    if (H == 0) {
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int i = 0; i < 16; ++i) s_fill[nb][i] = 0.f;
    }
#pragma unroll
    for (int k2 = 0; k2 < KH; ++k2)
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) s_fill[nb] = Mfma<T>::run(kf[k2], qf[nb][H * KH + k2], s_fill[nb]);
  }

  vec8 pn[2];
  float sum[2];
  half_step_p<T, H, !S_IN_VGPR<D>::value>(s_use, m_run, scale_log2, pn, sum);
  // Issue order of the block: each of its 2*D/16 large MFMAs is followed by a share of the P
  // arithmetic (3 plain VALU, 2 exp), so the softmax fills the issue slots behind every MFMA instead
  // of running as one burst after the last of them.  Measured 3 % faster than the scheduler's own order.
#pragma unroll
  for (int g = 0; g < 2 * D / 16; ++g) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
    __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);  // three VALU
    __builtin_amdgcn_sched_group_barrier(0x400, 2, 0);  // two transcendental
  }
  if (S_IN_VGPR<D>::value) {
    // The S^T MFMAs written as assembly get none of the compiler's wait states between an MFMA and a
    // vector instruction that reads its result.  They are all issued before this point, the MFMAs of
    // the sums after it, the matrix pipe completes in order, and the branch below waits for the sums:
    // so when the next block reads S^T, those MFMAs have completed.
    __builtin_amdgcn_sched_barrier(0);
    half_step_sums<T>(pn, sum);
  }
  // One compare for both query blocks: their sums are >= 0 or NaN, so the total is below the limit
  // only if both are.  Not "total >= limit": a NaN (row that has seen nothing yet) must take the rare
  // path too.
  const bool redo = !(sum[0] + sum[1] < HALF_SUM_LIMIT);
  if (__builtin_expect(__builtin_amdgcn_ballot_w64(redo) != 0, false)) {
    float alpha[2];
    half_step_rescale<T, D, H>(s_use, scale_log2, alpha, m_run, l_run, pn, sum);
    // the accumulators hold everything up to the previous half-step (its P.V was issued above; the
    // P.V of this half-step is added by the next block, under the new exponents)
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[db][nb][i] *= alpha[nb];
  }
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
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
__global__ __launch_bounds__(WG_THREADS, (D <= 64 ? 2 : 1)) void ha_attn_fwd_kernel(const ha_attn_kernel_params p) {
  typedef typename ElemTraits<T>::vec8 vec8;
  typedef typename ElemTraits<T>::vec4 vec4;
  constexpr int DV = D;
  constexpr int KSTEPS = D / 16;  // MFMA k-steps of Q.K^T
  constexpr int DB = DV / 32;     // 32-row blocks of O^T
  constexpr int PR = D / 8;       // 16-byte pieces per row

  // Separate LDS objects (two K tiles, two V tiles of KC rows, the query rows): the compiler then
  // knows that a tile being filled from HBM and a tile being read do not alias, and does not
  // serialise them.  The query region (one tile per wave) is reused for the output rows at the end.
  constexpr int TILE_BYTES = KC * D * 2;
  // The key tiles ask for the larger alignment only to be placed first: LDS offsets below 64 KB fit
  // the immediate field of the LDS reads, which matters at d = 128 where the workgroup uses 130 KB.
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

  auto run_tile = [&](const int qt) __attribute__((always_inline)) {
  // ---- row numbers of the queries: the first thing the workgroup has to wait for, so they are asked
  // for before the rest of the set-up (sorted query positions of this head: entries of 4 or 8 bytes,
  // the row number in the low word) ------------------------------------------------------------------
  constexpr int ROWS_PER_LOAD = 64 / PR;
  const int my_pp = lane % PR;  // physical piece of this lane's LDS slot in a tile load
  const int my_lr = lane / PR;  // row inside one tile load
  const int wave_q_first = qt * WG_QUERIES + wave * 64;
  const int idx_shift = p.idx64 ? 3 : 2;
  const int64_t qidx_off = b * p.qi_sb + h * p.qi_sh + (int64_t)seg * p.n_q * p.qi_sn;
  const unsigned char* const q_idx_base = (const unsigned char*)p.q_idx + (qidx_off << idx_shift);
  const uint32_t qi_rb = (uint32_t)p.qi_sn << idx_shift;
  int q_rows[PR];  // rows of this wave's query tile, in the order of its PR loads
  int qrow[2];     // original row of the query a lane's S^T / O^T columns belong to
#pragma unroll
  for (int j = 0; j < PR; ++j) {
    // positions past the end load the index of position 0 (replaced by -1 once all the index loads
    // of the prologue are in flight)
    const int pq = wave_q_first + j * ROWS_PER_LOAD + my_lr;
    q_rows[j] = GATHER ? *reinterpret_cast<const int*>(row_address(q_idx_base, pq < p.n_q ? pq : 0, qi_rb, 0)) : pq;
  }
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const int pq = wave_q_first + nb * 32 + col;
    qrow[nb] = GATHER ? *reinterpret_cast<const int*>(row_address(q_idx_base, pq < p.n_q ? pq : 0, qi_rb, 0)) : pq;
  }
  if (GATHER) __builtin_amdgcn_sched_barrier(0);

  // bases of this (virtual) head as byte pointers, row strides in bytes
  const unsigned char* qb = (const unsigned char*)((const T*)p.q + b * p.q_sb + h * p.q_sh + (p.q_seg_off + (int64_t)seg * p.seg_stride) * p.q_sn);
  const unsigned char* kb = (const unsigned char*)((const T*)p.k + b * p.k_sb + hk * p.k_sh + (p.k_seg_off + (int64_t)seg * p.seg_stride) * p.k_sn);
  const unsigned char* vb = (const unsigned char*)((const T*)p.v + b * p.v_sb + hk * p.v_sh + (p.k_seg_off + (int64_t)seg * p.seg_stride) * p.v_sn);
  unsigned char* ob = (unsigned char*)((T*)p.out + b * p.o_sb + h * p.o_sh + (p.q_seg_off + (int64_t)seg * p.seg_stride) * p.o_sn);
  const uint32_t q_rb = (uint32_t)p.q_sn * 2, k_rb = (uint32_t)p.k_sn * 2, v_rb = (uint32_t)p.v_sn * 2, o_rb = (uint32_t)p.o_sn * 2;
  float* lb = p.lse + b * p.lse_sb + h * p.lse_sh + p.q_seg_off + (int64_t)seg * p.seg_stride;
  const int64_t kidx_off = b * p.ki_sb + hk * p.ki_sh + (int64_t)seg * p.n_k * p.ki_sn;
  const int64_t sidx_off = b * p.si_sb + hk * p.si_sh;

  // ---- key-chunk schedule -------------------------------------------------------------------
  // chunk positions are in units of KC sorted keys, "unwrapped" (taken modulo n_k/KC when used)
  const int nk_chunks = p.n_k / KC;  // GATHER only (n_k % 128 == 0)
  int uni_start = 0, n_blk_chunks = 0, my_lo = 0, my_hi = 0, n_chunks = 0;
  if (GATHER) {
    int start[2], end[2];
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      const int t = qt * 2 + t2;  // reference query tile of 128
      const int block_id = fast_div(t, p.div_block_tiles);
      const int first = block_id * p.block_tiles * 128;
      int last = (block_id + 1) * p.block_tiles * 128;
      last = last < p.n_k ? last : p.n_k;
      int cnt = last > first ? (last - first) / KC : 0;
      if (t * 128 >= p.n_q) cnt = 0;
      int s = first / KC;
      if (!PLAIN && p.smooth) {
        // the window starts (block_tiles - 1) * 64 keys before the tile's own keys, modulo the sequence
        // (src/hyper_attn_triton.py:101,105-106); reduced to 0..n_k-1 here, also when the block is
        // longer than the sequence, and kept behind the first tile's window for the second tile
        int sk = (first + (t - block_id * p.block_tiles) * 128 - ((p.block_tiles - 1) * 128) / 2) % p.n_k;
        sk += sk < 0 ? p.n_k : 0;
        s = sk / KC;
        if (t2 == 1 && s < start[0]) s += nk_chunks;
      }
      start[t2] = s;
      end[t2] = s + cnt;
    }
    if (end[1] == start[1]) { start[1] = end[0]; end[1] = end[0]; }
    uni_start = start[0];
    const int uni_end = end[1] > end[0] ? end[1] : end[0];
    n_blk_chunks = uni_end - uni_start;
    my_lo = start[wave_s >> 1];
    my_hi = end[wave_s >> 1];
    n_chunks = n_blk_chunks + p.sample_chunks;
  } else {
    int kend = p.n_k;
    if (CAUSAL) {
      const int qend = (qt + 1) * WG_QUERIES;
      kend = kend < qend ? kend : qend;
    }
    n_chunks = (kend + KC - 1) / KC;
  }

  // ---- rows: HBM -> LDS without passing through registers -----------------------------------------
  // One global_load_lds moves 16 bytes per lane to 1 KB of consecutive LDS: 64/PR rows of a tile.
  // Wave w issues loads LPW*w .. LPW*w + LPW-1 of a key tile and all PR loads of its own query tile.
  // A lane's LDS slot is (row, physical piece lane % PR); it fetches the logical piece that the
  // swizzle puts there.  Original row numbers are fetched one tile ahead of the rows, so a row load
  // never waits for an index load.
  constexpr int LPW = PR / 4;  // loads per wave per key tile

  // Gathered kernel: original rows of keys kk0 + j*ROWS_PER_LOAD + my_lr (j < LPW) of chunk ci, one
  // register per tile load of the wave.  The source of a chunk is wave-uniform: a run of an index array
  // (sorted keys of the block part, or an explicit sample list), consecutive rows (default samples), or
  // nothing (chunks outside 0..n_chunks-1 read row 0: finite data whose scores are never used).  Index
  // arrays are read as 4-byte words at a stride of 4 or 8 bytes (row numbers fit the low word of an
  // int64).  Row numbers are fetched one iteration before the tile load that uses them and every
  // iteration ends by waiting for all loads, so the loads stay in flight through the iteration's
  // arithmetic, and a register is never written (by the next fetch, load or not) with a load pending.
  // Exact attention needs none of this: its tile loads take their rows from the chunk number.
  struct RowSource {
    int rows[LPW];
  };
  const unsigned char* const blk_idx = (const unsigned char*)p.k_idx + (kidx_off << idx_shift);
  const uint32_t blk_idx_rb = (uint32_t)p.ki_sn << idx_shift;  // bytes between entries of the key order
  const unsigned char* const smp_idx =
      !PLAIN && p.sampled_idx ? (const unsigned char*)p.sampled_idx + (sidx_off << idx_shift) : nullptr;
  // Smooth windows of neighbouring workgroups overlap (a workgroup's window is 640 keys wide and the next
  // one starts 256 keys later).  Every workgroup therefore walks its window in the same phase of the global
  // chunk number: it starts with the chunk whose number is a multiple of the window length and wraps
  // around, so that workgroups running side by side read a chunk they share in the same iteration and one
  // of them finds it in L2.  (The order in which a row's keys are summed changes, nothing else.)
  int blk_rot = 0;
  if (GATHER && !PLAIN && p.smooth && n_blk_chunks > 0) {
    const int phase = uni_start % n_blk_chunks;
    blk_rot = phase ? n_blk_chunks - phase : 0;
  }
  // window position (chunk, from the window's first) of block-part iteration ci
  auto blk_pos = [&](int ci) -> int {
    const int c = ci + blk_rot;
    return c >= n_blk_chunks ? c - n_blk_chunks : c;
  };
  auto fetch_rows = [&](int ci, int kk0, RowSource& rs) {
    // Consecutive rows (or row 0 for every lane) are written first and without a branch; an index run
    // then overwrites them by loads.  A vector write behind a branch that follows a load of the same
    // register would make the compiler wait for every load in flight, the tile loads included.
    const bool in_range = ci >= 0 && ci < n_chunks;
    const int first = in_range ? (ci - n_blk_chunks) * KC + kk0 : 0;
    const uint32_t per_lane = in_range ? 1u : 0u;
#pragma unroll
    for (int j = 0; j < LPW; ++j) rs.rows[j] = (int)__umul24((uint32_t)(j * ROWS_PER_LOAD + my_lr), per_lane) + first;
    if (in_range) {
      if (ci < n_blk_chunks) {
        int u = uni_start + (PLAIN ? ci : blk_pos(ci));
        if (!PLAIN) {  // smooth windows wrap around the key sequence
          u -= u >= nk_chunks ? nk_chunks : 0;
          u -= u >= nk_chunks ? nk_chunks : 0;
        }
        const unsigned char* const src = blk_idx + (uint32_t)(u * KC) * blk_idx_rb;
#pragma unroll
        for (int j = 0; j < LPW; ++j)
          rs.rows[j] = *reinterpret_cast<const int*>(row_address(src, kk0 + j * ROWS_PER_LOAD + my_lr, blk_idx_rb, 0));
      } else if (smp_idx) {
        const unsigned char* const src = smp_idx + ((uint32_t)(ci - n_blk_chunks) * KC << idx_shift);
#pragma unroll
        for (int j = 0; j < LPW; ++j)
          rs.rows[j] = *reinterpret_cast<const int*>(row_address(src, kk0 + j * ROWS_PER_LOAD + my_lr, 1u << idx_shift, 0));
      }
    }
  };
  // V tile c holds keys 0..63 of chunk c.  K tile c holds keys 32..63 of chunk c-1 in its rows 0..31
  // and keys 0..31 of chunk c in its rows 32..63: waves 0,1 load the former, waves 2,3 the latter.
  const int v_kk0 = wave_s * (LPW * ROWS_PER_LOAD);
  const int k_kk0 = (v_kk0 + 32) & 63;
  const int k_chunk_shift = (wave_s >> 1) - 1;
#define HA_FETCH_ROWS_K(tile_c, rs) if (GATHER) fetch_rows((tile_c) + k_chunk_shift, k_kk0, rs);
#define HA_FETCH_ROWS_V(ci, rs) if (GATHER) fetch_rows((ci), v_kk0, rs);
// Gathered kernel: one multiply-add per lane and load turns a row number into an address.  Exact
// attention: the first row of the load goes into the wave-uniform base, the lane's own row and piece
// are loop constants; only a tile that reaches past the last key (or lies before the first chunk:
// row0 < 0, every lane reads row 0) computes and clamps row numbers per lane.  All branches are
// wave-uniform.
#define HA_LOAD_TILE(base, stride, rs, chunk, kk0, tile, SWZ, LIM)                                         \
  if (GATHER) {                                                                                          \
    _Pragma("unroll") for (int j = 0; j < LPW; ++j) {                                                    \
      const int r = (wave_s * LPW + j) * ROWS_PER_LOAD + my_lr;                                          \
      global_to_lds_16(piece_address<NARROW>(base, rs.rows[j], stride, my_pp ^ SWZ(r), LIM),             \
                       (tile) + (wave_s * LPW + j) * 1024);                                              \
    }                                                                                                    \
  } else {                                                                                               \
    /* chunk c is rows 64 c ..; a chunk before the first reads row 0 */                                  \
    const int row0 = (chunk) < 0 ? -1 : (chunk) * KC + (kk0);                                            \
    if (__builtin_expect(row0 >= 0 && row0 + LPW * ROWS_PER_LOAD <= p.n_k, true)) {                      \
      _Pragma("unroll") for (int j = 0; j < LPW; ++j) {                                                  \
        const int r = (wave_s * LPW + j) * ROWS_PER_LOAD + my_lr;                                        \
        const uint32_t first_row = __builtin_amdgcn_readfirstlane((uint32_t)(row0 + j * ROWS_PER_LOAD) * (stride)); \
        global_to_lds_16(piece_address<NARROW>(base + first_row, my_lr, stride, my_pp ^ SWZ(r), LIM),    \
                         (tile) + (wave_s * LPW + j) * 1024);                                            \
      }                                                                                                  \
    } else {                                                                                             \
      _Pragma("unroll") for (int j = 0; j < LPW; ++j) {                                                  \
        const int r = (wave_s * LPW + j) * ROWS_PER_LOAD + my_lr;                                        \
        int row = row0 + j * ROWS_PER_LOAD + my_lr;                                                      \
        if (row0 < 0 || row >= p.n_k) row = 0;                                                           \
        global_to_lds_16(piece_address<NARROW>(base, row, stride, my_pp ^ SWZ(r), LIM),                  \
                         (tile) + (wave_s * LPW + j) * 1024);                                            \
      }                                                                                                  \
    }                                                                                                    \
  }

  // ---- first loads: row numbers of the queries and of the first key tiles, then the rows ----------
  unsigned char* const my_q = lds_q + wave * TILE_BYTES;
  RowSource rows_k, rows_v;
#pragma unroll
  for (int j = 0; j < LPW; ++j) rows_k.rows[j] = rows_v.rows[j] = 0;
  {
    RowSource rows_k1;
#pragma unroll
    for (int j = 0; j < LPW; ++j) rows_k1.rows[j] = 0;
    HA_FETCH_ROWS_K(0, rows_k)
    HA_FETCH_ROWS_V(0, rows_v)
    HA_FETCH_ROWS_K(1, rows_k1)
#pragma unroll
    for (int j = 0; j < PR; ++j)
      if (wave_q_first + j * ROWS_PER_LOAD + my_lr >= p.n_q) q_rows[j] = -1;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
      if (wave_q_first + nb * 32 + col >= p.n_q) qrow[nb] = -1;
    HA_LOAD_TILE(kb, k_rb, rows_k, k_chunk_shift, k_kk0, lds_k0, k_swizzle, p.qk_pieces)
#pragma unroll
    for (int j = 0; j < PR; ++j) {
      // positions past the end read row 0 (finite data; their results are never written)
      const int r = j * ROWS_PER_LOAD + my_lr;
      global_to_lds_16(piece_address<NARROW>(qb, q_rows[j] < 0 ? 0 : q_rows[j], q_rb, my_pp ^ (r & 7), p.qk_pieces),
                       my_q + j * 1024);
      if (my_pp == 0) lds_qrow[wave * 64 + r] = q_rows[j];
    }
    HA_LOAD_TILE(vb, v_rb, rows_v, 0, v_kk0, lds_v0, v_swizzle, p.v_pieces)
    HA_LOAD_TILE(kb, k_rb, rows_k1, 1 + k_chunk_shift, k_kk0, lds_k1, k_swizzle, p.qk_pieces)
  }
  HA_FETCH_ROWS_K(2, rows_k)
  HA_FETCH_ROWS_V(1, rows_v)

  // ---- soft-max state, accumulators ----------------------------------------------------------------
  float m_run[2], l_run[2], m_init[2];
  f32x16 acc[DB][2];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    m_run[nb] = M_FLOOR;
    l_run[nb] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[db][nb][i] = 0.f;
    if (p.accumulate && qrow[nb] >= 0) {
      // resume from a previous partial attention: it enters with weight exp(lse_prev - m) = 1; its
      // normalised output rows are added when the result is written
      // (a previous result of -inf, a row that had no key at all, enters with weight 0)
      const float m_prev = lb[qrow[nb]] * LOG2E;
      if (m_prev > M_FLOOR) {
        m_run[nb] = m_prev;
        l_run[nb] = hi == 0 ? 1.f : 0.f;
      }
    }
    m_init[nb] = m_run[nb];
  }

  // per-lane LDS offsets of the MFMA operand reads
  LaneOffsets<D> lo;
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) lo.k[ks] = tile_offset<D>(col, ks * 2 + hi);
  {
    // transposing read: lane s = 4j + w of a 16-lane group addresses key j (+4 for the upper lane
    // half), dv word w of the 16 dv columns of its group
    const int g = lane >> 4, sl = lane & 15;
    const int key = (g >> 1) * 4 + (sl >> 2);
    const int w = sl & 3;
#pragma unroll
    for (int db = 0; db < DB; ++db)
      lo.v[db] = v_tile_offset<D>(key, db * 4 + (g & 1) * 2 + (w >> 1)) + (w & 1) * 8;
  }

  // every wave's part of Q, K tile 0, V tile 0, K tile 1 has landed before anyone reads the tiles
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  __syncthreads();

  // ---- masks (wave-uniform decision per chunk) -------------------------------------------------
  auto chunk_masked = [&](int ci) -> bool {
    if (PLAIN) return false;
    if (GATHER) {
      if (ci >= n_blk_chunks) return false;
      const int u = uni_start + blk_pos(ci);
      return !(u >= my_lo && u < my_hi);
    }
    const int k_first = ci * KC;
    return (CAUSAL && k_first + KC - 1 > wave_q_first) || (k_first + KC > p.n_k);
  };
  // element i of a lane is key  first + 8*(i/4) + i%4  with first = chunk*64 + mb*32 + 4*hi; it is
  // dead when that exceeds `limit` = min(n_k - 1, query position).  In gather mode a masked chunk is
  // one whose keys belong to the other half of the workgroup: everything is dead.
#define HA_APPLY_MASK(ci, mb, s)                                                        \
  asm volatile("" ::); /* keeps this a branch: masked chunks are the exception */       \
  _Pragma("unroll") for (int nb = 0; nb < 2; ++nb) {                                    \
    const int first = (ci) * KC + (mb) * 32 + 4 * hi;                                   \
    int limit = p.n_k - 1;                                                              \
    if (CAUSAL) limit = min(limit, wave_q_first + nb * 32 + col);                       \
    const int slack = GATHER ? -1 : limit - first;                                      \
    _Pragma("unroll") for (int i = 0; i < 16; ++i)                                      \
      if (8 * (i >> 2) + (i & 3) > slack) s[nb][i] = -INFINITY;                         \
  }

  // Residual estimator (REWEIGHT instances of the general gathered kernel): the scores of the sampled
  // chunks get a bias (log of the sample weight, in raw q.k units), and a sampled key that is among the
  // block keys of this wave's query tile is dead.  Element i of a lane is slot
  // (chunk - n_blk_chunks)*64 + mb*32 + 4*hi + 8*(i/4) + i%4 of the sample list; its key's position in the
  // sorted order comes from sampled_pos (the same for all lanes of a lane half: broadcast loads).
  const int32_t* const smp_pos = REWEIGHT && p.sampled_pos ? p.sampled_pos + sidx_off : nullptr;
  const int win_first = my_lo - (my_lo >= nk_chunks ? nk_chunks : 0);  // first chunk of the tile's key window
  const int win_chunks = my_hi - my_lo;
#define HA_REWEIGHT(ci, mb, s)                                                          \
  if (REWEIGHT && (ci) >= n_blk_chunks) {                                               \
    const int slot0 = ((ci) - n_blk_chunks) * KC + (mb) * 32 + 4 * hi;                  \
    _Pragma("unroll") for (int i = 0; i < 16; ++i) {                                    \
      bool dead = false;                                                                \
      if (smp_pos) {                                                                    \
        int c = (smp_pos[slot0 + 8 * (i >> 2) + (i & 3)] >> 6) - win_first;             \
        c += c < 0 ? nk_chunks : 0;                                                     \
        dead = c < win_chunks;                                                          \
      }                                                                                 \
      _Pragma("unroll") for (int nb = 0; nb < 2; ++nb)                                  \
        s[nb][i] = dead ? -INFINITY : s[nb][i] + p.sample_bias_raw;                     \
    }                                                                                   \
  }

  // ---- Q fragments (B operand), S^T of the first 32 keys ---------------------------------------
  vec8 qf[2][KSTEPS];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb)
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) qf[nb][ks] = lds_read_k<T>(my_q, lo.k[ks] + nb * 32 * D * 2);
  // s_a / s_b hold S^T of keys 0..31 / 32..63 of the chunk being consumed
  f32x16 s_a[2], s_b[2];
  {
    vec8 kf[KSTEPS];
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) kf[ks] = lds_read_k<T>(lds_k0, lo.k[ks] + 32 * D * 2);
    if (S_IN_VGPR<D>::value) {
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) Mfma<T>::run_vgpr_acc(kf[ks], qf[nb][ks], s_a[nb], ks == 0);
    } else {
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int i = 0; i < 16; ++i) s_a[nb][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) s_a[nb] = Mfma<T>::run(kf[ks], qf[nb][ks], s_a[nb]);
    }
  }
  // the P.V of "the half-step before the first" adds nothing
  vec8 pb[2], vf[DB];
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) pb[nb] = vec8{};
#pragma unroll
  for (int db = 0; db < DB; ++db) vf[db] = vec8{};
  bool pending = false;  // pb/vf hold a half-step whose P.V has not been issued
  // all waves hold their operands of K tile 0: its buffer may be overwritten from iteration 0 on
  __syncthreads();

  // ---- main loop -----------------------------------------------------------------------------------
  // Iteration ci consumes chunk ci: its steps 0 and 1 soft-max s_a and s_b, read V tile ci, and fill
  // s_b and (for chunk ci+1) s_a from K tile ci+1.  Meanwhile K tile ci+2 streams into the buffer K
  // tile ci was read from during iteration ci-1, and V tile ci+1 into the buffer of V tile ci-1.
  // The loop is unrolled by two so that every tile access names its LDS object statically.
#define HA_PV_DRAIN()                                                                                       \
  _Pragma("unroll") for (int db = 0; db < DB; ++db) _Pragma("unroll") for (int nb = 0; nb < 2; ++nb)        \
      acc[db][nb] = Mfma<T>::run(vf[db], pb[nb], acc[db][nb]);
  /* consecutive rows known to lie inside the keys: no row numbers, no bounds */                             \
#define HA_LOAD_TILE_INSIDE(base, stride, chunk, kk0, tile, SWZ, LIM)                                         \
  _Pragma("unroll") for (int j = 0; j < LPW; ++j) {                                                         \
    const int r = (wave_s * LPW + j) * ROWS_PER_LOAD + my_lr;                                               \
    const uint32_t first_row =                                                                              \
        __builtin_amdgcn_readfirstlane((uint32_t)((chunk) * KC + (kk0) + j * ROWS_PER_LOAD) * (stride));    \
    global_to_lds_16(piece_address<NARROW>(base + first_row, my_lr, stride, my_pp ^ SWZ(r), LIM),           \
                     (tile) + (wave_s * LPW + j) * 1024);                                                   \
  }
  // INTERIOR (exact attention only): every row of the tiles the iteration loads exists and no score of
  // the chunk it consumes is masked for any wave, so all of that bookkeeping is compiled out
#define HA_ITERATION(ci, K_RD, K_WR, V_CUR, V_WR, INTERIOR)                                                 \
  {                                                                                                         \
    if (INTERIOR) {                                                                                         \
      HA_LOAD_TILE_INSIDE(kb, k_rb, (ci) + 2 + k_chunk_shift, k_kk0, K_WR, k_swizzle, p.qk_pieces)                       \
      HA_LOAD_TILE_INSIDE(vb, v_rb, (ci) + 1, v_kk0, V_WR, v_swizzle, p.v_pieces)                                       \
    } else {                                                                                                \
      if (__builtin_expect((ci) + 2 <= n_chunks, true)) {                                                   \
        HA_LOAD_TILE(kb, k_rb, rows_k, (ci) + 2 + k_chunk_shift, k_kk0, K_WR, k_swizzle, p.qk_pieces) /* K tile ci+2 */  \
      }                                                                                                     \
      if (__builtin_expect((ci) + 1 < n_chunks, true)) {                                                    \
        HA_LOAD_TILE(vb, v_rb, rows_v, (ci) + 1, v_kk0, V_WR, v_swizzle, p.v_pieces) /* V tile ci+1 */                  \
      }                                                                                                     \
      HA_FETCH_ROWS_K((ci) + 3, rows_k)                                                                     \
      HA_FETCH_ROWS_V((ci) + 2, rows_v)                                                                     \
    }                                                                                                       \
    /* causal: once a chunk lies wholly above this wave's queries, so do all later ones */                  \
    if (INTERIOR || !(CAUSAL && (ci) * KC > wave_q_first + 63)) {                                           \
      const bool masked = INTERIOR ? false : chunk_masked(ci);                                              \
      if (__builtin_expect(masked, false)) { HA_APPLY_MASK(ci, 0, s_a) }                                    \
      HA_REWEIGHT(ci, 0, s_a)                                                                               \
      half_step<T, D, 0>(s_a, s_b, K_RD, 0, V_CUR, 0, lo, qf, acc, m_run, l_run, pb, vf,                    \
                         p.scale_log2);                                                                     \
      half_step<T, D, 1>(s_a, s_b, K_RD, 0, V_CUR, 16 * D * 2, lo, qf, acc, m_run, l_run, pb, vf,           \
                         p.scale_log2);                                                                     \
      if (__builtin_expect(masked, false)) { HA_APPLY_MASK(ci, 1, s_b) }                                    \
      HA_REWEIGHT(ci, 1, s_b)                                                                               \
      half_step<T, D, 0>(s_b, s_a, K_RD, 32 * D * 2, V_CUR, 32 * D * 2, lo, qf, acc, m_run, l_run, pb, vf,  \
                         p.scale_log2);                                                                     \
      half_step<T, D, 1>(s_b, s_a, K_RD, 32 * D * 2, V_CUR, 48 * D * 2, lo, qf, acc, m_run, l_run, pb, vf,  \
                         p.scale_log2);                                                                     \
      pending = true;                                                                                       \
    } else if (pending) {                                                                                   \
      HA_PV_DRAIN()                                                                                         \
      pending = false;                                                                                      \
    }                                                                                                       \
    __builtin_amdgcn_s_waitcnt(0x0F70); /* this wave's parts of K tile ci+2, V tile ci+1 have landed */     \
    __syncthreads();                                                                                        \
  }
  int ci = 0;
  if (!GATHER) {
    // chunks 0 .. n_interior-1 (an even number): chunk ci + 2 is not the last one, so all its rows
    // exist, and causal chunks end at or before the first query of the workgroup
    int n_interior = n_chunks - 3;
    if (CAUSAL) n_interior = min(n_interior, qt * (WG_QUERIES / KC));
    n_interior = max(n_interior, 0) & ~1;
    for (; ci < n_interior; ci += 2) {
      HA_ITERATION(ci, lds_k1, lds_k0, lds_v0, lds_v1, true)
      HA_ITERATION(ci + 1, lds_k0, lds_k1, lds_v1, lds_v0, true)
    }
  }
  for (; ci < n_chunks; ci += 2) {
    HA_ITERATION(ci, lds_k1, lds_k0, lds_v0, lds_v1, false)
    if (ci + 1 < n_chunks) HA_ITERATION(ci + 1, lds_k0, lds_k1, lds_v1, lds_v0, false)
  }
  if (pending) { HA_PV_DRAIN() }
#undef HA_ITERATION
#undef HA_LOAD_TILE_INSIDE
#undef HA_PV_DRAIN

  // ---- epilogue: normalise, stage O through LDS, write whole rows ---------------------------------
  // A wave's 64 output rows are exactly one tile (64 rows of DV elements): it stages them in its
  // query tile and writes them out itself, so no further workgroup barrier is needed.  Piece j of a
  // lane belongs to the row its j-th query load fetched.
  constexpr int OUT_PIECES = PR;  // 16-byte pieces per lane
  int out_row[OUT_PIECES];
  vec8 prev[OUT_PIECES];
#pragma unroll
  for (int j = 0; j < OUT_PIECES; ++j) out_row[j] = lds_qrow[wave * 64 + j * ROWS_PER_LOAD + my_lr];
  if (p.accumulate) {
#pragma unroll
    for (int j = 0; j < OUT_PIECES; ++j) {
      // positions past the end read row 0 (never written back): an unconditional load needs no zero fill
      prev[j] = *reinterpret_cast<const vec8*>(
          piece_address<NARROW>(ob, out_row[j] < 0 ? 0 : out_row[j], o_rb, my_pp, p.v_pieces));
    }
  }
  T* const lds_o = reinterpret_cast<T*>(my_q);
#pragma unroll
  for (int nb = 0; nb < 2; ++nb) {
    const float l_tot = ha_sum_xor32(l_run[nb]);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int lrow = nb * 32 + col;
    if (hi == 0) {
      if (qrow[nb] >= 0) lb[qrow[nb]] = l_tot > 0.f && m_run[nb] > M_FLOOR ? (m_run[nb] + __builtin_amdgcn_logf(l_tot)) * LN2 : -INFINITY;
      // weight of the resumed rows: exp(lse_prev - m_final) / l_tot
      lds_w[wave * 64 + lrow] = m_init[nb] > M_FLOOR ? __builtin_amdgcn_exp2f(m_init[nb] - m_run[nb]) * inv : 0.f;
    }
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
  __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wave's LDS writes are done
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int j = 0; j < OUT_PIECES; ++j) {
    const int lrow = j * ROWS_PER_LOAD + my_lr;
    if (out_row[j] >= 0 && (!NARROW || my_pp < p.v_pieces)) {
      vec8 o = *reinterpret_cast<const vec8*>(&lds_o[lrow * DV + ((my_pp ^ (lrow & 7)) * 8)]);
      if (p.accumulate) {
        const float w = lds_w[wave * 64 + lrow];
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (T)__builtin_fmaf(w, (float)prev[j][e], (float)o[e]);
      }
      *reinterpret_cast<vec8*>(const_cast<unsigned char*>(row_address(ob, out_row[j], o_rb, my_pp * 16))) = o;
    }
  }
#undef HA_FETCH_ROWS_K
#undef HA_FETCH_ROWS_V
#undef HA_LOAD_TILE
#undef HA_APPLY_MASK
#undef HA_REWEIGHT
  };  // run_tile
  if (PAIRED) {
    // the long tile first.  No barrier between the two: the last iteration of a tile ends with one, and after
    // it a wave touches only its own part of the query region.
    const int t_long = qtiles - 1 - slot;
    run_tile(t_long);
    if (slot != t_long) run_tile(slot);
  } else {
    run_tile(slot);
  }
}

namespace {

template <typename T, int D, bool GATHER, bool CAUSAL, bool PLAIN = false, bool NARROW = false, bool REWEIGHT = false>
int launch_one(const ha_attn_kernel_params& p, int grid, hipStream_t stream, const char* what) {
  hipLaunchKernelGGL((ha_attn_fwd_kernel<T, D, GATHER, CAUSAL, PLAIN, NARROW, REWEIGHT>), dim3(grid), dim3(WG_THREADS), 0,
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
