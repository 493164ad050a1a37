// MFMA attention backward kernels for gfx950: gradients of the sorted block-diagonal + sampled-column
// attention and of exact (flash) attention with respect to q, k and v.
//
// Reference semantics: _hyper_attn_backward with _bwd_preprocess_do_o_dot,
// _bwd_permuted_block_diagonal_kernel and _bwd_sampled_col_kernel (src/hyper_attn_triton.py:195-665,
// :745-893) and _flash_attn_backward (src/flash_attn_triton.py:270-792, :875-992): given dO, the
// forward's O and its log-sum-exp L (a gradient arriving for L itself is ignored, as in
// HyperAttnFunc.backward, src/hyper_attn_triton.py:922-945),
//   D_i  = sum_c dO_ic O_ic,            P_ij = exp(scale q_i.k_j - L_i),
//   dV_j = sum_i P_ij dO_i,             dS_ij = P_ij (dO_i.v_j - D_i) scale,
//   dQ_i = sum_j dS_ij k_j,             dK_j = sum_i dS_ij q_i,
// over exactly the (query, key) pairs the forward visits: a key that is both in a query's block and in
// the sample list counts twice.  P and dS are rounded to the input type before the products, as the
// reference does.
//
// One kernel body serves five passes.  A workgroup of 4 waves keeps 128 "stationary" rows (32 per
// wave, as B operands in registers) and streams tiles of 64 rows of the other side through LDS:
//   dQ passes    stationary = queries (Q, dO), streamed = keys (K, V):      dQ^T += K^T dS^T
//   dK/dV passes stationary = keys (K, V),     streamed = queries (Q, dO):  dK^T += Q^T dS, dV^T += dO^T P
// Both compute S' = Y1 X1^T and dP' = Y2 X2^T (streamed rows as MFMA rows, stationary rows as MFMA
// columns), so a lane holds 16 streamed rows of ONE stationary row and P', dS' are the B operands of
// the products that follow, whose A operands (Y^T) come from the transposing LDS reads.  The dQ passes
// see all keys of a query in one workgroup and store dQ.  The dK/dV pass of exact attention sees all
// queries of a key (of every query head of the key head's group, streamed one head after the other)
// and stores dK, dV.  With sorted blocks a key gets one contribution from its block (complete in one
// workgroup: stored like the exact pass's) and, if it is in the sample list, one from every query:
// those are computed per range of queries and summed with atomics in small fp32 rows, one per slot of
// the sample list, which a last kernel adds to the keys' rows of dK, dV.
#include "ha_common.h"
#include "attn_tiles.h"
#include "attn_fwd.h"
#include "attn_bwd.h"

#include <type_traits>

namespace {

constexpr int WG_THREADS = 256;
constexpr int ST_ROWS = 128;       // stationary rows per workgroup
constexpr int YC = 64;             // streamed rows per LDS tile
constexpr int MAX_SMOOTH_TILES = 1024;  // query tiles that can attend one 128-key tile (smoothed blocks)

// LDS layout of a streamed tile: row-major [64][D] 2-byte elements, the 16-byte pieces of a row XOR-ed
// with a function of the row number chosen so that BOTH ways the tile is read are free of bank
// conflicts (the LDS serves 16 lanes, 64 banks of 4 bytes, at a time):
//   row reads (ds_read_b128): 16 lanes read the same piece of 16 consecutive rows -> the 16 rows
//     must land in 16 different 16-byte slots of the 256-byte bank window;
//   transposing reads (ds_read_b64_tr_b16): 16 lanes read 2 adjacent pieces of 4 consecutive rows
//     (starting at a multiple of 4) -> the four pairs must differ in a bit above the lowest.
// d = 64 (a row is half a bank window, so rows of equal parity compete for 8 slots): the bits 1,2,3
// of the row number, in reversed order.  d = 128 (16 slots per row): the low four bits of the row
// number with the two pairs of bits exchanged.
template <int D>
__device__ __forceinline__ int bwd_swizzle(int row) {
  if (D == 64) return (((row >> 1) & 1) << 2) | (((row >> 2) & 1) << 1) | ((row >> 3) & 1);
  return ((row & 3) << 2) | ((row >> 2) & 3);
}
template <int D>
__device__ __forceinline__ int bwd_tile_offset(int row, int piece) {
  return row * D * 2 + ((piece ^ bwd_swizzle<D>(row)) << 4);
}

// 8 streamed rows x 1 column, transposed by the LDS unit: rows 0..3 and 8..11 (+4 for the upper lane
// half) relative to the row the offsets were computed for
template <typename T>
__device__ __forceinline__ typename ElemTraits<T>::vec8 bwd_read_tr(const unsigned char* tile, int off_lo, int off_hi) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(tile + off_lo));
  const s16x4 hi8 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(tile + off_hi));
  const s16x8 both = __builtin_shufflevector(lo, hi8, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(typename ElemTraits<T>::vec8, both);
#else
  return typename ElemTraits<T>::vec8{};
#endif
}

template <typename T, int D, int PASS, bool CAUSAL>
__global__ __launch_bounds__(WG_THREADS, (D <= 64 || PASS == HA_BWD_DQ_BLOCK ? 2 : 1)) void ha_attn_bwd_kernel(const ha_attn_bwd_params p) {
  typedef typename ElemTraits<T>::vec8 vec8;
  typedef typename ElemTraits<T>::vec4 vec4;
  constexpr bool KEY_ST = PASS == HA_BWD_DKV_EXACT || PASS == HA_BWD_DKV_BLOCK || PASS == HA_BWD_DKV_SAMPLED;
  // the gathered dK/dV passes start their dP accumulators from -D (below); the exact pass, at its register
  // limit, subtracts D * scale per pair like the dQ passes
  constexpr bool FOLD_D = PASS == HA_BWD_DKV_BLOCK || PASS == HA_BWD_DKV_SAMPLED;
  constexpr int KSTEPS = D / 16;  // MFMA k-steps over the head dim
  constexpr int DB = D / 32;      // 32-row blocks of the transposed gradients
  constexpr int PR = D / 8;       // 16-byte pieces per row
  constexpr int RPL = 64 / PR;    // rows per tile load (one load = 64 lanes x 16 bytes)
  constexpr int LPW = PR / 4;     // tile loads per wave per tile
  constexpr int TILE_BYTES = YC * D * 2;

  __shared__ __attribute__((aligned(1024))) unsigned char lds_y1[2][TILE_BYTES];
  __shared__ __attribute__((aligned(1024))) unsigned char lds_y2[2][TILE_BYTES];
  __shared__ __attribute__((aligned(16))) float lds_lse[2][YC];    // dK/dV passes: L (log2 units) of the streamed queries
  __shared__ __attribute__((aligned(16))) float lds_delta[2][YC];  // and their -D (gathered passes) or D * scale (exact pass)
  constexpr bool STAGE_X = KEY_ST || D <= 64;
  __shared__ __attribute__((aligned(1024))) unsigned char lds_x1[STAGE_X ? ST_ROWS * D * 2 : 16];  // staging of the
  __shared__ __attribute__((aligned(1024))) unsigned char lds_x2[STAGE_X ? ST_ROWS * D * 2 : 16];  // stationary rows
  __shared__ int lds_tiles[PASS == HA_BWD_DKV_BLOCK ? MAX_SMOOTH_TILES : 1];
  __shared__ int lds_ntiles;

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int wave_s = __builtin_amdgcn_readfirstlane(wave);
  const int hi = lane >> 5, col = lane & 31;

  // ---- which head, which stationary tile ------------------------------------------------------
  const int st_total = PASS == HA_BWD_DKV_SAMPLED ? p.sample_size : (KEY_ST ? p.n_k : p.n_q);
  const int st_tiles = (st_total + ST_ROWS - 1) / ST_ROWS;
  const int splits = PASS == HA_BWD_DKV_SAMPLED ? (p.n_q + p.q_split - 1) / p.q_split : 1;
  int rest = xcd_contiguous_id(blockIdx.x, gridDim.x);
  int tile = rest % st_tiles;
  rest /= st_tiles;
  // causal dq: the tiles with the most keys first, so that the last workgroups of the grid are short
  // (the dk/dv tiles are in that order as they come: the first key tile streams the most queries)
  if (PASS == HA_BWD_DQ_EXACT && CAUSAL) tile = st_tiles - 1 - tile;
  const int split = rest % splits;
  const int vseq = rest / splits;   // (batch, head, segment)
  const int seg = vseq % p.segs;
  const int bh = vseq / p.segs;
  // The dK/dV passes that see every query of a key (exact attention, the blocks) take one workgroup per
  // KEY head and stream the queries of all the query heads of its group, one head after the other, so
  // that the sums are complete in registers; the other passes take one workgroup per query head.
  constexpr bool GROUP_LOOP = PASS == HA_BWD_DKV_EXACT || PASS == HA_BWD_DKV_BLOCK;
  const int kv_heads = p.heads / p.kv_group;
  int b, h0, hk;
  if (GROUP_LOOP) {
    b = bh / kv_heads;
    hk = bh - b * kv_heads;
    h0 = hk * p.kv_group;
  } else {
    b = bh / p.heads;
    h0 = bh - b * p.heads;
    hk = h0 / p.kv_group;
  }
  const int n_group = GROUP_LOOP ? p.kv_group : 1;
  // first row of this segment in the query-side and in the key-side tensors
  const int64_t q_row0 = p.q_seg_off + (int64_t)seg * p.seg_stride;
  const int64_t k_row0 = p.k_seg_off + (int64_t)seg * p.seg_stride;

  // query-side tensors of query head h0 + gi
  auto q_head = [&](int gi) { return (const unsigned char*)((const T*)p.q + b * p.q_sb + (h0 + gi) * p.q_sh + q_row0 * p.q_sn); };
  auto do_head = [&](int gi) { return (const unsigned char*)((const T*)p.dout + b * p.do_sb + (h0 + gi) * p.do_sh + q_row0 * p.do_sn); };
  // per query: {L in log2 units, -D} with D_i = sum_c dO_ic O_ic (src/hyper_attn_triton.py:195-226),
  // written by the dq pass of the call
  auto stats_head = [&](int gi) { return p.stats + ((int64_t)(b * p.heads + h0 + gi) * p.segs + seg) * p.n_q; };
  const int idx_shift = p.idx64 ? 3 : 2;
  auto q_idx_head = [&](int gi) {
    return (const unsigned char*)p.q_idx + ((b * p.qi_sb + (h0 + gi) * p.qi_sh + (int64_t)seg * p.n_q * p.qi_sn) << idx_shift);
  };
  const unsigned char* const kb = (const unsigned char*)((const T*)p.k + b * p.k_sb + hk * p.k_sh + k_row0 * p.k_sn);
  const unsigned char* const vb = (const unsigned char*)((const T*)p.v + b * p.v_sb + hk * p.v_sh + k_row0 * p.v_sn);
  const uint32_t q_rb = (uint32_t)p.q_sn * 2, k_rb = (uint32_t)p.k_sn * 2, v_rb = (uint32_t)p.v_sn * 2,
                 do_rb = (uint32_t)p.do_sn * 2;
  const unsigned char* const k_idx = (const unsigned char*)p.k_idx + ((b * p.ki_sb + hk * p.ki_sh + (int64_t)seg * p.n_k * p.ki_sn) << idx_shift);
  const unsigned char* const s_idx =
      p.sampled_idx ? (const unsigned char*)p.sampled_idx + ((b * p.si_sb + hk * p.si_sh) << idx_shift) : nullptr;
  const uint32_t qi_rb = (uint32_t)p.qi_sn << idx_shift, ki_rb = (uint32_t)p.ki_sn << idx_shift;
  const uint32_t si_rb = 1u << idx_shift;

  // stationary (X) and streamed (Y) operands of this pass
  const unsigned char* const x1b = KEY_ST ? kb : q_head(0);
  const unsigned char* const x2b = KEY_ST ? vb : do_head(0);
  const uint32_t x1_rb = KEY_ST ? k_rb : q_rb, x2_rb = KEY_ST ? v_rb : do_rb;
  const uint32_t y1_rb = KEY_ST ? q_rb : k_rb, y2_rb = KEY_ST ? do_rb : v_rb;
  const int n_y = KEY_ST ? p.n_q : p.n_k;  // rows on the streamed side

  // ---- the stationary row of this lane's MFMA column ------------------------------------------
  const int st_pos = tile * ST_ROWS + wave * 32 + col;  // position in the stationary order
  const bool st_valid = st_pos < st_total;
  int st_row;  // original row
  {
    const int pos = st_valid ? st_pos : 0;
    if (PASS == HA_BWD_DQ_BLOCK)
      st_row = *reinterpret_cast<const int*>(row_address(q_idx_head(0), pos, qi_rb, 0));
    else if (PASS == HA_BWD_DKV_BLOCK)
      st_row = *reinterpret_cast<const int*>(row_address(k_idx, pos, ki_rb, 0));
    else if (PASS == HA_BWD_DKV_SAMPLED)
      st_row = s_idx ? *reinterpret_cast<const int*>(row_address(s_idx, pos, si_rb, 0)) : pos;
    else
      st_row = pos;
  }
  // ---- the streamed chunks of this workgroup ---------------------------------------------------
  const int T_blk = p.block_tiles;
  const int nkc = p.n_k / YC;  // gathered passes: n_k % 128 == 0
  int nc = 0;                  // number of streamed chunks
  int y_first = 0;             // exact / sampled passes: first streamed row
  int y_end = n_y;             // exact / sampled passes: end of the valid streamed rows
  int blk_start = 0, n_blk = 0;  // dQ of the gathered kernel: first chunk (sorted keys) and count of the block part
  int t_first = 0;               // dK/dV of the block part, plain blocks: first attending query tile
  if (PASS == HA_BWD_DQ_EXACT) {
    if (CAUSAL) {
      const int qend = (tile + 1) * ST_ROWS;
      y_end = y_end < qend ? y_end : qend;
    }
    nc = (y_end + YC - 1) / YC;
  } else if (PASS == HA_BWD_DKV_EXACT) {
    y_first = CAUSAL ? tile * ST_ROWS : 0;
    nc = y_end > y_first ? (y_end - y_first + YC - 1) / YC : 0;
  } else if (PASS == HA_BWD_DKV_SAMPLED) {
    y_first = split * p.q_split;
    const int e = y_first + p.q_split;
    y_end = e < p.n_q ? e : p.n_q;
    nc = (y_end - y_first + YC - 1) / YC;
  } else if (PASS == HA_BWD_DQ_BLOCK) {
    // the key window of reference query tile `tile` (src/hyper_attn_triton.py:99-107)
    const int block_id = tile / T_blk;
    const int first = block_id * T_blk * 128;
    int last = first + T_blk * 128;
    last = last < p.n_k ? last : p.n_k;
    n_blk = last > first ? (last - first) / YC : 0;
    blk_start = first / YC;
    if (p.smooth) {
      int sk = (tile * 128 - (T_blk - 1) * 64) % p.n_k;
      sk += sk < 0 ? p.n_k : 0;
      blk_start = sk / YC;
    }
    nc = n_blk + p.sample_size / YC;
  } else {  // HA_BWD_DKV_BLOCK: the query tiles whose window holds this key tile
    const int n_qt = p.n_q / 128;
    if (!p.smooth) {
      const int block_id = tile / T_blk;
      t_first = block_id * T_blk;
      int t_last = t_first + T_blk;
      t_last = t_last < n_qt ? t_last : n_qt;
      nc = t_last > t_first ? 2 * (t_last - t_first) : 0;
    } else {
      // list them (ascending), with one flag per 64-key half of this tile: bit 30 lower, bit 31 upper
      if (wave_s == 0) {
        int count = 0;
        for (int t0 = 0; t0 < n_qt; t0 += 64) {
          const int t = t0 + lane;
          bool m0 = false, m1 = false;
          if (t < n_qt) {
            const int block_id = t / T_blk;
            const int first = block_id * T_blk * 128;
            int last = first + T_blk * 128;
            last = last < p.n_k ? last : p.n_k;
            const int cnt = last > first ? (last - first) / YC : 0;
            int sk = (t * 128 - (T_blk - 1) * 64) % p.n_k;
            sk += sk < 0 ? p.n_k : 0;
            int o0 = 2 * tile - sk / YC;
            o0 += o0 < 0 ? nkc : 0;
            int o1 = 2 * tile + 1 - sk / YC;
            o1 += o1 < 0 ? nkc : 0;
            m0 = o0 < cnt;
            m1 = o1 < cnt;
          }
          const bool any = m0 || m1;
          const uint64_t mask = __ballot(any);
          if (any) {
            const int pos = count + __popcll(mask & ((1ull << lane) - 1));
            if (pos < MAX_SMOOTH_TILES) lds_tiles[pos] = t | (m0 ? 1 << 30 : 0) | (m1 ? (int)(1u << 31) : 0);
          }
          count += __popcll(mask);
        }
        if (lane == 0) lds_ntiles = count < MAX_SMOOTH_TILES ? count : MAX_SMOOTH_TILES;
      }
      __syncthreads();
      nc = 2 * lds_ntiles;
    }
  }
  const int nc_head = __builtin_amdgcn_readfirstlane(nc);  // chunks per query head
  nc = nc_head * n_group;

  // Original row of streamed row r (0..63) of chunk c, clamped to rows that exist; chunks past the
  // end repeat the last one.  Gathered passes read an index array here.
  auto attending_tile = [&](int k) -> int {  // dK/dV of the block part: k-th attending query tile with its flags
    if (PASS != HA_BWD_DKV_BLOCK) return 0;
    return p.smooth ? lds_tiles[k] : ((t_first + k) | (int)(3u << 30));
  };
  auto group_of = [&](int c) -> int { return n_group == 1 ? 0 : (c < nc ? c : nc - 1) / nc_head; };
  auto stream_row = [&](int c, int r) -> int {
    c = c < nc ? c : nc - 1;
    const int gi = group_of(c);
    c -= gi * nc_head;
    if (PASS == HA_BWD_DQ_BLOCK) {
      if (c < n_blk) {
        int u = blk_start + c;
        u -= u >= nkc ? nkc : 0;
        return *reinterpret_cast<const int*>(row_address(k_idx, u * YC + r, ki_rb, 0));
      }
      const int s = (c - n_blk) * YC + r;
      return s_idx ? *reinterpret_cast<const int*>(row_address(s_idx, s, si_rb, 0)) : s;
    } else if (PASS == HA_BWD_DKV_BLOCK) {
      const int t = attending_tile(c >> 1) & 0x3fffffff;
      return *reinterpret_cast<const int*>(row_address(q_idx_head(gi), t * 128 + (c & 1) * YC + r, qi_rb, 0));
    } else {
      const int row = y_first + c * YC + r;
      return row < n_y ? row : n_y - 1;
    }
  };

  if (nc <= 0) {
    // nothing attends (or is attended by) this tile: its gradient is zero
    if (PASS != HA_BWD_DKV_SAMPLED && st_valid) {
      const vec4 zero = {(T)0.f, (T)0.f, (T)0.f, (T)0.f};
      unsigned char* const dqb = (unsigned char*)((T*)p.dq + b * p.dq_sb + h0 * p.dq_sh + q_row0 * p.dq_sn) + (int64_t)st_row * p.dq_sn * 2;
      unsigned char* const dkb = (unsigned char*)((T*)p.dk + b * p.dk_sb + hk * p.dk_sh + k_row0 * p.dk_sn) + (int64_t)st_row * p.dk_sn * 2;
      unsigned char* const dvb = (unsigned char*)((T*)p.dv + b * p.dv_sb + hk * p.dv_sh + k_row0 * p.dv_sn) + (int64_t)st_row * p.dv_sn * 2;
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int dd = 32 * db + 8 * g + 4 * hi;
          if (!KEY_ST) {
            if (!p.accumulate) *reinterpret_cast<vec4*>(dqb + dd * 2) = zero;
          } else if (!p.accumulate) {
            *reinterpret_cast<vec4*>(dkb + dd * 2) = zero;
            *reinterpret_cast<vec4*>(dvb + dd * 2) = zero;
          }
        }
    }
    return;
  }

  // ---- tile loads: HBM -> LDS, 16 bytes per lane, whole rows, swizzle applied on the source side ----
  const int my_pp = lane % PR;  // physical piece of this lane's LDS slot
  const int my_lr = lane / PR;  // row inside one tile load
  int rows_next[LPW];           // source rows of this wave's loads of the next tile
  int group_next = 0;           // the query head (within the group) those rows belong to
  int stat_row_next = 0;        // dK/dV passes: source row of streamed row 16 * wave + lane % 16 of the next tile
                                // (every wave fetches the statistics of 16 rows: no wave has more to do)
  bool stat_past_end_next = false;
  float stat_lse = 0.f, stat_delta = 0.f;
  auto fetch_rows = [&](int c) {
#pragma unroll
    for (int j = 0; j < LPW; ++j) rows_next[j] = stream_row(c, (wave_s * LPW + j) * RPL + my_lr);
    if (KEY_ST) {
      stat_row_next = stream_row(c, wave_s * 16 + (lane & 15));
      // sampled keys: a streamed query past the end of the workgroup's range gets L = +inf below, so that
      // P = 2^(s - inf) = 0 and dS = 0 * finite = 0 with no mask in the chunk
      if (PASS == HA_BWD_DKV_SAMPLED) {
        const int cc = (c < nc ? c : nc - 1) - group_of(c) * nc_head;
        stat_past_end_next = y_first + cc * YC + wave_s * 16 + (lane & 15) >= y_end;
      }
    }
    group_next = group_of(c);
  };
  auto load_tile = [&](int buf) {  // the tile whose rows are in rows_next
    const unsigned char* const y1b = KEY_ST ? q_head(group_next) : kb;
    const unsigned char* const y2b = KEY_ST ? do_head(group_next) : vb;
#pragma unroll
    for (int j = 0; j < LPW; ++j) {
      const int r = (wave_s * LPW + j) * RPL + my_lr;
      const uint32_t piece = (uint32_t)((my_pp ^ bwd_swizzle<D>(r)) << 4);
      unsigned char* const dst1 = lds_y1[buf] + (wave_s * LPW + j) * 1024;
      unsigned char* const dst2 = lds_y2[buf] + (wave_s * LPW + j) * 1024;
      global_to_lds_16(row_address(y1b, rows_next[j], y1_rb, piece), dst1);
      global_to_lds_16(row_address(y2b, rows_next[j], y2_rb, piece), dst2);
    }
    if (KEY_ST) {
      const f32x2 sd = stats_head(group_next)[stat_row_next];
      stat_lse = stat_past_end_next ? __builtin_inff() : sd[0];
      stat_delta = FOLD_D ? sd[1] : -sd[1] * p.scale;  // the word holds -D
    }
  };

  // the row numbers of the first tile are asked for before the stationary rows, so that the two chains
  // index -> rows run side by side
  fetch_rows(0);
  vec8 x1f[KSTEPS], x2f[KSTEPS];
  float st_lse2 = 0.f, st_delta = 0.f;  // dQ passes: L (log2 units) and D * scale of the lane's query
  f32x16 neg_d;  // dQ passes: -D in every element, what the dP accumulators of a chunk start from
#pragma unroll
  for (int i = 0; i < 16; ++i) neg_d[i] = 0.f;
  vec8 of[KSTEPS];  // dQ passes: the lane's pieces of its query's output row
  const unsigned char* const ob = (const unsigned char*)((const T*)p.out + b * p.o_sb + h0 * p.o_sh + q_row0 * p.o_sn);
  const uint32_t o_rb = (uint32_t)p.o_sn * 2;
  if (!KEY_ST) {
    if (!STAGE_X) {
#pragma unroll
      for (int ks = 0; ks < KSTEPS; ++ks)
        of[ks] = *reinterpret_cast<const vec8*>(row_address(ob, st_row, o_rb, (ks * 16 + hi * 8) * 2));
    }
  }
  if (!STAGE_X) {
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      x1f[ks] = *reinterpret_cast<const vec8*>(row_address(x1b, st_row, x1_rb, (ks * 16 + hi * 8) * 2));
      x2f[ks] = *reinterpret_cast<const vec8*>(row_address(x2b, st_row, x2_rb, (ks * 16 + hi * 8) * 2));
    }
  } else {
    // The stationary rows come through LDS (dK/dV passes; dQ passes at d = 64, where the 32 KB fit beside
    // two workgroups per CU): whole rows per 8 or 16 consecutive lanes (one 128- or 256-byte request per
    // row) instead of one 16-byte piece of 64 different rows per instruction.  Each wave stages its own
    // 32 rows, so only the wave itself has to wait.  The row numbers (stationary rows, first tile) are
    // waited for first; then the stationary rows, the queries' output rows (dQ passes: into the second
    // pair of tile buffers, which the loop fills only after its first barrier) and the first tile are all
    // asked for together: two memory round trips before the first chunk instead of three or four.
    constexpr int ROWS_PER_LOAD = 64 / PR;
    const int row_in_load = lane / PR, phys_piece = lane % PR;
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the row numbers
    unsigned char* const o_stage = (wave_s < 2 ? lds_y1[1] : lds_y2[1]) + (wave_s & 1) * 32 * D * 2;
#pragma unroll
    for (int j = 0; j < 32 / ROWS_PER_LOAD; ++j) {
      const int r = j * ROWS_PER_LOAD + row_in_load;  // 0..31: a stationary row of this wave
      const int row = __shfl(st_row, r);
      const uint32_t piece = (uint32_t)((phys_piece ^ bwd_swizzle<D>(r)) << 4);
      const int dst = (wave_s * 32 + j * ROWS_PER_LOAD) * D * 2;
      global_to_lds_16(row_address(x1b, row, x1_rb, piece), lds_x1 + dst);
      global_to_lds_16(row_address(x2b, row, x2_rb, piece), lds_x2 + dst);
      if (!KEY_ST) global_to_lds_16(row_address(ob, row, o_rb, piece), o_stage + j * ROWS_PER_LOAD * D * 2);
    }
  }

  if (!KEY_ST) st_lse2 = p.lse[b * p.lse_sb + h0 * p.lse_sh + q_row0 + st_row] * LOG2E;
  load_tile(0);
  fetch_rows(1);

  if (STAGE_X) {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the stationary rows (and the first tile) have landed
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks) {
      const int off = bwd_tile_offset<D>(wave_s * 32 + col, ks * 2 + hi);
      x1f[ks] = lds_read_k<T>(lds_x1, off);
      x2f[ks] = lds_read_k<T>(lds_x2, off);
      if (!KEY_ST) {
        const unsigned char* const o_stage = (wave_s < 2 ? lds_y1[1] : lds_y2[1]) + (wave_s & 1) * 32 * D * 2;
        of[ks] = lds_read_k<T>(o_stage, bwd_tile_offset<D>(col, ks * 2 + hi));
      }
    }
  }
  if (!KEY_ST) {
    // D = sum_c dO * O of the lane's query: the two lanes of a column hold complementary pieces of the row.
    // The dK/dV passes of the call read both statistics from the workspace.
    float part = 0.f;
#pragma unroll
    for (int ks = 0; ks < KSTEPS; ++ks)
#pragma unroll
      for (int e = 0; e < 8; ++e) part = __builtin_fmaf((float)of[ks][e], (float)x2f[ks][e], part);
    const float d_row = ha_sum_xor32(part);
    st_delta = d_row * p.scale;
#pragma unroll
    for (int i = 0; i < 16; ++i) neg_d[i] = -d_row;
    if (hi == 0 && st_valid) p.stats[((int64_t)(b * p.heads + h0) * p.segs + seg) * p.n_q + st_row] = f32x2{st_lse2, -d_row};
  }

  // per-lane LDS offsets of the operand reads
  int off_rows[KSTEPS];  // piece of k-step ks of tile row lane%32, 16-byte read
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) off_rows[ks] = bwd_tile_offset<D>(col, ks * 2 + hi);
  // transposing read: lane s = 4j + w of a 16-lane group addresses streamed row j (+4 for the upper lane
  // half), 8-byte word w of the 16 columns of its group; a second read takes the rows 8 further on
  int off_tr_lo[DB], off_tr_hi[DB];
  {
    const int g = lane >> 4, sl = lane & 15;
    const int key = (g >> 1) * 4 + (sl >> 2);
    const int w = sl & 3;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      off_tr_lo[db] = bwd_tile_offset<D>(key, db * 4 + (g & 1) * 2 + (w >> 1)) + (w & 1) * 8;
      off_tr_hi[db] = bwd_tile_offset<D>(key + 8, db * 4 + (g & 1) * 2 + (w >> 1)) + (w & 1) * 8;
    }
  }

  f32x16 acc1[DB], acc2[DB];  // dQ^T, or dK^T and dV^T: rows = head dim, column = the lane's stationary row
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      acc1[db][i] = 0.f;
      acc2[db][i] = 0.f;
    }

  for (int c = 0; c < nc; ++c) {
    const int buf = c & 1;
    if (KEY_ST && lane < 16) {
      lds_lse[buf][wave_s * 16 + lane] = stat_lse;
      lds_delta[buf][wave_s * 16 + lane] = stat_delta;
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's part of tile c has landed
    __syncthreads();
    if (c + 1 < nc) {
      load_tile(buf ^ 1);
      fetch_rows(c + 2);
    }

    // does this wave take part in the chunk at all (smoothed blocks: the window of a query tile can end
    // between the two 64-key halves of the stationary tile)
    const int cc = c - group_of(c) * nc_head;  // chunk number within its query head
    bool wave_in = true;      // does the wave have any pair in this chunk
    bool needs_mask = false;  // and are some of its pairs masked
    const int y_lo = y_first + cc * YC, y_hi = y_lo + YC - 1;             // streamed rows of the chunk (exact, sampled)
    const int st_lo = tile * ST_ROWS + wave_s * 32, st_hi = st_lo + 31;  // stationary positions of the wave
    if (PASS == HA_BWD_DKV_BLOCK) {
      wave_in = (attending_tile(cc >> 1) >> (30 + (wave_s >> 1))) & 1;
    } else if (PASS == HA_BWD_DQ_EXACT) {
      wave_in = !CAUSAL || y_lo <= st_hi;
      needs_mask = y_hi >= p.n_k || (CAUSAL && y_hi > st_lo);
    } else if (PASS == HA_BWD_DKV_EXACT) {
      wave_in = !CAUSAL || y_hi >= st_lo;
      needs_mask = y_hi >= p.n_q || (CAUSAL && y_lo < st_hi);
    }

    // One chunk of one wave as straight-line code, one copy with the mask and one without: the
    // scheduler is free to mix the soft-max arithmetic of one 32-row half with the MFMAs of the other
    // (forcing a particular interleave with scheduling groups made no difference).
    auto chunk_body = [&](auto masked_tag) {
      constexpr bool MASKED = decltype(masked_tag)::value;
      const unsigned char* const y1 = lds_y1[buf];
      const unsigned char* const y2 = lds_y2[buf];
      f32x16 s[2], dp[2];
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          s[rb][i] = 0.f;
          dp[rb][i] = 0.f;
        }
        if (!KEY_ST) dp[rb] = neg_d;
        if (FOLD_D) {
          // dP' starts from -D of its streamed query (accumulator element 4g + e is row 8g + 4 hi + e of the
          // 32-row block): the MFMAs then leave dP - D, and dS' = P' (dP - D) is one product; its factor
          // `scale` is applied to the sums of dK at the end
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const f32x4 nd = *reinterpret_cast<const f32x4*>(&lds_delta[buf][rb * 32 + g * 8 + hi * 4]);
#pragma unroll
            for (int e = 0; e < 4; ++e) dp[rb][g * 4 + e] = nd[e];
          }
        }
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ++ks) {
          const vec8 a1 = lds_read_k<T>(y1, off_rows[ks] + rb * 32 * D * 2);
          const vec8 a2 = lds_read_k<T>(y2, off_rows[ks] + rb * 32 * D * 2);
          s[rb] = Mfma<T>::run(a1, x1f[ks], s[rb]);
          dp[rb] = Mfma<T>::run(a2, x2f[ks], dp[rb]);
        }
      }

      // P' and dS' of the lane's 32 (streamed row, stationary row) pairs, rounded to the input type.
      // Only chunks that touch the diagonal or the end of the sequence pay for the mask.
      vec8 pb[2][2], dsb[2][2];
      {
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const int r0 = rb * 32 + g * 8 + hi * 4;  // streamed rows r0..r0+3 of the chunk
            f32x4 l4 = {st_lse2, st_lse2, st_lse2, st_lse2}, d4 = {st_delta, st_delta, st_delta, st_delta};
            if (KEY_ST) l4 = *reinterpret_cast<const f32x4*>(&lds_lse[buf][r0]);
            if (KEY_ST && !FOLD_D) d4 = *reinterpret_cast<const f32x4*>(&lds_delta[buf][r0]);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int i = g * 4 + e;
              float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(s[rb][i], p.scale_log2, -l4[e]));
              if (MASKED) {
                bool ok = true;
                if (PASS == HA_BWD_DQ_EXACT) {
                  const int key = cc * YC + r0 + e;
                  ok = key < p.n_k && (!CAUSAL || key <= st_pos);
                } else if (PASS == HA_BWD_DKV_EXACT) {
                  const int query = y_first + cc * YC + r0 + e;
                  ok = query < p.n_q && (!CAUSAL || st_pos <= query);
                }
                pv = ok ? pv : 0.f;
              }
              // d4 holds D * scale: dS = P (dP - D) scale in one FMA and one product; the gathered dK/dV passes
              // hold dP - D in dp already
              const float dsv = (FOLD_D || !KEY_ST) ? pv * dp[rb][i] : pv * __builtin_fmaf(dp[rb][i], p.scale, -d4[e]);
              pb[rb][i >> 3][i & 7] = (T)pv;
              dsb[rb][i >> 3][i & 7] = (T)dsv;
            }
          }
      }

      // the products that contract over the streamed rows
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int kk = 0; kk < 2; ++kk)
#pragma unroll
          for (int db = 0; db < DB; ++db) {
            const int row_off = (rb * 32 + kk * 16) * D * 2;
            const vec8 t1 = bwd_read_tr<T>(y1, off_tr_lo[db] + row_off, off_tr_hi[db] + row_off);
            acc1[db] = Mfma<T>::run(t1, dsb[rb][kk], acc1[db]);
            if (KEY_ST) {
              const vec8 t2 = bwd_read_tr<T>(y2, off_tr_lo[db] + row_off, off_tr_hi[db] + row_off);
              acc2[db] = Mfma<T>::run(t2, pb[rb][kk], acc2[db]);
            }
          }
    };
    // the passes whose pairs are masked one by one: the diagonal and the end of the sequence in exact
    // attention (the sampled keys' pass handles the end of its query range through L)
    constexpr bool CAN_MASK = PASS == HA_BWD_DQ_EXACT || PASS == HA_BWD_DKV_EXACT;
    if (wave_in) {
      if (CAN_MASK && needs_mask)
        chunk_body(std::true_type{});
      else
        chunk_body(std::false_type{});
    }
  }

  if (FOLD_D || !KEY_ST) {
    // dK (dQ) was summed without the factor `scale` of dS
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc1[db][i] *= p.scale;
  }

  // ---- results -------------------------------------------------------------------------------
  // A lane holds 4 consecutive elements of 16 pieces of ONE row.  In the gathered passes, whose rows lie
  // all over the head, each wave turns its 32 x D results around in LDS (its quarter of the first tile
  // buffer pair, free once every wave has left the loop), so that 8 or 16 consecutive lanes write one
  // whole row, 16 bytes each, instead of every lane 8 bytes of its own row per instruction (3.5 %; the
  // exact passes, whose rows are neighbours anyway, lose 1-3 % to the extra barrier and registers).
  constexpr bool TURN_RESULTS = PASS == HA_BWD_DQ_BLOCK || PASS == HA_BWD_DKV_BLOCK;
  if (TURN_RESULTS) {
    constexpr int ROWS_PER_STORE = 64 / PR;
    constexpr int NJ = 32 / ROWS_PER_STORE;
    const int row_in_store = lane / PR, out_piece = lane % PR;
    unsigned char* const base1 =
        KEY_ST ? (unsigned char*)((T*)p.dk + b * p.dk_sb + hk * p.dk_sh + k_row0 * p.dk_sn)
               : (unsigned char*)((T*)p.dq + b * p.dq_sb + h0 * p.dq_sh + q_row0 * p.dq_sn);
    unsigned char* const base2 = (unsigned char*)((T*)p.dv + b * p.dv_sb + hk * p.dv_sh + k_row0 * p.dv_sn);
    const int64_t stride1 = (KEY_ST ? p.dk_sn : p.dq_sn) * 2, stride2 = p.dv_sn * 2;
    // the rows this lane writes (a piece of NJ rows of its wave), and, when the call adds to what is there,
    // their present values: all asked for at once, ahead of the barrier and the turn through LDS (one
    // memory round trip; fetched where each row is stored they were NJ round trips per tensor, one after
    // the other, and a third of the block pass's time)
    int rows_j[NJ];
    bool valid_j[NJ];
    vec8 old1[NJ], old2[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int r = j * ROWS_PER_STORE + row_in_store;
      rows_j[j] = __shfl(st_row, r);  // lanes past the end hold the first row: a valid address
      valid_j[j] = __shfl((int)st_valid, r) != 0;
    }
    if (p.accumulate) {
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        old1[j] = *reinterpret_cast<const vec8*>(base1 + rows_j[j] * stride1 + out_piece * 16);
        if (KEY_ST) old2[j] = *reinterpret_cast<const vec8*>(base2 + rows_j[j] * stride2 + out_piece * 16);
      }
    }
    __syncthreads();
    unsigned char* const turn = lds_y1[0] + wave_s * (32 * D * 2);
    auto store_rows = [&](const f32x16 (&acc)[DB], unsigned char* base, int64_t row_stride_bytes, const vec8 (&old)[NJ]) {
      // [row][D] in the output type, 16-byte pieces XOR-ed with the row number
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          vec4 o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = (T)acc[db][g * 4 + e];
          const int piece = (4 * db + g) ^ (col & (PR - 1));
          *reinterpret_cast<vec4*>(turn + col * (D * 2) + piece * 16 + hi * 8) = o;
        }
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int r = j * ROWS_PER_STORE + row_in_store;
        vec8 o = *reinterpret_cast<const vec8*>(turn + r * (D * 2) + ((out_piece ^ (r & (PR - 1))) << 4));
        if (p.accumulate) {
#pragma unroll
          for (int e = 0; e < 8; ++e) o[e] = (T)((float)o[e] + (float)old[j][e]);
        }
        if (valid_j[j]) *reinterpret_cast<vec8*>(base + rows_j[j] * row_stride_bytes + out_piece * 16) = o;
      }
    };
    store_rows(acc1, base1, stride1, old1);
    if (KEY_ST) store_rows(acc2, base2, stride2, old2);
  }
  if (!TURN_RESULTS && !KEY_ST && st_valid) {
    unsigned char* const dqb = (unsigned char*)((T*)p.dq + b * p.dq_sb + h0 * p.dq_sh + q_row0 * p.dq_sn) + (int64_t)st_row * p.dq_sn * 2;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        vec4* const dst = reinterpret_cast<vec4*>(dqb + (32 * db + 8 * g + 4 * hi) * 2);
        vec4 o;
        if (p.accumulate) {
          const vec4 old = *dst;
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = (T)(acc1[db][g * 4 + e] + (float)old[e]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = (T)acc1[db][g * 4 + e];
        }
        *dst = o;
      }
  } else if (!TURN_RESULTS && (PASS == HA_BWD_DKV_EXACT || PASS == HA_BWD_DKV_BLOCK) && st_valid) {
    // complete sums (of the blocks: every key is in exactly one tile of the sorted order): straight to dk, dv
    unsigned char* const dkb = (unsigned char*)((T*)p.dk + b * p.dk_sb + hk * p.dk_sh + k_row0 * p.dk_sn) + (int64_t)st_row * p.dk_sn * 2;
    unsigned char* const dvb = (unsigned char*)((T*)p.dv + b * p.dv_sb + hk * p.dv_sh + k_row0 * p.dv_sn) + (int64_t)st_row * p.dv_sn * 2;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        vec4* const dst_k = reinterpret_cast<vec4*>(dkb + (32 * db + 8 * g + 4 * hi) * 2);
        vec4* const dst_v = reinterpret_cast<vec4*>(dvb + (32 * db + 8 * g + 4 * hi) * 2);
        vec4 ok_, ov_;
        if (p.accumulate) {
          const vec4 old_k = *dst_k, old_v = *dst_v;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            ok_[e] = (T)(acc1[db][g * 4 + e] + (float)old_k[e]);
            ov_[e] = (T)(acc2[db][g * 4 + e] + (float)old_v[e]);
          }
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            ok_[e] = (T)acc1[db][g * 4 + e];
            ov_[e] = (T)acc2[db][g * 4 + e];
          }
        }
        *dst_k = ok_;
        *dst_v = ov_;
      }
  }
  if (PASS == HA_BWD_DKV_SAMPLED) {
    // Sampled keys: partial sums over one range of queries of one query head, added with atomics to the
    // fp32 row of the key's SLOT in the sample list (batch, kv_heads, sample_size, D).  Each wave turns its
    // 32 x D results around in LDS (its quarter of the tile buffers, free once every wave has left the
    // loop) so that one atomic instruction covers 64 consecutive floats of one row instead of one float of
    // each of 64 rows.
    __syncthreads();
    float* const turn = reinterpret_cast<float*>(wave_s < 2 ? lds_y1[wave_s] : lds_y2[wave_s - 2]);
    const int64_t head_base = ((int64_t)(b * kv_heads + hk) * p.segs + seg) * p.sample_size * D;
#pragma unroll
    for (int which = 0; which < 2; ++which) {
      float* const dst = (which == 0 ? p.dk32 : p.dv32) + head_base;
      // [key][D] fp32, the 16-byte pieces of a row XOR-ed with the key number: conflict-free both ways
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const f32x16& a = which == 0 ? acc1[db] : acc2[db];
          const int piece = (8 * db + 2 * g + hi) ^ (col & 15);
          *reinterpret_cast<f32x4*>(turn + col * D + piece * 4) = f32x4{a[g * 4], a[g * 4 + 1], a[g * 4 + 2], a[g * 4 + 3]};
        }
      for (int r = 0; r < 32; ++r) {
        const int slot = tile * ST_ROWS + wave_s * 32 + r;  // < sample_size: a multiple of 128
#pragma unroll
        for (int part = 0; part < D / 64; ++part) {
          const int dd = part * 64 + lane;
          const float val = turn[r * D + (((dd >> 2) ^ (r & 15)) << 2) + (dd & 3)];
          unsafeAtomicAdd(dst + (int64_t)slot * D + dd, val);
        }
      }
    }
  }
}

__global__ __launch_bounds__(256) void ha_bwd_zero_kernel(f32x4* __restrict__ buf, int64_t n4) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n4) buf[i] = f32x4{0.f, 0.f, 0.f, 0.f};
}

// Sums of the sampled keys (fp32, one row per slot of the sample list) added to the rows of dk, dv, 8
// elements per lane.  A row that is listed several times is handled by its first slot alone, which adds
// the sums of all of them: no two lanes write the same row, whatever the list holds.
template <typename T, int D>
__global__ __launch_bounds__(256) void ha_bwd_add_samples_kernel(const float* __restrict__ sk32, const float* __restrict__ sv32,
                                                                 T* __restrict__ dk, T* __restrict__ dv,
                                                                 const void* __restrict__ sampled_idx, int idx64,
                                                                 int64_t si_sb, int64_t si_sh, int kv_heads, int sample_size,
                                                                 int64_t dk_sb, int64_t dk_sh, int64_t dk_sn, int64_t dv_sb,
                                                                 int64_t dv_sh, int64_t dv_sn, int64_t total_slots,
                                                                 int segs, int64_t seg_stride, int64_t k_seg_off) {
  typedef typename ElemTraits<T>::vec8 vec8;
  constexpr int PR = D / 8;
  const int64_t item = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t gslot = item / PR;
  const int piece = (int)(item % PR);
  if (gslot >= total_slots) return;
  const int64_t bhs = gslot / sample_size;   // (batch, kv head, segment)
  const int slot = (int)(gslot - bhs * sample_size);
  const int64_t bh = bhs / segs, seg = bhs - bh * segs;
  const int64_t b = bh / kv_heads, h = bh - b * kv_heads;
  const int64_t row0 = k_seg_off + seg * seg_stride;
  int row = slot;
  float sum_k[8], sum_v[8];
  const float* const bk = sk32 + (bhs * sample_size) * D + piece * 8;
  const float* const bv = sv32 + (bhs * sample_size) * D + piece * 8;
  auto add_slot = [&](int s2) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      sum_k[e] += bk[(int64_t)s2 * D + e];
      sum_v[e] += bv[(int64_t)s2 * D + e];
    }
  };
#pragma unroll
  for (int e = 0; e < 8; ++e) sum_k[e] = sum_v[e] = 0.f;
  if (sampled_idx) {
    const int64_t list = b * si_sb + h * si_sh;
    row = ha_load_idx(sampled_idx, list + slot, idx64);
    for (int s2 = 0; s2 < slot; ++s2)
      if (ha_load_idx(sampled_idx, list + s2, idx64) == row) return;  // an earlier slot owns this row
    add_slot(slot);
    for (int s2 = slot + 1; s2 < sample_size; ++s2)
      if (ha_load_idx(sampled_idx, list + s2, idx64) == row) add_slot(s2);
  } else {
    add_slot(slot);
  }
  vec8* const dst_k = reinterpret_cast<vec8*>(dk + b * dk_sb + h * dk_sh + (row0 + row) * dk_sn + piece * 8);
  vec8* const dst_v = reinterpret_cast<vec8*>(dv + b * dv_sb + h * dv_sh + (row0 + row) * dv_sn + piece * 8);
  vec8 ok = *dst_k, ov = *dst_v;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    ok[e] = (T)((float)ok[e] + sum_k[e]);
    ov[e] = (T)((float)ov[e] + sum_v[e]);
  }
  *dst_k = ok;
  *dst_v = ov;
}

template <typename T, int D, int PASS, bool CAUSAL>
int launch_pass(const ha_attn_bwd_params& p, int64_t grid, hipStream_t stream, const char* what) {
  if (grid <= 0) return HA_OK;
  if (grid >= (1ll << 31)) return ha_fail(HA_ERR_SHAPE, "%s: grid of %lld workgroups", what, (long long)grid);
  hipLaunchKernelGGL((ha_attn_bwd_kernel<T, D, PASS, CAUSAL>), dim3((unsigned)grid), dim3(WG_THREADS), 0, stream, p);
  return ha_launch_status(what);
}

inline int64_t align256(int64_t v) { return (v + 255) & ~(int64_t)255; }

struct Workspace {
  f32x2* stats;  // per query {L * log2(e), -D}
  float* dk32;  // sums of the sampled keys, (batch, kv_heads, sample_size, d) fp32
  float* dv32;
  int64_t acc_floats;  // per accumulator
  int64_t bytes;
};

Workspace carve(const ha_attn_operands& t, int64_t sample_size, void* base) {
  Workspace w;
  const int64_t delta_bytes = align256(t.batch * t.heads * t.segs * t.n_q * 8);
  w.acc_floats = t.batch * (t.heads / t.kv_group) * t.segs * sample_size * t.d;
  const int64_t acc_bytes = align256(w.acc_floats * 4);
  w.stats = (f32x2*)base;
  w.dk32 = (float*)((char*)base + delta_bytes);
  w.dv32 = (float*)((char*)base + delta_bytes + acc_bytes);
  w.bytes = delta_bytes + 2 * acc_bytes;
  return w;
}

int check_grads(const ha_attn_operands& t, int64_t sample_size, const ha_attn_grads& g, const char* who) {
  HA_REQUIRE(g.dout && g.dq && g.dk && g.dv, HA_ERR_NULL, "%s: null gradient pointer", who);
  HA_REQUIRE((t.d == 64 || t.d == 128) && t.dv == t.d, HA_ERR_UNSUPPORTED,
             "%s: the backward is built for head dims 64 and 128 with a value dim equal to them", who);
  const int64_t strides[] = {g.do_stride_b, g.do_stride_h, g.do_stride_n, g.dq_stride_b, g.dq_stride_h, g.dq_stride_n,
                             g.dk_stride_b, g.dk_stride_h, g.dk_stride_n, g.dv_stride_b, g.dv_stride_h, g.dv_stride_n};
  for (int64_t s : strides) HA_REQUIRE(s % 8 == 0, HA_ERR_SHAPE, "%s: gradient rows must be 16-byte aligned", who);
  HA_REQUIRE(((uintptr_t)g.dout % 16) == 0 && ((uintptr_t)g.dq % 16) == 0 && ((uintptr_t)g.dk % 16) == 0 &&
                 ((uintptr_t)g.dv % 16) == 0,
             HA_ERR_SHAPE, "%s: gradient tensors must be 16-byte aligned", who);
  const int64_t row_strides[] = {g.do_stride_n, g.dq_stride_n, g.dk_stride_n, g.dv_stride_n};
  const int64_t row_counts[] = {t.n_q, t.n_q, t.n_k, t.n_k};
  for (int i = 0; i < 4; ++i) {
    HA_REQUIRE(row_strides[i] > 0 && row_strides[i] * 2 < (1ll << 24), HA_ERR_UNSUPPORTED,
               "%s: gradient row strides must be positive and below 16 MiB", who);
    HA_REQUIRE((row_counts[i] - 1) * row_strides[i] * 2 + t.d * 2 <= (1ll << 32), HA_ERR_UNSUPPORTED,
               "%s: one head of a gradient tensor may span 4 GiB at most", who);
  }
  const Workspace w = carve(t, sample_size, nullptr);
  HA_REQUIRE(g.workspace && g.workspace_bytes >= w.bytes && ((uintptr_t)g.workspace % 256) == 0, HA_ERR_WORKSPACE,
             "%s: workspace of %lld bytes (256-byte aligned) required", who, (long long)w.bytes);
  return HA_OK;
}

void fill_bwd_params(const ha_attn_operands& t, const ha_attn_grads& g, const Workspace& w, ha_attn_bwd_params& p) {
  p.q = t.q; p.k = t.k; p.v = t.v; p.dout = g.dout;
  p.out = t.out; p.lse = t.lse;
  p.o_sb = t.o_stride_b; p.o_sh = t.o_stride_h; p.o_sn = t.o_stride_n;
  p.lse_sb = t.lse_stride_b; p.lse_sh = t.lse_stride_h;
  p.stats = w.stats;
  p.dq = g.dq; p.dk = g.dk; p.dv = g.dv; p.dk32 = w.dk32; p.dv32 = w.dv32;
  p.q_sb = t.q_stride_b; p.q_sh = t.q_stride_h; p.q_sn = t.q_stride_n;
  p.k_sb = t.k_stride_b; p.k_sh = t.k_stride_h; p.k_sn = t.k_stride_n;
  p.v_sb = t.v_stride_b; p.v_sh = t.v_stride_h; p.v_sn = t.v_stride_n;
  p.do_sb = g.do_stride_b; p.do_sh = g.do_stride_h; p.do_sn = g.do_stride_n;
  p.dq_sb = g.dq_stride_b; p.dq_sh = g.dq_stride_h; p.dq_sn = g.dq_stride_n;
  p.dk_sb = g.dk_stride_b; p.dk_sh = g.dk_stride_h; p.dk_sn = g.dk_stride_n;
  p.dv_sb = g.dv_stride_b; p.dv_sh = g.dv_stride_h; p.dv_sn = g.dv_stride_n;
  p.q_idx = p.k_idx = p.sampled_idx = nullptr;
  p.qi_sb = p.qi_sh = p.qi_sn = 0;
  p.ki_sb = p.ki_sh = p.ki_sn = 0;
  p.si_sb = p.si_sh = 0;
  p.batch = (int)t.batch; p.heads = (int)t.heads; p.kv_group = (int)t.kv_group;
  p.segs = (int)t.segs; p.seg_stride = t.seg_stride_rows; p.q_seg_off = t.q_seg_offset; p.k_seg_off = t.k_seg_offset;
  p.n_q = (int)t.n_q; p.n_k = (int)t.n_k;
  p.block_tiles = 1; p.sample_size = 0; p.smooth = 0; p.idx64 = 0;
  p.accumulate = g.accumulate != 0;
  p.q_split = (int)t.n_q;
  p.scale = t.scale;
  p.scale_log2 = t.scale * LOG2E;
}

// the sampled keys' sums onto their rows of dk, dv
template <typename T, int D>
int launch_add_samples(const ha_block_attn_args& a, const ha_attn_grads& g, const Workspace& w, hipStream_t stream) {
  const ha_attn_operands& t = a.t;
  const int64_t kv_heads = t.heads / t.kv_group;
  const int64_t slots = t.batch * kv_heads * t.segs * a.sample_size;
  const int64_t items = slots * (D / 8);
  hipLaunchKernelGGL((ha_bwd_add_samples_kernel<T, D>), dim3((unsigned)((items + 255) / 256)), dim3(256), 0, stream,
                     w.dk32, w.dv32, (T*)g.dk, (T*)g.dv, a.sampled_idx, (int)(a.idx_type == HA_IDX_I64),
                     a.sampled_stride_b, a.sampled_stride_h, (int)kv_heads, (int)a.sample_size, g.dk_stride_b,
                     g.dk_stride_h, g.dk_stride_n, g.dv_stride_b, g.dv_stride_h, g.dv_stride_n, slots, (int)t.segs,
                     t.seg_stride_rows, t.k_seg_offset);
  return ha_launch_status("attention backward: sampled keys");
}

template <typename T, int D>
int run_block_bwd(const ha_block_attn_args& a, const ha_attn_grads& g, hipStream_t stream) {
  const ha_attn_operands& t = a.t;
  const Workspace w = carve(t, a.sample_size, g.workspace);
  int st;
  ha_attn_bwd_params p;
  fill_bwd_params(t, g, w, p);
  p.q_idx = a.q_idx; p.k_idx = a.k_idx; p.sampled_idx = a.sampled_idx;
  p.qi_sb = a.q_idx_stride_b; p.qi_sh = a.q_idx_stride_h; p.qi_sn = a.q_idx_stride_n;
  p.ki_sb = a.k_idx_stride_b; p.ki_sh = a.k_idx_stride_h; p.ki_sn = a.k_idx_stride_n;
  p.si_sb = a.sampled_stride_b; p.si_sh = a.sampled_stride_h;
  p.block_tiles = (int)((a.block_size + 127) / 128);
  p.sample_size = (int)a.sample_size;
  p.smooth = a.smooth_block != 0;
  p.idx64 = a.idx_type == HA_IDX_I64;
  const int64_t bh = t.batch * t.heads * t.segs, bhk = t.batch * (t.heads / t.kv_group) * t.segs;
  st = launch_pass<T, D, HA_BWD_DQ_BLOCK, false>(p, bh * (t.n_q / ST_ROWS), stream, "ha_block_attn_bwd: dq");
  if (st != HA_OK) return st;
  st = launch_pass<T, D, HA_BWD_DKV_BLOCK, false>(p, bhk * (t.n_k / ST_ROWS), stream, "ha_block_attn_bwd: dk, dv of the blocks");
  if (st != HA_OK) return st;
  if (a.sample_size > 0) {
    // the two arrays of sums lie one behind the other in the workspace (each a multiple of 256 bytes): one fill
    const int64_t n4 = (int64_t)(((char*)w.dv32 - (char*)w.dk32) + align256(w.acc_floats * 4)) / 16;
    hipLaunchKernelGGL(ha_bwd_zero_kernel, dim3((unsigned)((n4 + 255) / 256)), dim3(256), 0, stream, (f32x4*)w.dk32, n4);
    st = ha_launch_status("attention backward: clear");
    if (st != HA_OK) return st;
    // every query attends every sampled key: the queries are cut into ranges, as long as possible (each
    // range ends in one atomic add per element of the sampled rows) while two workgroups per CU remain
    int64_t q_split = 8192;
    while (q_split > 512 && bh * (a.sample_size / ST_ROWS) * ((t.n_q + q_split - 1) / q_split) < 512) q_split /= 2;
    p.q_split = (int)q_split;
    const int64_t splits = (t.n_q + q_split - 1) / q_split;
    st = launch_pass<T, D, HA_BWD_DKV_SAMPLED, false>(p, bh * (a.sample_size / ST_ROWS) * splits, stream,
                                                      "ha_block_attn_bwd: dk, dv of the sampled keys");
    if (st != HA_OK) return st;
    return launch_add_samples<T, D>(a, g, w, stream);
  }
  return HA_OK;
}

template <typename T, int D>
int run_flash_bwd(const ha_attn_operands& t, bool causal, const ha_attn_grads& g, hipStream_t stream) {
  const Workspace w = carve(t, 0, g.workspace);
  int st;
  ha_attn_bwd_params p;
  fill_bwd_params(t, g, w, p);
  const int64_t bh = t.batch * t.heads * t.segs, bhk = t.batch * (t.heads / t.kv_group) * t.segs;
  const int64_t q_tiles = (t.n_q + ST_ROWS - 1) / ST_ROWS, k_tiles = (t.n_k + ST_ROWS - 1) / ST_ROWS;
  if (causal) {
    st = launch_pass<T, D, HA_BWD_DQ_EXACT, true>(p, bh * q_tiles, stream, "ha_flash_attn_bwd: dq");
    if (st != HA_OK) return st;
    st = launch_pass<T, D, HA_BWD_DKV_EXACT, true>(p, bhk * k_tiles, stream, "ha_flash_attn_bwd: dk, dv");
  } else {
    st = launch_pass<T, D, HA_BWD_DQ_EXACT, false>(p, bh * q_tiles, stream, "ha_flash_attn_bwd: dq");
    if (st != HA_OK) return st;
    st = launch_pass<T, D, HA_BWD_DKV_EXACT, false>(p, bhk * k_tiles, stream, "ha_flash_attn_bwd: dk, dv");
  }
  return st;
}

}  // namespace

extern "C" int64_t ha_attn_bwd_workspace_bytes(const ha_attn_operands* t, int64_t sample_size) {
  if (!t || t->batch <= 0 || t->heads <= 0 || t->n_q <= 0 || t->n_k <= 0 || t->d <= 0 || t->kv_group <= 0 ||
      t->heads % t->kv_group != 0 || sample_size < 0 || t->segs < 1)
    return ha_fail(HA_ERR_SHAPE, "ha_attn_bwd_workspace_bytes: sizes must be positive, kv_group dividing heads, segs >= 1");
  return carve(*t, sample_size, nullptr).bytes;
}

extern "C" int ha_block_attn_bwd(const ha_block_attn_args* args, const ha_attn_grads* grads, void* stream) {
  HA_REQUIRE(args && grads, HA_ERR_NULL, "ha_block_attn_bwd: null argument");
  const ha_block_attn_args& a = *args;
  int st = ha_check_block_attn_args(a, "ha_block_attn_bwd");
  if (st != HA_OK) return st;
  st = check_grads(a.t, a.sample_size, *grads, "ha_block_attn_bwd");
  if (st != HA_OK) return st;
  HA_REQUIRE(!a.accumulate, HA_ERR_UNSUPPORTED, "ha_block_attn_bwd: no backward of the fused merge (accumulate)");
  HA_REQUIRE(a.sample_bias == 0.f && !a.mask_sampled_in_block, HA_ERR_UNSUPPORTED,
             "ha_block_attn_bwd: no backward of the residual estimator (sample_bias, mask_sampled_in_block)");
  HA_REQUIRE(!a.smooth_block || a.block_size <= 128 * (MAX_SMOOTH_TILES - 1), HA_ERR_UNSUPPORTED,
             "ha_block_attn_bwd: smoothed blocks longer than %d rows are not built", 128 * (MAX_SMOOTH_TILES - 1));
  hipStream_t s = (hipStream_t)stream;
  if (a.t.dtype == HA_F16) return a.t.d == 64 ? run_block_bwd<f16_t, 64>(a, *grads, s) : run_block_bwd<f16_t, 128>(a, *grads, s);
  return a.t.d == 64 ? run_block_bwd<bf16_t, 64>(a, *grads, s) : run_block_bwd<bf16_t, 128>(a, *grads, s);
}

extern "C" int ha_flash_attn_bwd(const ha_attn_operands* t, int causal, const ha_attn_grads* grads, void* stream) {
  HA_REQUIRE(t && grads, HA_ERR_NULL, "ha_flash_attn_bwd: null argument");
  int st = ha_check_operands(*t, "ha_flash_attn_bwd");
  if (st != HA_OK) return st;
  st = check_grads(*t, 0, *grads, "ha_flash_attn_bwd");
  if (st != HA_OK) return st;
  hipStream_t s = (hipStream_t)stream;
  if (t->dtype == HA_F16)
    return t->d == 64 ? run_flash_bwd<f16_t, 64>(*t, causal != 0, *grads, s) : run_flash_bwd<f16_t, 128>(*t, causal != 0, *grads, s);
  return t->d == 64 ? run_flash_bwd<bf16_t, 64>(*t, causal != 0, *grads, s) : run_flash_bwd<bf16_t, 128>(*t, causal != 0, *grads, s);
}
