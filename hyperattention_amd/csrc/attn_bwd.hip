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
  // Exact causal attention: a workgroup takes the pair of stationary tiles (s, T-1-s), the one that streams more
  // rows first (the last query tile sees every key, the first key tile is seen by every query), so that every
  // workgroup of a launch streams the same number of rows.  The hardware hands out workgroups in order, and a
  // slot freed by a short one stays empty until the ones queued before it are placed.
  constexpr bool PAIRED = CAUSAL && (PASS == HA_BWD_DQ_EXACT || PASS == HA_BWD_DKV_EXACT);
  const int wg_per_seq = PAIRED ? (st_tiles + 1) / 2 : st_tiles;
  int rest = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int slot = rest % wg_per_seq;
  rest /= wg_per_seq;
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
  const int64_t o_row0 = p.o_seg_off + (int64_t)seg * p.o_seg_stride;  // in the forward's out and lse

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

  if constexpr (!PAIRED) {
    const int tile = slot;
#include "attn_bwd_tile.inc"
  } else {
    const int t_long = PASS == HA_BWD_DQ_EXACT ? st_tiles - 1 - slot : slot;
    const int t_short = st_tiles - 1 - t_long;
    {
      const int tile = t_long;
#include "attn_bwd_tile.inc"
    }
    if (t_short != t_long) {  // an odd number of tiles: the middle one has no partner
      // the first tile's last reads of the staging areas and the streamed tiles are behind every wave
      __syncthreads();
      const int tile = t_short;
#include "attn_bwd_tile.inc"
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
  p.o_seg_stride = t.o_seg_stride_rows > 0 ? t.o_seg_stride_rows : t.seg_stride_rows;
  p.o_seg_off = t.o_seg_stride_rows > 0 ? t.o_seg_offset : t.q_seg_offset;
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
    // one workgroup per pair of stationary tiles
    st = launch_pass<T, D, HA_BWD_DQ_EXACT, true>(p, bh * ((q_tiles + 1) / 2), stream, "ha_flash_attn_bwd: dq");
    if (st != HA_OK) return st;
    st = launch_pass<T, D, HA_BWD_DKV_EXACT, true>(p, bhk * ((k_tiles + 1) / 2), stream, "ha_flash_attn_bwd: dk, dv");
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
