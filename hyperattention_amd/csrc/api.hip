// C entry points for the attention operators and the whole-forward orchestration.
// Argument checks mirror the reference's assertions (src/hyper_attn_triton.py:678-695, :911,
// src/flash_attn_triton.py:797-804, hyper_attention.py:45); nothing is launched when a check fails.
#include "ha_common.h"
#include "attn_fwd.h"
#include "bucket_sort.h"

#include <math.h>
#include <string.h>
#include <algorithm>

char* ha_error_buffer() {
  static thread_local char buf[512] = {0};
  return buf;
}

extern "C" int ha_abi_version(void) { return HA_ABI_VERSION; }
extern "C" const char* ha_last_error(void) { return ha_error_buffer(); }

namespace {

constexpr float LOG2E_F = 1.4426950408889634f;

}  // namespace

int ha_check_operands(const ha_attn_operands& t, const char* who) {
  HA_REQUIRE(t.q && t.k && t.v && t.out && t.lse, HA_ERR_NULL, "%s: null tensor pointer", who);
  HA_REQUIRE(t.dtype == HA_F16 || t.dtype == HA_BF16, HA_ERR_DTYPE, "%s: Only support fp16 and bf16", who);
  HA_REQUIRE(t.batch > 0 && t.heads > 0 && t.n_q > 0 && t.n_k > 0, HA_ERR_SHAPE, "%s: sizes must be positive", who);
  // the kernels address a row as a per-head base plus a 32-bit byte offset computed with a 24-bit multiply
  HA_REQUIRE(t.n_q < (1ll << 24) && t.n_k < (1ll << 24), HA_ERR_SHAPE, "%s: sequence too long (2^24 rows at most)", who);
  HA_REQUIRE(t.d <= 128 && t.dv <= 128, HA_ERR_HEADDIM, "%s: FlashAttention only support head dimensions up to 128", who);
  HA_REQUIRE(t.d >= 8 && t.dv >= 8 && t.d % 8 == 0 && t.dv % 8 == 0, HA_ERR_UNSUPPORTED,
             "%s: head dims must be multiples of 8 (got %lld and %lld)", who, (long long)t.d, (long long)t.dv);
  HA_REQUIRE(t.segs >= 1 && t.kv_group >= 1 && t.heads % t.kv_group == 0, HA_ERR_SHAPE,
             "%s: segs >= 1 and kv_group dividing heads required", who);
  HA_REQUIRE(t.scale > 0.f && isfinite(t.scale), HA_ERR_SHAPE, "%s: softmax scale must be positive and finite", who);
  const int64_t strides[] = {t.q_stride_b, t.q_stride_h, t.q_stride_n, t.k_stride_b, t.k_stride_h, t.k_stride_n,
                             t.v_stride_b, t.v_stride_h, t.v_stride_n, t.o_stride_b, t.o_stride_h, t.o_stride_n};
  for (int64_t s : strides) HA_REQUIRE(s % 8 == 0, HA_ERR_SHAPE, "%s: rows must be 16-byte aligned", who);
  HA_REQUIRE(((uintptr_t)t.q % 16) == 0 && ((uintptr_t)t.k % 16) == 0 && ((uintptr_t)t.v % 16) == 0 &&
                 ((uintptr_t)t.out % 16) == 0,
             HA_ERR_SHAPE, "%s: tensors must be 16-byte aligned", who);
  const int64_t row_strides[] = {t.q_stride_n, t.k_stride_n, t.v_stride_n, t.o_stride_n};
  const int64_t row_counts[] = {t.n_q, t.n_k, t.n_k, t.n_q};
  for (int i = 0; i < 4; ++i) {
    HA_REQUIRE(row_strides[i] > 0 && row_strides[i] * 2 < (1ll << 24), HA_ERR_UNSUPPORTED,
               "%s: row strides must be positive and below 16 MiB", who);
    HA_REQUIRE((row_counts[i] - 1) * row_strides[i] * 2 + 128 * 2 <= (1ll << 32), HA_ERR_UNSUPPORTED,
               "%s: one head of a tensor may span 4 GiB at most", who);
  }
  return HA_OK;
}

int ha_check_block_attn_args(const ha_block_attn_args& a, const char* who) {
  int st = ha_check_operands(a.t, who);
  if (st != HA_OK) return st;
  HA_REQUIRE(a.q_idx && a.k_idx, HA_ERR_NULL, "%s: null index pointer", who);
  HA_REQUIRE(a.idx_type == HA_IDX_I32 || a.idx_type == HA_IDX_I64, HA_ERR_DTYPE, "%s: bad idx_type", who);
  HA_REQUIRE(a.t.n_k % 128 == 0, HA_ERR_SHAPE, "%s: keys sequence length must be divisible by 128", who);
  HA_REQUIRE(a.t.n_q % 128 == 0, HA_ERR_SHAPE, "%s: query sequence length must be divisible by 128", who);
  HA_REQUIRE(a.sample_size >= 0 && a.sample_size % 128 == 0, HA_ERR_SHAPE,
             "%s: sample_size must be a non-negative multiple of 128", who);
  HA_REQUIRE(a.block_size > 0, HA_ERR_SHAPE, "%s: block_size must be positive", who);
  HA_REQUIRE(a.sampled_idx || a.sample_size <= a.t.n_k, HA_ERR_SHAPE,
             "%s: default sampled rows 0..sample_size-1 exceed the key length", who);
  {
    const int64_t esz = a.idx_type == HA_IDX_I64 ? 8 : 4;
    HA_REQUIRE(a.q_idx_stride_n > 0 && a.k_idx_stride_n > 0 && a.q_idx_stride_n * esz < (1ll << 24) &&
                   a.k_idx_stride_n * esz < (1ll << 24) && (a.t.n_q - 1) * a.q_idx_stride_n * esz < (1ll << 32) &&
                   (a.t.n_k - 1) * a.k_idx_stride_n * esz < (1ll << 32),
               HA_ERR_UNSUPPORTED, "%s: index strides must be positive, below 16 MiB, and span 4 GiB at most", who);
  }
  return HA_OK;
}

namespace {

void fill_params(const ha_attn_operands& t, ha_attn_kernel_params& p) {
  p.q = t.q; p.k = t.k; p.v = t.v; p.out = t.out; p.lse = t.lse;
  p.q_idx = nullptr; p.k_idx = nullptr; p.sampled_idx = nullptr;
  p.q_sb = t.q_stride_b; p.q_sh = t.q_stride_h; p.q_sn = t.q_stride_n;
  p.k_sb = t.k_stride_b; p.k_sh = t.k_stride_h; p.k_sn = t.k_stride_n;
  p.v_sb = t.v_stride_b; p.v_sh = t.v_stride_h; p.v_sn = t.v_stride_n;
  p.o_sb = t.o_stride_b; p.o_sh = t.o_stride_h; p.o_sn = t.o_stride_n;
  p.lse_sb = t.lse_stride_b; p.lse_sh = t.lse_stride_h;
  p.qi_sb = p.qi_sh = p.qi_sn = 0;
  p.ki_sb = p.ki_sh = p.ki_sn = 0;
  p.si_sb = p.si_sh = 0;
  p.seg_stride = t.seg_stride_rows; p.q_seg_off = t.q_seg_offset; p.k_seg_off = t.k_seg_offset;
  p.o_seg_stride = t.o_seg_stride_rows > 0 ? t.o_seg_stride_rows : t.seg_stride_rows;
  p.o_seg_off = t.o_seg_stride_rows > 0 ? t.o_seg_offset : t.q_seg_offset;
  p.batch = (int)t.batch; p.heads = (int)t.heads; p.segs = (int)t.segs; p.kv_group = (int)t.kv_group;
  p.n_q = (int)t.n_q; p.n_k = (int)t.n_k;
  p.block_tiles = 1; p.sample_chunks = 0; p.smooth = 0; p.accumulate = 0; p.idx64 = 0;
  p.sampled_pos = nullptr; p.sample_bias_raw = 0.f;
  p.n_q_last = (int)t.n_q;
  p.tiles_per_wg = 1;
  p.rag_levels = -1; p.rag_split = 0; p.rag_n = 0;
  for (int& c : p.rag_half) c = 0;
  p.scale_log2 = t.scale * LOG2E_F;
}

// n_q_last: queries of the last segment of every head that exist (see ha_attn_kernel_params), or -1
int block_attn(const ha_block_attn_args& a, hipStream_t stream, int64_t n_q_last = -1) {
  int st = ha_check_block_attn_args(a, "ha_block_attn_fwd");
  if (st != HA_OK) return st;
  ha_attn_kernel_params p;
  fill_params(a.t, p);
  p.q_idx = a.q_idx; p.k_idx = a.k_idx; p.sampled_idx = a.sampled_idx;
  p.qi_sb = a.q_idx_stride_b; p.qi_sh = a.q_idx_stride_h; p.qi_sn = a.q_idx_stride_n;
  p.ki_sb = a.k_idx_stride_b; p.ki_sh = a.k_idx_stride_h; p.ki_sn = a.k_idx_stride_n;
  p.si_sb = a.sampled_stride_b; p.si_sh = a.sampled_stride_h;
  p.block_tiles = (int)((a.block_size + 127) / 128);
  p.sample_chunks = (int)(a.sample_size / 64);
  p.smooth = a.smooth_block != 0;
  p.accumulate = a.accumulate != 0;
  p.idx64 = a.idx_type == HA_IDX_I64;
  if (n_q_last >= 0) p.n_q_last = (int)n_q_last;
  const bool reweight = a.sample_bias != 0.f || a.mask_sampled_in_block != 0;
  if (reweight) {
    HA_REQUIRE(isfinite(a.sample_bias), HA_ERR_SHAPE, "ha_block_attn_fwd: sample_bias must be finite");
    HA_REQUIRE(!a.mask_sampled_in_block || a.sampled_pos, HA_ERR_NULL,
               "ha_block_attn_fwd: mask_sampled_in_block needs sampled_pos");
    HA_REQUIRE(a.t.d == a.t.dv && (a.t.d == 64 || a.t.d == 128), HA_ERR_UNSUPPORTED,
               "ha_block_attn_fwd: the residual estimator is built for d == dv in {64, 128}");
    p.sampled_pos = a.mask_sampled_in_block ? a.sampled_pos : nullptr;
    p.sample_bias_raw = a.sample_bias / a.t.scale;
  }
  return ha_attn_launch(p, (int)a.t.d, (int)a.t.dv, a.t.dtype, true, false, reweight, stream);
}

// Ragged segments of an exact launch inside a causal recursion with odd lengths (see ha_attn_kernel_params)
struct Ragged {
  int levels, split, n;
  int half[HA_MAX_RAGGED_LEVELS + 1];
};

int flash_attn(const ha_attn_operands& t, int causal, int accumulate, hipStream_t stream, const Ragged* rag = nullptr) {
  int st = ha_check_operands(t, "ha_flash_attn_fwd");
  if (st != HA_OK) return st;
  ha_attn_kernel_params p;
  fill_params(t, p);
  p.accumulate = accumulate != 0;
  if (rag) {
    p.rag_levels = rag->levels; p.rag_split = rag->split; p.rag_n = rag->n;
    for (int i = 0; i <= HA_MAX_RAGGED_LEVELS; ++i) p.rag_half[i] = rag->half[i];
  }
  return ha_attn_launch(p, (int)t.d, (int)t.dv, t.dtype, false, causal != 0, false, stream);
}

inline int64_t align256(int64_t v) { return (v + 255) & ~(int64_t)255; }

// Static shape of the causal divide-and-conquer (hyper_attention.py:51-96).  A virtual head of odd length
// gets a zero row appended before it is cut in two (:61-64), so lengths are counted with those rows: len[j]
// is the length of a level-j virtual head as the recursion sees it, half[j] = ceil(len[j] / 2) the length of
// its two halves.  Appended rows sit at the end of their virtual head, and so of every last descendant.
struct Plan {
  int levels;            // number of halvings
  int64_t len[48];       // len[levels] = leaf
  int64_t half[48];
  bool level_hyper[48];  // off-diagonal of level j uses the hashed kernel (else exact, hyper_attention.py:109)
  bool any_hyper;
  bool ragged;           // an odd length somewhere
  int64_t n_hashed;      // rows per head as the hashed levels see them: n, plus the appended row of an odd n
  int64_t granule;       // length of the shortest hashed half (n_hashed is a multiple of it)
};

int make_plan(const ha_forward_args& a, Plan& pl) {
  pl.levels = 0;
  pl.any_hyper = false;
  pl.ragged = false;
  pl.len[0] = a.n;
  pl.n_hashed = a.n;
  pl.granule = a.n;
  if (!a.causal) {
    pl.level_hyper[0] = !(a.min_seq_len > a.n);  // hyper_attention.py:109
    pl.any_hyper = pl.level_hyper[0];
    if (pl.any_hyper) {
      HA_REQUIRE(a.n % 128 == 0, HA_ERR_SHAPE, "ha_forward: keys sequence length must be divisible by 128");
      HA_REQUIRE(a.sampled_idx || a.sample_size <= a.n, HA_ERR_SHAPE,
                 "ha_forward: default sampled rows 0..sample_size-1 exceed the key length");
    }
    return HA_OK;
  }
  // Only n itself can be odd: a level whose halves are hashed has halves of a multiple of 128 rows, and a
  // level whose halves are shorter than min_seq_len is the last one.
  while (pl.len[pl.levels] > a.min_seq_len) {  // hyper_attention.py:52
    const int j = pl.levels;
    const int64_t cur = pl.len[j];
    pl.ragged = pl.ragged || (cur & 1);
    const int64_t half = (cur + 1) / 2;
    pl.half[j] = half;
    pl.level_hyper[j] = !(a.min_seq_len > half);
    if (pl.level_hyper[j]) {
      HA_REQUIRE(half % 128 == 0, HA_ERR_SHAPE, "ha_forward: keys sequence length must be divisible by 128");
      HA_REQUIRE(a.sampled_idx || a.sample_size <= half, HA_ERR_SHAPE,
                 "ha_forward: default sampled rows 0..sample_size-1 exceed the key length %lld of a level",
                 (long long)half);
      pl.any_hyper = true;
      pl.granule = half;
    }
    pl.len[++pl.levels] = half;
    HA_REQUIRE(pl.levels < HA_MAX_RAGGED_LEVELS, HA_ERR_SHAPE, "ha_forward: recursion too deep");
  }
  // a hashed half is a multiple of 128, so every hashed level but the first has an even length: the hashed
  // levels see the sequence with at most one appended row, the one of an odd n
  if (pl.any_hyper) pl.n_hashed = a.n + (a.n & 1);
  return HA_OK;
}

struct Workspace {
  bool units;                          // one ranking for all levels (byte-sized ids), else a sort per level
  ha_unit_grid grid;
  int64_t buckets_q, buckets_k;        // byte offsets; one byte per id with `units`, else int32
  int64_t sorted_q, sorted_k;          // with `units`: per-unit orders
  int64_t unit_hist_q, unit_hist_k;    // with `units`: per-unit bucket counts
  int64_t qidx[48], kidx[48];          // per hyper level (index 0 for the non-causal case)
  int64_t hist_q[48], hist_k[48];      // without `units`: per-level chunk histograms
  int64_t tmp_q[48][2], tmp_k[48][2];  // without `units`, more than 256 buckets: orders between the two passes
  int64_t total;
};

// A placement workgroup adds up the bucket counts of all units of its segment and moves one unit's rows: the
// longest hashed segment may span this many units before the per-level sort is the better choice.
inline int64_t max_units_per_segment(int unit) { return std::max<int64_t>(64, unit / 4); }

void layout_workspace(const ha_forward_args& a, const Plan& pl, Workspace& w) {
  int64_t off = 0;
  memset(&w, 0, sizeof(w));
  const int nlev = a.causal ? pl.levels : 1;
  const int64_t nh = pl.n_hashed;  // rows per head as the hashed levels see them
  if (pl.any_hyper) {
    ha_unit_grid& g = w.grid;
    g.n = nh;
    g.granule = pl.granule;
    g.units_per_granule = (int)((g.granule + HA_SORT_CHUNK - 1) / HA_SORT_CHUNK);
    g.unit = (int)std::min<int64_t>(g.granule, HA_SORT_CHUNK);
    g.units_per_seq = (int)(nh / g.granule) * g.units_per_granule;
    int64_t longest = 0;
    for (int j = 0; j < nlev; ++j)
      if (pl.level_hyper[j]) longest = std::max<int64_t>(longest, a.causal ? pl.half[j] : a.n);
    w.units = a.lsh_num_projs <= 8 && longest / g.granule * g.units_per_granule <= max_units_per_segment(g.unit) &&
              nh % g.granule == 0;
    const int64_t id_bytes = w.units ? 1 : 4;
    w.buckets_q = off; off += align256(a.batch * a.heads * nh * id_bytes);
    w.buckets_k = off; off += align256(a.batch * a.kv_heads * nh * id_bytes);
    if (w.units) {
      w.sorted_q = off; off += align256(a.batch * a.heads * nh * 4);
      w.sorted_k = off; off += align256(a.batch * a.kv_heads * nh * 4);
      w.unit_hist_q = off; off += align256(a.batch * a.heads * g.units_per_seq * 256 * 4);
      w.unit_hist_k = off; off += align256(a.batch * a.kv_heads * g.units_per_seq * 256 * 4);
    }
  }
  for (int j = 0; j < nlev; ++j) {
    if (!pl.level_hyper[j]) continue;
    const int64_t seg_len = a.causal ? pl.half[j] : a.n;
    const int64_t segs = a.causal ? (1ll << j) : 1;
    const int64_t chunks = (seg_len + HA_SORT_CHUNK - 1) / HA_SORT_CHUNK;
    w.qidx[j] = off; off += align256(a.batch * a.heads * segs * seg_len * 4);
    w.kidx[j] = off; off += align256(a.batch * a.kv_heads * segs * seg_len * 4);
    if (w.units) continue;
    w.hist_q[j] = off; off += align256(a.batch * a.heads * segs * chunks * 256 * 4);
    w.hist_k[j] = off; off += align256(a.batch * a.kv_heads * segs * chunks * 256 * 4);
    if (a.lsh_num_projs > 8)
      for (int t = 0; t < 2; ++t) {
        w.tmp_q[j][t] = off; off += align256(a.batch * a.heads * segs * seg_len * 4);
        w.tmp_k[j][t] = off; off += align256(a.batch * a.kv_heads * segs * seg_len * 4);
      }
  }
  w.total = off > 0 ? off : 256;
}

int check_forward(const ha_forward_args& a) {
  HA_REQUIRE(a.q && a.k && a.v && a.out && a.lse, HA_ERR_NULL, "ha_forward: null tensor pointer");
  HA_REQUIRE(a.dtype == HA_F16 || a.dtype == HA_BF16, HA_ERR_DTYPE, "ha_forward: Only support fp16 and bf16");
  HA_REQUIRE(a.batch > 0 && a.heads > 0 && a.kv_heads > 0 && a.n > 0, HA_ERR_SHAPE, "ha_forward: sizes must be positive");
  HA_REQUIRE(a.heads % a.kv_heads == 0, HA_ERR_SHAPE, "ha_forward: kv_heads must divide heads");
  HA_REQUIRE(a.n < (1ll << 30), HA_ERR_SHAPE, "ha_forward: sequence too long");
  HA_REQUIRE(a.d <= 128 && a.dv <= 128, HA_ERR_HEADDIM, "ha_forward: FlashAttention only support head dimensions up to 128");
  HA_REQUIRE(a.d >= 8 && a.dv >= 8 && a.d % 8 == 0 && a.dv % 8 == 0, HA_ERR_UNSUPPORTED,
             "ha_forward: head dims must be multiples of 8 (got %lld and %lld)", (long long)a.d, (long long)a.dv);
  HA_REQUIRE(a.scale > 0.f && isfinite(a.scale), HA_ERR_SHAPE, "ha_forward: softmax scale must be positive and finite");
  HA_REQUIRE(a.block_size > 0 && a.sample_size >= 0 && a.sample_size % 128 == 0 && a.min_seq_len >= 0, HA_ERR_SHAPE,
             "ha_forward: block_size > 0 and sample_size a non-negative multiple of 128 required");
  return HA_OK;
}

// (batch, heads, n, d) operands of the whole forward pass: contiguous unless strides are given
void forward_operands(const ha_forward_args& a, ha_attn_operands& t) {
  t = ha_attn_operands{};  // segments as the callers set them; out and lse follow q (o_seg_stride_rows = 0)
  t.q = a.q; t.k = a.k; t.v = a.v; t.out = a.out; t.lse = a.lse;
  t.batch = a.batch; t.heads = a.heads; t.d = a.d; t.dv = a.dv;
  t.q_stride_b = a.heads * a.n * a.d; t.q_stride_h = a.n * a.d; t.q_stride_n = a.d;
  t.k_stride_b = a.kv_heads * a.n * a.d; t.k_stride_h = a.n * a.d; t.k_stride_n = a.d;
  t.v_stride_b = a.kv_heads * a.n * a.dv; t.v_stride_h = a.n * a.dv; t.v_stride_n = a.dv;
  t.o_stride_b = a.heads * a.n * a.dv; t.o_stride_h = a.n * a.dv; t.o_stride_n = a.dv;
  if (a.q_stride_b || a.q_stride_h || a.q_stride_n) {
    t.q_stride_b = a.q_stride_b; t.q_stride_h = a.q_stride_h; t.q_stride_n = a.q_stride_n;
  }
  if (a.k_stride_b || a.k_stride_h || a.k_stride_n) {
    t.k_stride_b = a.k_stride_b; t.k_stride_h = a.k_stride_h; t.k_stride_n = a.k_stride_n;
  }
  if (a.v_stride_b || a.v_stride_h || a.v_stride_n) {
    t.v_stride_b = a.v_stride_b; t.v_stride_h = a.v_stride_h; t.v_stride_n = a.v_stride_n;
  }
  t.lse_stride_b = a.heads * a.n; t.lse_stride_h = a.n;
  t.kv_group = a.heads / a.kv_heads;
  t.scale = a.scale;
  t.dtype = a.dtype;
}

// Row alignment of the tensors a forward pass reads and writes, checked before the first launch (the hash
// and the attention kernels move rows in 16-byte pieces).
int check_forward_layout(const ha_attn_operands& t, bool with_values, const char* who) {
  HA_REQUIRE(((uintptr_t)t.q % 16) == 0 && ((uintptr_t)t.k % 16) == 0, HA_ERR_SHAPE, "%s: tensors must be 16-byte aligned", who);
  const int64_t qk[] = {t.q_stride_b, t.q_stride_h, t.q_stride_n, t.k_stride_b, t.k_stride_h, t.k_stride_n};
  for (int64_t s : qk) HA_REQUIRE(s % 8 == 0, HA_ERR_SHAPE, "%s: rows must be 16-byte aligned", who);
  if (with_values) {
    HA_REQUIRE(((uintptr_t)t.v % 16) == 0 && ((uintptr_t)t.out % 16) == 0, HA_ERR_SHAPE, "%s: tensors must be 16-byte aligned", who);
    const int64_t vo[] = {t.v_stride_b, t.v_stride_h, t.v_stride_n};
    for (int64_t s : vo) HA_REQUIRE(s % 8 == 0, HA_ERR_SHAPE, "%s: rows must be 16-byte aligned", who);
  }
  return HA_OK;
}

// Bucket ids of q and k, then the stable bucket order of the query and key segment of every hashed level
// (hyper_attention.py:112-117 at every level of the recursion), as int32 rows local to the segment.
int hash_and_sort(const ha_forward_args& a, const Plan& pl, const Workspace& w, const ha_attn_operands& t,
                  hipStream_t stream) {
  unsigned char* ws = (unsigned char*)a.workspace;
  const int nlev = a.causal ? pl.levels : 1;
  int st;
  if (w.units) {
    const int64_t qs[3] = {t.q_stride_b, t.q_stride_h, t.q_stride_n}, ks[3] = {t.k_stride_b, t.k_stride_h, t.k_stride_n};
    st = ha_hash_pair_u8(a.q, a.k, a.proj, ws + w.buckets_q, ws + w.buckets_k, a.batch, a.heads, a.kv_heads, pl.n_hashed,
                         a.n, a.d, a.lsh_num_projs, qs, ks, a.dtype, stream);
    if (st != HA_OK) return st;
    const uint8_t* ids[2] = {ws + w.buckets_q, ws + w.buckets_k};
    uint32_t* sorted[2] = {(uint32_t*)(ws + w.sorted_q), (uint32_t*)(ws + w.sorted_k)};
    uint32_t* hist[2] = {(uint32_t*)(ws + w.unit_hist_q), (uint32_t*)(ws + w.unit_hist_k)};
    const int64_t seqs[2] = {a.batch * a.heads, a.batch * a.kv_heads};
    st = ha_rank_units(ids, sorted, hist, seqs, w.grid, stream);
    if (st != HA_OK) return st;
    ha_place_jobs jobs;
    jobs.num_jobs = 0;
    jobs.grid = w.grid;
    int64_t blocks = 0;
    for (int j = 0; j < nlev; ++j) {
      if (!pl.level_hyper[j]) continue;
      const int64_t seg_len = a.causal ? pl.half[j] : a.n;
      const int64_t segs = a.causal ? (1ll << j) : 1;
      for (int side = 0; side < 2; ++side) {
        HA_REQUIRE(jobs.num_jobs < HA_SORT_MAX_JOBS, HA_ERR_SHAPE, "ha_forward: too many sort jobs");
        ha_place_job& job = jobs.job[jobs.num_jobs++];
        job.sorted = sorted[side];
        job.hist = hist[side];
        job.out = (int32_t*)(ws + (side == 0 ? w.qidx[j] : w.kidx[j]));
        job.seg_stride = a.causal ? 2 * seg_len : a.n;
        job.seg_offset = (a.causal && side == 0) ? seg_len : 0;  // queries: second halves, keys: first halves
        job.seg_len = (int)seg_len;
        job.segs_per_seq = (int)segs;
        job.units_per_seg = (int)(seg_len / w.grid.granule) * w.grid.units_per_granule;
        job.first_block = (int)blocks;
        blocks += seqs[side] * segs * job.units_per_seg;
        HA_REQUIRE(blocks < (1ll << 30), HA_ERR_SHAPE, "ha_forward: too many sort units");
      }
    }
    return ha_place_units(jobs, (int)blocks, stream);
  }

  int32_t* bq = (int32_t*)(ws + w.buckets_q);
  int32_t* bk = (int32_t*)(ws + w.buckets_k);
  st = ha_hash_i32(a.q, a.proj, bq, a.batch, a.heads, pl.n_hashed, a.n, a.d, a.lsh_num_projs, t.q_stride_b, t.q_stride_h,
                   t.q_stride_n, 0, 0, a.dtype, stream);
  if (st != HA_OK) return st;
  st = ha_hash_i32(a.k, a.proj, bk, a.batch, a.kv_heads, pl.n_hashed, a.n, a.d, a.lsh_num_projs, t.k_stride_b, t.k_stride_h,
                   t.k_stride_n, 0, 0, a.dtype, stream);
  if (st != HA_OK) return st;
  // all segmented sorts of all levels in one batch of launches per 8-bit digit
  const int passes = a.lsh_num_projs > 8 ? 2 : 1;
  for (int pass = 0; pass < passes; ++pass) {
    const bool last = pass == passes - 1;
    ha_sort_jobs jobs;
    jobs.num_jobs = 0;
    jobs.shift = 8 * pass;
    jobs.idx64 = 0;
    int blocks = 0, segments = 0;
    bool multi = false;
    for (int j = 0; j < nlev; ++j) {
      if (!pl.level_hyper[j]) continue;
      const int64_t seg_len = a.causal ? pl.half[j] : a.n;
      const int64_t segs = a.causal ? (1ll << j) : 1;
      const int64_t stride = a.causal ? 2 * seg_len : a.n;
      const int64_t chunks = (seg_len + HA_SORT_CHUNK - 1) / HA_SORT_CHUNK;
      for (int side = 0; side < 2; ++side) {
        HA_REQUIRE(jobs.num_jobs < HA_SORT_MAX_JOBS, HA_ERR_SHAPE, "ha_forward: too many sort jobs");
        ha_sort_job& job = jobs.job[jobs.num_jobs++];
        const int64_t nseg = a.batch * (side == 0 ? a.heads : a.kv_heads) * segs;
        const int64_t* tmp = side == 0 ? w.tmp_q[j] : w.tmp_k[j];
        job.keys = side == 0 ? bq : bk;
        job.prev = pass == 0 ? nullptr : (const int32_t*)(ws + tmp[(pass - 1) & 1]);
        job.out = last ? ws + (side == 0 ? w.qidx[j] : w.kidx[j]) : ws + tmp[pass & 1];
        job.hist = (uint32_t*)(ws + (side == 0 ? w.hist_q[j] : w.hist_k[j]));
        job.seg_stride = stride;
        job.seg_offset = (a.causal && side == 0) ? seg_len : 0;  // queries: second halves, keys: first halves
        job.seg_len = (int)seg_len;
        job.num_segments = (int)nseg;
        job.chunks_per_seg = (int)chunks;
        job.first_block = blocks;
        job.first_segment = segments;
        HA_REQUIRE(nseg * chunks + blocks < (1ll << 30), HA_ERR_SHAPE, "ha_forward: too many sort chunks");
        blocks += (int)(nseg * chunks);
        segments += (int)nseg;
        multi = multi || chunks > 1;
      }
    }
    st = ha_sort_launch(jobs, blocks, segments, multi, stream);
    if (st != HA_OK) return st;
  }
  return HA_OK;
}

// checks shared by ha_forward and ha_forward_sort once the plan and the workspace layout are known
int check_hashing(const ha_forward_args& a, const Workspace& w, const char* who) {
  HA_REQUIRE(a.proj, HA_ERR_NULL, "%s: null projection matrix", who);
  HA_REQUIRE(a.lsh_num_projs >= 1, HA_ERR_SHAPE, "%s: Invalid value for num_projs", who);
  HA_REQUIRE(a.lsh_num_projs <= 16, HA_ERR_UNSUPPORTED, "%s: lsh_num_projs above 16 is not built", who);
  HA_REQUIRE(a.workspace && a.workspace_bytes >= w.total, HA_ERR_WORKSPACE, "%s: workspace of %lld bytes needed", who,
             (long long)w.total);
  return HA_OK;
}

}  // namespace

extern "C" int ha_block_attn_fwd(const ha_block_attn_args* args, void* stream) {
  HA_REQUIRE(args, HA_ERR_NULL, "ha_block_attn_fwd: null argument block");
  return block_attn(*args, (hipStream_t)stream);
}

extern "C" int ha_flash_attn_fwd(const ha_attn_operands* t, int causal, void* stream) {
  HA_REQUIRE(t, HA_ERR_NULL, "ha_flash_attn_fwd: null argument block");
  return flash_attn(*t, causal, 0, (hipStream_t)stream);
}

extern "C" int64_t ha_forward_workspace_bytes(const ha_forward_args* args) {
  if (!args) return ha_fail(HA_ERR_NULL, "ha_forward_workspace_bytes: null argument block");
  ha_forward_args a = *args;
  // pointers are not needed to size the workspace
  Plan pl;
  if (a.batch <= 0 || a.heads <= 0 || a.kv_heads <= 0 || a.n <= 0 || a.min_seq_len < 0)
    return ha_fail(HA_ERR_SHAPE, "ha_forward_workspace_bytes: sizes must be positive");
  int st = make_plan(a, pl);
  if (st != HA_OK) return st;
  Workspace w;
  layout_workspace(a, pl, w);
  return w.total;
}

extern "C" int ha_forward_sort(const ha_forward_args* args, int64_t* q_idx_offset, int64_t* k_idx_offset,
                               int* num_levels, void* stream) {
  HA_REQUIRE(args && q_idx_offset && k_idx_offset && num_levels, HA_ERR_NULL, "ha_forward_sort: null argument");
  const ha_forward_args& a = *args;
  HA_REQUIRE(a.q && a.k, HA_ERR_NULL, "ha_forward_sort: null tensor pointer");
  HA_REQUIRE(a.dtype == HA_F16 || a.dtype == HA_BF16, HA_ERR_DTYPE, "ha_forward_sort: Only support fp16 and bf16");
  HA_REQUIRE(a.batch > 0 && a.heads > 0 && a.kv_heads > 0 && a.n > 0 && a.min_seq_len >= 0 && a.heads % a.kv_heads == 0,
             HA_ERR_SHAPE, "ha_forward_sort: sizes must be positive and kv_heads must divide heads");
  HA_REQUIRE(a.n < (1ll << 30), HA_ERR_SHAPE, "ha_forward_sort: sequence too long");
  HA_REQUIRE(a.d >= 8 && a.d <= 128 && a.d % 8 == 0, HA_ERR_UNSUPPORTED,
             "ha_forward_sort: head dim must be a multiple of 8 up to 128 (got %lld)", (long long)a.d);
  Plan pl;
  int st = make_plan(a, pl);
  if (st != HA_OK) return st;
  Workspace w;
  layout_workspace(a, pl, w);
  const int nlev = a.causal ? pl.levels : 1;
  *num_levels = nlev;
  for (int j = 0; j < nlev; ++j) {
    q_idx_offset[j] = pl.level_hyper[j] ? w.qidx[j] : -1;
    k_idx_offset[j] = pl.level_hyper[j] ? w.kidx[j] : -1;
  }
  if (!pl.any_hyper) return HA_OK;
  st = check_hashing(a, w, "ha_forward_sort");
  if (st != HA_OK) return st;
  ha_attn_operands t;
  ha_forward_args b = a;
  b.dv = a.d;
  forward_operands(b, t);
  st = check_forward_layout(t, false, "ha_forward_sort");
  if (st != HA_OK) return st;
  return hash_and_sort(a, pl, w, t, (hipStream_t)stream);
}

extern "C" int ha_forward(const ha_forward_args* args, void* stream_) {
  HA_REQUIRE(args, HA_ERR_NULL, "ha_forward: null argument block");
  const ha_forward_args& a = *args;
  hipStream_t stream = (hipStream_t)stream_;
  int st = check_forward(a);
  if (st != HA_OK) return st;
  Plan pl;
  st = make_plan(a, pl);
  if (st != HA_OK) return st;
  Workspace w;
  layout_workspace(a, pl, w);
  if (pl.any_hyper) {
    st = check_hashing(a, w, "ha_forward");
    if (st != HA_OK) return st;
  }
  unsigned char* ws = (unsigned char*)a.workspace;

  ha_attn_operands t;
  forward_operands(a, t);
  st = check_forward_layout(t, true, "ha_forward");
  if (st != HA_OK) return st;

  // 1. bucket ids, once for the whole tensors (the projection does not depend on the level), and
  // 2. the bucket order of every segment of every hashed level
  if (pl.any_hyper) {
    st = hash_and_sort(a, pl, w, t, stream);
    if (st != HA_OK) return st;
  }

  auto hyper_level = [&](int j, bool accumulate) -> int {
    const int64_t seg_len = a.causal ? pl.half[j] : a.n;
    const int64_t segs = a.causal ? (1ll << j) : 1;
    ha_block_attn_args b = {};
    b.t = t;
    b.t.n_q = b.t.n_k = seg_len;
    b.t.segs = segs;
    b.t.seg_stride_rows = a.causal ? 2 * seg_len : a.n;
    b.t.q_seg_offset = a.causal ? seg_len : 0;
    b.t.k_seg_offset = 0;
    b.q_idx = ws + w.qidx[j];
    b.k_idx = ws + w.kidx[j];
    b.sampled_idx = a.sampled_idx;
    b.idx_type = HA_IDX_I32;
    b.q_idx_stride_b = a.heads * segs * seg_len; b.q_idx_stride_h = segs * seg_len; b.q_idx_stride_n = 1;
    b.k_idx_stride_b = a.kv_heads * segs * seg_len; b.k_idx_stride_h = segs * seg_len; b.k_idx_stride_n = 1;
    b.sampled_stride_b = b.sampled_stride_h = 0;
    b.block_size = a.block_size;
    b.sample_size = a.sample_size;
    b.smooth_block = a.smooth_block;
    b.accumulate = accumulate;
    // an odd n: the last query of the last segment is the appended zero row; it is placed by its bucket like
    // any other row and its result is dropped
    return block_attn(b, stream, seg_len - (pl.n_hashed - a.n));
  };

  if (!a.causal) {
    if (pl.level_hyper[0]) return hyper_level(0, false);
    ha_attn_operands f = t;
    f.n_q = f.n_k = a.n;
    f.segs = 1; f.seg_stride_rows = a.n; f.q_seg_offset = f.k_seg_offset = 0;
    return flash_attn(f, 0, 0, stream);
  }

  // Exact launches over the segments of level `level` (leaves: level == pl.levels, whole segments with the
  // causal mask; else the off-diagonal part of that level: second halves against first halves).  With an odd
  // length somewhere the segments are ragged: the kernel finds each segment's rows from the plan.
  auto exact_level = [&](int level, bool leaves) -> int {
    ha_attn_operands f = t;
    const int64_t rows = leaves ? pl.len[level] : pl.half[level];
    f.n_q = f.n_k = rows;
    f.segs = 1ll << level;
    f.seg_stride_rows = leaves ? rows : 2 * rows;
    f.q_seg_offset = leaves ? 0 : rows;
    f.k_seg_offset = 0;
    if (!pl.ragged) return flash_attn(f, leaves ? 1 : 0, leaves ? 0 : 1, stream);
    Ragged rag = {};
    rag.levels = level;
    rag.split = leaves ? 0 : 1;
    rag.n = (int)a.n;
    for (int i = 0; i <= level && i < pl.levels; ++i) rag.half[i] = (int)pl.half[i];
    return flash_attn(f, leaves ? 1 : 0, leaves ? 0 : 1, stream, &rag);
  };

  // 3. leaves: exact causal attention on every segment of the deepest level
  st = exact_level(pl.levels, true);
  if (st != HA_OK) return st;
  // 4. off-diagonal parts, deepest level first, merged in place into the second halves
  for (int j = pl.levels - 1; j >= 0; --j) {
    st = pl.level_hyper[j] ? hyper_level(j, true) : exact_level(j, false);
    if (st != HA_OK) return st;
  }
  return HA_OK;
}
