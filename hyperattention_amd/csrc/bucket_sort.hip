// Segmented stable counting sort (argsort) of small integer keys.
// Stands in for torch.sort(buckets, dim=2, stable=True) at hyper_attention.py:116-117 of the
// reference: within every segment the output lists row numbers by non-decreasing key, ties in
// ascending row number.
//
// A segment is cut into chunks of SORT_CHUNK keys, one workgroup each.  Ranking inside a wave
// uses ballot matching (8 ballots give every lane the set of lanes holding the same 8-bit digit),
// so skewed key distributions cost the same as uniform ones and no LDS atomics are needed for the
// order-sensitive part.  Segments longer than one chunk use two launches (per-chunk histograms, then a
// scatter in which every workgroup adds up the histograms of its segment for itself), and beyond
// SORT_DIRECT_CHUNKS chunks per segment a third one between them (per-segment scan); shorter ones a single
// launch.  Keys above 255 take one extra
// least-significant-digit pass per byte.  Several jobs (for instance all recursion levels of a
// causal forward) share one launch through a small by-value job table.
#include "ha_common.h"
#include "bucket_sort.h"

#include <mutex>

namespace {

constexpr int SORT_THREADS = 256;
constexpr int SORT_WAVES = SORT_THREADS / HA_WAVE;
constexpr int SORT_STEPS = HA_SORT_CHUNK / SORT_THREADS;  // 64-key steps per wave per chunk
// up to this many chunks per segment a scatter workgroup reads the histograms of all chunks of its segment
// (256 counters each, from L2) rather than wait for a scan launch that has one workgroup per segment
constexpr int SORT_DIRECT_CHUNKS = 64;

struct BlockRef {
  int job, seg, chunk;
};

// Workgroups go to the 8 XCDs round-robin by their number, and each XCD has its own L2.  Re-numbered so that
// an XCD works through consecutive chunks (units): the rows of a bucket from neighbouring chunks of a segment
// are neighbours in the output, and their short runs then meet in one L2 line before it is written back.
__device__ __forceinline__ int xcd_contiguous_block() {
  const int total = (int)gridDim.x, lin = (int)blockIdx.x;
  const int xq = total / 8, xr = total % 8, xcd = lin % 8;
  return xcd * xq + (xcd < xr ? xcd : xr) + lin / 8;
}

__device__ __forceinline__ BlockRef locate_block(const ha_sort_jobs& jobs, int block, bool per_segment) {
  int j = 0;
  while (j + 1 < jobs.num_jobs &&
         block >= (per_segment ? jobs.job[j + 1].first_segment : jobs.job[j + 1].first_block))
    ++j;
  BlockRef r;
  r.job = j;
  if (per_segment) {
    r.seg = block - jobs.job[j].first_segment;
    r.chunk = 0;
  } else {
    const int local = block - jobs.job[j].first_block;
    r.seg = local / jobs.job[j].chunks_per_seg;
    r.chunk = local % jobs.job[j].chunks_per_seg;
  }
  return r;
}

// lanes of the wave holding the same digit as this lane, restricted to valid lanes.  Per bit: the
// lane's own bit spread over a word (0 or ~0), one ballot, and per mask half one three-input bit
// operation "keep the lanes whose bit equals mine".
__device__ __forceinline__ uint64_t match_digit(int digit, bool valid) {
  const uint64_t all = __ballot(valid);
  uint32_t lo = (uint32_t)all, hi = (uint32_t)(all >> 32);
#pragma unroll
  for (int bit = 0; bit < 8; ++bit) {
    const uint32_t mine = (uint32_t)((int32_t)((uint32_t)digit << (31 - bit)) >> 31);
    const uint64_t b = __ballot(mine != 0u);
    lo &= ~((uint32_t)b ^ mine);
    hi &= ~((uint32_t)(b >> 32) ^ mine);
  }
  return ((uint64_t)hi << 32) | lo;
}

// number of set bits of `mask` below this lane
__device__ __forceinline__ uint32_t rank_below(uint64_t mask) {
  return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
}

// Digits (and source rows) of positions first + s*stride (s < SORT_STEPS) of a segment.  Positions past the
// end are clamped to the last one, so every load is unconditional and all of them are in flight
// together: one memory round trip per pass instead of one per step.
__device__ __forceinline__ void load_digits(const ha_sort_job& job, const int32_t* prev, int64_t seg_base, int first,
                                            int stride, int shift, int (&src)[SORT_STEPS], int (&digit)[SORT_STEPS]) {
#pragma unroll
  for (int s = 0; s < SORT_STEPS; ++s) {
    const int i = min(first + s * stride, job.seg_len - 1);
    src[s] = prev ? prev[i] : i;
  }
#pragma unroll
  for (int s = 0; s < SORT_STEPS; ++s) digit[s] = (job.keys[seg_base + src[s]] >> shift) & 255;
}

// ---- per-chunk histograms (only for segments longer than one chunk) -------------------------
// Counting needs no order, so it uses LDS atomics.
__global__ __launch_bounds__(SORT_THREADS) void sort_hist_kernel(ha_sort_jobs jobs) {
  __shared__ uint32_t hist[256];
  const BlockRef br = locate_block(jobs, blockIdx.x, false);
  const ha_sort_job& job = jobs.job[br.job];
  const int tid = threadIdx.x;
  hist[tid] = 0;
  __syncthreads();
  const int64_t seg_base = job.seg_offset + (int64_t)br.seg * job.seg_stride;
  const int32_t* prev = job.prev ? job.prev + (int64_t)br.seg * job.seg_len : nullptr;
  const int chunk_start = br.chunk * HA_SORT_CHUNK;
  int src[SORT_STEPS], digit[SORT_STEPS];
  load_digits(job, prev, seg_base, chunk_start + tid, SORT_THREADS, jobs.shift, src, digit);
#pragma unroll
  for (int s = 0; s < SORT_STEPS; ++s)
    if (chunk_start + s * SORT_THREADS + tid < job.seg_len) atomicAdd(&hist[digit[s]], 1u);
  __syncthreads();
  job.hist[((int64_t)br.seg * job.chunks_per_seg + br.chunk) * 256 + tid] = hist[tid];
}

// exclusive scan of one value per thread over a 256-thread block
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v, uint32_t* wave_totals) {
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  uint32_t incl = v;
#pragma unroll
  for (int off = 1; off < HA_WAVE; off <<= 1) {
    const uint32_t up = __shfl_up(incl, off);
    if (lane >= off) incl += up;
  }
  if (lane == HA_WAVE - 1) wave_totals[wave] = incl;
  __syncthreads();
  uint32_t base = 0;
  for (int w = 0; w < wave; ++w) base += wave_totals[w];
  __syncthreads();
  return base + incl - v;
}

// ---- per-segment scan: hist[c][k] -> first output slot of (chunk c, key k) -------------------
__global__ __launch_bounds__(SORT_THREADS) void sort_scan_kernel(ha_sort_jobs jobs) {
  __shared__ uint32_t wave_totals[SORT_WAVES];
  const BlockRef br = locate_block(jobs, blockIdx.x, true);
  const ha_sort_job& job = jobs.job[br.job];
  const int k = threadIdx.x;
  uint32_t* h = job.hist + (int64_t)br.seg * job.chunks_per_seg * 256;
  uint32_t running = 0;
  for (int c = 0; c < job.chunks_per_seg; ++c) {
    const uint32_t t = h[c * 256 + k];
    h[c * 256 + k] = running;
    running += t;
  }
  const uint32_t base = block_exclusive_scan(running, wave_totals);
  for (int c = 0; c < job.chunks_per_seg; ++c) h[c * 256 + k] += base;
}

// ---- stable scatter --------------------------------------------------------------------------
// A wave owns a contiguous run of the chunk (wave order = key order) and holds its digits in registers.
// Pass 1 counts digits per wave with LDS atomics; pass 2 ranks the keys inside each 64-key step by
// ballot matching, which is what keeps equal keys in ascending row order.  The chunk is
// put in order in LDS first and then written out by consecutive threads, so that the runs of equal
// keys leave as whole cache lines instead of scattered 4-byte writes.
__global__ __launch_bounds__(SORT_THREADS) void sort_scatter_kernel(ha_sort_jobs jobs) {
  __shared__ uint32_t wave_hist[SORT_WAVES][256];
  __shared__ uint32_t wave_totals[SORT_WAVES];
  __shared__ int32_t to_global[256];            // global slot minus chunk-local slot, per digit
  __shared__ uint32_t staged[HA_SORT_CHUNK];    // (digit << 24) | row, in chunk-local sorted order
  const BlockRef br = locate_block(jobs, xcd_contiguous_block(), false);
  const ha_sort_job& job = jobs.job[br.job];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
#pragma unroll
  for (int w = 0; w < SORT_WAVES; ++w) wave_hist[w][tid] = 0;
  __syncthreads();

  const int64_t seg_base = job.seg_offset + (int64_t)br.seg * job.seg_stride;
  const int32_t* prev = job.prev ? job.prev + (int64_t)br.seg * job.seg_len : nullptr;
  const int chunk_start = br.chunk * HA_SORT_CHUNK;
  const int wave_start = chunk_start + wave * (SORT_STEPS * HA_WAVE);
  const bool stage = job.seg_len <= (1 << 24);  // rows fit 24 bits next to the digit

  int src_all[SORT_STEPS], digit_all[SORT_STEPS];
  load_digits(job, prev, seg_base, wave_start + lane, HA_WAVE, jobs.shift, src_all, digit_all);
#pragma unroll
  for (int s = 0; s < SORT_STEPS; ++s)
    if (wave_start + s * HA_WAVE + lane < job.seg_len) atomicAdd(&wave_hist[wave][digit_all[s]], 1u);
  __syncthreads();

  // chunk-local first slot of key tid, and the global first slot of (this chunk, key tid): from the
  // scan kernel, or equal to the local one when the segment is a single chunk
  uint32_t total = 0;
#pragma unroll
  for (int w = 0; w < SORT_WAVES; ++w) total += wave_hist[w][tid];
  const uint32_t local_base = block_exclusive_scan(total, wave_totals);
  uint32_t global_base = local_base;
  if (job.chunks_per_seg > 1 && jobs.scanned) {
    global_base = job.hist[((int64_t)br.seg * job.chunks_per_seg + br.chunk) * 256 + tid];
  } else if (job.chunks_per_seg > 1) {
    // raw counts: keys tid of the whole segment and of the chunks before this one, eight loads in flight
    const uint32_t* h = job.hist + (int64_t)br.seg * job.chunks_per_seg * 256 + tid;
    uint32_t tot = 0, before = 0;
    for (int c0 = 0; c0 < job.chunks_per_seg; c0 += 8) {
      uint32_t c[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) c[i] = c0 + i < job.chunks_per_seg ? h[(int64_t)(c0 + i) * 256] : 0u;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        before += c0 + i < br.chunk ? c[i] : 0u;
        tot += c[i];
      }
    }
    global_base = block_exclusive_scan(tot, wave_totals) + before;
  }
  to_global[tid] = (int32_t)(global_base - local_base);
  // turn the per-wave counts into per-wave chunk-local first slots
  uint32_t run = local_base;
#pragma unroll
  for (int w = 0; w < SORT_WAVES; ++w) {
    const uint32_t c = wave_hist[w][tid];
    wave_hist[w][tid] = run;
    run += c;
  }
  __syncthreads();

  const int64_t out_base = (int64_t)br.seg * job.seg_len;
#pragma unroll
  for (int s = 0; s < SORT_STEPS; ++s) {
    const int i = wave_start + s * HA_WAVE + lane;
    const bool valid = i < job.seg_len;
    const int src = src_all[s], digit = digit_all[s];
    const uint64_t m = match_digit(digit, valid);
    const uint32_t below = rank_below(m);
    if (valid) {
      const uint32_t slot = wave_hist[wave][digit] + below;
      if (stage) {
        staged[slot] = ((uint32_t)digit << 24) | (uint32_t)src;
      } else {
        const int64_t g = out_base + (int64_t)slot + to_global[digit];
        if (jobs.idx64)
          ((int64_t*)job.out)[g] = src;
        else
          ((int32_t*)job.out)[g] = src;
      }
    }
    // every lane of the wave has read its slot before the first lane of each digit advances it
    // (same wave: LDS operations complete in program order)
    __builtin_amdgcn_wave_barrier();
    if (valid && below == 0) wave_hist[wave][digit] += (uint32_t)__popcll(m);
    __builtin_amdgcn_wave_barrier();
  }
  if (!stage) return;
  __syncthreads();
  const int count = min(HA_SORT_CHUNK, job.seg_len - chunk_start);
  for (int pos = tid; pos < count; pos += SORT_THREADS) {
    const uint32_t v = staged[pos];
    const int64_t g = out_base + pos + to_global[v >> 24];
    if (jobs.idx64)
      ((int64_t*)job.out)[g] = (int64_t)(v & 0xFFFFFFu);
    else
      ((int32_t*)job.out)[g] = (int32_t)(v & 0xFFFFFFu);
  }
}


// ---- one ranking for all levels ---------------------------------------------------------------------
struct RankArgs {
  const uint8_t* ids[2];
  uint32_t* sorted[2];
  uint32_t* hist[2];
  int units0;   // units of the first tensor (seqs * units_per_seq)
  ha_unit_grid grid;
};

// One workgroup per unit: bucket order of the unit's rows and its bucket counts.  Same ranking as the
// scatter kernel above (a wave owns a contiguous run, ballot matching inside 64-row steps).
__global__ __launch_bounds__(SORT_THREADS) void rank_units_kernel(RankArgs a) {
  __shared__ uint32_t wave_hist[SORT_WAVES][256];
  __shared__ uint32_t wave_totals[SORT_WAVES];
  __shared__ uint32_t staged[HA_SORT_CHUNK];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int which = (int)blockIdx.x >= a.units0 ? 1 : 0;
  const int unit_id = (int)blockIdx.x - (which ? a.units0 : 0);
  const ha_unit_grid& g = a.grid;
  const int seq = unit_id / g.units_per_seq, u = unit_id % g.units_per_seq;
  const int gran = u / g.units_per_granule, w = u % g.units_per_granule;
  const int64_t row0 = (int64_t)seq * g.n + (int64_t)gran * g.granule + (int64_t)w * g.unit;
  const int len = (int)min((int64_t)g.unit, g.granule - (int64_t)w * g.unit);
  const uint8_t* ids = a.ids[which] + row0;
#pragma unroll
  for (int k = 0; k < SORT_WAVES; ++k) wave_hist[k][tid] = 0;
  __syncthreads();

  const int per_wave = ((len + SORT_THREADS - 1) / SORT_THREADS) * HA_WAVE;  // rows per wave, whole steps
  const int wave_start = wave * per_wave;
  int digit_all[SORT_STEPS];
#pragma unroll
  for (int s = 0; s < SORT_STEPS; ++s) digit_all[s] = ids[min(wave_start + s * HA_WAVE + lane, len - 1)];
#pragma unroll
  for (int s = 0; s < SORT_STEPS; ++s)
    if (s * HA_WAVE < per_wave && wave_start + s * HA_WAVE + lane < len) atomicAdd(&wave_hist[wave][digit_all[s]], 1u);
  __syncthreads();
  uint32_t total = 0;
#pragma unroll
  for (int k = 0; k < SORT_WAVES; ++k) total += wave_hist[k][tid];
  a.hist[which][(int64_t)unit_id * 256 + tid] = total;
  uint32_t run = block_exclusive_scan(total, wave_totals);
#pragma unroll
  for (int k = 0; k < SORT_WAVES; ++k) {
    const uint32_t c = wave_hist[k][tid];
    wave_hist[k][tid] = run;
    run += c;
  }
  __syncthreads();
#pragma unroll
  for (int s = 0; s < SORT_STEPS; ++s) {
    if (s * HA_WAVE >= per_wave) break;  // the same for every lane of the workgroup
    const int i = wave_start + s * HA_WAVE + lane;
    const bool valid = i < len;
    const int digit = digit_all[s];
    const uint64_t m = match_digit(digit, valid);
    const uint32_t below = rank_below(m);
    if (valid) staged[wave_hist[wave][digit] + below] = ((uint32_t)digit << 16) | (uint32_t)i;
    __builtin_amdgcn_wave_barrier();
    if (valid && below == 0) wave_hist[wave][digit] += (uint32_t)__popcll(m);
    __builtin_amdgcn_wave_barrier();
  }
  __syncthreads();
  uint32_t* out = a.sorted[which] + row0;
  for (int pos = tid; pos < len; pos += SORT_THREADS) out[pos] = staged[pos];
}

// One workgroup per (job, segment, unit): where the unit's rows of every bucket start in the segment's
// order, then a copy of the unit's order to those places.
__global__ __launch_bounds__(SORT_THREADS) void place_units_kernel(ha_place_jobs jobs) {
  __shared__ uint32_t wave_totals[SORT_WAVES];
  __shared__ int32_t delta[256];   // segment slot minus unit slot, per bucket
  const int block = xcd_contiguous_block();
  int j = 0;
  while (j + 1 < jobs.num_jobs && block >= jobs.job[j + 1].first_block) ++j;
  const ha_place_job& job = jobs.job[j];
  const ha_unit_grid& g = jobs.grid;
  const int tid = threadIdx.x;
  const int local = block - job.first_block;
  const int seg = local / job.units_per_seg, u = local % job.units_per_seg;
  const int seq = seg / job.segs_per_seq, sis = seg % job.segs_per_seq;
  const int64_t first_row = job.seg_offset + (int64_t)sis * job.seg_stride;   // of the segment, in its sequence
  const int64_t first_unit = (int64_t)seq * g.units_per_seq + (first_row / g.granule) * g.units_per_granule;
  const uint32_t* h = job.hist + first_unit * 256 + tid;
  // eight independent loads in flight at a time: one after the other, a segment of 32 units would cost the
  // workgroup 32 memory round trips before it moves a single row
  uint32_t tot = 0, before = 0, mine = 0;
  for (int k0 = 0; k0 < job.units_per_seg; k0 += 8) {
    uint32_t c[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) c[i] = k0 + i < job.units_per_seg ? h[(int64_t)(k0 + i) * 256] : 0u;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      before += k0 + i < u ? c[i] : 0u;
      mine = k0 + i == u ? c[i] : mine;
      tot += c[i];
    }
  }
  const uint32_t seg_first = block_exclusive_scan(tot, wave_totals);
  const uint32_t unit_first = block_exclusive_scan(mine, wave_totals);
  delta[tid] = (int32_t)(seg_first + before) - (int32_t)unit_first;
  __syncthreads();
  const int gran = u / g.units_per_granule, w = u % g.units_per_granule;
  const int64_t row0 = (int64_t)gran * g.granule + (int64_t)w * g.unit;   // of the unit, in its segment
  const int len = (int)min((int64_t)g.unit, g.granule - (int64_t)w * g.unit);
  const uint32_t* src = job.sorted + (int64_t)seq * g.n + first_row + row0;
  int32_t* out = job.out + (int64_t)seg * job.seg_len;
  for (int pos0 = tid; pos0 < len; pos0 += 8 * SORT_THREADS) {
    uint32_t v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = src[min(pos0 + i * SORT_THREADS, len - 1)];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int pos = pos0 + i * SORT_THREADS;
      if (pos < len) out[pos + delta[v[i] >> 16]] = (int32_t)row0 + (int32_t)(v[i] & 0xFFFFu);
    }
  }
}

}  // namespace

int ha_rank_units(const uint8_t* const ids[2], uint32_t* const sorted[2], uint32_t* const hist[2], const int64_t seqs[2],
                  const ha_unit_grid& grid, hipStream_t stream) {
  RankArgs a;
  for (int i = 0; i < 2; ++i) {
    a.ids[i] = ids[i];
    a.sorted[i] = sorted[i];
    a.hist[i] = hist[i];
  }
  a.grid = grid;
  const int64_t units = (seqs[0] + seqs[1]) * grid.units_per_seq;
  HA_REQUIRE(units < (1ll << 31) && grid.unit >= 1 && grid.unit <= HA_SORT_CHUNK, HA_ERR_SHAPE,
             "ha_forward: too many sort units");
  a.units0 = (int)(seqs[0] * grid.units_per_seq);
  hipLaunchKernelGGL(rank_units_kernel, dim3((unsigned)units), dim3(SORT_THREADS), 0, stream, a);
  return ha_launch_status("ha_forward (rank)");
}

int ha_place_units(const ha_place_jobs& jobs, int total_blocks, hipStream_t stream) {
  hipLaunchKernelGGL(place_units_kernel, dim3(total_blocks), dim3(SORT_THREADS), 0, stream, jobs);
  return ha_launch_status("ha_forward (place)");
}

int ha_sort_launch(const ha_sort_jobs& jobs_in, int total_blocks, int total_segments, bool any_multi_chunk,
                   hipStream_t stream) {
  ha_sort_jobs jobs = jobs_in;
  int most_chunks = 1;
  for (int j = 0; j < jobs.num_jobs; ++j) most_chunks = jobs.job[j].chunks_per_seg > most_chunks ? jobs.job[j].chunks_per_seg : most_chunks;
  jobs.scanned = most_chunks > SORT_DIRECT_CHUNKS;
  if (any_multi_chunk) {
    hipLaunchKernelGGL(sort_hist_kernel, dim3(total_blocks), dim3(SORT_THREADS), 0, stream, jobs);
    if (jobs.scanned) hipLaunchKernelGGL(sort_scan_kernel, dim3(total_segments), dim3(SORT_THREADS), 0, stream, jobs);
  }
  hipLaunchKernelGGL(sort_scatter_kernel, dim3(total_blocks), dim3(SORT_THREADS), 0, stream, jobs);
  return ha_launch_status("ha_bucket_argsort");
}

static inline int64_t align256(int64_t v) { return (v + 255) & ~(int64_t)255; }

extern "C" int64_t ha_bucket_argsort_workspace_bytes(int64_t num_segments, int64_t seg_len, int64_t num_keys) {
  if (num_segments <= 0 || seg_len <= 0) return 0;
  const int64_t chunks = (seg_len + HA_SORT_CHUNK - 1) / HA_SORT_CHUNK;
  int64_t bytes = align256(num_segments * chunks * 256 * (int64_t)sizeof(uint32_t));
  if (num_keys > 256) bytes += 2 * align256(num_segments * seg_len * (int64_t)sizeof(int32_t));
  return bytes;
}

static int bucket_argsort(const int32_t* keys, void* idx_out, int idx_type, int64_t num_segments, int64_t seg_len,
                          int64_t seg_stride, int64_t seg_offset, int64_t num_keys, void* workspace,
                          int64_t workspace_bytes, void* stream) {
  HA_REQUIRE(keys && idx_out, HA_ERR_NULL, "ha_bucket_argsort: null pointer");
  HA_REQUIRE(idx_type == HA_IDX_I32 || idx_type == HA_IDX_I64, HA_ERR_DTYPE, "ha_bucket_argsort: bad idx_type");
  HA_REQUIRE(num_segments > 0 && seg_len > 0, HA_ERR_SHAPE, "ha_bucket_argsort: sizes must be positive");
  HA_REQUIRE(seg_len < (1ll << 31) && num_segments < (1ll << 24), HA_ERR_SHAPE, "ha_bucket_argsort: too large");
  HA_REQUIRE(num_keys >= 1 && num_keys <= 65536, HA_ERR_UNSUPPORTED, "ha_bucket_argsort: num_keys must be in [1, 65536]");
  const int64_t need = ha_bucket_argsort_workspace_bytes(num_segments, seg_len, num_keys);
  HA_REQUIRE(workspace && workspace_bytes >= need, HA_ERR_WORKSPACE,
             "ha_bucket_argsort: workspace of %lld bytes needed", (long long)need);
  const int64_t chunks = (seg_len + HA_SORT_CHUNK - 1) / HA_SORT_CHUNK;
  HA_REQUIRE(num_segments * chunks < (1ll << 31), HA_ERR_SHAPE, "ha_bucket_argsort: too many chunks");

  ha_sort_jobs jobs;
  jobs.num_jobs = 1;
  ha_sort_job& j = jobs.job[0];
  j.keys = keys;
  j.seg_stride = seg_stride;
  j.seg_offset = seg_offset;
  j.seg_len = (int)seg_len;
  j.num_segments = (int)num_segments;
  j.chunks_per_seg = (int)chunks;
  j.first_block = 0;
  j.first_segment = 0;
  j.hist = (uint32_t*)workspace;
  unsigned char* ws = (unsigned char*)workspace + align256(num_segments * chunks * 256 * (int64_t)sizeof(uint32_t));
  const int passes = num_keys > 256 ? 2 : 1;
  int32_t* tmp[2] = {nullptr, nullptr};
  if (passes > 1) {
    tmp[0] = (int32_t*)ws;
    tmp[1] = (int32_t*)(ws + align256(num_segments * seg_len * (int64_t)sizeof(int32_t)));
  }
  const int32_t* prev = nullptr;
  for (int p = 0; p < passes; ++p) {
    const bool last = p == passes - 1;
    j.prev = prev;
    j.out = last ? idx_out : (void*)tmp[p & 1];
    jobs.shift = 8 * p;
    jobs.idx64 = last && idx_type == HA_IDX_I64;
    int st = ha_sort_launch(jobs, (int)(num_segments * chunks), (int)num_segments, chunks > 1, (hipStream_t)stream);
    if (st != HA_OK) return st;
    prev = tmp[p & 1];
  }
  return HA_OK;
}

extern "C" int ha_bucket_argsort(const int32_t* keys, void* idx_out, int idx_type, int64_t num_segments,
                                 int64_t seg_len, int64_t seg_stride, int64_t seg_offset, int64_t num_keys,
                                 void* workspace, int64_t workspace_bytes, void* stream) {
  return bucket_argsort(keys, idx_out, idx_type, num_segments, seg_len, seg_stride, seg_offset, num_keys, workspace,
                        workspace_bytes, stream);
}

// ---- the same sort for callers that cannot allocate ------------------------------------------------
// The histograms (and, for keys above 255, the two intermediate orders) live in a device array that is
// part of the library's image: one copy per GPU, held until the process ends.  On the host the array's
// name is only a handle; its device address is asked for once per device, with that device current, and
// that address is what the kernels are given.
static __device__ __align__(256) unsigned char scratch[HA_SORT_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex scratch_mutex;
void* scratch_ptr[MAX_DEVICES] = {nullptr};

// device address of `scratch` on the current device (0 on failure, with the status in *st).  The address is
// asked for on the first call on a device; that call must not sit inside a stream capture (the runtime may
// have to load the code object and the array then), so a first call under capture is refused.
void* scratch_on_current_device(hipStream_t stream, int* st) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    *st = ha_fail(e != hipSuccess ? (int)e : HA_ERR_UNSUPPORTED, "ha_bucket_argsort_static: no usable current device");
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (!scratch_ptr[dev]) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone) {
      (void)hipGetLastError();
      *st = ha_fail(HA_ERR_UNSUPPORTED, "ha_bucket_argsort_static: the first call on a device must be made outside "
                    "stream capture (it looks up the scratch array's address)");
      return nullptr;
    }
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      *st = ha_fail(e != hipSuccess ? (int)e : HA_ERR_WORKSPACE, "ha_bucket_argsort_static: hipGetSymbolAddress: %s",
                    hipGetErrorString(e));
      return nullptr;
    }
    scratch_ptr[dev] = p;
  }
  *st = HA_OK;
  return scratch_ptr[dev];
}
}  // namespace

extern "C" int ha_bucket_argsort_static(const int32_t* keys, void* idx_out, int idx_type, int64_t num_segments,
                                        int64_t seg_len, int64_t seg_stride, int64_t seg_offset, int64_t num_keys,
                                        void* stream) {
  HA_REQUIRE(num_segments > 0 && seg_len > 0, HA_ERR_SHAPE, "ha_bucket_argsort_static: sizes must be positive");
  HA_REQUIRE(num_segments < (1ll << 24) && seg_len < (1ll << 31), HA_ERR_SHAPE, "ha_bucket_argsort_static: too large");
  const int64_t need = ha_bucket_argsort_workspace_bytes(num_segments, seg_len, num_keys);
  HA_REQUIRE(need <= (int64_t)HA_SORT_SCRATCH_BYTES, HA_ERR_WORKSPACE,
             "ha_bucket_argsort_static: this sort needs %lld bytes of scratch, the built-in array holds %lld; use "
             "ha_bucket_argsort with a workspace",
             (long long)need, (long long)HA_SORT_SCRATCH_BYTES);
  int st = HA_OK;
  void* ws = scratch_on_current_device((hipStream_t)stream, &st);
  if (!ws) return st;
  // every histogram entry and intermediate order that is read is written by the same call first: nothing
  // has to start at zero
  return bucket_argsort(keys, idx_out, idx_type, num_segments, seg_len, seg_stride, seg_offset, num_keys, ws,
                        (int64_t)HA_SORT_SCRATCH_BYTES, stream);
}
