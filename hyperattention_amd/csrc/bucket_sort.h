// Job table shared by the sort kernels and the fused forward pass.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define HA_SORT_CHUNK 4096   // keys per workgroup
#define HA_SORT_MAX_JOBS 40

struct ha_sort_job {
  const int32_t* keys;   // key array; segment s starts at keys[seg_offset + s*seg_stride]
  const int32_t* prev;   // previous pass' order (num_segments*seg_len), or null for 0..seg_len-1
  void* out;             // (num_segments, seg_len) int32 or int64 row numbers local to the segment
  uint32_t* hist;        // (num_segments, chunks_per_seg, 256) scratch, used when chunks_per_seg > 1
  int64_t seg_stride;
  int64_t seg_offset;
  int seg_len;
  int num_segments;
  int chunks_per_seg;
  int first_block;       // first workgroup of this job in the hist/scatter launches
  int first_segment;     // first workgroup of this job in the scan launch
};

struct ha_sort_jobs {
  ha_sort_job job[HA_SORT_MAX_JOBS];
  int num_jobs;
  int shift;   // bit offset of the 8-bit digit sorted in this pass
  int idx64;   // output width of this pass
  int scanned; // set by ha_sort_launch: the histograms hold first output slots (scan launch) rather than counts
};

int ha_sort_launch(const ha_sort_jobs& jobs, int total_blocks, int total_segments, bool any_multi_chunk,
                   hipStream_t stream);

// ---- all levels of one forward pass from one ranking --------------------------------------------
// Every segment of the causal recursion is a whole number of leaf-length granules.  A granule is cut
// into units of at most HA_SORT_CHUNK rows; each unit is put in bucket order once (ha_rank_units), and
// the order of any segment follows from its units' orders and bucket counts (ha_place_units): all rows
// of bucket b come before those of bucket b+1, inside a bucket unit after unit.
struct ha_unit_grid {
  int64_t n;            // rows per sequence
  int64_t granule;      // leaf length (n for the non-causal case); divides n
  int unit;             // rows per unit, <= HA_SORT_CHUNK; the last unit of a granule may be shorter
  int units_per_granule;
  int units_per_seq;
};

struct ha_place_job {
  const uint32_t* sorted;  // (seqs, n): per unit, (bucket << 16) | row inside the unit, in bucket order
  const uint32_t* hist;    // (seqs * units_per_seq, 256) rows per bucket of every unit
  int32_t* out;            // (num_segments, seg_len) rows local to the segment
  int64_t seg_stride;      // rows between segments of one sequence
  int64_t seg_offset;      // first row of the first segment of a sequence
  int seg_len;
  int segs_per_seq;
  int units_per_seg;
  int first_block;
};

struct ha_place_jobs {
  ha_place_job job[HA_SORT_MAX_JOBS];
  int num_jobs;
  ha_unit_grid grid;
};

// ids: byte-sized bucket ids of two tensors, (seqs[i], n) each
int ha_rank_units(const uint8_t* const ids[2], uint32_t* const sorted[2], uint32_t* const hist[2], const int64_t seqs[2],
                  const ha_unit_grid& grid, hipStream_t stream);
int ha_place_units(const ha_place_jobs& jobs, int total_blocks, hipStream_t stream);

// Bucket ids of the queries and keys of one forward pass as one byte each (at most 8 projections, one shared
// projection matrix), one launch.  Strides: batch, head, row, in elements.  Defined in lsh_hash.hip.
// Only the first n_read <= n rows of a sequence exist; the ids of the others are those of zero rows.
int ha_hash_pair_u8(const void* q, const void* k, const void* proj, uint8_t* ids_q, uint8_t* ids_k, int64_t batch,
                    int64_t heads, int64_t kv_heads, int64_t n, int64_t n_read, int64_t d, int64_t r,
                    const int64_t (&q_strides)[3], const int64_t (&k_strides)[3], int dtype, hipStream_t stream);
// ha_lsh_hash (int32 ids) with the same n / n_read distinction
int ha_hash_i32(const void* x, const void* proj, int32_t* buckets, int64_t batch, int64_t heads, int64_t n,
                int64_t n_read, int64_t d, int64_t r, int64_t x_stride_b, int64_t x_stride_h, int64_t x_stride_n,
                int64_t proj_stride_b, int64_t proj_stride_h, int dtype, hipStream_t stream);
