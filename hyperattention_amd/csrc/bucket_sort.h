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
};

int ha_sort_launch(const ha_sort_jobs& jobs, int total_blocks, int total_segments, bool any_multi_chunk,
                   hipStream_t stream);
