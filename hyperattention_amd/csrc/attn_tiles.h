// Building blocks shared by the attention kernels (forward and backward) for gfx950: the MFMA
// wrappers, the swizzled row-major LDS tile layouts with their operand reads, and the HBM -> LDS
// row loads.  Everything sits in an unnamed namespace: each kernel file gets its own copy.
#pragma once

#include "ha_common.h"

namespace {

constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;
constexpr int NUM_XCD = 8;

// Workgroups are handed to the 8 XCDs round-robin by their linear id, and each XCD has its own L2.
// Re-number them so that every XCD works through one contiguous range of (head, tile): the
// tiles that share a head's rows then meet in the same L2.
__device__ __forceinline__ int xcd_contiguous_id(int linear, int total) {
  const int xcd = (unsigned)linear % NUM_XCD, k = (unsigned)linear / NUM_XCD;
  const int q = (unsigned)total / NUM_XCD, r = (unsigned)total % NUM_XCD;
  return xcd * q + (xcd < r ? xcd : r) + k;
}


template <typename T>
struct Mfma;
template <>
struct Mfma<f16_t> {
  static __device__ __forceinline__ f32x16 run(f16x8 a, f16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  // c[*] + a[0] + a[1] + a[2] + a[3] on the matrix pipe: the 4x4x4 MFMA works on 16 independent
  // blocks of 4 lanes; with an all-ones A a lane's four results are all the sum of its own four B values
  static __device__ __forceinline__ f32x4 quad_sum(f16x4 a, f32x4 c) {
    const f16x4 ones = {(f16_t)1.0f, (f16_t)1.0f, (f16_t)1.0f, (f16_t)1.0f};
    return __builtin_amdgcn_mfma_f32_4x4x4f16(ones, a, c, 0, 0, 0);
  }
};
template <>
struct Mfma<bf16_t> {
  static __device__ __forceinline__ f32x16 run(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 quad_sum(bf16x4 a, f32x4 c) {
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    const bf16x4 ones = {(bf16_t)1.0f, (bf16_t)1.0f, (bf16_t)1.0f, (bf16_t)1.0f};
    return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(s16x4, ones), __builtin_bit_cast(s16x4, a), c, 0, 0, 0);
  }
};

// A lane's value and the value of the lane 32 away, in one of the two orders (symmetric uses only: max,
// sum).  v_permlane32_swap exchanges the upper half of one register with the lower half of another; with
// both holding v, every lane ends up with its own value in one of them and its partner's in the other.
// No lane id and no LDS crossbar (ds_bpermute) are involved.  The s_nop covers the wait states the
// instruction needs after a VALU write of its operands, which the compiler does not count for inline asm.
__device__ __forceinline__ void ha_with_lane_xor32(float v, float& a, float& b) {
  a = v;
  b = v;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float ha_max_xor32(float v) {
  float a, b;
  ha_with_lane_xor32(v, a, b);
  return fmaxf(a, b);
}
__device__ __forceinline__ float ha_sum_xor32(float v) {
  float a, b;
  ha_with_lane_xor32(v, a, b);
  return a + b;
}

// Address of 16-byte piece `piece_bytes` of row `row`: a wave-uniform base plus a 32-bit byte offset,
// so that a lane spends one 24-bit multiply-add on it instead of a 64-bit multiplication.  The entry
// points check that row numbers and row strides in bytes stay below 2^24 and their products below 2^32.
__device__ __forceinline__ const unsigned char* row_address(const unsigned char* base, int row, uint32_t stride_bytes,
                                                            uint32_t piece_bytes) {
  return base + (uint32_t)(__umul24((uint32_t)row, stride_bytes) + piece_bytes);
}

// 16-byte piece `piece` of row `row` of a row-major [rows][D] 2-byte tile, XOR-swizzled; byte offset.
// Q and K tiles are read 16 bytes per lane, 16 lanes (16 consecutive rows, the same piece of each) at a time
// over the 64 banks: they move a piece by the row number modulo the pieces of a row (8 at D = 64, where rows
// r and r + 8 still share a bank group: a row is half a bank window; 16 at D = 128, where the 16 rows then
// fall into 16 different groups).  V tiles are read by the transposing loads, 16 lanes at a time: 4
// consecutive rows x 32 bytes; they move a PAIR of pieces by the row number mod 4, so that the four rows fall
// into four different 32-byte bank groups.
template <int D>
__device__ __forceinline__ int k_swizzle(int row) { return row & (D / 8 - 1) & 15; }
__device__ __forceinline__ int v_swizzle(int row) { return (row & 3) << 1; }
template <int D>
__device__ __forceinline__ int tile_offset(int row, int piece) {
  return row * D * 2 + ((piece ^ k_swizzle<D>(row)) << 4);
}
template <int D>
__device__ __forceinline__ int v_tile_offset(int row, int piece) {
  return row * D * 2 + ((piece ^ v_swizzle(row)) << 4);
}

template <typename T>
__device__ __forceinline__ typename ElemTraits<T>::vec8 lds_read_k(const unsigned char* tile, int off) {
  return *reinterpret_cast<const typename ElemTraits<T>::vec8*>(tile + off);
}

// 8 keys x 1 dv column of V, transposed by the LDS unit: two 4-key reads
template <typename T>
__device__ __forceinline__ typename ElemTraits<T>::vec8 lds_read_vt(const unsigned char* tile, int off, int row_bytes) {
#if defined(__HIP_DEVICE_COMPILE__)  // the builtin only exists in the device pass
  typedef short s16x4 __attribute__((ext_vector_type(4)));
  typedef short s16x8 __attribute__((ext_vector_type(8)));
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(tile + off));
  const s16x4 hi8 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(tile + off + 8 * row_bytes));
  const s16x8 both = __builtin_shufflevector(lo, hi8, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(typename ElemTraits<T>::vec8, both);
#else
  return typename ElemTraits<T>::vec8{};
#endif
}

// 16 bytes per lane from global memory straight into LDS at lds_dst + lane*16 (lds_dst wave-uniform)
__device__ __forceinline__ void global_to_lds_16(const void* src, unsigned char* lds_dst) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef __attribute__((address_space(3))) unsigned char lds_byte;
  __builtin_amdgcn_global_load_lds(src, (lds_byte*)lds_dst, 16, 0, 0);
#endif
}

}  // namespace
