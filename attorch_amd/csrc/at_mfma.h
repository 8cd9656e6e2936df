// Building blocks shared by the 16-bit MFMA kernels (GEMM and implicit-GEMM convolution):
// the 32x32x16 matrix instruction, buffer resources, direct global->LDS loads and the LDS
// image of an operand tile whose rows are contiguous along the contraction index.
#pragma once

#include "at_common.h"

namespace at_hip {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef short s16x4 __attribute__((ext_vector_type(4)));

// D(32x32, fp32) += X(32 x 16) * Y(32 x 16)^T.  Each lane supplies 8 consecutive k of row
// lane % 32 (k half lane / 32) of both operands and receives, in register r, the element
//   D[row of X = (r / 4) * 8 + (lane / 32) * 4 + r % 4][row of Y = lane % 32].
template <typename T> struct Mfma16;
template <> struct Mfma16<bf16_t> {
  static __device__ __forceinline__ f32x16 run(const uint4& x, const uint4& y, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, x), __builtin_bit_cast(bf16x8, y),
                                                   c, 0, 0, 0);
  }
};
template <> struct Mfma16<f16_t> {
  static __device__ __forceinline__ f32x16 run(const uint4& x, const uint4& y, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, x), __builtin_bit_cast(f16x8, y),
                                                  c, 0, 0, 0);
  }
};

__device__ __forceinline__ bool aligned16_dev(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Byte offset of 16-byte chunk `chunk` (0..7) of row `row` inside a [rows][64] 16-bit tile
// (128 bytes per row).  The XOR spreads the 32 rows a fragment read touches over the banks.
__device__ __forceinline__ int lds_chunk_offset(int row, int chunk) {
  return row * 128 + ((chunk ^ ((row ^ (row >> 3)) & 7)) << 4);
}

// Raw buffer resource over [base, base + bytes): loads past the end return zeros.
__device__ __forceinline__ i32x4 make_buffer_rsrc(const void* base, int64_t bytes) {
  const uint64_t addr = reinterpret_cast<uint64_t>(base);
  i32x4 r;
  r.x = (int)(uint32_t)addr;
  r.y = (int)(uint32_t)((addr >> 32) & 0xffffu);   // stride 0: raw buffer
  r.z = (int)bytes;                                  // num_records in bytes
  r.w = 0x00020000;                                  // 32-bit untyped data format
  return r;
}

constexpr int kOobOffset = (int)0x80000000u;  // beyond any buffer these kernels accept (< 2 GiB)

// Global -> LDS without passing through registers (buffer_load ... lds): each wave-wide load
// moves 64 lanes x 16 bytes into one contiguous KiB of LDS, each lane choosing its own global
// address.  Buffer addressing gives zero fill for offsets past the end of the tensor.
// The loads are issued as inline assembly on purpose: the compiler cannot tell that a load into
// one LDS stage does not alias the fragment reads of the other stage and would otherwise wait
// for every outstanding load (vmcnt(0)) before the next LDS read.  The kernels wait for them
// themselves, once, before the barrier that publishes the stage.
__device__ __forceinline__ void lds_dma_16(const i32x4& rsrc, int byte_offset, const char* lds_dst) {
  // LDS byte address of lane 0's 16 bytes; wave-uniform by construction, made so for the compiler
  const unsigned m0 = (unsigned)__builtin_amdgcn_readfirstlane((int)(uintptr_t)lds_dst);
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(m0), "v"(byte_offset), "s"(rsrc)
               : "m0");
}

__device__ __forceinline__ void lds_dma_wait_all() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// Waits for all loads of the wave except the N issued last (the counter runs in issue order).
template <int N>
__device__ __forceinline__ void lds_dma_wait_newest() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

// Fragment (32 rows x 16 k, 8 consecutive k per lane) of a tile laid out by lds_chunk_offset.
__device__ __forceinline__ uint4 read_frag_kc(const char* tile, int row_base, int ks) {
  const int lane = threadIdx.x & 63;
  return *reinterpret_cast<const uint4*>(tile + lds_chunk_offset(row_base + (lane & 31), ks * 2 + (lane >> 5)));
}

}  // namespace at_hip
