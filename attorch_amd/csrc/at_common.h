// Shared device/host helpers for the gfx950 (CDNA4, wave64) kernels of libattorch_hip.
//
// Conventions used by every kernel in this library:
//   * storage dtypes are fp32 / fp16 / bf16, all arithmetic is fp32
//   * a "chunk" is the unit one lane moves with one 128-bit access of the narrowest
//     tensor involved (8 x 16-bit or 4 x fp32 elements)
//   * cross-lane reductions use wave64 shuffles first and LDS across waves; nothing
//     uses floating-point atomics, so results are bit-reproducible run to run
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/attorch_hip.h"

namespace at_hip {

typedef __bf16 bf16_t;
typedef _Float16 f16_t;

constexpr int kWave = 64;

template <typename T> struct dtype_of;
template <> struct dtype_of<float>  { static constexpr int value = AT_DTYPE_F32; };
template <> struct dtype_of<f16_t>  { static constexpr int value = AT_DTYPE_F16; };
template <> struct dtype_of<bf16_t> { static constexpr int value = AT_DTYPE_BF16; };

__host__ __device__ inline int dtype_size(int dt) { return dt == AT_DTYPE_F32 ? 4 : 2; }
inline bool dtype_valid(int dt) { return dt == AT_DTYPE_F32 || dt == AT_DTYPE_F16 || dt == AT_DTYPE_BF16; }

template <typename T> __device__ __forceinline__ float to_f32(T v) { return static_cast<float>(v); }
template <typename T> __device__ __forceinline__ T from_f32(float v) { return static_cast<T>(v); }

// ---- N-element contiguous load/store through the widest access the byte count allows ----
template <int BYTES> struct raw_vec;
template <> struct raw_vec<2>  { typedef uint16_t type; };
template <> struct raw_vec<4>  { typedef uint32_t type; };
template <> struct raw_vec<8>  { typedef uint2 type; };
template <> struct raw_vec<16> { typedef uint4 type; };

// Loads N elements of T starting at p (p must be aligned to min(16, N*sizeof(T))) and
// widens them to fp32.
template <typename T, int N>
__device__ __forceinline__ void load_f32(const T* __restrict__ p, float (&out)[N]) {
  constexpr int BYTES = N * (int)sizeof(T);
  if constexpr (BYTES <= 16) {
    typedef typename raw_vec<BYTES>::type R;
    union { R r; T e[N]; } u;
    u.r = *reinterpret_cast<const R*>(p);
#pragma unroll
    for (int i = 0; i < N; ++i) out[i] = to_f32(u.e[i]);
  } else {
    constexpr int PER = 16 / (int)sizeof(T);
#pragma unroll
    for (int j = 0; j < N / PER; ++j) {
      union { uint4 r; T e[PER]; } u;
      u.r = reinterpret_cast<const uint4*>(p)[j];
#pragma unroll
      for (int i = 0; i < PER; ++i) out[j * PER + i] = to_f32(u.e[i]);
    }
  }
}

template <typename T, int N>
__device__ __forceinline__ void store_f32(T* __restrict__ p, const float (&v)[N]) {
  constexpr int BYTES = N * (int)sizeof(T);
  if constexpr (BYTES <= 16) {
    typedef typename raw_vec<BYTES>::type R;
    union { R r; T e[N]; } u;
#pragma unroll
    for (int i = 0; i < N; ++i) u.e[i] = from_f32<T>(v[i]);
    *reinterpret_cast<R*>(p) = u.r;
  } else {
    constexpr int PER = 16 / (int)sizeof(T);
#pragma unroll
    for (int j = 0; j < N / PER; ++j) {
      union { uint4 r; T e[PER]; } u;
#pragma unroll
      for (int i = 0; i < PER; ++i) u.e[i] = from_f32<T>(v[j * PER + i]);
      reinterpret_cast<uint4*>(p)[j] = u.r;
    }
  }
}

// Parameter vectors (weight / bias) may be stored in a dtype different from the
// activations; they are small and cache resident, so a runtime dtype switch is enough.
template <int N>
__device__ __forceinline__ void load_param_f32(const void* __restrict__ p, int dt, int64_t idx,
                                               float (&out)[N]) {
  if (dt == AT_DTYPE_F32) load_f32<float, N>(reinterpret_cast<const float*>(p) + idx, out);
  else if (dt == AT_DTYPE_F16) load_f32<f16_t, N>(reinterpret_cast<const f16_t*>(p) + idx, out);
  else load_f32<bf16_t, N>(reinterpret_cast<const bf16_t*>(p) + idx, out);
}

__device__ __forceinline__ float load_scalar_f32(const void* __restrict__ p, int dt, int64_t idx) {
  if (dt == AT_DTYPE_F32) return reinterpret_cast<const float*>(p)[idx];
  if (dt == AT_DTYPE_F16) return to_f32(reinterpret_cast<const f16_t*>(p)[idx]);
  return to_f32(reinterpret_cast<const bf16_t*>(p)[idx]);
}

__device__ __forceinline__ void store_scalar_f32(void* __restrict__ p, int dt, int64_t idx, float v) {
  if (dt == AT_DTYPE_F32) reinterpret_cast<float*>(p)[idx] = v;
  else if (dt == AT_DTYPE_F16) reinterpret_cast<f16_t*>(p)[idx] = from_f32<f16_t>(v);
  else reinterpret_cast<bf16_t*>(p)[idx] = from_f32<bf16_t>(v);
}

// ---- packed access to raw 32-bit words (keeps register-cached rows packed) ----
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

template <typename T> struct Word;   // view of one 32-bit register holding 1 (fp32) or 2 elements
template <> struct Word<float> {
  static constexpr int N = 1;
  static constexpr uint32_t kNegInf = 0xff800000u;
  template <int K> static __device__ __forceinline__ float get(uint32_t w) { return __uint_as_float(w); }
  static __device__ __forceinline__ uint32_t pack(float a, float) { return __float_as_uint(a); }
};
template <> struct Word<f16_t> {
  static constexpr int N = 2;
  static constexpr uint32_t kNegInf = 0xfc00fc00u;
  template <int K> static __device__ __forceinline__ float get(uint32_t w) {
    const f16x2_t h = __builtin_bit_cast(f16x2_t, w);
    return static_cast<float>(K == 0 ? h.x : h.y);
  }
  static __device__ __forceinline__ uint32_t pack(float a, float b) {
    f16x2_t h;
    h.x = static_cast<f16_t>(a);
    h.y = static_cast<f16_t>(b);
    return __builtin_bit_cast(uint32_t, h);
  }
};
template <> struct Word<bf16_t> {
  static constexpr int N = 2;
  static constexpr uint32_t kNegInf = 0xff80ff80u;
  template <int K> static __device__ __forceinline__ float get(uint32_t w) {
    return __uint_as_float(K == 0 ? (w << 16) : (w & 0xffff0000u));
  }
  static __device__ __forceinline__ uint32_t pack(float a, float b) {
    bf16x2_t h;
    h.x = static_cast<bf16_t>(a);
    h.y = static_cast<bf16_t>(b);
    return __builtin_bit_cast(uint32_t, h);
  }
};

// Widens the 16 / sizeof(T) elements of a raw 128-bit vector.
template <typename T>
__device__ __forceinline__ void unpack16(const uint4& r, float (&f)[16 / sizeof(T)]) {
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (Word<T>::N == 1) f[i] = Word<T>::template get<0>(w[i]);
    else { f[2 * i] = Word<T>::template get<0>(w[i]); f[2 * i + 1] = Word<T>::template get<1>(w[i]); }
  }
}

template <typename T>
__device__ __forceinline__ uint4 pack16(const float (&f)[16 / sizeof(T)]) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (Word<T>::N == 1) w[i] = Word<T>::pack(f[i], 0.f);
    else w[i] = Word<T>::pack(f[2 * i], f[2 * i + 1]);
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// Optimisation barrier on a register-resident 128-bit value: the compiler must treat it as
// modified, so values derived from it earlier (e.g. widened copies) are not kept alive.
__device__ __forceinline__ void keep_raw(uint4& v) {
  asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w));
}

// ---- reductions over a group of `group` consecutive lanes (power of two, <= 1024) ----
struct SumOp { __device__ __forceinline__ float operator()(float a, float b) const { return a + b; } };
struct MaxOp { __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); } };

template <typename Op>
__device__ __forceinline__ float wave_reduce(float v, int width, Op op) {
  for (int o = width >> 1; o > 0; o >>= 1) v = op(v, __shfl_xor(v, o, kWave));
  return v;
}

// All lanes of the group receive the result. `scratch` holds blockDim.x / 64 floats and is
// only touched when a group spans several waves. Every thread of the block must call this
// (it contains block-wide barriers when group > 64).
template <typename Op>
__device__ __forceinline__ float group_reduce(float v, int group, float* scratch, Op op, float identity) {
  if (group <= kWave) return wave_reduce(v, group, op);
  v = wave_reduce(v, kWave, op);
  const int wave = threadIdx.x / kWave;
  const int waves_per_group = group / kWave;
  __syncthreads();
  if ((threadIdx.x & (kWave - 1)) == 0) scratch[wave] = v;
  __syncthreads();
  const int first = (wave / waves_per_group) * waves_per_group;
  float r = identity;
  for (int i = 0; i < waves_per_group; ++i) r = op(r, scratch[first + i]);
  return r;
}

// ---- host side ----
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int device_cu_count() {
  static int cached = 0;  // written once with the same value by any racing thread
  if (cached == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cached = n;
  }
  return cached;
}

inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? AT_OK : static_cast<int>(e);
}

inline int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int next_pow2(int64_t v) { int p = 1; while (p < v) p <<= 1; return p; }

}  // namespace at_hip
