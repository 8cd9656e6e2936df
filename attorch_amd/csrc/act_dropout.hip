// Standalone activation layers with fused dropout, and dropout on its own: flat elementwise
// passes (one read, one write forward; two reads, one write backward), 128-bit accesses.
//
//   forward : y  = dropout(act(x))
//   backward: dx = dropout'(dy) * act'(x)      (the same mask, recomputed from the seed)
//
// The dropout mask is a pure function of (seed, element index): Philox4x32-7 keyed by the seed
// with the counter set to index / 8 yields four 32-bit words = eight 16-bit numbers, element
// index % 8 takes its number u, and the element is dropped when u / 65536 is below drop_p; kept
// elements are scaled by 1 / (1 - drop_p).  Forward and backward therefore agree without a
// stored mask, for every dtype and launch shape.  The generator's integer arithmetic, not memory,
// is what bounds this kernel: 16 bits per element halve its cost (the drop probability is exact
// to 2^-16), and seven rounds instead of the customary ten — the fewest for which Philox4x32
// passes the BigCrush battery (Salmon et al., SC11) — take another 30 % off.
#include <type_traits>

#include "at_act.h"

namespace at_hip {
namespace {

struct Philox4 { uint32_t x, y, z, w; };

__device__ __forceinline__ Philox4 philox4x32_7(uint32_t c0, uint32_t c1, uint32_t k0, uint32_t k1) {
  constexpr uint32_t kMulA = 0xD2511F53u, kMulB = 0xCD9E8D57u, kWeylA = 0x9E3779B9u, kWeylB = 0xBB67AE85u;
  uint32_t c2 = 0u, c3 = 0u;
#pragma unroll
  for (int r = 0; r < 7; ++r) {
    const uint32_t hi0 = __umulhi(kMulA, c0), lo0 = kMulA * c0;
    const uint32_t hi1 = __umulhi(kMulB, c2), lo1 = kMulB * c2;
    c0 = hi1 ^ c1 ^ k0;
    c1 = lo1;
    c2 = hi0 ^ c3 ^ k1;
    c3 = lo0;
    k0 += kWeylA;
    k1 += kWeylB;
  }
  return Philox4{c0, c1, c2, c3};
}

__device__ __forceinline__ float uniform16(uint32_t bits16) { return (float)bits16 * (1.0f / 65536.0f); }

// keep[j] = 1 / (1 - drop_p) for kept elements, 0 for dropped ones, for the VEC elements from
// `first` on (first % VEC == 0; VEC is 8, 4 or 1).
template <int VEC>
__device__ __forceinline__ void dropout_factors(int64_t first, uint32_t seed, float drop_p, float inv_keep,
                                                float (&keep)[VEC]) {
  static_assert(VEC == 8 || VEC == 4 || VEC == 1, "a vector is a whole or half generator output, or one element");
  const uint64_t ctr = (uint64_t)first >> 3;
  const Philox4 r = philox4x32_7((uint32_t)ctr, (uint32_t)(ctr >> 32), seed, 0u);
  const uint32_t words[4] = {r.x, r.y, r.z, r.w};
  if (VEC == 8) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const uint32_t u = (j & 1) ? words[j >> 1] >> 16 : words[j >> 1] & 0xffffu;
      keep[j] = uniform16(u) < drop_p ? 0.f : inv_keep;
    }
  } else if (VEC == 4) {
    const bool upper = (first >> 2) & 1;
    const uint32_t w0 = upper ? words[2] : words[0], w1 = upper ? words[3] : words[1];
    keep[VEC == 4 ? 0 : 0] = uniform16(w0 & 0xffffu) < drop_p ? 0.f : inv_keep;
    keep[VEC == 4 ? 1 : 0] = uniform16(w0 >> 16) < drop_p ? 0.f : inv_keep;
    keep[VEC == 4 ? 2 : 0] = uniform16(w1 & 0xffffu) < drop_p ? 0.f : inv_keep;
    keep[VEC == 4 ? 3 : 0] = uniform16(w1 >> 16) < drop_p ? 0.f : inv_keep;
  } else {
    const int e = (int)(first & 7);
    uint32_t w = words[0];
    if ((e >> 1) == 1) w = words[1];
    if ((e >> 1) == 2) w = words[2];
    if ((e >> 1) == 3) w = words[3];
    keep[0] = uniform16((e & 1) ? w >> 16 : w & 0xffffu) < drop_p ? 0.f : inv_keep;
  }
}

// BACKWARD = false: out = dropout(act(in0)).  BACKWARD = true: out = dropout'(in0) * act'(in1)
// (in0 = output gradient, in1 = forward input; in1 is not read when act == AT_ACT_NONE).
constexpr int kActBlock = 256, kActUnroll = 1;
template <typename T, bool BACKWARD, bool VECTOR>
__global__ __launch_bounds__(kActBlock) void act_dropout_kernel(const T* __restrict__ in0, const T* __restrict__ in1,
                                                          T* __restrict__ out, int64_t n, int act, float param,
                                                          float drop_p, float inv_keep, uint32_t seed) {
  constexpr int VEC = VECTOR ? 16 / (int)sizeof(T) : 1;
  // One vector per lane, and as a rule one step per workgroup (the grid covers the tensor): short
  // waves that end behind their store keep more bytes in flight than a few long-lived ones, whose
  // next loads queue behind the acknowledgement of their own stores (measured: 6.0-6.4 TB/s
  // against 4.7-5.6 for a grid capped at 16 workgroups per CU, and 5.8 with four vectors per lane).
  constexpr int U = kActUnroll;
  const bool dropout = drop_p > 0.f;
  const int64_t n_vec = VECTOR ? n / VEC : n;
  const int64_t stride = (int64_t)gridDim.x * (kActBlock * U);
  for (int64_t v0 = (int64_t)blockIdx.x * (kActBlock * U) + threadIdx.x; v0 < n_vec; v0 += stride) {
    float a[U][VEC], b[U][VEC];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t v = v0 + u * kActBlock;
      const int64_t first = (v < n_vec ? v : v0) * VEC;   // past the end: a vector that exists, loaded again
      load_f32<T, VEC>(in0 + first, a[u]);
      if (BACKWARD && act != AT_ACT_NONE) load_f32<T, VEC>(in1 + first, b[u]);
    }
    // the activation is chosen once per step, not once per element
    float o[U][VEC];
    auto apply = [&](auto act_c) {
      constexpr int ACT = decltype(act_c)::value;
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          if (BACKWARD) o[u][j] = ACT != AT_ACT_NONE ? act_derivative(ACT, b[u][j], param) : 1.f;
          else o[u][j] = ACT != AT_ACT_NONE ? act_forward(ACT, a[u][j], param) : a[u][j];
        }
    };
    AT_ACT_DISPATCH(act, apply(std::integral_constant<int, ACT>()));
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t v = v0 + u * kActBlock;
      if (v >= n_vec) break;
      const int64_t first = v * VEC;
      if (dropout) {
        float keep[VEC];
        dropout_factors<VEC>(first, seed, drop_p, inv_keep, keep);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          // a dropped element is an exact zero whatever it held (inf * 0 would not be)
          if (BACKWARD) a[u][j] = keep[j] == 0.f ? 0.f : a[u][j] * keep[j];
          else o[u][j] = keep[j] == 0.f ? 0.f : o[u][j] * keep[j];
        }
      }
      if (BACKWARD) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) o[u][j] = a[u][j] * o[u][j];
      }
      store_f32<T, VEC>(out + first, o[u]);
    }
  }
  if (VECTOR) {
    // tail of fewer than VEC elements: one lane each
    const int64_t done = n_vec * VEC;
    const int64_t e = done + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (e < n) {
      const float x0 = to_f32(in0[e]);
      float val;
      if (BACKWARD) val = act != AT_ACT_NONE ? act_derivative(act, to_f32(in1[e]), param) : 1.f;
      else val = act != AT_ACT_NONE ? act_forward(act, x0, param) : x0;
      float g = x0;
      if (dropout) {
        float keep[1];
        dropout_factors<1>(e, seed, drop_p, inv_keep, keep);
        if (BACKWARD) g = keep[0] == 0.f ? 0.f : g * keep[0];
        else val = keep[0] == 0.f ? 0.f : val * keep[0];
      }
      out[e] = from_f32<T>(BACKWARD ? g * val : val);
    }
  }
}

template <typename F>
inline int dispatch_dtype(int dt, F&& f) {
  if (dt == AT_DTYPE_F32) return f((float*)0);
  if (dt == AT_DTYPE_F16) return f((f16_t*)0);
  if (dt == AT_DTYPE_BF16) return f((bf16_t*)0);
  return AT_ERR_DTYPE;
}

template <bool BACKWARD>
int launch(const void* in0, const void* in1, void* out, int64_t n, int act, float param, float drop_p,
           uint32_t seed, int dtype, hipStream_t stream) {
  if (!in0 || !out) return AT_ERR_NULL;
  if (!dtype_valid(dtype)) return AT_ERR_DTYPE;
  if (!act_valid(act)) return AT_ERR_ACT;
  if (BACKWARD && act != AT_ACT_NONE && !in1) return AT_ERR_NULL;
  if (n < 0 || !(drop_p >= 0.f && drop_p <= 1.f)) return AT_ERR_DIM;
  if (n == 0) return AT_OK;
  const float inv_keep = drop_p < 1.f ? 1.0f / (1.0f - drop_p) : 0.f;
  const bool vec = aligned16(in0) && aligned16(out) && (!in1 || aligned16(in1));
  return dispatch_dtype(dtype, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    constexpr int VEC = 16 / (int)sizeof(T);
    const int64_t items = vec ? cdiv64(n, VEC) : n;
    int64_t blocks = cdiv64(items, kActBlock * kActUnroll);
    const int64_t cap = (int64_t)1 << 22;   // beyond that a workgroup takes several steps
    if (blocks > cap) blocks = cap;
    if (vec)
      hipLaunchKernelGGL((act_dropout_kernel<T, BACKWARD, true>), dim3((unsigned)blocks), dim3(kActBlock), 0, stream,
                         (const T*)in0, (const T*)in1, (T*)out, n, act, param, drop_p, inv_keep, seed);
    else
      hipLaunchKernelGGL((act_dropout_kernel<T, BACKWARD, false>), dim3((unsigned)blocks), dim3(kActBlock), 0, stream,
                         (const T*)in0, (const T*)in1, (T*)out, n, act, param, drop_p, inv_keep, seed);
    return launch_status();
  });
}

}  // namespace
}  // namespace at_hip

using namespace at_hip;

extern "C" {

int at_act_dropout_fwd(const void* input, void* output, int64_t size, int act, float param, float drop_p,
                       uint32_t seed, int dtype, at_stream_t stream) {
  return launch<false>(input, nullptr, output, size, act, param, drop_p, seed, dtype, (hipStream_t)stream);
}

int at_act_dropout_bwd(const void* output_grad, const void* input, void* input_grad, int64_t size, int act,
                       float param, float drop_p, uint32_t seed, int dtype, at_stream_t stream) {
  return launch<true>(output_grad, input, input_grad, size, act, param, drop_p, seed, dtype, (hipStream_t)stream);
}

}  // extern "C"
