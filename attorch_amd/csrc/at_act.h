// The 21 activation functions accepted by the Linear / BatchNorm epilogues and their
// derivatives, as fp32 device functions (formulas of attorch/act_kernels.py:13-628; the
// piecewise ones keep the reference's <= / < choices at the joints so gradients agree at the
// boundary points attorch's tests probe).  tanh is 2*sigmoid(2x) - 1 as in the reference (:81).
#pragma once

#include "at_common.h"

namespace at_hip {

inline bool act_valid(int act) { return act >= AT_ACT_NONE && act < AT_ACT_COUNT; }
inline bool act_needs_param(int act) { return act >= AT_ACT_LEAKY_RELU && act <= AT_ACT_SOFTSHRINK; }

// 1 / x by the hardware reciprocal (1 ulp) instead of the correctly rounded division sequence,
// which is an order of magnitude longer; every use below feeds a result that is rounded again.
__device__ __forceinline__ float act_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

__device__ __forceinline__ float act_sigmoid(float x) { return act_rcp(1.f + __expf(-x)); }
__device__ __forceinline__ float act_tanh(float x) { return 2.f * act_sigmoid(2.f * x) - 1.f; }

// erf by Abramowitz & Stegun 7.1.26 (absolute error < 1.5e-7): small enough to inline into the
// fully unrolled GEMM epilogue, which the libm erff is not.
__device__ __forceinline__ float act_erf(float x) {
  const float ax = fabsf(x);
  const float t = act_rcp(1.f + 0.3275911f * ax);
  const float poly = ((((1.061405429f * t - 1.453152027f) * t + 1.421413741f) * t - 0.284496736f) * t +
                      0.254829592f) * t;
  return copysignf(1.f - poly * __expf(-ax * ax), x);
}

constexpr float kSeluScale = 1.0507009873554804934193349852946f;
constexpr float kSeluAlpha = 1.6732632423543772848170429916717f;

__device__ __forceinline__ float act_forward(int act, float x, float p) {
  switch (act) {
    case AT_ACT_SIGMOID: return act_sigmoid(x);
    case AT_ACT_LOGSIGMOID: return __logf(act_sigmoid(x));
    case AT_ACT_TANH: return act_tanh(x);
    case AT_ACT_RELU: return fmaxf(0.f, x);
    case AT_ACT_GELU: return 0.5f * (1.f + act_erf(0.707106781f * x)) * x;
    // 0.5 * (1 + tanh(u)) = sigmoid(2u)
    case AT_ACT_GELUAPPROX: {
      // x * sigmoid(2u) with 2u = 1.5957691216 x (1 + 0.044715 x^2), as x / (1 + 2^(-2u log2 e)):
      // the constants folded into one polynomial in front of the exponential (5 plain operations
      // and 2 transcendental ones per element; the epilogue of the large GEMM is bound by them)
      constexpr float k1 = -1.5957691216f * 1.4426950409f, k3 = k1 * 0.044715f;
      return x * act_rcp(1.f + __builtin_amdgcn_exp2f(x * fmaf(k3, x * x, k1)));
    }
    case AT_ACT_SILU: return x * act_sigmoid(x);
    case AT_ACT_RELU6: return fminf(fmaxf(0.f, x), 6.f);
    case AT_ACT_HARDSIGMOID: return fmaxf(0.f, fminf(1.f, x / 6.f + 0.5f));
    case AT_ACT_HARDTANH: return fmaxf(-1.f, fminf(1.f, x));
    case AT_ACT_HARDSWISH: return x * fminf(fmaxf(0.f, x + 3.f), 6.f) / 6.f;
    case AT_ACT_SELU: return kSeluScale * (fmaxf(0.f, x) + fminf(0.f, kSeluAlpha * (__expf(x) - 1.f)));
    case AT_ACT_MISH: return x * act_tanh(__logf(1.f + __expf(x)));
    case AT_ACT_SOFTPLUS: return __logf(1.f + __expf(x));
    case AT_ACT_SOFTSIGN: return x / (1.f + fabsf(x));
    case AT_ACT_TANHSHRINK: return x - act_tanh(x);
    case AT_ACT_LEAKY_RELU: return fmaxf(0.f, x) + p * fminf(0.f, x);
    case AT_ACT_ELU: return x <= 0.f ? p * (__expf(x) - 1.f) : x;
    case AT_ACT_CELU: return fmaxf(0.f, x) + fminf(0.f, p * (__expf(x / p) - 1.f));
    case AT_ACT_HARDSHRINK: return fabsf(x) <= p ? 0.f : x;
    case AT_ACT_SOFTSHRINK: return x > p ? x - p : (x < -p ? x + p : 0.f);
    default: return x;
  }
}

__device__ __forceinline__ float act_derivative(int act, float x, float p) {
  switch (act) {
    case AT_ACT_SIGMOID: { const float s = act_sigmoid(x); return s * (1.f - s); }
    case AT_ACT_LOGSIGMOID: return act_rcp(1.f + __expf(x));
    case AT_ACT_TANH: { const float t = act_tanh(x); return 1.f - t * t; }
    case AT_ACT_RELU: return x <= 0.f ? 0.f : 1.f;
    case AT_ACT_GELU: {
      const float cdf = 0.5f * (1.f + act_erf(0.707106781f * x));
      return 0.39894228f * __expf(-0.5f * x * x) * x + cdf;
    }
    case AT_ACT_GELUAPPROX: {
      // with s = sigmoid(2u), 2u = 1.5957691216 x (1 + 0.044715 x^2): 0.5 (1 + tanh u) = s and
      // 0.5 (1 - tanh^2 u) = 2 s (1 - s), so the derivative is s + x s (1 - s) d(2u)/dx with
      // d(2u)/dx = 1.5957691216 (1 + 3 * 0.044715 x^2); constants folded as in the forward form
      constexpr float k1 = -1.5957691216f * 1.4426950409f, k3 = k1 * 0.044715f;
      constexpr float c1 = 1.5957691216f, c3 = 1.5957691216f * 3.f * 0.044715f;
      const float x2 = x * x;
      const float sg = act_rcp(1.f + __builtin_amdgcn_exp2f(x * fmaf(k3, x2, k1)));
      return fmaf(fmaf(-sg, sg, sg), x * fmaf(c3, x2, c1), sg);
    }
    case AT_ACT_SILU: { const float s = act_sigmoid(x); return s * (x * (1.f - s) + 1.f); }
    case AT_ACT_RELU6: return (0.f < x && x < 6.f) ? 1.f : 0.f;
    case AT_ACT_HARDSIGMOID: return (-3.f < x && x < 3.f) ? (1.f / 6.f) : 0.f;
    case AT_ACT_HARDTANH: return (-1.f < x && x < 1.f) ? 1.f : 0.f;
    case AT_ACT_HARDSWISH: return x < -3.f ? 0.f : (x <= 3.f ? x / 3.f + 0.5f : 1.f);
    case AT_ACT_SELU: return kSeluScale * (x <= 0.f ? kSeluAlpha * __expf(x) : 1.f);
    case AT_ACT_MISH: {
      if (x > 20.f) return 1.f;  // the ratio is 1 to fp32 precision and exp(4x) would overflow
      const float e = __expf(x);
      const float d = e * (e + 2.f) + 2.f;
      return e * (e * ((4.f * x + 6.f) + e * (e + 4.f)) + 4.f * (x + 1.f)) / (d * d);
    }
    case AT_ACT_SOFTPLUS: return act_sigmoid(x);
    case AT_ACT_SOFTSIGN: { const float d = 1.f + fabsf(x); return 1.f / (d * d); }
    case AT_ACT_TANHSHRINK: { const float t = act_tanh(x); return t * t; }
    case AT_ACT_LEAKY_RELU: return x <= 0.f ? p : 1.f;
    case AT_ACT_ELU: return x <= 0.f ? p * __expf(x) : 1.f;
    case AT_ACT_CELU: return x <= 0.f ? __expf(x / p) : 1.f;
    case AT_ACT_HARDSHRINK:
    case AT_ACT_SOFTSHRINK: return fabsf(x) <= p ? 0.f : 1.f;
    default: return 1.f;
  }
}

// Runs the statement(s) with `ACT` a compile-time constant equal to the runtime id: inside, calls
// of act_forward(ACT, ...) / act_derivative(ACT, ...) fold to the one formula, so a loop over many
// elements pays for the choice once instead of once per element.
#define AT_ACT_DISPATCH(ACT_VALUE, ...)                                                               \
  switch (ACT_VALUE) {                                                                                \
    case 0: { constexpr int ACT = 0; __VA_ARGS__; break; }   case 1: { constexpr int ACT = 1; __VA_ARGS__; break; }   \
    case 2: { constexpr int ACT = 2; __VA_ARGS__; break; }   case 3: { constexpr int ACT = 3; __VA_ARGS__; break; }   \
    case 4: { constexpr int ACT = 4; __VA_ARGS__; break; }   case 5: { constexpr int ACT = 5; __VA_ARGS__; break; }   \
    case 6: { constexpr int ACT = 6; __VA_ARGS__; break; }   case 7: { constexpr int ACT = 7; __VA_ARGS__; break; }   \
    case 8: { constexpr int ACT = 8; __VA_ARGS__; break; }   case 9: { constexpr int ACT = 9; __VA_ARGS__; break; }   \
    case 10: { constexpr int ACT = 10; __VA_ARGS__; break; } case 11: { constexpr int ACT = 11; __VA_ARGS__; break; } \
    case 12: { constexpr int ACT = 12; __VA_ARGS__; break; } case 13: { constexpr int ACT = 13; __VA_ARGS__; break; } \
    case 14: { constexpr int ACT = 14; __VA_ARGS__; break; } case 15: { constexpr int ACT = 15; __VA_ARGS__; break; } \
    case 16: { constexpr int ACT = 16; __VA_ARGS__; break; } case 17: { constexpr int ACT = 17; __VA_ARGS__; break; } \
    case 18: { constexpr int ACT = 18; __VA_ARGS__; break; } case 19: { constexpr int ACT = 19; __VA_ARGS__; break; } \
    case 20: { constexpr int ACT = 20; __VA_ARGS__; break; } default: { constexpr int ACT = 21; __VA_ARGS__; break; } \
  }

}  // namespace at_hip
