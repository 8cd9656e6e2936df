// Gated linear unit with an arbitrary activation: the gated dimension is cut in two halves,
//   forward : y = x1 * act(x2)
//   backward: dx1 = dy * act(x2),  dx2 = dy * x1 * act'(x2)
//
// The input is addressed in place as [outer][2][half] (half = elements of one half of the gated
// dimension times everything inside it), so neither the halves nor the two gradients are ever
// copied: the forward pass reads the input once and writes the output once, the backward pass
// reads dy and the input and writes the whole input gradient.  128-bit accesses when `half` is
// a whole number of vectors.
#include <type_traits>

#include "at_act.h"

namespace at_hip {
namespace {

template <typename T, typename IDX, bool BACKWARD, bool VECTOR>
__global__ __launch_bounds__(256) void glu_kernel(const T* __restrict__ input, const T* __restrict__ output_grad,
                                                  T* __restrict__ out, IDX outer, IDX half, int act, float param) {
  constexpr int VEC = VECTOR ? 16 / (int)sizeof(T) : 1;
  const IDX per_row = half / VEC;            // VECTOR: half % VEC == 0
  const IDX n_items = outer * per_row;
  const IDX stride = (IDX)gridDim.x * 256;
  for (IDX item = (IDX)blockIdx.x * 256 + threadIdx.x; item < n_items; item += stride) {
    const IDX o = item / per_row;
    const IDX l = (item - o * per_row) * VEC;
    const T* x1p = input + (o * 2) * half + l;
    float x1[VEC], x2[VEC];
    load_f32<T, VEC>(x1p, x1);
    load_f32<T, VEC>(x1p + half, x2);
    if (!BACKWARD) {
      float y[VEC];
      // the activation's formula is chosen once per vector, not once per element
      AT_ACT_DISPATCH(act, _Pragma("unroll") for (int j = 0; j < VEC; ++j) y[j] = x1[j] * act_forward(ACT, x2[j], param));
      store_f32<T, VEC>(out + o * half + l, y);
    } else {
      float dy[VEC], d1[VEC], d2[VEC];
      load_f32<T, VEC>(output_grad + o * half + l, dy);
      AT_ACT_DISPATCH(act, _Pragma("unroll") for (int j = 0; j < VEC; ++j) {
        d1[j] = dy[j] * act_forward(ACT, x2[j], param);
        d2[j] = dy[j] * x1[j] * act_derivative(ACT, x2[j], param);
      });
      T* g1 = out + (o * 2) * half + l;
      store_f32<T, VEC>(g1, d1);
      store_f32<T, VEC>(g1 + half, d2);
    }
  }
}

template <bool BACKWARD>
int launch(const void* input, const void* output_grad, void* out, int64_t outer, int64_t half, int act, float param,
           int dtype, hipStream_t stream) {
  if (!input || !out || (BACKWARD && !output_grad)) return AT_ERR_NULL;
  if (!dtype_valid(dtype)) return AT_ERR_DTYPE;
  if (!act_valid(act) || act == AT_ACT_NONE) return AT_ERR_ACT;
  if (outer < 0 || half < 0) return AT_ERR_DIM;
  if (outer == 0 || half == 0) return AT_OK;
  const int vec = 16 / dtype_size(dtype);
  const bool vector = half % vec == 0 && aligned16(input) && aligned16(out) && (!BACKWARD || aligned16(output_grad));
  const int64_t items = outer * (vector ? half / vec : half);
  int64_t blocks = cdiv64(items, 256);
  // as a rule one vector per lane and one step per workgroup: short-lived waves keep more bytes
  // in flight than a capped grid whose lanes loop (their next loads queue behind their own stores)
  const int64_t cap = (int64_t)1 << 22;
  if (blocks > cap) blocks = cap;
  const bool small = outer * half * 2 + 16 < ((int64_t)1 << 31);
  auto go = [&](auto* tp, auto idx, auto vflag) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    typedef decltype(idx) IDX;
    hipLaunchKernelGGL((glu_kernel<T, IDX, BACKWARD, decltype(vflag)::value>), dim3((unsigned)blocks), dim3(256), 0,
                       stream, (const T*)input, (const T*)output_grad, (T*)out, (IDX)outer, (IDX)half, act, param);
    return launch_status();
  };
  auto by_type = [&](auto* tp) -> int {
    if (small) return vector ? go(tp, (uint32_t)0, std::true_type()) : go(tp, (uint32_t)0, std::false_type());
    return vector ? go(tp, (int64_t)0, std::true_type()) : go(tp, (int64_t)0, std::false_type());
  };
  if (dtype == AT_DTYPE_F32) return by_type((float*)0);
  if (dtype == AT_DTYPE_F16) return by_type((f16_t*)0);
  return by_type((bf16_t*)0);
}

}  // namespace
}  // namespace at_hip

using namespace at_hip;

extern "C" {

int at_glu_fwd(const void* input, void* output, int64_t outer, int64_t half, int act, float param, int dtype,
               at_stream_t stream) {
  return launch<false>(input, nullptr, output, outer, half, act, param, dtype, (hipStream_t)stream);
}

int at_glu_bwd(const void* output_grad, const void* input, void* input_grad, int64_t outer, int64_t half, int act,
               float param, int dtype, at_stream_t stream) {
  return launch<true>(input, output_grad, input_grad, outer, half, act, param, dtype, (hipStream_t)stream);
}

}  // extern "C"
