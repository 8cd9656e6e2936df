// Elementwise regression losses of d = input - target, reductions none / mean / sum:
//   AT_P_LOSS_SMOOTH_L1: |d| < beta ? d^2 / (2 beta) : |d| - beta / 2
//   AT_P_LOSS_L1       : |d|
//   AT_P_LOSS_MSE      : d^2
//   AT_P_LOSS_HUBER    : |d| < delta ? d^2 / 2 : delta (|d| - delta / 2)
// and their gradients with respect to input (the target's is the negative).  One read of both
// tensors forward; the reductions add per-workgroup partial sums in a fixed order.
#include <type_traits>

#include "at_common.h"

namespace at_hip {
namespace {

constexpr int kLossBlock = 256;
constexpr int kLossMaxBlocks = 2048;

__device__ __forceinline__ float p_loss_value(int kind, float d, float param) {
  const float a = fabsf(d);
  switch (kind) {
    case AT_P_LOSS_SMOOTH_L1: return a < param ? 0.5f * d * d / param : a - 0.5f * param;
    case AT_P_LOSS_L1: return a;
    case AT_P_LOSS_MSE: return d * d;
    default: return a < param ? 0.5f * d * d : param * (a - 0.5f * param);
  }
}

// d(loss)/d(input); the sign at d == 0 is +1, as in the reference (tl.where(0 <= diff, 1, -1)).
__device__ __forceinline__ float p_loss_slope(int kind, float d, float param) {
  const float sign = 0.f <= d ? 1.f : -1.f;
  switch (kind) {
    case AT_P_LOSS_SMOOTH_L1: return fabsf(d) < param ? d / param : sign;
    case AT_P_LOSS_L1: return sign;
    case AT_P_LOSS_MSE: return 2.f * d;
    default: return fabsf(d) < param ? d : param * sign;
  }
}

template <typename T, typename TO, bool VECTOR>
__global__ __launch_bounds__(kLossBlock) void p_loss_fwd_kernel(
    const T* __restrict__ input, const T* __restrict__ target, TO* __restrict__ output, float* __restrict__ part,
    int64_t size, int kind, float param, bool reduce) {
  constexpr int VEC = VECTOR ? 16 / (int)sizeof(T) : 1;
  __shared__ float scratch[kLossBlock / kWave];
  const int64_t n_vec = VECTOR ? size / VEC : size;
  const int64_t stride = (int64_t)gridDim.x * kLossBlock;
  float sum = 0.f;
  for (int64_t v = (int64_t)blockIdx.x * kLossBlock + threadIdx.x; v < n_vec; v += stride) {
    float x[VEC], t[VEC], e[VEC];
    load_f32<T, VEC>(input + v * VEC, x);
    load_f32<T, VEC>(target + v * VEC, t);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      e[j] = p_loss_value(kind, x[j] - t[j], param);
      sum += e[j];
    }
    if (!reduce) store_f32<TO, VEC>(output + v * VEC, e);
  }
  if (VECTOR) {
    const int64_t e0 = n_vec * VEC + (int64_t)blockIdx.x * kLossBlock + threadIdx.x;   // tail: one lane each
    if (e0 < size) {
      const float e = p_loss_value(kind, to_f32(input[e0]) - to_f32(target[e0]), param);
      sum += e;
      if (!reduce) output[e0] = from_f32<TO>(e);
    }
  }
  if (!reduce) return;
  sum = group_reduce(sum, kLossBlock, scratch, SumOp(), 0.f);
  if (threadIdx.x == 0) part[blockIdx.x] = sum;
}

template <typename TO>
__global__ __launch_bounds__(kLossBlock) void p_loss_finish_kernel(const float* __restrict__ part, int parts,
                                                                   TO* __restrict__ output, float scale) {
  __shared__ float scratch[kLossBlock / kWave];
  float sum = 0.f;
  for (int i = threadIdx.x; i < parts; i += kLossBlock) sum += part[i];
  sum = group_reduce(sum, kLossBlock, scratch, SumOp(), 0.f);
  if (threadIdx.x == 0) output[0] = from_f32<TO>(sum * scale);
}

template <typename T, typename TG, typename TO, bool VECTOR>
__global__ __launch_bounds__(kLossBlock) void p_loss_bwd_kernel(
    const TG* __restrict__ output_grad, const T* __restrict__ input, const T* __restrict__ target,
    TO* __restrict__ input_grad, TO* __restrict__ target_grad, int64_t size, int kind, float param, bool reduced,
    float scale) {
  constexpr int VEC = VECTOR ? 16 / (int)sizeof(T) : 1;
  const int64_t n_vec = VECTOR ? size / VEC : size;
  const int64_t stride = (int64_t)gridDim.x * kLossBlock;
  const float upstream = reduced ? to_f32(output_grad[0]) * scale : scale;
  auto one = [&](int64_t e) {
    float g = p_loss_slope(kind, to_f32(input[e]) - to_f32(target[e]), param) * upstream;
    if (!reduced) g *= to_f32(output_grad[e]);
    if (input_grad) input_grad[e] = from_f32<TO>(g);
    if (target_grad) target_grad[e] = from_f32<TO>(-g);
  };
  for (int64_t v = (int64_t)blockIdx.x * kLossBlock + threadIdx.x; v < n_vec; v += stride) {
    if (!VECTOR) { one(v); continue; }
    float x[VEC], t[VEC], dy[VEC], g[VEC], ng[VEC];
    load_f32<T, VEC>(input + v * VEC, x);
    load_f32<T, VEC>(target + v * VEC, t);
    if (!reduced) load_f32<TG, VEC>(output_grad + v * VEC, dy);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      g[j] = p_loss_slope(kind, x[j] - t[j], param) * upstream;
      if (!reduced) g[j] *= dy[j];
      ng[j] = -g[j];
    }
    if (input_grad) store_f32<TO, VEC>(input_grad + v * VEC, g);
    if (target_grad) store_f32<TO, VEC>(target_grad + v * VEC, ng);
  }
  if (VECTOR) {
    const int64_t e0 = n_vec * VEC + (int64_t)blockIdx.x * kLossBlock + threadIdx.x;
    if (e0 < size) one(e0);
  }
}

template <typename F>
inline int dispatch_dtype(int dt, F&& f) {
  if (dt == AT_DTYPE_F32) return f((float*)0);
  if (dt == AT_DTYPE_F16) return f((f16_t*)0);
  if (dt == AT_DTYPE_BF16) return f((bf16_t*)0);
  return AT_ERR_DTYPE;
}

inline bool kind_valid(int k) { return k >= AT_P_LOSS_SMOOTH_L1 && k <= AT_P_LOSS_HUBER; }
inline bool reduction_valid(int r) {
  return r == AT_REDUCTION_NONE || r == AT_REDUCTION_MEAN || r == AT_REDUCTION_SUM;
}

inline int grid_blocks(int64_t size, int vec) {
  int64_t blocks = cdiv64(cdiv64(size, vec), kLossBlock);
  if (blocks > kLossMaxBlocks) blocks = kLossMaxBlocks;
  return (int)(blocks < 1 ? 1 : blocks);
}

}  // namespace
}  // namespace at_hip

using namespace at_hip;

extern "C" {

int64_t at_p_loss_workspace_bytes(int64_t size) {
  if (size <= 0) return 0;
  return (int64_t)kLossMaxBlocks * (int64_t)sizeof(float);
}

int at_p_loss_fwd(const void* input, const void* target, void* output, void* workspace, int64_t workspace_bytes,
                  int64_t size, int p_loss, int reduction, float param, int in_dtype, int out_dtype,
                  at_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!input || !target || !output) return AT_ERR_NULL;
  if (!dtype_valid(in_dtype) || !dtype_valid(out_dtype)) return AT_ERR_DTYPE;
  if (!kind_valid(p_loss) || !reduction_valid(reduction)) return AT_ERR_UNSUPPORTED;
  if (size <= 0) return AT_ERR_DIM;
  const bool reduce = reduction != AT_REDUCTION_NONE;
  if (reduce) {
    if (!workspace || workspace_bytes < at_p_loss_workspace_bytes(size)) return AT_ERR_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(workspace) & 3u) != 0) return AT_ERR_ALIGN;
  }
  const int vec = 16 / dtype_size(in_dtype);
  const bool vector = aligned16(input) && aligned16(target) && (reduce || aligned16(output));
  const int blocks = grid_blocks(size, vector ? vec : 1);
  return dispatch_dtype(in_dtype, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    return dispatch_dtype(out_dtype, [&](auto* op) -> int {
      typedef std::remove_pointer_t<decltype(op)> TO;
      if (vector)
        hipLaunchKernelGGL((p_loss_fwd_kernel<T, TO, true>), dim3(blocks), dim3(kLossBlock), 0, stream,
                           (const T*)input, (const T*)target, (TO*)output, (float*)workspace, size, p_loss, param,
                           reduce);
      else
        hipLaunchKernelGGL((p_loss_fwd_kernel<T, TO, false>), dim3(blocks), dim3(kLossBlock), 0, stream,
                           (const T*)input, (const T*)target, (TO*)output, (float*)workspace, size, p_loss, param,
                           reduce);
      int rc = launch_status();
      if (rc || !reduce) return rc;
      const float scale = reduction == AT_REDUCTION_MEAN ? 1.0f / (float)size : 1.0f;
      hipLaunchKernelGGL((p_loss_finish_kernel<TO>), dim3(1), dim3(kLossBlock), 0, stream,
                         (const float*)workspace, blocks, (TO*)output, scale);
      return launch_status();
    });
  });
}

int at_p_loss_bwd(const void* output_grad, const void* input, const void* target, void* input_grad,
                  void* target_grad, int64_t size, int p_loss, int reduction, float param, int in_dtype,
                  int grad_dtype, int out_dtype, at_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!output_grad || !input || !target || (!input_grad && !target_grad)) return AT_ERR_NULL;
  if (!dtype_valid(in_dtype) || !dtype_valid(grad_dtype) || !dtype_valid(out_dtype)) return AT_ERR_DTYPE;
  if (!kind_valid(p_loss) || !reduction_valid(reduction)) return AT_ERR_UNSUPPORTED;
  if (size <= 0) return AT_ERR_DIM;
  const int vec = 16 / dtype_size(in_dtype);
  const bool reduced = reduction != AT_REDUCTION_NONE;
  const bool vector = aligned16(input) && aligned16(target) && (!input_grad || aligned16(input_grad)) &&
                      (!target_grad || aligned16(target_grad)) && (reduced || aligned16(output_grad));
  int64_t blocks = cdiv64(cdiv64(size, vector ? vec : 1), kLossBlock);
  const int64_t cap = (int64_t)device_cu_count() * 16;
  if (blocks > cap) blocks = cap;
  const float scale = reduction == AT_REDUCTION_MEAN ? 1.0f / (float)size : 1.0f;
  return dispatch_dtype(in_dtype, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    return dispatch_dtype(grad_dtype, [&](auto* gp) -> int {
      typedef std::remove_pointer_t<decltype(gp)> TG;
      return dispatch_dtype(out_dtype, [&](auto* op) -> int {
        typedef std::remove_pointer_t<decltype(op)> TO;
        if (vector)
          hipLaunchKernelGGL((p_loss_bwd_kernel<T, TG, TO, true>), dim3((unsigned)blocks), dim3(kLossBlock), 0, stream,
                             (const TG*)output_grad, (const T*)input, (const T*)target, (TO*)input_grad,
                             (TO*)target_grad, size, p_loss, param, reduced, scale);
        else
          hipLaunchKernelGGL((p_loss_bwd_kernel<T, TG, TO, false>), dim3((unsigned)blocks), dim3(kLossBlock), 0, stream,
                             (const TG*)output_grad, (const T*)input, (const T*)target, (TO*)input_grad,
                             (TO*)target_grad, size, p_loss, param, reduced, scale);
        return launch_status();
      });
    });
  });
}

}  // extern "C"
