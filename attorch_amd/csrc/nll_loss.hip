// Negative log likelihood loss over log-probabilities [batch, feat, spatial] with integer
// targets [batch, spatial], optional class weights, reductions none / mean / sum.
//
//   forward : l[b, s] = -w[t] * x[b, t, s],  t = target[b, s]     (w = 1 without weights)
//             none: l;  sum: sum(l);  mean: sum(l) / sum(w[t])  (= sum(l) / (batch * spatial) unweighted)
//   backward: dx[b, c, s] = -dy * w[c] / denominator  where c == target[b, s], 0 elsewhere
//
// The forward pass gathers one element per (b, s) and is tiny; the backward pass writes the
// whole gradient once (zeros included, no separate memset), so it runs at the write bandwidth
// of HBM.  Partial sums are added in a fixed order (no floating-point atomics).  A target
// outside [0, feat) contributes neither loss, weight nor gradient.
#include <type_traits>

#include "at_common.h"

namespace at_hip {
namespace {

constexpr int kNllBlock = 256;
constexpr int kNllMaxBlocks = 1024;   // partial sums of the forward pass

// reduction != none: part[block] = (sum of losses, sum of weights) of the block's elements.
template <typename T>
__global__ __launch_bounds__(kNllBlock) void nll_fwd_kernel(
    const T* __restrict__ input, const int64_t* __restrict__ target, const void* __restrict__ weight, int wdt,
    void* __restrict__ output, int out_dt, float2* __restrict__ part, int64_t batch, int feat, int64_t spatial,
    int reduction) {
  __shared__ float scratch[kNllBlock / kWave];
  const int64_t total = batch * spatial;
  float loss_sum = 0.f, weight_sum = 0.f;
  for (int64_t e = (int64_t)blockIdx.x * kNllBlock + threadIdx.x; e < total; e += (int64_t)gridDim.x * kNllBlock) {
    const int64_t b = e / spatial, s = e - b * spatial;
    const int64_t t = target[e];
    float loss = 0.f, w = 0.f;
    if (t >= 0 && t < feat) {
      w = weight ? load_scalar_f32(weight, wdt, t) : 1.f;
      loss = -to_f32(input[(b * feat + t) * spatial + s]) * w;
    }
    if (reduction == AT_REDUCTION_NONE) store_scalar_f32(output, out_dt, e, loss);
    loss_sum += loss;
    weight_sum += w;
  }
  if (reduction == AT_REDUCTION_NONE) return;
  loss_sum = group_reduce(loss_sum, kNllBlock, scratch, SumOp(), 0.f);
  weight_sum = group_reduce(weight_sum, kNllBlock, scratch, SumOp(), 0.f);
  if (threadIdx.x == 0) part[blockIdx.x] = make_float2(loss_sum, weight_sum);
}

__global__ __launch_bounds__(kNllBlock) void nll_finish_kernel(
    const float2* __restrict__ part, int parts, void* __restrict__ output, int out_dt,
    float* __restrict__ sum_weights, int reduction, bool weighted, float count) {
  __shared__ float scratch[kNllBlock / kWave];
  float loss_sum = 0.f, weight_sum = 0.f;
  for (int i = threadIdx.x; i < parts; i += kNllBlock) {
    loss_sum += part[i].x;
    weight_sum += part[i].y;
  }
  loss_sum = group_reduce(loss_sum, kNllBlock, scratch, SumOp(), 0.f);
  weight_sum = group_reduce(weight_sum, kNllBlock, scratch, SumOp(), 0.f);
  if (threadIdx.x != 0) return;
  float result = loss_sum;
  if (reduction == AT_REDUCTION_MEAN) result = weighted ? loss_sum / weight_sum : loss_sum / count;
  store_scalar_f32(output, out_dt, 0, result);
  if (sum_weights) sum_weights[0] = weight_sum;
}

// One lane per 16-byte vector of the gradient, walked through the flat [batch][feat][spatial]
// index with carries; the target is re-read only when (b, s) changes.
template <typename TG, typename TO>
__global__ __launch_bounds__(kNllBlock) void nll_bwd_kernel(
    const TG* __restrict__ output_grad, const int64_t* __restrict__ target, const void* __restrict__ weight, int wdt,
    const float* __restrict__ sum_weights, TO* __restrict__ input_grad, int64_t batch, int feat, int64_t spatial,
    int reduction, float inv_count, bool vector_ok) {
  constexpr int VEC = 16 / (int)sizeof(TO);
  const int64_t total = batch * feat * spatial;
  float scale = -1.f;
  if (reduction == AT_REDUCTION_MEAN) scale = weight ? -1.f / sum_weights[0] : -inv_count;
  if (reduction != AT_REDUCTION_NONE) scale *= to_f32(output_grad[0]);
  const int64_t n_vec = (total + VEC - 1) / VEC;
  for (int64_t v = (int64_t)blockIdx.x * kNllBlock + threadIdx.x; v < n_vec; v += (int64_t)gridDim.x * kNllBlock) {
    const int64_t f0 = v * VEC;
    int64_t b = f0 / (feat * spatial);
    const int64_t r = f0 - b * feat * spatial;
    int c = (int)(r / spatial);
    int64_t s = r - (int64_t)c * spatial;
    float g[VEC];
    int64_t t = -1;
    bool have = false;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      g[j] = 0.f;
      if (f0 + j < total) {
        if (!have || spatial != 1) t = target[b * spatial + s];
        have = true;
        if (t == c) {
          float coef = scale;
          if (reduction == AT_REDUCTION_NONE) coef *= to_f32(output_grad[b * spatial + s]);
          if (weight) coef *= load_scalar_f32(weight, wdt, c);
          g[j] = coef;
        }
        if (++s == spatial) {
          s = 0;
          if (++c == feat) { c = 0; ++b; have = false; }
        }
      }
    }
    if (vector_ok && f0 + VEC <= total) {
      store_f32<TO, VEC>(input_grad + f0, g);
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j)
        if (f0 + j < total) input_grad[f0 + j] = from_f32<TO>(g[j]);
    }
  }
}

// spatial == 1 (a [batch, feat] matrix): the gradient is zero except at flat position
// row * feat + target[row] of every row.  A workgroup owns one 16 KB piece of the flat gradient:
// it clears the piece in LDS, the rows that overlap it (found with two divisions per workgroup,
// not one per vector) drop their value into it, and the piece leaves as whole 16-byte vectors.
// Every byte of the gradient is written exactly once (no memset, no second launch), and the
// per-vector work is a few instructions, so the pass runs at the speed of a plain fill.
constexpr int kNllTileBytes = 16384;
template <typename TG, typename TO>
__global__ __launch_bounds__(kNllBlock) void nll_bwd_rows_kernel(
    const TG* __restrict__ output_grad, const int64_t* __restrict__ target, const void* __restrict__ weight, int wdt,
    const float* __restrict__ sum_weights, TO* __restrict__ input_grad, int64_t batch, int64_t feat, int reduction,
    float inv_count) {
  constexpr int VEC = 16 / (int)sizeof(TO);
  constexpr int kTileElems = kNllTileBytes / (int)sizeof(TO);
  constexpr int kVecPerLane = kNllTileBytes / 16 / kNllBlock;
  __shared__ __attribute__((aligned(16))) TO tile[kTileElems];
  const int64_t total = batch * feat;
  float scale = -1.f;
  if (reduction == AT_REDUCTION_MEAN) scale = weight ? -1.f / sum_weights[0] : -inv_count;
  if (reduction != AT_REDUCTION_NONE) scale *= to_f32(output_grad[0]);
  for (int64_t e0 = (int64_t)blockIdx.x * kTileElems; e0 < total; e0 += (int64_t)gridDim.x * kTileElems) {
    const int64_t e1 = e0 + kTileElems < total ? e0 + kTileElems : total;
    // 32-bit division whenever the tensor allows it
    int64_t row_lo, row_hi;
    if (total <= (int64_t)UINT32_MAX) {
      row_lo = (uint32_t)e0 / (uint32_t)feat;
      row_hi = (uint32_t)(e1 - 1) / (uint32_t)feat;
    } else {
      row_lo = e0 / feat;
      row_hi = (e1 - 1) / feat;
    }
#pragma unroll
    for (int i = 0; i < kVecPerLane; ++i)
      reinterpret_cast<uint4*>(tile)[threadIdx.x + i * kNllBlock] = make_uint4(0u, 0u, 0u, 0u);
    __syncthreads();
    for (int64_t r = row_lo + threadIdx.x; r <= row_hi; r += kNllBlock) {
      const int64_t t = target[r];
      if (t < 0 || t >= feat) continue;
      const int64_t pos = r * feat + t;
      if (pos < e0 || pos >= e1) continue;
      float coef = scale;
      if (reduction == AT_REDUCTION_NONE) coef *= to_f32(output_grad[r]);
      if (weight) coef *= load_scalar_f32(weight, wdt, t);
      tile[pos - e0] = from_f32<TO>(coef);
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kVecPerLane; ++i) {
      const int v = threadIdx.x + i * kNllBlock;
      const int64_t f0 = e0 + (int64_t)v * VEC;
      if (f0 + VEC <= total) {
        reinterpret_cast<uint4*>(input_grad + e0)[v] = reinterpret_cast<const uint4*>(tile)[v];
      } else {
        for (int j = 0; j < VEC; ++j)
          if (f0 + j < total) input_grad[f0 + j] = tile[v * VEC + j];
      }
    }
    __syncthreads();   // the piece has left before the next one is cleared
  }
}

template <typename F>
inline int dispatch_dtype(int dt, F&& f) {
  if (dt == AT_DTYPE_F32) return f((float*)0);
  if (dt == AT_DTYPE_F16) return f((f16_t*)0);
  if (dt == AT_DTYPE_BF16) return f((bf16_t*)0);
  return AT_ERR_DTYPE;
}

inline bool reduction_valid(int r) {
  return r == AT_REDUCTION_NONE || r == AT_REDUCTION_MEAN || r == AT_REDUCTION_SUM;
}

inline int forward_blocks(int64_t total) {
  const int64_t blocks = cdiv64(total, kNllBlock);
  return (int)(blocks < kNllMaxBlocks ? blocks : kNllMaxBlocks);
}

}  // namespace
}  // namespace at_hip

using namespace at_hip;

extern "C" {

int64_t at_nll_loss_workspace_bytes(int64_t batch, int64_t spatial) {
  if (batch <= 0 || spatial <= 0) return 0;
  return (int64_t)kNllMaxBlocks * (int64_t)sizeof(float2);
}

int at_nll_loss_fwd(const void* input, const int64_t* target, const void* weight, void* output,
                    float* sum_weights, void* workspace, int64_t workspace_bytes, int64_t batch, int64_t feat,
                    int64_t spatial, int reduction, int in_dtype, int weight_dtype, int out_dtype,
                    at_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!input || !target || !output) return AT_ERR_NULL;
  if (!dtype_valid(in_dtype) || !dtype_valid(out_dtype) || (weight && !dtype_valid(weight_dtype)))
    return AT_ERR_DTYPE;
  if (!reduction_valid(reduction)) return AT_ERR_UNSUPPORTED;
  if (batch <= 0 || feat <= 0 || spatial <= 0 || feat > ((int64_t)1 << 30)) return AT_ERR_DIM;
  if (reduction != AT_REDUCTION_NONE) {
    if (!workspace || workspace_bytes < at_nll_loss_workspace_bytes(batch, spatial)) return AT_ERR_WORKSPACE;
    if ((reinterpret_cast<uintptr_t>(workspace) & 7u) != 0) return AT_ERR_ALIGN;
  }
  const int blocks = forward_blocks(batch * spatial);
  int rc = dispatch_dtype(in_dtype, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    hipLaunchKernelGGL((nll_fwd_kernel<T>), dim3(blocks), dim3(kNllBlock), 0, stream, (const T*)input, target,
                       weight, weight_dtype, output, out_dtype, (float2*)workspace, batch, (int)feat, spatial,
                       reduction);
    return launch_status();
  });
  if (rc || reduction == AT_REDUCTION_NONE) return rc;
  hipLaunchKernelGGL(nll_finish_kernel, dim3(1), dim3(kNllBlock), 0, stream, (const float2*)workspace, blocks,
                     output, out_dtype, sum_weights, reduction, weight != nullptr, (float)(batch * spatial));
  return launch_status();
}

int at_nll_loss_bwd(const void* output_grad, const int64_t* target, const void* weight, const float* sum_weights,
                    void* input_grad, int64_t batch, int64_t feat, int64_t spatial, int reduction,
                    int grad_dtype, int weight_dtype, int out_dtype, at_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!output_grad || !target || !input_grad) return AT_ERR_NULL;
  if (!dtype_valid(grad_dtype) || !dtype_valid(out_dtype) || (weight && !dtype_valid(weight_dtype)))
    return AT_ERR_DTYPE;
  if (!reduction_valid(reduction)) return AT_ERR_UNSUPPORTED;
  if (batch <= 0 || feat <= 0 || spatial <= 0 || feat > ((int64_t)1 << 30)) return AT_ERR_DIM;
  if (reduction == AT_REDUCTION_MEAN && weight && !sum_weights) return AT_ERR_NULL;
  const int64_t total = batch * feat * spatial;
  const int64_t n_vec = cdiv64(total, 16 / dtype_size(out_dtype));
  int64_t blocks = cdiv64(n_vec, kNllBlock);
  // as a rule one step per workgroup: short-lived waves keep more bytes in flight than a capped
  // grid whose lanes loop (their next loads queue behind their own stores)
  const int64_t cap = (int64_t)1 << 22;
  if (blocks > cap) blocks = cap;
  const float inv_count = 1.0f / (float)(batch * spatial);
  const bool vector_ok = aligned16(input_grad);
  return dispatch_dtype(grad_dtype, [&](auto* gp) -> int {
    typedef std::remove_pointer_t<decltype(gp)> TG;
    return dispatch_dtype(out_dtype, [&](auto* op) -> int {
      typedef std::remove_pointer_t<decltype(op)> TO;
      if (spatial == 1 && vector_ok) {
        int64_t tiles = cdiv64(total * (int64_t)sizeof(TO), kNllTileBytes);
        if (tiles > cap) tiles = cap;
        hipLaunchKernelGGL((nll_bwd_rows_kernel<TG, TO>), dim3((unsigned)tiles), dim3(kNllBlock), 0, stream,
                           (const TG*)output_grad, target, weight, weight_dtype, sum_weights, (TO*)input_grad, batch,
                           feat, reduction, inv_count);
        return launch_status();
      }
      hipLaunchKernelGGL((nll_bwd_kernel<TG, TO>), dim3((unsigned)blocks), dim3(kNllBlock), 0, stream,
                         (const TG*)output_grad, target, weight, weight_dtype, sum_weights, (TO*)input_grad, batch,
                         (int)feat, spatial, reduction, inv_count, vector_ok);
      return launch_status();
    });
  });
}

}  // extern "C"
