// BatchNorm over [N, C, S] tensors (S = flattened spatial extent, 1 for 2D inputs) with fused
// affine, residual add, pre-activation store and activation; forward and backward.
//
// HBM-bound.  The reference gives one program to each channel (C workgroups, a quarter of the
// chip for C = 64); here every pass is spread over C x P workgroups:
//   forward : partial (count, mean, M2) per (channel, split) -> per-channel finalize (Chan
//             merge in fixed order, running-stat EMA) -> elementwise apply
//   backward: partial (sum g, sum g*x_hat) per (channel, split), writing g = dy * act'(z) on
//             the way -> per-channel finalize (weight/bias gradients, coefficients) ->
//             elementwise input gradient
// All cross-workgroup combination goes through small fp32 workspaces and is order-fixed.
#include <type_traits>

#include "at_act.h"
#include "at_common.h"

namespace at_hip {
namespace {

constexpr int kBnBlock = 256;

struct Welford { float n, mean, m2; };

__device__ __forceinline__ Welford wf_merge(const Welford& a, const Welford& b) {
  const float n = a.n + b.n;
  if (n == 0.f) return Welford{0.f, 0.f, 0.f};
  const float d = b.mean - a.mean;
  const float f = b.n / n;
  return Welford{n, a.mean + d * f, a.m2 + b.m2 + d * d * a.n * f};
}

__device__ __forceinline__ Welford wf_block_reduce(Welford v, Welford* smem /* blockDim/64 */) {
  for (int o = 32; o > 0; o >>= 1) {
    Welford other{__shfl_xor(v.n, o, 64), __shfl_xor(v.mean, o, 64), __shfl_xor(v.m2, o, 64)};
    // merge in a lane-symmetric order so both partners compute identical bits
    v = (threadIdx.x & o) ? wf_merge(other, v) : wf_merge(v, other);
  }
  const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) smem[wave] = v;
  __syncthreads();
  Welford r = smem[0];
  for (int i = 1; i < nw; ++i) r = wf_merge(r, smem[i]);
  return r;
}

__device__ __forceinline__ float block_sum(float v, float* smem) {
  return group_reduce(v, (int)blockDim.x, smem, SumOp(), 0.f);
}

// Enumerates the VEC-element chunks of channel c that belong to split p of P and calls
// f(element_offset).  Planes with many chunks are walked plane by plane; small planes are
// flattened so the lanes stay busy.
template <int VEC, typename F>
__device__ __forceinline__ void for_channel_chunks(int c, int p, int P, int64_t N, int C, int S, F&& f) {
  const int sp = S / VEC;  // chunks per plane (S % VEC == 0 on the vector path, VEC == 1 otherwise)
  if (sp >= kBnBlock) {
    for (int64_t n = p; n < N; n += P) {
      const int64_t base = (n * C + c) * (int64_t)S;
      for (int i = threadIdx.x; i < sp; i += kBnBlock) f(base + (int64_t)i * VEC);
    }
  } else {
    const int64_t planes = (N - p + P - 1) / P;  // planes n = p, p + P, ...
    const int64_t total = planes * sp;
    for (int64_t q = threadIdx.x; q < total; q += kBnBlock) {
      const int64_t k = q / sp;
      const int i = (int)(q - k * sp);
      f(((p + k * P) * C + c) * (int64_t)S + (int64_t)i * VEC);
    }
  }
}

template <typename T, int VEC>
__global__ __launch_bounds__(kBnBlock) void bn_stats_kernel(const T* __restrict__ x, float* __restrict__ part,
                                                           int64_t N, int C, int S, int P) {
  __shared__ Welford smem[kBnBlock / 64];
  const int c = blockIdx.x, p = blockIdx.y;
  Welford acc{0.f, 0.f, 0.f};
  for_channel_chunks<VEC>(c, p, P, N, C, S, [&](int64_t off) {
    float v[VEC];
    load_f32<T, VEC>(x + off, v);
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < VEC; ++j) s += v[j];
    const float m = s * (1.0f / VEC);
    float m2 = 0.f;
#pragma unroll
    for (int j = 0; j < VEC; ++j) m2 += (v[j] - m) * (v[j] - m);
    const float n = acc.n + VEC;
    const float d = m - acc.mean;
    const float f = __fdividef((float)VEC, n);
    acc.m2 += m2 + d * d * acc.n * f;
    acc.mean += d * f;
    acc.n = n;
  });
  const Welford r = wf_block_reduce(acc, smem);
  if (threadIdx.x == 0) {
    float* dst = part + ((int64_t)c * P + p) * 3;
    dst[0] = r.n; dst[1] = r.mean; dst[2] = r.m2;
  }
}

// One wave per channel: merges the P partials, derives mean / inv_std, updates the running
// statistics (unbiased variance) and leaves {mean, inv_std} in stat[c].
__global__ __launch_bounds__(64) void bn_stats_finalize_kernel(
    const float* __restrict__ part, int P, float* __restrict__ stat, float* __restrict__ mean_out,
    float* __restrict__ inv_std_out, void* __restrict__ running_mean, void* __restrict__ running_var,
    int rdt, float momentum, float eps) {
  const int c = blockIdx.x;
  Welford acc{0.f, 0.f, 0.f};
  for (int p = threadIdx.x; p < P; p += 64) {
    const float* src = part + ((int64_t)c * P + p) * 3;
    acc = wf_merge(acc, Welford{src[0], src[1], src[2]});
  }
  for (int o = 32; o > 0; o >>= 1) {
    Welford other{__shfl_xor(acc.n, o, 64), __shfl_xor(acc.mean, o, 64), __shfl_xor(acc.m2, o, 64)};
    acc = (threadIdx.x & o) ? wf_merge(other, acc) : wf_merge(acc, other);
  }
  if (threadIdx.x == 0) {
    const float var = acc.m2 / acc.n;
    const float inv_std = rsqrtf(var + eps);
    stat[2 * c] = acc.mean;
    stat[2 * c + 1] = inv_std;
    if (mean_out) mean_out[c] = acc.mean;
    if (inv_std_out) inv_std_out[c] = inv_std;
    if (running_mean && running_var) {
      const float rm = load_scalar_f32(running_mean, rdt, c), rv = load_scalar_f32(running_var, rdt, c);
      store_scalar_f32(running_mean, rdt, c, (1.f - momentum) * rm + momentum * acc.mean);
      store_scalar_f32(running_var, rdt, c, (1.f - momentum) * rv + momentum * var * acc.n / (acc.n - 1.f));
    }
  }
}

__global__ void bn_eval_stats_kernel(const void* __restrict__ running_mean, const void* __restrict__ running_var,
                                     int rdt, float* __restrict__ stat, float* __restrict__ mean_out,
                                     float* __restrict__ inv_std_out, int C, float eps) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const float m = load_scalar_f32(running_mean, rdt, c);
  const float r = rsqrtf(load_scalar_f32(running_var, rdt, c) + eps);
  stat[2 * c] = m;
  stat[2 * c + 1] = r;
  if (mean_out) mean_out[c] = m;
  if (inv_std_out) inv_std_out[c] = r;
}

// y = act(w * (x - mean) * inv_std + b (+ residual)); one workgroup per slice of a plane.
// grid.x = planes (n * C + c), grid.y = slices of the plane.
template <typename T, int VEC, int ACT>
__global__ __launch_bounds__(kBnBlock) void bn_apply_kernel(
    const T* __restrict__ x, const T* __restrict__ res, T* __restrict__ pre_act, T* __restrict__ y,
    const float* __restrict__ stat, const void* __restrict__ w, const void* __restrict__ b, int wdt,
    int C, int S, float param, int64_t total_planes) {
  const int sp = S / VEC;
  for (int64_t plane = blockIdx.x; plane < total_planes; plane += gridDim.x) {
    const int c = (int)(plane % C);
    const float mean = stat[2 * c], inv_std = stat[2 * c + 1];
    const float wt = w ? load_scalar_f32(w, wdt, c) : 1.f;
    const float bs = b ? load_scalar_f32(b, wdt, c) : 0.f;
    const int64_t base = plane * (int64_t)S;
    for (int i = blockIdx.y * kBnBlock + threadIdx.x; i < sp; i += gridDim.y * kBnBlock) {
      const int64_t off = base + (int64_t)i * VEC;
      float v[VEC];
      load_f32<T, VEC>(x + off, v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = wt * (v[j] - mean) * inv_std + bs;
      if (res) {
        float r[VEC];
        load_f32<T, VEC>(res + off, r);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] += r[j];
      }
      if (ACT != AT_ACT_NONE) {
        if (pre_act) store_f32<T, VEC>(pre_act + off, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = act_forward(ACT, v[j], param);
      }
      store_f32<T, VEC>(y + off, v);
    }
  }
}

// Backward partial sums per (channel, split); writes g = dy * act'(pre_act) to g_out when an
// activation is fused (g_out then feeds the apply pass and doubles as the residual gradient).
template <typename T, int VEC, int ACT>
__global__ __launch_bounds__(kBnBlock) void bn_bwd_reduce_kernel(
    const T* __restrict__ dy, const T* __restrict__ pre_act, const T* __restrict__ x, T* __restrict__ g_out,
    const float* __restrict__ mean_in, const float* __restrict__ inv_std_in, float* __restrict__ part,
    int64_t N, int C, int S, int P, float param) {
  __shared__ float smem[16];
  const int c = blockIdx.x, p = blockIdx.y;
  const float mean = mean_in[c], inv_std = inv_std_in[c];
  float s1 = 0.f, s2 = 0.f;
  for_channel_chunks<VEC>(c, p, P, N, C, S, [&](int64_t off) {
    float g[VEC], xv[VEC];
    load_f32<T, VEC>(dy + off, g);
    load_f32<T, VEC>(x + off, xv);
    if (ACT != AT_ACT_NONE) {
      float z[VEC];
      load_f32<T, VEC>(pre_act + off, z);
#pragma unroll
      for (int j = 0; j < VEC; ++j) g[j] *= act_derivative(ACT, z[j], param);
      store_f32<T, VEC>(g_out + off, g);
      // the reference rounds pre_act_grad to the storage dtype before reducing it
#pragma unroll
      for (int j = 0; j < VEC; ++j) g[j] = to_f32(from_f32<T>(g[j]));
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      s1 += g[j] * (xv[j] - mean) * inv_std;
      s2 += g[j];
    }
  });
  s1 = block_sum(s1, smem);
  s2 = block_sum(s2, smem);
  if (threadIdx.x == 0) {
    float* dst = part + ((int64_t)c * P + p) * 2;
    dst[0] = s1; dst[1] = s2;
  }
}

__global__ __launch_bounds__(64) void bn_bwd_finalize_kernel(
    const float* __restrict__ part, int P, const void* __restrict__ w, int wdt, float count,
    float* __restrict__ coef, float* __restrict__ weight_grad, float* __restrict__ bias_grad) {
  const int c = blockIdx.x;
  float s1 = 0.f, s2 = 0.f;
  for (int p = threadIdx.x; p < P; p += 64) {
    s1 += part[((int64_t)c * P + p) * 2];
    s2 += part[((int64_t)c * P + p) * 2 + 1];
  }
  s1 = wave_reduce(s1, 64, SumOp());
  s2 = wave_reduce(s2, 64, SumOp());
  if (threadIdx.x == 0) {
    const float wt = w ? load_scalar_f32(w, wdt, c) : 1.f;
    coef[2 * c] = s1 * wt / count;
    coef[2 * c + 1] = s2 * wt / count;
    if (weight_grad) weight_grad[c] = s1;
    if (bias_grad) bias_grad[c] = s2;
  }
}

template <typename T, int VEC>
__global__ __launch_bounds__(kBnBlock) void bn_bwd_apply_kernel(
    const T* __restrict__ g, const T* __restrict__ x, T* __restrict__ dx, const float* __restrict__ mean_in,
    const float* __restrict__ inv_std_in, const float* __restrict__ coef, const void* __restrict__ w, int wdt,
    int C, int S, int64_t total_planes) {
  const int sp = S / VEC;
  for (int64_t plane = blockIdx.x; plane < total_planes; plane += gridDim.x) {
    const int c = (int)(plane % C);
    const float mean = mean_in[c], inv_std = inv_std_in[c];
    const float t1 = coef[2 * c], t2 = coef[2 * c + 1];
    const float wt = w ? load_scalar_f32(w, wdt, c) : 1.f;
    const int64_t base = plane * (int64_t)S;
    for (int i = blockIdx.y * kBnBlock + threadIdx.x; i < sp; i += gridDim.y * kBnBlock) {
      const int64_t off = base + (int64_t)i * VEC;
      float gv[VEC], xv[VEC];
      load_f32<T, VEC>(g + off, gv);
      load_f32<T, VEC>(x + off, xv);
#pragma unroll
      for (int j = 0; j < VEC; ++j)
        gv[j] = inv_std * (wt * gv[j] - (t1 * (xv[j] - mean) * inv_std + t2));
      store_f32<T, VEC>(dx + off, gv);
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

// Compile-time activation ids for the unrolled element loops; everything goes through one
// switch so each kernel is instantiated once per activation.
#define AT_BN_ACT_SWITCH(ACT_VALUE, ...)                                                              \
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

inline int bn_splits(int64_t N, int C) {
  // aim for ~8 workgroups per CU over the whole grid, at most one split per batch entry
  int64_t want = cdiv64((int64_t)device_cu_count() * 8, C);
  if (want > N) want = N;
  if (want < 1) want = 1;
  if (want > 1024) want = 1024;
  return (int)want;
}

inline void apply_grid(int64_t planes, int S, int vec, dim3* grid) {
  const int sp = S / vec;
  int gy = (int)cdiv64(sp, kBnBlock * 2);
  if (gy < 1) gy = 1;
  if (gy > 64) gy = 64;
  int64_t gx = planes;
  const int64_t cap = (int64_t)device_cu_count() * 64;
  if (gx > cap) gx = cap;
  *grid = dim3((unsigned)gx, (unsigned)gy);
}

constexpr int kMaxSplits = 1024;

}  // namespace
}  // namespace at_hip

using namespace at_hip;

extern "C" {

int64_t at_batch_norm_workspace_bytes(int64_t feat) {
  if (feat <= 0) return 0;
  // partials (3 floats per split) + {mean, inv_std} / coefficient pairs
  return feat * ((int64_t)kMaxSplits * 3 + 4) * (int64_t)sizeof(float);
}

int at_batch_norm_fwd(const void* input, const void* weight, const void* bias, float* mean, float* inv_std,
                      const void* pre_act_add, void* pre_act, void* output, void* running_mean,
                      void* running_var, void* workspace, int64_t workspace_bytes, int64_t batch,
                      int64_t feat, int64_t spatial, float momentum, float eps, int act, float param,
                      int track_running_stats, int is_train, int dtype, int param_dtype, int running_dtype,
                      at_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!input || !output) return AT_ERR_NULL;
  if (!dtype_valid(dtype) || ((weight || bias) && !dtype_valid(param_dtype)) ||
      ((running_mean || running_var) && !dtype_valid(running_dtype)))
    return AT_ERR_DTYPE;
  if (!act_valid(act)) return AT_ERR_ACT;
  if (batch <= 0 || feat <= 0 || spatial <= 0 || feat > INT32_MAX || spatial > INT32_MAX) return AT_ERR_DIM;
  const bool batch_stats = is_train || !track_running_stats;
  if (!batch_stats && (!running_mean || !running_var)) return AT_ERR_NULL;
  if (!workspace || workspace_bytes < at_batch_norm_workspace_bytes(feat)) return AT_ERR_WORKSPACE;
  if (!(weight && bias)) weight = bias = nullptr;  // affine only with both (batch_norm_layer.py:116)
  if (pre_act == output) pre_act = nullptr;

  float* part = (float*)workspace;
  float* stat = part + feat * (int64_t)kMaxSplits * 3;
  const int C = (int)feat, S = (int)spatial;
  const int es = dtype_size(dtype);
  const int vfull = 16 / es;
  const bool vec_ok = S % vfull == 0 && aligned16(input) && aligned16(output) &&
                      (!pre_act_add || aligned16(pre_act_add)) && (!pre_act || aligned16(pre_act));

  return dispatch_dtype(dtype, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    constexpr int VEC = 16 / (int)sizeof(T);
    if (batch_stats) {
      const int P = bn_splits(batch, C);
      if (vec_ok)
        hipLaunchKernelGGL((bn_stats_kernel<T, VEC>), dim3(C, P), dim3(kBnBlock), 0, stream, (const T*)input,
                           part, batch, C, S, P);
      else
        hipLaunchKernelGGL((bn_stats_kernel<T, 1>), dim3(C, P), dim3(kBnBlock), 0, stream, (const T*)input,
                           part, batch, C, S, P);
      const bool update = track_running_stats && is_train && running_mean && running_var;
      hipLaunchKernelGGL(bn_stats_finalize_kernel, dim3(C), dim3(64), 0, stream, part, P, stat, mean, inv_std,
                         update ? running_mean : nullptr, update ? running_var : nullptr, running_dtype,
                         momentum, eps);
    } else {
      hipLaunchKernelGGL(bn_eval_stats_kernel, dim3((unsigned)cdiv64(C, 256)), dim3(256), 0, stream,
                         running_mean, running_var, running_dtype, stat, mean, inv_std, C, eps);
    }
    dim3 grid;
    const int64_t planes = batch * feat;
    apply_grid(planes, S, vec_ok ? VEC : 1, &grid);
    if (vec_ok) {
      AT_BN_ACT_SWITCH(act, hipLaunchKernelGGL((bn_apply_kernel<T, VEC, ACT>), grid, dim3(kBnBlock), 0, stream,
                                               (const T*)input, (const T*)pre_act_add, (T*)pre_act, (T*)output,
                                               stat, weight, bias, param_dtype, C, S, param, planes));
    } else {
      AT_BN_ACT_SWITCH(act, hipLaunchKernelGGL((bn_apply_kernel<T, 1, ACT>), grid, dim3(kBnBlock), 0, stream,
                                               (const T*)input, (const T*)pre_act_add, (T*)pre_act, (T*)output,
                                               stat, weight, bias, param_dtype, C, S, param, planes));
    }
    return launch_status();
  });
}

int at_batch_norm_bwd(const void* output_grad, const void* pre_act, const void* input, const float* mean,
                      const float* inv_std, const void* weight, void* input_grad, void* pre_act_grad,
                      float* weight_grad, float* bias_grad, void* workspace, int64_t workspace_bytes,
                      int64_t batch, int64_t feat, int64_t spatial, int act, float param, int dtype,
                      int param_dtype, at_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!output_grad || !input || !mean || !inv_std || !input_grad) return AT_ERR_NULL;
  if (!dtype_valid(dtype) || (weight && !dtype_valid(param_dtype))) return AT_ERR_DTYPE;
  if (!act_valid(act)) return AT_ERR_ACT;
  if (act != AT_ACT_NONE && (!pre_act || !pre_act_grad)) return AT_ERR_NULL;
  if (batch <= 0 || feat <= 0 || spatial <= 0 || feat > INT32_MAX || spatial > INT32_MAX) return AT_ERR_DIM;
  if (!workspace || workspace_bytes < at_batch_norm_workspace_bytes(feat)) return AT_ERR_WORKSPACE;

  float* part = (float*)workspace;
  float* coef = part + feat * (int64_t)kMaxSplits * 3;
  const int C = (int)feat, S = (int)spatial;
  const int vfull = 16 / dtype_size(dtype);
  const bool vec_ok = S % vfull == 0 && aligned16(output_grad) && aligned16(input) && aligned16(input_grad) &&
                      (!pre_act || aligned16(pre_act)) && (!pre_act_grad || aligned16(pre_act_grad));
  const void* g_for_apply = act != AT_ACT_NONE ? pre_act_grad : output_grad;

  return dispatch_dtype(dtype, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    constexpr int VEC = 16 / (int)sizeof(T);
    const int P = bn_splits(batch, C);
    if (vec_ok) {
      AT_BN_ACT_SWITCH(act, hipLaunchKernelGGL((bn_bwd_reduce_kernel<T, VEC, ACT>), dim3(C, P), dim3(kBnBlock), 0,
                                               stream, (const T*)output_grad, (const T*)pre_act, (const T*)input,
                                               (T*)pre_act_grad, mean, inv_std, part, batch, C, S, P, param));
    } else {
      AT_BN_ACT_SWITCH(act, hipLaunchKernelGGL((bn_bwd_reduce_kernel<T, 1, ACT>), dim3(C, P), dim3(kBnBlock), 0,
                                               stream, (const T*)output_grad, (const T*)pre_act, (const T*)input,
                                               (T*)pre_act_grad, mean, inv_std, part, batch, C, S, P, param));
    }
    hipLaunchKernelGGL(bn_bwd_finalize_kernel, dim3(C), dim3(64), 0, stream, part, P, weight, param_dtype,
                       (float)(batch * spatial), coef, weight_grad, bias_grad);
    dim3 grid;
    const int64_t planes = batch * feat;
    apply_grid(planes, S, vec_ok ? VEC : 1, &grid);
    if (vec_ok)
      hipLaunchKernelGGL((bn_bwd_apply_kernel<T, VEC>), grid, dim3(kBnBlock), 0, stream, (const T*)g_for_apply,
                         (const T*)input, (T*)input_grad, mean, inv_std, coef, weight, param_dtype, C, S, planes);
    else
      hipLaunchKernelGGL((bn_bwd_apply_kernel<T, 1>), grid, dim3(kBnBlock), 0, stream, (const T*)g_for_apply,
                         (const T*)input, (T*)input_grad, mean, inv_std, coef, weight, param_dtype, C, S, planes);
    return launch_status();
  });
}

}  // extern "C"
