// BatchNorm over [N, C, S] tensors (S = flattened spatial extent, 1 for 2D inputs) with fused
// affine, residual add, pre-activation store and activation; forward and backward.
//
// HBM-bound.  The reference gives one program to each channel (C workgroups, a quarter of the
// chip for C = 64); here every pass is spread over C x P workgroups:
//   forward : partial (count, mean, M2) per (channel, split) -> elementwise apply
//   backward: partial (sum g, sum g*x_hat) per (channel, split), writing g = dy * act'(z) on
//             the way -> elementwise input gradient
// Two launches per direction: every workgroup of an apply pass merges the partials of its
// channel itself (a few dozen values, in a fixed order, so all of them get the same bits), and
// the workgroup that owns the channel's first plane also writes the per-channel outputs
// (statistics, running-statistics update, weight / bias gradients).  Each lane keeps several
// independent 16-byte loads in flight: these passes are bound by memory latency otherwise.
// All cross-workgroup combination goes through small fp32 workspaces and is order-fixed.
#include <type_traits>

#include "at_act.h"
#include "at_common.h"

namespace at_hip {
namespace {

constexpr int kBnBlock = 256;
constexpr int kBnBwdBatch = 4;   // chunks per lane whose loads the backward reduce pass issues together

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

// Tensors below this size are read through buffer addressing by the passes that sum over a channel.
constexpr int64_t kBufferedBytes = (int64_t)1 << 31;

// Raw 16-byte (or narrower) image of VEC elements, widened on use: loads are issued into these
// so that nothing has to wait before the next load is issued.
template <typename T, int VEC>
struct RawVec {
  typename raw_vec<(int)sizeof(T) * VEC>::type r;
  __device__ __forceinline__ void load(const T* p) { r = *reinterpret_cast<const decltype(r)*>(p); }
  // Through a buffer resource (16-byte chunks of a tensor below 2 GiB): a chunk that does not
  // exist is asked for past the end of the buffer, which yields zeros and no request to memory.
  __device__ __forceinline__ void load(const __amdgpu_buffer_rsrc_t& rs, int64_t element_offset, bool exists) {
    static_assert(sizeof(T) * VEC == 16, "whole 16-byte chunks");
    const int byte_offset = exists ? (int)(element_offset * (int64_t)sizeof(T)) : (int)0x80000000u;
    r = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rs, byte_offset, 0, 0));
  }
  __device__ __forceinline__ void get(float (&f)[VEC]) const {
    union { decltype(r) raw; T e[VEC]; } u;
    u.raw = r;
#pragma unroll
    for (int j = 0; j < VEC; ++j) f[j] = to_f32(u.e[j]);
  }
};

// Buffer resource over a whole [N, C, S] tensor for the kernels instantiated with BUF (the host
// picks them for tensors below 2 GiB); an empty one otherwise.
template <bool BUF, typename T>
__device__ __forceinline__ __amdgpu_buffer_rsrc_t tensor_rsrc(const T* base, int64_t N, int C, int S) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(base), 0,
                                           BUF ? (int)(N * C * (int64_t)S * (int64_t)sizeof(T)) : 0, 0x00020000);
}

// The VEC-element chunks of channel c that split p of P owns (planes n = p, p + P, ..., flattened
// so that the lanes stay busy whatever the plane size), U at a time per thread:
// issue(u, element_offset, exists) is called for the U chunks of a batch first — it should only
// start loads — and use(u) afterwards for those of them that exist.  The loads of a batch are thus
// in flight together; a chunk that does not exist is issued all the same, so that no load sits
// inside a branch (the compiler waits for such a load on the spot), with the offset of the
// batch's first chunk (which exists).  A second request for a line that is still on its way is
// not always merged with the first — on c5's 56 x 56 planes these duplicates made the backward
// sums fetch 10 % more than they read — so the kernels go through buffer addressing where they
// can (see RawVec) and such a chunk then costs no request at all.
template <int VEC, int U, typename ISSUE, typename USE>
__device__ __forceinline__ void for_channel_chunks_batched(int c, int p, int P, int64_t N, int C, int S,
                                                           ISSUE&& issue, USE&& use) {
  const uint32_t sp = (uint32_t)(S / VEC);
  const int64_t planes = (N - p + P - 1) / P;   // planes n = p, p + P, ...
  const int64_t total = planes * sp;
  auto offset_of = [&](int64_t q) {
    int64_t k;
    uint32_t i;
    if (total <= (int64_t)UINT32_MAX) {
      const uint32_t q32 = (uint32_t)q, k32 = q32 / sp;
      k = k32;
      i = q32 - k32 * sp;
    } else {
      k = q / sp;
      i = (uint32_t)(q - k * sp);
    }
    return ((p + k * P) * C + c) * (int64_t)S + (int64_t)i * VEC;
  };
  for (int64_t q0 = threadIdx.x; q0 < total; q0 += (int64_t)kBnBlock * U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t q = q0 + (int64_t)u * kBnBlock;
      const bool exists = q < total;
      issue(u, offset_of(exists ? q : q0), exists);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (q0 + (int64_t)u * kBnBlock < total) use(u);
  }
}

template <typename T, int VEC, bool BUF>
__global__ __launch_bounds__(kBnBlock) void bn_stats_kernel(const T* __restrict__ x, float* __restrict__ part,
                                                           int64_t N, int C, int S, int P) {
  __shared__ Welford smem[kBnBlock / 64];
  const int c = blockIdx.x, p = blockIdx.y;
  Welford acc{0.f, 0.f, 0.f};
  constexpr int U = 8;   // all of a workgroup's chunks in one round of loads at the usual sizes
  RawVec<T, VEC> raw[U];
  const __amdgpu_buffer_rsrc_t rs_x = tensor_rsrc<BUF>(x, N, C, S);
  for_channel_chunks_batched<VEC, U>(
      c, p, P, N, C, S,
      [&](int u, int64_t off, bool exists) {
        if constexpr (BUF) raw[u].load(rs_x, off, exists);
        else raw[u].load(x + off);
      },
      [&](int u) {
        float v[VEC];
        raw[u].get(v);
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

// Statistics of channel c for an apply workgroup.  Every thread calls this.
//   part != nullptr: every wave merges the P partial (count, mean, M2) triples by itself with three
//     sums over its lanes (total count; count-weighted mean; M2 plus count * squared distance of
//     each partial mean from the merged one) — the same order in every wave of every workgroup, so
//     all of them get the same bits, and no barrier or LDS is needed; `count` receives the number
//     of elements.
//   part == nullptr: the running statistics (evaluation mode).
__device__ __forceinline__ void channel_stats(const float* __restrict__ part, int P, int c,
                                              const void* __restrict__ running_mean,
                                              const void* __restrict__ running_var, int rdt, float& mean,
                                              float& var, float& count) {
  if (!part) {
    mean = load_scalar_f32(running_mean, rdt, c);
    var = load_scalar_f32(running_var, rdt, c);
    count = 0.f;
    return;
  }
  const int lane = threadIdx.x & 63;
  // the lane's first triple stays in registers for the second sum (with up to 64 splits nothing
  // is read twice)
  float n = 0.f, nm = 0.f, first[3] = {0.f, 0.f, 0.f};
  for (int p = lane; p < P; p += 64) {
    const float* src = part + ((int64_t)c * P + p) * 3;
    const float pn = src[0], pm = src[1], pq = src[2];
    if (p == lane) {
      first[0] = pn; first[1] = pm; first[2] = pq;
    }
    n += pn;
    nm += pn * pm;
  }
  n = wave_reduce(n, 64, SumOp());
  nm = wave_reduce(nm, 64, SumOp());
  const float m = nm / n;
  float m2 = 0.f;
  for (int p = lane; p < P; p += 64) {
    const float* src = part + ((int64_t)c * P + p) * 3;
    const bool cached = p == lane;
    const float pn = cached ? first[0] : src[0], pm = cached ? first[1] : src[1], pq = cached ? first[2] : src[2];
    const float d = pm - m;
    m2 += pq + pn * d * d;
  }
  m2 = wave_reduce(m2, 64, SumOp());
  mean = m;
  var = m2 / n;
  count = n;
}

// y = act(w * (x - mean) * inv_std + b (+ residual)); one workgroup per slice of a plane.
// grid.x = planes (n * C + c), grid.y = slices of the plane.  The workgroup of slice 0 of a
// channel's first plane (n = 0) also writes mean / inv_std and updates the running statistics
// (unbiased variance) of that channel.
template <typename T, int VEC, int ACT>
__global__ __launch_bounds__(kBnBlock) void bn_apply_kernel(
    const T* __restrict__ x, const T* __restrict__ res, T* __restrict__ pre_act, T* __restrict__ y,
    const float* __restrict__ part, int P, float* __restrict__ mean_out, float* __restrict__ inv_std_out,
    void* __restrict__ running_mean, void* __restrict__ running_var, int rdt, int update_running,
    float momentum, float eps, const void* __restrict__ w, const void* __restrict__ b, int wdt, int C, int S,
    float param, int64_t total_planes) {
  const int sp = S / VEC;
  const int step = gridDim.y * kBnBlock;
  int merged_c = -1;   // the channel whose statistics the workgroup holds (planes a multiple of C apart share it)
  float mean = 0.f, var = 0.f, count = 0.f;
  for (int64_t plane = blockIdx.x; plane < total_planes; plane += gridDim.x) {
    const int c = (int)(plane % C);
    const int64_t base = plane * (int64_t)S;
    // Two chunks per lane and pass, their loads (input and residual) issued together; those of the
    // first pass go out before the statistics of the channel are merged, so both latencies overlap.
    int i0 = blockIdx.y * kBnBlock + threadIdx.x;
    bool has1;
    int64_t off[2];
    RawVec<T, VEC> xin[2], rin[2];
    auto issue = [&](int i) {   // i < sp
      has1 = i + step < sp;
      off[0] = base + (int64_t)i * VEC;
      off[1] = base + (int64_t)(has1 ? i + step : i) * VEC;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        xin[u].load(x + off[u]);
        if (res) rin[u].load(res + off[u]);   // uniform
      }
    };
    issue(i0 < sp ? i0 : 0);
    if (c != merged_c) {   // uniform
      merged_c = c;
      channel_stats(part, P, c, running_mean, running_var, rdt, mean, var, count);
    }
    const float inv_std = rsqrtf(var + eps);
    if (plane < C && blockIdx.y == 0 && threadIdx.x == 0) {
      if (mean_out) mean_out[c] = mean;
      if (inv_std_out) inv_std_out[c] = inv_std;
      if (update_running) {
        const float rm = load_scalar_f32(running_mean, rdt, c), rv = load_scalar_f32(running_var, rdt, c);
        store_scalar_f32(running_mean, rdt, c, (1.f - momentum) * rm + momentum * mean);
        store_scalar_f32(running_var, rdt, c, (1.f - momentum) * rv + momentum * var * count / (count - 1.f));
      }
    }
    const float wt = w ? load_scalar_f32(w, wdt, c) : 1.f;
    const float bs = b ? load_scalar_f32(b, wdt, c) : 0.f;
    while (i0 < sp) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        if (u == 1 && !has1) break;
        float v[VEC];
        xin[u].get(v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = wt * (v[j] - mean) * inv_std + bs;
        if (res) {
          float r[VEC];
          rin[u].get(r);
#pragma unroll
          for (int j = 0; j < VEC; ++j) v[j] += r[j];
        }
        if (ACT != AT_ACT_NONE) {
          if (pre_act) store_f32<T, VEC>(pre_act + off[u], v);
#pragma unroll
          for (int j = 0; j < VEC; ++j) v[j] = act_forward(ACT, v[j], param);
        }
        store_f32<T, VEC>(y + off[u], v);
      }
      i0 += 2 * step;
      if (i0 < sp) issue(i0);
    }
  }
}

// Backward partial sums per (channel, split); writes g = dy * act'(pre_act) to g_out when an
// activation is fused (g_out then feeds the apply pass and doubles as the residual gradient).
template <typename T, int VEC, int ACT, bool BUF>
__global__ __launch_bounds__(kBnBlock) void bn_bwd_reduce_kernel(
    const T* __restrict__ dy, const T* __restrict__ pre_act, const T* __restrict__ x, T* __restrict__ g_out,
    const float* __restrict__ mean_in, const float* __restrict__ inv_std_in, float* __restrict__ part,
    int64_t N, int C, int S, int P, float param) {
  __shared__ float smem[16];
  const int c = blockIdx.x, p = blockIdx.y;
  const float mean = mean_in[c], inv_std = inv_std_in[c];
  float s1 = 0.f, s2 = 0.f;
  constexpr int U = kBnBwdBatch;
  RawVec<T, VEC> rg[U], rx[U], rz[ACT != AT_ACT_NONE ? U : 1];
  int64_t offs[U];
  const __amdgpu_buffer_rsrc_t rs_dy = tensor_rsrc<BUF>(dy, N, C, S), rs_x = tensor_rsrc<BUF>(x, N, C, S),
                               rs_z = tensor_rsrc<BUF && ACT != AT_ACT_NONE>(pre_act, N, C, S);
  for_channel_chunks_batched<VEC, U>(
      c, p, P, N, C, S,
      [&](int u, int64_t off, bool exists) {
        offs[u] = off;
        if constexpr (BUF) {
          rg[u].load(rs_dy, off, exists);
          rx[u].load(rs_x, off, exists);
          if constexpr (ACT != AT_ACT_NONE) rz[u].load(rs_z, off, exists);
        } else {
          rg[u].load(dy + off);
          rx[u].load(x + off);
          if constexpr (ACT != AT_ACT_NONE) rz[u].load(pre_act + off);
        }
      },
      [&](int u) {
        float g[VEC], xv[VEC];
        rg[u].get(g);
        rx[u].get(xv);
        if constexpr (ACT != AT_ACT_NONE) {
          float z[VEC];
          rz[u].get(z);
#pragma unroll
          for (int j = 0; j < VEC; ++j) g[j] *= act_derivative(ACT, z[j], param);
          store_f32<T, VEC>(g_out + offs[u], g);
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

// input_grad = inv_std * (w * g - (t1 * x_hat + t2)) with t1 = w * sum(g x_hat) / count and
// t2 = w * sum(g) / count.  Every workgroup sums the P partial pairs of its channel itself (wave 0,
// lane-strided then a tree: the same order everywhere); the workgroup of slice 0 of the channel's
// first plane also writes the weight and bias gradients.
template <typename T, int VEC>
__global__ __launch_bounds__(kBnBlock) void bn_bwd_apply_kernel(
    const T* __restrict__ g, const T* __restrict__ x, T* __restrict__ dx, const float* __restrict__ mean_in,
    const float* __restrict__ inv_std_in, const float* __restrict__ part, int P, float count,
    float* __restrict__ weight_grad, float* __restrict__ bias_grad, const void* __restrict__ w, int wdt,
    int C, int S, int64_t total_planes) {
  __shared__ float smem[2];
  const int sp = S / VEC;
  const int step = gridDim.y * kBnBlock;
  int summed_c = -1;   // the channel whose sums the workgroup holds (planes a multiple of C apart share it)
  float s1 = 0.f, s2 = 0.f;
  for (int64_t plane = blockIdx.x; plane < total_planes; plane += gridDim.x) {
    const int c = (int)(plane % C);
    const int64_t base = plane * (int64_t)S;
    int i0 = blockIdx.y * kBnBlock + threadIdx.x;
    bool has1;
    int64_t off[2];
    RawVec<T, VEC> gin[2], xin[2];
    auto issue = [&](int i) {   // i < sp
      has1 = i + step < sp;
      off[0] = base + (int64_t)i * VEC;
      off[1] = base + (int64_t)(has1 ? i + step : i) * VEC;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        gin[u].load(g + off[u]);
        xin[u].load(x + off[u]);
      }
    };
    issue(i0 < sp ? i0 : 0);   // in flight while the partial sums of the channel are added up
    if (c != summed_c) {       // uniform
      summed_c = c;
      __syncthreads();   // previous readers of smem are done
      if (threadIdx.x < 64) {
        float a1 = 0.f, a2 = 0.f;
        for (int p = threadIdx.x; p < P; p += 64) {
          a1 += part[((int64_t)c * P + p) * 2];
          a2 += part[((int64_t)c * P + p) * 2 + 1];
        }
        a1 = wave_reduce(a1, 64, SumOp());
        a2 = wave_reduce(a2, 64, SumOp());
        if (threadIdx.x == 0) {
          smem[0] = a1;
          smem[1] = a2;
        }
      }
      __syncthreads();
      s1 = smem[0];
      s2 = smem[1];
    }
    if (plane < C && blockIdx.y == 0 && threadIdx.x == 0) {
      if (weight_grad) weight_grad[c] = s1;
      if (bias_grad) bias_grad[c] = s2;
    }
    const float mean = mean_in[c], inv_std = inv_std_in[c];
    const float wt = w ? load_scalar_f32(w, wdt, c) : 1.f;
    const float t1 = s1 * wt / count, t2 = s2 * wt / count;
    while (i0 < sp) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        if (u == 1 && !has1) break;
        float gv[VEC], xv[VEC];
        gin[u].get(gv);
        xin[u].get(xv);
#pragma unroll
        for (int j = 0; j < VEC; ++j)
          gv[j] = inv_std * (wt * gv[j] - (t1 * (xv[j] - mean) * inv_std + t2));
        store_f32<T, VEC>(dx + off[u], gv);
      }
      i0 += 2 * step;
      if (i0 < sp) issue(i0);
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

// Grid of an apply pass: x walks over the planes with at most per_cu workgroups for every CU
// (a workgroup then loops over planes), y splits long planes.
inline void apply_grid(int64_t planes, int S, int vec, int per_cu, dim3* grid) {
  const int sp = S / vec;
  int gy = (int)cdiv64(sp, kBnBlock * 2);
  if (gy < 1) gy = 1;
  if (gy > 64) gy = 64;
  int64_t gx = planes;
  const int64_t cap = (int64_t)device_cu_count() * per_cu;
  if (gx > cap) gx = cap;
  *grid = dim3((unsigned)gx, (unsigned)gy);
}

constexpr int kMaxSplits = 1024;

// ------------------------------------------------------------------------------------------
// Channels-last tensors: a [rows = N * S][C] matrix, statistics per column.
// A row is C / VEC 16-byte chunks (at most 256 of them); lane t of a 256-lane workgroup owns chunk
// t % chunks_per_row of the rows (t / chunks_per_row) + k * rows_per_step it is given, so its VEC
// channels never change and their parameters live in registers.  Every pass reads whole rows,
// fully coalesced.  Passes: partial statistics per (row slice, channel) -> one wave per channel
// merges them (same arithmetic as the channels-first path) and leaves mean / inv_std (forward) or
// the three coefficients of the input gradient (backward) in the workspace -> elementwise pass.
// ------------------------------------------------------------------------------------------
struct LastRows {
  int64_t rows;
  int C;                // channels the workgroups cover (a slab of the row when the row is wider)
  int64_t stride;       // elements from one row to the next
  int chunks_per_row;   // C / VEC
  int rows_per_step;    // 256 / chunks_per_row
  int64_t rows_per_block;
};

// Whether the rows of a step that share a chunk sit in the lanes of one wave, every lane of the
// workgroup in use: chunks_per_row a power of two of at most 64.
__device__ __forceinline__ bool last_wave_fold(const LastRows& g) {
  return g.chunks_per_row <= 64 && (g.chunks_per_row & (g.chunks_per_row - 1)) == 0;
}

template <int VEC>
__device__ __forceinline__ bool last_lane(const LastRows& g, int& chunk, int& row_in_step) {
  chunk = threadIdx.x % g.chunks_per_row;
  row_in_step = threadIdx.x / g.chunks_per_row;
  return row_in_step < g.rows_per_step;
}

// Rows r0 + row_in_step + k * rows_per_step (< r1) of this lane's chunk, U at a time: issue(u, offset)
// for all of a batch first (rows that do not exist are issued at the batch's first row), then
// use(u) for those that exist.
template <int VEC, int U, typename ISSUE, typename USE>
__device__ __forceinline__ void for_rows_batched(const LastRows& g, int64_t r0, int64_t r1, int chunk,
                                                 int row_in_step, ISSUE&& issue, USE&& use) {
  for (int64_t r = r0 + row_in_step; r < r1; r += (int64_t)g.rows_per_step * U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t ru = r + (int64_t)u * g.rows_per_step;
      issue(u, (ru < r1 ? ru : r) * g.stride + (int64_t)chunk * VEC);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (r + (int64_t)u * g.rows_per_step < r1) use(u);
  }
}

// part[(c * P + p) * 3 + {0, 1, 2}] = (count, mean, M2) of channel c over row slice p.
template <typename T, int VEC>
__global__ __launch_bounds__(kBnBlock) void bn_last_stats_kernel(const T* __restrict__ x, float* __restrict__ part,
                                                                LastRows g, int P) {
  __shared__ float sm[kBnBlock * (2 * VEC + 1)];
  int chunk, row_in_step;
  const bool active = last_lane<VEC>(g, chunk, row_in_step);
  const int p = blockIdx.x;
  const int64_t r0 = p * g.rows_per_block;
  const int64_t r1 = r0 + g.rows_per_block < g.rows ? r0 + g.rows_per_block : g.rows;
  float n = 0.f, mean[VEC], m2[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) mean[j] = m2[j] = 0.f;
  if (active) {
    constexpr int U = 8;
    RawVec<T, VEC> raw[U];
    for_rows_batched<VEC, U>(
        g, r0, r1, chunk, row_in_step, [&](int u, int64_t off) { raw[u].load(x + off); },
        [&](int u) {
          float v[VEC];
          raw[u].get(v);
          n += 1.f;
          const float inv_n = __fdividef(1.f, n);
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            const float d = v[j] - mean[j];
            mean[j] += d * inv_n;
            m2[j] += d * (v[j] - mean[j]);
          }
        });
  }
  if (last_wave_fold(g)) {
    // Rows of a step sit in the lanes of a wave (lane = row * chunks_per_row + chunk): a butterfly
    // over the lanes merges them, the four waves meet in LDS once, value v of wave w and chunk c
    // at sm[(v * 4 + w) * chunks_per_row + c], and lane (j, c) merges the four triples of its channel.
    const int cpr = g.chunks_per_row;
    for (int o = cpr; o < 64; o <<= 1) {
      const float nb = __shfl_xor(n, o);
      const float nn = n + nb;
      const float f = nn > 0.f ? nb / nn : 0.f;
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float d = __shfl_xor(mean[j], o) - mean[j];
        m2[j] += __shfl_xor(m2[j], o) + d * d * n * f;
        mean[j] += d * f;
      }
      n = nn;
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane < cpr) {
      sm[wave * cpr + lane] = n;
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        sm[((1 + j) * 4 + wave) * cpr + lane] = mean[j];
        sm[((1 + VEC + j) * 4 + wave) * cpr + lane] = m2[j];
      }
    }
    __syncthreads();
    for (int o = threadIdx.x; o < cpr * VEC; o += kBnBlock) {
      const int c = o % cpr, j = o / cpr;
      float tn = sm[c], tm = sm[(1 + j) * 4 * cpr + c], tq = sm[(1 + VEC + j) * 4 * cpr + c];
      for (int w = 1; w < 4; ++w) {
        const float nb = sm[w * cpr + c];
        const float nn = tn + nb;
        if (nn > 0.f) {
          const float f = nb / nn;
          const float d = sm[((1 + j) * 4 + w) * cpr + c] - tm;
          tq += sm[((1 + VEC + j) * 4 + w) * cpr + c] + d * d * tn * f;
          tm += d * f;
        }
        tn = nn;
      }
      float* dst = part + ((int64_t)(c * VEC + j) * P + p) * 3;
      dst[0] = tn; dst[1] = tm; dst[2] = tq;
    }
    return;
  }
  // lanes of one chunk, one per row of a step: merged pairwise through LDS, row r taking in row
  // r + s for s = the largest power of two below the row count, then half of it, ... (a fixed tree)
  float* mine = sm + threadIdx.x * (2 * VEC + 1);
  int s = 1;
  while (s * 2 < g.rows_per_step) s *= 2;
  for (; s > 0; s >>= 1) {
    mine[0] = n;
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      mine[1 + j] = mean[j];
      mine[1 + VEC + j] = m2[j];
    }
    __syncthreads();
    if (active && row_in_step < s && row_in_step + s < g.rows_per_step) {
      const float* other = sm + ((row_in_step + s) * g.chunks_per_row + chunk) * (2 * VEC + 1);
      const float nb = other[0];
      const float nn = n + nb;
      if (nn > 0.f) {
        const float f = nb / nn;
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float d = other[1 + j] - mean[j];
          m2[j] += other[1 + VEC + j] + d * d * n * f;
          mean[j] += d * f;
        }
      }
      n = nn;
    }
    __syncthreads();
  }
  if (active && row_in_step == 0) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      float* dst = part + ((int64_t)(chunk * VEC + j) * P + p) * 3;
      dst[0] = n; dst[1] = mean[j]; dst[2] = m2[j];
    }
  }
}

// The per-channel values of a pass, staged once per workgroup: value v of channel c at sm[v * C + c].
// f(c, out) computes the NV values of channel c.  Returns after a barrier.
template <int NV, typename F>
__device__ __forceinline__ void stage_channel_values(float* sm, int C, F&& f) {
  for (int c = threadIdx.x; c < C; c += kBnBlock) {
    float out[NV];
    f(c, out);
#pragma unroll
    for (int v = 0; v < NV; ++v) sm[v * C + c] = out[v];
  }
  __syncthreads();
}
constexpr int kLastMaxC = kBnBlock * 8;   // channels of a row: at most 256 chunks of 8

// One wave per channel: merges the partial statistics (or takes the running ones), leaves
// stat[c] = mean, stat[C + c] = inv_std in the workspace, writes the optional outputs and
// updates the running statistics.
__global__ __launch_bounds__(64) void bn_last_finalize_kernel(
    const float* __restrict__ part, int P, float* __restrict__ stat, float* __restrict__ mean_out,
    float* __restrict__ inv_std_out, void* __restrict__ running_mean, void* __restrict__ running_var, int rdt,
    int update_running, float momentum, float eps, int C) {
  const int c = blockIdx.x;
  float mean, var, count;
  channel_stats(part, P, c, running_mean, running_var, rdt, mean, var, count);
  if (threadIdx.x != 0) return;
  const float inv_std = rsqrtf(var + eps);
  stat[c] = mean;
  stat[C + c] = inv_std;
  if (mean_out) mean_out[c] = mean;
  if (inv_std_out) inv_std_out[c] = inv_std;
  if (update_running) {
    const float rm = load_scalar_f32(running_mean, rdt, c), rv = load_scalar_f32(running_var, rdt, c);
    store_scalar_f32(running_mean, rdt, c, (1.f - momentum) * rm + momentum * mean);
    store_scalar_f32(running_var, rdt, c, (1.f - momentum) * rv + momentum * var * count / (count - 1.f));
  }
}

// y = act(w * (x - mean) * inv_std + b (+ residual)), rows in slices of rows_per_block.
template <typename T, int VEC, int ACT>
__global__ __launch_bounds__(kBnBlock) void bn_last_apply_kernel(
    const T* __restrict__ x, const T* __restrict__ res, T* __restrict__ pre_act, T* __restrict__ y,
    const float* __restrict__ stat, const void* __restrict__ w, const void* __restrict__ b, int wdt, LastRows g,
    float param) {
  __shared__ float sm[2 * kLastMaxC];
  int chunk, row_in_step;
  const bool active = last_lane<VEC>(g, chunk, row_in_step);
  const int64_t r0 = blockIdx.x * g.rows_per_block;
  const int64_t r1 = r0 + g.rows_per_block < g.rows ? r0 + g.rows_per_block : g.rows;
  constexpr int U = 4;
  RawVec<T, VEC> xin[U], rin[U];
  int64_t offs[U];
  auto issue = [&](int u, int64_t off) {
    offs[u] = off;
    xin[u].load(x + off);
    if (res) rin[u].load(res + off);   // uniform
  };
  // The first batch of rows is requested ahead of the parameters, which every lane needs before it
  // can use a row (a lane without a row asks for the slice's first one, which exists).
  int64_t r = r0 + row_in_step;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int64_t ru = r + (int64_t)u * g.rows_per_step;
    issue(u, ((active && ru < r1) ? ru : r0) * g.stride + (int64_t)(active ? chunk : 0) * VEC);
  }
  stage_channel_values<2>(sm, g.C, [&](int c, float (&out)[2]) {
    const float wt = w ? load_scalar_f32(w, wdt, c) : 1.f;
    const float bs = b ? load_scalar_f32(b, wdt, c) : 0.f;
    out[0] = wt * stat[g.C + c];
    out[1] = bs - stat[c] * out[0];
  });
  if (!active) return;
  float scale[VEC], shift[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) {
    scale[j] = sm[chunk * VEC + j];
    shift[j] = sm[g.C + chunk * VEC + j];
  }
  auto use = [&](int u) {
    float v[VEC];
    xin[u].get(v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) v[j] = fmaf(v[j], scale[j], shift[j]);
    if (res) {
      float rv[VEC];
      rin[u].get(rv);
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] += rv[j];
    }
    if (ACT != AT_ACT_NONE) {
      if (pre_act) store_f32<T, VEC>(pre_act + offs[u], v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = act_forward(ACT, v[j], param);
    }
    store_f32<T, VEC>(y + offs[u], v);
  };
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (r + (int64_t)u * g.rows_per_step < r1) use(u);
  for_rows_batched<VEC, U>(g, r0 + (int64_t)g.rows_per_step * U, r1, chunk, row_in_step, issue, use);
}

// part[(c * P + p) * 2 + {0, 1}] = (sum g x_hat, sum g) of channel c over row slice p, with
// g = dy * act'(pre_act), which is also written to g_out when an activation is fused.
template <typename T, int VEC, int ACT>
__global__ __launch_bounds__(kBnBlock) void bn_last_bwd_reduce_kernel(
    const T* __restrict__ dy, const T* __restrict__ pre_act, const T* __restrict__ x, T* __restrict__ g_out,
    const float* __restrict__ mean_in, const float* __restrict__ inv_std_in, float* __restrict__ part, LastRows g,
    int P, float param) {
  __shared__ float sm[kBnBlock * 2 * VEC];
  int chunk, row_in_step;
  const bool active = last_lane<VEC>(g, chunk, row_in_step);
  const int p = blockIdx.x;
  const int64_t r0 = p * g.rows_per_block;
  const int64_t r1 = r0 + g.rows_per_block < g.rows ? r0 + g.rows_per_block : g.rows;
  float s1[VEC], s2[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) s1[j] = s2[j] = 0.f;
  if (active) {
    float mean[VEC], inv_std[VEC];
    if (((reinterpret_cast<uintptr_t>(mean_in) | reinterpret_cast<uintptr_t>(inv_std_in)) & 15) == 0) {
      load_f32<float, VEC>(mean_in + chunk * VEC, mean);
      load_f32<float, VEC>(inv_std_in + chunk * VEC, inv_std);
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        mean[j] = mean_in[chunk * VEC + j];
        inv_std[j] = inv_std_in[chunk * VEC + j];
      }
    }
    constexpr int U = 4;
    RawVec<T, VEC> rg[U], rx[U], rz[ACT != AT_ACT_NONE ? U : 1];
    int64_t offs[U];
    for_rows_batched<VEC, U>(
        g, r0, r1, chunk, row_in_step,
        [&](int u, int64_t off) {
          offs[u] = off;
          rg[u].load(dy + off);
          rx[u].load(x + off);
          if constexpr (ACT != AT_ACT_NONE) rz[u].load(pre_act + off);
        },
        [&](int u) {
          float gv[VEC], xv[VEC];
          rg[u].get(gv);
          rx[u].get(xv);
          if constexpr (ACT != AT_ACT_NONE) {
            float z[VEC];
            rz[u].get(z);
#pragma unroll
            for (int j = 0; j < VEC; ++j) gv[j] *= act_derivative(ACT, z[j], param);
            store_f32<T, VEC>(g_out + offs[u], gv);
            // the reference rounds pre_act_grad to the storage dtype before reducing it
#pragma unroll
            for (int j = 0; j < VEC; ++j) gv[j] = to_f32(from_f32<T>(gv[j]));
          }
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            s1[j] += gv[j] * (xv[j] - mean[j]) * inv_std[j];
            s2[j] += gv[j];
          }
        });
  }
  if (last_wave_fold(g)) {   // as in the statistics pass
    const int cpr = g.chunks_per_row;
    for (int o = cpr; o < 64; o <<= 1) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        s1[j] += __shfl_xor(s1[j], o);
        s2[j] += __shfl_xor(s2[j], o);
      }
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane < cpr) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        sm[(j * 4 + wave) * cpr + lane] = s1[j];
        sm[((VEC + j) * 4 + wave) * cpr + lane] = s2[j];
      }
    }
    __syncthreads();
    for (int o = threadIdx.x; o < cpr * 2 * VEC; o += kBnBlock) {
      const int c = o % cpr, v = o / cpr;   // v < VEC: s1[v], else s2[v - VEC]
      const float* src = sm + v * 4 * cpr + c;
      const float t = ((src[0] + src[cpr]) + src[2 * cpr]) + src[3 * cpr];
      const int j = v < VEC ? v : v - VEC;
      part[((int64_t)(c * VEC + j) * P + p) * 2 + (v < VEC ? 0 : 1)] = t;
    }
    return;
  }
  float* mine = sm + threadIdx.x * 2 * VEC;
  int s = 1;
  while (s * 2 < g.rows_per_step) s *= 2;
  for (; s > 0; s >>= 1) {   // the same fixed tree as in the statistics pass
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      mine[j] = s1[j];
      mine[VEC + j] = s2[j];
    }
    __syncthreads();
    if (active && row_in_step < s && row_in_step + s < g.rows_per_step) {
      const float* other = sm + ((row_in_step + s) * g.chunks_per_row + chunk) * 2 * VEC;
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        s1[j] += other[j];
        s2[j] += other[VEC + j];
      }
    }
    __syncthreads();
  }
  if (active && row_in_step == 0) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      float* dst = part + ((int64_t)(chunk * VEC + j) * P + p) * 2;
      dst[0] = s1[j]; dst[1] = s2[j];
    }
  }
}

// One wave per channel: sums the partial pairs, writes the weight and bias gradients and leaves
// the coefficients of input_grad = a * g - (b1 * (x - mean) + b2) in the workspace:
// coef[c] = a = inv_std * w, coef[C + c] = b1, coef[2C + c] = b2, coef[3C + c] = mean.
__global__ __launch_bounds__(64) void bn_last_bwd_finalize_kernel(
    const float* __restrict__ part, int P, float count, const float* __restrict__ mean_in,
    const float* __restrict__ inv_std_in, const void* __restrict__ w, int wdt, float* __restrict__ coef,
    float* __restrict__ weight_grad, float* __restrict__ bias_grad, int C) {
  const int c = blockIdx.x;
  float s1 = 0.f, s2 = 0.f;
  for (int p = threadIdx.x; p < P; p += 64) {
    s1 += part[((int64_t)c * P + p) * 2];
    s2 += part[((int64_t)c * P + p) * 2 + 1];
  }
  s1 = wave_reduce(s1, 64, SumOp());
  s2 = wave_reduce(s2, 64, SumOp());
  if (threadIdx.x != 0) return;
  if (weight_grad) weight_grad[c] = s1;
  if (bias_grad) bias_grad[c] = s2;
  const float inv_std = inv_std_in[c];
  const float wt = w ? load_scalar_f32(w, wdt, c) : 1.f;
  const float t1 = s1 * wt / count, t2 = s2 * wt / count;
  coef[c] = inv_std * wt;
  coef[C + c] = inv_std * t1 * inv_std;
  coef[2 * C + c] = inv_std * t2;
  coef[3 * C + c] = mean_in[c];
}

template <typename T, int VEC>
__global__ __launch_bounds__(kBnBlock) void bn_last_bwd_apply_kernel(const T* __restrict__ gin, const T* __restrict__ x,
                                                                    T* __restrict__ dx, const float* __restrict__ coef,
                                                                    LastRows g) {
  int chunk, row_in_step;
  if (!last_lane<VEC>(g, chunk, row_in_step)) return;
  float a[VEC], b1[VEC], b2[VEC], mean[VEC];
  {
    // 16-byte loads: the coefficient arrays are laid out by channel and chunk * VEC is a multiple of 4
    float tmp[4][VEC];
#pragma unroll
    for (int v = 0; v < 4; ++v) load_f32<float, VEC>(coef + (int64_t)v * g.C + chunk * VEC, tmp[v]);
#pragma unroll
    for (int j = 0; j < VEC; ++j) { a[j] = tmp[0][j]; b1[j] = tmp[1][j]; b2[j] = tmp[2][j]; mean[j] = tmp[3][j]; }
  }
  const int64_t r0 = blockIdx.x * g.rows_per_block;
  const int64_t r1 = r0 + g.rows_per_block < g.rows ? r0 + g.rows_per_block : g.rows;
  constexpr int U = 4;
  RawVec<T, VEC> rg[U], rx[U];
  int64_t offs[U];
  for_rows_batched<VEC, U>(
      g, r0, r1, chunk, row_in_step,
      [&](int u, int64_t off) {
        offs[u] = off;
        rg[u].load(gin + off);
        rx[u].load(x + off);
      },
      [&](int u) {
        float gv[VEC], xv[VEC];
        rg[u].get(gv);
        rx[u].get(xv);
#pragma unroll
        for (int j = 0; j < VEC; ++j) gv[j] = a[j] * gv[j] - (b1[j] * (xv[j] - mean[j]) + b2[j]);
        store_f32<T, VEC>(dx + offs[u], gv);
      });
}

// Geometry of the channels-last passes, or false when the layout does not fit them.
inline bool last_rows(int64_t rows, int64_t feat, int64_t stride, int dtype, int64_t chunks_per_block,
                      int64_t max_blocks, LastRows* g, int* blocks) {
  const int vec = 16 / dtype_size(dtype);
  if (feat % vec != 0 || feat / vec > kBnBlock) return false;
  g->rows = rows;
  g->C = (int)feat;
  g->stride = stride;
  g->chunks_per_row = (int)(feat / vec);
  g->rows_per_step = kBnBlock / g->chunks_per_row;
  // rows per block: whole steps, about chunks_per_block 16-byte chunks per lane
  int64_t steps = chunks_per_block;
  int64_t per_block = steps * g->rows_per_step;
  int64_t nb = cdiv64(rows, per_block);
  if (nb > max_blocks) {
    per_block = cdiv64(cdiv64(rows, max_blocks), g->rows_per_step) * g->rows_per_step;
    nb = cdiv64(rows, per_block);
  }
  g->rows_per_block = per_block;
  *blocks = (int)nb;
  return true;
}

// Row slices of a summing pass: per_cu for every CU, within what the workspace holds.
inline int64_t last_slices(int per_cu) {
  const int64_t n = (int64_t)device_cu_count() * per_cu;
  return n < kMaxSplits ? n : kMaxSplits;
}

// p + elems elements (null stays null): the column slab of a tensor or of a parameter vector
inline const void* slab_of(const void* p, int64_t elems, int dt) {
  return p ? (const char*)p + elems * dtype_size(dt) : nullptr;
}
inline void* slab_of_mut(void* p, int64_t elems, int dt) { return p ? (char*)p + elems * dtype_size(dt) : nullptr; }
inline float* slab_of_f32(float* p, int64_t elems) { return p ? p + elems : nullptr; }
inline const float* slab_of_f32c(const float* p, int64_t elems) { return p ? p + elems : nullptr; }

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
  const int C = (int)feat, S = (int)spatial;
  const int es = dtype_size(dtype);
  const int vfull = 16 / es;
  const bool vec_ok = S % vfull == 0 && aligned16(input) && aligned16(output) &&
                      (!pre_act_add || aligned16(pre_act_add)) && (!pre_act || aligned16(pre_act));
  const bool buffered = batch * feat * spatial * es < kBufferedBytes;

  return dispatch_dtype(dtype, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    constexpr int VEC = 16 / (int)sizeof(T);
    int P = 0;
    if (batch_stats) {
      P = bn_splits(batch, C);
      if (vec_ok && buffered)
        hipLaunchKernelGGL((bn_stats_kernel<T, VEC, true>), dim3(C, P), dim3(kBnBlock), 0, stream, (const T*)input,
                           part, batch, C, S, P);
      else if (vec_ok)
        hipLaunchKernelGGL((bn_stats_kernel<T, VEC, false>), dim3(C, P), dim3(kBnBlock), 0, stream,
                           (const T*)input, part, batch, C, S, P);
      else
        hipLaunchKernelGGL((bn_stats_kernel<T, 1, false>), dim3(C, P), dim3(kBnBlock), 0, stream, (const T*)input,
                           part, batch, C, S, P);
    }
    const int update = batch_stats && track_running_stats && is_train && running_mean && running_var;
    const float* part_in = batch_stats ? part : nullptr;   // null: the apply pass reads the running statistics
    dim3 grid;
    const int64_t planes = batch * feat;
    apply_grid(planes, S, vec_ok ? VEC : 1, 64, &grid);
    if (vec_ok) {
      AT_BN_ACT_SWITCH(act, hipLaunchKernelGGL((bn_apply_kernel<T, VEC, ACT>), grid, dim3(kBnBlock), 0, stream,
                                               (const T*)input, (const T*)pre_act_add, (T*)pre_act, (T*)output,
                                               part_in, P, mean, inv_std, running_mean, running_var,
                                               running_dtype, update, momentum, eps, weight, bias, param_dtype, C,
                                               S, param, planes));
    } else {
      AT_BN_ACT_SWITCH(act, hipLaunchKernelGGL((bn_apply_kernel<T, 1, ACT>), grid, dim3(kBnBlock), 0, stream,
                                               (const T*)input, (const T*)pre_act_add, (T*)pre_act, (T*)output,
                                               part_in, P, mean, inv_std, running_mean, running_var,
                                               running_dtype, update, momentum, eps, weight, bias, param_dtype, C,
                                               S, param, planes));
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
  const int C = (int)feat, S = (int)spatial;
  const int vfull = 16 / dtype_size(dtype);
  const bool vec_ok = S % vfull == 0 && aligned16(output_grad) && aligned16(input) && aligned16(input_grad) &&
                      (!pre_act || aligned16(pre_act)) && (!pre_act_grad || aligned16(pre_act_grad));
  const void* g_for_apply = act != AT_ACT_NONE ? pre_act_grad : output_grad;
  const bool buffered = batch * feat * spatial * dtype_size(dtype) < kBufferedBytes;

  return dispatch_dtype(dtype, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    constexpr int VEC = 16 / (int)sizeof(T);
    int P = bn_splits(batch, C);
    if (vec_ok) {
      // At least as many splits as give a workgroup no more planes than one round of its loads
      // covers: a lane that loops waits for the acknowledgement of the gradient it has just stored
      // before the next round's loads count as arrived (c5: 70.6 -> 68.9 us for the backward pass).
      const int64_t per = (int64_t)kBnBlock * kBnBwdBatch / (S / VEC);
      const int64_t want = cdiv64(batch, per < 1 ? 1 : per);
      if (want > P) P = (int)(want > kMaxSplits ? kMaxSplits : want);
    }
    if (vec_ok && buffered) {
      AT_BN_ACT_SWITCH(act, hipLaunchKernelGGL((bn_bwd_reduce_kernel<T, VEC, ACT, true>), dim3(C, P), dim3(kBnBlock),
                                               0, stream, (const T*)output_grad, (const T*)pre_act, (const T*)input,
                                               (T*)pre_act_grad, mean, inv_std, part, batch, C, S, P, param));
    } else if (vec_ok) {
      AT_BN_ACT_SWITCH(act, hipLaunchKernelGGL((bn_bwd_reduce_kernel<T, VEC, ACT, false>), dim3(C, P), dim3(kBnBlock),
                                               0, stream, (const T*)output_grad, (const T*)pre_act, (const T*)input,
                                               (T*)pre_act_grad, mean, inv_std, part, batch, C, S, P, param));
    } else {
      AT_BN_ACT_SWITCH(act, hipLaunchKernelGGL((bn_bwd_reduce_kernel<T, 1, ACT, false>), dim3(C, P), dim3(kBnBlock), 0,
                                               stream, (const T*)output_grad, (const T*)pre_act, (const T*)input,
                                               (T*)pre_act_grad, mean, inv_std, part, batch, C, S, P, param));
    }
    dim3 grid;
    const int64_t planes = batch * feat;
    // Two planes per workgroup at c5's size, of one channel when the grid is a multiple of C: the
    // channel's sums are then added up once for both (c5: 72 -> 69 us for the backward pass; the
    // forward pass is best at one plane each).
    apply_grid(planes, S, vec_ok ? VEC : 1, 16, &grid);
    const float count = (float)(batch * spatial);
    if (vec_ok)
      hipLaunchKernelGGL((bn_bwd_apply_kernel<T, VEC>), grid, dim3(kBnBlock), 0, stream, (const T*)g_for_apply,
                         (const T*)input, (T*)input_grad, mean, inv_std, part, P, count, weight_grad, bias_grad,
                         weight, param_dtype, C, S, planes);
    else
      hipLaunchKernelGGL((bn_bwd_apply_kernel<T, 1>), grid, dim3(kBnBlock), 0, stream, (const T*)g_for_apply,
                         (const T*)input, (T*)input_grad, mean, inv_std, part, P, count, weight_grad, bias_grad,
                         weight, param_dtype, C, S, planes);
    return launch_status();
  });
}

int at_batch_norm_nhwc_supported(int64_t feat, int dtype) {
  if (!dtype_valid(dtype) || feat <= 0) return 0;
  // rows wider than one workgroup's 256 chunks of 16 bytes are processed in column slabs
  return feat % (16 / dtype_size(dtype)) == 0 ? 1 : 0;
}


int at_batch_norm_fwd_nhwc(const void* input, const void* weight, const void* bias, float* mean, float* inv_std,
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
  if (!at_batch_norm_nhwc_supported(feat, dtype)) return AT_ERR_UNSUPPORTED;
  if (!aligned16(input) || !aligned16(output) || (pre_act_add && !aligned16(pre_act_add)) ||
      (pre_act && !aligned16(pre_act)))
    return AT_ERR_ALIGN;
  if (!(weight && bias)) weight = bias = nullptr;  // affine only with both (batch_norm_layer.py:116)
  if (pre_act == output) pre_act = nullptr;

  float* part = (float*)workspace;
  const int64_t rows = batch * spatial;
  const int64_t slab = (int64_t)(16 / dtype_size(dtype)) * kBnBlock;   // channels one workgroup row covers
  for (int64_t c0 = 0; c0 < feat; c0 += slab) {
    const int C = (int)(feat - c0 < slab ? feat - c0 : slab);
    float* stat = part + (int64_t)C * kMaxSplits * 3;   // mean[C], inv_std[C]
    LastRows gs, ga;
    int P = 0, blocks = 0;
    // statistics: two row slices per CU; apply: one round of four rows per lane and workgroup
    // (c5: 64.7 -> 62 us for the pass against eight rows in two rounds)
    if (!last_rows(rows, C, feat, dtype, 16, last_slices(2), &gs, &P) ||
        !last_rows(rows, C, feat, dtype, 4, 65535, &ga, &blocks))
      return AT_ERR_UNSUPPORTED;
    const void* x = slab_of(input, c0, dtype);
    const void* res = slab_of(pre_act_add, c0, dtype);
    void* pre = slab_of_mut(pre_act, c0, dtype);
    void* y = slab_of_mut(output, c0, dtype);
    const void* w = slab_of(weight, c0, param_dtype);
    const void* b = slab_of(bias, c0, param_dtype);
    void* rm = slab_of_mut(running_mean, c0, running_dtype);
    void* rv = slab_of_mut(running_var, c0, running_dtype);
    float* mean_c = slab_of_f32(mean, c0);
    float* inv_std_c = slab_of_f32(inv_std, c0);
    const int rc = dispatch_dtype(dtype, [&](auto* tp) -> int {
      typedef std::remove_pointer_t<decltype(tp)> T;
      constexpr int VEC = 16 / (int)sizeof(T);
      if (batch_stats)
        hipLaunchKernelGGL((bn_last_stats_kernel<T, VEC>), dim3(P), dim3(kBnBlock), 0, stream, (const T*)x, part, gs, P);
      const int update = batch_stats && track_running_stats && is_train && running_mean && running_var;
      hipLaunchKernelGGL(bn_last_finalize_kernel, dim3(C), dim3(64), 0, stream, batch_stats ? part : nullptr, P, stat,
                         mean_c, inv_std_c, rm, rv, running_dtype, update, momentum, eps, C);
      AT_BN_ACT_SWITCH(act, hipLaunchKernelGGL((bn_last_apply_kernel<T, VEC, ACT>), dim3(blocks), dim3(kBnBlock), 0,
                                               stream, (const T*)x, (const T*)res, (T*)pre, (T*)y, stat, w, b,
                                               param_dtype, ga, param));
      return launch_status();
    });
    if (rc) return rc;
  }
  return AT_OK;
}

int at_batch_norm_bwd_nhwc(const void* output_grad, const void* pre_act, const void* input, const float* mean,
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
  if (!at_batch_norm_nhwc_supported(feat, dtype)) return AT_ERR_UNSUPPORTED;
  if (!aligned16(output_grad) || !aligned16(input) || !aligned16(input_grad) || (pre_act && !aligned16(pre_act)) ||
      (pre_act_grad && !aligned16(pre_act_grad)))
    return AT_ERR_ALIGN;

  float* part = (float*)workspace;
  const int64_t rows = batch * spatial;
  const int64_t slab = (int64_t)(16 / dtype_size(dtype)) * kBnBlock;
  for (int64_t c0 = 0; c0 < feat; c0 += slab) {
    const int C = (int)(feat - c0 < slab ? feat - c0 : slab);
    float* coef = part + (int64_t)C * kMaxSplits * 3;   // 4 floats per channel
    LastRows gs, ga;
    int P = 0, blocks = 0;
    // sums: one row slice per CU (three tensors in and one out per row: c5 78.7 -> 76.5 us for the
    // pass against two); apply as in the forward pass
    if (!last_rows(rows, C, feat, dtype, 16, last_slices(1), &gs, &P) ||
        !last_rows(rows, C, feat, dtype, 4, 65535, &ga, &blocks))
      return AT_ERR_UNSUPPORTED;
    const void* dy = slab_of(output_grad, c0, dtype);
    const void* pre = slab_of(pre_act, c0, dtype);
    const void* x = slab_of(input, c0, dtype);
    void* dx = slab_of_mut(input_grad, c0, dtype);
    void* dpre = slab_of_mut(pre_act_grad, c0, dtype);
    const void* w = slab_of(weight, c0, param_dtype);
    const float* mean_c = slab_of_f32c(mean, c0);
    const float* inv_std_c = slab_of_f32c(inv_std, c0);
    float* wg = slab_of_f32(weight_grad, c0);
    float* bg = slab_of_f32(bias_grad, c0);
    const void* g_for_apply = act != AT_ACT_NONE ? dpre : dy;
    const int rc = dispatch_dtype(dtype, [&](auto* tp) -> int {
      typedef std::remove_pointer_t<decltype(tp)> T;
      constexpr int VEC = 16 / (int)sizeof(T);
      AT_BN_ACT_SWITCH(act, hipLaunchKernelGGL((bn_last_bwd_reduce_kernel<T, VEC, ACT>), dim3(P), dim3(kBnBlock), 0,
                                               stream, (const T*)dy, (const T*)pre, (const T*)x, (T*)dpre, mean_c,
                                               inv_std_c, part, gs, P, param));
      hipLaunchKernelGGL(bn_last_bwd_finalize_kernel, dim3(C), dim3(64), 0, stream, part, P, (float)rows, mean_c,
                         inv_std_c, w, param_dtype, coef, wg, bg, C);
      hipLaunchKernelGGL((bn_last_bwd_apply_kernel<T, VEC>), dim3(blocks), dim3(kBnBlock), 0, stream,
                         (const T*)g_for_apply, (const T*)x, (T*)dx, coef, ga);
      return launch_status();
    });
    if (rc) return rc;
  }
  return AT_OK;
}

}  // extern "C"
