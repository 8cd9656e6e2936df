// Row-reduction kernels: RMSNorm, LayerNorm, Softmax/LogSoftmax/Softmin, forward and backward.
//
// These are HBM-bound: every element is read once and written once per pass.  A row is owned
// by a "group" of 2^k consecutive lanes (a fraction of a wave for narrow rows, one wave, or
// several waves of one workgroup for wide rows).  Each lane keeps its chunks of the row in
// registers (ITERS chunks of VEC elements, 128-bit accesses on the vector path), so the row is
// read from memory exactly once even though the math needs two or three sweeps.  Rows wider
// than the register budget use the streaming instantiation (ITERS == 0), which re-reads the
// row from cache.  Parameter gradients of the norms are accumulated per lane across a
// persistent grid, reduced across the workgroup through LDS, written as one partial row per
// workgroup and summed by a second launch in fixed order (deterministic, no atomics).
#include <type_traits>

#include "at_common.h"

namespace at_hip {
namespace {

template <int ITERS> constexpr int cache_len() { return ITERS > 0 ? ITERS : 1; }

struct RowPlan {
  int vec;         // elements per chunk: 8 / 4 on the vector path, 1 on the scalar path
  int group_log2;  // lanes per row = 1 << group_log2
  int iters;       // template ITERS to use: 1, 2, 4, 8, or 0 (streaming)
  int block;       // threads per workgroup
};

inline RowPlan plan_rows(int64_t feat, int vec, int min_block, int wave_rows_iters, int max_group) {
  RowPlan p;
  p.vec = vec;
  const int64_t chunks = cdiv64(feat, vec);
  // Prefer one wave per row (no workgroup barriers in the reductions) while the row fits in
  // wave_rows_iters chunks per lane; narrower rows use a fraction of a wave with one chunk per
  // lane; wider rows spread over several waves.
  int group;
  if (chunks <= kWave) group = next_pow2(chunks);
  else if (chunks <= (int64_t)kWave * wave_rows_iters) group = kWave;
  else group = next_pow2(cdiv64(chunks, wave_rows_iters));
  if (group > max_group) group = max_group;
  int iters = (int)cdiv64(chunks, group);
  if (iters > 8) p.iters = 0;
  else p.iters = iters <= 1 ? 1 : iters <= 2 ? 2 : iters <= 4 ? 4 : 8;
  p.group_log2 = 0;
  while ((1 << p.group_log2) < group) ++p.group_log2;
  p.block = group > min_block ? group : min_block;
  return p;
}

// ------------------------------------------------------------------------------------------
// Norm forward.  LAYER = true: LayerNorm (mean subtracted, optional bias); false: RMSNorm.
// ------------------------------------------------------------------------------------------
template <bool LAYER, typename TX, typename TY, int VEC, int ITERS>
__global__ __launch_bounds__(1024) void norm_fwd_kernel(
    const TX* __restrict__ x, const void* __restrict__ w, const void* __restrict__ b,
    float* __restrict__ mean_out, float* __restrict__ rstd_out, TY* __restrict__ y,
    int64_t batch, int feat, int64_t xs, int64_t ys, float eps, int wdt, int group_log2) {
  __shared__ float scratch[16];
  const int group = 1 << group_log2;
  const int lane = threadIdx.x & (group - 1);
  const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> group_log2) + (threadIdx.x >> group_log2);
  const bool valid = row < batch;
  const int chunks = feat / VEC;
  const int n_it = ITERS > 0 ? ITERS : (chunks + group - 1) / group;
  const TX* xr = x + (valid ? row : 0) * xs;
  float cache[cache_len<ITERS>()][VEC];
  const float inv_feat = 1.0f / (float)feat;

  float mean = 0.f;
  if (LAYER) {
    float s = 0.f;
#pragma unroll
    for (int it = 0; it < n_it; ++it) {
      const int c = lane + it * group;
      float v[VEC];
      if (valid && c < chunks) load_f32<TX, VEC>(xr + (int64_t)c * VEC, v);
      else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = 0.f;
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        s += v[j];
        if (ITERS > 0) cache[ITERS > 0 ? it : 0][j] = v[j];
      }
    }
    mean = group_reduce(s, group, scratch, SumOp(), 0.f) * inv_feat;
  }

  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < n_it; ++it) {
    const int c = lane + it * group;
    float v[VEC];
    if (ITERS > 0 && LAYER) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = cache[ITERS > 0 ? it : 0][j];
    } else {
      if (valid && c < chunks) load_f32<TX, VEC>(xr + (int64_t)c * VEC, v);
      else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = 0.f;
      }
      if (ITERS > 0) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) cache[ITERS > 0 ? it : 0][j] = v[j];
      }
    }
    if (c < chunks) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float d = v[j] - mean;
        ss += d * d;
      }
    }
  }
  ss = group_reduce(ss, group, scratch, SumOp(), 0.f);
  const float rstd = rsqrtf(ss * inv_feat + eps);

  if (valid && lane == 0) {
    if (LAYER && mean_out) mean_out[row] = mean;
    if (rstd_out) rstd_out[row] = rstd;
  }
  if (!valid) return;

  TY* yr = y + row * ys;
#pragma unroll
  for (int it = 0; it < n_it; ++it) {
    const int c = lane + it * group;
    if (c < chunks) {
      float v[VEC];
      if (ITERS > 0) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = cache[ITERS > 0 ? it : 0][j];
      } else {
        load_f32<TX, VEC>(xr + (int64_t)c * VEC, v);
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = (v[j] - mean) * rstd;
      if (w) {
        float wv[VEC];
        load_param_f32<VEC>(w, wdt, (int64_t)c * VEC, wv);
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] *= wv[j];
        if (LAYER && b) {
          float bv[VEC];
          load_param_f32<VEC>(b, wdt, (int64_t)c * VEC, bv);
#pragma unroll
          for (int j = 0; j < VEC; ++j) v[j] += bv[j];
        }
      }
      store_f32<TY, VEC>(yr + (int64_t)c * VEC, v);
    }
  }
}

// ------------------------------------------------------------------------------------------
// Norm backward over a persistent grid.  Each workgroup walks row-blocks with a grid stride;
// each lane accumulates the parameter gradients of the columns it owns.
//   part_w / part_b: [gridDim.x, feat] fp32 partial rows (null when not wanted).
// Dynamic LDS: blockDim.x * VEC floats (only used when a workgroup holds several rows).
// ------------------------------------------------------------------------------------------
template <bool LAYER, typename TDY, typename TX, typename TDX, int VEC, int ITERS>
__global__ __launch_bounds__(512) void norm_bwd_kernel(
    const TDY* __restrict__ dy, const TX* __restrict__ x, const float* __restrict__ mean_in,
    const float* __restrict__ rstd_in, const void* __restrict__ w, TDX* __restrict__ dx,
    float* __restrict__ part_w, float* __restrict__ part_b, int64_t batch, int feat,
    int64_t dys, int64_t xs, int64_t dxs, int wdt, int group_log2) {
  static_assert(ITERS > 0, "the persistent backward kernel caches the row in registers");
  __shared__ float scratch[16];
  extern __shared__ float red[];
  const int group = 1 << group_log2;
  const int lane = threadIdx.x & (group - 1);
  const int rpb = blockDim.x >> group_log2;
  const int rib = threadIdx.x >> group_log2;
  const int chunks = feat / VEC;
  const float inv_feat = 1.0f / (float)feat;
  const int64_t row_blocks = (batch + rpb - 1) / rpb;

  float acc_w[ITERS][VEC], acc_b[ITERS][VEC];
#pragma unroll
  for (int it = 0; it < ITERS; ++it)
#pragma unroll
    for (int j = 0; j < VEC; ++j) { acc_w[it][j] = 0.f; acc_b[it][j] = 0.f; }

  float wv[ITERS][VEC];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int c = lane + it * group;
    if (w && c < chunks) load_param_f32<VEC>(w, wdt, (int64_t)c * VEC, wv[it]);
    else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) wv[it][j] = 1.f;
    }
  }

  for (int64_t rb = blockIdx.x; rb < row_blocks; rb += gridDim.x) {
    const int64_t row = rb * rpb + rib;
    const bool valid = row < batch;
    const int64_t rr = valid ? row : 0;
    const TDY* dyr = dy + rr * dys;
    const TX* xr = x + rr * xs;
    const float mean = (LAYER && valid) ? mean_in[rr] : 0.f;
    const float rstd = valid ? rstd_in[rr] : 0.f;

    float xh[ITERS][VEC], g[ITERS][VEC];
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int c = lane + it * group;
      float dv[VEC], xv[VEC];
      if (valid && c < chunks) {
        load_f32<TDY, VEC>(dyr + (int64_t)c * VEC, dv);
        load_f32<TX, VEC>(xr + (int64_t)c * VEC, xv);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float h = (xv[j] - mean) * rstd;
          const float gg = dv[j] * wv[it][j];
          xh[it][j] = h;
          g[it][j] = gg;
          s1 += h * gg;
          s2 += gg;
          acc_w[it][j] += dv[j] * h;
          acc_b[it][j] += dv[j];
        }
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) { xh[it][j] = 0.f; g[it][j] = 0.f; }
      }
    }
    s1 = group_reduce(s1, group, scratch, SumOp(), 0.f) * inv_feat;
    if (LAYER) s2 = group_reduce(s2, group, scratch, SumOp(), 0.f) * inv_feat;
    else s2 = 0.f;

    if (valid) {
      TDX* dxr = dx + row * dxs;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int c = lane + it * group;
        if (c < chunks) {
          float o[VEC];
#pragma unroll
          for (int j = 0; j < VEC; ++j) o[j] = rstd * (g[it][j] - (xh[it][j] * s1 + s2));
          store_f32<TDX, VEC>(dxr + (int64_t)c * VEC, o);
        }
      }
    }
  }

  if (!part_w && !part_b) return;
  // Fold the row-groups of this workgroup together, then emit one partial row.
  const int n_out = (part_w ? 1 : 0) + ((LAYER && part_b) ? 1 : 0);
  for (int which = 0; which < n_out; ++which) {
    const bool is_w = (which == 0 && part_w);
    float* part = is_w ? part_w : part_b;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int c = lane + it * group;
      float v[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = is_w ? acc_w[it][j] : acc_b[it][j];
      if (rpb > 1) {
        __syncthreads();
#pragma unroll
        for (int j = 0; j < VEC; ++j) red[(rib * group + lane) * VEC + j] = v[j];
        __syncthreads();
        if (rib == 0) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            float s = 0.f;
            for (int r = 0; r < rpb; ++r) s += red[(r * group + lane) * VEC + j];
            v[j] = s;
          }
        }
      }
      if (rib == 0 && c < chunks) {
        float* dst = part + (int64_t)blockIdx.x * feat + (int64_t)c * VEC;
#pragma unroll
        for (int j = 0; j < VEC; ++j) dst[j] = v[j];
      }
    }
  }
}

// Streaming fallback for rows too wide for the register cache: input gradient only.
template <bool LAYER, typename TDY, typename TX, typename TDX, int VEC>
__global__ __launch_bounds__(1024) void norm_bwd_stream_kernel(
    const TDY* __restrict__ dy, const TX* __restrict__ x, const float* __restrict__ mean_in,
    const float* __restrict__ rstd_in, const void* __restrict__ w, TDX* __restrict__ dx,
    int64_t batch, int feat, int64_t dys, int64_t xs, int64_t dxs, int wdt) {
  __shared__ float scratch[16];
  const int group = blockDim.x;
  const int lane = threadIdx.x;
  const int64_t row = blockIdx.x;
  const int chunks = feat / VEC;
  const float inv_feat = 1.0f / (float)feat;
  const TDY* dyr = dy + row * dys;
  const TX* xr = x + row * xs;
  TDX* dxr = dx + row * dxs;
  const float mean = LAYER ? mean_in[row] : 0.f;
  const float rstd = rstd_in[row];
  float s1 = 0.f, s2 = 0.f;
  for (int c = lane; c < chunks; c += group) {
    float dv[VEC], xv[VEC], wv[VEC];
    load_f32<TDY, VEC>(dyr + (int64_t)c * VEC, dv);
    load_f32<TX, VEC>(xr + (int64_t)c * VEC, xv);
    if (w) load_param_f32<VEC>(w, wdt, (int64_t)c * VEC, wv);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float gg = w ? dv[j] * wv[j] : dv[j];
      s1 += (xv[j] - mean) * rstd * gg;
      s2 += gg;
    }
  }
  s1 = group_reduce(s1, group, scratch, SumOp(), 0.f) * inv_feat;
  s2 = LAYER ? group_reduce(s2, group, scratch, SumOp(), 0.f) * inv_feat : 0.f;
  for (int c = lane; c < chunks; c += group) {
    float dv[VEC], xv[VEC], wv[VEC], o[VEC];
    load_f32<TDY, VEC>(dyr + (int64_t)c * VEC, dv);
    load_f32<TX, VEC>(xr + (int64_t)c * VEC, xv);
    if (w) load_param_f32<VEC>(w, wdt, (int64_t)c * VEC, wv);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float gg = w ? dv[j] * wv[j] : dv[j];
      o[j] = rstd * (gg - ((xv[j] - mean) * rstd * s1 + s2));
    }
    store_f32<TDX, VEC>(dxr + (int64_t)c * VEC, o);
  }
}

// Column partial sums for the streaming fallback: one thread per column, a slice of rows per
// blockIdx.y; partial rows are [gridDim.y, feat].
template <bool LAYER, typename TDY, typename TX>
__global__ void norm_param_grad_cols_kernel(
    const TDY* __restrict__ dy, const TX* __restrict__ x, const float* __restrict__ mean_in,
    const float* __restrict__ rstd_in, float* __restrict__ part_w, float* __restrict__ part_b,
    int64_t batch, int feat, int64_t dys, int64_t xs, int64_t rows_per_slice) {
  const int col = blockIdx.x * blockDim.x + threadIdx.x;
  if (col >= feat) return;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_slice;
  const int64_t r1 = r0 + rows_per_slice < batch ? r0 + rows_per_slice : batch;
  float aw = 0.f, ab = 0.f;
  for (int64_t r = r0; r < r1; ++r) {
    const float d = to_f32(dy[r * dys + col]);
    const float mean = LAYER ? mean_in[r] : 0.f;
    aw += d * (to_f32(x[r * xs + col]) - mean) * rstd_in[r];
    ab += d;
  }
  if (part_w) part_w[(int64_t)blockIdx.y * feat + col] = aw;
  if (LAYER && part_b) part_b[(int64_t)blockIdx.y * feat + col] = ab;
}

// out[f] = sum over p of part[p, f], fixed order.  Block = 256 threads = 16 column quads x 16
// row slices; grid.x covers the columns in steps of 64, grid.y selects the gradient.
__global__ __launch_bounds__(256) void reduce_partials_kernel(
    const float* __restrict__ part0, float* __restrict__ out0, const float* __restrict__ part1,
    float* __restrict__ out1, int parts, int feat) {
  __shared__ float sm[16][65];
  const float* part = blockIdx.y == 0 ? part0 : part1;
  float* out = blockIdx.y == 0 ? out0 : out1;
  if (!part || !out) return;
  const int cq = threadIdx.x & 15, slice = threadIdx.x >> 4;
  const int col = blockIdx.x * 64 + cq * 4;
  float a[4] = {0.f, 0.f, 0.f, 0.f};
  for (int p = slice; p < parts; p += 16) {
    const float* src = part + (int64_t)p * feat + col;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (col + j < feat) a[j] += src[j];
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) sm[slice][cq * 4 + j] = a[j];
  __syncthreads();
  if (threadIdx.x < 64) {
    float s = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) s += sm[r][threadIdx.x];
    const int c = blockIdx.x * 64 + threadIdx.x;
    if (c < feat) out[c] = s;
  }
}

// ------------------------------------------------------------------------------------------
// Softmax family.
// ------------------------------------------------------------------------------------------
template <typename TX, typename TY, int VEC, int ITERS>
__global__ __launch_bounds__(1024) void softmax_fwd_kernel(
    const TX* __restrict__ x, TY* __restrict__ y, int64_t batch, int feat, int64_t xs, int64_t ys,
    int neg, int log, int group_log2) {
  __shared__ float scratch[16];
  const int group = 1 << group_log2;
  const int lane = threadIdx.x & (group - 1);
  const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> group_log2) + (threadIdx.x >> group_log2);
  const bool valid = row < batch;
  const int chunks = feat / VEC;
  const int n_it = ITERS > 0 ? ITERS : (chunks + group - 1) / group;
  const TX* xr = x + (valid ? row : 0) * xs;
  const float sign = neg ? -1.f : 1.f;
  float cache[cache_len<ITERS>()][VEC];

  float m = -INFINITY;
#pragma unroll
  for (int it = 0; it < n_it; ++it) {
    const int c = lane + it * group;
    float v[VEC];
    if (valid && c < chunks) {
      load_f32<TX, VEC>(xr + (int64_t)c * VEC, v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] *= sign;
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) v[j] = -INFINITY;
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      m = fmaxf(m, v[j]);
      if (ITERS > 0) cache[ITERS > 0 ? it : 0][j] = v[j];
    }
  }
  m = group_reduce(m, group, scratch, MaxOp(), -INFINITY);

  float s = 0.f;
#pragma unroll
  for (int it = 0; it < n_it; ++it) {
    const int c = lane + it * group;
    if (ITERS > 0) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float d = cache[ITERS > 0 ? it : 0][j] - m;
        const float e = __expf(d);
        s += e;
        cache[ITERS > 0 ? it : 0][j] = log ? d : e;
      }
    } else if (valid && c < chunks) {
      float v[VEC];
      load_f32<TX, VEC>(xr + (int64_t)c * VEC, v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) s += __expf(v[j] * sign - m);
    }
  }
  s = group_reduce(s, group, scratch, SumOp(), 0.f);
  if (!valid) return;
  const float inv = 1.0f / s;
  const float lg = __logf(s);

  TY* yr = y + row * ys;
#pragma unroll
  for (int it = 0; it < n_it; ++it) {
    const int c = lane + it * group;
    if (c < chunks) {
      float v[VEC];
      if (ITERS > 0) {
#pragma unroll
        for (int j = 0; j < VEC; ++j)
          v[j] = log ? cache[ITERS > 0 ? it : 0][j] - lg : cache[ITERS > 0 ? it : 0][j] * inv;
      } else {
        load_f32<TX, VEC>(xr + (int64_t)c * VEC, v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float d = v[j] * sign - m;
          v[j] = log ? d - lg : __expf(d) * inv;
        }
      }
      store_f32<TY, VEC>(yr + (int64_t)c * VEC, v);
    }
  }
}

template <typename TDY, typename TY, typename TDX, int VEC, int ITERS>
__global__ __launch_bounds__(1024) void softmax_bwd_kernel(
    const TDY* __restrict__ dy, const TY* __restrict__ y, TDX* __restrict__ dx, int64_t batch,
    int feat, int64_t dys, int64_t ys, int64_t dxs, int neg, int log, int group_log2) {
  __shared__ float scratch[16];
  const int group = 1 << group_log2;
  const int lane = threadIdx.x & (group - 1);
  const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> group_log2) + (threadIdx.x >> group_log2);
  const bool valid = row < batch;
  const int chunks = feat / VEC;
  const int n_it = ITERS > 0 ? ITERS : (chunks + group - 1) / group;
  const int64_t rr = valid ? row : 0;
  const TDY* dyr = dy + rr * dys;
  const TY* yr = y + rr * ys;
  float cdy[cache_len<ITERS>()][VEC], cy[cache_len<ITERS>()][VEC];

  float s = 0.f;
#pragma unroll
  for (int it = 0; it < n_it; ++it) {
    const int c = lane + it * group;
    float dv[VEC], yv[VEC];
    if (valid && c < chunks) {
      load_f32<TDY, VEC>(dyr + (int64_t)c * VEC, dv);
      load_f32<TY, VEC>(yr + (int64_t)c * VEC, yv);
    } else {
#pragma unroll
      for (int j = 0; j < VEC; ++j) { dv[j] = 0.f; yv[j] = 0.f; }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      s += log ? dv[j] : dv[j] * yv[j];
      if (ITERS > 0) { cdy[ITERS > 0 ? it : 0][j] = dv[j]; cy[ITERS > 0 ? it : 0][j] = yv[j]; }
    }
  }
  s = group_reduce(s, group, scratch, SumOp(), 0.f);
  if (!valid) return;
  const float sign = neg ? -1.f : 1.f;

  TDX* dxr = dx + row * dxs;
#pragma unroll
  for (int it = 0; it < n_it; ++it) {
    const int c = lane + it * group;
    if (c < chunks) {
      float dv[VEC], yv[VEC], o[VEC];
      if (ITERS > 0) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) { dv[j] = cdy[ITERS > 0 ? it : 0][j]; yv[j] = cy[ITERS > 0 ? it : 0][j]; }
      } else {
        load_f32<TDY, VEC>(dyr + (int64_t)c * VEC, dv);
        load_f32<TY, VEC>(yr + (int64_t)c * VEC, yv);
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j)
        o[j] = sign * (log ? dv[j] - __expf(yv[j]) * s : yv[j] * (dv[j] - s));
      store_f32<TDX, VEC>(dxr + (int64_t)c * VEC, o);
    }
  }
}

// ------------------------------------------------------------------------------------------
// Host-side dispatch.
// ------------------------------------------------------------------------------------------
inline bool rows_vectorizable(const void* p, int64_t stride, int dt) {
  return aligned16(p) && ((stride * dtype_size(dt)) & 15) == 0;
}

inline int narrow_vec(int dt_a, int dt_b, int dt_c) {
  // chunk = one 128-bit access of the narrowest dtype involved
  return (dt_a == AT_DTYPE_F32 && dt_b == AT_DTYPE_F32 && dt_c == AT_DTYPE_F32) ? 4 : 8;
}

#define AT_DISPATCH_ITERS(ITERS_VALUE, ...)                       \
  switch (ITERS_VALUE) {                                           \
    case 1: { constexpr int ITERS = 1; __VA_ARGS__; break; }       \
    case 2: { constexpr int ITERS = 2; __VA_ARGS__; break; }       \
    case 4: { constexpr int ITERS = 4; __VA_ARGS__; break; }       \
    case 8: { constexpr int ITERS = 8; __VA_ARGS__; break; }       \
    default: { constexpr int ITERS = 0; __VA_ARGS__; break; }      \
  }

#define AT_DISPATCH_ITERS_CACHED(ITERS_VALUE, ...)                 \
  switch (ITERS_VALUE) {                                           \
    case 1: { constexpr int ITERS = 1; __VA_ARGS__; break; }       \
    case 2: { constexpr int ITERS = 2; __VA_ARGS__; break; }       \
    case 4: { constexpr int ITERS = 4; __VA_ARGS__; break; }       \
    default: { constexpr int ITERS = 8; __VA_ARGS__; break; }      \
  }

// Allowed (in, out) storage pairs: out == in, or out == fp32 (autocast-to-fp32 policy).
template <typename F>
inline int dispatch_pair(int in_dt, int out_dt, F&& f) {
  if (in_dt == AT_DTYPE_F32 && out_dt == AT_DTYPE_F32) return f((float*)0, (float*)0);
  if (in_dt == AT_DTYPE_F16 && out_dt == AT_DTYPE_F16) return f((f16_t*)0, (f16_t*)0);
  if (in_dt == AT_DTYPE_F16 && out_dt == AT_DTYPE_F32) return f((f16_t*)0, (float*)0);
  if (in_dt == AT_DTYPE_BF16 && out_dt == AT_DTYPE_BF16) return f((bf16_t*)0, (bf16_t*)0);
  if (in_dt == AT_DTYPE_BF16 && out_dt == AT_DTYPE_F32) return f((bf16_t*)0, (float*)0);
  return AT_ERR_DTYPE;
}

inline int check_rows(int64_t batch, int64_t feat, int64_t s0, int64_t s1, int64_t s2) {
  if (batch < 0 || feat <= 0 || feat > (int64_t)1 << 30) return AT_ERR_DIM;
  if (s0 < feat || s1 < feat || s2 < feat) return AT_ERR_DIM;
  return AT_OK;
}

template <bool LAYER>
int norm_fwd(const void* x, const void* weight, const void* bias, float* mean, float* rstd, void* y,
             int64_t batch, int64_t feat, int64_t xs, int64_t ys, float eps, int xdt, int wdt,
             int ydt, hipStream_t stream) {
  if (!x || !y) return AT_ERR_NULL;
  if (!dtype_valid(xdt) || !dtype_valid(ydt) || (weight && !dtype_valid(wdt))) return AT_ERR_DTYPE;
  int rc = check_rows(batch, feat, xs, ys, feat);
  if (rc) return rc;
  if (batch == 0) return AT_OK;
  if (!weight) bias = nullptr;
  int vec = narrow_vec(xdt, ydt, AT_DTYPE_F32);
  const bool vector_ok = feat % vec == 0 && rows_vectorizable(x, xs, xdt) &&
                         rows_vectorizable(y, ys, ydt) && (!weight || aligned16(weight)) &&
                         (!bias || aligned16(bias));
  if (!vector_ok) vec = 1;
  const RowPlan p = plan_rows(feat, vec, 256, 8, 1024);
  const int rpb = p.block >> p.group_log2;
  const dim3 grid((unsigned)cdiv64(batch, rpb));
  return dispatch_pair(xdt, ydt, [&](auto* tx, auto* ty) -> int {
    typedef std::remove_pointer_t<decltype(tx)> TX;
    typedef std::remove_pointer_t<decltype(ty)> TY;
    constexpr int VECW = sizeof(TX) == 4 && sizeof(TY) == 4 ? 4 : 8;
    if (vec != 1) {
      AT_DISPATCH_ITERS(p.iters, hipLaunchKernelGGL((norm_fwd_kernel<LAYER, TX, TY, VECW, ITERS>), grid,
                                                    dim3(p.block), 0, stream, (const TX*)x, weight, bias,
                                                    mean, rstd, (TY*)y, batch, (int)feat, xs, ys, eps,
                                                    wdt, p.group_log2));
    } else {
      AT_DISPATCH_ITERS(p.iters, hipLaunchKernelGGL((norm_fwd_kernel<LAYER, TX, TY, 1, ITERS>), grid,
                                                    dim3(p.block), 0, stream, (const TX*)x, weight, bias,
                                                    mean, rstd, (TY*)y, batch, (int)feat, xs, ys, eps,
                                                    wdt, p.group_log2));
    }
    return launch_status();
  });
}

constexpr int kBwdBlock = 512;        // 8 waves: room for 256 VGPRs per lane
constexpr int kStreamSlices = 256;    // row slices of the column kernel in the streaming fallback
constexpr int kMaxPartialRows = 1024; // upper bound on partial rows (CU count or kStreamSlices)

inline int bwd_grid_blocks(int64_t row_blocks) {
  int64_t cap = (int64_t)device_cu_count();
  if (cap > kMaxPartialRows) cap = kMaxPartialRows;
  return (int)(row_blocks < cap ? row_blocks : cap);
}

template <bool LAYER>
int norm_bwd(const void* dy, const void* x, const float* mean, const float* rstd, const void* weight,
             void* dx, float* weight_grad, float* bias_grad, void* workspace, int64_t workspace_bytes,
             int64_t batch, int64_t feat, int64_t dys, int64_t xs, int64_t dxs, int dydt, int xdt,
             int wdt, int dxdt, hipStream_t stream) {
  if (!dy || !x || !rstd || !dx || (LAYER && !mean)) return AT_ERR_NULL;
  if (!dtype_valid(dydt) || !dtype_valid(xdt) || !dtype_valid(dxdt) || (weight && !dtype_valid(wdt)))
    return AT_ERR_DTYPE;
  if (dxdt != dydt) return AT_ERR_DTYPE;  // the input gradient is produced in the output dtype
  int rc = check_rows(batch, feat, dys, xs, dxs);
  if (rc) return rc;
  if (!LAYER) bias_grad = nullptr;
  const int n_grads = (weight_grad ? 1 : 0) + (bias_grad ? 1 : 0);
  if (bias_grad && !weight_grad) return AT_ERR_NULL;
  if (n_grads) {
    if (!workspace) return AT_ERR_WORKSPACE;
    if (workspace_bytes < at_norm_bwd_workspace_bytes(batch, feat, n_grads)) return AT_ERR_WORKSPACE;
  }
  if (batch == 0) {
    if (n_grads)  // zero partial rows: the reduction writes exact zeros
      hipLaunchKernelGGL(reduce_partials_kernel, dim3((unsigned)cdiv64(feat, 64), bias_grad ? 2 : 1),
                         dim3(256), 0, stream, (const float*)workspace, weight_grad,
                         (const float*)workspace, bias_grad, 0, (int)feat);
    return launch_status();
  }
  int vec = narrow_vec(dydt, xdt, dxdt);
  const bool vector_ok = feat % vec == 0 && rows_vectorizable(dy, dys, dydt) &&
                         rows_vectorizable(x, xs, xdt) && rows_vectorizable(dx, dxs, dxdt) &&
                         (!weight || aligned16(weight));
  if (!vector_ok) vec = 1;
  const RowPlan p = plan_rows(feat, vec, kBwdBlock, vec == 4 ? 8 : 4, kBwdBlock);
  float* part_w = weight_grad ? (float*)workspace : nullptr;
  int parts = 0;

  rc = dispatch_pair(xdt, dydt, [&](auto* tx, auto* tdy) -> int {
    typedef std::remove_pointer_t<decltype(tx)> TX;
    typedef std::remove_pointer_t<decltype(tdy)> TDY;
    constexpr int VECW = sizeof(TX) == 4 && sizeof(TDY) == 4 ? 4 : 8;
    if (p.iters != 0) {
      const int rpb = p.block >> p.group_log2;
      parts = bwd_grid_blocks(cdiv64(batch, rpb));
      float* part_b = bias_grad ? part_w + (int64_t)parts * feat : nullptr;
      if (vec != 1) {
        const size_t lds = rpb > 1 ? (size_t)p.block * VECW * sizeof(float) : 0;
        AT_DISPATCH_ITERS_CACHED(p.iters, hipLaunchKernelGGL(
            (norm_bwd_kernel<LAYER, TDY, TX, TDY, VECW, ITERS>), dim3(parts), dim3(p.block), lds, stream,
            (const TDY*)dy, (const TX*)x, mean, rstd, weight, (TDY*)dx, part_w, part_b, batch, (int)feat,
            dys, xs, dxs, wdt, p.group_log2));
      } else {
        const size_t lds = rpb > 1 ? (size_t)p.block * sizeof(float) : 0;
        AT_DISPATCH_ITERS_CACHED(p.iters, hipLaunchKernelGGL(
            (norm_bwd_kernel<LAYER, TDY, TX, TDY, 1, ITERS>), dim3(parts), dim3(p.block), lds, stream,
            (const TDY*)dy, (const TX*)x, mean, rstd, weight, (TDY*)dx, part_w, part_b, batch, (int)feat,
            dys, xs, dxs, wdt, p.group_log2));
      }
    } else {
      if (vec != 1)
        hipLaunchKernelGGL((norm_bwd_stream_kernel<LAYER, TDY, TX, TDY, VECW>), dim3((unsigned)batch),
                           dim3(1024), 0, stream, (const TDY*)dy, (const TX*)x, mean, rstd, weight,
                           (TDY*)dx, batch, (int)feat, dys, xs, dxs, wdt);
      else
        hipLaunchKernelGGL((norm_bwd_stream_kernel<LAYER, TDY, TX, TDY, 1>), dim3((unsigned)batch),
                           dim3(1024), 0, stream, (const TDY*)dy, (const TX*)x, mean, rstd, weight,
                           (TDY*)dx, batch, (int)feat, dys, xs, dxs, wdt);
      if (n_grads) {
        parts = (int)(batch < kStreamSlices ? batch : kStreamSlices);
        const int64_t rows_per_slice = cdiv64(batch, parts);
        parts = (int)cdiv64(batch, rows_per_slice);
        float* part_b = bias_grad ? part_w + (int64_t)parts * feat : nullptr;
        hipLaunchKernelGGL((norm_param_grad_cols_kernel<LAYER, TDY, TX>),
                           dim3((unsigned)cdiv64(feat, 256), parts), dim3(256), 0, stream,
                           (const TDY*)dy, (const TX*)x, mean, rstd, part_w, part_b, batch, (int)feat,
                           dys, xs, rows_per_slice);
      }
    }
    return launch_status();
  });
  if (rc) return rc;
  if (n_grads) {
    float* part_b = bias_grad ? part_w + (int64_t)parts * feat : nullptr;
    hipLaunchKernelGGL(reduce_partials_kernel, dim3((unsigned)cdiv64(feat, 64), bias_grad ? 2 : 1),
                       dim3(256), 0, stream, part_w, weight_grad, part_b, bias_grad, parts, (int)feat);
    rc = launch_status();
  }
  return rc;
}

}  // namespace
}  // namespace at_hip

using namespace at_hip;

extern "C" {

int64_t at_norm_bwd_workspace_bytes(int64_t batch, int64_t feat, int n_param_grads) {
  if (batch < 0 || feat <= 0 || n_param_grads <= 0) return 0;
  const int64_t rows = batch < kMaxPartialRows ? (batch > 0 ? batch : 1) : kMaxPartialRows;
  return rows * feat * (int64_t)sizeof(float) * n_param_grads;
}

int at_rms_norm_fwd(const void* x, const void* weight, float* inv_rms, void* y, int64_t batch,
                    int64_t feat, int64_t x_stride, int64_t y_stride, float eps, int x_dtype,
                    int weight_dtype, int y_dtype, at_stream_t stream) {
  return norm_fwd<false>(x, weight, nullptr, nullptr, inv_rms, y, batch, feat, x_stride, y_stride, eps,
                         x_dtype, weight_dtype, y_dtype, (hipStream_t)stream);
}

int at_rms_norm_bwd(const void* dy, const void* x, const float* inv_rms, const void* weight, void* dx,
                    float* weight_grad, void* workspace, int64_t workspace_bytes, int64_t batch,
                    int64_t feat, int64_t dy_stride, int64_t x_stride, int64_t dx_stride, int dy_dtype,
                    int x_dtype, int weight_dtype, int dx_dtype, at_stream_t stream) {
  return norm_bwd<false>(dy, x, nullptr, inv_rms, weight, dx, weight_grad, nullptr, workspace,
                         workspace_bytes, batch, feat, dy_stride, x_stride, dx_stride, dy_dtype, x_dtype,
                         weight_dtype, dx_dtype, (hipStream_t)stream);
}

int at_layer_norm_fwd(const void* x, const void* weight, const void* bias, float* mean, float* inv_std,
                      void* y, int64_t batch, int64_t feat, int64_t x_stride, int64_t y_stride,
                      float eps, int x_dtype, int weight_dtype, int y_dtype, at_stream_t stream) {
  return norm_fwd<true>(x, weight, bias, mean, inv_std, y, batch, feat, x_stride, y_stride, eps, x_dtype,
                        weight_dtype, y_dtype, (hipStream_t)stream);
}

int at_layer_norm_bwd(const void* dy, const void* x, const float* mean, const float* inv_std,
                      const void* weight, void* dx, float* weight_grad, float* bias_grad, void* workspace,
                      int64_t workspace_bytes, int64_t batch, int64_t feat, int64_t dy_stride,
                      int64_t x_stride, int64_t dx_stride, int dy_dtype, int x_dtype, int weight_dtype,
                      int dx_dtype, at_stream_t stream) {
  return norm_bwd<true>(dy, x, mean, inv_std, weight, dx, weight_grad, bias_grad, workspace,
                        workspace_bytes, batch, feat, dy_stride, x_stride, dx_stride, dy_dtype, x_dtype,
                        weight_dtype, dx_dtype, (hipStream_t)stream);
}

int at_softmax_fwd(const void* x, void* y, int64_t batch, int64_t feat, int64_t x_stride,
                   int64_t y_stride, int neg, int log, int x_dtype, int y_dtype, at_stream_t stream) {
  if (!x || !y) return AT_ERR_NULL;
  if (!dtype_valid(x_dtype) || !dtype_valid(y_dtype)) return AT_ERR_DTYPE;
  int rc = check_rows(batch, feat, x_stride, y_stride, feat);
  if (rc) return rc;
  if (batch == 0) return AT_OK;
  int vec = narrow_vec(x_dtype, y_dtype, AT_DTYPE_F32);
  if (!(feat % vec == 0 && rows_vectorizable(x, x_stride, x_dtype) && rows_vectorizable(y, y_stride, y_dtype)))
    vec = 1;
  const RowPlan p = plan_rows(feat, vec, 256, 8, 1024);
  const dim3 grid((unsigned)cdiv64(batch, p.block >> p.group_log2));
  return dispatch_pair(x_dtype, y_dtype, [&](auto* tx, auto* ty) -> int {
    typedef std::remove_pointer_t<decltype(tx)> TX;
    typedef std::remove_pointer_t<decltype(ty)> TY;
    constexpr int VECW = sizeof(TX) == 4 && sizeof(TY) == 4 ? 4 : 8;
    if (vec != 1) {
      AT_DISPATCH_ITERS(p.iters, hipLaunchKernelGGL((softmax_fwd_kernel<TX, TY, VECW, ITERS>), grid,
                                                    dim3(p.block), 0, (hipStream_t)stream, (const TX*)x,
                                                    (TY*)y, batch, (int)feat, x_stride, y_stride, neg,
                                                    log, p.group_log2));
    } else {
      AT_DISPATCH_ITERS(p.iters, hipLaunchKernelGGL((softmax_fwd_kernel<TX, TY, 1, ITERS>), grid,
                                                    dim3(p.block), 0, (hipStream_t)stream, (const TX*)x,
                                                    (TY*)y, batch, (int)feat, x_stride, y_stride, neg,
                                                    log, p.group_log2));
    }
    return launch_status();
  });
}

int at_softmax_bwd(const void* dy, const void* y, void* dx, int64_t batch, int64_t feat,
                   int64_t dy_stride, int64_t y_stride, int64_t dx_stride, int neg, int log,
                   int dy_dtype, int y_dtype, int dx_dtype, at_stream_t stream) {
  if (!dy || !y || !dx) return AT_ERR_NULL;
  if (!dtype_valid(dy_dtype) || !dtype_valid(y_dtype) || !dtype_valid(dx_dtype)) return AT_ERR_DTYPE;
  if (dx_dtype != y_dtype) return AT_ERR_DTYPE;  // input_grad = empty_like(output), softmax_layers.py:78
  int rc = check_rows(batch, feat, dy_stride, y_stride, dx_stride);
  if (rc) return rc;
  if (batch == 0) return AT_OK;
  int vec = narrow_vec(dy_dtype, y_dtype, dx_dtype);
  if (!(feat % vec == 0 && rows_vectorizable(dy, dy_stride, dy_dtype) &&
        rows_vectorizable(y, y_stride, y_dtype) && rows_vectorizable(dx, dx_stride, dx_dtype)))
    vec = 1;
  const RowPlan p = plan_rows(feat, vec, 256, vec == 4 ? 8 : 4, 1024);
  const dim3 grid((unsigned)cdiv64(batch, p.block >> p.group_log2));
  return dispatch_pair(dy_dtype, y_dtype, [&](auto* tdy, auto* ty) -> int {
    typedef std::remove_pointer_t<decltype(tdy)> TDY;
    typedef std::remove_pointer_t<decltype(ty)> TY;
    constexpr int VECW = sizeof(TDY) == 4 && sizeof(TY) == 4 ? 4 : 8;
    if (vec != 1) {
      AT_DISPATCH_ITERS(p.iters, hipLaunchKernelGGL((softmax_bwd_kernel<TDY, TY, TY, VECW, ITERS>), grid,
                                                    dim3(p.block), 0, (hipStream_t)stream, (const TDY*)dy,
                                                    (const TY*)y, (TY*)dx, batch, (int)feat, dy_stride,
                                                    y_stride, dx_stride, neg, log, p.group_log2));
    } else {
      AT_DISPATCH_ITERS(p.iters, hipLaunchKernelGGL((softmax_bwd_kernel<TDY, TY, TY, 1, ITERS>), grid,
                                                    dim3(p.block), 0, (hipStream_t)stream, (const TDY*)dy,
                                                    (const TY*)y, (TY*)dx, batch, (int)feat, dy_stride,
                                                    y_stride, dx_stride, neg, log, p.group_log2));
    }
    return launch_status();
  });
}

}  // extern "C"
