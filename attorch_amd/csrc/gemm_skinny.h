// Linear layers with at most 16 output features (classifier heads): the three products on vector
// ALUs.  A 64-wide matrix tile would be three quarters padding and, worse, such outputs give the
// tiled kernels a few dozen workgroups; these kernels are bound by reading (or writing) the wide
// [rows, features] operand once.
//   forward     : Y[m, n]  = act(sum_k X[m, k] W[k, n] + b[n])
//   input grad  : dX[m, k] = sum_n dZ[m, n] W[k, n]
//   weight grad : dW[k, n] = sum_m X[m, k] dZ[m, n]   (fp32 partials per slice of rows, summed in
//                                                      fixed order by gemm_split_finish_kernel)
// A lane owns 16 bytes (VEC elements) of the wide dimension k; the narrow operand (a chunk of W, or
// the dZ rows of a slice) sits in LDS as fp32.
#pragma once

#include "at_act.h"
#include "at_common.h"

namespace at_hip {
namespace {

constexpr int kSkinnyCols = 16;   // widest narrow dimension the kernels take
// Rows per workgroup.  Forward: one per wave, several workgroups per CU hide each other's load and
// reduction latencies.  Input gradient: four per wave, the staged weights serve more rows.
constexpr int kSkinnyRowsFwd = 4;
constexpr int kSkinnyRowsDx = 16;
constexpr int kSkinnySlice = 64;  // rows whose dZ is staged at once in the weight-gradient kernel
constexpr int kSkinnyMaxSlices = 128;

struct SkinnyArgs {
  const void* x;     // [M, K] rows, stride ldx (forward, weight gradient)
  const void* w;     // [K, N] rows, stride ldw (forward, input gradient)
  const void* dz;    // [M, N] rows, stride ldz (input gradient, weight gradient)
  void* out;         // Y [M, N] / dX [M, K] (stride ldo) / fp32 partials [slices][K][kSkinnyCols]
  void* pre_act;     // optional, stride ldp
  const void* bias;
  int bias_dt;
  int M, N, K;
  int64_t ldx, ldw, ldz, ldo, ldp;
  int act;
  float param;
  int rows_per_slice;
};

// W[k0 .. k0 + CH, 0 .. N) -> wl[n][k] as fp32 (zeros past K), by the whole workgroup.
template <typename T, int CH, int THREADS>
__device__ __forceinline__ void skinny_stage_w(const T* __restrict__ W, int64_t ldw, int k0, int K, int N,
                                               float (*wl)[CH + 4]) {
  // a lane takes whole rows k (N consecutive elements each): no index arithmetic beyond an add, and
  // consecutive lanes write consecutive LDS words
#pragma unroll
  for (int kk = 0; kk < CH / THREADS; ++kk) {
    const int k = threadIdx.x + kk * THREADS;
    const bool ok = k0 + k < K;
    const T* row = W + (int64_t)(ok ? k0 + k : 0) * ldw;
#pragma unroll
    for (int n = 0; n < kSkinnyCols; ++n)
      if (n < N) wl[n][k] = ok ? to_f32(row[n]) : 0.f;
  }
}

template <typename T, typename TO>
__global__ __launch_bounds__(256) void skinny_fwd_kernel(SkinnyArgs g) {
  constexpr int VEC = 16 / (int)sizeof(T), CH = 64 * VEC, RW = kSkinnyRowsFwd / 4;
  __shared__ __align__(16) float wl[kSkinnyCols][CH + 4];
  const T* __restrict__ X = reinterpret_cast<const T*>(g.x);
  const T* __restrict__ W = reinterpret_cast<const T*>(g.w);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row0 = (int64_t)blockIdx.x * kSkinnyRowsFwd + wave * RW;
  float acc[RW][kSkinnyCols];
#pragma unroll
  for (int r = 0; r < RW; ++r)
#pragma unroll
    for (int n = 0; n < kSkinnyCols; ++n) acc[r][n] = 0.f;

  for (int k0 = 0; k0 < g.K; k0 += CH) {
    // this chunk of the rows is requested first: it travels while the weights are staged
    const int k = k0 + lane * VEC;
    float xv[RW][VEC];
#pragma unroll
    for (int r = 0; r < RW; ++r) {
      if (row0 + r < g.M && k < g.K) {
        load_f32<T, VEC>(X + (row0 + r) * g.ldx + k, xv[r]);
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) xv[r][j] = 0.f;
      }
    }
    __syncthreads();   // the previous chunk has been read
    skinny_stage_w<T, CH, 256>(W, g.ldw, k0, g.K, g.N, wl);
    __syncthreads();
#pragma unroll
    for (int n = 0; n < kSkinnyCols; ++n) {
      if (n < g.N) {
        float wv[VEC];
#pragma unroll
        for (int j = 0; j < VEC; j += 4) {
          const float4 q = *reinterpret_cast<const float4*>(&wl[n][lane * VEC + j]);
          wv[j] = q.x; wv[j + 1] = q.y; wv[j + 2] = q.z; wv[j + 3] = q.w;
        }
#pragma unroll
        for (int r = 0; r < RW; ++r)
#pragma unroll
          for (int j = 0; j < VEC; ++j) acc[r][n] = fmaf(xv[r][j], wv[j], acc[r][n]);
      }
    }
  }

  TO* __restrict__ Y = reinterpret_cast<TO*>(g.out);
  TO* __restrict__ P = g.act != AT_ACT_NONE ? reinterpret_cast<TO*>(g.pre_act) : nullptr;
#pragma unroll
  for (int r = 0; r < RW; ++r) {
    float mine = 0.f;   // lane n keeps column n of this row
#pragma unroll
    for (int n = 0; n < kSkinnyCols; ++n) {
      if (n < g.N) {
        const float s = wave_reduce(acc[r][n], kWave, SumOp());
        if (lane == n) mine = s;
      }
    }
    const int64_t row = row0 + r;
    if (lane < g.N && row < g.M) {
      float v = mine + (g.bias ? load_scalar_f32(g.bias, g.bias_dt, lane) : 0.f);
      if (P) P[row * g.ldp + lane] = from_f32<TO>(v);
      if (g.act != AT_ACT_NONE) v = act_forward(g.act, v, g.param);
      Y[row * g.ldo + lane] = from_f32<TO>(v);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void skinny_dx_kernel(SkinnyArgs g) {
  constexpr int VEC = 16 / (int)sizeof(T), CH = 64 * VEC, RW = kSkinnyRowsDx / 4;
  __shared__ __align__(16) float wl[kSkinnyCols][CH + 4];
  __shared__ float dzl[kSkinnyRowsDx][kSkinnyCols];
  const T* __restrict__ W = reinterpret_cast<const T*>(g.w);
  const T* __restrict__ dZ = reinterpret_cast<const T*>(g.dz);
  T* __restrict__ dX = reinterpret_cast<T*>(g.out);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t block_row = (int64_t)blockIdx.x * kSkinnyRowsDx;
  if (threadIdx.x < kSkinnyRowsDx * kSkinnyCols) {
    const int r = threadIdx.x / kSkinnyCols, n = threadIdx.x % kSkinnyCols;
    dzl[r][n] = (block_row + r < g.M && n < g.N) ? to_f32(dZ[(block_row + r) * g.ldz + n]) : 0.f;
  }
  for (int k0 = 0; k0 < g.K; k0 += CH) {
    __syncthreads();
    skinny_stage_w<T, CH, 256>(W, g.ldw, k0, g.K, g.N, wl);
    __syncthreads();
    const int k = k0 + lane * VEC;
    float out[RW][VEC];
#pragma unroll
    for (int r = 0; r < RW; ++r)
#pragma unroll
      for (int j = 0; j < VEC; ++j) out[r][j] = 0.f;
#pragma unroll
    for (int n = 0; n < kSkinnyCols; ++n) {
      if (n < g.N) {
        float wv[VEC];
#pragma unroll
        for (int j = 0; j < VEC; j += 4) {
          const float4 q = *reinterpret_cast<const float4*>(&wl[n][lane * VEC + j]);
          wv[j] = q.x; wv[j + 1] = q.y; wv[j + 2] = q.z; wv[j + 3] = q.w;
        }
#pragma unroll
        for (int r = 0; r < RW; ++r) {
          const float d = dzl[wave * RW + r][n];
#pragma unroll
          for (int j = 0; j < VEC; ++j) out[r][j] = fmaf(d, wv[j], out[r][j]);
        }
      }
    }
    if (k < g.K) {
#pragma unroll
      for (int r = 0; r < RW; ++r) {
        const int64_t row = block_row + wave * RW + r;
        if (row < g.M) store_f32<T, VEC>(dX + row * g.ldo + k, out[r]);
      }
    }
  }
}

// grid (cdiv(K, 64 VEC), slices).  The four waves of a workgroup own the same 64 VEC columns k and
// take every fourth row of the slice; their accumulators are added through LDS in four passes, wave
// p finishing the p-th quarter of the VEC x 16 values per lane.
template <typename T>
__global__ __launch_bounds__(256) void skinny_dw_kernel(SkinnyArgs g) {
  constexpr int VEC = 16 / (int)sizeof(T);
  constexpr int QUARTER = VEC * kSkinnyCols / 4;   // accumulators per lane and pass
  __shared__ float dzl[kSkinnySlice][kSkinnyCols];
  __shared__ float fold[4][QUARTER][64];
  const T* __restrict__ X = reinterpret_cast<const T*>(g.x);
  const T* __restrict__ dZ = reinterpret_cast<const T*>(g.dz);
  float* __restrict__ part = reinterpret_cast<float*>(g.out);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int k = (blockIdx.x * 64 + lane) * VEC;
  const bool k_ok = k < g.K;
  const int64_t m_begin = (int64_t)blockIdx.y * g.rows_per_slice;
  const int64_t m_end = m_begin + g.rows_per_slice < g.M ? m_begin + g.rows_per_slice : g.M;
  float acc[VEC * kSkinnyCols];   // [j][n]
#pragma unroll
  for (int i = 0; i < VEC * kSkinnyCols; ++i) acc[i] = 0.f;

  for (int64_t mb = m_begin; mb < m_end; mb += kSkinnySlice) {
    const int rows = (int)(m_end - mb < kSkinnySlice ? m_end - mb : kSkinnySlice);
    __syncthreads();
#pragma unroll 4
    for (int e = threadIdx.x; e < kSkinnySlice * kSkinnyCols; e += 256) {
      const int r = e / kSkinnyCols, n = e % kSkinnyCols;
      dzl[r][n] = (r < rows && n < g.N) ? to_f32(dZ[(mb + r) * g.ldz + n]) : 0.f;
    }
    __syncthreads();
    constexpr int U = 4;   // rows in flight per wave: r = wave + 4 (r0 + u)
    for (int r0 = 0; r0 < kSkinnySlice / 4; r0 += U) {
      float xv[U][VEC];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int r = wave + 4 * (r0 + u);
        if (k_ok && r < rows) {
          load_f32<T, VEC>(X + (mb + r) * g.ldx + k, xv[u]);
        } else {
#pragma unroll
          for (int j = 0; j < VEC; ++j) xv[u][j] = 0.f;
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int r = wave + 4 * (r0 + u);   // rows past the end were staged as zeros
#pragma unroll
        for (int n = 0; n < kSkinnyCols; ++n) {
          if (n < g.N) {
            const float d = dzl[r][n];
#pragma unroll
            for (int j = 0; j < VEC; ++j) acc[j * kSkinnyCols + n] = fmaf(xv[u][j], d, acc[j * kSkinnyCols + n]);
          }
        }
      }
    }
  }
  float mine[QUARTER];
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < QUARTER; ++i) fold[wave][i][lane] = acc[pass * QUARTER + i];
    __syncthreads();
    if (wave == pass) {
#pragma unroll
      for (int i = 0; i < QUARTER; ++i)
        mine[i] = (fold[0][i][lane] + fold[1][i][lane]) + (fold[2][i][lane] + fold[3][i][lane]);
    }
  }
  if (k_ok) {
    // wave p holds [j][n] for the flat indices p * QUARTER ... of the lane's VEC x 16 block
    float* dst = part + ((int64_t)blockIdx.y * g.K + k) * kSkinnyCols + wave * QUARTER;
#pragma unroll
    for (int i = 0; i < QUARTER; i += 4)
      *reinterpret_cast<float4*>(dst + i) = make_float4(mine[i], mine[i + 1], mine[i + 2], mine[i + 3]);
  }
}

// Rows of the wide operand per slice of the weight gradient, and the slice count that follows.
inline int64_t skinny_rows_per_slice(int64_t M) {
  int64_t rows = cdiv64(M, kSkinnyMaxSlices);
  rows = cdiv64(rows, kSkinnySlice) * kSkinnySlice;
  return rows < kSkinnySlice ? kSkinnySlice : rows;
}

inline int64_t skinny_dw_workspace_bytes(int64_t M, int64_t K) {
  return cdiv64(M, skinny_rows_per_slice(M)) * K * kSkinnyCols * (int64_t)sizeof(float);
}

// Whether the wide operand (rows of `wide` elements, stride ld) allows the 16-byte lane accesses.
inline bool skinny_rows_ok(const void* p, int64_t wide, int64_t ld, int dt) {
  const int vec = 16 / dtype_size(dt);
  return aligned16(p) && wide % vec == 0 && ld % vec == 0 && wide >= 4 * 64;
}

}  // namespace
}  // namespace at_hip
