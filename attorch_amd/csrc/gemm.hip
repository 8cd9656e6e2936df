// Linear layer GEMMs: Y = act(X W + b) and the two backward products, fp32 accumulate.
//
// Two kernels:
//  * gemm_mfma16_kernel — bf16/fp16 operands on v_mfma_f32_32x32x16 (MFMA-bound).  256x256x64
//    macro-tile per 256-lane workgroup (4 waves, 128x128 each, 256 accumulator registers per
//    lane), LDS double-buffered (2 x 64 KiB), one barrier per k-tile, global loads of tile
//    k+1 in flight while tile k is multiplied.  LDS tiles are [row][k] with the 16-byte chunk
//    index XOR-swizzled by the row, so both the 128-bit fragment reads and the tile writes are
//    bank-conflict free.  Operands whose contraction index is not the contiguous one in
//    memory (W in the forward product, X and dZ in the weight gradient) are transposed 8x8 in
//    registers (byte permutes) between the global load and the LDS write.  Workgroup ids are
//    remapped so that each XCD (own L2) works on a compact block of output tiles.
//  * gemm_simple_kernel — any dtype, any strides, fp32 MFMA (32x32x2), 64x64 tile; used for
//    fp32 tensors and for 16-bit shapes the fast kernel cannot address with 128-bit accesses.
// Both fuse bias, the optional pre-activation store and the activation into the epilogue.
#include <type_traits>

#include "at_act.h"
#include "at_common.h"

namespace at_hip {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

struct GemmArgs {
  const void* a;      // A(m, k)
  const void* b;      // B(k, n)
  void* c;            // C[m, n], row stride ldc
  void* pre_act;      // optional copy of the accumulator before the activation, row stride ldp
  const void* bias;   // optional [n]
  int M, N, K;
  int64_t lda, ldb, ldc, ldp;  // A: row stride of [M,K] (KC) or of [K,M] (MC); B: of [K,N] (NC) or [N,K] (KC)
  int act;
  float param;
  int bias_dt;
};

template <typename T> struct Mfma16;
template <> struct Mfma16<bf16_t> {
  static __device__ __forceinline__ f32x16 run(const uint4& a, const uint4& b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b),
                                                   c, 0, 0, 0);
  }
};
template <> struct Mfma16<f16_t> {
  static __device__ __forceinline__ f32x16 run(const uint4& a, const uint4& b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b),
                                                  c, 0, 0, 0);
  }
};

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kGemmThreads = 256;
constexpr int kTileBytes = BM * BK * 2;  // one operand tile, 32 KiB

// Byte offset of 16-byte chunk `chunk` (0..7) of row `row` inside a [256][64] 16-bit tile.
__device__ __forceinline__ int lds_chunk_offset(int row, int chunk) {
  return row * (BK * 2) + ((chunk ^ ((row ^ (row >> 3)) & 7)) << 4);
}

// 8x8 transpose of 16-bit elements held as 8 rows of 128 bits: out[c] = column c.
__device__ __forceinline__ void transpose8x8(const uint4 (&in)[8], uint4 (&out)[8]) {
  const uint32_t w[8][4] = {{in[0].x, in[0].y, in[0].z, in[0].w}, {in[1].x, in[1].y, in[1].z, in[1].w},
                            {in[2].x, in[2].y, in[2].z, in[2].w}, {in[3].x, in[3].y, in[3].z, in[3].w},
                            {in[4].x, in[4].y, in[4].z, in[4].w}, {in[5].x, in[5].y, in[5].z, in[5].w},
                            {in[6].x, in[6].y, in[6].z, in[6].w}, {in[7].x, in[7].y, in[7].z, in[7].w}};
#pragma unroll
  for (int c = 0; c < 8; ++c) {
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // rows 2j (low half) and 2j+1 (high half), column c lives in word c/2, half c%2
      o[j] = (c & 1) ? __builtin_amdgcn_perm(w[2 * j + 1][c >> 1], w[2 * j][c >> 1], 0x07060302u)
                     : __builtin_amdgcn_perm(w[2 * j + 1][c >> 1], w[2 * j][c >> 1], 0x05040100u);
    }
    out[c] = make_uint4(o[0], o[1], o[2], o[3]);
  }
}

// Operand staging.  CONTRACT_CONTIG: memory is [outer][k] (k contiguous); otherwise [k][outer].
template <typename T, bool CONTRACT_CONTIG>
struct OperandStage {
  uint4 r[8];

  __device__ __forceinline__ void load(const T* __restrict__ base, int64_t ld, int outer0, int outer_total,
                                       int k0, int K) {
    const int t = threadIdx.x;
    if (CONTRACT_CONTIG) {
      const int c = t & 7;
      const int k = k0 + c * 8;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int o = outer0 + (t >> 3) + 32 * i;
        r[i] = (o < outer_total && k < K) ? *reinterpret_cast<const uint4*>(base + (int64_t)o * ld + k)
                                          : make_uint4(0, 0, 0, 0);
      }
    } else {
      const int o = outer0 + (t & 31) * 8;
      const int kb = k0 + (t >> 5) * 8;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int k = kb + i;
        r[i] = (o < outer_total && k < K) ? *reinterpret_cast<const uint4*>(base + (int64_t)k * ld + o)
                                          : make_uint4(0, 0, 0, 0);
      }
    }
  }

  __device__ __forceinline__ void store(char* tile) const {
    const int t = threadIdx.x;
    if (CONTRACT_CONTIG) {
      const int c = t & 7;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int row = (t >> 3) + 32 * i;
        *reinterpret_cast<uint4*>(tile + lds_chunk_offset(row, c)) = r[i];
      }
    } else {
      uint4 tr[8];
      transpose8x8(r, tr);
      const int chunk = t >> 5;
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const int row = (t & 31) * 8 + c;
        *reinterpret_cast<uint4*>(tile + lds_chunk_offset(row, chunk)) = tr[c];
      }
    }
  }
};

// ACT is the compile-time activation id of the epilogue (the act switch must fold away: the
// epilogue is fully unrolled over 256 accumulator registers).
template <typename T, bool A_MC, bool B_KC, int ACT>
__global__ __launch_bounds__(kGemmThreads) void gemm_mfma16_kernel(GemmArgs g) {
  __shared__ __attribute__((aligned(16))) char lds[4 * kTileBytes];  // [stage][A|B]
  const T* __restrict__ A = reinterpret_cast<const T*>(g.a);
  const T* __restrict__ B = reinterpret_cast<const T*>(g.b);

  // ---- workgroup -> output tile, XCD aware ----
  const int nbm = (g.M + BM - 1) / BM, nbn = (g.N + BN - 1) / BN;
  const int total = nbm * nbn;
  int logical;
  {
    const int bid = blockIdx.x, xcd = bid & 7, idx = bid >> 3;
    const int q = total >> 3, rem = total & 7;
    logical = xcd * q + (xcd < rem ? xcd : rem) + idx;
  }
  constexpr int GROUP = 8;
  const int per_group = GROUP * nbn;
  const int first_m = (logical / per_group) * GROUP;
  const int gsz = nbm - first_m < GROUP ? nbm - first_m : GROUP;
  const int in_group = logical % per_group;
  const int m0 = (first_m + in_group % gsz) * BM;
  const int n0 = (in_group / gsz) * BN;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  OperandStage<T, !A_MC> sa;
  OperandStage<T, B_KC> sb;
  const int KT = (g.K + BK - 1) / BK;

  sa.load(A, g.lda, m0, g.M, 0, g.K);
  sb.load(B, g.ldb, n0, g.N, 0, g.K);
  sa.store(lds);
  sb.store(lds + kTileBytes);
  __syncthreads();

  const int frag_row = lane & 31, frag_half = lane >> 5;
  for (int kt = 0; kt < KT; ++kt) {
    char* cur = lds + (kt & 1) * 2 * kTileBytes;
    char* nxt = lds + ((kt & 1) ^ 1) * 2 * kTileBytes;
    const bool more = kt + 1 < KT;
    if (more) {
      sa.load(A, g.lda, m0, g.M, (kt + 1) * BK, g.K);
      sb.load(B, g.ldb, n0, g.N, (kt + 1) * BK, g.K);
    }
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      uint4 af[4], bf[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        af[i] = *reinterpret_cast<const uint4*>(cur + lds_chunk_offset(wm * 128 + i * 32 + frag_row, ks * 2 + frag_half));
        bf[i] = *reinterpret_cast<const uint4*>(cur + kTileBytes +
                                                lds_chunk_offset(wn * 128 + i * 32 + frag_row, ks * 2 + frag_half));
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          // operands swapped: the accumulator holds C^T, i.e. 4 consecutive n per lane
          acc[i][j] = Mfma16<T>::run(bf[j], af[i], acc[i][j]);
    }
    if (more) {
      sa.store(nxt);
      sb.store(nxt + kTileBytes);
    }
    __syncthreads();
  }

  // ---- epilogue: lane holds, for tile (i, j) and register group rg, C[m][n .. n+3] with
  //      m = m0 + wm*128 + i*32 + lane%32, n = n0 + wn*128 + j*32 + rg*8 + (lane/32)*4 ----
  T* __restrict__ C = reinterpret_cast<T*>(g.c);
  T* __restrict__ P = reinterpret_cast<T*>(g.pre_act);
  const bool vec_ok = ((g.ldc & 3) == 0) && ((reinterpret_cast<uintptr_t>(C) & 7u) == 0) &&
                      (!P || (((g.ldp & 3) == 0) && ((reinterpret_cast<uintptr_t>(P) & 7u) == 0)));
#pragma unroll
  for (int j = 0; j < 4; ++j) {
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
      const int n = n0 + wn * 128 + j * 32 + rg * 8 + frag_half * 4;
      float bv[4] = {0.f, 0.f, 0.f, 0.f};
      if (g.bias) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < g.N) bv[e] = load_scalar_f32(g.bias, g.bias_dt, n + e);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int m = m0 + wm * 128 + i * 32 + frag_row;
        if (m >= g.M || n >= g.N) continue;
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[i][j][rg * 4 + e] + bv[e];
        const bool full = vec_ok && n + 3 < g.N;
        if (ACT != AT_ACT_NONE) {
          if (P) {
            T* pp = P + (int64_t)m * g.ldp + n;
            if (full) store_f32<T, 4>(pp, v);
            else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (n + e < g.N) pp[e] = from_f32<T>(v[e]);
            }
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = act_forward(ACT, v[e], g.param);
        }
        T* cp = C + (int64_t)m * g.ldc + n;
        if (full) store_f32<T, 4>(cp, v);
        else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < g.N) cp[e] = from_f32<T>(v[e]);
        }
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// Generic kernel: element strides for both operands, fp32 MFMA 32x32x2, 64x64x16 tiles.
// ------------------------------------------------------------------------------------------
struct SimpleArgs {
  const void* a; const void* b; void* c; void* pre_act; const void* bias;
  int M, N, K;
  int64_t sam, sak, sbk, sbn, ldc, ldp;
  int act; float param; int bias_dt;
};

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void gemm_simple_kernel(SimpleArgs g) {
  constexpr int TM = 64, TN = 64, TK = 16;
  __shared__ float sa[TK][TM + 1];
  __shared__ float sb[TK][TN + 1];
  const TI* __restrict__ A = reinterpret_cast<const TI*>(g.a);
  const TI* __restrict__ B = reinterpret_cast<const TI*>(g.b);
  const int nbn = (g.N + TN - 1) / TN;
  const int m0 = (blockIdx.x / nbn) * TM, n0 = (blockIdx.x % nbn) * TN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  f32x16 acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0.f;

  // Tile loads: pick the thread->element mapping that follows the unit stride of each operand.
  const bool a_k_fast = g.sak == 1;
  const bool b_n_fast = g.sbn == 1;
  for (int k0 = 0; k0 < g.K; k0 += TK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = threadIdx.x + i * 256;  // 1024 elements per operand tile
      int mm, kk;
      if (a_k_fast) { kk = e & 15; mm = e >> 4; } else { mm = e & 63; kk = e >> 6; }
      const int m = m0 + mm, k = k0 + kk;
      sa[kk][mm] = (m < g.M && k < g.K) ? to_f32(A[(int64_t)m * g.sam + (int64_t)k * g.sak]) : 0.f;
      int nn, kb;
      if (b_n_fast) { nn = e & 63; kb = e >> 6; } else { kb = e & 15; nn = e >> 4; }
      const int n = n0 + nn, k2 = k0 + kb;
      sb[kb][nn] = (n < g.N && k2 < g.K) ? to_f32(B[(int64_t)k2 * g.sbk + (int64_t)n * g.sbn]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < TK; ks += 2) {
      // operands swapped so that a lane ends up with 4 consecutive n of one m
      const float bval = sb[ks + (lane >> 5)][wn * 32 + (lane & 31)];
      const float aval = sa[ks + (lane >> 5)][wm * 32 + (lane & 31)];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(bval, aval, acc, 0, 0, 0);
    }
    __syncthreads();
  }

  TO* __restrict__ C = reinterpret_cast<TO*>(g.c);
  TO* __restrict__ P = reinterpret_cast<TO*>(g.pre_act);
  const int m = m0 + wm * 32 + (lane & 31);
  if (m >= g.M) return;
#pragma unroll
  for (int rg = 0; rg < 4; ++rg) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int n = n0 + wn * 32 + rg * 8 + (lane >> 5) * 4 + e;
      if (n >= g.N) continue;
      float v = acc[rg * 4 + e];
      if (g.bias) v += load_scalar_f32(g.bias, g.bias_dt, n);
      if (g.act != AT_ACT_NONE) {
        if (P) P[(int64_t)m * g.ldp + n] = from_f32<TO>(v);
        v = act_forward(g.act, v, g.param);
      }
      C[(int64_t)m * g.ldc + n] = from_f32<TO>(v);
    }
  }
}

// ------------------------------------------------------------------------------------------
// Elementwise activation backward with fused column sum (bias gradient).
//   dz = dy * act'(z);  bias partials: one fp32 row per workgroup row-slice.
// ------------------------------------------------------------------------------------------
template <typename TDY, typename TZ>
__global__ __launch_bounds__(256) void act_bwd_kernel(
    const TDY* __restrict__ dy, const TZ* __restrict__ z, TZ* __restrict__ dz, int64_t M, int N,
    int64_t dys, int64_t zs, int64_t dzs, int act, float param, int vec_ok) {
  constexpr int VEC = 8;
  const int64_t chunks_per_row = (N + VEC - 1) / VEC;
  const int64_t total = M * chunks_per_row;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int64_t r = i / chunks_per_row;
    const int c = (int)(i - r * chunks_per_row) * VEC;
    if (vec_ok) {
      float d[VEC], zz[VEC];
      load_f32<TDY, VEC>(dy + r * dys + c, d);
      load_f32<TZ, VEC>(z + r * zs + c, zz);
#pragma unroll
      for (int j = 0; j < VEC; ++j) d[j] *= act_derivative(act, zz[j], param);
      store_f32<TZ, VEC>(dz + r * dzs + c, d);
    } else {
      for (int j = 0; j < VEC && c + j < N; ++j)
        dz[r * dzs + c + j] =
            from_f32<TZ>(to_f32(dy[r * dys + c + j]) * act_derivative(act, to_f32(z[r * zs + c + j]), param));
    }
  }
}

// Column sums of a [M, N] matrix: partial[slice, n] over a slice of rows, then a fixed-order
// reduction; grid = (ceil(N / 256), slices).
template <typename T>
__global__ __launch_bounds__(256) void colsum_partial_kernel(const T* __restrict__ x, float* __restrict__ part,
                                                            int64_t M, int N, int64_t xs,
                                                            int64_t rows_per_slice) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  if (n >= N) return;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_slice;
  const int64_t r1 = r0 + rows_per_slice < M ? r0 + rows_per_slice : M;
  float s = 0.f;
  for (int64_t r = r0; r < r1; ++r) s += to_f32(x[r * xs + n]);
  part[(int64_t)blockIdx.y * N + n] = s;
}

__global__ __launch_bounds__(256) void colsum_final_kernel(const float* __restrict__ part, void* __restrict__ out,
                                                          int out_dt, int slices, int N) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  if (n >= N) return;
  float s = 0.f;
  for (int p = 0; p < slices; ++p) s += part[(int64_t)p * N + n];
  store_scalar_f32(out, out_dt, n, s);
}

template <typename F>
inline int dispatch_dtype(int dt, F&& f) {
  if (dt == AT_DTYPE_F32) return f((float*)0);
  if (dt == AT_DTYPE_F16) return f((f16_t*)0);
  if (dt == AT_DTYPE_BF16) return f((bf16_t*)0);
  return AT_ERR_DTYPE;
}

enum Layout { kFwd = 0, kDx = 1, kDw = 2 };

// C[M,N] = A(m,k) B(k,n) for the three products of the linear layer.
//   kFwd: A = [M,K] rows,  B = [K,N] rows          (X, W)
//   kDx : A = [M,K] rows,  B = [N,K] rows          (dZ, W: contraction over W's columns)
//   kDw : A = [K,M] rows,  B = [K,N] rows          (X, dZ: contraction over rows of both)
int run_gemm(Layout layout, const void* a, const void* b, void* c, void* pre_act, const void* bias, int64_t M,
             int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int64_t ldp, int act, float param,
             int in_dt, int bias_dt, int out_dt, hipStream_t stream) {
  if (!a || !b || !c) return AT_ERR_NULL;
  if (!dtype_valid(in_dt) || !dtype_valid(out_dt) || (bias && !dtype_valid(bias_dt))) return AT_ERR_DTYPE;
  if (!act_valid(act)) return AT_ERR_ACT;
  if (M < 0 || N <= 0 || K <= 0 || M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return AT_ERR_DIM;
  const int64_t a_min = layout == kDw ? M : K, b_min = layout == kDx ? K : N;
  if (lda < a_min || ldb < b_min || ldc < N || (pre_act && ldp < N)) return AT_ERR_DIM;
  if (M == 0) return AT_OK;

  const bool a_contig_k = layout != kDw, b_contig_k = layout == kDx;
  bool fast = in_dt != AT_DTYPE_F32 && out_dt == in_dt && aligned16(a) && aligned16(b) && (lda % 8) == 0 &&
              (ldb % 8) == 0 && (K % 8) == 0;
  if (!a_contig_k) fast = fast && (M % 8) == 0;
  if (!b_contig_k) fast = fast && (N % 8) == 0;
  // Small problems do not fill 256x256 tiles; the generic kernel has finer tiles.
  if (M * N < (int64_t)BM * BN / 2 || M < 64 || N < 64) fast = false;

  if (fast) {
    GemmArgs g{a, b, c, pre_act, bias, (int)M, (int)N, (int)K, lda, ldb, ldc, ldp, act, param, bias_dt};
    const unsigned grid = (unsigned)(cdiv64(M, BM) * cdiv64(N, BN));
    return dispatch_dtype(in_dt, [&](auto* tp) -> int {
      typedef std::remove_pointer_t<decltype(tp)> T;
      if constexpr (std::is_same<T, float>::value) {
        return AT_ERR_DTYPE;
      } else {
        if (layout == kDx) {
          hipLaunchKernelGGL((gemm_mfma16_kernel<T, false, true, AT_ACT_NONE>), dim3(grid), dim3(kGemmThreads), 0, stream, g);
        } else if (layout == kDw) {
          hipLaunchKernelGGL((gemm_mfma16_kernel<T, true, false, AT_ACT_NONE>), dim3(grid), dim3(kGemmThreads), 0, stream, g);
        } else {
          switch (act) {
#define AT_FWD_CASE(ID) case ID: hipLaunchKernelGGL((gemm_mfma16_kernel<T, false, false, ID>), dim3(grid), dim3(kGemmThreads), 0, stream, g); break;
            AT_FWD_CASE(AT_ACT_NONE) AT_FWD_CASE(AT_ACT_SIGMOID) AT_FWD_CASE(AT_ACT_LOGSIGMOID)
            AT_FWD_CASE(AT_ACT_TANH) AT_FWD_CASE(AT_ACT_RELU) AT_FWD_CASE(AT_ACT_GELU)
            AT_FWD_CASE(AT_ACT_GELUAPPROX) AT_FWD_CASE(AT_ACT_SILU) AT_FWD_CASE(AT_ACT_RELU6)
            AT_FWD_CASE(AT_ACT_HARDSIGMOID) AT_FWD_CASE(AT_ACT_HARDTANH) AT_FWD_CASE(AT_ACT_HARDSWISH)
            AT_FWD_CASE(AT_ACT_SELU) AT_FWD_CASE(AT_ACT_MISH) AT_FWD_CASE(AT_ACT_SOFTPLUS)
            AT_FWD_CASE(AT_ACT_SOFTSIGN) AT_FWD_CASE(AT_ACT_TANHSHRINK) AT_FWD_CASE(AT_ACT_LEAKY_RELU)
            AT_FWD_CASE(AT_ACT_ELU) AT_FWD_CASE(AT_ACT_CELU) AT_FWD_CASE(AT_ACT_HARDSHRINK)
            AT_FWD_CASE(AT_ACT_SOFTSHRINK)
#undef AT_FWD_CASE
            default: return AT_ERR_ACT;
          }
        }
        return launch_status();
      }
    });
  }

  SimpleArgs s{a, b, c, pre_act, bias, (int)M, (int)N, (int)K,
               a_contig_k ? lda : 1, a_contig_k ? 1 : lda, b_contig_k ? 1 : ldb, b_contig_k ? ldb : 1,
               ldc, ldp, act, param, bias_dt};
  const unsigned grid = (unsigned)(cdiv64(M, 64) * cdiv64(N, 64));
  return dispatch_dtype(in_dt, [&](auto* ti) -> int {
    typedef std::remove_pointer_t<decltype(ti)> TI;
    return dispatch_dtype(out_dt, [&](auto* to) -> int {
      typedef std::remove_pointer_t<decltype(to)> TO;
      hipLaunchKernelGGL((gemm_simple_kernel<TI, TO>), dim3(grid), dim3(256), 0, stream, s);
      return launch_status();
    });
  });
}

constexpr int kColsumSlices = 64;

}  // namespace
}  // namespace at_hip

using namespace at_hip;

extern "C" {

int at_linear_fwd(const void* input, const void* weight, const void* bias, void* pre_act, void* output,
                  int64_t batch, int64_t in_feat, int64_t out_feat, int64_t input_stride,
                  int64_t weight_stride, int64_t pre_act_stride, int64_t output_stride, int act, float param,
                  int in_dtype, int bias_dtype, int out_dtype, at_stream_t stream) {
  if (pre_act == output) pre_act = nullptr;  // the reference aliases them when nothing is saved
  return run_gemm(kFwd, input, weight, output, pre_act, bias, batch, out_feat, in_feat, input_stride,
                  weight_stride, output_stride, pre_act_stride, act, param, in_dtype, bias_dtype, out_dtype,
                  (hipStream_t)stream);
}

int at_linear_bwd_input(const void* pre_act_grad, const void* weight, void* input_grad, int64_t batch,
                        int64_t in_feat, int64_t out_feat, int64_t grad_stride, int64_t weight_stride,
                        int64_t input_grad_stride, int in_dtype, int out_dtype, at_stream_t stream) {
  return run_gemm(kDx, pre_act_grad, weight, input_grad, nullptr, nullptr, batch, in_feat, out_feat,
                  grad_stride, weight_stride, input_grad_stride, 0, AT_ACT_NONE, 0.f, in_dtype, 0, out_dtype,
                  (hipStream_t)stream);
}

int at_linear_bwd_weight(const void* input, const void* pre_act_grad, void* weight_grad, int64_t batch,
                         int64_t in_feat, int64_t out_feat, int64_t input_stride, int64_t grad_stride,
                         int64_t weight_grad_stride, int in_dtype, int out_dtype, at_stream_t stream) {
  if (batch <= 0) return AT_ERR_DIM;
  return run_gemm(kDw, input, pre_act_grad, weight_grad, nullptr, nullptr, in_feat, out_feat, batch,
                  input_stride, grad_stride, weight_grad_stride, 0, AT_ACT_NONE, 0.f, in_dtype, 0, out_dtype,
                  (hipStream_t)stream);
}

int at_act_bwd(const void* output_grad, const void* input, void* input_grad, int64_t rows, int64_t cols,
               int64_t output_grad_stride, int64_t input_stride, int64_t input_grad_stride, int act,
               float param, int grad_dtype, int input_dtype, at_stream_t stream) {
  if (!output_grad || !input || !input_grad) return AT_ERR_NULL;
  if (!dtype_valid(grad_dtype) || !dtype_valid(input_dtype)) return AT_ERR_DTYPE;
  if (!act_valid(act) || act == AT_ACT_NONE) return AT_ERR_ACT;
  if (rows < 0 || cols <= 0 || cols > INT32_MAX) return AT_ERR_DIM;
  if (output_grad_stride < cols || input_stride < cols || input_grad_stride < cols) return AT_ERR_DIM;
  if (rows == 0) return AT_OK;
  const int gs = dtype_size(grad_dtype), is = dtype_size(input_dtype);
  const int vec_ok = cols % 8 == 0 && aligned16(output_grad) && aligned16(input) && aligned16(input_grad) &&
                     (output_grad_stride * gs) % 16 == 0 && (input_stride * is) % 16 == 0 &&
                     (input_grad_stride * is) % 16 == 0;
  const int64_t chunks = rows * cdiv64(cols, 8);
  int64_t blocks = cdiv64(chunks, 256);
  const int64_t cap = (int64_t)device_cu_count() * 16;
  if (blocks > cap) blocks = cap;
  return dispatch_dtype(grad_dtype, [&](auto* tg) -> int {
    typedef std::remove_pointer_t<decltype(tg)> TG;
    return dispatch_dtype(input_dtype, [&](auto* tz) -> int {
      typedef std::remove_pointer_t<decltype(tz)> TZ;
      hipLaunchKernelGGL((act_bwd_kernel<TG, TZ>), dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                         (const TG*)output_grad, (const TZ*)input, (TZ*)input_grad, rows, (int)cols,
                         output_grad_stride, input_stride, input_grad_stride, act, param, vec_ok);
      return launch_status();
    });
  });
}

int64_t at_colsum_workspace_bytes(int64_t rows, int64_t cols) {
  if (rows <= 0 || cols <= 0) return 0;
  return (int64_t)kColsumSlices * cols * (int64_t)sizeof(float);
}

int at_colsum(const void* x, void* out, void* workspace, int64_t workspace_bytes, int64_t rows, int64_t cols,
              int64_t x_stride, int x_dtype, int out_dtype, at_stream_t stream) {
  if (!x || !out) return AT_ERR_NULL;
  if (!dtype_valid(x_dtype) || !dtype_valid(out_dtype)) return AT_ERR_DTYPE;
  if (rows <= 0 || cols <= 0 || cols > INT32_MAX || x_stride < cols) return AT_ERR_DIM;
  if (!workspace || workspace_bytes < at_colsum_workspace_bytes(rows, cols)) return AT_ERR_WORKSPACE;
  int slices = (int)(rows < kColsumSlices ? rows : kColsumSlices);
  const int64_t rows_per_slice = cdiv64(rows, slices);
  slices = (int)cdiv64(rows, rows_per_slice);
  const unsigned gx = (unsigned)cdiv64(cols, 256);
  int rc = dispatch_dtype(x_dtype, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    hipLaunchKernelGGL((colsum_partial_kernel<T>), dim3(gx, slices), dim3(256), 0, (hipStream_t)stream,
                       (const T*)x, (float*)workspace, rows, (int)cols, x_stride, rows_per_slice);
    return launch_status();
  });
  if (rc) return rc;
  hipLaunchKernelGGL(colsum_final_kernel, dim3(gx), dim3(256), 0, (hipStream_t)stream,
                     (const float*)workspace, out, out_dtype, slices, (int)cols);
  return launch_status();
}

}  // extern "C"
