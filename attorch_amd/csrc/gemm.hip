// Linear layer GEMMs: Y = act(X W + b) and the two backward products, fp32 accumulate.
//
// Two kernels:
//  * gemm_mfma16_kernel — bf16/fp16 operands on v_mfma_f32_32x32x16 (MFMA-bound).  256x256x64
//    macro-tile per 256-lane workgroup (4 waves, 128x128 each, 256 accumulator registers per
//    lane), LDS double-buffered, one barrier per k-tile.  Tiles go from global memory straight
//    into LDS (buffer_load ... lds), the loads of tile k+1 in flight while tile k is
//    multiplied.  An operand whose contraction index is contiguous in memory is kept as
//    [row][k] with the 16-byte chunk index XOR-swizzled by the row (bank-conflict-free 128-bit
//    fragment reads); an operand stored the other way round (W in the forward product, X and
//    dZ in the weight gradient) is kept as loaded and transposed by the fragment reads
//    themselves (ds_read_b64_tr_b16).  Fragments are double-buffered in registers, and the
//    finished tile leaves through LDS as whole 512-byte row segments.  Workgroup ids are
//    remapped so that each XCD (own L2) works on a compact block of output tiles.
//  * gemm_simple_kernel — any dtype, any strides, fp32 MFMA (32x32x2), 64x64x64 tile, next k-tile
//    prefetched into registers; used for fp32 tensors and for 16-bit shapes the fast kernel cannot
//    address with 128-bit accesses.
// Both fuse bias, the optional pre-activation store and the activation into the epilogue.
#include <type_traits>

#include "at_act.h"
#include "at_mfma.h"

namespace at_hip {
namespace {

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

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kGemmThreads = 256;
constexpr int kTileBytes = BM * BK * 2;  // one operand tile, 32 KiB
constexpr int kEpiPitch = BN * 2 + 16;   // bytes per row of the epilogue tile in LDS (padded against bank conflicts)
constexpr int kEpiBytes = BM * kEpiPitch;

typedef __attribute__((address_space(3))) void lds_void_t;

// LDS image of one operand tile of a k-tile.
//  * CONTRACT_CONTIG (memory [outer][k]): 256 rows x 128 bytes, 16-byte chunks XOR-swizzled by
//    the row (lds_chunk_offset); fragments are plain 128-bit reads.
//  * otherwise (memory [k][outer]): 64 k-rows x 512 bytes kept as loaded; every pair of rows
//    is one contiguous KiB (one wave-wide load) followed by 64 bytes of padding, which
//    spreads the 8 rows a transposing fragment read touches evenly over the banks.
constexpr int kPairPitch = 1024 + 64;
template <bool CONTRACT_CONTIG> constexpr int operand_tile_bytes() { return CONTRACT_CONTIG ? kTileBytes : 32 * kPairPitch; }

template <typename T, bool CONTRACT_CONTIG>
struct OperandLoader {
  i32x4 rsrc;
  int lane_off;   // byte offset of this lane's first load at k-tile 0
  int blk_step;   // bytes between the 8 loads of a lane
  int k_step;     // bytes per k-tile
  int k_lane;     // k of this lane inside a k-tile (contract-contiguous layout only)
  int K;

  __device__ __forceinline__ void init(const T* base, int64_t ld, int outer0, int outer_total, int K_) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    K = K_;
    if (CONTRACT_CONTIG) {
      rsrc = make_buffer_rsrc(base, outer_total * ld * 2);
      // load i of wave w fills rows 8q .. 8q+7 (q = 8w + i); lane -> (row, position), and the
      // position holds chunk (position ^ swizzle(row)) so that the reads find chunk c at c ^ swizzle
      const int row = wave * 64 + (lane >> 3);            // + 8 i
      k_lane = 0;
      lane_off = (int)(((int64_t)(outer0 + row) * ld) * 2);
      blk_step = (int)(8 * ld * 2);
      k_step = BK * 2;
    } else {
      rsrc = make_buffer_rsrc(base, K_ * ld * 2);
      // load i of wave w fills k-rows 2q, 2q+1 (q = 8w + i); lane -> k-row 2q + lane/32, 8 columns at (lane%32)*8
      const int krow = wave * 16 + (lane >> 5);            // + 2 i
      k_lane = 0;
      lane_off = (int)(((int64_t)krow * ld + outer0 + (lane & 31) * 8) * 2);
      blk_step = (int)(2 * ld * 2);
      k_step = (int)(BK * ld * 2);
    }
  }

  // Issues the 8 loads of this lane for k-tile `kt` into `tile` (LDS).
  __device__ __forceinline__ void issue(int kt, char* tile) const {
#pragma unroll
    for (int i = 0; i < 8; ++i) issue_one(kt, tile, i);
  }

  // Load i (0..7) of this lane for k-tile `kt`.
  __device__ __forceinline__ void issue_one(int kt, char* tile, int i) const {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    {
      const int q = wave * 8 + i;
      int off;
      char* dst;
      if (CONTRACT_CONTIG) {
        const int row = q * 8 + (lane >> 3);
        const int chunk = (lane & 7) ^ ((row ^ (row >> 3)) & 7);
        const int k = kt * BK + chunk * 8;
        off = k < K ? lane_off + i * blk_step + k * 2 : kOobOffset;   // K tail reads as zeros
        dst = tile + q * 1024;
      } else {
        off = lane_off + i * blk_step + kt * k_step;                  // k-rows past K fall out of range
        dst = tile + q * kPairPitch;
      }
      lds_dma_16(rsrc, off, dst);
    }
  }
};

// Fragment of 32 rows (outer index) x 16 k for one MFMA operand: 8 consecutive k per lane.
template <bool CONTRACT_CONTIG>
__device__ __forceinline__ uint4 read_frag(const char* tile, int outer_base, int ks) {
  const int lane = threadIdx.x & 63;
  if (CONTRACT_CONTIG) {
    return read_frag_kc(tile, outer_base, ks);
  } else {
    // ds_read_b64_tr_b16: within 16 lanes, result[l][e] = source[4e + l/4][l%4]; the source lane
    // 4e + q therefore points at k-row (k0 + e), columns 4q .. 4q+3, and lane l receives
    // k0 .. k0+3 of column l.  Two reads give the 8 k of this lane's half.
    const int i = lane & 15, g = lane >> 4;
    const int col = outer_base + (g & 1) * 16 + (i & 3) * 4;
    const int krow = ks * 16 + (g >> 1) * 8 + (i >> 2);
    const char* p0 = tile + (krow >> 1) * kPairPitch + (krow & 1) * 512 + col * 2;
    const int krow1 = krow + 4;
    const char* p1 = tile + (krow1 >> 1) * kPairPitch + (krow1 & 1) * 512 + col * 2;
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p0);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p1);
    const uint2 a = __builtin_bit_cast(uint2, lo), b = __builtin_bit_cast(uint2, hi);
    return make_uint4(a.x, a.y, b.x, b.y);
  }
}

// ACT is the compile-time activation id of the epilogue (the act switch must fold away: the
// epilogue is fully unrolled over 256 accumulator registers).
template <typename T, bool A_MC, bool B_KC, int ACT>
__global__ __launch_bounds__(kGemmThreads) void gemm_mfma16_kernel(GemmArgs g) {
  constexpr bool A_KC = !A_MC;
  constexpr int kATile = operand_tile_bytes<A_KC>(), kBTile = operand_tile_bytes<B_KC>();
  constexpr int kStage = kATile + kBTile;
  constexpr int kLds = 2 * kStage > kEpiBytes ? 2 * kStage : kEpiBytes;
  __shared__ __attribute__((aligned(1024))) char lds[kLds];  // main loop: [stage][A|B]; epilogue: output tile
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
  const int frag_row = lane & 31, frag_half = lane >> 5;

  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  OperandLoader<T, A_KC> la;
  OperandLoader<T, B_KC> lb;
  la.init(A, g.lda, m0, g.M, g.K);
  lb.init(B, g.ldb, n0, g.N, g.K);
  const int KT = (g.K + BK - 1) / BK;

  la.issue(0, lds);
  lb.issue(0, lds + kATile);
  lds_dma_wait_all();
  __syncthreads();

  auto load_frags = [&](const char* stage, int ks, uint4 (&af)[4], uint4 (&bf)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      af[i] = read_frag<A_KC>(stage, wm * 128 + i * 32, ks);
      bf[i] = read_frag<B_KC>(stage + kATile, wn * 128 + i * 32, ks);
    }
  };

  // One k-tile = four k-steps of 16 MFMAs (512 matrix-pipe cycles each).  With a single wave
  // per SIMD nothing else hides latency, so the other instructions of the iteration are
  // slotted between MFMAs: the 16 global->LDS loads of the next tile during k-step 0, the
  // fragment reads of k-step s+1 during k-step s.  The loads of tile kt+1 stay in flight for
  // the whole iteration and are only waited for at the barrier that ends it.
  // (sched_group_barrier masks: 0x8 MFMA, 0x2 VALU, 0x20 VMEM read, 0x100 LDS read.)
  for (int kt = 0; kt < KT; ++kt) {
    char* cur = lds + (kt & 1) * kStage;
    char* nxt = lds + ((kt & 1) ^ 1) * kStage;
    uint4 af[2][4], bf[2][4];
    load_frags(cur, 0, af[0], bf[0]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      if (ks + 1 < BK / 16) load_frags(cur, ks + 1, af[(ks + 1) & 1], bf[(ks + 1) & 1]);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          // One global->LDS load of the next tile behind each MFMA of k-step 0.  Unconditional:
          // past the last k-tile every offset is out of range and the loads write zeros into
          // a stage nobody reads, so the loop body has no branches.
          if (ks == 0) {
            if (i < 2) la.issue_one(kt + 1, nxt, i * 4 + j);
            else lb.issue_one(kt + 1, nxt + kATile, (i - 2) * 4 + j);
          }
          // operands swapped: the accumulator holds C^T, i.e. 4 consecutive n per lane
          acc[i][j] = Mfma16<T>::run(bf[ks & 1][j], af[ks & 1][i], acc[i][j]);
        }
      if (ks < BK / 16 - 1) {
#pragma unroll
        for (int q = 0; q < 16; ++q) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    lds_dma_wait_all();   // this wave's part of the next stage has landed
    __syncthreads();      // ... and so has everybody else's; the current stage may be overwritten
  }

  // ---- epilogue ----
  // A lane holds, for tile (i, j) and register group rg, C[m][n .. n+3] with
  //   m = wm*128 + i*32 + lane%32,  n = wn*128 + j*32 + rg*8 + (lane/32)*4   (tile-local).
  // Storing that straight to memory touches 32 rows per instruction with 16 bytes each; instead
  // the finished tile goes through LDS (free after the main loop) and leaves as whole rows:
  // 32 lanes x 16 bytes = one 512-byte row segment per half-wave.
  T* __restrict__ C = reinterpret_cast<T*>(g.c);
  T* __restrict__ P = reinterpret_cast<T*>(g.pre_act);
  const bool rows16 = ((g.ldc & 7) == 0) && aligned16_dev(C) && (n0 + BN <= g.N) &&
                      (!P || (((g.ldp & 7) == 0) && aligned16_dev(P)));
  constexpr int n_out = ACT != AT_ACT_NONE ? 2 : 1;
#pragma unroll
  for (int pass = 0; pass < n_out; ++pass) {
    const bool is_pre = (n_out == 2 && pass == 0);
    T* __restrict__ dst = is_pre ? P : C;
    const int64_t ldd = is_pre ? g.ldp : g.ldc;
    if (is_pre && !P) continue;   // uniform
    __syncthreads();              // previous readers of LDS (main loop or previous pass) are done
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        const int nl = wn * 128 + j * 32 + rg * 8 + frag_half * 4;
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (g.bias) {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n0 + nl + e < g.N) bv[e] = load_scalar_f32(g.bias, g.bias_dt, n0 + nl + e);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v[e] = acc[i][j][rg * 4 + e] + bv[e];
            if (ACT != AT_ACT_NONE && !is_pre) v[e] = act_forward(ACT, v[e], g.param);
          }
          const int ml = wm * 128 + i * 32 + frag_row;
          store_f32<T, 4>(reinterpret_cast<T*>(lds + ml * kEpiPitch) + nl, v);
        }
      }
    __syncthreads();
    // 256 lanes: 8 rows per sweep, 32 lanes x 16 bytes per row
    const int rsub = threadIdx.x >> 5, cseg = (threadIdx.x & 31) * 8;
#pragma unroll 4
    for (int r0 = 0; r0 < BM; r0 += 8) {
      const int ml = r0 + rsub;
      const int m = m0 + ml;
      if (m >= g.M) continue;
      const uint4 v = *reinterpret_cast<const uint4*>(lds + ml * kEpiPitch + cseg * 2);
      T* out = dst + (int64_t)m * ldd + n0 + cseg;
      if (rows16) {
        *reinterpret_cast<uint4*>(out) = v;
      } else {
        union { uint4 raw; T e[8]; } u;
        u.raw = v;
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (n0 + cseg + e < g.N) out[e] = u.e[e];
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
  constexpr int TM = 64, TN = 64, TK = 64;
  constexpr int PER = TM * TK / 256;   // elements of each operand tile per lane
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

  // Tile loads: the thread->element mapping follows the unit stride of each operand.  The next
  // k-tile is fetched into registers while the current one is multiplied (small problems are
  // bound by the latency of these loads, not by their volume).
  const bool a_k_fast = g.sak == 1;
  const bool b_n_fast = g.sbn == 1;
  float ra[PER], rb[PER];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = threadIdx.x + i * 256;
      int mm, kk;
      if (a_k_fast) { kk = e & (TK - 1); mm = e / TK; } else { mm = e & (TM - 1); kk = e / TM; }
      const int m = m0 + mm, k = k0 + kk;
      ra[i] = (m < g.M && k < g.K) ? to_f32(A[(int64_t)m * g.sam + (int64_t)k * g.sak]) : 0.f;
      int nn, kb;
      if (b_n_fast) { nn = e & (TN - 1); kb = e / TN; } else { kb = e & (TK - 1); nn = e / TK; }
      const int n = n0 + nn, k2 = k0 + kb;
      rb[i] = (n < g.N && k2 < g.K) ? to_f32(B[(int64_t)k2 * g.sbk + (int64_t)n * g.sbn]) : 0.f;
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = threadIdx.x + i * 256;
      int mm, kk;
      if (a_k_fast) { kk = e & (TK - 1); mm = e / TK; } else { mm = e & (TM - 1); kk = e / TM; }
      sa[kk][mm] = ra[i];
      int nn, kb;
      if (b_n_fast) { nn = e & (TN - 1); kb = e / TN; } else { kb = e & (TK - 1); nn = e / TK; }
      sb[kb][nn] = rb[i];
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < g.K; k0 += TK) {
    stage();
    __syncthreads();
    if (k0 + TK < g.K) fetch(k0 + TK);
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
// Elementwise activation backward, optionally with the bias gradient fused in:
//   dz = dy * act'(z);  part[slice, n] = sum over the rows of the slice of dz (rounded as stored).
// grid = (column groups of 256 * 8, row slices); each lane owns 8 consecutive columns and walks
// the rows of its slice, so the column sums need no cross-lane traffic.
// ------------------------------------------------------------------------------------------
template <typename TDY, typename TZ, bool VEC_OK>
__global__ __launch_bounds__(256) void act_bwd_kernel(
    const TDY* __restrict__ dy, const TZ* __restrict__ z, TZ* __restrict__ dz, float* __restrict__ part,
    int64_t M, int N, int64_t dys, int64_t zs, int64_t dzs, int act, float param, int64_t rows_per_slice) {
  constexpr int VEC = 8;
  const int c = (blockIdx.x * 256 + threadIdx.x) * VEC;
  if (c >= N) return;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_slice;
  const int64_t r1 = r0 + rows_per_slice < M ? r0 + rows_per_slice : M;
  float sum[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) sum[j] = 0.f;
  constexpr int ROWS = 4;  // rows in flight per lane
  for (int64_t rb = r0; rb < r1; rb += ROWS) {
    float d[ROWS][VEC], zz[ROWS][VEC];
#pragma unroll
    for (int u = 0; u < ROWS; ++u) {
      const int64_t r = rb + u;
      if (r < r1) {
        if (VEC_OK) {
          load_f32<TDY, VEC>(dy + r * dys + c, d[u]);
          load_f32<TZ, VEC>(z + r * zs + c, zz[u]);
        } else {
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            const bool ok = c + j < N;
            d[u][j] = ok ? to_f32(dy[r * dys + c + j]) : 0.f;
            zz[u][j] = ok ? to_f32(z[r * zs + c + j]) : 0.f;
          }
        }
      }
    }
#pragma unroll
    for (int u = 0; u < ROWS; ++u) {
      const int64_t r = rb + u;
      if (r < r1) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          d[u][j] = to_f32(from_f32<TZ>(d[u][j] * act_derivative(act, zz[u][j], param)));  // summed as stored
          sum[j] += d[u][j];
        }
        if (VEC_OK) store_f32<TZ, VEC>(dz + r * dzs + c, d[u]);
        else {
#pragma unroll
          for (int j = 0; j < VEC; ++j)
            if (c + j < N) dz[r * dzs + c + j] = from_f32<TZ>(d[u][j]);
        }
      }
    }
  }
  if (part) {
#pragma unroll
    for (int j = 0; j < VEC; ++j)
      if (c + j < N) part[(int64_t)blockIdx.y * N + c + j] = sum[j];
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

// out[n] = sum over slices of part[slice][n], fixed order.  A workgroup owns 16 columns: 4 column
// quads x 64 slice lanes, folded through LDS.
constexpr int kColsumFinalCols = 16;
__global__ __launch_bounds__(256) void colsum_final_kernel(const float* __restrict__ part, void* __restrict__ out,
                                                          int out_dt, int slices, int N) {
  __shared__ float sm[64][kColsumFinalCols + 1];
  const int cq = threadIdx.x & 3, lane_slice = threadIdx.x >> 2;
  const int col = blockIdx.x * kColsumFinalCols + cq * 4;
  float a[4] = {0.f, 0.f, 0.f, 0.f};
  if (col + 3 < N && (N & 3) == 0 && aligned16_dev(part)) {
#pragma unroll 4
    for (int p = lane_slice; p < slices; p += 64) {
      const float4 v = *reinterpret_cast<const float4*>(part + (int64_t)p * N + col);
      a[0] += v.x; a[1] += v.y; a[2] += v.z; a[3] += v.w;
    }
  } else {
    for (int p = lane_slice; p < slices; p += 64)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (col + j < N) a[j] += part[(int64_t)p * N + col + j];
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) sm[lane_slice][cq * 4 + j] = a[j];
  __syncthreads();
  if (threadIdx.x < kColsumFinalCols) {
    float s = 0.f;
#pragma unroll
    for (int r = 0; r < 64; ++r) s += sm[r][threadIdx.x];
    const int n = blockIdx.x * kColsumFinalCols + threadIdx.x;
    if (n < N) store_scalar_f32(out, out_dt, n, s);
  }
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
  // buffer descriptors address each operand with 32-bit byte offsets below 2 GiB
  const int64_t a_bytes = (a_contig_k ? M : K) * lda * 2, b_bytes = (b_contig_k ? N : K) * ldb * 2;
  if (a_bytes >= ((int64_t)1 << 31) || b_bytes >= ((int64_t)1 << 31)) fast = false;
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
            AT_FWD_CASE(AT_ACT_NONE) AT_FWD_CASE(AT_ACT_RELU) AT_FWD_CASE(AT_ACT_GELUAPPROX)
#ifndef AT_QUICK_BUILD  // development builds instantiate three epilogues only
            AT_FWD_CASE(AT_ACT_SIGMOID) AT_FWD_CASE(AT_ACT_LOGSIGMOID)
            AT_FWD_CASE(AT_ACT_TANH) AT_FWD_CASE(AT_ACT_GELU)
            AT_FWD_CASE(AT_ACT_SILU) AT_FWD_CASE(AT_ACT_RELU6)
            AT_FWD_CASE(AT_ACT_HARDSIGMOID) AT_FWD_CASE(AT_ACT_HARDTANH) AT_FWD_CASE(AT_ACT_HARDSWISH)
            AT_FWD_CASE(AT_ACT_SELU) AT_FWD_CASE(AT_ACT_MISH) AT_FWD_CASE(AT_ACT_SOFTPLUS)
            AT_FWD_CASE(AT_ACT_SOFTSIGN) AT_FWD_CASE(AT_ACT_TANHSHRINK) AT_FWD_CASE(AT_ACT_LEAKY_RELU)
            AT_FWD_CASE(AT_ACT_ELU) AT_FWD_CASE(AT_ACT_CELU) AT_FWD_CASE(AT_ACT_HARDSHRINK)
            AT_FWD_CASE(AT_ACT_SOFTSHRINK)
#endif
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
constexpr int kActBwdMaxSlices = 512;

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

int64_t at_act_bwd_workspace_bytes(int64_t rows, int64_t cols) {
  if (rows <= 0 || cols <= 0) return 0;
  return (int64_t)kActBwdMaxSlices * cols * (int64_t)sizeof(float);
}

int at_act_bwd(const void* output_grad, const void* input, void* input_grad, void* bias_grad, void* workspace,
               int64_t workspace_bytes, int64_t rows, int64_t cols, int64_t output_grad_stride,
               int64_t input_stride, int64_t input_grad_stride, int act, float param, int grad_dtype,
               int input_dtype, int bias_grad_dtype, at_stream_t stream) {
  if (!output_grad || !input || !input_grad) return AT_ERR_NULL;
  if (!dtype_valid(grad_dtype) || !dtype_valid(input_dtype) || (bias_grad && !dtype_valid(bias_grad_dtype)))
    return AT_ERR_DTYPE;
  if (!act_valid(act) || act == AT_ACT_NONE) return AT_ERR_ACT;
  if (rows < 0 || cols <= 0 || cols > INT32_MAX) return AT_ERR_DIM;
  if (output_grad_stride < cols || input_stride < cols || input_grad_stride < cols) return AT_ERR_DIM;
  if (bias_grad && (!workspace || workspace_bytes < at_act_bwd_workspace_bytes(rows, cols))) return AT_ERR_WORKSPACE;
  if (rows == 0) return bias_grad ? AT_ERR_DIM : AT_OK;
  const int gs = dtype_size(grad_dtype), is = dtype_size(input_dtype);
  const bool vec_ok = cols % 8 == 0 && aligned16(output_grad) && aligned16(input) && aligned16(input_grad) &&
                      (output_grad_stride * gs) % 16 == 0 && (input_stride * is) % 16 == 0 &&
                      (input_grad_stride * is) % 16 == 0;
  // enough workgroups to fill the chip, few enough row slices to keep the partial buffer small
  const unsigned gx = (unsigned)cdiv64(cols, 256 * 8);
  int64_t slices = cdiv64((int64_t)device_cu_count() * 16, gx);
  if (slices > kActBwdMaxSlices) slices = kActBwdMaxSlices;
  if (slices > rows) slices = rows;
  const int64_t rows_per_slice = cdiv64(rows, slices);
  slices = cdiv64(rows, rows_per_slice);
  float* part = bias_grad ? (float*)workspace : nullptr;
  int rc = dispatch_dtype(grad_dtype, [&](auto* tg) -> int {
    typedef std::remove_pointer_t<decltype(tg)> TG;
    return dispatch_dtype(input_dtype, [&](auto* tz) -> int {
      typedef std::remove_pointer_t<decltype(tz)> TZ;
      if (vec_ok)
        hipLaunchKernelGGL((act_bwd_kernel<TG, TZ, true>), dim3(gx, (unsigned)slices), dim3(256), 0,
                           (hipStream_t)stream, (const TG*)output_grad, (const TZ*)input, (TZ*)input_grad, part, rows,
                           (int)cols, output_grad_stride, input_stride, input_grad_stride, act, param, rows_per_slice);
      else
        hipLaunchKernelGGL((act_bwd_kernel<TG, TZ, false>), dim3(gx, (unsigned)slices), dim3(256), 0,
                           (hipStream_t)stream, (const TG*)output_grad, (const TZ*)input, (TZ*)input_grad, part, rows,
                           (int)cols, output_grad_stride, input_stride, input_grad_stride, act, param, rows_per_slice);
      return launch_status();
    });
  });
  if (rc || !bias_grad) return rc;
  hipLaunchKernelGGL(colsum_final_kernel, dim3((unsigned)cdiv64(cols, kColsumFinalCols)), dim3(256), 0, (hipStream_t)stream,
                     (const float*)workspace, bias_grad, bias_grad_dtype, (int)slices, (int)cols);
  return launch_status();
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
  hipLaunchKernelGGL(colsum_final_kernel, dim3((unsigned)cdiv64(cols, kColsumFinalCols)), dim3(256), 0,
                     (hipStream_t)stream, (const float*)workspace, out, out_dtype, slices, (int)cols);
  return launch_status();
}

}  // extern "C"
