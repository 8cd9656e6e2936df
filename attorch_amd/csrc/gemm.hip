// Linear layer GEMMs: Y = act(X W + b) and the two backward products, fp32 accumulate.
//
// Five kernels:
//  * gemm_mfma16_kernel — bf16/fp16 operands on v_mfma_f32_32x32x16 (MFMA-bound).  256x256x64
//    macro-tile per 512-lane workgroup (8 waves, 128x64 each, 128 accumulator registers per
//    lane, two waves per SIMD), LDS double-buffered, one barrier per k-tile.  Tiles go from global memory straight
//    into LDS (buffer_load ... lds), the loads of tile k+1 in flight while tile k is
//    multiplied.  An operand whose contraction index is contiguous in memory is kept as
//    [row][k] with the 16-byte chunk index XOR-swizzled by the row (bank-conflict-free 128-bit
//    fragment reads); an operand stored the other way round (W in the forward product, X and
//    dZ in the weight gradient) is kept as loaded and transposed by the fragment reads
//    themselves (ds_read_b64_tr_b16).  Fragments are double-buffered in registers, and the
//    finished tile leaves through LDS as whole 512-byte row segments.  Workgroup ids are
//    remapped so that each XCD (own L2) works on a compact block of output tiles.
//  * gemm_mid16_kernel — the same operands in 128x128x64 tiles, two workgroups per CU, for
//    problems with too few 256x256 tiles to fill the chip; for the weight gradient it can also
//    split the contraction (the batch) over blockIdx.y into fp32 partial tiles that
//    gemm_split_finish_kernel adds up in a fixed order.
//  * gemm_small16_kernel — bf16/fp16 operands with any strides and extents (16-byte loads where
//    an operand allows them, element loads otherwise), 64x64 or 128x32 tiles: skinny outputs,
//    small problems, rows that are not 16-byte aligned; 32x32 tiles with the contraction split
//    over the four waves when the larger tiles would leave most CUs idle.
//  * gemm_skinny.h — at most 16 output features (classifier heads): vector-ALU kernels bound by
//    one pass over the wide operand.
//  * gemm_f32_kernel — fp32 operands with 16-byte aligned rows on v_mfma_f32_32x32x2f32: 128x128x16
//    (or 64x64x16) tiles straight from global memory into LDS, two stages.
//  * gemm_simple_kernel — fp32 operands, any strides, fp32 MFMA (32x32x2), 64x64x64 tile, next
//    k-tile prefetched into registers.
// All fuse bias, the optional pre-activation store and the activation into the epilogue.
#include <type_traits>

#include "at_act.h"
#include "at_mfma.h"
#include "gemm_skinny.h"

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
  // split of the contraction (128x128 kernel only): blockIdx.y takes k-tiles
  // [y * kt_per_split, (y + 1) * kt_per_split) and stores its fp32 partial tile to
  // partial[y][m][n] (row pitch ldw) instead of C
  float* partial;
  int kt_per_split;
  int ldw;
  int round_dt;       // generic kernels: results are rounded to this dtype before they are stored (fp32: as they are)
};

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kGemmThreads = 256;
// Waves of the 256x256 kernel: 2 along m (128 rows each) x 4 along n (64 columns each), two per
// SIMD.  (Four waves of 128x128 read less from LDS per MFMA but leave each SIMD with a single
// wave and nothing to cover its stalls: measured 10 % slower.)
constexpr int kBigWaves = 8;
constexpr int kBigThreads = kBigWaves * 64;
constexpr int kBigLoads = 32 / kBigWaves;          // wave-wide loads per operand tile and wave
constexpr int kBigWaveN = BN / (kBigWaves / 2);    // columns per wave
constexpr int kBigNJ = kBigWaveN / 32;             // 32-column MFMA tiles per wave
constexpr int kTileBytes = BM * BK * 2;  // one operand tile, 32 KiB
constexpr int kEpiPitch = BN * 2 + 16;   // bytes per row of the epilogue tile in LDS (padded against bank conflicts)

typedef __attribute__((address_space(3))) void lds_void_t;

// LDS image of one operand tile of a k-tile.
//  * CONTRACT_CONTIG (memory [outer][k]): 256 rows x 128 bytes, 16-byte chunks XOR-swizzled by
//    the row (lds_chunk_offset); fragments are plain 128-bit reads.
//  * otherwise (memory [k][outer]): 64 k-rows x 512 bytes; every pair of rows is one KiB (one
//    wave-wide load) followed by 128 bytes of padding, and inside the KiB the two rows alternate in
//    pieces of 64 bytes (piece 2 c + r holds columns 32 c .. 32 c + 31 of row r of the pair).  A
//    transposing fragment read takes 64 bytes from each of four consecutive k-rows per half-wave:
//    the two rows of a pair then sit 64 bytes apart and consecutive pairs 128 bytes further, so
//    the four pieces cover all 64 banks once.  (With the rows of a pair kept whole, 512 bytes
//    apart, they share their banks: the counters showed every second LDS cycle of such reads as a
//    bank conflict.)
constexpr int kPairPitch = 1024 + 128;
template <bool CONTRACT_CONTIG> constexpr int operand_tile_bytes() { return CONTRACT_CONTIG ? kTileBytes : 32 * kPairPitch; }

template <typename T, bool CONTRACT_CONTIG>
struct OperandLoader {
  i32x4 rsrc;
  int lane_off;   // byte offset of this lane's first load at k-tile 0
  int blk_step;   // bytes between the 8 loads of a lane
  int k_step;     // bytes per k-tile
  int k_lane;     // k of this lane inside a k-tile (contract-contiguous layout only)
  int K;
  int tid;        // threadIdx.x, or a copy of it that the compiler cannot see through (see the caller)

  __device__ __forceinline__ void init(const T* base, int64_t ld, int outer0, int outer_total, int K_, int tid_) {
    tid = tid_;
    const int lane = tid & 63, wave = tid >> 6;
    K = K_;
    if (CONTRACT_CONTIG) {
      rsrc = make_buffer_rsrc(base, ((int64_t)(outer_total - 1) * ld + K_) * 2);   // the last row ends at its last element
      // load i of wave w fills rows 8q .. 8q+7 (q = kBigLoads w + i); lane -> (row, position), and the
      // position holds chunk (position ^ swizzle(row)) so that the reads find chunk c at c ^ swizzle
      const int row = wave * (kBigLoads * 8) + (lane >> 3);   // + 8 i
      k_lane = 0;
      lane_off = (int)(((int64_t)(outer0 + row) * ld) * 2);
      blk_step = (int)(8 * ld * 2);
      k_step = BK * 2;
    } else {
      // up to the end of the 16-byte unit that holds the last element (rows start on such units,
      // and the range check drops a dword that is only partly inside)
      rsrc = make_buffer_rsrc(base, ((int64_t)(K_ - 1) * ld + ((outer_total + 7) & ~7)) * 2);
      // load i of wave w fills k-rows 2q, 2q+1 (q = kBigLoads w + i); the lane's 16 bytes land at
      // 16 * lane of the KiB, i.e. in piece lane / 4: row (lane / 4) % 2 of the pair, columns
      // 32 * (lane / 8) + 8 * (lane % 4) ...
      const int krow = wave * (kBigLoads * 2) + ((lane >> 2) & 1);  // + 2 i
      k_lane = 0;
      lane_off = (int)(((int64_t)krow * ld + outer0 + (lane >> 3) * 32 + (lane & 3) * 8) * 2);
      blk_step = (int)(2 * ld * 2);
      k_step = (int)(BK * ld * 2);
    }
  }

  // Issues the loads of this lane for k-tile `kt` into `tile` (LDS).
  __device__ __forceinline__ void issue(int kt, char* tile) const {
#pragma unroll
    for (int i = 0; i < kBigLoads; ++i) issue_one(kt, tile, i);
  }

  // Load i (0 .. kBigLoads-1) of this lane for k-tile `kt`; kt < 0 gives an offset that is out of
  // range (the load writes zeros).
  __device__ __forceinline__ void issue_one(int kt, char* tile, int i) const {
    const int lane = tid & 63, wave = tid >> 6;
    {
      const int q = wave * kBigLoads + i;
      int off;
      char* dst;
      if (CONTRACT_CONTIG) {
        const int row = q * 8 + (lane >> 3);
        const int chunk = (lane & 7) ^ ((row ^ (row >> 3)) & 7);
        const int k = kt * BK + chunk * 8;
        off = (kt >= 0 && k < K) ? lane_off + i * blk_step + k * 2 : kOobOffset;   // K tail reads as zeros
        dst = tile + q * 1024;
      } else {
        off = kt >= 0 ? lane_off + i * blk_step + kt * k_step : kOobOffset;        // k-rows past K fall out of range
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
    const int in_piece = ((col >> 5) * 2) * 64 + (col & 31) * 2;   // + 64 for the odd row of a pair
    const char* p0 = tile + (krow >> 1) * kPairPitch + (krow & 1) * 64 + in_piece;
    const int krow1 = krow + 4;
    const char* p1 = tile + (krow1 >> 1) * kPairPitch + (krow1 & 1) * 64 + in_piece;
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p0);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p1);
    const uint2 a = __builtin_bit_cast(uint2, lo), b = __builtin_bit_cast(uint2, hi);
    return make_uint4(a.x, a.y, b.x, b.y);
  }
}

// Epilogue of the 256x256 kernels: bias, optional pre-activation copy and activation, out through LDS.
// The tile leaves in four chunks of 64 rows through a staging area of 33 KB that does not touch the
// first stage of either operand, so that `prefetch_next` — called once all waves are done with the
// main loop's buffers — can already request the first k-tile of the workgroup's next output
// tile: it lands while this tile is written out, and the next tile starts without waiting for its
// first loads or, on this architecture's single in-order memory counter, for this tile's stores.
// Returns the number of global stores each lane issued after `prefetch_next` when that number is
// the same for every lane (a full tile with 16-byte aligned rows), -1 otherwise.
constexpr int kEpiRows = BM / 4;                               // rows per chunk
constexpr int kEpiStageBytes = kEpiRows * kEpiPitch;           // 33 792
constexpr int kEpiBiasBytes = BN * 4;                          // the tile's bias values as floats, behind the chunk
constexpr int kEpiSweeps = kEpiRows / (kBigThreads / 32);      // 16-byte stores per lane and chunk
// TO is T, or float for a product whose result is wanted in fp32 although the operands have 16 bits
// (the backward products under autocast: autograd would widen the 16-bit result anyway): the tile
// is staged rounded to T as always and widened by the store sweep, which then writes 1 KiB of a row
// per wave and takes twice the sweeps.
template <typename T, int ACT, typename TO, typename Prefetch>
__device__ __forceinline__ int big_tile_epilogue(f32x16 (&acc)[4][kBigNJ], char* stage, const GemmArgs& g, int m0,
                                                 int n0, Prefetch&& prefetch_next) {
  constexpr bool WIDE = !std::is_same<T, TO>::value;
  static_assert(!WIDE || (std::is_same<TO, float>::value && ACT == AT_ACT_NONE), "fp32 results only without activation");
  constexpr int NJ = kBigNJ;
  // a thread index the compiler takes for a new value: what the epilogue derives from it is worked
  // out here and not kept in registers across the main loop
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave / (kBigWaves / 2), wn = wave % (kBigWaves / 2);
  const int frag_row = lane & 31, frag_half = lane >> 5;
  // A lane holds, for tile (i, j) and register group rg, C[m][n .. n+3] with
  //   m = wm*128 + i*32 + lane%32,  n = wn*kBigWaveN + j*32 + rg*8 + (lane/32)*4   (tile-local).
  // Storing that straight to memory touches 32 rows per instruction with 16 bytes each; instead
  // the rows go through LDS and leave whole: 32 lanes x 16 bytes = one 512-byte row segment per
  // half-wave.  Chunk c holds row tile c of every wave, so that all eight share the work of each
  // chunk: rows 32 c .. 32 c + 31 of the upper and of the lower half of the tile.
  T* __restrict__ C = reinterpret_cast<T*>(g.c);
  T* __restrict__ P = reinterpret_cast<T*>(g.pre_act);
  const bool rows16 = WIDE ? (((g.ldc & 3) == 0) && aligned16_dev(g.c) && (n0 + BN <= g.N))
                           : (((g.ldc & 7) == 0) && aligned16_dev(C) && (n0 + BN <= g.N) &&
                              (!P || (((g.ldp & 7) == 0) && aligned16_dev(P))));
  const bool exact = rows16 && m0 + BM <= g.M;
  float* const bias_tile = reinterpret_cast<float*>(stage + kEpiStageBytes);
  // the bias of the tile's columns goes to LDS before anything else: a global load further down
  // would make the compiler wait for every store issued before it
  float bias_value = 0.f;
  if (g.bias && tid < BN && n0 + (int)tid < g.N)
    bias_value = load_scalar_f32(g.bias, g.bias_dt, n0 + tid);
  __syncthreads();              // every wave is done with the main loop's reads of LDS
  if (tid < BN) bias_tile[tid] = bias_value;
  // a use of the loaded value on every path: the compiler's wait for it comes here, not as a wait
  // for everything in flight somewhere behind the request below
  asm volatile("" ::"v"(bias_value));
  prefetch_next();
  constexpr int n_out = ACT != AT_ACT_NONE ? 2 : 1;
  int outputs = 0;
#pragma unroll
  for (int pass = 0; pass < n_out; ++pass) {
    const bool is_pre = (n_out == 2 && pass == 0);
    T* __restrict__ dst = is_pre ? P : C;
    const int64_t ldd = is_pre ? g.ldp : g.ldc;
    if (is_pre && !P) continue;   // uniform
    ++outputs;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      __syncthreads();            // previous readers of the staging area are done (and the bias is in place)
#pragma unroll
      for (int j = 0; j < NJ; ++j)
#pragma unroll
        for (int rg = 0; rg < 4; ++rg) {
          const int nl = wn * kBigWaveN + j * 32 + rg * 8 + frag_half * 4;
          const float4 bv = *reinterpret_cast<const float4*>(bias_tile + nl);
          float v[4] = {acc[c][j][rg * 4 + 0] + bv.x, acc[c][j][rg * 4 + 1] + bv.y, acc[c][j][rg * 4 + 2] + bv.z,
                        acc[c][j][rg * 4 + 3] + bv.w};
          if (ACT != AT_ACT_NONE && !is_pre) {
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = act_forward(ACT, v[e], g.param);
          }
          store_f32<T, 4>(reinterpret_cast<T*>(stage + (wm * 32 + frag_row) * kEpiPitch) + nl, v);
        }
      __syncthreads();
      if constexpr (WIDE) {
        // one row per wave and sweep: 64 lanes x 4 values, 16 bytes of fp32 each
        float* __restrict__ Cw = reinterpret_cast<float*>(g.c);
        const int rw = tid >> 6, cw = (tid & 63) * 4;
#pragma unroll
        for (int r0 = 0; r0 < kEpiRows; r0 += kBigThreads / 64) {
          const int ml = r0 + rw;
          const int m = m0 + (ml >> 5) * (BM / 2) + c * 32 + (ml & 31);
          if (m >= g.M) continue;
          float v[4];
          load_f32<T, 4>(reinterpret_cast<const T*>(stage + ml * kEpiPitch) + cw, v);
          float* out = Cw + (int64_t)m * g.ldc + n0 + cw;
          if (rows16) {
            *reinterpret_cast<float4*>(out) = make_float4(v[0], v[1], v[2], v[3]);
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n0 + cw + e < g.N) out[e] = v[e];
          }
        }
        continue;
      }
      // 2 rows per wave and sweep, 32 lanes x 16 bytes per row
      const int rsub = tid >> 5, cseg = (tid & 31) * 8;
#pragma unroll
      for (int r0 = 0; r0 < kEpiRows; r0 += kBigThreads / 32) {
        const int ml = r0 + rsub;
        const int m = m0 + (ml >> 5) * (BM / 2) + c * 32 + (ml & 31);
        if (m >= g.M) continue;
        if (rows16) {
          const uint4 v = *reinterpret_cast<const uint4*>(stage + ml * kEpiPitch + cseg * 2);
          *reinterpret_cast<uint4*>(dst + (int64_t)m * ldd + n0 + cseg) = v;
        } else {
          // Rows that do not start on 16-byte boundaries (an odd row stride) or a tile that sticks
          // out over the last column: the row segment is still written as whole 16-byte vectors
          // wherever memory allows — lane j takes the j-th aligned vector inside the segment and
          // gathers its 8 elements from LDS — and only the few elements before the first and after
          // the last aligned vector go out one by one.
          const int j = tid & 31;
          const int ncols = g.N - n0 < BN ? g.N - n0 : BN;
          T* seg = dst + (int64_t)m * ldd + n0;
          const T* src = reinterpret_cast<const T*>(stage + ml * kEpiPitch);
          const int head = (int)(((16 - (reinterpret_cast<uintptr_t>(seg) & 15)) & 15) >> 1);   // elements before the first boundary
          const int first = head < ncols ? head : ncols;
          const int nfull = (ncols - first) >> 3;
          if (j < nfull) {
            union { uint4 raw; T e[8]; } u;
#pragma unroll
            for (int e = 0; e < 8; ++e) u.e[e] = src[first + j * 8 + e];
            *reinterpret_cast<uint4*>(seg + first + j * 8) = u.raw;
          }
          if (j < first) seg[j] = src[j];
          const int tail0 = first + nfull * 8;
          if (tail0 + j < ncols && j < 8) seg[tail0 + j] = src[tail0 + j];
        }
      }
    }
  }
  return exact ? outputs * 4 * kEpiSweeps * (WIDE ? 2 : 1) : -1;
}

// ACT is the compile-time activation id of the epilogue (the act switch must fold away: the
// epilogue is fully unrolled over the accumulator registers).
template <typename T, bool A_MC, bool B_KC, int ACT, typename TO = T>
__global__ __launch_bounds__(kBigThreads) void gemm_mfma16_kernel(GemmArgs g) {
  constexpr bool A_KC = !A_MC;
  constexpr int kATile = operand_tile_bytes<A_KC>(), kBTile = operand_tile_bytes<B_KC>();
  // When both operands are contraction-contiguous (32 KB tiles) the A tiles live in a ring of
  // three stages and the B tiles in one of two — all of the CU's 160 KB: A's loads then run two
  // k-tiles ahead of their use, B's one (see the main loop); that product gains 6 %.  The other
  // layouts have padded tiles that do not fit a third stage (and the forward product, tried with
  // unpadded tiles, gains under 1 % from it): two stages each.
  constexpr int kAStages = (A_KC && B_KC) ? 3 : 2;
  constexpr int kARing = kAStages * kATile;
  constexpr int kLds = kARing + 2 * kBTile;
  static_assert(kLds <= 160 * 1024, "the stages fill the LDS of a CU exactly");
  // The epilogue's staging area lies behind the first stage of A where A's later stages hold it,
  // else in B's second stage: the first stage of either operand stays free for the next tile.
  constexpr int kEpiNeed = kEpiStageBytes + kEpiBiasBytes;
  constexpr int kEpiOff = (kAStages - 1) * kATile >= kEpiNeed ? kATile : kARing + kBTile;
  static_assert(kEpiOff == kATile || kBTile >= kEpiNeed, "the staging area fits behind the first stages");
  __shared__ __attribute__((aligned(1024))) char lds[kLds];  // A ring | B ring; the epilogue stages chunks of the output at kEpiOff
  const T* __restrict__ A = reinterpret_cast<const T*>(g.a);
  const T* __restrict__ B = reinterpret_cast<const T*>(g.b);

  // ---- workgroup -> output tiles, XCD aware.  The grid may be smaller than the number of tiles
  // (a multiple of 8 workgroups, so that a workgroup's tiles all carry its XCD number): a
  // workgroup then takes tiles blockIdx.x, blockIdx.x + gridDim.x, ... one after the other ----
  const int nbm = (g.M + BM - 1) / BM, nbn = (g.N + BN - 1) / BN;
  const int total = nbm * nbn;
  auto tile_origin = [&](int bid, int& m0_, int& n0_) {
    const int xcd = bid & 7, idx = bid >> 3;
    const int q = total >> 3, rem = total & 7;
    const int logical = xcd * q + (xcd < rem ? xcd : rem) + idx;
    constexpr int GROUP = 8;
    const int per_group = GROUP * nbn;
    const int first_m = (logical / per_group) * GROUP;
    const int gsz = nbm - first_m < GROUP ? nbm - first_m : GROUP;
    const int in_group = logical % per_group;
    m0_ = (first_m + in_group % gsz) * BM;
    n0_ = (in_group / gsz) * BN;
  };
  char* const a_ring = lds;
  char* const b_ring = lds + kARing;
  // k-tile 0 of a tile after the workgroup's first is requested from inside the epilogue of the
  // tile before it; `stores_behind` is what that epilogue issued after the request (-1: unknown)
  bool requested = false;
  int stores_behind = -1;
  for (int tile_id = blockIdx.x; tile_id < total; tile_id += gridDim.x) {
  int m0, n0;
  tile_origin(tile_id, m0, n0);

  const int wave = threadIdx.x >> 6;
  constexpr int NJ = kBigNJ;
  const int wm = wave / (kBigWaves / 2), wn = wave % (kBigWaves / 2);

  f32x16 acc[4][NJ];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  OperandLoader<T, A_KC> la;
  OperandLoader<T, B_KC> lb;
  int tid = threadIdx.x;
  asm volatile("" : "+v"(tid));   // keeps the lane's offsets from being hoisted out of the tile loop and held across the epilogue
  la.init(A, g.lda, m0, g.M, g.K, tid);
  lb.init(B, g.ldb, n0, g.N, g.K, tid);
  const int KT = (g.K + BK - 1) / BK;

  auto load_frags = [&](const char* a_stage, const char* b_stage, int ks, uint4 (&af)[4], uint4 (&bf)[NJ]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) af[i] = read_frag<A_KC>(a_stage, wm * 128 + i * 32, ks);
#pragma unroll
    for (int j = 0; j < NJ; ++j) bf[j] = read_frag<B_KC>(b_stage, wn * kBigWaveN + j * 32, ks);
  };

  if (!requested) {
    la.issue(0, a_ring);
    lb.issue(0, b_ring);
  }
  // The memory counter runs in issue order and counts stores too: leaving exactly the stores of
  // the last epilogue outstanding waits for k-tile 0 and not for their acknowledgements.
  if (stores_behind == 4 * kEpiSweeps) lds_dma_wait_newest<4 * kEpiSweeps>();
  else if (stores_behind == 8 * kEpiSweeps) lds_dma_wait_newest<8 * kEpiSweeps>();
  else lds_dma_wait_all();
  __syncthreads();      // k-tile 0 is everybody's; the last epilogue's readers of the staging area are done
  // k-tiles 1 (both operands) and 2 (A) travel while k-tile 0 is multiplied (zeros when there are
  // none).  A's tile 2 is issued last: the in-order counter then lets it stay in flight across the
  // first wait.
  la.issue(1, a_ring + kATile);
  lb.issue(1, b_ring + kBTile);
  if (kAStages == 3) la.issue(2 < KT ? 2 : -1, a_ring + 2 * kATile);
  uint4 af[2][4], bf[2][NJ];
  load_frags(a_ring, b_ring, 0, af[0], bf[0]);

  // One k-tile = four k-steps of 4 * NJ MFMAs per wave, the other instructions slotted between
  // them.  K-steps 0..2 multiply while the fragments of the following k-step are read.  Before
  // k-step 3 every fragment of the current stage is in registers, so the one barrier of the
  // iteration both publishes k-tile kt+1 and frees the current stages: k-step 3 multiplies while
  // B's k-tile kt+2 and then A's k-tile kt+3 are issued into them and the first fragments of
  // k-tile kt+1 are read, so the MFMAs run on across the barrier.  The wait before the barrier
  // leaves the newest kBigLoads loads of the wave (A's k-tile kt+2, issued last in the previous
  // iteration) in flight: A's tiles have two iterations to arrive, B's one.
  // (sched_group_barrier masks: 0x8 MFMA, 0x2 VALU, 0x20 VMEM read, 0x100 LDS read.)
  int a_slot = 0;   // kt % kAStages
  for (int kt = 0; kt < KT; ++kt) {
    const int a_this = kAStages == 3 ? a_slot : (kt & 1);
    const int a_next = kAStages == 3 ? (a_slot == 2 ? 0 : a_slot + 1) : (a_this ^ 1);
    char* a_cur = a_ring + a_this * kATile;
    char* a_nxt = a_ring + a_next * kATile;
    char* b_cur = b_ring + (kt & 1) * kBTile;
    char* b_nxt = b_ring + ((kt & 1) ^ 1) * kBTile;
    a_slot = a_next;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int ks = 0; ks < BK / 16 - 1; ++ks) {
      load_frags(a_cur, b_cur, ks + 1, af[(ks + 1) & 1], bf[(ks + 1) & 1]);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
          // operands swapped: the accumulator holds C^T, i.e. 4 consecutive n per lane
          acc[i][j] = Mfma16<T>::run(bf[ks & 1][j], af[ks & 1][i], acc[i][j]);
#pragma unroll
      for (int q = 0; q < 4 * NJ; ++q) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // k-tile kt+1: this wave's part has landed
    if (kAStages == 3) lds_dma_wait_newest<kBigLoads>(); else lds_dma_wait_all();
    __syncthreads();                    // ... and everybody's; nobody reads the current stages any more
    // Past the last k-tile the loads are issued all the same, with offsets that are out of range:
    // they write zeros into a stage nobody reads, and the loop body has no branches.
    const int kt2 = kt + 2 < KT ? kt + 2 : -1;
    const int kt3 = kt + kAStages < KT ? kt + kAStages : -1;   // A's next tile: two or three ahead
    load_frags(a_nxt, b_nxt, 0, af[0], bf[0]);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        // one global->LDS load behind each MFMA (2 * kBigLoads = 4 * NJ of either)
        const int t = i * NJ + j;
        // with three A stages A's loads must be the wave's newest (they stay in flight over the wait)
        if ((t < kBigLoads) == (kAStages == 3)) lb.issue_one(kt2, b_cur, t % kBigLoads);
        else la.issue_one(kt3, a_cur, t % kBigLoads);
        acc[i][j] = Mfma16<T>::run(bf[1][j], af[1][i], acc[i][j]);
      }
#pragma unroll
    for (int q = 0; q < 4 * NJ; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  lds_dma_wait_all();   // the zero-fill loads past the end: the epilogue reuses the stages

  const int next_id = tile_id + gridDim.x;
  requested = next_id < total;
  stores_behind = big_tile_epilogue<T, ACT, TO>(acc, lds + kEpiOff, g, m0, n0, [&] {
    if (!requested) return;
    int m1, n1;
    tile_origin(next_id, m1, n1);
    // The lane's offsets are worked out afresh from a thread index the compiler takes for a new
    // value: shared with the main loop's loaders they would be kept across it, in registers it
    // does not have.
    int tid1 = threadIdx.x;
    asm volatile("" : "+v"(tid1));
    OperandLoader<T, A_KC> la1;
    OperandLoader<T, B_KC> lb1;
    la1.init(A, g.lda, m1, g.M, g.K, tid1);
    lb1.init(B, g.ldb, n1, g.N, g.K, tid1);
    la1.issue(0, a_ring);
    lb1.issue(0, b_ring);
  });
  }
}

// ------------------------------------------------------------------------------------------
// Mid-size problems: 128x128x64 tiles, 2x2 waves of 64x64.  The same operands as the kernel above
// for shapes whose 256x256 tiling would leave most of the CUs idle.  Two workgroups share a CU
// (64 accumulator registers per lane, 66 KB of LDS) and cover each other's latencies, so the
// loop is plain: issue the loads of tile kt+1, multiply tile kt, one barrier.  The activation
// is applied after the accumulators have been staged in LDS as fp32, in a rolled loop, so one
// kernel serves every activation.
// ------------------------------------------------------------------------------------------
constexpr int MT = 128;                          // tile edge
constexpr int kMidTileBytes = MT * BK * 2;       // one operand tile, 16 KiB
constexpr int kMidStage = 2 * kMidTileBytes;
constexpr int kMidEpiPitch = MT + 4;             // floats per row of the staged output tile

// LDS image of an operand tile stored [k][outer] in memory: 64 k-rows x 256 bytes as loaded,
// four rows per KiB (one wave-wide load), the 16-byte chunk index XORed with 4 * (k-row % 4) so
// that the four rows a transposing fragment read touches fall on different banks.
template <typename T, bool CONTRACT_CONTIG>
struct MidLoader {
  i32x4 rsrc;
  int lane_off, blk_step, k_step, K;

  int tid;   // thread index inside the four waves that load a tile together

  __device__ __forceinline__ void init(const T* base, int64_t ld, int outer0, int outer_total, int K_, int tid_) {
    tid = tid_;
    const int lane = tid & 63, wave = tid >> 6;
    K = K_;
    if (CONTRACT_CONTIG) {
      rsrc = make_buffer_rsrc(base, ((int64_t)(outer_total - 1) * ld + K_) * 2);
      lane_off = (int)(((int64_t)(outer0 + wave * 32 + (lane >> 3)) * ld) * 2);   // + 8 rows per load
      blk_step = (int)(8 * ld * 2);
      k_step = BK * 2;
    } else {
      rsrc = make_buffer_rsrc(base, ((int64_t)(K_ - 1) * ld + ((outer_total + 7) & ~7)) * 2);
      const int krow = wave * 16 + (lane >> 4);                                    // + 4 k-rows per load
      const int chunk = (lane & 15) ^ ((krow & 3) << 2);
      lane_off = (int)(((int64_t)krow * ld + outer0 + chunk * 8) * 2);
      blk_step = (int)(4 * ld * 2);
      k_step = (int)(BK * ld * 2);
    }
  }
  __device__ __forceinline__ void issue(int kt, char* tile) const {
    const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = wave * 4 + i;
      int off;
      if (CONTRACT_CONTIG) {
        const int row = q * 8 + (lane >> 3);
        const int chunk = (lane & 7) ^ ((row ^ (row >> 3)) & 7);
        const int k = kt * BK + chunk * 8;
        off = k < K ? lane_off + i * blk_step + k * 2 : kOobOffset;
      } else {
        // k-rows at or past K lie past the end of the buffer and read as zeros
        off = kt * BK < K ? lane_off + i * blk_step + kt * k_step : kOobOffset;
      }
      lds_dma_16(rsrc, off, tile + q * 1024);
    }
  }
};

template <bool CONTRACT_CONTIG>
__device__ __forceinline__ uint4 read_frag_mid(const char* tile, int outer_base, int ks) {
  const int lane = threadIdx.x & 63;
  if (CONTRACT_CONTIG) {
    return read_frag_kc(tile, outer_base, ks);
  } else {
    // see read_frag: source lane 4e + q of a 16-lane group points at k-row k0 + e, columns 4q .. 4q+3
    const int i = lane & 15, g = lane >> 4;
    const int col = outer_base + (g & 1) * 16 + (i & 3) * 4;
    const int krow = ks * 16 + (g >> 1) * 8 + (i >> 2);
    const char* p0 = tile + (krow >> 2) * 1024 + (krow & 3) * 256 + ((((col >> 3) ^ ((krow & 3) << 2)) & 15) << 4) +
                     (col & 7) * 2;
    const char* p1 = p0 + 1024;   // k-row + 4: the next KiB, same position
    typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p0);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)p1);
    const uint2 a = __builtin_bit_cast(uint2, lo), b = __builtin_bit_cast(uint2, hi);
    return make_uint4(a.x, a.y, b.x, b.y);
  }
}

// TO as in big_tile_epilogue: T, or float for the value rounded to T and widened (no activation).
// KG = 2: for problems with at most one tile per CU.  The workgroup has eight waves in two groups
// of four; each group multiplies every other k-tile of the same output tile from LDS stages of its
// own, and the two sets of accumulators are added while the tile is staged for the epilogue.  A CU
// then has two waves per SIMD to cover each other's waits, as it has with two workgroups of four.
template <typename T, bool A_MC, bool B_KC, bool SPLIT, typename TO = T, int KG = 1>
__global__ __launch_bounds__(kGemmThreads * KG, KG == 1 ? 2 : 1) void gemm_mid16_kernel(GemmArgs g) {
  constexpr bool A_KC = !A_MC;
  static_assert(KG == 1 || (KG == 2 && !SPLIT), "one or two k-groups; no k-groups inside a split of the contraction");
  constexpr int kStagesBytes = KG * 2 * kMidStage;
  constexpr int kEpiBytes = KG * MT * kMidEpiPitch * 4;
  __shared__ __attribute__((aligned(1024))) char lds[kStagesBytes > kEpiBytes ? kStagesBytes : kEpiBytes];
  const T* __restrict__ A = reinterpret_cast<const T*>(g.a);
  const T* __restrict__ B = reinterpret_cast<const T*>(g.b);

  // workgroup -> output tile: consecutive ids go round the XCDs, so each XCD gets a contiguous
  // run of tiles, walked in groups of 8 tile rows
  const int nbm = (g.M + MT - 1) / MT, nbn = (g.N + MT - 1) / MT;
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
  const int m0 = (first_m + in_group % gsz) * MT;
  const int n0 = (in_group / gsz) * MT;

  const int lane = threadIdx.x & 63, wave = (threadIdx.x >> 6) & 3;
  const int kgroup = KG == 1 ? 0 : (int)(threadIdx.x >> 8);
  const int wm = wave >> 1, wn = wave & 1;
  char* const stages = lds + kgroup * 2 * kMidStage;   // this k-group's two stages

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  MidLoader<T, A_KC> la;
  MidLoader<T, B_KC> lb;
  la.init(A, g.lda, m0, g.M, g.K, threadIdx.x & 255);
  lb.init(B, g.ldb, n0, g.N, g.K, threadIdx.x & 255);
  int kt0 = 0, KT = (g.K + BK - 1) / BK;
  if (SPLIT) {
    kt0 = blockIdx.y * g.kt_per_split;
    KT = kt0 + g.kt_per_split < KT ? kt0 + g.kt_per_split : KT;   // the host leaves no split empty
  }
  // k-group q takes k-tiles kt0 + q, kt0 + q + KG, ...; both groups make the same number of steps (a
  // k-tile past the end reads as zeros), so every wave passes every barrier
  kt0 += kgroup;
  la.issue(kt0, stages);
  lb.issue(kt0, stages + kMidTileBytes);
  lds_dma_wait_all();
  __syncthreads();

  for (int kt = kt0, step = 0; kt - kgroup < KT; kt += KG, ++step) {
    const char* cur = stages + (step & 1) * kMidStage;
    char* nxt = stages + ((step & 1) ^ 1) * kMidStage;
    if (kt - kgroup + KG < KT) {
      la.issue(kt + KG, nxt);
      lb.issue(kt + KG, nxt + kMidTileBytes);
    }
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      uint4 af[2], bf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        af[i] = read_frag_mid<A_KC>(cur, wm * 64 + i * 32, ks);
        bf[i] = read_frag_mid<B_KC>(cur + kMidTileBytes, wn * 64 + i * 32, ks);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = Mfma16<T>::run(bf[j], af[i], acc[i][j]);   // C^T: 4 consecutive n per lane
    }
    lds_dma_wait_all();
    __syncthreads();
  }

  // ---- epilogue: accumulators (+ bias) -> LDS as fp32 -> rows of 8 columns per lane ----
  // A lane holds, for tile (i, j) and register group rg, C[m][n .. n+3] with
  //   m = wm*64 + i*32 + lane%32,  n = wn*64 + j*32 + rg*8 + (lane/32)*4   (tile-local).
  float* stage = reinterpret_cast<float*>(lds) + kgroup * MT * kMidEpiPitch;   // k-group 1 stages its sums behind group 0's
  const bool with_bias = g.bias && kgroup == 0;
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
      const int nl = wn * 64 + j * 32 + rg * 8 + (lane >> 5) * 4;
      float bv[4] = {0.f, 0.f, 0.f, 0.f};
      if (with_bias) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n0 + nl + e < g.N) bv[e] = load_scalar_f32(g.bias, g.bias_dt, n0 + nl + e);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int ml = wm * 64 + i * 32 + (lane & 31);
        float4 v;
        v.x = acc[i][j][rg * 4 + 0] + bv[0];
        v.y = acc[i][j][rg * 4 + 1] + bv[1];
        v.z = acc[i][j][rg * 4 + 2] + bv[2];
        v.w = acc[i][j][rg * 4 + 3] + bv[3];
        *reinterpret_cast<float4*>(stage + ml * kMidEpiPitch + nl) = v;
      }
    }
  __syncthreads();
  // 16 rows per sweep and k-group, 16 lanes x 8 columns per row; the sums of the k-groups are added here
  const int rsub = threadIdx.x >> 4, cseg = (threadIdx.x & 15) * 8;
  constexpr int kSweepRows = 16 * KG;
  auto load8 = [&](int ml, float (&v)[8]) {
    const float* src = reinterpret_cast<const float*>(lds) + ml * kMidEpiPitch + cseg;
    *reinterpret_cast<float4*>(v) = *reinterpret_cast<const float4*>(src);
    *reinterpret_cast<float4*>(v + 4) = *reinterpret_cast<const float4*>(src + 4);
    if (KG == 2) {
      const float4 lo = *reinterpret_cast<const float4*>(src + MT * kMidEpiPitch);
      const float4 hi = *reinterpret_cast<const float4*>(src + MT * kMidEpiPitch + 4);
      v[0] += lo.x; v[1] += lo.y; v[2] += lo.z; v[3] += lo.w;
      v[4] += hi.x; v[5] += hi.y; v[6] += hi.z; v[7] += hi.w;
    }
  };
  if (SPLIT) {
    // partial tile as fp32; ldw is a multiple of 8, so whole segments stay inside the row
    float* part = g.partial + (int64_t)blockIdx.y * g.M * g.ldw;
    for (int r0 = 0; r0 < MT; r0 += 16) {
      const int ml = r0 + rsub, m = m0 + ml;
      if (m >= g.M || n0 + cseg >= g.N) continue;
      float* out = part + (int64_t)m * g.ldw + n0 + cseg;
      *reinterpret_cast<float4*>(out) = *reinterpret_cast<const float4*>(stage + ml * kMidEpiPitch + cseg);
      *reinterpret_cast<float4*>(out + 4) = *reinterpret_cast<const float4*>(stage + ml * kMidEpiPitch + cseg + 4);
    }
    return;
  }
  if constexpr (!std::is_same<T, TO>::value) {
    float* __restrict__ Cw = reinterpret_cast<float*>(g.c);
    const bool rows16w = ((g.ldc & 3) == 0) && aligned16_dev(Cw) && (n0 + MT <= g.N);
    for (int r0 = 0; r0 < MT; r0 += kSweepRows) {
      const int ml = r0 + rsub, m = m0 + ml;
      if (m >= g.M) continue;
      float v[8];
      load8(ml, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = to_f32(from_f32<T>(v[e]));
      float* out = Cw + (int64_t)m * g.ldc + n0 + cseg;
      if (rows16w) {
        *reinterpret_cast<float4*>(out) = *reinterpret_cast<const float4*>(v);
        *reinterpret_cast<float4*>(out + 4) = *reinterpret_cast<const float4*>(v + 4);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (n0 + cseg + e < g.N) out[e] = v[e];
      }
    }
    return;
  }
  T* __restrict__ C = reinterpret_cast<T*>(g.c);
  T* __restrict__ P = g.act != AT_ACT_NONE ? reinterpret_cast<T*>(g.pre_act) : nullptr;
  const bool rows16 = ((g.ldc & 7) == 0) && aligned16_dev(C) && (n0 + MT <= g.N) &&
                      (!P || (((g.ldp & 7) == 0) && aligned16_dev(P)));
  for (int r0 = 0; r0 < MT; r0 += kSweepRows) {
    const int ml = r0 + rsub, m = m0 + ml;
    if (m >= g.M) continue;
    float v[8];
    load8(ml, v);
    if (P) {
      T* out = P + (int64_t)m * g.ldp + n0 + cseg;
      if (rows16) {
        store_f32<T, 8>(out, v);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (n0 + cseg + e < g.N) out[e] = from_f32<T>(v[e]);
      }
    }
    if (g.act != AT_ACT_NONE) {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = act_forward(g.act, v[e], g.param);
    }
    T* out = C + (int64_t)m * g.ldc + n0 + cseg;
    if (rows16) {
      store_f32<T, 8>(out, v);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (n0 + cseg + e < g.N) out[e] = from_f32<T>(v[e]);
    }
  }
}

// C[m][n] = sum over the splits of partial[s][m][n], rounded once to T.  One lane per 8 columns.
// TO = T, or float for the rounded value widened (as in big_tile_epilogue).
template <typename T, typename TO = T>
__global__ __launch_bounds__(256) void gemm_split_finish_kernel(const float* __restrict__ partial, TO* __restrict__ C,
                                                                int M, int N, int ldw, int64_t ldc, int splits) {
  const int segs = ldw / 8;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)M * segs) return;
  const int m = (int)(idx / segs), n = (int)(idx % segs) * 8;
  if (n >= N) return;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  const float* src = partial + (int64_t)m * ldw + n;
#pragma unroll 4
  for (int sidx = 0; sidx < splits; ++sidx) {
    const float4 lo = *reinterpret_cast<const float4*>(src), hi = *reinterpret_cast<const float4*>(src + 4);
    acc[0] += lo.x; acc[1] += lo.y; acc[2] += lo.z; acc[3] += lo.w;
    acc[4] += hi.x; acc[5] += hi.y; acc[6] += hi.z; acc[7] += hi.w;
    src += (int64_t)M * ldw;
  }
  TO* out = C + (int64_t)m * ldc + n;
  if constexpr (!std::is_same<T, TO>::value) {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = to_f32(from_f32<T>(acc[e]));
  }
  constexpr int kPer = 16 / (int)sizeof(TO);   // elements per 16 bytes of output
  if (n + 8 <= N && (ldc % kPer) == 0 && aligned16_dev(C)) {
    store_f32<TO, 8>(out, acc);
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (n + e < N) out[e] = from_f32<TO>(acc[e]);
  }
}

// ------------------------------------------------------------------------------------------
// fp32 operands on v_mfma_f32_32x32x2f32 (MFMA-bound: one MFMA is 64 cycles for 512 bytes of
// operands, so LDS and the loads have time to spare).  (64 WT) x (64 WT) x 16 tiles, 2x2 waves,
// tiles straight from global memory into LDS, two stages, one barrier per k-tile.  The MFMA
// takes one value per lane and operand, so either memory layout is read with plain ds_read_b32:
//  * rows along the contraction ([outer][k]): 64-byte rows of 16 k, the 16-byte chunk index
//    XORed with (row / 4) % 4 so that 16 consecutive rows read at one k fall on different banks;
//  * the other way round ([k][outer]): rows of 64 WT * 4 bytes as loaded, consecutive lanes
//    read consecutive addresses.
// ------------------------------------------------------------------------------------------
constexpr int FK = 16;   // k per tile (the swizzle below is written for 64-byte rows)

template <int WT, bool CONTRACT_CONTIG>
struct F32Loader {
  static constexpr int TILE = 64 * WT;
  static constexpr int kBytes = TILE * FK * 4;
  static constexpr int kLoads = kBytes / 1024 / 4;   // wave-wide loads per wave
  i32x4 rsrc;
  int lane_off, blk_step, k_step, k_lane, K;

  __device__ __forceinline__ void init(const float* base, int64_t ld, int outer0, int outer_total, int K_) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    K = K_;
    if (CONTRACT_CONTIG) {
      rsrc = make_buffer_rsrc(base, ((int64_t)(outer_total - 1) * ld + K_) * 4);
      // a wave-wide load fills 16 rows of 64 bytes: lane -> row lane / 4, position lane % 4
      const int row = wave * (kLoads * 16) + (lane >> 2);          // + 16 i
      k_lane = ((lane & 3) ^ ((row >> 2) & 3)) * 4;                // the same for row + 16
      lane_off = (int)(((int64_t)(outer0 + row) * ld) * 4) + k_lane * 4;
      blk_step = (int)(16 * ld * 4);
      k_step = FK * 4;
    } else {
      rsrc = make_buffer_rsrc(base, ((int64_t)(K_ - 1) * ld + ((outer_total + 3) & ~3)) * 4);
      // a wave-wide load fills 1024 / (4 TILE) k-rows: lane -> k-row lane / TILE', 4 columns
      constexpr int LPR = TILE / 4;                                // lanes per k-row
      constexpr int RPL = 64 / LPR;                                // k-rows per load
      const int krow = wave * (kLoads * RPL) + lane / LPR;         // + RPL i
      k_lane = 0;
      lane_off = (int)(((int64_t)krow * ld + outer0 + (lane % LPR) * 4) * 4);
      blk_step = (int)(RPL * ld * 4);
      k_step = (int)(FK * ld * 4);
    }
  }
  __device__ __forceinline__ void issue(int kt, char* tile) const {
    const int wave = threadIdx.x >> 6;
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      int off;
      if (CONTRACT_CONTIG) off = kt * FK + k_lane < K ? lane_off + i * blk_step + kt * k_step : kOobOffset;
      else off = lane_off + i * blk_step + kt * k_step;          // k-rows past K fall out of range
      lds_dma_16(rsrc, off, tile + (wave * kLoads + i) * 1024);
    }
  }
  // value (outer, k) of the tile
  static __device__ __forceinline__ float read(const char* tile, int outer, int k) {
    if (CONTRACT_CONTIG)
      return *reinterpret_cast<const float*>(tile + outer * 64 + ((((k >> 2) ^ (outer >> 2)) & 3) << 4) + (k & 3) * 4);
    else
      return *reinterpret_cast<const float*>(tile + k * (TILE * 4) + outer * 4);
  }
};

template <int WT, bool A_MC, bool B_KC>
__global__ __launch_bounds__(256) void gemm_f32_kernel(GemmArgs g) {
  constexpr int TILE = 64 * WT;
  constexpr int kTile = TILE * FK * 4, kStage = 2 * kTile;
  // ring of NS stages, NS - 1 k-tiles of loads in flight: small tiles have little work per k-tile
  // to cover the load latency with, so they look further ahead
  constexpr int NS = WT == 1 ? 6 : 3;
  constexpr int kLoadsPerIter = 2 * (kTile / 1024 / 4);
  __shared__ __attribute__((aligned(1024))) char lds[NS * kStage];
  const float* __restrict__ A = reinterpret_cast<const float*>(g.a);
  const float* __restrict__ B = reinterpret_cast<const float*>(g.b);

  const int nbm = (g.M + TILE - 1) / TILE, nbn = (g.N + TILE - 1) / TILE;
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
  const int m0 = (first_m + in_group % gsz) * TILE;
  const int n0 = (in_group / gsz) * TILE;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  f32x16 acc[WT][WT];
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < WT; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  F32Loader<WT, !A_MC> la;
  F32Loader<WT, B_KC> lb;
  la.init(A, g.lda, m0, g.M, g.K);
  lb.init(B, g.ldb, n0, g.N, g.K);
  const int KT = (g.K + FK - 1) / FK;
  // loads past the last k-tile are issued all the same (they are out of range and write zeros into
  // stages nobody reads), so the number of loads in flight is the same in every iteration
#pragma unroll
  for (int t = 0; t < NS - 1; ++t) {
    la.issue(t, lds + t * kStage);
    lb.issue(t, lds + t * kStage + kTile);
  }
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoadsPerIter * (NS - 2)) : "memory");   // k-tile 0 has landed
  __syncthreads();

  int cur_stage = 0;
  for (int kt = 0; kt < KT; ++kt) {
    const char* cur = lds + cur_stage * kStage;
    {
      const int fill = cur_stage == 0 ? NS - 1 : cur_stage - 1;   // the stage the previous iteration left
      la.issue(kt + NS - 1, lds + fill * kStage);
      lb.issue(kt + NS - 1, lds + fill * kStage + kTile);
    }
    cur_stage = cur_stage + 1 == NS ? 0 : cur_stage + 1;
#pragma unroll
    for (int ks = 0; ks < FK / 2; ++ks) {
      const int k = ks * 2 + (lane >> 5);
      float av[WT], bv[WT];
#pragma unroll
      for (int i = 0; i < WT; ++i) {
        av[i] = F32Loader<WT, !A_MC>::read(cur, wm * 32 * WT + i * 32 + (lane & 31), k);
        bv[i] = F32Loader<WT, B_KC>::read(cur + kTile, wn * 32 * WT + i * 32 + (lane & 31), k);
      }
#pragma unroll
      for (int i = 0; i < WT; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[j], av[i], acc[i][j], 0, 0, 0);   // C^T: 4 consecutive n per lane
    }
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoadsPerIter * (NS - 2)) : "memory");   // k-tile kt + 1 has landed
    __syncthreads();
  }
  lds_dma_wait_all();   // the zero-fill loads past the end: the epilogue reuses the stages
  __syncthreads();

  // Epilogue.  A lane holds, for tile (i, j) and register group rg, C[m][n .. n+3] with
  //   m = wm*32*WT + i*32 + lane%32,  n = wn*32*WT + j*32 + rg*8 + (lane/32)*4   (tile-local).
  // Each wave passes its 32 x (32 WT) block of rows through a private piece of LDS and finishes it
  // in a rolled loop (bias, pre-activation copy, activation chosen at run time, 16-byte stores of
  // whole row segments), so the activation code exists once instead of once per accumulator.
  constexpr int W = 32 * WT, kPitch = W + 4;
  static_assert(4 * 32 * kPitch * 4 <= NS * kStage, "the wave blocks fit in the stages");
  float* block = reinterpret_cast<float*>(lds) + wave * 32 * kPitch;
  float* __restrict__ C = reinterpret_cast<float*>(g.c);
  float* __restrict__ P = g.act != AT_ACT_NONE ? reinterpret_cast<float*>(g.pre_act) : nullptr;
  const bool vec_c = (g.ldc & 3) == 0 && aligned16_dev(C), vec_p = P && (g.ldp & 3) == 0 && aligned16_dev(P);
  constexpr int SEGS = W / 4, ROWS_PER_IT = 64 / SEGS;
  const int seg = lane % SEGS, rsub = lane / SEGS;
  const int n = n0 + wn * W + seg * 4;
  float bias4[4] = {0.f, 0.f, 0.f, 0.f};
  if (g.bias) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (n + e < g.N) bias4[e] = load_scalar_f32(g.bias, g.bias_dt, n + e);
  }
#pragma unroll
  for (int i = 0; i < WT; ++i) {
#pragma unroll
    for (int jj = 0; jj < WT; ++jj)
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        const f32x16& a = acc[i][jj];
        *reinterpret_cast<float4*>(block + (lane & 31) * kPitch + jj * 32 + rg * 8 + (lane >> 5) * 4) =
            make_float4(a[rg * 4 + 0], a[rg * 4 + 1], a[rg * 4 + 2], a[rg * 4 + 3]);
      }
    // same wave: LDS operations complete in order; only the compiler has to keep them in place
    __builtin_amdgcn_wave_barrier();
#pragma unroll 1
    for (int it = 0; it < 32 / ROWS_PER_IT; ++it) {
      const int r = it * ROWS_PER_IT + rsub;
      const int m = m0 + wm * W + i * 32 + r;
      const float4 raw = *reinterpret_cast<const float4*>(block + r * kPitch + seg * 4);
      if (m >= g.M || n >= g.N) continue;
      float v[4] = {raw.x + bias4[0], raw.y + bias4[1], raw.z + bias4[2], raw.w + bias4[3]};
      const bool whole = n + 4 <= g.N;
      if (P) {
        float* out = P + (int64_t)m * g.ldp + n;
        if (whole && vec_p) {
          *reinterpret_cast<float4*>(out) = make_float4(v[0], v[1], v[2], v[3]);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < g.N) out[e] = v[e];
        }
      }
      if (g.act != AT_ACT_NONE) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = act_forward(g.act, v[e], g.param);
      }
      float* out = C + (int64_t)m * g.ldc + n;
      if (whole && vec_c) {
        *reinterpret_cast<float4*>(out) = make_float4(v[0], v[1], v[2], v[3]);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < g.N) out[e] = v[e];
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
}

// v rounded to a 16-bit dtype and widened again (fp32: v itself).
__device__ __forceinline__ float round_through(float v, int dt) {
  if (dt == AT_DTYPE_F16) return to_f32(from_f32<f16_t>(v));
  if (dt == AT_DTYPE_BF16) return to_f32(from_f32<bf16_t>(v));
  return v;
}

// Epilogue of the generic kernels: one 32x32 accumulator tile per wave (register r of a lane =
// C[m = lane % 32][n = (r / 4) * 8 + (lane / 32) * 4 + r % 4]) goes through a wave-private block
// of LDS (32 rows of 36 floats) and is finished in a rolled loop, so that the run-time activation
// switch exists once and not once per accumulator register.  `block` must not be in use by
// anybody else; rows are stored as segments of 4 consecutive columns.
template <typename TO, typename ARGS>
__device__ __forceinline__ void wave_tile_epilogue(const f32x16& acc, float* block, const ARGS& g, int m_base,
                                                   int n_base) {
  constexpr int kPitch = 36;
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int rg = 0; rg < 4; ++rg)
    *reinterpret_cast<float4*>(block + (lane & 31) * kPitch + rg * 8 + (lane >> 5) * 4) =
        make_float4(acc[rg * 4 + 0], acc[rg * 4 + 1], acc[rg * 4 + 2], acc[rg * 4 + 3]);
  __builtin_amdgcn_wave_barrier();   // same wave: LDS operations complete in order
  TO* __restrict__ C = reinterpret_cast<TO*>(g.c);
  TO* __restrict__ P = g.act != AT_ACT_NONE ? reinterpret_cast<TO*>(g.pre_act) : nullptr;
  const int seg = lane & 7, rsub = lane >> 3;
  const int n = n_base + seg * 4;
  float bias4[4] = {0.f, 0.f, 0.f, 0.f};
  if (g.bias) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (n + e < g.N) bias4[e] = load_scalar_f32(g.bias, g.bias_dt, n + e);
  }
#pragma unroll 1
  for (int it = 0; it < 4; ++it) {
    const int r = it * 8 + rsub;
    const int m = m_base + r;
    const float4 raw = *reinterpret_cast<const float4*>(block + r * kPitch + seg * 4);
    if (m >= g.M || n >= g.N) continue;
    float v[4] = {raw.x + bias4[0], raw.y + bias4[1], raw.z + bias4[2], raw.w + bias4[3]};
    if (P) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < g.N) P[(int64_t)m * g.ldp + n + e] = from_f32<TO>(v[e]);
    }
    if (g.act != AT_ACT_NONE) {
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = act_forward(g.act, v[e], g.param);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (n + e < g.N) C[(int64_t)m * g.ldc + n + e] = from_f32<TO>(round_through(v[e], g.round_dt));
  }
}

// ------------------------------------------------------------------------------------------
// Generic kernel for fp32 operands: element strides for both, fp32 MFMA 32x32x2, 64x64x64 tiles.
// ------------------------------------------------------------------------------------------
struct SimpleArgs {
  const void* a; const void* b; void* c; void* pre_act; const void* bias;
  int M, N, K;
  int64_t sam, sak, sbk, sbn, ldc, ldp;
  int act; float param; int bias_dt;
  int round_dt;   // results are rounded to this dtype before they are stored (fp32: as they are)
};

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void gemm_simple_kernel(SimpleArgs g) {
  constexpr int TM = 64, TN = 64, TK = 64;
  constexpr int PER = TM * TK / 256;   // elements of each operand tile per lane
  __shared__ float smem[2][TK][TM + 1];   // A and B tiles; reused by the epilogue
  float (*sa)[TM + 1] = smem[0];
  float (*sb)[TN + 1] = smem[1];
  static_assert(TM == TN, "one array for both tiles");
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

  // the operand tiles are dead (barrier above): 32 x 36 floats of them per wave for the epilogue
  static_assert(4 * 32 * 36 * 4 <= (int)sizeof(smem), "epilogue blocks fit in the tiles");
  wave_tile_epilogue<TO>(acc, &smem[0][0][0] + wave * 32 * 36, g, m0 + wm * 32, n0 + wn * 32);
}

// ------------------------------------------------------------------------------------------
// fp32 operands, outputs too small to give every CU a 64x64 tile (a 512 x 256 layer): 32x32 output
// tiles, four times as many workgroups, and the eight waves of a workgroup share the contraction —
// wave w multiplies k-steps w, w + 8, ... of every k-tile — so the serial chain of MFMAs per wave is
// an eighth as long; the eight accumulators are added through LDS in a fixed order.
// Such a launch lasts a few microseconds, most of them memory latency, so the loads run far ahead:
// a ring of STAGES k-tiles travels in registers (the whole contraction of a 784-wide layer is
// requested before the first multiply), and the LDS tiles are double-buffered, which leaves one
// barrier per k-tile.  Tiles are fetched with 16-byte loads along the contiguous index of each
// operand.
// ------------------------------------------------------------------------------------------
constexpr int kSplitWaves = 8, kSplitThreads = kSplitWaves * 64, kSplitStages = 4;

// output_grad * act'(pre_act) for four elements.  Kept out of line: it is called from every stage
// of an unrolled register ring, and the activation switch inlined at each call site makes a
// kernel of a few microseconds spend them fetching instructions.
__device__ __attribute__((noinline)) float4 pre_act_grad_vec(float4 g, float4 z, int act, float param) {
  return make_float4(g.x * act_derivative(act, z.x, param), g.y * act_derivative(act, z.y, param),
                     g.z * act_derivative(act, z.z, param), g.w * act_derivative(act, z.w, param));
}

// One 32x32 output tile of C = A B.  DZ names an operand that does not exist in memory: the
// gradient of the pre-activation, output_grad * act'(pre_act), formed while its tile is staged
// (DZ = 1: A, DZ = 2: B; `a` / `b` then point at output_grad and `p` at pre_act, both indexed
// alike, row strides lda / ldb and ldp).  COLSUM (with DZ = 2) also sums the columns of the B
// tiles this workgroup passes through LDS, i.e. the bias gradient of its 32 columns.
struct SplitTile {
  const float* a;
  const float* b;
  const float* p;
  int64_t lda, ldb, ldp;
  int M, N, K;     // extents of this product
  int m0, n0;      // origin of the tile
  int act;
  float param;
};

template <int TK>
struct SplitShape {
  static constexpr int kPitchK = TK + 4, kPitchO = 32 + 4;
  static constexpr int kTileFloats = 32 * kPitchK > TK * kPitchO ? 32 * kPitchK : TK * kPitchO;
  static constexpr int kFoldFloats = kSplitWaves * 16 * 64;
  static constexpr int kSmemFloats = 4 * kTileFloats > kFoldFloats ? 4 * kTileFloats : kFoldFloats;
};

// Returns the tile's accumulator (fragment layout of the 32x32 MFMA) in wave 0; the other waves
// return garbage.  On return every wave has passed a barrier after its last use of smem except
// wave 0's reads of the fold area, so wave 0 alone may go on using smem.
template <bool A_MC, bool B_KC, int TK, int DZ, bool COLSUM>
__device__ __forceinline__ f32x16 split_tile(const SplitTile& t, float* smem, float* colsum_out) {
  constexpr int NV = TK * 8 / kSplitThreads;   // 16-byte vectors per lane, operand and k-tile
  static_assert(NV >= 1 && (TK / 2) % kSplitWaves == 0, "k-tile too small for the workgroup");
  static_assert(!COLSUM || (DZ == 2 && !B_KC && TK % 16 == 0), "column sums are taken from a [k][n] tile");
  // LDS image of a tile: as in memory, rows padded by 4 floats (16-byte aligned rows, and the 32
  // lanes of a fragment read spread over the banks): [outer][TK + 4] for an operand whose rows
  // run along the contraction, [k][32 + 4] for the other layout.
  constexpr int kPitchK = SplitShape<TK>::kPitchK, kPitchO = SplitShape<TK>::kPitchO;
  constexpr int kTileFloats = SplitShape<TK>::kTileFloats;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

  // Each lane fetches NV 16-byte vectors per operand and k-tile: 4 consecutive k of one outer index
  // or 4 consecutive outer indices of one k, whichever is contiguous in memory.  Extents along the
  // vectors are multiples of 4 (host check), so a vector is inside or outside as a whole.
  float4 ra[kSplitStages][NV], rb[kSplitStages][NV], rp[DZ ? kSplitStages : 1][NV];
  auto where = [&](bool outer_contig, int idx, int& o, int& k) {
    if (outer_contig) { k = idx >> 3; o = (idx & 7) * 4; } else { o = idx / (TK / 4); k = (idx % (TK / 4)) * 4; }
  };
  auto fetch_one = [&](const float* base, int64_t ld, bool outer_contig, int o0, int o_lim, int k0, int idx) {
    int o, k;
    where(outer_contig, idx, o, k);
    const int go = o0 + o, gk = k0 + k;
    if (go >= o_lim || gk >= t.K) return make_float4(0.f, 0.f, 0.f, 0.f);
    return *reinterpret_cast<const float4*>(base + (outer_contig ? (int64_t)gk * ld + go : (int64_t)go * ld + gk));
  };
  auto fetch = [&](int st, int k0) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      ra[st][i] = fetch_one(t.a, t.lda, A_MC, t.m0, t.M, k0, threadIdx.x + i * kSplitThreads);
      rb[st][i] = fetch_one(t.b, t.ldb, !B_KC, t.n0, t.N, k0, threadIdx.x + i * kSplitThreads);
      if constexpr (DZ == 1) rp[st][i] = fetch_one(t.p, t.ldp, A_MC, t.m0, t.M, k0, threadIdx.x + i * kSplitThreads);
      if constexpr (DZ == 2) rp[st][i] = fetch_one(t.p, t.ldp, !B_KC, t.n0, t.N, k0, threadIdx.x + i * kSplitThreads);
    }
  };
  auto pre_act_grad = [&](const float4& g, const float4& z) {   // zero where the fetch was outside
    if (t.act == AT_ACT_RELU)
      return make_float4(z.x <= 0.f ? 0.f : g.x, z.y <= 0.f ? 0.f : g.y, z.z <= 0.f ? 0.f : g.z, z.w <= 0.f ? 0.f : g.w);
    return pre_act_grad_vec(g, z, t.act, t.param);
  };
  auto stage_one = [&](float* tile, bool outer_contig, const float4& v, int idx) {
    int o, k;
    where(outer_contig, idx, o, k);
    *reinterpret_cast<float4*>(tile + (outer_contig ? k * kPitchO + o : o * kPitchK + k)) = v;
  };
  auto value = [&](const float* tile, bool outer_contig, int o, int k) {
    return tile[outer_contig ? k * kPitchO + o : o * kPitchK + k];
  };

  f32x16 acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0.f;
  float colsum = 0.f;   // COLSUM: column (threadIdx.x & 31), rows (threadIdx.x >> 5) + 16 j of every k-tile
#pragma unroll
  for (int st = 0; st < kSplitStages; ++st)
    if (st * TK < t.K) fetch(st, st * TK);
  // k-tile i sits in register stage i % STAGES and goes through LDS buffer i % 2.  The barrier of
  // tile i is passed only after every wave has finished reading tile i - 1, so writing buffer
  // (i + 1) % 2 after it cannot disturb a reader; one barrier per tile is enough.
  for (int k_ring = 0; k_ring < t.K; k_ring += kSplitStages * TK) {
#pragma unroll
    for (int st = 0; st < kSplitStages; ++st) {
      const int k0 = k_ring + st * TK;
      if (k0 < t.K) {
        float* const sa = smem + (st & 1) * 2 * kTileFloats;
        float* const sb = sa + kTileFloats;
#pragma unroll
        for (int i = 0; i < NV; ++i) {
          if constexpr (DZ == 1) ra[st][i] = pre_act_grad(ra[st][i], rp[st][i]);
          if constexpr (DZ == 2) rb[st][i] = pre_act_grad(rb[st][i], rp[st][i]);
          stage_one(sa, A_MC, ra[st][i], threadIdx.x + i * kSplitThreads);
          stage_one(sb, !B_KC, rb[st][i], threadIdx.x + i * kSplitThreads);
        }
        __syncthreads();
        if (k0 + kSplitStages * TK < t.K) fetch(st, k0 + kSplitStages * TK);
#pragma unroll
        for (int q = 0; q < TK / (2 * kSplitWaves); ++q) {
          const int k = (q * kSplitWaves + wave) * 2 + (lane >> 5);   // k-step q * 8 + wave of this tile
          // operands swapped so that a lane ends up with 4 consecutive n of one m
          acc = __builtin_amdgcn_mfma_f32_32x32x2f32(value(sb, !B_KC, lane & 31, k), value(sa, A_MC, lane & 31, k),
                                                     acc, 0, 0, 0);
        }
        if constexpr (COLSUM) {   // rows beyond K were staged as zeros
#pragma unroll
          for (int j = 0; j < TK / 16; ++j) colsum += sb[((threadIdx.x >> 5) + 16 * j) * kPitchO + (threadIdx.x & 31)];
        }
      }
    }
  }
  __syncthreads();

  // the operand tiles are dead (barrier above): add the partial accumulators in wave order
  float* fold = smem;
#pragma unroll
  for (int r = 0; r < 16; ++r) fold[(r * kSplitWaves + wave) * 64 + lane] = acc[r];
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      float sum = fold[(r * kSplitWaves) * 64 + lane];
#pragma unroll
      for (int w = 1; w < kSplitWaves; ++w) sum += fold[(r * kSplitWaves + w) * 64 + lane];
      acc[r] = sum;
    }
  }
  if constexpr (COLSUM) {
    // 16 row slices per column, added in slice order by the first 32 lanes of wave 1 (wave 0 is
    // busy with the tile); the slices go through LDS behind the fold area's last reader
    __syncthreads();
    float* slices = smem;   // [16][32]
    slices[(threadIdx.x >> 5) * 32 + (threadIdx.x & 31)] = colsum;
    __syncthreads();
    if (wave == 1 && lane < 32) {
      float sum = slices[lane];
#pragma unroll
      for (int j = 1; j < 16; ++j) sum += slices[j * 32 + lane];
      *colsum_out = sum;
    }
    __syncthreads();
  }
  return acc;
}

template <bool A_MC, bool B_KC, int TK>
__global__ __launch_bounds__(kSplitThreads) void gemm_f32_split_kernel(GemmArgs g) {
  __shared__ __align__(16) float smem[SplitShape<TK>::kSmemFloats];
  const int nbn = (g.N + 31) / 32;
  // g.partial (weight-gradient layout only: both operands stored [k][row]): workgroup row y of
  // the grid contracts k-tiles [y * kt_per_split, (y + 1) * kt_per_split) and leaves its tile in
  // partial[y] for gemm_split_finish_kernel
  const int k_begin = g.partial ? (int)blockIdx.y * g.kt_per_split * TK : 0;
  const int k_len = g.partial ? (g.K - k_begin < g.kt_per_split * TK ? g.K - k_begin : g.kt_per_split * TK) : g.K;
  const SplitTile t{reinterpret_cast<const float*>(g.a) + (int64_t)k_begin * g.lda,
                    reinterpret_cast<const float*>(g.b) + (int64_t)k_begin * g.ldb, nullptr,
                    g.lda, g.ldb, 0, g.M, g.N, k_len, (int)(blockIdx.x / nbn) * 32, (int)(blockIdx.x % nbn) * 32,
                    AT_ACT_NONE, 0.f};
  const f32x16 acc = split_tile<A_MC, B_KC, TK, 0, false>(t, smem, nullptr);
  if (threadIdx.x >= 64) return;
  __builtin_amdgcn_wave_barrier();
  static_assert(32 * 36 <= SplitShape<TK>::kFoldFloats, "the epilogue block fits");
  if (g.partial) {
    GemmArgs to_partial = g;
    to_partial.c = g.partial + (int64_t)blockIdx.y * g.M * g.ldw;
    to_partial.ldc = g.ldw;
    wave_tile_epilogue<float>(acc, smem, to_partial, t.m0, t.n0);
  } else {
    wave_tile_epilogue<float>(acc, smem, g, t.m0, t.n0);
  }
}

// Slices of the batch for a small fp32 weight gradient (few 32x32 tiles, a long contraction):
// enough to give every CU two workgroups, each slice at least 8 k-tiles of 128 long.  1 = none.
inline int dw_split_count_f32(int64_t M, int64_t N, int64_t K) {
  const int64_t tiles = cdiv64(M, 32) * cdiv64(N, 32);
  const int64_t want = (int64_t)device_cu_count() * 2 / tiles;
  const int64_t kt = K / 128;
  int64_t splits = want < kt / 8 ? want : kt / 8;
  if (splits > 64) splits = 64;
  if (splits < 2) return 1;
  const int64_t per = cdiv64(cdiv64(K, 128), splits);
  return (int)cdiv64(cdiv64(K, 128), per);   // no empty slice
}

// Backward pass of a small fp32 linear layer with an activation in one launch: the first
// dx_tiles workgroups compute tiles of dX = dZ W^T, the others tiles of dW = X^T dZ, and the
// dW workgroups of the first row block also write the bias gradient (column sums of dZ).
// dZ = output_grad * act'(pre_act) is never stored: every workgroup forms the part it needs
// while staging its tiles.  The contraction runs over out_feat for dX (k-tiles of TKX) and over
// the batch for dW (k-tiles of TKW).
struct SmallBwdArgs {
  const float* output_grad;   // [batch, out_feat]
  const float* pre_act;       // [batch, out_feat]
  const float* input;         // [batch, in_feat]
  const float* weight;        // [in_feat, out_feat]
  float* input_grad;          // [batch, in_feat]
  float* weight_grad;         // [in_feat, out_feat]
  float* bias_grad;           // [out_feat] or null
  int batch, in_feat, out_feat;
  int64_t ld_g, ld_p, ld_x, ld_w, ld_dx, ld_dw;
  int act;
  float param;
  int dx_tiles;
};

template <int TKX, int TKW>
__global__ __launch_bounds__(kSplitThreads) void linear_bwd_small_kernel(SmallBwdArgs s) {
  constexpr int kSmem = SplitShape<TKX>::kSmemFloats > SplitShape<TKW>::kSmemFloats ? SplitShape<TKX>::kSmemFloats
                                                                                      : SplitShape<TKW>::kSmemFloats;
  __shared__ __align__(16) float smem[kSmem];
  GemmArgs g{};   // what the epilogue reads: plain stores of the tile
  g.act = AT_ACT_NONE;
  if ((int)blockIdx.x < s.dx_tiles) {
    // dX[batch, in_feat]: A = dZ (rows along the contraction), B(k, n) = W[n, k] (likewise)
    const int nbn = (s.in_feat + 31) / 32;
    const SplitTile t{s.output_grad, s.weight, s.pre_act, s.ld_g, s.ld_w, s.ld_p, s.batch, s.in_feat, s.out_feat,
                      (int)(blockIdx.x / nbn) * 32, (int)(blockIdx.x % nbn) * 32, s.act, s.param};
    const f32x16 acc = split_tile<false, true, TKX, 1, false>(t, smem, nullptr);
    if (threadIdx.x >= 64) return;
    __builtin_amdgcn_wave_barrier();
    g.c = s.input_grad; g.M = s.batch; g.N = s.in_feat; g.ldc = s.ld_dx;
    wave_tile_epilogue<float>(acc, smem, g, t.m0, t.n0);
  } else {
    // dW[in_feat, out_feat]: A(m, k) = X[k, m], B = dZ[k, n], contraction over the batch
    const int tile = (int)blockIdx.x - s.dx_tiles;
    const int nbn = (s.out_feat + 31) / 32;
    const SplitTile t{s.input, s.output_grad, s.pre_act, s.ld_x, s.ld_g, s.ld_p, s.in_feat, s.out_feat, s.batch,
                      (tile / nbn) * 32, (tile % nbn) * 32, s.act, s.param};
    f32x16 acc;
    if (t.m0 == 0 && s.bias_grad) {
      float column = 0.f;
      acc = split_tile<true, false, TKW, 2, true>(t, smem, &column);
      const int lane = threadIdx.x & 63;
      if ((threadIdx.x >> 6) == 1 && lane < 32 && t.n0 + lane < s.out_feat) s.bias_grad[t.n0 + lane] = column;
    } else {
      acc = split_tile<true, false, TKW, 2, false>(t, smem, nullptr);
    }
    if (threadIdx.x >= 64) return;
    __builtin_amdgcn_wave_barrier();
    g.c = s.weight_grad; g.M = s.in_feat; g.N = s.out_feat; g.ldc = s.ld_dw;
    wave_tile_epilogue<float>(acc, smem, g, t.m0, t.n0);
  }
}

// ------------------------------------------------------------------------------------------
// Generic kernel for 16-bit operands: any strides and extents, 32x32x16 MFMA, tiles of
// (32 WM) x (32 WN) x 64 staged through registers into LDS rows that are contiguous along the
// contraction index.  Each operand is fetched with 16-byte loads when its unit-stride dimension
// allows it and element by element otherwise.
// ------------------------------------------------------------------------------------------
constexpr int kSmallPitch = 72;   // 16-bit elements per LDS row: 64 k + 8 of padding (144 bytes)

template <typename T, int R>
struct SmallTile {   // R outer rows (m or n) x 64 k of one operand
  static constexpr int NV = R / 32, NS = R / 4;
  const T* p;
  int64_t ld;        // stride of the dimension that is not contiguous
  int o0, o_lim, K;
  bool outer_fast;   // the outer index (m or n) is the contiguous one
  bool vec;
  uint4 v[NV];
  unsigned short s[NS];

  __device__ __forceinline__ void where_vec(int idx, int& o, int& k) const {
    if (outer_fast) {
      // a wave takes 16 k x 4 vectors of 8 outer indices: 64 contiguous bytes per k-row on the
      // memory side, and LDS writes that spread over the banks (lanes of one k-row would all
      // fall on two banks)
      const int lane = idx & 63, blk = idx >> 6;
      o = ((blk % (R / 32)) * 4 + (lane >> 4)) * 8;
      k = (blk / (R / 32)) * 16 + (lane & 15);
    } else {
      o = idx >> 3;
      k = (idx & 7) * 8;
    }
  }
  __device__ __forceinline__ void where_one(int e, int& o, int& k) const {
    if (outer_fast) { o = e % R; k = e / R; } else { o = e >> 6; k = e & 63; }
  }
  __device__ __forceinline__ int64_t at(int go, int gk) const {
    return outer_fast ? (int64_t)gk * ld + go : (int64_t)go * ld + gk;
  }
  __device__ __forceinline__ void fetch(int k0) {
    if (vec) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        int o, k;
        where_vec(threadIdx.x + i * 256, o, k);
        const int go = o0 + o, gk = k0 + k;
        // the extent along the vector is a multiple of 8, so a vector is inside or outside as a whole
        v[i] = (go < o_lim && gk < K) ? *reinterpret_cast<const uint4*>(p + at(go, gk)) : make_uint4(0, 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        int o, k;
        where_one(threadIdx.x + i * 256, o, k);
        const int go = o0 + o, gk = k0 + k;
        s[i] = (go < o_lim && gk < K) ? __builtin_bit_cast(unsigned short, p[at(go, gk)]) : (unsigned short)0;
      }
    }
  }
  __device__ __forceinline__ void stage(unsigned short* lds) const {
    if (vec) {
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        int o, k;
        where_vec(threadIdx.x + i * 256, o, k);
        if (!outer_fast) {
          *reinterpret_cast<uint4*>(lds + o * kSmallPitch + k) = v[i];
        } else {
          const uint32_t w[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
#pragma unroll
          for (int j = 0; j < 8; ++j)
            lds[(o + j) * kSmallPitch + k] = (unsigned short)((j & 1) ? w[j >> 1] >> 16 : w[j >> 1] & 0xffffu);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < NS; ++i) {
        int o, k;
        where_one(threadIdx.x + i * 256, o, k);
        lds[o * kSmallPitch + k] = s[i];
      }
    }
  }
};

// KSPLIT: the four waves share one 32x32 output tile and each multiplies a quarter of every
// k-tile; their accumulators are added through LDS at the end.  Four times the workgroups of the
// 64x64 arrangement, for outputs too small to occupy the GPU otherwise (a 10-class head).
template <typename T, typename TO, int WM, int WN, bool KSPLIT = false>
__global__ __launch_bounds__(256) void gemm_small16_kernel(SimpleArgs g) {
  static_assert(KSPLIT ? (WM == 1 && WN == 1) : WM * WN == 4, "four waves");
  constexpr int TM = WM * 32, TN = WN * 32, TK = 64;
  constexpr int kTileShorts = (TM + TN) * kSmallPitch;
  constexpr int kFoldShorts = KSPLIT ? 4 * 64 * 16 * 2 : 0;   // four waves x 16 fp32 registers per lane
  // A and B tiles; reused by the epilogue
  __shared__ __align__(16) unsigned short smem[kTileShorts > kFoldShorts ? kTileShorts : kFoldShorts];
  unsigned short* const sa = smem;
  unsigned short* const sb = smem + TM * kSmallPitch;
  const T* A = reinterpret_cast<const T*>(g.a);
  const T* B = reinterpret_cast<const T*>(g.b);
  const int nbn = (g.N + TN - 1) / TN;
  const int m0 = (blockIdx.x / nbn) * TM, n0 = (blockIdx.x % nbn) * TN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = KSPLIT ? 0 : wave / WN, wn = KSPLIT ? 0 : wave % WN;

  SmallTile<T, TM> ta;
  ta.p = A; ta.o0 = m0; ta.o_lim = g.M; ta.K = g.K;
  ta.outer_fast = g.sak != 1;
  ta.ld = ta.outer_fast ? g.sak : g.sam;
  ta.vec = (ta.ld & 7) == 0 && aligned16_dev(A) && (((ta.outer_fast ? g.M : g.K) & 7) == 0);
  SmallTile<T, TN> tb;
  tb.p = B; tb.o0 = n0; tb.o_lim = g.N; tb.K = g.K;
  tb.outer_fast = g.sbk != 1;
  tb.ld = tb.outer_fast ? g.sbk : g.sbn;
  tb.vec = (tb.ld & 7) == 0 && aligned16_dev(B) && (((tb.outer_fast ? g.N : g.K) & 7) == 0);

  f32x16 acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0.f;
  ta.fetch(0);
  tb.fetch(0);
  for (int k0 = 0; k0 < g.K; k0 += TK) {
    ta.stage(sa);
    tb.stage(sb);
    __syncthreads();
    if (k0 + TK < g.K) {   // the next k-tile travels while this one is multiplied
      ta.fetch(k0 + TK);
      tb.fetch(k0 + TK);
    }
#pragma unroll
    for (int ks = 0; ks < TK / 16; ++ks) {
      if (KSPLIT && ks != wave) continue;
      const int k = ks * 16 + (lane >> 5) * 8;
      const uint4 xa = *reinterpret_cast<const uint4*>(sa + (wm * 32 + (lane & 31)) * kSmallPitch + k);
      const uint4 xb = *reinterpret_cast<const uint4*>(sb + (wn * 32 + (lane & 31)) * kSmallPitch + k);
      // B first: a lane ends up with 4 consecutive n of one m
      acc = Mfma16<T>::run(xb, xa, acc);
    }
    __syncthreads();
  }

  // the operand tiles are dead (barrier above)
  if (KSPLIT) {
    float* fold = reinterpret_cast<float*>(smem);
#pragma unroll
    for (int r = 0; r < 16; ++r) fold[(r * 4 + wave) * 64 + lane] = acc[r];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int r = 0; r < 16; ++r)
      acc[r] = (fold[(r * 4 + 0) * 64 + lane] + fold[(r * 4 + 1) * 64 + lane]) +
               (fold[(r * 4 + 2) * 64 + lane] + fold[(r * 4 + 3) * 64 + lane]);
    __builtin_amdgcn_wave_barrier();
  }
  // 32 x 36 floats of the tiles per wave for the epilogue
  static_assert((KSPLIT ? 1 : 4) * 32 * 36 * 4 <= (int)sizeof(smem), "epilogue blocks fit in the tiles");
  wave_tile_epilogue<TO>(acc, reinterpret_cast<float*>(smem) + wave * 32 * 36, g, m0 + wm * 32, n0 + wn * 32);
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
    if (VEC_OK) {
      // all loads of the row block first, none inside a branch: a row past the slice reads the last
      // row of the slice again (its values are not used), so no load waits for another
      constexpr int ND = (int)sizeof(TDY) * VEC / 16, NZ = (int)sizeof(TZ) * VEC / 16;   // 16-byte vectors per row
      uint4 rd[ROWS][ND], rz[ROWS][NZ];
#pragma unroll
      for (int u = 0; u < ROWS; ++u) {
        const int64_t r = rb + u < r1 ? rb + u : r1 - 1;
#pragma unroll
        for (int q = 0; q < ND; ++q) rd[u][q] = reinterpret_cast<const uint4*>(dy + r * dys + c)[q];
#pragma unroll
        for (int q = 0; q < NZ; ++q) rz[u][q] = reinterpret_cast<const uint4*>(z + r * zs + c)[q];
      }
#pragma unroll
      for (int u = 0; u < ROWS; ++u) {
        union { uint4 raw[ND]; TDY e[VEC]; } ud;
        union { uint4 raw[NZ]; TZ e[VEC]; } uz;
#pragma unroll
        for (int q = 0; q < ND; ++q) ud.raw[q] = rd[u][q];
#pragma unroll
        for (int q = 0; q < NZ; ++q) uz.raw[q] = rz[u][q];
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          d[u][j] = to_f32(ud.e[j]);
          zz[u][j] = to_f32(uz.e[j]);
        }
      }
    } else {
#pragma unroll
      for (int u = 0; u < ROWS; ++u) {
        const int64_t r = rb + u;
        if (r < r1) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            const bool ok = c + j < N;
            d[u][j] = ok ? to_f32(dy[r * dys + c + j]) : 0.f;
            zz[u][j] = ok ? to_f32(z[r * zs + c + j]) : 0.f;
          }
        }
      }
    }
    // the derivative's formula is chosen once per row block, not once per element
    auto derive = [&](auto act_c) {
      constexpr int ACT = decltype(act_c)::value;
#pragma unroll
      for (int u = 0; u < ROWS; ++u)
#pragma unroll
        for (int j = 0; j < VEC; ++j) zz[u][j] = act_derivative(ACT, zz[u][j], param);
    };
    AT_ACT_DISPATCH(act, derive(std::integral_constant<int, ACT>()));
#pragma unroll
    for (int u = 0; u < ROWS; ++u) {
      const int64_t r = rb + u;
      if (r < r1) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          d[u][j] = to_f32(from_f32<TZ>(d[u][j] * zz[u][j]));  // summed as stored
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

// The same pass for whole 16-byte vectors, shaped for bandwidth: a workgroup is 32 column lanes (8
// columns each) times 8 row lanes of kActTileRows / 8 rows each, i.e. one tile of 32 rows x 256
// columns per step, and as a rule one step per workgroup (grid = (N / 256, row slices of 32
// rows)).  Many short-lived workgroups keep more bytes in flight than few long-lived ones: in a
// loop the next loads queue behind the acknowledgement of the wave's own stores.  The column
// sums of the 8 row lanes are folded through LDS in a fixed order.
constexpr int kActTileRows = 32, kActTileCols = 256;
template <typename TDY, typename TZ>
__global__ __launch_bounds__(256) void act_bwd_tile_kernel(
    const TDY* __restrict__ dy, const TZ* __restrict__ z, TZ* __restrict__ dz, float* __restrict__ part,
    int64_t M, int N, int64_t dys, int64_t zs, int64_t dzs, int act, float param, int64_t rows_per_slice) {
  constexpr int VEC = 8, ROWS = kActTileRows / 8;
  constexpr int ND = (int)sizeof(TDY) * VEC / 16, NZ = (int)sizeof(TZ) * VEC / 16;   // 16-byte vectors per row
  __shared__ float fold[8][32][VEC + 1];
  const int cx = threadIdx.x & 31, ry = threadIdx.x >> 5;
  const int c = (blockIdx.x * 32 + cx) * VEC;
  const bool in_cols = c < N;
  const int cc = in_cols ? c : 0;   // lanes past the last column work on column 0 and drop the result
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_slice;
  const int64_t r1 = r0 + rows_per_slice < M ? r0 + rows_per_slice : M;
  float sum[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) sum[j] = 0.f;
  for (int64_t rb = r0 + ry * ROWS; rb < r1; rb += kActTileRows) {
    uint4 rd[ROWS][ND], rz[ROWS][NZ];
#pragma unroll
    for (int u = 0; u < ROWS; ++u) {
      const int64_t r = rb + u < r1 ? rb + u : r1 - 1;   // past the slice: its last row again, not used
#pragma unroll
      for (int q = 0; q < ND; ++q) rd[u][q] = reinterpret_cast<const uint4*>(dy + r * dys + cc)[q];
#pragma unroll
      for (int q = 0; q < NZ; ++q) rz[u][q] = reinterpret_cast<const uint4*>(z + r * zs + cc)[q];
    }
    float d[ROWS][VEC], zz[ROWS][VEC];
#pragma unroll
    for (int u = 0; u < ROWS; ++u) {
      union { uint4 raw[ND]; TDY e[VEC]; } ud;
      union { uint4 raw[NZ]; TZ e[VEC]; } uz;
#pragma unroll
      for (int q = 0; q < ND; ++q) ud.raw[q] = rd[u][q];
#pragma unroll
      for (int q = 0; q < NZ; ++q) uz.raw[q] = rz[u][q];
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        d[u][j] = to_f32(ud.e[j]);
        zz[u][j] = to_f32(uz.e[j]);
      }
    }
    auto derive = [&](auto act_c) {
      constexpr int ACT = decltype(act_c)::value;
#pragma unroll
      for (int u = 0; u < ROWS; ++u)
#pragma unroll
        for (int j = 0; j < VEC; ++j) zz[u][j] = act_derivative(ACT, zz[u][j], param);
    };
    AT_ACT_DISPATCH(act, derive(std::integral_constant<int, ACT>()));
#pragma unroll
    for (int u = 0; u < ROWS; ++u) {
      const int64_t r = rb + u;
      if (r < r1 && in_cols) {
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          d[u][j] = to_f32(from_f32<TZ>(d[u][j] * zz[u][j]));  // summed as stored
          sum[j] += d[u][j];
        }
        store_f32<TZ, VEC>(dz + r * dzs + c, d[u]);
      }
    }
  }
  if (part) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) fold[ry][cx][j] = sum[j];
    __syncthreads();
    // lane (cx, j') sums column cx * 8 + j' over the 8 row lanes, always in the same order
    const int col = threadIdx.x;   // 0 .. 255: column of the tile
    const int fx = col >> 3, fj = col & 7;
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < 8; ++k) t += fold[k][fx][fj];
    const int64_t gc = (int64_t)blockIdx.x * kActTileCols + col;
    if (gc < N) part[(int64_t)blockIdx.y * N + gc] = t;
  }
}

// Column sums of a [M, N] matrix: partial[slice, n] over a slice of rows, then a fixed-order
// reduction.  A workgroup is CT column lanes (8 columns each, one 16-byte load per row) times
// 256 / CT row lanes that stride the rows of the slice; the row lanes are folded through LDS in
// a fixed order.  grid = (ceil(N / (8 CT)), slices).
template <typename T, bool VEC_OK>
__global__ __launch_bounds__(256) void colsum_partial_kernel(const T* __restrict__ x, float* __restrict__ part,
                                                            int64_t M, int N, int64_t xs, int64_t rows_per_slice,
                                                            int ct_log2) {
  constexpr int VEC = 8;
  __shared__ float sm[256 * VEC];
  const int CT = 1 << ct_log2, RT = 256 >> ct_log2;
  const int cx = threadIdx.x & (CT - 1), ry = threadIdx.x >> ct_log2;
  const int c = (blockIdx.x * CT + cx) * VEC;
  const int64_t r0 = (int64_t)blockIdx.y * rows_per_slice;
  const int64_t r1 = r0 + rows_per_slice < M ? r0 + rows_per_slice : M;
  float s[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) s[j] = 0.f;
  if (c < N) {
    auto add_row = [&](int64_t r) {
      const T* p = x + r * xs + c;
      float v[VEC];
      if (VEC_OK) {
        load_f32<T, VEC>(p, v);
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) v[j] = c + j < N ? to_f32(p[j]) : 0.f;
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) s[j] += v[j];
    };
    int64_t r = r0 + ry;
    for (; r + 3 * RT < r1; r += 4 * RT) {   // four independent loads in flight
      add_row(r);
      add_row(r + RT);
      add_row(r + 2 * RT);
      add_row(r + 3 * RT);
    }
    for (; r < r1; r += RT) add_row(r);
  }
#pragma unroll
  for (int j = 0; j < VEC; ++j) sm[(ry * CT + cx) * VEC + j] = s[j];
  __syncthreads();
  if (ry == 0 && c < N) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      float t = 0.f;
      for (int q = 0; q < RT; ++q) t += sm[(q * CT + cx) * VEC + j];
      if (c + j < N) part[(int64_t)blockIdx.y * N + c + j] = t;
    }
  }
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

// Tile choice for a problem the 16-bit kernels can address.  One workgroup of the 256x256
// kernel occupies a CU, so its time goes in whole rounds of one tile per CU; the 128x128 kernel
// runs two workgroups per CU, a full round of 512 tiles taking about 0.7 of a round of 256 large
// ones (measured over fourteen layer shapes, 0.65-0.74).  Its rounds are whole too — a last round
// costs a round even when few tiles are left — unless that last round has at most one workgroup
// per CU, which then has the CU to itself (0.6 of a round).
inline bool prefer_mid_tiles(int64_t M, int64_t N) {
  const int64_t cus = device_cu_count();
  const double big = (double)cdiv64(cdiv64(M, BM) * cdiv64(N, BN), cus);
  const int64_t tiles = cdiv64(M, MT) * cdiv64(N, MT);
  const int64_t full = tiles / (2 * cus), rest = tiles - full * 2 * cus;
  const double mid = 0.7 * ((double)full + (rest == 0 ? 0.0 : rest <= cus ? 0.6 : 1.0));
  return mid < big;
}

// Number of splits of the contraction for the weight gradient (a [in, out] tile grid that is
// small next to the chip, a long contraction over the batch): enough to give every CU two
// workgroups, each split at least 4 k-tiles long.  1 = no split.
inline int dw_split_count(int64_t M, int64_t N, int64_t K) {
  const int64_t tiles = cdiv64(M, MT) * cdiv64(N, MT);
  const int64_t want = (int64_t)device_cu_count() * 2 / tiles;
  const int64_t kt = cdiv64(K, BK);
  int64_t splits = want < kt / 4 ? want : kt / 4;
  if (splits > 32) splits = 32;
  if (splits < 2) return 1;
  const int64_t per = cdiv64(kt, splits);
  return (int)cdiv64(kt, per);   // no empty split
}

inline int64_t dw_partial_pitch(int64_t N) { return (N + 7) / 8 * 8; }

// C[M,N] = A(m,k) B(k,n) for the three products of the linear layer.
//   kFwd: A = [M,K] rows,  B = [K,N] rows          (X, W)
//   kDx : A = [M,K] rows,  B = [N,K] rows          (dZ, W: contraction over W's columns)
//   kDw : A = [K,M] rows,  B = [K,N] rows          (X, dZ: contraction over rows of both)
int run_gemm(Layout layout, const void* a, const void* b, void* c, void* pre_act, const void* bias, int64_t M,
             int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc, int64_t ldp, int act, float param,
             int in_dt, int bias_dt, int out_dt, hipStream_t stream, void* workspace = nullptr,
             int64_t workspace_bytes = 0) {
  if (!a || !b || !c) return AT_ERR_NULL;
  if (!dtype_valid(in_dt) || !dtype_valid(out_dt) || (bias && !dtype_valid(bias_dt))) return AT_ERR_DTYPE;
  if (!act_valid(act)) return AT_ERR_ACT;
  if (M < 0 || N <= 0 || K <= 0 || M > INT32_MAX || N > INT32_MAX || K > INT32_MAX) return AT_ERR_DIM;
  const int64_t a_min = layout == kDw ? M : K, b_min = layout == kDx ? K : N;
  if (lda < a_min || ldb < b_min || ldc < N || (pre_act && ldp < N)) return AT_ERR_DIM;
  if (M == 0) return AT_OK;

  const bool a_contig_k = layout != kDw, b_contig_k = layout == kDx;
  // A backward product of 16-bit operands may be asked for in fp32: the value rounded to the operand
  // dtype, widened (what the 16-bit product followed by autograd's cast to an fp32 leaf gives).
  const bool wide = layout != kFwd && in_dt != AT_DTYPE_F32 && out_dt == AT_DTYPE_F32;
  // 16-byte loads need aligned rows; an operand whose rows run along the contraction index also
  // needs K in whole vectors (the other layout reads whole rows of k, and what a vector picks up
  // past M or N only reaches outputs that are not stored).
  bool fast = in_dt != AT_DTYPE_F32 && (out_dt == in_dt || wide) && aligned16(a) && aligned16(b) && (lda % 8) == 0 &&
              (ldb % 8) == 0;
  if (a_contig_k || b_contig_k) fast = fast && (K % 8) == 0;
  // buffer descriptors address each operand with 32-bit byte offsets below 2 GiB
  const int64_t a_bytes = (a_contig_k ? M : K) * lda * 2, b_bytes = (b_contig_k ? N : K) * ldb * 2;
  if (a_bytes >= ((int64_t)1 << 31) || b_bytes >= ((int64_t)1 << 31)) fast = false;
  // Small problems do not fill the tiles of these kernels; the generic kernel has finer ones.
  if (M * N < (int64_t)MT * MT || M < 64 || N < 64) fast = false;

  const int64_t big_tiles = cdiv64(M, BM) * cdiv64(N, BN);
  if (fast && prefer_mid_tiles(M, N)) {
    GemmArgs g{a, b, c, pre_act, bias, (int)M, (int)N, (int)K, lda, ldb, ldc, ldp, act, param, bias_dt, nullptr, 0, 0, AT_DTYPE_F32};
    const unsigned grid = (unsigned)(cdiv64(M, MT) * cdiv64(N, MT));
    int splits = 1;
    if (layout == kDw && workspace) {
      splits = dw_split_count(M, N, K);
      if (workspace_bytes < (int64_t)splits * M * dw_partial_pitch(N) * 4) splits = 1;
    }
    const bool two_groups = splits == 1 && (int64_t)grid <= device_cu_count() && cdiv64(K, BK) >= 4;
    return dispatch_dtype(in_dt, [&](auto* tp) -> int {
      typedef std::remove_pointer_t<decltype(tp)> T;
      if constexpr (std::is_same<T, float>::value) {
        return AT_ERR_DTYPE;
      } else {
        if (splits > 1) {
          g.partial = (float*)workspace;
          g.kt_per_split = (int)cdiv64(cdiv64(K, BK), splits);
          g.ldw = (int)dw_partial_pitch(N);
          hipLaunchKernelGGL((gemm_mid16_kernel<T, true, false, true>), dim3(grid, splits), dim3(kGemmThreads), 0,
                             stream, g);
          const int64_t items = M * (g.ldw / 8);
          if (wide)
            hipLaunchKernelGGL((gemm_split_finish_kernel<T, float>), dim3((unsigned)cdiv64(items, 256)), dim3(256), 0,
                               stream, (const float*)workspace, (float*)c, (int)M, (int)N, g.ldw, ldc, splits);
          else
            hipLaunchKernelGGL((gemm_split_finish_kernel<T>), dim3((unsigned)cdiv64(items, 256)), dim3(256), 0, stream,
                               (const float*)workspace, (T*)c, (int)M, (int)N, g.ldw, ldc, splits);
        } else if (two_groups) {
          // at most one tile per CU: eight waves per tile, two k-groups (see the kernel)
#define AT_MID2(AMC, BKC, TOUT) \
  hipLaunchKernelGGL((gemm_mid16_kernel<T, AMC, BKC, false, TOUT, 2>), dim3(grid), dim3(2 * kGemmThreads), 0, stream, g)
          if (layout == kDx) { if (wide) AT_MID2(false, true, float); else AT_MID2(false, true, T); }
          else if (layout == kDw) { if (wide) AT_MID2(true, false, float); else AT_MID2(true, false, T); }
          else AT_MID2(false, false, T);
#undef AT_MID2
        } else if (layout == kDx) {
          if (wide) hipLaunchKernelGGL((gemm_mid16_kernel<T, false, true, false, float>), dim3(grid), dim3(kGemmThreads), 0, stream, g);
          else hipLaunchKernelGGL((gemm_mid16_kernel<T, false, true, false>), dim3(grid), dim3(kGemmThreads), 0, stream, g);
        } else if (layout == kDw) {
          if (wide) hipLaunchKernelGGL((gemm_mid16_kernel<T, true, false, false, float>), dim3(grid), dim3(kGemmThreads), 0, stream, g);
          else hipLaunchKernelGGL((gemm_mid16_kernel<T, true, false, false>), dim3(grid), dim3(kGemmThreads), 0, stream, g);
        } else {
          hipLaunchKernelGGL((gemm_mid16_kernel<T, false, false, false>), dim3(grid), dim3(kGemmThreads), 0, stream, g);
        }
        return launch_status();
      }
    });
  }

  if (fast) {
    GemmArgs g{a, b, c, pre_act, bias, (int)M, (int)N, (int)K, lda, ldb, ldc, ldp, act, param, bias_dt, nullptr, 0, 0, AT_DTYPE_F32};
    // one workgroup per CU at a time (LDS): a grid of that many walks the tiles itself
    const int64_t resident = (int64_t)device_cu_count() / 8 * 8;
    const unsigned grid = (unsigned)(big_tiles > resident && resident > 0 ? resident : big_tiles);
    return dispatch_dtype(in_dt, [&](auto* tp) -> int {
      typedef std::remove_pointer_t<decltype(tp)> T;
      if constexpr (std::is_same<T, float>::value) {
        return AT_ERR_DTYPE;
      } else {
        if (layout == kDx) {
          if (wide) hipLaunchKernelGGL((gemm_mfma16_kernel<T, false, true, AT_ACT_NONE, float>), dim3(grid), dim3(kBigThreads), 0, stream, g);
          else hipLaunchKernelGGL((gemm_mfma16_kernel<T, false, true, AT_ACT_NONE>), dim3(grid), dim3(kBigThreads), 0, stream, g);
        } else if (layout == kDw) {
          if (wide) hipLaunchKernelGGL((gemm_mfma16_kernel<T, true, false, AT_ACT_NONE, float>), dim3(grid), dim3(kBigThreads), 0, stream, g);
          else hipLaunchKernelGGL((gemm_mfma16_kernel<T, true, false, AT_ACT_NONE>), dim3(grid), dim3(kBigThreads), 0, stream, g);
        } else {
          switch (act) {
#define AT_FWD_CASE(ID) case ID: hipLaunchKernelGGL((gemm_mfma16_kernel<T, false, false, ID>), dim3(grid), dim3(kBigThreads), 0, stream, g); break;
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

  // Classifier heads (at most 16 output features) on the vector ALUs.
  if (layout == kFwd && N <= kSkinnyCols && skinny_rows_ok(a, K, lda, in_dt)) {
    SkinnyArgs sk{a, b, nullptr, c, pre_act, bias, bias_dt, (int)M, (int)N, (int)K, lda, ldb, 0, ldc, ldp, act, param, 0};
    return dispatch_dtype(in_dt, [&](auto* ti) -> int {
      typedef std::remove_pointer_t<decltype(ti)> TI;
      return dispatch_dtype(out_dt, [&](auto* to) -> int {
        typedef std::remove_pointer_t<decltype(to)> TO;
        hipLaunchKernelGGL((skinny_fwd_kernel<TI, TO>), dim3((unsigned)cdiv64(M, kSkinnyRowsFwd)), dim3(256), 0, stream, sk);
        return launch_status();
      });
    });
  }
  if (layout == kDx && K <= kSkinnyCols && in_dt == out_dt && skinny_rows_ok(c, N, ldc, out_dt)) {
    // dX[M, N] = dZ[M, K] W[N, K]^T with the narrow dimension contracted
    SkinnyArgs sk{nullptr, b, a, c, nullptr, nullptr, 0, (int)M, (int)K, (int)N, 0, ldb, lda, ldc, 0, AT_ACT_NONE, 0.f, 0};
    return dispatch_dtype(in_dt, [&](auto* tp) -> int {
      typedef std::remove_pointer_t<decltype(tp)> T;
      hipLaunchKernelGGL((skinny_dx_kernel<T>), dim3((unsigned)cdiv64(M, kSkinnyRowsDx)), dim3(256), 0, stream, sk);
      return launch_status();
    });
  }
  if (layout == kDw && N <= kSkinnyCols && in_dt == out_dt && skinny_rows_ok(a, M, lda, in_dt) && workspace &&
      workspace_bytes >= skinny_dw_workspace_bytes(K, M)) {
    // dW[M, N] = X[K, M]^T dZ[K, N]: the batch (K here) is cut into slices of rows
    const int64_t rows_per_slice = skinny_rows_per_slice(K);
    const int slices = (int)cdiv64(K, rows_per_slice);
    SkinnyArgs sk{a, nullptr, b, workspace, nullptr, nullptr, 0, (int)K, (int)N, (int)M, lda, 0, ldb, 0, 0,
                  AT_ACT_NONE, 0.f, (int)rows_per_slice};
    return dispatch_dtype(in_dt, [&](auto* tp) -> int {
      typedef std::remove_pointer_t<decltype(tp)> T;
      constexpr int VEC = 16 / (int)sizeof(T);
      hipLaunchKernelGGL((skinny_dw_kernel<T>), dim3((unsigned)cdiv64(M, 64 * VEC), (unsigned)slices), dim3(256), 0,
                         stream, sk);
      const int64_t items = M * (kSkinnyCols / 8);
      hipLaunchKernelGGL((gemm_split_finish_kernel<T>), dim3((unsigned)cdiv64(items, 256)), dim3(256), 0, stream,
                         (const float*)workspace, (T*)c, (int)M, (int)N, kSkinnyCols, ldc, slices);
      return launch_status();
    });
  }

  // fp32 tensors whose rows allow 16-byte loads: the tiled fp32 MFMA kernel
  if (in_dt == AT_DTYPE_F32 && out_dt == AT_DTYPE_F32 && aligned16(a) && aligned16(b) && (lda % 4) == 0 &&
      (ldb % 4) == 0 && (!(a_contig_k || b_contig_k) || (K % 4) == 0) && M >= 32 && N >= 32 &&
      (a_contig_k ? M : K) * lda * 4 < ((int64_t)1 << 31) && (b_contig_k ? N : K) * ldb * 4 < ((int64_t)1 << 31)) {
    GemmArgs g{a, b, c, pre_act, bias, (int)M, (int)N, (int)K, lda, ldb, ldc, ldp, act, param, bias_dt, nullptr, 0, 0, AT_DTYPE_F32};
    // outputs with fewer 64x64 tiles than CUs: 32x32 tiles, the contraction shared by the waves
    if (cdiv64(M, 64) * cdiv64(N, 64) < device_cu_count() && K >= 128 && (M % 4) == 0 && (N % 4) == 0) {
      const unsigned grid = (unsigned)(cdiv64(M, 32) * cdiv64(N, 32));
      if (layout == kDw && workspace && K >= 512) {
        const int splits = dw_split_count_f32(M, N, K);
        const int64_t pitch = dw_partial_pitch(N);
        if (splits > 1 && workspace_bytes >= (int64_t)splits * M * pitch * 4) {
          g.partial = (float*)workspace;
          g.kt_per_split = (int)cdiv64(cdiv64(K, 128), splits);
          g.ldw = (int)pitch;
          hipLaunchKernelGGL((gemm_f32_split_kernel<true, false, 128>), dim3(grid, (unsigned)splits), dim3(kSplitThreads),
                             0, stream, g);
          const int64_t items = M * (pitch / 8);
          hipLaunchKernelGGL((gemm_split_finish_kernel<float>), dim3((unsigned)cdiv64(items, 256)), dim3(256), 0, stream,
                             (const float*)workspace, (float*)c, (int)M, (int)N, (int)pitch, ldc, splits);
          return launch_status();
        }
      }
#define AT_SPLIT_LAUNCH(TK)                                                                                              \
  {                                                                                                                      \
    if (layout == kDx)                                                                                                   \
      hipLaunchKernelGGL((gemm_f32_split_kernel<false, true, TK>), dim3(grid), dim3(kSplitThreads), 0, stream, g);       \
    else if (layout == kDw)                                                                                              \
      hipLaunchKernelGGL((gemm_f32_split_kernel<true, false, TK>), dim3(grid), dim3(kSplitThreads), 0, stream, g);       \
    else                                                                                                                 \
      hipLaunchKernelGGL((gemm_f32_split_kernel<false, false, TK>), dim3(grid), dim3(kSplitThreads), 0, stream, g);      \
  }
      if (K >= 512) AT_SPLIT_LAUNCH(128) else AT_SPLIT_LAUNCH(64)
#undef AT_SPLIT_LAUNCH
      return launch_status();
    }
    // 128x128 tiles once they give every CU a workgroup, 64x64 tiles below that
    const bool big = cdiv64(M, 128) * cdiv64(N, 128) >= device_cu_count();
    const unsigned grid = (unsigned)(big ? cdiv64(M, 128) * cdiv64(N, 128) : cdiv64(M, 64) * cdiv64(N, 64));
#define AT_F32_LAUNCH(WT)                                                                                     \
  {                                                                                                           \
    if (layout == kDx) hipLaunchKernelGGL((gemm_f32_kernel<WT, false, true>), dim3(grid), dim3(256), 0, stream, g);       \
    else if (layout == kDw) hipLaunchKernelGGL((gemm_f32_kernel<WT, true, false>), dim3(grid), dim3(256), 0, stream, g);  \
    else hipLaunchKernelGGL((gemm_f32_kernel<WT, false, false>), dim3(grid), dim3(256), 0, stream, g);                    \
  }
    if (big) AT_F32_LAUNCH(2) else AT_F32_LAUNCH(1)
#undef AT_F32_LAUNCH
    return launch_status();
  }

  SimpleArgs s{a, b, c, pre_act, bias, (int)M, (int)N, (int)K,
               a_contig_k ? lda : 1, a_contig_k ? 1 : lda, b_contig_k ? 1 : ldb, b_contig_k ? ldb : 1,
               ldc, ldp, act, param, bias_dt, wide ? in_dt : AT_DTYPE_F32};
  return dispatch_dtype(in_dt, [&](auto* ti) -> int {
    typedef std::remove_pointer_t<decltype(ti)> TI;
    return dispatch_dtype(out_dt, [&](auto* to) -> int {
      typedef std::remove_pointer_t<decltype(to)> TO;
      if constexpr (std::is_same<TI, float>::value) {
        const unsigned grid = (unsigned)(cdiv64(M, 64) * cdiv64(N, 64));
        hipLaunchKernelGGL((gemm_simple_kernel<TI, TO>), dim3(grid), dim3(256), 0, stream, s);
      } else {
        // skinny outputs put all four waves along m; outputs that leave most CUs without a
        // workgroup split the contraction over the waves instead (four times the workgroups)
        const int64_t blocks = N <= 32 ? cdiv64(M, 128) * cdiv64(N, 32) : cdiv64(M, 64) * cdiv64(N, 64);
        if (blocks * 2 <= device_cu_count() && K >= 256) {
          const unsigned grid = (unsigned)(cdiv64(M, 32) * cdiv64(N, 32));
          hipLaunchKernelGGL((gemm_small16_kernel<TI, TO, 1, 1, true>), dim3(grid), dim3(256), 0, stream, s);
        } else if (N <= 32) {
          hipLaunchKernelGGL((gemm_small16_kernel<TI, TO, 4, 1>), dim3((unsigned)blocks), dim3(256), 0, stream, s);
        } else {
          hipLaunchKernelGGL((gemm_small16_kernel<TI, TO, 2, 2>), dim3((unsigned)blocks), dim3(256), 0, stream, s);
        }
      }
      return launch_status();
    });
  });
}

constexpr int kColsumSlices = 256;   // at most; fewer when the columns alone fill the GPU
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

int at_linear_bwd_wide_output_supported(int64_t batch, int64_t in_feat, int64_t out_feat, int dtype) {
  if (dtype != AT_DTYPE_F16 && dtype != AT_DTYPE_BF16) return 0;
  // the conditions under which run_gemm takes a tiled 16-bit kernel for dX = dZ W^T and dW = X^T dZ
  // when every row stride equals the row's extent
  if ((in_feat % 8) || (out_feat % 8)) return 0;
  if (batch < 64 || in_feat < 64 || out_feat < 64) return 0;
  if (batch * in_feat < (int64_t)MT * MT || in_feat * out_feat < (int64_t)MT * MT) return 0;
  const int64_t limit = (int64_t)1 << 31;
  if (batch * out_feat * 2 >= limit || in_feat * out_feat * 2 >= limit || batch * in_feat * 2 >= limit) return 0;
  return 1;
}

int at_linear_bwd_small_supported(int64_t batch, int64_t in_feat, int64_t out_feat, int dtype) {
  if (dtype != AT_DTYPE_F32) return 0;
  if (batch < 128 || in_feat < 32 || out_feat < 128) return 0;          // contractions of at least two k-tiles
  if ((in_feat % 4) || (out_feat % 4)) return 0;                         // 16-byte vectors along the features
  // small enough that neither product gives every CU a 64x64 tile (the same bound as the
  // single products use for the 32x32 tiles)
  const int64_t cus = device_cu_count();
  if (cdiv64(batch, 64) * cdiv64(in_feat, 64) >= cus || cdiv64(in_feat, 64) * cdiv64(out_feat, 64) >= cus) return 0;
  return 1;
}

int at_linear_bwd_small(const void* output_grad, const void* pre_act, const void* input, const void* weight,
                        void* input_grad, void* weight_grad, void* bias_grad, int64_t batch, int64_t in_feat,
                        int64_t out_feat, int64_t output_grad_stride, int64_t pre_act_stride, int64_t input_stride,
                        int64_t weight_stride, int64_t input_grad_stride, int64_t weight_grad_stride, int act,
                        float param, int dtype, at_stream_t stream) {
  if (!output_grad || !input || !weight || !weight_grad) return AT_ERR_NULL;   // input_grad is optional
  if (!act_valid(act)) return AT_ERR_ACT;
  if (act != AT_ACT_NONE && !pre_act) return AT_ERR_NULL;
  if (!at_linear_bwd_small_supported(batch, in_feat, out_feat, dtype)) return AT_ERR_UNSUPPORTED;
  if (output_grad_stride < out_feat || (pre_act && pre_act_stride < out_feat) || input_stride < in_feat ||
      weight_stride < out_feat || (input_grad && input_grad_stride < in_feat) || weight_grad_stride < out_feat)
    return AT_ERR_DIM;
  const int64_t strides[] = {output_grad_stride, pre_act ? pre_act_stride : 0, input_stride, weight_stride};
  for (int64_t st : strides)
    if (st % 4) return AT_ERR_ALIGN;
  if (!aligned16(output_grad) || (pre_act && !aligned16(pre_act)) || !aligned16(input) || !aligned16(weight))
    return AT_ERR_ALIGN;
  const int64_t limit = (int64_t)1 << 31;
  if (batch * output_grad_stride * 4 >= limit || batch * input_stride * 4 >= limit || in_feat * weight_stride * 4 >= limit)
    return AT_ERR_UNSUPPORTED;
  SmallBwdArgs s{};
  s.output_grad = (const float*)output_grad;
  // without an activation the derivative is 1 whatever it is evaluated at: any readable tensor of
  // the gradient's shape serves as the second stream
  s.pre_act = pre_act ? (const float*)pre_act : (const float*)output_grad;
  s.input = (const float*)input;
  s.weight = (const float*)weight;
  s.input_grad = (float*)input_grad;
  s.weight_grad = (float*)weight_grad;
  s.bias_grad = (float*)bias_grad;
  s.batch = (int)batch; s.in_feat = (int)in_feat; s.out_feat = (int)out_feat;
  s.ld_g = output_grad_stride; s.ld_p = pre_act ? pre_act_stride : output_grad_stride;
  s.ld_x = input_stride; s.ld_w = weight_stride; s.ld_dx = input_grad_stride; s.ld_dw = weight_grad_stride;
  s.act = act; s.param = param;
  s.dx_tiles = input_grad ? (int)(cdiv64(batch, 32) * cdiv64(in_feat, 32)) : 0;
  const unsigned grid = (unsigned)(s.dx_tiles + cdiv64(in_feat, 32) * cdiv64(out_feat, 32));
  // k-tiles of 128 for contractions of 512 and more, 64 below (the ring holds four of them)
  const bool long_x = out_feat >= 512, long_w = batch >= 512;
  hipStream_t hs = (hipStream_t)stream;
  if (long_x && long_w) hipLaunchKernelGGL((linear_bwd_small_kernel<128, 128>), dim3(grid), dim3(kSplitThreads), 0, hs, s);
  else if (long_x) hipLaunchKernelGGL((linear_bwd_small_kernel<128, 64>), dim3(grid), dim3(kSplitThreads), 0, hs, s);
  else if (long_w) hipLaunchKernelGGL((linear_bwd_small_kernel<64, 128>), dim3(grid), dim3(kSplitThreads), 0, hs, s);
  else hipLaunchKernelGGL((linear_bwd_small_kernel<64, 64>), dim3(grid), dim3(kSplitThreads), 0, hs, s);
  return launch_status();
}

int64_t at_linear_bwd_weight_workspace_bytes(int64_t batch, int64_t in_feat, int64_t out_feat, int dtype) {
  if (batch <= 0 || in_feat <= 0 || out_feat <= 0 || !dtype_valid(dtype)) return 0;
  if (out_feat <= kSkinnyCols) return skinny_dw_workspace_bytes(batch, in_feat);
  if (dtype == AT_DTYPE_F32) {
    // the condition under which run_gemm takes the 32x32-tile kernel, and its slices of the batch
    if (cdiv64(in_feat, 64) * cdiv64(out_feat, 64) >= device_cu_count() || batch < 512 || in_feat % 4 || out_feat % 4 ||
        in_feat < 32 || out_feat < 32)
      return 0;
    const int splits = dw_split_count_f32(in_feat, out_feat, batch);
    return splits > 1 ? (int64_t)splits * in_feat * dw_partial_pitch(out_feat) * 4 : 0;
  }
  if (dtype != AT_DTYPE_F16 && dtype != AT_DTYPE_BF16) return 0;
  if (in_feat < 64 || out_feat < 64 || in_feat * out_feat < (int64_t)MT * MT) return 0;
  if (!prefer_mid_tiles(in_feat, out_feat)) return 0;
  const int splits = dw_split_count(in_feat, out_feat, batch);
  return splits > 1 ? (int64_t)splits * in_feat * dw_partial_pitch(out_feat) * 4 : 0;
}

int at_linear_bwd_weight(const void* input, const void* pre_act_grad, void* weight_grad, void* workspace,
                         int64_t workspace_bytes, int64_t batch, int64_t in_feat, int64_t out_feat,
                         int64_t input_stride, int64_t grad_stride, int64_t weight_grad_stride, int in_dtype,
                         int out_dtype, at_stream_t stream) {
  if (batch <= 0) return AT_ERR_DIM;
  return run_gemm(kDw, input, pre_act_grad, weight_grad, nullptr, nullptr, in_feat, out_feat, batch,
                  input_stride, grad_stride, weight_grad_stride, 0, AT_ACT_NONE, 0.f, in_dtype, 0, out_dtype,
                  (hipStream_t)stream, workspace, workspace_bytes);
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
  float* part = bias_grad ? (float*)workspace : nullptr;
  if (vec_ok) {
    // tiles of 32 rows x 256 columns, one per workgroup unless the partial buffer would outgrow
    // its slices (then a workgroup walks down several tiles)
    const unsigned gx = (unsigned)cdiv64(cols, kActTileCols);
    int64_t slices = cdiv64(rows, kActTileRows);
    const int64_t max_slices = bias_grad ? kActBwdMaxSlices : 65535;
    if (slices > max_slices) slices = max_slices;
    int64_t rows_per_slice = cdiv64(cdiv64(rows, slices), kActTileRows) * kActTileRows;
    slices = cdiv64(rows, rows_per_slice);
    int rc = dispatch_dtype(grad_dtype, [&](auto* tg) -> int {
      typedef std::remove_pointer_t<decltype(tg)> TG;
      return dispatch_dtype(input_dtype, [&](auto* tz) -> int {
        typedef std::remove_pointer_t<decltype(tz)> TZ;
        hipLaunchKernelGGL((act_bwd_tile_kernel<TG, TZ>), dim3(gx, (unsigned)slices), dim3(256), 0,
                           (hipStream_t)stream, (const TG*)output_grad, (const TZ*)input, (TZ*)input_grad, part, rows,
                           (int)cols, output_grad_stride, input_stride, input_grad_stride, act, param, rows_per_slice);
        return launch_status();
      });
    });
    if (rc || !bias_grad) return rc;
    hipLaunchKernelGGL(colsum_final_kernel, dim3((unsigned)cdiv64(cols, kColsumFinalCols)), dim3(256), 0,
                       (hipStream_t)stream, (const float*)workspace, bias_grad, bias_grad_dtype, (int)slices, (int)cols);
    return launch_status();
  }
  // enough workgroups to fill the chip, few enough row slices to keep the partial buffer small
  const unsigned gx = (unsigned)cdiv64(cols, 256 * 8);
  int64_t slices = cdiv64((int64_t)device_cu_count() * 16, gx);
  if (slices > kActBwdMaxSlices) slices = kActBwdMaxSlices;
  if (slices > rows) slices = rows;
  const int64_t rows_per_slice = cdiv64(rows, slices);
  slices = cdiv64(rows, rows_per_slice);
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
  // column lanes: enough for the columns, at most a whole workgroup; slices: about 1024 workgroups
  int ct_log2 = 0;
  while (ct_log2 < 8 && ((int64_t)8 << ct_log2) < cols) ++ct_log2;
  const unsigned gx = (unsigned)cdiv64(cols, (int64_t)8 << ct_log2);
  int64_t want = cdiv64(1024, gx);
  if (want < 16) want = 16;
  if (want > kColsumSlices) want = kColsumSlices;
  int slices = (int)(rows < want ? rows : want);
  const int64_t rows_per_slice = cdiv64(rows, slices);
  slices = (int)cdiv64(rows, rows_per_slice);
  const bool vec_ok = cols % 8 == 0 && x_stride % 8 == 0 && aligned16(x);
  int rc = dispatch_dtype(x_dtype, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    if (vec_ok)
      hipLaunchKernelGGL((colsum_partial_kernel<T, true>), dim3(gx, slices), dim3(256), 0, (hipStream_t)stream,
                         (const T*)x, (float*)workspace, rows, (int)cols, x_stride, rows_per_slice, ct_log2);
    else
      hipLaunchKernelGGL((colsum_partial_kernel<T, false>), dim3(gx, slices), dim3(256), 0, (hipStream_t)stream,
                         (const T*)x, (float*)workspace, rows, (int)cols, x_stride, rows_per_slice, ct_log2);
    return launch_status();
  });
  if (rc) return rc;
  hipLaunchKernelGGL(colsum_final_kernel, dim3((unsigned)cdiv64(cols, kColsumFinalCols)), dim3(256), 0,
                     (hipStream_t)stream, (const float*)workspace, out, out_dtype, slices, (int)cols);
  return launch_status();
}

}  // extern "C"
