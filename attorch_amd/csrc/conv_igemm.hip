// Implicit-GEMM convolution kernels for 16-bit tensors on v_mfma_f32_32x32x16 (see conv_igemm.h).
//
//   forward / input gradient (conv_igemm_kernel):
//     out[(n,oh,ow), co] = sum over taps (kh,kw) and channels c of
//                          act[n, oh*s+kh-p, ow*s+kw-p, c] * wt[co, (kh,kw), c]
//     GEMM rows are output pixels, columns output channels, the contraction runs tap-major and
//     channel-minor; a k-tile of 64 is 64 channels of one tap, so an operand row of the
//     activations is 128 contiguous bytes of a channels-last pixel (or zeros outside the image).
//     128 x 64 x 64 tiles, 4 waves, operand tiles straight from global memory into LDS, double
//     buffered; the finished tile is transposed through LDS and leaves as NCHW rows.
//     The input gradient is the same product over dY with the taps mirrored and the roles of
//     the channel counts exchanged (stride 1).
//   weight gradient (conv_dw_kernel):
//     dW[co, (kh,kw), c] = sum over pixels of dY[pixel, co] * X[pixel shifted by the tap, c]
//     Both operands have the contraction index (the pixel) as their row index: they are kept
//     in LDS as loaded and transposed by the fragment reads (ds_read_b64_tr_b16).  The pixel
//     range is split over workgroups; fp32 partial tiles are summed in fixed order afterwards.
#include "conv_igemm.h"

#include <type_traits>

#include "at_mfma.h"

namespace at_hip {
namespace {

// q = n / d for 0 <= n < 2^31 with one multiply-high and a shift.
struct FastDiv {
  uint32_t mul;
  int shift;   // < 0: d == 1
  uint32_t d;
};

inline FastDiv make_fastdiv(int64_t d) {
  FastDiv f;
  f.d = (uint32_t)d;
  if (d <= 1) {
    f.mul = 0;
    f.shift = -1;
    return f;
  }
  int l = 0;
  while (((int64_t)1 << l) < d) ++l;
  const unsigned __int128 num = (unsigned __int128)1 << (31 + l);
  f.mul = (uint32_t)((num + (unsigned __int128)d - 1) / (unsigned __int128)d);
  f.shift = l - 1;
  return f;
}

__device__ __forceinline__ int fast_div(int n, const FastDiv& f) {
  return f.shift < 0 ? n : (int)(__umulhi((uint32_t)n, f.mul) >> f.shift);
}

// ------------------------------------------------------------------------------------------
// Layout changes.
// ------------------------------------------------------------------------------------------
// [N][C][HW] -> [N][HW'][C'] through a 64 x 64 LDS tile; 128-bit accesses on both sides when the
// shapes allow (vec_in: HW % 8 == 0 and aligned source; the target rows are 16-byte aligned by
// construction when vec_out is set).  The target may be wider than the source in two ways:
//  * channels: every group of Cg source channels becomes Cgp >= Cg target channels (Cgp a
//    multiple of 64 when it differs from Cg), the extra ones zero — the products below contract
//    over whole 64-channel tiles;
//  * pixels: source pixel (h, w) of a row of W lands at ((h * sh) * Wd + w * sw); the pixels in
//    between are not written (the caller clears the target first when sh * sw > 1) — the input
//    gradient of a strided layer is a stride-1 product over the gradient spread out like this.
struct LayoutCopyArgs {
  int C, HW;          // source channels and pixels per image
  int Cg, Cgp;        // channels per group in the source and in the target
  int W, Wd, sh, sw;  // source row length, target row length, pixel spreading
  int HWd;            // target pixels per image
  int vec_in, vec_out;
};

template <typename T>
__global__ __launch_bounds__(256) void nchw_to_nhwc_kernel(const T* __restrict__ src, T* __restrict__ dst,
                                                            LayoutCopyArgs a) {
  __shared__ uint32_t tile[64][33];   // [channel][pixel pair], padded
  const int n = blockIdx.z;
  const int p0 = blockIdx.x * 64;
  // blockIdx.y counts 64-channel tiles of the target; without padding groups play no role
  const bool padded = a.Cgp != a.Cg;
  const int tiles_per_group = padded ? a.Cgp / 64 : 1;
  const int grp = padded ? (int)blockIdx.y / tiles_per_group : 0;
  const int in_group0 = padded ? ((int)blockIdx.y % tiles_per_group) * 64 : (int)blockIdx.y * 64;
  const int src_c0 = grp * a.Cg + in_group0;                    // first source channel of the tile
  const int src_c_end = padded ? grp * a.Cg + a.Cg : a.C;       // one past the last valid one
  const int dst_c0 = blockIdx.y * 64;
  const int Cd = padded ? (a.C / a.Cg) * a.Cgp : a.C;           // target channels
  const T* s = src + (int64_t)n * a.C * a.HW;
  T* d = dst + (int64_t)n * a.HWd * Cd;
  const int t = threadIdx.x;
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int cl = pass * 32 + (t >> 3), pv = (t & 7) * 8;
    const int c = src_c0 + cl, p = p0 + pv;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (c < src_c_end) {
      const T* q = s + (int64_t)c * a.HW + p;
      if (a.vec_in && p + 8 <= a.HW) {
        v = *reinterpret_cast<const uint4*>(q);
      } else {
        union { uint4 raw; T e[8]; } u;
        u.raw = v;
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (p + e < a.HW) u.e[e] = q[e];
        v = u.raw;
      }
    }
    tile[cl][pv / 2 + 0] = v.x;
    tile[cl][pv / 2 + 1] = v.y;
    tile[cl][pv / 2 + 2] = v.z;
    tile[cl][pv / 2 + 3] = v.w;
  }
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int pl = pass * 32 + (t >> 3), cv = (t & 7) * 8;
    const int p = p0 + pl, c = dst_c0 + cv;
    if (p >= a.HW || c >= Cd) continue;
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t lo = tile[cv + 2 * e][pl >> 1], hi = tile[cv + 2 * e + 1][pl >> 1];
      const int sft = (pl & 1) * 16;
      w[e] = ((lo >> sft) & 0xffffu) | (((hi >> sft) & 0xffffu) << 16);
    }
    int pd = p;
    if (a.sh != 1 || a.sw != 1) {
      const int h = p / a.W;
      pd = (h * a.sh) * a.Wd + (p - h * a.W) * a.sw;
    }
    T* q = d + (int64_t)pd * Cd + c;
    if (a.vec_out && c + 8 <= Cd) {
      *reinterpret_cast<uint4*>(q) = make_uint4(w[0], w[1], w[2], w[3]);
    } else {
      union { uint32_t raw[4]; T e[8]; } u;
#pragma unroll
      for (int e = 0; e < 4; ++e) u.raw[e] = w[e];
#pragma unroll
      for (int e = 0; e < 8; ++e)
        if (c + e < Cd) q[e] = u.e[e];
    }
  }
}

// Clears `count16` 16-byte units (a kernel, not a memset: the calls may be captured in a HIP graph).
__global__ __launch_bounds__(256) void conv_clear_kernel(uint4* __restrict__ dst, int64_t count16) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < count16; i += stride)
    dst[i] = make_uint4(0, 0, 0, 0);
}

// W[O][Cg][KH][KW] -> wt[rows][taps * colsp]; the columns of a tap are padded with zeros from
// cols to colsp (the contraction channels per group as the products see them):
//   forward  (flip = 0): wt[o][tap][c]              = W[o][c][tap]               (rows O,  cols Cg)
//   dX       (flip = 1): wt[g*Cg + c][tap'][o in g] = W[g*Og + o][c][taps-1-tap'] (rows C, cols Og)
template <typename T>
__global__ void conv_weight_taps_kernel(const T* __restrict__ w, T* __restrict__ wt, int O, int Cg, int Og,
                                        int taps, int flip, int colsp, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int col = (int)(i % colsp);
  const int tap = (int)((i / colsp) % taps);
  const int row = (int)(i / ((int64_t)colsp * taps));
  T v = from_f32<T>(0.f);
  if (!flip) {
    if (col < Cg) v = w[((int64_t)row * Cg + col) * taps + tap];
  } else if (col < Og) {
    const int g = row / Cg, c = row - g * Cg;   // row = g * Cg + c
    v = w[(((int64_t)g * Og + col) * Cg + c) * taps + (taps - 1 - tap)];
  }
  wt[i] = v;
}

// W[O][Cg][KH][KW] -> fragment-major copy of wt (as defined above) for the kernel that reads the
// weights straight into registers: the 64 lanes x 16 bytes of one operand fragment (32 rows x 16 k)
// are contiguous, ordered [group][row tile of 32][k / 16][lane]; rows past Og are zeros.
// k = tap * Cg + c for the forward product (flip = 0); for the input gradient (flip = 1) the roles
// of the channel counts are swapped and the taps mirrored.  Cg = contraction channels per group,
// Cgp = the same padded to what the products contract over (a multiple of 16; channels from Cg on
// are zeros), Og = rows per group.
template <typename T>
__global__ void conv_weight_frags_direct_kernel(const T* __restrict__ w, T* __restrict__ wf, int Cg, int Cgp, int Og,
                                                int taps, int flip, int ntiles, int64_t total_chunks) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total_chunks) return;
  const int lane = (int)(i & 63);
  const int64_t frag = i >> 6;
  const int ksteps = taps * Cgp / 16;
  const int kstep = (int)(frag % ksteps);
  const int tile = (int)((frag / ksteps) % ntiles);
  const int grp = (int)(frag / ((int64_t)ksteps * ntiles));
  const int co = tile * 32 + (lane & 31);
  const int k0 = kstep * 16 + (lane >> 5) * 8;
  const int tap = k0 / Cgp, c = k0 - tap * Cgp;
  union { uint4 raw; T e[8]; } u;
  u.raw = make_uint4(0, 0, 0, 0);
  if (co < Og) {
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (c + e < Cg)
        u.e[e] = flip ? w[(((int64_t)grp * Cg + c + e) * Og + co) * taps + (taps - 1 - tap)]
                      : w[(((int64_t)grp * Og + co) * Cg + c + e) * taps + tap];
  }
  reinterpret_cast<uint4*>(wf)[i] = u.raw;
}

// ------------------------------------------------------------------------------------------
// Forward / input-gradient kernel.
// ------------------------------------------------------------------------------------------
constexpr int CBM = 128, CBN = 64, CBK = 64;
constexpr int kCATile = CBM * 128, kCBTile = CBN * 128, kCStage = kCATile + kCBTile;
constexpr int kCEpiPitch = CBM * 2 + 16;   // bytes per output-channel row of the epilogue tile

struct IgemmArgs {
  const void* act;    // [N][IH][IW][Ctot]
  const void* wt;     // [groups * Og][taps * Cg]
  void* wf;           // fragment-major copy of wt (room for groups * ceil32(Og) * K elements)
  void* out;          // [N][groups * Og][OH][OW]
  const void* bias;   // [groups * Og] or null
  int bias_dt;
  int IH, IW, Ctot, Cg, Og, KW, OW, OHW, sh, sw, ph, pw;
  int M;              // N * OH * OW
  int K;              // taps * Cg
  int KT;             // K / 64
  int tiles_per_tap;  // Cg / 64
  int nbn;            // column tiles per group
  int vec_store;      // 16-byte stores: OHW % 8 == 0 (channels-first) or Og and the channel total % 8 == 0, aligned output
  int out_last;       // the output is channels-last, [N][OH][OW][groups * Og]
  int64_t act_bytes, wt_bytes;
  FastDiv div_ohw, div_ow;
};

// Epilogue of the forward / input-gradient kernels: the 128 x 64 tile goes through LDS (dead after
// the main loop; the caller has synchronised) and leaves in 16-byte pieces.
//   Channels-first output: a lane holds, for tile t and register r, pixel wm*64 + t*32 + (r/4)*8 +
//   (lane/32)*4 + r%4 of output channel wn*32 + lane%32; the tile is laid down as
//   [channel][pixel] and leaves as runs of 8 pixels of one channel (NCHW rows).
//   Channels-last output (MFMA operands the other way round): a lane holds channel wn*32 +
//   (r/4)*8 + (lane/32)*4 + r%4 of pixel wm*64 + t*32 + lane%32; the tile is laid down as
//   [pixel][channel] and leaves as 8 channels of one pixel — consecutive pixels are consecutive
//   rows of groups * Og channels, so no division is needed to place them.
constexpr int kCEpiPitchLast = CBN * 2 + 16;   // bytes per pixel row of the channels-last epilogue tile

// First half: accumulators (+ bias) into the LDS tile, barrier, and this thread's four 16-byte
// pieces back into registers.  `bias_tile`, when given, holds the 64 bias values of the tile's
// channels as floats in LDS (a workgroup that walks over many tiles loads them once).
template <typename T, bool OUT_LAST>
__device__ __forceinline__ void igemm_epilogue_stage(const f32x16 (&acc)[2], char* lds, const IgemmArgs& g, int grp,
                                                     int n0, int wm, int wn, int tid, const float* bias_tile,
                                                     uint4 (&piece)[4]) {
  const int lane = tid & 63;
  if (OUT_LAST) {
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
      const int ch = wn * 32 + rg * 8 + (lane >> 5) * 4;
      float bv4[4] = {0.f, 0.f, 0.f, 0.f};
      if (bias_tile) {
#pragma unroll
        for (int e = 0; e < 4; ++e) bv4[e] = bias_tile[ch + e];
      } else if (g.bias) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n0 + ch + e < g.Og) bv4[e] = load_scalar_f32(g.bias, g.bias_dt, grp * g.Og + n0 + ch + e);
      }
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc[t][rg * 4 + e] + bv4[e];
        const int pix = wm * 64 + t * 32 + (lane & 31);
        store_f32<T, 4>(reinterpret_cast<T*>(lds + pix * kCEpiPitchLast) + ch, v);
      }
    }
    __syncthreads();
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int id = tid + 256 * s;
      const int pix = id >> 3, ch = (id & 7) * 8;
      piece[s] = *reinterpret_cast<const uint4*>(lds + pix * kCEpiPitchLast + ch * 2);
    }
    return;
  }
  const int col = wn * 32 + (lane & 31);
  float bv = 0.f;
  if (bias_tile) bv = bias_tile[col];
  else if (g.bias && n0 + col < g.Og) bv = load_scalar_f32(g.bias, g.bias_dt, grp * g.Og + n0 + col);
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int rg = 0; rg < 4; ++rg) {
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = acc[t][rg * 4 + e] + bv;
      const int pix = wm * 64 + t * 32 + rg * 8 + (lane >> 5) * 4;
      store_f32<T, 4>(reinterpret_cast<T*>(lds + col * kCEpiPitch) + pix, v);
    }
  __syncthreads();
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const int id = tid + 256 * s;
    const int col2 = id >> 4, pc = id & 15;
    piece[s] = *reinterpret_cast<const uint4*>(lds + col2 * kCEpiPitch + pc * 16);
  }
}

// Second half: the four pieces out to memory.
template <typename T, bool OUT_LAST>
__device__ __forceinline__ void igemm_epilogue_store(const uint4 (&piece)[4], const IgemmArgs& g, int grp, int m0,
                                                     int n0, int tid) {
  T* __restrict__ out = reinterpret_cast<T*>(g.out);
  const int Otot = g.Og * (int)gridDim.z;
  if (OUT_LAST) {
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int id = tid + 256 * s;
      const int pix = id >> 3, ch = (id & 7) * 8;
      const int co = n0 + ch, m = m0 + pix;
      if (co >= g.Og || m >= g.M) continue;
      T* dst = out + (int64_t)m * Otot + grp * g.Og + co;
      if (g.vec_store) {
        *reinterpret_cast<uint4*>(dst) = piece[s];
      } else {
        union { uint4 raw; T e[8]; } u;
        u.raw = piece[s];
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (co + e < g.Og) dst[e] = u.e[e];
      }
    }
    return;
  }
#pragma unroll
  for (int s = 0; s < 4; ++s) {
    const int id = tid + 256 * s;
    const int col2 = id >> 4, pc = id & 15;
    const int co = n0 + col2, m = m0 + pc * 8;
    if (co >= g.Og || m >= g.M) continue;
    if (g.vec_store) {
      const int n = fast_div(m, g.div_ohw);
      const int p = m - n * g.OHW;
      *reinterpret_cast<uint4*>(out + ((int64_t)n * Otot + grp * g.Og + co) * g.OHW + p) = piece[s];
    } else {
      union { uint4 raw; T e[8]; } u;
      u.raw = piece[s];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int mm = m + e;
        if (mm < g.M) {
          const int n = fast_div(mm, g.div_ohw);
          const int p = mm - n * g.OHW;
          out[((int64_t)n * Otot + grp * g.Og + co) * g.OHW + p] = u.e[e];
        }
      }
    }
  }
}

template <typename T, bool OUT_LAST>
__device__ __forceinline__ void igemm_epilogue(const f32x16 (&acc)[2], char* lds, const IgemmArgs& g, int grp, int m0,
                                               int n0, int wm, int wn, int tid) {
  uint4 piece[4];
  igemm_epilogue_stage<T, OUT_LAST>(acc, lds, g, grp, n0, wm, wn, tid, nullptr, piece);
  igemm_epilogue_store<T, OUT_LAST>(piece, g, grp, m0, n0, tid);
}

template <typename T, bool OUT_LAST>
__global__ __launch_bounds__(256) void conv_igemm_kernel(IgemmArgs g) {
  __shared__ __attribute__((aligned(1024))) char lds[2 * kCStage];
  const int grp = blockIdx.z;
  const int tile_m = blockIdx.x / g.nbn, tile_n = blockIdx.x - tile_m * g.nbn;
  const int m0 = tile_m * CBM, n0 = tile_n * CBN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // ---- operand loaders: a wave-wide load fills 8 tile rows of 128 bytes ----
  const i32x4 ra = make_buffer_rsrc(g.act, g.act_bytes);
  const i32x4 rb = make_buffer_rsrc(g.wt, g.wt_bytes);
  int a_ih0[4], a_iw0[4], a_base[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = (wave * 4 + i) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row ^ (row >> 3)) & 7);   // the chunk that belongs at this lane's LDS position
    const int m = m0 + row;
    if (m < g.M) {
      const int n = fast_div(m, g.div_ohw);
      const int p = m - n * g.OHW;
      const int oh = fast_div(p, g.div_ow);
      const int ow = p - oh * g.OW;
      a_ih0[i] = oh * g.sh - g.ph;
      a_iw0[i] = ow * g.sw - g.pw;
      // element offset of the lane's chunk at input pixel (0, 0) of image n
      a_base[i] = n * g.IH * g.IW * g.Ctot + grp * g.Cg + chunk * 8;
    } else {
      a_ih0[i] = -(1 << 24);   // never inside the image
      a_iw0[i] = 0;
      a_base[i] = 0;
    }
  }
  int b_off[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = (wave * 2 + i) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row ^ (row >> 3)) & 7);
    const int co = n0 + row;
    b_off[i] = co < g.Og ? ((grp * g.Og + co) * g.K + chunk * 8) * 2 : kOobOffset;
  }

  // k-tile to issue next: tap (kh, kw) and first channel
  int nk_kh = 0, nk_kw = 0, nk_ct = 0, nk = 0;
  auto issue = [&](char* stage) {
    const int cb = nk_ct * 64;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int ih = a_ih0[i] + nk_kh, iw = a_iw0[i] + nk_kw;
      const bool ok = (unsigned)ih < (unsigned)g.IH && (unsigned)iw < (unsigned)g.IW;
      const int off = (a_base[i] + (ih * g.IW + iw) * g.Ctot + cb) * 2;
      lds_dma_16(ra, ok ? off : kOobOffset, stage + (wave * 4 + i) * 1024);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
      lds_dma_16(rb, b_off[i] == kOobOffset ? kOobOffset : b_off[i] + nk * (CBK * 2),
                 stage + kCATile + (wave * 2 + i) * 1024);
    ++nk;
    if (++nk_ct == g.tiles_per_tap) {
      nk_ct = 0;
      if (++nk_kw == g.KW) {
        nk_kw = 0;
        ++nk_kh;
      }
    }
  };

  f32x16 acc[2];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[t][e] = 0.f;

  issue(lds);
  lds_dma_wait_all();
  __syncthreads();
  for (int kt = 0; kt < g.KT; ++kt) {
    const char* cur = lds + (kt & 1) * kCStage;
    char* nxt = lds + ((kt & 1) ^ 1) * kCStage;
    if (kt + 1 < g.KT) issue(nxt);
#pragma unroll
    for (int ks = 0; ks < CBK / 16; ++ks) {
      const uint4 a0 = read_frag_kc(cur, wm * 64, ks);
      const uint4 a1 = read_frag_kc(cur, wm * 64 + 32, ks);
      const uint4 b = read_frag_kc(cur + kCATile, wn * 32, ks);
      // which operand goes first decides what a lane ends up with: four consecutive pixels of
      // one channel (channels-first output) or four consecutive channels of one pixel
      acc[0] = OUT_LAST ? Mfma16<T>::run(b, a0, acc[0]) : Mfma16<T>::run(a0, b, acc[0]);
      acc[1] = OUT_LAST ? Mfma16<T>::run(b, a1, acc[1]) : Mfma16<T>::run(a1, b, acc[1]);
    }
    lds_dma_wait_all();   // this wave's part of the next stage has landed
    __syncthreads();      // ... and everybody else's; the current stage may be overwritten
  }

  igemm_epilogue<T, OUT_LAST>(acc, lds, g, grp, m0, n0, wm, wn, threadIdx.x);
}

// ------------------------------------------------------------------------------------------
// Forward / input-gradient kernel, input window resident in LDS.
// ------------------------------------------------------------------------------------------
// The 128 output pixels of a tile read, over all taps, a contiguous range of channels-last input
// pixels (flattened over image, row, column): tap (kh, kw) of output pixel m sits at
// q(m) + kh*IW + kw with q(m) growing with m.  When that range fits in LDS it is loaded once per
// 64-channel chunk (instead of once per tap), the operand fragments of every tap are read from it
// at shifted rows, and taps outside the image read a row of zeros.  The weights go from cache
// straight into registers, so the main loop needs no barrier.
constexpr int kHaloRows = 288;                       // input pixels a tile may span
constexpr int kHaloBytes = (kHaloRows + 1) * 128;    // + the zero row

template <typename T, bool OUT_LAST>
__global__ __launch_bounds__(256) void conv_igemm_halo_kernel(IgemmArgs g) {
  __shared__ __attribute__((aligned(1024))) char lds[kHaloBytes];
  const int grp = blockIdx.z;
  const int tile_m = blockIdx.x / g.nbn, tile_n = blockIdx.x - tile_m * g.nbn;
  const int m0 = tile_m * CBM, n0 = tile_n * CBN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int KH = g.KT / (g.tiles_per_tap * g.KW);

  // q of (tap 0,0) for an output pixel, and whether the pixel exists
  auto q_of = [&](int m, int& ih0, int& iw0) -> int {
    const int n = fast_div(m, g.div_ohw);
    const int p = m - n * g.OHW;
    const int oh = fast_div(p, g.div_ow);
    const int ow = p - oh * g.OW;
    ih0 = oh * g.sh - g.ph;
    iw0 = ow * g.sw - g.pw;
    return (n * g.IH + ih0) * g.IW + iw0;
  };
  int dummy0, dummy1;
  const int m_last = m0 + CBM - 1 < g.M ? m0 + CBM - 1 : g.M - 1;
  const int q_lo = q_of(m0, dummy0, dummy1);
  const int rows = q_of(m_last, dummy0, dummy1) + (KH - 1) * g.IW + g.KW - q_lo;   // <= kHaloRows (host check)

  // this lane's two fragment rows (output pixels) and its weight row
  int f_ih0[2], f_iw0[2], f_row[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int m = m0 + wm * 64 + t * 32 + (lane & 31);
    if (m < g.M) {
      f_row[t] = q_of(m, f_ih0[t], f_iw0[t]) - q_lo;
    } else {
      f_ih0[t] = -(1 << 24);
      f_iw0[t] = 0;
      f_row[t] = 0;
    }
  }
  // byte offset of this lane inside the first fragment of its channel tile (fragment-major
  // weights: one fragment = 64 lanes x 16 bytes, K / 16 fragments per tile)
  const int ntiles32 = (g.Og + 31) >> 5;
  const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
      g.wf, 0, (int)((int64_t)gridDim.z * ntiles32 * g.K * 64), 0x00020000);
  const int wrow = ((grp * ntiles32 + (n0 >> 5) + wn) * (g.K >> 4)) * 1024 + lane * 16;

  if (threadIdx.x < 32) reinterpret_cast<uint32_t*>(lds + kHaloRows * 128)[threadIdx.x] = 0u;   // the zero row

  const i32x4 ra = make_buffer_rsrc(g.act, g.act_bytes);
  f32x16 acc[2];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[t][e] = 0.f;

  for (int cc = 0; cc < g.tiles_per_tap; ++cc) {
    if (cc > 0) __syncthreads();   // everybody is done with the previous chunk's window
    // Straight-line and unconditional on purpose (offsets first, then the loads back to back; a
    // load past the window writes zeros into unused rows): any wait the compiler inserts for
    // loads it tracks would also wait for the loads issued here, one after the other.
    int doff[kHaloRows / 32];
#pragma unroll
    for (int i = 0; i < kHaloRows / 32; ++i) {
      const int row = (wave + 4 * i) * 8 + (lane >> 3);
      // A fragment read takes 16 consecutive window rows (128 bytes each) starting anywhere: with
      // the chunk index XORed with (row / 2) % 8 those rows occupy the 16 different 16-byte
      // columns of the banks, whatever the first row is.
      const int chunk = (lane & 7) ^ ((row >> 1) & 7);
      const int off = ((q_lo + row) * g.Ctot + grp * g.Cg + cc * 64 + chunk * 8) * 2;   // negative: out of range
      doff[i] = row < rows ? off : kOobOffset;
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < kHaloRows / 32; ++i) lds_dma_16(ra, doff[i], lds + (wave + 4 * i) * 1024);
    lds_dma_wait_all();
    __syncthreads();

    const int wk = wrow + cc * 4096;   // 4 fragments per 64 channels
    const int taps = KH * g.KW;
    // weight fragments of a whole tap (4 k-steps) per buffer; the next tap's are fetched while
    // this tap multiplies
    uint4 b0[4], b1[4];
    // Buffer loads without a branch around them (a missing channel reads zeros; one tap past
    // the end reads values nobody uses): with conditional loads the compiler cannot count what is
    // in flight and waits for the fragments it has just requested.
    // The tap and k-step go into the scalar offset, so the vector offset is one register that
    // never changes: no address arithmetic competes for the registers the loads land in.
    auto fetch = [&](uint4 (&dst)[4], int tap) {
      const int tap_bytes = tap < taps ? tap * g.tiles_per_tap * 4096 : 0;   // one past the end: any valid tap
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
        dst[ks] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rw, wk, tap_bytes + ks * 1024, 0));
    };
    int kh = 0, kw = 0;
    auto multiply = [&](const uint4 (&bw)[4]) {
      int rowaddr[2], swz[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int ih = f_ih0[t] + kh, iw = f_iw0[t] + kw;
        const bool ok = (unsigned)ih < (unsigned)g.IH && (unsigned)iw < (unsigned)g.IW;
        const int row = ok ? f_row[t] + kh * g.IW + kw : kHaloRows;
        rowaddr[t] = row * 128;
        swz[t] = (row >> 1) & 7;
      }
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const int chunk = ks * 2 + (lane >> 5);
        const uint4 a0 = *reinterpret_cast<const uint4*>(lds + rowaddr[0] + ((chunk ^ swz[0]) << 4));
        const uint4 a1 = *reinterpret_cast<const uint4*>(lds + rowaddr[1] + ((chunk ^ swz[1]) << 4));
        acc[0] = OUT_LAST ? Mfma16<T>::run(bw[ks], a0, acc[0]) : Mfma16<T>::run(a0, bw[ks], acc[0]);
        acc[1] = OUT_LAST ? Mfma16<T>::run(bw[ks], a1, acc[1]) : Mfma16<T>::run(a1, bw[ks], acc[1]);
      }
      if (++kw == g.KW) {
        kw = 0;
        ++kh;
      }
    };
    fetch(b0, 0);
#pragma unroll 1
    for (int tap = 0; tap < taps; tap += 2) {
      fetch(b1, tap + 1);
      multiply(b0);
      if (tap + 1 < taps) {
        fetch(b0, tap + 2);
        multiply(b1);
      }
    }
  }
  __syncthreads();   // the window is dead: LDS becomes the output tile
  igemm_epilogue<T, OUT_LAST>(acc, lds, g, grp, m0, n0, wm, wn, threadIdx.x);
}

// ------------------------------------------------------------------------------------------
// Forward / input-gradient kernel, input window in LDS and the weights resident in registers.
// ------------------------------------------------------------------------------------------
// With 64 contraction channels per group and TAPS taps, the weights a wave multiplies by (32
// output channels x K = 64 TAPS) are TAPS * 16 registers per lane: 144 for a 3x3 filter.  A
// workgroup then fetches them once and walks over many tiles of 128 output pixels: the window of
// the next tile travels into the second of two LDS buffers while the current one is multiplied
// (fragments of every tap read at shifted rows, as in the kernel above), and the buffer just
// multiplied from serves as the staging area of the epilogue.  Two workgroups share a CU (two
// waves per SIMD, 256 registers each).  The tiles of the grid are dealt out in eight contiguous
// ranges, one per XCD (workgroup b runs on XCD b % 8), so that the input rows two neighbouring
// tiles share are fetched into one L2 only.
constexpr int kStatWin = (kHaloRows + 1) * 128;    // window + the zero row

template <typename T, bool OUT_LAST, int TAPS>
__global__ __launch_bounds__(256, 2) void conv_igemm_stationary_kernel(IgemmArgs g, int tiles_m) {
  __shared__ __attribute__((aligned(1024))) char lds[2 * kStatWin + CBN * 4];
  float* const bias_tile = reinterpret_cast<float*>(lds + 2 * kStatWin);   // the tile's bias values, if any
  const int grp = blockIdx.z;
  const int n0 = blockIdx.y * CBN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int KH = TAPS / g.KW;

  const int xcd = blockIdx.x & 7, per_xcd = gridDim.x >> 3;   // the grid is a multiple of 8 wide
  const int t_end = (int)(((int64_t)(xcd + 1) * tiles_m) >> 3);
  int tile = (int)(((int64_t)xcd * tiles_m) >> 3) + (blockIdx.x >> 3);
  if (tile >= t_end) return;

  // q of (tap 0,0) for an output pixel
  auto q_of = [&](int m, int& ih0, int& iw0) -> int {
    const int n = fast_div(m, g.div_ohw);
    const int p = m - n * g.OHW;
    const int oh = fast_div(p, g.div_ow);
    const int ow = p - oh * g.OW;
    ih0 = oh * g.sh - g.ph;
    iw0 = ow * g.sw - g.pw;
    return (n * g.IH + ih0) * g.IW + iw0;
  };
  const i32x4 ra = make_buffer_rsrc(g.act, g.act_bytes);
  // Starts the loads of tile t's window into `win` (offsets first, then the loads back to back;
  // rows past the window read zeros).
  auto issue_window = [&](int t, char* win) {
    // the lane's part of the offsets is recomputed per tile on purpose (the empty asm hides that
    // it never changes): kept across the main loop it would take the registers the fragment
    // prefetch needs
    int lane_v = lane;
    asm volatile("" : "+v"(lane_v));
    int d0, d1;
    const int m0 = t * CBM;
    const int m_last = m0 + CBM - 1 < g.M ? m0 + CBM - 1 : g.M - 1;
    const int q_lo = q_of(m0, d0, d1);
    const int rows = q_of(m_last, d0, d1) + (KH - 1) * g.IW + g.KW - q_lo;   // <= kHaloRows (host check)
    int doff[kHaloRows / 32];
#pragma unroll
    for (int i = 0; i < kHaloRows / 32; ++i) {
      const int row = (wave + 4 * i) * 8 + (lane_v >> 3);
      const int chunk = (lane_v & 7) ^ ((row >> 1) & 7);   // as in the kernel above
      const int off = ((q_lo + row) * g.Ctot + grp * g.Cg + chunk * 8) * 2;   // negative: out of range
      doff[i] = row < rows ? off : kOobOffset;
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < kHaloRows / 32; ++i) lds_dma_16(ra, doff[i], win + (wave + 4 * i) * 1024);
  };

  if (threadIdx.x < 64)   // the zero rows of both buffers
    reinterpret_cast<uint32_t*>(lds + (threadIdx.x >> 5) * kStatWin + kHaloRows * 128)[threadIdx.x & 31] = 0u;
  issue_window(tile, lds);
  if (g.bias && threadIdx.x < CBN)
    bias_tile[threadIdx.x] =
        n0 + (int)threadIdx.x < g.Og ? load_scalar_f32(g.bias, g.bias_dt, grp * g.Og + n0 + threadIdx.x) : 0.f;

  // this wave's weights: fragment-major, one fragment = 64 lanes x 16 bytes, K / 16 fragments per
  // tile of 32 output channels
  const int ntiles32 = (g.Og + 31) >> 5;
  const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
      g.wf, 0, (int)((int64_t)gridDim.z * ntiles32 * g.K * 64), 0x00020000);
  const int wrow = ((grp * ntiles32 + (n0 >> 5) + wn) * (g.K >> 4)) * 1024 + lane * 16;
  uint4 wreg[TAPS * 4];
#pragma unroll
  for (int i = 0; i < TAPS * 4; ++i)
    wreg[i] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rw, wrow, i * 1024, 0));

  lds_dma_wait_all();
  __syncthreads();
  // The window of the next tile is always on its way while a tile is worked on: it is requested
  // as soon as the buffer it goes into has been emptied by the epilogue of the tile before, and
  // waited for only after the next epilogue's LDS work, a whole tile later.
  if (tile + per_xcd < t_end) issue_window(tile + per_xcd, lds + kStatWin);
  int buf = 0;
  for (; tile < t_end; tile += per_xcd) {
    char* const win = lds + buf * kStatWin;

    const int m0 = tile * CBM;
    int d0, d1;
    const int q_lo = q_of(m0, d0, d1);
    int f_ih0[2], f_iw0[2], f_row[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int m = m0 + wm * 64 + t * 32 + (lane & 31);
      if (m < g.M) {
        f_row[t] = q_of(m, f_ih0[t], f_iw0[t]) - q_lo;
      } else {
        f_ih0[t] = -(1 << 24);
        f_iw0[t] = 0;
        f_row[t] = 0;
      }
    }
    f32x16 acc[2];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[t][e] = 0.f;

    // Fragment address of k-step 0 of a tap: row * 128 + ((lane / 32) ^ (row / 2)) % 8 * 16; k-step ks
    // sits at that address with ks XORed into bits 5-6 (the chunk swizzle is an XOR as well).
    // The fragments are fetched two k-steps ahead of the MFMAs that use them.
    int kh = 0, kw = 0;
    auto tap_address = [&](int t) -> int {
      const int ih = f_ih0[t] + kh, iw = f_iw0[t] + kw;
      const bool ok = (unsigned)ih < (unsigned)g.IH && (unsigned)iw < (unsigned)g.IW;
      const int row = ok ? f_row[t] + kh * g.IW + kw : kHaloRows;
      return row * 128 + ((((lane >> 5) ^ (row >> 1)) & 7) << 4);
    };
    auto next_tap = [&]() {
      if (++kw == g.KW) {
        kw = 0;
        ++kh;
      }
    };
    constexpr int kSteps = TAPS * 4, kAhead = 2;
    uint4 af[kAhead + 1][2];
    int abase[2] = {tap_address(0), tap_address(1)};
    auto fetch = [&](int step) {
      if (step > 0 && (step & 3) == 0) {
        next_tap();
        abase[0] = tap_address(0);
        abase[1] = tap_address(1);
      }
#pragma unroll
      for (int t = 0; t < 2; ++t)
        af[step % (kAhead + 1)][t] = *reinterpret_cast<const uint4*>(win + (abase[t] ^ ((step & 3) << 5)));
    };
#pragma unroll
    for (int st = 0; st < kAhead; ++st) fetch(st);
#pragma unroll
    for (int st = 0; st < kSteps; ++st) {
      __builtin_amdgcn_sched_barrier(0);   // a k-step's address arithmetic stays in its k-step
      if (st + kAhead < kSteps) fetch(st + kAhead);
      const uint4 bw = wreg[st];
#pragma unroll
      for (int t = 0; t < 2; ++t)
        acc[t] = OUT_LAST ? Mfma16<T>::run(bw, af[st % (kAhead + 1)][t], acc[t])
                          : Mfma16<T>::run(af[st % (kAhead + 1)][t], bw, acc[t]);
    }
    __syncthreads();      // nobody reads the current window any more: it becomes the output tile
    {
      // as for the window offsets: what the epilogue derives from the thread index is recomputed per tile
      int tid = threadIdx.x;
      asm volatile("" : "+v"(tid));
      uint4 piece[4];
      igemm_epilogue_stage<T, OUT_LAST>(acc, win, g, grp, n0, tid >> 7, (tid >> 6) & 1, tid, g.bias ? bias_tile : nullptr,
                                        piece);
      lds_dma_wait_all();   // this wave's part of the next window (requested a tile ago) has landed
      __syncthreads();      // ... and everybody's; the output tile has been read: its buffer is free
      if (tile + 2 * per_xcd < t_end) issue_window(tile + 2 * per_xcd, win);
      igemm_epilogue_store<T, OUT_LAST>(piece, g, grp, m0, n0, tid);
    }
    buf ^= 1;
  }
}

// ------------------------------------------------------------------------------------------
// Forward / input-gradient kernel for channels-last 3x3 layers with stride 1 and padding 1 over 64
// contraction channels: weights resident in registers, image rows in a ring of LDS slots.
// ------------------------------------------------------------------------------------------
// The image is cut into bands of 28 output columns and each band into steps of 8 output rows.  A
// workgroup (4 waves = 2 halves of 64 output channels x 2 groups of 4 rows) walks down a range of
// consecutive steps.  A 32-pixel MFMA operand is a piece of ONE image row (28 columns used), so the
// fragment of input row y, column shift kw serves the taps (0, kw), (1, kw) and (2, kw) of the
// output rows y + 1, y and y - 1: 72 fragment reads feed the 144 MFMAs of a wave and step, half of
// what pixel tiles cut from the flattened image need.  Rows live in 18 slots of 30 pixels x 128
// bytes (band + one neighbour column each side, zeros outside the image by way of out-of-range
// loads): the 10 rows of the step being multiplied and the at most 8 or 9 new ones of the next
// step, requested a whole step ahead; a step keeps the two bottom rows of the step before.  The
// 16-byte chunks of a pixel are XORed with (pixel / 2) % 8, which spreads any 16 consecutive
// pixels over all banks (no bank conflicts measured).  Rows above and below the image are never
// loaded: their fragments are read from 128 bytes of zeros.  Outputs leave straight from the
// accumulators (see the epilogue) as buffer stores with out-of-range offsets for what must not be
// written, always 8 per wave and step: the in-order memory counter then lets the wave wait for its
// row loads (issued before those stores) without waiting for the stores themselves.  One barrier
// per step, no LDS staging of the output.
constexpr int kRingBand = 28;                           // output columns per band
constexpr int kRingCols = kRingBand + 2;                // window columns
constexpr int kRingRow = kRingCols * 128;               // bytes per slot
constexpr int kRingSlots = 18;
constexpr int kRingStep = 8;                            // output rows per step
constexpr int kRingRows = kRingSlots * kRingRow + 4 * 128;   // + what lanes 28..31 read past the last slot
constexpr int kRingZero = kRingRows + CBN * 4;          // 128 bytes of zeros, 128-byte aligned
constexpr int kRingLds = kRingZero + 128;
constexpr int kRingRowChunks = kRingCols * 8;           // 16-byte chunks per slot
constexpr int kRingStores = 8;                          // stores per wave and step

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

struct RingArgs {
  int bands, steps_per_strip, total_steps;
  int64_t out_bytes;
  FastDiv div_steps, div_bands;
};

template <typename T>
__device__ __forceinline__ uint2 pack4(const float (&v)[4]) {
  union { uint2 raw; T e[4]; } u;
#pragma unroll
  for (int e = 0; e < 4; ++e) u.e[e] = from_f32<T>(v[e]);
  return u.raw;
}

template <typename T>
__global__ __launch_bounds__(256, 2) void conv_igemm_ring_kernel(IgemmArgs g, RingArgs ra) {
  __shared__ __attribute__((aligned(1024))) char lds[kRingLds];
  float* const bias_tile = reinterpret_cast<float*>(lds + kRingRows);
  const int grp = blockIdx.z;
  const int n0 = blockIdx.y * CBN;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int wn = wave & 1, wr = wave >> 1;

  // Ranges of steps are cut in an order in which workgroups b and b + grid / 2 are neighbours:
  // those two share a CU (the second half of the grid is placed once every CU has one workgroup,
  // measurably later), and when the steps do not divide evenly the one that starts first gets the
  // longer range.
  const int half = (int)gridDim.x >> 1;   // the grid is even
  const int bx = (int)blockIdx.x;
  const int v = bx < half ? 2 * bx + 1 : 2 * (bx - half);
  int q = (int)(((int64_t)v * ra.total_steps) / (int)gridDim.x);
  const int q_end = (int)(((int64_t)(v + 1) * ra.total_steps) / (int)gridDim.x);
  if (q >= q_end) return;

  auto decode = [&](int qq, int& n, int& b, int& s) {
    const int strip = fast_div(qq, ra.div_steps);
    s = qq - strip * ra.steps_per_strip;
    n = fast_div(strip, ra.div_bands);
    b = strip - n * ra.bands;
  };
  const i32x4 rin = make_buffer_rsrc(g.act, g.act_bytes);

  // Requests the rows step qq needs and the step before it (same strip) does not hold; `fresh`:
  // nothing is held.  Returns the strip's anchor: image row r lives in slot (anchor + r) % 18.
  int next_slot = 0;
  auto issue_rows = [&](int qq, bool fresh, int anchor_prev) -> int {
    int n, b, s;
    decode(qq, n, b, s);
    const int y0 = s * kRingStep;
    const int r_hi = y0 + kRingStep < g.IH ? y0 + kRingStep : g.IH - 1;
    int r_lo, anchor;
    if (fresh || s == 0) {
      r_lo = y0 > 0 ? y0 - 1 : 0;
      anchor = ((next_slot - r_lo) % kRingSlots + kRingSlots) % kRingSlots;
    } else {
      r_lo = y0 + 1;
      anchor = anchor_prev;
    }
    // what a lane fetches of a row: LDS chunk c = 64 j + lane is position c % 8 of window pixel
    // c / 8 and holds the pixel's chunk (c % 8) ^ (pixel / 2) % 8.  Recomputed per call on purpose
    // (the empty asm hides that only the band changes): kept across the main loop it would take
    // registers from it.
    int lane_v = lane;
    asm volatile("" : "+v"(lane_v));
    int loff[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = j * 64 + lane_v;
      const int px = c >> 3, chunk = (c ^ (px >> 1)) & 7;
      const int col = b * kRingBand + px - 1;
      const bool ok = px < kRingCols && (unsigned)col < (unsigned)g.IW;
      loff[j] = ok ? (px - 1) * g.Ctot * 2 + chunk * 16 : kOobOffset;
    }
    for (int r = r_lo + wave; r <= r_hi; r += 4) {
      const int slot = (anchor + r) % kRingSlots;
      const unsigned row_off = (unsigned)((((n * g.IH + r) * g.IW + b * kRingBand) * g.Ctot + grp * g.Cg) * 2);
      char* const dst = lds + slot * kRingRow;
#pragma unroll
      for (int j = 0; j < 3; ++j) lds_dma_16(rin, (int)((unsigned)loff[j] + row_off), dst + j * 1024);
      if (lane_v < kRingRowChunks - 192) lds_dma_16(rin, (int)((unsigned)loff[3] + row_off), dst + 3072);
    }
    if (r_hi >= r_lo) next_slot = (anchor + r_hi + 1) % kRingSlots;
    return anchor;
  };

  int anchor_cur = issue_rows(q, true, 0);
  if (threadIdx.x < 32) reinterpret_cast<uint32_t*>(lds + kRingZero)[threadIdx.x] = 0u;
  if (g.bias && threadIdx.x < CBN)
    bias_tile[threadIdx.x] =
        n0 + (int)threadIdx.x < g.Og ? load_scalar_f32(g.bias, g.bias_dt, grp * g.Og + n0 + threadIdx.x) : 0.f;

  // this wave's weights: fragment-major, 36 fragments of 64 lanes x 16 bytes
  const int ntiles32 = (g.Og + 31) >> 5;
  const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(
      g.wf, 0, (int)((int64_t)gridDim.z * ntiles32 * g.K * 64), 0x00020000);
  const int wrow = ((grp * ntiles32 + (n0 >> 5) + wn) * (g.K >> 4)) * 1024 + lane * 16;
  uint4 wreg[36];
#pragma unroll
  for (int i = 0; i < 36; ++i)
    wreg[i] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rw, wrow, i * 1024, 0));
  const __amdgpu_buffer_rsrc_t rout = __builtin_amdgcn_make_buffer_rsrc(g.out, 0, (int)ra.out_bytes, 0x00020000);
  const int Otot = g.Og * (int)gridDim.z;

  bool first = true;
  for (; q < q_end; ++q) {
    int n, b, s;
    decode(q, n, b, s);
    // the rows of this step were requested before the stores of the step before
    if (first) lds_dma_wait_all();
    else lds_dma_wait_newest<kRingStores>();
    __syncthreads();   // everybody's rows are there; nobody reads the rows of the step before any more
    int anchor_next = anchor_cur;

    const int y = s * kRingStep + wr * 4;   // this wave's first output row
    // fragment address of (input row i, column shift kw, k-step kc): (row_base[i] + t[kw]) ^ (kc << 5);
    // the row bases are wave-uniform and multiples of 128, the XOR only touches bits 5-6.  A row
    // above or below the image reads the 128 zero bytes instead (every lane the same 16).
    int row_base[6], t[3];
    bool inside[6];
    {
      int lane_v = lane;
      asm volatile("" : "+v"(lane_v));
#pragma unroll
      for (int kw = 0; kw < 3; ++kw) {
        const int px = (lane_v & 31) + kw;
        t[kw] = px * 128 + ((((lane_v >> 5) ^ (px >> 1)) & 7) << 4);
      }
#pragma unroll
      for (int i = 0; i < 6; ++i) {
        const int r = y - 1 + i;
        inside[i] = (unsigned)r < (unsigned)g.IH;
        row_base[i] = ((anchor_cur + (inside[i] ? r : 0)) % kRingSlots) * kRingRow;
      }
    }
    f32x16 acc[4];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[r][e] = 0.f;

    // fragment f = (input row i, column shift kw, k-step kc), fetched three fragments ahead
    {
      constexpr int kFrags = 72, kAhead = 3, kSplit = 12;
      uint4 af[kAhead + 1];
      auto fetch = [&](int f) {
        const int i = f / 12, kw = (f % 12) / 4, kc = f % 4;
        const int at = inside[i] ? row_base[i] + t[kw] : kRingZero;
        af[f % (kAhead + 1)] = *reinterpret_cast<const uint4*>(lds + (at ^ (kc << 5)));
      };
#pragma unroll
      for (int f = 0; f < kAhead; ++f) fetch(f);
      auto run = [&](auto from, auto to) {
#pragma unroll
        for (int f = decltype(from)::value; f < decltype(to)::value; ++f) {
          __builtin_amdgcn_sched_barrier(0);
          if (f + kAhead < kFrags) fetch(f + kAhead);
          const int i = f / 12, kw = (f % 12) / 4, kc = f % 4;
          const uint4 a = af[f % (kAhead + 1)];
#pragma unroll
          for (int kh = 0; kh < 3; ++kh) {
            const int r = i - kh;
            if (r < 0 || r > 3) continue;
            // operands this way round: a lane ends up with 4 consecutive channels of one pixel
            acc[r] = Mfma16<T>::run(wreg[(kh * 3 + kw) * 4 + kc], a, acc[r]);
          }
        }
      };
      // the next step's rows are requested behind the first MFMAs, whose run time covers the address
      // arithmetic of the requests
      run(std::integral_constant<int, 0>{}, std::integral_constant<int, kSplit>{});
      __builtin_amdgcn_sched_barrier(0);
      if (q + 1 < q_end) anchor_next = issue_rows(q + 1, false, anchor_cur);
      run(std::integral_constant<int, kSplit>{}, std::integral_constant<int, kFrags>{});
    }

    // ---- outputs ----
    // A lane holds channels rg*8 + (lane/32)*4 .. +3 of pixel lane % 32 of each of its 4 rows.
    // Exchanging the packed values of an even and an odd register group between the two halves
    // of the wave (v_permlane32_swap) leaves lane (pixel, 0) with channels 16 p .. 16 p + 7 and
    // lane (pixel, 1) with 16 p + 8 .. 16 p + 15: 16 bytes per lane, 32 contiguous bytes per pixel
    // and store, without a trip through LDS.
    {
      int lane_v = lane;
      asm volatile("" : "+v"(lane_v));
      const int ch0 = wn * 32 + (lane_v >> 5) * 4;
      float bv[4][4];
#pragma unroll
      for (int rg = 0; rg < 4; ++rg) {
        float4 t4 = make_float4(0.f, 0.f, 0.f, 0.f);
        if (g.bias) t4 = *reinterpret_cast<const float4*>(bias_tile + ch0 + rg * 8);
        bv[rg][0] = t4.x; bv[rg][1] = t4.y; bv[rg][2] = t4.z; bv[rg][3] = t4.w;
      }
      const int x = lane_v & 31, xg = b * kRingBand + x;
      const int chs = wn * 32 + (lane_v >> 5) * 8;   // + 16 p: first of the lane's 8 channels after the exchange
      bool ook[2];
      unsigned ooff[2];
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        ook[p] = x < kRingBand && xg < g.OW && n0 + chs + 16 * p < g.Og;
        ooff[p] = (unsigned)(((n * g.IH) * g.OW + xg) * Otot + grp * g.Og + n0 + chs + 16 * p) * 2u;
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const bool row_ok = y + r < g.IH;
        const unsigned row_off = (unsigned)((y + r) * g.OW * Otot * 2);
#pragma unroll
        for (int p = 0; p < 2; ++p) {
          uint2 part[2];
#pragma unroll
          for (int k = 0; k < 2; ++k) {
            const int rg = 2 * p + k;
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] = acc[r][rg * 4 + e] + bv[rg][e];
            part[k] = pack4<T>(o);
          }
          const auto sx = __builtin_amdgcn_permlane32_swap(part[0].x, part[1].x, false, false);
          const auto sy = __builtin_amdgcn_permlane32_swap(part[0].y, part[1].y, false, false);
          u32x4 d;
          d[0] = sx[0]; d[1] = sy[0]; d[2] = sx[1]; d[3] = sy[1];
          __builtin_amdgcn_raw_buffer_store_b128(d, rout, ook[p] && row_ok ? (int)(ooff[p] + row_off) : kOobOffset, 0, 0);
        }
      }
    }
    anchor_cur = anchor_next;
    first = false;
  }
}

// ------------------------------------------------------------------------------------------
// Weight-gradient kernel.
// ------------------------------------------------------------------------------------------
// Operand tile in LDS: 64 pixel rows x 128 bytes (64 channels) as loaded, the 16-byte chunk
// index XORed with 2 * (row % 4): the four consecutive rows a transposing read touches then
// sit in four different 32-byte bank groups.
__device__ __forceinline__ int dw_chunk_swizzle(int row) { return (row & 3) << 1; }

// Fragment of 32 channels x 16 pixels for one MFMA operand: 8 consecutive pixels per lane.
// ds_read_b64_tr_b16: within 16 lanes, result[l][e] = source[4e + l/4][l%4]; source lane 4e + q
// points at pixel row (k0 + e), channels 4q .. 4q+3, and lane l receives k0 .. k0+3 of channel l.
__device__ __forceinline__ uint4 read_frag_tr(const char* tile, int ch_base, int ks) {
  const int lane = threadIdx.x & 63;
  const int i = lane & 15, gq = lane >> 4;
  const int byte = (ch_base + (gq & 1) * 16 + (i & 3) * 4) * 2;
  const int krow = ks * 16 + (gq >> 1) * 8 + (i >> 2);
  const int krow1 = krow + 4;   // same row % 4: same swizzle
  const int inrow = (((byte >> 4) ^ dw_chunk_swizzle(krow)) << 4) + (byte & 15);
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(tile + krow * 128 + inrow));
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(tile + krow1 * 128 + inrow));
  const uint2 a = __builtin_bit_cast(uint2, lo), b = __builtin_bit_cast(uint2, hi);
  return make_uint4(a.x, a.y, b.x, b.y);
}

constexpr int kDwTile = 64 * 128;        // one operand tile: 64 pixels x 64 channels
constexpr int kDwStage = 2 * kDwTile;

struct DwArgs {
  const void* dy;     // [N*OH*OW][Otot]
  const void* x;      // [N][H][W][Ctot]
  float* part;        // [splits][Otot][taps * Cg]
  int H, W, Ctot, Otot, Cg, Og, KW, OW, OHW, sh, sw, ph, pw;
  int P;              // N * OH * OW
  int K;              // taps * Cg
  int tiles_per_tap;  // Cg / 64
  int nbn;            // column tiles (taps * Cg / 64)
  int mtiles;         // row tiles (Og / 64)
  int splits;         // pixel ranges
  int p_per_split;    // pixels per split, a multiple of 64
  int64_t dy_bytes, x_bytes;
  FastDiv div_ohw, div_ow;
};

template <typename T>
__global__ __launch_bounds__(256) void conv_dw_kernel(DwArgs g) {
  __shared__ __attribute__((aligned(1024))) char lds[2 * kDwStage];
  // Consecutive workgroup ids go to different XCDs (each with its own L2).  The tiles of one
  // pixel range all read the same rows of dY and X, so they are given to one XCD: id -> (XCD,
  // position on it) -> split = XCD + 8 * (position / tiles), tile = position % tiles.
  const int grp = blockIdx.z;
  const int tiles = g.mtiles * g.nbn;
  const int xcd = blockIdx.x & 7, pos = blockIdx.x >> 3;
  const int split = xcd + 8 * (pos / tiles);
  if (split >= g.splits) return;   // padding of the grid, uniform for the workgroup
  const int tile = pos % tiles;
  const int tile_m = tile / g.nbn, tile_n = tile - tile_m * g.nbn;
  const int co0 = tile_m * 64;                               // within the group
  const int tap = tile_n / g.tiles_per_tap;
  const int c0 = (tile_n - tap * g.tiles_per_tap) * 64;      // within the group
  const int kh = tap / g.KW, kw = tap - kh * g.KW;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  const int p_begin = split * g.p_per_split;
  const int p_end = p_begin + g.p_per_split < g.P ? p_begin + g.p_per_split : g.P;
  const int KT = (p_end - p_begin + 63) / 64;

  const i32x4 ra = make_buffer_rsrc(g.dy, g.dy_bytes);
  const i32x4 rb = make_buffer_rsrc(g.x, g.x_bytes);
  // a wave-wide load fills 8 pixel rows; lane -> (row, position), fetching the chunk that belongs there
  int row_l[2], a_col[2], b_col[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = (wave * 2 + i) * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ dw_chunk_swizzle(row);
    row_l[i] = row;
    // channels past the end of the group read as zeros (their products are never stored)
    a_col[i] = co0 + chunk * 8 < g.Og ? grp * g.Og + co0 + chunk * 8 : -1;
    b_col[i] = c0 + chunk * 8 < g.Cg ? grp * g.Cg + c0 + chunk * 8 : -1;
  }

  auto issue = [&](int kt, char* stage) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int p = p_begin + kt * 64 + row_l[i];
      const bool live = p < p_end;
      int offa = kOobOffset, offb = kOobOffset;
      if (live) {
        if (a_col[i] >= 0) offa = (p * g.Otot + a_col[i]) * 2;
        const int n = fast_div(p, g.div_ohw);
        const int q = p - n * g.OHW;
        const int oh = fast_div(q, g.div_ow);
        const int ow = q - oh * g.OW;
        const int ih = oh * g.sh - g.ph + kh, iw = ow * g.sw - g.pw + kw;
        if (b_col[i] >= 0 && (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W)
          offb = (((n * g.H + ih) * g.W + iw) * g.Ctot + b_col[i]) * 2;
      }
      lds_dma_16(ra, offa, stage + (wave * 2 + i) * 1024);
      lds_dma_16(rb, offb, stage + kDwTile + (wave * 2 + i) * 1024);
    }
  };

  f32x16 acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0.f;

  if (KT > 0) {
    issue(0, lds);
    lds_dma_wait_all();
  }
  __syncthreads();
  for (int kt = 0; kt < KT; ++kt) {
    const char* cur = lds + (kt & 1) * kDwStage;
    char* nxt = lds + ((kt & 1) ^ 1) * kDwStage;
    if (kt + 1 < KT) issue(kt + 1, nxt);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const uint4 a = read_frag_tr(cur, wm * 32, ks);
      const uint4 b = read_frag_tr(cur + kDwTile, wn * 32, ks);
      acc = Mfma16<T>::run(a, b, acc);
    }
    lds_dma_wait_all();
    __syncthreads();
  }

  // lane holds, in register r, output channel wm*32 + (r/4)*8 + (lane/32)*4 + r%4 and column
  // wn*32 + lane%32: 32 lanes write 32 consecutive floats of one partial row
  float* part = g.part + (int64_t)split * g.Otot * g.K;
  const int c = c0 + wn * 32 + (lane & 31);
  if (c < g.Cg) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int co = co0 + wm * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
      if (co < g.Og) part[(int64_t)(grp * g.Og + co) * g.K + tap * g.Cg + c] = acc[r];
    }
  }
}

// ------------------------------------------------------------------------------------------
// Weight gradient of 3x3 / stride 1 / padding 1 layers with rows of at most 64 pixels: all nine
// taps in one workgroup.  A k-tile is TR whole output rows of one image (TR * OW <= 64 pixels,
// padded with zero rows of dY to 64); the input rows they touch, TR + 2 rows of W + 2 pixels with
// the out-of-image positions as zeros, sit in LDS once and every tap reads its operand fragments
// from them at shifted positions.  Against one workgroup per tap this moves a third of the bytes
// into LDS and multiplies nine times as much per barrier.
// ------------------------------------------------------------------------------------------
constexpr int kRowsWinMax = 208;                              // window pixels at most
constexpr int kRowsSlots = 36;                                // wave-wide loads per k-tile: 8 + 26 + 2 spare
constexpr int kRowsStage = kRowsSlots * 1024;                 // dY tile, then the window (+ spare rows)
constexpr int kRowsStages = 4;                                // k-tiles in LDS: a pair multiplied, a pair in flight

struct DwRowsArgs {
  const void* dy;     // [N*OH*OW][Otot]
  const void* x;      // [N][H][W][Ctot]
  float* part;        // [splits][Otot][9 * Cg]
  int H, W, Ctot, Otot, Cg, Og;
  int TR;             // output rows per k-tile
  int Wp;             // W + 2
  int win_px;         // (TR + 2) * Wp
  int tiles_per_image, total_tiles, tiles_per_split, splits;
  int K;              // 9 * Cg
  int mtiles, ctiles;
  int64_t dy_bytes, x_bytes;
  FastDiv div_ow, div_wp, div_tpi;
};

// Twelve waves: wave = (k-steps 0-1 | 2-3 of every k-tile) x (filter row kh) x (32-channel half of
// the tile's 64 input channels); it holds 64 output channels x 32 input channels x 3 taps (six
// accumulator tiles) and reads two dY fragments and three window fragments per k-step for six
// MFMAs.  The transposing LDS reads bound this kernel: the fragments are shared as widely as the
// register file allows, and the k-steps are split over two sets of waves (added through LDS at the
// end) only to have enough waves asking for them.
constexpr int kRowsWaves = 12;

template <typename T>
__global__ __launch_bounds__(kRowsWaves * 64) void conv_dw_rows_kernel(DwRowsArgs g) {
  __shared__ __attribute__((aligned(1024))) char lds[kRowsStages * kRowsStage];
  const int grp = blockIdx.z;
  const int tiles = g.mtiles * g.ctiles;
  const int xcd = blockIdx.x & 7, pos = blockIdx.x >> 3;
  const int split = xcd + 8 * (pos / tiles);
  if (split >= g.splits) return;   // padding of the grid, uniform for the workgroup
  const int tile = pos % tiles;
  const int tile_m = tile / g.ctiles;
  const int co0 = tile_m * 64, c0 = (tile - tile_m * g.ctiles) * 64;   // within the group
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int khalf = wave / 6, w6 = wave % 6;   // which k-steps; position among the six accumulator owners
  const int wn = w6 & 1, kh = w6 >> 1;

  const int t_begin = split * g.tiles_per_split;
  const int t_end = t_begin + g.tiles_per_split < g.total_tiles ? t_begin + g.tiles_per_split : g.total_tiles;

  const i32x4 ra = make_buffer_rsrc(g.dy, g.dy_bytes);
  const i32x4 rb = make_buffer_rsrc(g.x, g.x_bytes);
  // Every wave issues exactly kRowsSlots / kRowsWaves loads per k-tile (slots past the data fetch
  // zeros into spare rows), so that "k-tile t has landed" is a fixed count of outstanding loads.
  // What a lane fetches differs between k-tiles only by the tile's first pixel (n, oh0, 0): the rest
  // of the byte offset, and whether the position exists at all, are fixed per slot.
  constexpr int kLoads = kRowsSlots / kRowsWaves;
  int slot_const[kLoads], slot_row[kLoads], slot_pitch[kLoads];
  bool slot_ok[kLoads];
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    const int slot = wave + kRowsWaves * i;
    if (slot < 8) {
      // dY tile: pixel k of the k-tile is (row k / OW, column k % OW); rows past TR are zeros
      const int k = slot * 8 + (lane >> 3);
      const int r = fast_div(k, g.div_ow), ow = k - r * g.W;
      const int chunk = (lane & 7) ^ dw_chunk_swizzle(k);
      slot_ok[i] = r < g.TR && co0 + chunk * 8 < g.Og;
      slot_row[i] = r;
      slot_pitch[i] = g.Otot * 2;
      slot_const[i] = ((r * g.W + ow) * g.Otot + grp * g.Og + co0 + chunk * 8) * 2;
    } else {
      const int j = (slot - 8) * 8 + (lane >> 3);           // window pixel
      const int chunk = (lane & 7) ^ dw_chunk_swizzle(j);
      const int wr = fast_div(j, g.div_wp), wc = j - wr * g.Wp;
      slot_ok[i] = j < g.win_px && (unsigned)(wc - 1) < (unsigned)g.W && c0 + chunk * 8 < g.Cg;
      slot_row[i] = wr - 1;
      slot_pitch[i] = g.Ctot * 2;
      slot_const[i] = (((wr - 1) * g.W + wc - 1) * g.Ctot + grp * g.Cg + c0 + chunk * 8) * 2;
    }
  }
  auto issue = [&](int t, char* stage) {
    const bool live = t < t_end;
    const int n = fast_div(t, g.div_tpi);
    const int oh0 = (t - n * g.tiles_per_image) * g.TR;
    const int first_px = (n * g.H + oh0) * g.W;
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const int slot = wave + kRowsWaves * i;
      const bool ok = live && slot_ok[i] && (unsigned)(oh0 + slot_row[i]) < (unsigned)g.H;
      const int off = ok ? first_px * slot_pitch[i] + slot_const[i] : kOobOffset;
      if (slot < 8) lds_dma_16(ra, off, stage + slot * 1024);   // uniform for the wave
      else lds_dma_16(rb, off, stage + slot * 1024);
    }
  };

  // LDS positions (relative to a stage) of the fragments this lane reads per k-tile; they do not
  // change from k-tile to k-tile.  dY fragments as in read_frag_tr.  Window fragments: pixel k ->
  // (row r, column ow) -> window row (r + kh) * Wp + ow + kw; padding pixels (their dY is zero) are
  // kept inside the window.
  const int li = lane & 15, gq = lane >> 4;
  int a_rel[2][2][2], b_rel[2][3][2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int k = (khalf * 2 + kk) * 16 + (gq >> 1) * 8 + (li >> 2) + h * 4;
#pragma unroll
      for (int f = 0; f < 2; ++f) {
        const int byte = (f * 32 + (gq & 1) * 16 + (li & 3) * 4) * 2;
        a_rel[kk][f][h] = k * 128 + (((byte >> 4) ^ dw_chunk_swizzle(k)) << 4) + (byte & 15);
      }
      int r = fast_div(k, g.div_ow);
      const int ow = k - r * g.W;
      if (r >= g.TR) r = g.TR - 1;
      const int byte = (wn * 32 + (gq & 1) * 16 + (li & 3) * 4) * 2;
#pragma unroll
      for (int kw = 0; kw < 3; ++kw) {
        const int row = (r + kh) * g.Wp + ow + kw;
        b_rel[kk][kw][h] = kDwTile + row * 128 + (((byte >> 4) ^ dw_chunk_swizzle(row)) << 4) + (byte & 15);
      }
    }

  f32x16 acc[2][3];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int t = 0; t < 3; ++t)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][t][e] = 0.f;

  // k-tiles are multiplied in pairs between barriers: while the pair in stages {0, 1} (or {2, 3}) is
  // multiplied, the next pair travels into the other two stages.  One barrier, one wait for loads
  // and one ramp-up of the fragment reads per two k-tiles.
  issue(t_begin, lds);
  issue(t_begin + 1, lds + kRowsStage);
  typedef __attribute__((address_space(3))) s16x4 lds_s16x4;
  for (int t = t_begin; t < t_end; t += 2) {
    const int half = ((t - t_begin) >> 1) & 1;
    lds_dma_wait_all();
    __syncthreads();   // this pair is in LDS for everybody, and nobody reads the pair before any more
    issue(t + 2, lds + ((half ^ 1) * 2) * kRowsStage);
    issue(t + 3, lds + ((half ^ 1) * 2 + 1) * kRowsStage);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      if (t + u >= t_end) break;   // uniform
      const char* cur = lds + (half * 2 + u) * kRowsStage;
      auto frag = [&](const int (&rel)[2]) {
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(cur + rel[0]));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(cur + rel[1]));
        const uint2 x0 = __builtin_bit_cast(uint2, lo), x1 = __builtin_bit_cast(uint2, hi);
        return make_uint4(x0.x, x0.y, x1.x, x1.y);
      };
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const uint4 a0 = frag(a_rel[kk][0]), a1 = frag(a_rel[kk][1]);
#pragma unroll
        for (int kw = 0; kw < 3; ++kw) {
          const uint4 b = frag(b_rel[kk][kw]);
          acc[0][kw] = Mfma16<T>::run(a0, b, acc[0][kw]);
          acc[1][kw] = Mfma16<T>::run(a1, b, acc[1][kw]);
        }
      }
    }
  }
  lds_dma_wait_all();   // the loads issued past the end of the range have nothing to deliver, but must land
  // The waves of the second k-step set hand their sums to their partners through LDS, one
  // 32-output-channel half (48 floats per lane) at a time.
  float* fold = reinterpret_cast<float*>(lds);
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    __syncthreads();
    if (khalf == 1) {
#pragma unroll
      for (int kw = 0; kw < 3; ++kw)
#pragma unroll
        for (int r = 0; r < 16; ++r) fold[((w6 * 48 + kw * 16 + r) << 6) + lane] = acc[i][kw][r];
    }
    __syncthreads();
    if (khalf == 0) {
#pragma unroll
      for (int kw = 0; kw < 3; ++kw)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][kw][r] += fold[((w6 * 48 + kw * 16 + r) << 6) + lane];
    }
  }
  if (khalf == 1) return;

  // register r of a 32 x 32 accumulator = output channel (r/4)*8 + (lane/32)*4 + r%4, column lane%32
  float* part = g.part + (int64_t)split * g.Otot * g.K;
  const int c = c0 + wn * 32 + (lane & 31);
  if (c < g.Cg) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int kw = 0; kw < 3; ++kw)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int co = co0 + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
          if (co < g.Og) part[(int64_t)(grp * g.Og + co) * g.K + (kh * 3 + kw) * g.Cg + c] = acc[i][kw][r];
        }
  }
}

// dW[o][c][tap] = sum over splits of part[split][o][tap * Cg + c], fixed order.  A workgroup
// owns 64 consecutive partial columns; its four waves each sum every fourth split.
template <typename T>
__global__ __launch_bounds__(256) void conv_dw_finish_kernel(const float* __restrict__ part, T* __restrict__ dw,
                                                              int splits, int Cg, int taps, int64_t total) {
  // 16 lanes of 4 consecutive partial elements each (one 16-byte load per split) times 16 slice
  // lanes that stride the splits, 8 loads in flight per lane; the 16 slice sums are folded
  // through LDS in a fixed order.  total % 4 == 0 (the contraction channels are padded to 64).
  __shared__ float4 sm[16][16];
  const int col = threadIdx.x & 15, slice = threadIdx.x >> 4;
  const int64_t i = ((int64_t)blockIdx.x * 16 + col) * 4;   // index into a partial: (o, tap, c)
  float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
  if (i < total) {
    const float* src = part + i;
    for (int sp0 = slice; sp0 < splits; sp0 += 16 * 8) {
      float4 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int sp = sp0 + 16 * u;
        v[u] = *reinterpret_cast<const float4*>(src + (int64_t)(sp < splits ? sp : sp0) * total);
      }
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (sp0 + 16 * u < splits) {
          s.x += v[u].x; s.y += v[u].y; s.z += v[u].z; s.w += v[u].w;
        }
    }
  }
  sm[slice][col] = s;
  __syncthreads();
  if (slice < 4 && i < total) {
    // lane (col, e = slice) finishes element i + e
    const int e = slice;
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < 16; ++k) t += reinterpret_cast<const float*>(&sm[k][col])[e];
    const int64_t idx = i + e;
    const int c = (int)(idx % Cg);
    const int tap = (int)((idx / Cg) % taps);
    const int64_t o = idx / ((int64_t)Cg * taps);
    dw[(o * Cg + c) * taps + tap] = from_f32<T>(t);
  }
}

// ------------------------------------------------------------------------------------------
// Host side.
// ------------------------------------------------------------------------------------------
constexpr int64_t kMaxBytes = (int64_t)1 << 31;   // 32-bit buffer offsets
constexpr int kDwMaxSplits = 256;

inline int64_t round256(int64_t v) { return (v + 255) & ~(int64_t)255; }
inline bool is16(int dt) { return dt == AT_DTYPE_F16 || dt == AT_DTYPE_BF16; }

template <typename F>
inline int dispatch16(int dt, F&& f) {
  if (dt == AT_DTYPE_F16) return f((f16_t*)0);
  if (dt == AT_DTYPE_BF16) return f((bf16_t*)0);
  return AT_ERR_DTYPE;
}

inline bool sizes_ok(const ConvProblem& p) {
  const int64_t x_bytes = p.N * p.C * p.H * p.W * 2, y_bytes = p.N * p.O * p.OH * p.OW * 2;
  const int64_t w_bytes = p.O * (p.C / p.groups) * p.KH * p.KW * 2;
  return x_bytes < kMaxBytes && y_bytes < kMaxBytes && w_bytes < kMaxBytes && p.groups <= 65535 &&
         p.N <= 65535;
}

inline int64_t pad64(int64_t v) { return (v + 63) / 64 * 64; }

// Contraction channels per group: the products take whole 64-channel tiles, so other counts are
// padded with zero channels in the channels-last copy and in the reordered weights.  From 16
// channels on (at most four times the arithmetic) that still beats the kernels that gather.
inline bool contract_ok(int64_t per_group) { return per_group % 64 == 0 || per_group >= 16; }

// [N][C][H*W] -> [N][Hd*Wd][groups * Cgp]: channels of every group padded from C / groups to Cgp,
// pixel (h, w) at (h * sh, w * sw) of an image of Hd x Wd = ((H-1) sh + 1) x ((W-1) sw + 1).
int to_nhwc_ex(const void* src, void* dst, int64_t N, int64_t C, int64_t H, int64_t W, int64_t groups, int64_t Cgp,
               int64_t sh, int64_t sw, int dt, hipStream_t stream) {
  const int64_t Cg = C / groups, HW = H * W;
  const bool padded = Cgp != Cg;
  const int64_t Cd = padded ? groups * Cgp : C;
  const int64_t Hd = (H - 1) * sh + 1, Wd = (W - 1) * sw + 1;
  LayoutCopyArgs a{};
  a.C = (int)C; a.HW = (int)HW; a.Cg = (int)Cg; a.Cgp = (int)Cgp;
  a.W = (int)W; a.Wd = (int)Wd; a.sh = (int)sh; a.sw = (int)sw; a.HWd = (int)(Hd * Wd);
  a.vec_in = (HW % 8 == 0) && aligned16(src);
  a.vec_out = (Cd % 8 == 0) && aligned16(dst);
  const dim3 grid((unsigned)cdiv64(HW, 64), (unsigned)(padded ? groups * (Cgp / 64) : cdiv64(C, 64)), (unsigned)N);
  if (sh * sw > 1) {   // the pixels in between stay zero
    const int64_t count16 = cdiv64(N * Hd * Wd * Cd * 2, 16);
    int64_t blocks = cdiv64(count16, 256 * 4);
    if (blocks > 65535) blocks = 65535;
    hipLaunchKernelGGL(conv_clear_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (uint4*)dst, count16);
  }
  return dispatch16(dt, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    hipLaunchKernelGGL((nchw_to_nhwc_kernel<T>), grid, dim3(256), 0, stream, (const T*)src, (T*)dst, a);
    return launch_status();
  });
}

int to_nhwc(const void* src, void* dst, int64_t N, int64_t C, int64_t HW, int dt, hipStream_t stream) {
  return to_nhwc_ex(src, dst, N, C, 1, HW, 1, C, 1, 1, dt, stream);
}

// colsp: contraction channels per group as padded for the product
int weight_taps(const void* w, void* wt, const ConvProblem& p, int flip, int64_t colsp, hipStream_t stream) {
  const int64_t rows = flip ? p.C : p.O;
  const int64_t total = rows * p.KH * p.KW * colsp;
  return dispatch16(p.dtype, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    hipLaunchKernelGGL((conv_weight_taps_kernel<T>), dim3((unsigned)cdiv64(total, 256)), dim3(256), 0, stream,
                       (const T*)w, (T*)wt, (int)p.O, (int)(p.C / p.groups), (int)(p.O / p.groups),
                       (int)(p.KH * p.KW), flip, (int)colsp, total);
    return launch_status();
  });
}

// Largest number of input pixels (flattened over image, row, column) that the taps of one tile of
// 128 consecutive output pixels span, or -1 when the position of tap (0, 0) does not grow with the
// output pixel (very wide padding) or the answer would take too long to find.
int64_t halo_rows_needed(const IgemmArgs& g, int64_t n_img, int64_t OH, int KH) {
  const int64_t OW = g.OW, OHW = OH * OW, M = n_img * OHW;
  if ((int64_t)g.sh * g.IW < (OW - 1) * g.sw) return -1;
  if ((int64_t)g.IH * g.IW < (OH - 1) * g.sh * g.IW + (OW - 1) * g.sw) return -1;
  auto q_of = [&](int64_t m) {
    const int64_t n = m / OHW, p = m % OHW, oh = p / OW, ow = p % OW;
    return (n * g.IH + oh * g.sh - g.ph) * g.IW + ow * g.sw - g.pw;
  };
  // The span depends only on where the tile starts inside its image, and that offset repeats
  // with period OHW / gcd(OHW, 128) tiles.
  int64_t a = OHW, b = CBM;
  while (b) { const int64_t r = a % b; a = b; b = r; }
  const int64_t period = OHW / a;
  const int64_t tiles = cdiv64(M, CBM);
  const int64_t walk = tiles < period ? tiles : period;
  if (walk > 16384) return -1;
  int64_t worst = 0;
  for (int64_t t = 0; t < walk; ++t) {
    const int64_t m0 = t * CBM;
    const int64_t m_last = m0 + CBM - 1 < M ? m0 + CBM - 1 : M - 1;
    const int64_t span = q_of(m_last) + (int64_t)(KH - 1) * g.IW + g.KW - q_of(m0);
    if (span > worst) worst = span;
  }
  return worst;
}

// One product out[(n,oh,ow), co] over channels-last `act`; see IgemmArgs for the meaning of the fields.
// cg_real: contraction channels per group in the weight tensor (g.Cg is that count padded to 64s).
int run_igemm(IgemmArgs g, const void* w, const ConvProblem& p, int flip, int cg_real, int64_t n_img, int64_t OH,
              int groups, int dt, hipStream_t stream) {
  g.OHW = (int)(OH * g.OW);
  g.M = (int)(n_img * g.OHW);
  g.K = g.KT * 64;
  g.tiles_per_tap = g.Cg / 64;
  g.nbn = (int)cdiv64(g.Og, CBN);
  g.vec_store = g.out_last ? (g.Og % 8 == 0) && aligned16(g.out) : (g.OHW % 8 == 0) && aligned16(g.out);
  g.div_ohw = make_fastdiv(g.OHW);
  g.div_ow = make_fastdiv(g.OW);
  const dim3 grid((unsigned)(cdiv64(g.M, CBM) * g.nbn), 1, (unsigned)groups);
  const int KH = g.KT / (g.tiles_per_tap * g.KW);
  const int64_t window = halo_rows_needed(g, n_img, OH, KH);
  const bool resident = window > 0 && window <= kHaloRows;
  return dispatch16(dt, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    // weights in registers: 3x3-sized filters over 64 channels, enough tiles for every resident
    // workgroup (two per CU) to walk over several
    const int64_t tiles_m = cdiv64(g.M, CBM);
    const int stat_grid = device_cu_count() * 2 / 8 * 8;
    const bool stationary = resident && g.tiles_per_tap == 1 && g.KT == 9 && stat_grid >= 8 && tiles_m >= 4 * stat_grid;
    // rows in a ring of LDS slots: channels-last 3x3 layers with stride 1 and padding 1, bands of 28
    // columns that waste little of the 32-pixel operands, and at least one step of 8 rows for
    // every resident workgroup
    RingArgs ra{};
    ra.bands = (int)cdiv64(g.IW, kRingBand);
    ra.steps_per_strip = (int)cdiv64(g.IH, kRingStep);
    const int64_t ring_steps = n_img * ra.bands * ra.steps_per_strip;
    const bool ring = g.out_last && g.tiles_per_tap == 1 && g.KT == 9 && g.KW == 3 && g.sh == 1 && g.sw == 1 &&
                      g.ph == 1 && g.pw == 1 && OH == g.IH && g.OW == g.IW && stat_grid >= 8 &&
                      ring_steps >= stat_grid && ring_steps < INT32_MAX && g.IW * 5 >= ra.bands * 32 * 4 &&
                      g.Og % 8 == 0 && (reinterpret_cast<uintptr_t>(g.out) & 15u) == 0;
    if (resident || ring) {
      const int ntiles = (g.Og + 31) / 32;
      const int64_t chunks = (int64_t)groups * ntiles * (g.K / 16) * 64;
      hipLaunchKernelGGL((conv_weight_frags_direct_kernel<T>), dim3((unsigned)cdiv64(chunks, 256)), dim3(256), 0,
                         stream, (const T*)w, (T*)g.wf, cg_real, g.Cg, g.Og, (int)(p.KH * p.KW), flip, ntiles,
                         chunks);
      if (ring) {
        ra.total_steps = (int)ring_steps;
        ra.out_bytes = (int64_t)g.M * g.Og * groups * 2;
        ra.div_steps = make_fastdiv(ra.steps_per_strip);
        ra.div_bands = make_fastdiv(ra.bands);
        const dim3 rgrid((unsigned)stat_grid, (unsigned)g.nbn, (unsigned)groups);
        hipLaunchKernelGGL((conv_igemm_ring_kernel<T>), rgrid, dim3(256), 0, stream, g, ra);
      } else if (stationary) {
        const dim3 sgrid((unsigned)stat_grid, (unsigned)g.nbn, (unsigned)groups);
        if (g.out_last)
          hipLaunchKernelGGL((conv_igemm_stationary_kernel<T, true, 9>), sgrid, dim3(256), 0, stream, g, (int)tiles_m);
        else
          hipLaunchKernelGGL((conv_igemm_stationary_kernel<T, false, 9>), sgrid, dim3(256), 0, stream, g, (int)tiles_m);
      } else if (g.out_last) {
        hipLaunchKernelGGL((conv_igemm_halo_kernel<T, true>), grid, dim3(256), 0, stream, g);
      } else {
        hipLaunchKernelGGL((conv_igemm_halo_kernel<T, false>), grid, dim3(256), 0, stream, g);
      }
    } else {
      const int rc = weight_taps(w, const_cast<void*>(g.wt), p, flip, g.Cg, stream);
      if (rc) return rc;
      if (g.out_last) hipLaunchKernelGGL((conv_igemm_kernel<T, true>), grid, dim3(256), 0, stream, g);
      else hipLaunchKernelGGL((conv_igemm_kernel<T, false>), grid, dim3(256), 0, stream, g);
    }
    return launch_status();
  });
}

}  // namespace

namespace {
// bytes of the fragment-major weight copy: output channels per group padded to 32
inline int64_t frag_weight_bytes(int64_t groups, int64_t out_per_group, int64_t K) {
  return groups * ((out_per_group + 31) / 32 * 32) * K * 2;
}
}  // namespace

namespace {
// sizes of the channels-last copies the products read
inline int64_t fwd_act_bytes(const ConvProblem& p) { return p.N * p.H * p.W * p.groups * pad64(p.C / p.groups) * 2; }
inline int64_t dx_rows(const ConvProblem& p) { return (p.OH - 1) * p.sh + 1; }
inline int64_t dx_cols(const ConvProblem& p) { return (p.OW - 1) * p.sw + 1; }
inline int64_t dx_act_bytes(const ConvProblem& p) {
  return p.N * dx_rows(p) * dx_cols(p) * p.groups * pad64(p.O / p.groups) * 2;
}
}  // namespace

bool conv_igemm_supports_fwd(const ConvProblem& p) {
  return is16(p.dtype) && contract_ok(p.C / p.groups) && sizes_ok(p) && fwd_act_bytes(p) < kMaxBytes &&
         p.O * pad64(p.C / p.groups) * p.KH * p.KW * 2 < kMaxBytes && p.N * p.OH * p.OW < kMaxBytes;
}

// The input gradient of a strided layer is the stride-1 product over the output gradient spread
// out by the strides (zeros in between): sh * sw times the arithmetic, so strides up to 2 x 2.
bool conv_igemm_supports_dx(const ConvProblem& p) {
  return is16(p.dtype) && contract_ok(p.O / p.groups) && sizes_ok(p) && p.sh * p.sw <= 4 &&
         p.ph <= p.KH - 1 && p.pw <= p.KW - 1 && dx_act_bytes(p) < kMaxBytes &&
         p.C * pad64(p.O / p.groups) * p.KH * p.KW * 2 < kMaxBytes && p.N * p.H * p.W < kMaxBytes;
}

bool conv_igemm_fwd_leaves_nhwc(const ConvProblem& p) {
  return conv_igemm_supports_fwd(p) && (p.C / p.groups) % 64 == 0;
}

bool conv_igemm_supports_dw(const ConvProblem& p) {
  return is16(p.dtype) && (p.C / p.groups) % 8 == 0 && (p.O / p.groups) % 8 == 0 && sizes_ok(p) &&
         p.N * p.OH * p.OW < kMaxBytes - 64 * kDwMaxSplits;
}

int64_t conv_igemm_fwd_workspace(const ConvProblem& p) {
  if (!conv_igemm_supports_fwd(p)) return 0;
  const int64_t cgp = pad64(p.C / p.groups);
  return round256(fwd_act_bytes(p)) + round256(p.O * cgp * p.KH * p.KW * 2) +
         round256(frag_weight_bytes(p.groups, p.O / p.groups, cgp * p.KH * p.KW));
}

int64_t conv_igemm_dx_workspace(const ConvProblem& p) {
  if (!conv_igemm_supports_dx(p)) return 0;
  const int64_t ogp = pad64(p.O / p.groups);
  return round256(dx_act_bytes(p)) + round256(p.C * ogp * p.KH * p.KW * 2) +
         round256(frag_weight_bytes(p.groups, p.C / p.groups, ogp * p.KH * p.KW));
}

namespace {
inline int dw_split_count(const ConvProblem& p) {
  const int64_t P = p.N * p.OH * p.OW;
  const int64_t tiles = cdiv64(p.O / p.groups, 64) * (p.KH * p.KW * cdiv64(p.C / p.groups, 64)) * p.groups;
  int64_t want = cdiv64((int64_t)device_cu_count() * 4, tiles);
  const int64_t by_len = cdiv64(P, 256);   // at least four k-tiles per split
  if (want > by_len) want = by_len;
  if (want > kDwMaxSplits) want = kDwMaxSplits;
  return (int)(want < 1 ? 1 : want);
}
inline int64_t dw_padded_k(const ConvProblem& p) { return p.KH * p.KW * (p.C / p.groups); }
}  // namespace

int64_t conv_igemm_dw_workspace(const ConvProblem& p) {
  if (!conv_igemm_supports_dw(p)) return 0;
  return round256(p.N * p.O * p.OH * p.OW * 2) + round256(p.N * p.C * p.H * p.W * 2) +
         round256((int64_t)kDwMaxSplits * p.O * dw_padded_k(p) * 4);
}

int conv_igemm_fwd(const ConvProblem& p, const void* x, const void* w, const void* bias, int bias_dt,
                   void* y, void* workspace, hipStream_t stream) {
  char* ws = static_cast<char*>(workspace);
  const int64_t cg = p.C / p.groups, cgp = pad64(cg);
  void* xh = ws;
  void* wt = ws + round256(fwd_act_bytes(p));
  int rc = to_nhwc_ex(x, xh, p.N, p.C, p.H, p.W, p.groups, cgp, 1, 1, p.dtype, stream);
  if (rc) return rc;
  IgemmArgs g{};
  g.act = xh; g.wt = wt; g.out = y; g.bias = bias; g.bias_dt = bias_dt;
  g.wf = static_cast<char*>(wt) + round256(p.O * cgp * p.KH * p.KW * 2);
  g.IH = (int)p.H; g.IW = (int)p.W; g.Ctot = (int)(p.groups * cgp); g.Cg = (int)cgp; g.Og = (int)(p.O / p.groups);
  g.KW = (int)p.KW; g.OW = (int)p.OW; g.sh = (int)p.sh; g.sw = (int)p.sw; g.ph = (int)p.ph; g.pw = (int)p.pw;
  g.KT = (int)(p.KH * p.KW * (g.Cg / 64));
  g.act_bytes = fwd_act_bytes(p);
  g.wt_bytes = p.O * cgp * p.KH * p.KW * 2;
  return run_igemm(g, w, p, 0, (int)cg, p.N, p.OH, (int)p.groups, p.dtype, stream);
}

// ---- channels-last tensors in and out: no copies, the workspace holds the reordered weights only ----
bool conv_igemm_supports_fwd_last(const ConvProblem& p) {
  return is16(p.dtype) && (p.C / p.groups) % 64 == 0 && sizes_ok(p) && p.N * p.OH * p.OW < kMaxBytes;
}

bool conv_igemm_supports_dx_last(const ConvProblem& p) {
  return is16(p.dtype) && (p.O / p.groups) % 64 == 0 && sizes_ok(p) && p.sh == 1 && p.sw == 1 &&
         p.ph <= p.KH - 1 && p.pw <= p.KW - 1 && p.N * p.H * p.W < kMaxBytes;
}

namespace {
inline int64_t last_weight_workspace(const ConvProblem& p, int64_t rows_per_group, int64_t contract_per_group) {
  const int64_t taps = p.KH * p.KW;
  return round256(p.groups * rows_per_group * contract_per_group * taps * 2) +
         round256(frag_weight_bytes(p.groups, rows_per_group, contract_per_group * taps));
}
}  // namespace

int64_t conv_igemm_fwd_last_workspace(const ConvProblem& p) {
  return conv_igemm_supports_fwd_last(p) ? last_weight_workspace(p, p.O / p.groups, p.C / p.groups) : 0;
}

int64_t conv_igemm_dx_last_workspace(const ConvProblem& p) {
  return conv_igemm_supports_dx_last(p) ? last_weight_workspace(p, p.C / p.groups, p.O / p.groups) : 0;
}

int conv_igemm_fwd_last(const ConvProblem& p, const void* x_last, const void* w, const void* bias, int bias_dt,
                        void* y_last, void* workspace, hipStream_t stream) {
  char* wt = static_cast<char*>(workspace);
  const int64_t cg = p.C / p.groups;
  IgemmArgs g{};
  g.act = x_last; g.wt = wt; g.out = y_last; g.bias = bias; g.bias_dt = bias_dt; g.out_last = 1;
  g.wf = wt + round256(p.O * cg * p.KH * p.KW * 2);
  g.IH = (int)p.H; g.IW = (int)p.W; g.Ctot = (int)p.C; g.Cg = (int)cg; g.Og = (int)(p.O / p.groups);
  g.KW = (int)p.KW; g.OW = (int)p.OW; g.sh = (int)p.sh; g.sw = (int)p.sw; g.ph = (int)p.ph; g.pw = (int)p.pw;
  g.KT = (int)(p.KH * p.KW * (g.Cg / 64));
  g.act_bytes = p.N * p.C * p.H * p.W * 2;
  g.wt_bytes = p.O * cg * p.KH * p.KW * 2;
  return run_igemm(g, w, p, 0, (int)cg, p.N, p.OH, (int)p.groups, p.dtype, stream);
}

int conv_igemm_dx_last(const ConvProblem& p, const void* dy_last, const void* w, void* dx_last, void* workspace,
                       hipStream_t stream) {
  char* wt = static_cast<char*>(workspace);
  const int64_t og = p.O / p.groups;
  IgemmArgs g{};
  g.act = dy_last; g.wt = wt; g.out = dx_last; g.bias = nullptr; g.bias_dt = 0; g.out_last = 1;
  g.wf = wt + round256(p.C * og * p.KH * p.KW * 2);
  g.IH = (int)p.OH; g.IW = (int)p.OW; g.Ctot = (int)p.O; g.Cg = (int)og; g.Og = (int)(p.C / p.groups);
  g.KW = (int)p.KW; g.OW = (int)p.W; g.sh = 1; g.sw = 1; g.ph = (int)(p.KH - 1 - p.ph); g.pw = (int)(p.KW - 1 - p.pw);
  g.KT = (int)(p.KH * p.KW * (g.Cg / 64));
  g.act_bytes = p.N * p.O * p.OH * p.OW * 2;
  g.wt_bytes = p.C * og * p.KH * p.KW * 2;
  return run_igemm(g, w, p, 1, (int)og, p.N, p.H, (int)p.groups, p.dtype, stream);
}

int conv_nchw_to_nhwc(const void* src, void* dst, int64_t N, int64_t C, int64_t HW, int dtype,
                      hipStream_t stream) {
  if (!is16(dtype)) return AT_ERR_DTYPE;
  if (N <= 0 || C <= 0 || HW <= 0 || N > 65535 || C > INT32_MAX || HW > INT32_MAX) return AT_ERR_DIM;
  return to_nhwc(src, dst, N, C, HW, dtype, stream);
}

int conv_igemm_dx(const ConvProblem& p, const void* dy, const void* dy_nhwc, const void* w, void* dx,
                  void* workspace, hipStream_t stream) {
  char* ws = static_cast<char*>(workspace);
  const int64_t og = p.O / p.groups, ogp = pad64(og);
  // the caller's channels-last copy serves only when the product reads dY as it is
  const void* dyh = (ogp == og && p.sh == 1 && p.sw == 1) ? dy_nhwc : nullptr;
  void* wt = ws + round256(dx_act_bytes(p));
  int rc = AT_OK;
  if (!dyh) {
    rc = to_nhwc_ex(dy, ws, p.N, p.O, p.OH, p.OW, p.groups, ogp, p.sh, p.sw, p.dtype, stream);
    dyh = ws;
  }
  if (rc) return rc;
  // dX[n, c, ih, iw] = sum_{taps', o} dY[n, ih + kh' - (KH-1-ph), iw + kw' - (KW-1-pw), o] * W[o, c, mirrored tap]
  IgemmArgs g{};
  g.act = dyh; g.wt = wt; g.out = dx; g.bias = nullptr; g.bias_dt = 0;
  g.wf = static_cast<char*>(wt) + round256(p.C * ogp * p.KH * p.KW * 2);
  g.IH = (int)dx_rows(p); g.IW = (int)dx_cols(p); g.Ctot = (int)(p.groups * ogp); g.Cg = (int)ogp;
  g.Og = (int)(p.C / p.groups);
  g.KW = (int)p.KW; g.OW = (int)p.W; g.sh = 1; g.sw = 1; g.ph = (int)(p.KH - 1 - p.ph); g.pw = (int)(p.KW - 1 - p.pw);
  g.KT = (int)(p.KH * p.KW * (g.Cg / 64));
  g.act_bytes = dx_act_bytes(p);
  g.wt_bytes = p.C * ogp * p.KH * p.KW * 2;
  return run_igemm(g, w, p, 1, (int)og, p.N, p.H, (int)p.groups, p.dtype, stream);
}

int conv_igemm_dw(const ConvProblem& p, const void* dy, const void* dy_nhwc, const void* x, const void* x_nhwc,
                  void* dw, void* workspace, hipStream_t stream) {
  char* ws = static_cast<char*>(workspace);
  const void* dyh = dy_nhwc;
  const void* xh = x_nhwc;
  float* part = reinterpret_cast<float*>(ws + round256(p.N * p.O * p.OH * p.OW * 2) +
                                         round256(p.N * p.C * p.H * p.W * 2));
  int rc = AT_OK;
  if (!dyh) {
    rc = to_nhwc(dy, ws, p.N, p.O, p.OH * p.OW, p.dtype, stream);
    dyh = ws;
  }
  if (rc) return rc;
  if (!xh) {
    void* dst = ws + round256(p.N * p.O * p.OH * p.OW * 2);
    rc = to_nhwc(x, dst, p.N, p.C, p.H * p.W, p.dtype, stream);
    xh = dst;
  }
  if (rc) return rc;
  if (p.KH == 3 && p.KW == 3 && p.sh == 1 && p.sw == 1 && p.ph == 1 && p.pw == 1 && p.OW <= 64) {
    DwRowsArgs r{};
    r.dy = dyh; r.x = xh; r.part = part;
    r.H = (int)p.H; r.W = (int)p.W; r.Ctot = (int)p.C; r.Otot = (int)p.O; r.Cg = (int)(p.C / p.groups);
    r.Og = (int)(p.O / p.groups);
    r.TR = (int)(64 / p.OW < p.OH ? 64 / p.OW : p.OH);
    r.Wp = (int)p.W + 2;
    r.win_px = (r.TR + 2) * r.Wp;
    if (r.win_px <= kRowsWinMax) {
      r.tiles_per_image = (int)cdiv64(p.OH, r.TR);
      r.total_tiles = (int)(p.N * r.tiles_per_image);
      r.K = 9 * r.Cg;
      r.mtiles = (int)cdiv64(r.Og, 64);
      r.ctiles = (int)cdiv64(r.Cg, 64);
      // two workgroups per CU over the whole grid, at least four k-tiles each
      int64_t want = cdiv64((int64_t)device_cu_count() * 2, (int64_t)r.mtiles * r.ctiles * p.groups);
      const int64_t by_len = cdiv64(r.total_tiles, 4);
      if (want > by_len) want = by_len;
      if (want > kDwMaxSplits) want = kDwMaxSplits;
      if (want < 1) want = 1;
      r.tiles_per_split = (int)cdiv64(r.total_tiles, want);
      r.splits = (int)cdiv64(r.total_tiles, r.tiles_per_split);
    }
    // small problems give this kernel too few workgroups (one per pixel range and 64 x 64 tile of
    // all taps); the per-tap kernel below has nine times as many
    if (r.win_px <= kRowsWinMax &&
        (int64_t)r.mtiles * r.ctiles * p.groups * r.splits * 2 >= device_cu_count()) {
      r.dy_bytes = p.N * p.O * p.OH * p.OW * 2;
      r.x_bytes = p.N * p.C * p.H * p.W * 2;
      r.div_ow = make_fastdiv(p.OW);
      r.div_wp = make_fastdiv(r.Wp);
      r.div_tpi = make_fastdiv(r.tiles_per_image);
      const dim3 grid((unsigned)(r.mtiles * r.ctiles * (cdiv64(r.splits, 8) * 8)), 1, (unsigned)p.groups);
      const int64_t total = p.O * (int64_t)r.K;
      return dispatch16(p.dtype, [&](auto* tp) -> int {
        typedef std::remove_pointer_t<decltype(tp)> T;
        hipLaunchKernelGGL((conv_dw_rows_kernel<T>), grid, dim3(kRowsWaves * 64), 0, stream, r);
        int rc2 = launch_status();
        if (rc2) return rc2;
        hipLaunchKernelGGL((conv_dw_finish_kernel<T>), dim3((unsigned)cdiv64(total, 64)), dim3(256), 0, stream,
                           (const float*)part, (T*)dw, r.splits, r.Cg, 9, total);
        return launch_status();
      });
    }
  }
  DwArgs g{};
  g.dy = dyh; g.x = xh; g.part = part;
  g.H = (int)p.H; g.W = (int)p.W; g.Ctot = (int)p.C; g.Otot = (int)p.O; g.Cg = (int)(p.C / p.groups);
  g.Og = (int)(p.O / p.groups); g.KW = (int)p.KW; g.OW = (int)p.OW; g.OHW = (int)(p.OH * p.OW);
  g.sh = (int)p.sh; g.sw = (int)p.sw; g.ph = (int)p.ph; g.pw = (int)p.pw;
  g.P = (int)(p.N * p.OH * p.OW);
  g.K = (int)dw_padded_k(p);
  g.tiles_per_tap = (int)cdiv64(g.Cg, 64);
  g.nbn = (int)(p.KH * p.KW) * g.tiles_per_tap;
  const int splits = dw_split_count(p);
  g.p_per_split = (int)(cdiv64(cdiv64(g.P, splits), 64) * 64);
  g.dy_bytes = p.N * p.O * p.OH * p.OW * 2;
  g.x_bytes = p.N * p.C * p.H * p.W * 2;
  g.div_ohw = make_fastdiv(g.OHW);
  g.div_ow = make_fastdiv(g.OW);
  const int real_splits = (int)cdiv64(g.P, g.p_per_split);
  g.mtiles = (int)cdiv64(g.Og, 64);
  g.splits = real_splits;
  const dim3 grid((unsigned)(g.mtiles * g.nbn * (cdiv64(real_splits, 8) * 8)), 1, (unsigned)p.groups);
  const int64_t total = p.O * (int64_t)g.K;
  return dispatch16(p.dtype, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    hipLaunchKernelGGL((conv_dw_kernel<T>), grid, dim3(256), 0, stream, g);
    int rc2 = launch_status();
    if (rc2) return rc2;
    hipLaunchKernelGGL((conv_dw_finish_kernel<T>), dim3((unsigned)cdiv64(total, 64)), dim3(256), 0, stream,
                       (const float*)part, (T*)dw, real_splits, g.Cg, (int)(p.KH * p.KW), total);
    return launch_status();
  });
}

}  // namespace at_hip
