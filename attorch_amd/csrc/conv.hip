// 2D convolution (NCHW, zero padding, stride, groups, no dilation) as implicit GEMM: forward,
// input gradient and weight gradient.
//
// The im2col matrix is never materialised: the operand tiles are gathered straight from the
// NCHW tensors into LDS, multiplied with fp32-accumulating MFMA (v_mfma_f32_32x32x2f32) in
// 64x64 output tiles, and scattered back to NCHW.
//   forward      : Y[(n,oh,ow), co]   = sum_{c,kh,kw} X[n,c,oh*s-p+kh,ow*s-p+kw] * W[co,c,kh,kw]
//   input grad   : dX[(n,ih,iw), c]   = sum_{co,kh,kw} dY[n,co,(ih+p-kh)/s,(iw+p-kw)/s] * W[co,c,kh,kw]
//   weight grad  : dW[co, (c,kh,kw)]  = sum_{n,oh,ow} dY[n,co,oh,ow] * X[n,c,oh*s-p+kh,ow*s-p+kw]
// The weight gradient contracts over batch x space, so it is split over many workgroups that
// write fp32 partial tiles, summed by a second launch in fixed order.
#include <type_traits>

#include "at_common.h"
#include "conv_igemm.h"

namespace at_hip {
namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));

enum ConvMode { kConvFwd = 0, kConvDx = 1, kConvDw = 2 };

struct ConvArgs {
  const void* a;     // fwd: X, dx: dY, dw: dY
  const void* b;     // fwd: W, dx: W,  dw: X
  void* out;         // fwd: Y, dx: dX, dw: fp32 partials
  const void* bias;  // fwd only, nullable
  int bias_dt;
  int N, C, H, W, O, KH, KW, OH, OW, sh, sw, ph, pw, groups;
  int Cg, Og;        // channels per group (input / output)
  int64_t M, K;      // GEMM rows and contraction length
  int cols;          // GEMM columns
  int64_t k_per_split;
};

constexpr int TM = 64, TN = 64, TK = 16;

// A position a * (nb * nc) + b * nc + c, moved forward by a fixed step with two carries.
struct MixedRadix {
  int a, b, c;
  int da, db, dc;
  __device__ __forceinline__ void init(int64_t pos, int nb, int nc) {
    c = (int)(pos % nc);
    const int64_t t = pos / nc;
    b = (int)(t % nb);
    a = (int)(t / nb);
  }
  __device__ __forceinline__ void set_step(int step, int nb, int nc) {
    dc = step % nc;
    const int t = step / nc;
    db = t % nb;
    da = t / nb;
  }
  __device__ __forceinline__ void advance(int nb, int nc) {
    c += dc;
    if (c >= nc) { c -= nc; ++b; }
    b += db;
    if (b >= nb) { b -= nb; ++a; }
    a += da;
  }
  __device__ __forceinline__ void next(int nb, int nc) {
    if (++c >= nc) {
      c = 0;
      if (++b >= nb) { b = 0; ++a; }
    }
  }
};

template <int MODE, typename TI, typename TO>
__global__ __launch_bounds__(256) void conv_gemm_kernel(ConvArgs g) {
  __shared__ float sa[TK][TM + 1];
  __shared__ float sb[TK][TN + 1];
  const TI* __restrict__ A = reinterpret_cast<const TI*>(g.a);
  const TI* __restrict__ B = reinterpret_cast<const TI*>(g.b);
  const int grp = blockIdx.z;
  const int nbn = (g.cols + TN - 1) / TN;
  const int64_t m0 = (int64_t)(blockIdx.x / nbn) * TM;
  const int n0 = (blockIdx.x % nbn) * TN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int KK = g.KH * g.KW;

  int64_t k_begin = 0, k_end = g.K;
  if (MODE == kConvDw) {
    k_begin = (int64_t)blockIdx.y * g.k_per_split;
    k_end = k_begin + g.k_per_split < g.K ? k_begin + g.k_per_split : g.K;
  }

  // Tile elements per thread.  "Gather" operands (the A tile of fwd / dx: contiguous along the image
  // row, i.e. along m) give a thread one m and four consecutive k; "k-fast" operands (contiguous
  // along k) give it one k and four rows 16 apart.  The (channel, kh, kw) or (n, oh, ow) split of a
  // thread's k is carried from k-tile to k-tile by adding the split of TK with two carries
  // (MixedRadix), so the main loop holds no integer division.
  const int tid = threadIdx.x;
  const int m_lane = tid & 63, kq = tid >> 6;
  const int k_lane = tid & 15, x_lane = tid >> 4;

  // fwd / dx gather state
  bool a_row_ok = false;
  int a_n = 0, a_p = 0, a_q = 0;  // (n, oh, ow) for fwd, (n, ih, iw) for dx
  int64_t a_base = 0;
  MixedRadix ga{};                // (channel, kh, kw) of k0 + 4 kq
  // fwd: k of the B element; dx: (co, tap) of it; dw: (n, oh, ow) of both operands' k
  int64_t k_cur = k_begin + k_lane;
  MixedRadix gb{};
  int dw_c[4] = {0, 0, 0, 0}, dw_kh[4] = {0, 0, 0, 0}, dw_kw[4] = {0, 0, 0, 0};
  bool dw_ok[4] = {false, false, false, false};

  if (MODE != kConvDw) {
    const int64_t m = m0 + m_lane;
    a_row_ok = m < g.M;
    const int pw_ = MODE == kConvFwd ? g.OW : g.W, ph_ = MODE == kConvFwd ? g.OH : g.H;
    const int64_t t = a_row_ok ? m : 0;
    a_q = (int)(t % pw_);
    a_p = (int)((t / pw_) % ph_);
    a_n = (int)(t / ((int64_t)pw_ * ph_));
    ga.init(k_begin + 4 * kq, g.KH, g.KW);
    ga.set_step(TK, g.KH, g.KW);
    if (MODE == kConvFwd) {
      // X[n, grp*Cg + c, a_p*sh - ph + kh, a_q*sw - pw + kw] = X[a_base + (c*H + kh)*W + kw]
      a_base = (((int64_t)a_n * g.C + grp * g.Cg) * g.H + (a_p * g.sh - g.ph)) * g.W + (a_q * g.sw - g.pw);
    } else {
      gb.init(k_begin + k_lane, 1, KK);
      gb.set_step(TK, 1, KK);
    }
  } else {
    gb.init(k_begin + k_lane, g.OH, g.OW);
    gb.set_step(TK, g.OH, g.OW);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int j = n0 + x_lane + 16 * i;
      dw_ok[i] = j < g.cols;
      const int jj = dw_ok[i] ? j : 0;
      const int r = jj % KK;
      dw_c[i] = jj / KK;
      dw_kh[i] = r / g.KW;
      dw_kw[i] = r % g.KW;
    }
  }

  // Loads one k-tile's elements of both operands into registers and moves the state on by TK.
  auto fetch = [&](float (&ra)[4], float (&rb)[4]) {
    if (MODE == kConvFwd) {
      MixedRadix e = ga;
      const int ih0 = a_p * g.sh - g.ph, iw0 = a_q * g.sw - g.pw;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = 0.f;
        if (a_row_ok && e.a < g.Cg && (unsigned)(ih0 + e.b) < (unsigned)g.H && (unsigned)(iw0 + e.c) < (unsigned)g.W)
          v = to_f32(A[a_base + ((int64_t)e.a * g.H + e.b) * g.W + e.c]);
        ra[i] = v;
        e.next(g.KH, g.KW);
      }
      ga.advance(g.KH, g.KW);
      // B(k, co) = W[co, k], contiguous over k
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int co = n0 + x_lane + 16 * i;
        rb[i] = (co < g.Og && k_cur < k_end) ? to_f32(B[((int64_t)grp * g.Og + co) * g.K + k_cur]) : 0.f;
      }
    } else if (MODE == kConvDx) {
      MixedRadix e = ga;
      const int th0 = a_p + g.ph, tw0 = a_q + g.pw;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = 0.f;
        int oh = th0 - e.b, ow = tw0 - e.c;
        bool ok = a_row_ok && e.a < g.Og && oh >= 0 && ow >= 0;
        if (g.sh != 1) {
          const int q = oh / g.sh;
          ok = ok && q * g.sh == oh;
          oh = q;
        }
        if (g.sw != 1) {
          const int q = ow / g.sw;
          ok = ok && q * g.sw == ow;
          ow = q;
        }
        if (ok && oh < g.OH && ow < g.OW)
          v = to_f32(A[(((int64_t)a_n * g.O + grp * g.Og + e.a) * g.OH + oh) * g.OW + ow]);
        ra[i] = v;
        e.next(g.KH, g.KW);
      }
      ga.advance(g.KH, g.KW);
      // B(k = (co, tap), c) = W[co, c, tap]
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int c = n0 + x_lane + 16 * i;
        rb[i] = (c < g.Cg && gb.a < g.Og)
                    ? to_f32(B[(((int64_t)grp * g.Og + gb.a) * g.Cg + c) * KK + gb.c]) : 0.f;
      }
      gb.advance(1, KK);
    } else {
      const bool k_ok = k_cur < k_end;
      // A(co, k) = dY[n, co, oh, ow]
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int co = (int)m0 + x_lane + 16 * i;
        ra[i] = (k_ok && co < g.Og)
                    ? to_f32(A[(((int64_t)gb.a * g.O + grp * g.Og + co) * g.OH + gb.b) * g.OW + gb.c]) : 0.f;
      }
      // B(k, j = (c, kh, kw)) = X[n, c, oh*s-p+kh, ow*s-p+kw]
      const int ih0 = gb.b * g.sh - g.ph, iw0 = gb.c * g.sw - g.pw;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int ih = ih0 + dw_kh[i], iw = iw0 + dw_kw[i];
        float v = 0.f;
        if (k_ok && dw_ok[i] && (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W)
          v = to_f32(B[(((int64_t)gb.a * g.C + grp * g.Cg + dw_c[i]) * g.H + ih) * g.W + iw]);
        rb[i] = v;
      }
      gb.advance(g.OH, g.OW);
    }
    k_cur += TK;
  };

  f32x16 acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0.f;

  float ra[4], rb[4];
  if (k_begin < k_end) fetch(ra, rb);
  for (int64_t k0 = k_begin; k0 < k_end; k0 += TK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (MODE == kConvDw) sa[k_lane][x_lane + 16 * i] = ra[i];
      else sa[4 * kq + i][m_lane] = ra[i];
      sb[k_lane][x_lane + 16 * i] = rb[i];
    }
    __syncthreads();
    // the next tile's loads are in flight while this one is multiplied
    if (k0 + TK < k_end) fetch(ra, rb);
#pragma unroll
    for (int ks = 0; ks < TK; ks += 2) {
      const float av = sa[ks + (lane >> 5)][wm * 32 + (lane & 31)];
      const float bv = sb[ks + (lane >> 5)][wn * 32 + (lane & 31)];
      // fwd / dx outputs are contiguous along m, so the operands are swapped there: a lane then
      // owns one m (lane % 32) and 16 columns, and 32 consecutive lanes store consecutive addresses
      acc = MODE == kConvDw ? __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc, 0, 0, 0)
                            : __builtin_amdgcn_mfma_f32_32x32x2f32(bv, av, acc, 0, 0, 0);
    }
    __syncthreads();
  }

  // acc[r] belongs to (row, column) = (sub, lane % 32) for dw and (lane % 32, sub) otherwise,
  // with sub = (r/4)*8 + (lane/32)*4 + r%4.
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int sub = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
    const int64_t m = m0 + wm * 32 + (MODE == kConvDw ? sub : (lane & 31));
    const int col = n0 + wn * 32 + (MODE == kConvDw ? (lane & 31) : sub);
    if (m >= g.M || col >= g.cols) continue;
    const float v = acc[r];
    if (MODE == kConvFwd) {
      const int ow = (int)(m % g.OW), oh = (int)((m / g.OW) % g.OH);
      const int64_t n = m / ((int64_t)g.OW * g.OH);
      const int co = grp * g.Og + col;
      const float bb = g.bias ? load_scalar_f32(g.bias, g.bias_dt, co) : 0.f;
      reinterpret_cast<TO*>(g.out)[((n * g.O + co) * g.OH + oh) * g.OW + ow] = from_f32<TO>(v + bb);
    } else if (MODE == kConvDx) {
      const int iw = (int)(m % g.W), ih = (int)((m / g.W) % g.H);
      const int64_t n = m / ((int64_t)g.W * g.H);
      reinterpret_cast<TO*>(g.out)[((n * g.C + grp * g.Cg + col) * g.H + ih) * g.W + iw] = from_f32<TO>(v);
    } else {
      // partial [split][O][cols]
      float* part = reinterpret_cast<float*>(g.out);
      part[((int64_t)blockIdx.y * g.O + grp * g.Og + m) * g.cols + col] = v;
    }
  }
}

template <typename TO>
__global__ void conv_dw_reduce_kernel(const float* __restrict__ part, TO* __restrict__ out, int splits,
                                      int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  float s = 0.f;
#pragma unroll 8
  for (int p = 0; p < splits; ++p) s += part[(int64_t)p * total + i];
  out[i] = from_f32<TO>(s);
}

// ------------------------------------------------------------------------------------------
// Thin groups (depthwise convolutions, pooling written as a convolution, a three-channel input
// gradient): 64-wide matrix tiles would be mostly padding, so a lane owns one output element and
// walks the few channels and taps of its group in fp32.
// ------------------------------------------------------------------------------------------
constexpr int kThinFeat = 8;         // at most this many output columns of the implicit GEMM
constexpr int kThinWalkFwd = 512;    // channels x taps walked per output element (fwd, dw)
constexpr int kThinWalkDx = 4096;    // output channels x taps walked per input-gradient element
constexpr int kThinTaps = 16;        // taps accumulated at once per lane in the weight gradient

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void conv_direct_fwd_kernel(ConvArgs g) {
  const TI* __restrict__ X = reinterpret_cast<const TI*>(g.a);
  const TI* __restrict__ Wt = reinterpret_cast<const TI*>(g.b);
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= g.M) return;  // M = N * O * OH * OW
  const int ow = (int)(idx % g.OW);
  int64_t t = idx / g.OW;
  const int oh = (int)(t % g.OH);
  t /= g.OH;
  const int co = (int)(t % g.O);
  const int64_t n = t / g.O;
  const int grp = co / g.Og;
  const TI* xg = X + (n * g.C + (int64_t)grp * g.Cg) * g.H * g.W;
  const TI* wg = Wt + (int64_t)co * g.Cg * g.KH * g.KW;
  const int ih0 = oh * g.sh - g.ph, iw0 = ow * g.sw - g.pw;
  float acc = 0.f;
  for (int c = 0; c < g.Cg; ++c) {
    for (int kh = 0; kh < g.KH; ++kh) {
      const int ih = ih0 + kh;
      if ((unsigned)ih >= (unsigned)g.H) continue;
      const TI* xr = xg + ((int64_t)c * g.H + ih) * g.W;
      const TI* wr = wg + (c * g.KH + kh) * g.KW;
#pragma unroll 4
      for (int kw = 0; kw < g.KW; ++kw) {
        const int iw = iw0 + kw;
        if ((unsigned)iw < (unsigned)g.W) acc = fmaf(to_f32(xr[iw]), to_f32(wr[kw]), acc);
      }
    }
  }
  if (g.bias) acc += load_scalar_f32(g.bias, g.bias_dt, co);
  reinterpret_cast<TO*>(g.out)[idx] = from_f32<TO>(acc);
}

// grid (N * C, cdiv(H * W, 256)): a workgroup stays inside one input-gradient plane, so the
// Og x KH x KW weights that plane needs are staged in LDS once.
template <typename T>
__global__ __launch_bounds__(256) void conv_direct_dx_kernel(ConvArgs g) {
  __shared__ float wl[kThinWalkDx];
  const T* __restrict__ dY = reinterpret_cast<const T*>(g.a);
  const T* __restrict__ Wt = reinterpret_cast<const T*>(g.b);
  const int c = blockIdx.x % g.C;
  const int64_t n = blockIdx.x / g.C;
  const int grp = c / g.Cg, cl = c % g.Cg;
  const int KK = g.KH * g.KW;
  for (int i = threadIdx.x; i < g.Og * KK; i += 256) {
    const int co = i / KK, tap = i % KK;
    wl[i] = to_f32(Wt[(((int64_t)grp * g.Og + co) * g.Cg + cl) * KK + tap]);
  }
  __syncthreads();
  const int pix = blockIdx.y * 256 + threadIdx.x;
  if (pix >= g.H * g.W) return;
  const int ih = pix / g.W, iw = pix % g.W;
  const int64_t plane = (int64_t)g.OH * g.OW;
  const T* dyg = dY + (n * g.O + (int64_t)grp * g.Og) * plane;
  float acc = 0.f;
  // only the taps kh = (ih + ph) mod sh, + sh, ... reach an output row, which then steps down by one
  const int th = ih + g.ph, tw = iw + g.pw;
  const int kh0 = th % g.sh, kw0 = tw % g.sw, oh0 = th / g.sh, ow0 = tw / g.sw;
  for (int kh = kh0, oh = oh0; kh < g.KH && oh >= 0; kh += g.sh, --oh) {
    if (oh >= g.OH) continue;
    for (int kw = kw0, ow = ow0; kw < g.KW && ow >= 0; kw += g.sw, --ow) {
      if (ow >= g.OW) continue;
      const T* dyp = dyg + (int64_t)oh * g.OW + ow;
      const float* wp = wl + kh * g.KW + kw;
      // independent loads in flight together: one at a time the walk is bound by memory latency
#pragma unroll 8
      for (int co = 0; co < g.Og; ++co) acc = fmaf(to_f32(dyp[co * plane]), wp[co * KK], acc);
    }
  }
  reinterpret_cast<T*>(g.out)[((n * g.C + c) * g.H) * g.W + pix] = from_f32<T>(acc);
}

// grid (O * Cg, splits): a workgroup sums one filter plane dW[co, c, :, :] over its share of the
// batch x space positions and writes the fp32 partial [split][O][Cg * KH * KW].
template <typename T>
__global__ __launch_bounds__(256) void conv_direct_dw_kernel(ConvArgs g) {
  __shared__ float fold[4][kThinTaps];
  const T* __restrict__ dY = reinterpret_cast<const T*>(g.a);
  const T* __restrict__ X = reinterpret_cast<const T*>(g.b);
  float* __restrict__ part = reinterpret_cast<float*>(g.out);
  const int co = blockIdx.x / g.Cg, cl = blockIdx.x % g.Cg;
  const int c = (co / g.Og) * g.Cg + cl;
  const int KK = g.KH * g.KW;
  const int64_t p_begin = (int64_t)blockIdx.y * g.k_per_split;
  const int64_t p_end = p_begin + g.k_per_split < g.K ? p_begin + g.k_per_split : g.K;  // K = N * OH * OW
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float* out = part + (((int64_t)blockIdx.y * g.O + co) * g.Cg + cl) * KK;

  for (int t0 = 0; t0 < KK; t0 += kThinTaps) {
    int tkh[kThinTaps], tkw[kThinTaps];
#pragma unroll
    for (int j = 0; j < kThinTaps; ++j) {
      const int tap = t0 + j < KK ? t0 + j : 0;
      tkh[j] = tap / g.KW;
      tkw[j] = tap % g.KW;
    }
    float acc[kThinTaps];
#pragma unroll
    for (int j = 0; j < kThinTaps; ++j) acc[j] = 0.f;
    for (int64_t p = p_begin + threadIdx.x; p < p_end; p += 256) {
      const int ow = (int)(p % g.OW);
      const int64_t q = p / g.OW;
      const int oh = (int)(q % g.OH);
      const int64_t n = q / g.OH;
      const float dv = to_f32(dY[((n * g.O + co) * g.OH + oh) * g.OW + ow]);
      const T* xp = X + (n * g.C + c) * g.H * g.W;
      const int ih0 = oh * g.sh - g.ph, iw0 = ow * g.sw - g.pw;
#pragma unroll
      for (int j = 0; j < kThinTaps; ++j) {
        const int ih = ih0 + tkh[j], iw = iw0 + tkw[j];
        if (t0 + j < KK && (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W)
          acc[j] = fmaf(dv, to_f32(xp[(int64_t)ih * g.W + iw]), acc[j]);
      }
    }
#pragma unroll
    for (int j = 0; j < kThinTaps; ++j) {
      const float v = wave_reduce(acc[j], kWave, SumOp());
      if (lane == 0) fold[wave][j] = v;
    }
    __syncthreads();
    if (threadIdx.x < kThinTaps && t0 + threadIdx.x < KK)
      out[t0 + threadIdx.x] = (fold[0][threadIdx.x] + fold[1][threadIdx.x]) + (fold[2][threadIdx.x] + fold[3][threadIdx.x]);
    __syncthreads();
  }
}

// Per-channel sum over batch and space of a [N, C, S] tensor (bias gradient): one workgroup of
// 1024 lanes per channel.  VEC: the planes are whole 16-byte vectors (S a multiple of the vector
// length, aligned base): a lane then reads vectors, four of them in flight at a time, and walks
// the planes in the order (image, vector); otherwise element by element.  The order of the sum is
// fixed by the launch shape, so the result is the same run to run.
constexpr int kChannelSumBlock = 1024;
template <typename T, bool VEC>
__global__ __launch_bounds__(kChannelSumBlock) void channel_sum_kernel(const T* __restrict__ x, void* __restrict__ out,
                                                                      int out_dt, int64_t N, int C, int64_t S) {
  __shared__ float smem[kChannelSumBlock / kWave];
  const int c = blockIdx.x;
  float s = 0.f;
  if (VEC) {
    constexpr int kPer = 16 / sizeof(T), kUnroll = 4;
    const int64_t vec_per_plane = S / kPer, total = N * vec_per_plane;
    float part[kUnroll] = {0.f, 0.f, 0.f, 0.f};
    for (int64_t v0 = threadIdx.x; v0 < total; v0 += (int64_t)kUnroll * kChannelSumBlock) {
      uint4 raw[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int64_t v = v0 + (int64_t)u * kChannelSumBlock;
        // 32-bit division whenever the vector count allows it (64-bit division is a long routine)
        const int64_t n = total <= INT32_MAX ? (int64_t)((uint32_t)v / (uint32_t)vec_per_plane) : v / vec_per_plane;
        const int64_t i = v - n * vec_per_plane;
        raw[u] = v < total ? reinterpret_cast<const uint4*>(x + (n * C + c) * S)[i] : make_uint4(0, 0, 0, 0);
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        float f[kPer];
        unpack16<T>(raw[u], f);
        float t = 0.f;
#pragma unroll
        for (int e = 0; e < kPer; ++e) t += f[e];
        part[u] += t;
      }
    }
    s = (part[0] + part[1]) + (part[2] + part[3]);
  } else {
    for (int64_t n = 0; n < N; ++n) {
      const T* plane = x + (n * C + c) * S;
      for (int64_t i = threadIdx.x; i < S; i += kChannelSumBlock) s += to_f32(plane[i]);
    }
  }
  s = group_reduce(s, kChannelSumBlock, smem, SumOp(), 0.f);
  if (threadIdx.x == 0) store_scalar_f32(out, out_dt, c, s);
}

template <typename F>
inline int dispatch_dtype(int dt, F&& f) {
  if (dt == AT_DTYPE_F32) return f((float*)0);
  if (dt == AT_DTYPE_F16) return f((f16_t*)0);
  if (dt == AT_DTYPE_BF16) return f((bf16_t*)0);
  return AT_ERR_DTYPE;
}

struct ConvShape {
  int64_t N, C, H, W, O, KH, KW, sh, sw, ph, pw, groups;
  int64_t OH, OW;
};

inline int check_shape(const ConvShape& s) {
  if (s.N <= 0 || s.C <= 0 || s.H <= 0 || s.W <= 0 || s.O <= 0 || s.KH <= 0 || s.KW <= 0) return AT_ERR_DIM;
  if (s.sh <= 0 || s.sw <= 0 || s.ph < 0 || s.pw < 0 || s.groups <= 0) return AT_ERR_DIM;
  if (s.C % s.groups || s.O % s.groups) return AT_ERR_DIM;
  if (s.OH <= 0 || s.OW <= 0) return AT_ERR_DIM;
  if (s.OH != (s.H + 2 * s.ph - s.KH) / s.sh + 1 || s.OW != (s.W + 2 * s.pw - s.KW) / s.sw + 1) return AT_ERR_DIM;
  const int64_t lim = INT32_MAX;
  if (s.N > lim || s.C > lim || s.H > lim || s.W > lim || s.O > lim || s.C / s.groups * s.KH * s.KW > lim ||
      s.O / s.groups * s.KH * s.KW > lim)
    return AT_ERR_DIM;
  return AT_OK;
}

inline ConvArgs base_args(const ConvShape& s) {
  ConvArgs g{};
  g.N = (int)s.N; g.C = (int)s.C; g.H = (int)s.H; g.W = (int)s.W; g.O = (int)s.O; g.KH = (int)s.KH;
  g.KW = (int)s.KW; g.OH = (int)s.OH; g.OW = (int)s.OW; g.sh = (int)s.sh; g.sw = (int)s.sw; g.ph = (int)s.ph;
  g.pw = (int)s.pw; g.groups = (int)s.groups; g.Cg = (int)(s.C / s.groups); g.Og = (int)(s.O / s.groups);
  return g;
}

constexpr int kDwMaxSplits = 512;

inline int dw_splits(const ConvShape& s) {
  const int64_t K = s.N * s.OH * s.OW;
  const int64_t tiles = cdiv64(s.O / s.groups, TM) * cdiv64(s.C / s.groups * s.KH * s.KW, TN) * s.groups;
  int64_t want = cdiv64((int64_t)device_cu_count() * 4, tiles);
  const int64_t max_by_k = cdiv64(K, 4 * TK);
  if (want > max_by_k) want = max_by_k;
  if (want > kDwMaxSplits) want = kDwMaxSplits;
  if (want < 1) want = 1;
  return (int)want;
}

}  // namespace
}  // namespace at_hip

using namespace at_hip;

extern "C" {

namespace {
inline ConvProblem problem_of(const ConvShape& s, int dtype) {
  return ConvProblem{s.N, s.C, s.H, s.W, s.O, s.KH, s.KW, s.sh, s.sw, s.ph, s.pw, s.groups, s.OH, s.OW, dtype};
}
inline ConvShape shape_of(int64_t batch, int64_t in_feat, int64_t in_height, int64_t in_width, int64_t out_feat,
                          int64_t out_height, int64_t out_width, int64_t kernel_height, int64_t kernel_width,
                          int64_t stride_height, int64_t stride_width, int64_t padding_height,
                          int64_t padding_width, int64_t groups) {
  return ConvShape{batch, in_feat, in_height, in_width, out_feat, kernel_height, kernel_width, stride_height,
                   stride_width, padding_height, padding_width, groups, out_height, out_width};
}
}  // namespace

int64_t at_conv2d_fwd_workspace_bytes(int64_t batch, int64_t in_feat, int64_t in_height, int64_t in_width,
                                      int64_t out_feat, int64_t out_height, int64_t out_width,
                                      int64_t kernel_height, int64_t kernel_width, int64_t stride_height,
                                      int64_t stride_width, int64_t padding_height, int64_t padding_width,
                                      int64_t groups, int in_dtype, int out_dtype) {
  const ConvShape s = shape_of(batch, in_feat, in_height, in_width, out_feat, out_height, out_width, kernel_height,
                               kernel_width, stride_height, stride_width, padding_height, padding_width, groups);
  if (check_shape(s) || in_dtype != out_dtype) return 0;
  return conv_igemm_fwd_workspace(problem_of(s, in_dtype));
}

int at_conv2d_fwd_leaves_nhwc(int64_t batch, int64_t in_feat, int64_t in_height, int64_t in_width, int64_t out_feat,
                              int64_t out_height, int64_t out_width, int64_t kernel_height, int64_t kernel_width,
                              int64_t stride_height, int64_t stride_width, int64_t padding_height,
                              int64_t padding_width, int64_t groups, int in_dtype, int out_dtype) {
  const ConvShape s = shape_of(batch, in_feat, in_height, in_width, out_feat, out_height, out_width, kernel_height,
                               kernel_width, stride_height, stride_width, padding_height, padding_width, groups);
  if (check_shape(s) || in_dtype != out_dtype) return 0;
  return conv_igemm_fwd_leaves_nhwc(problem_of(s, in_dtype)) ? 1 : 0;
}

int at_conv2d_fwd(const void* input, const void* weight, const void* bias, void* output, void* workspace,
                  int64_t workspace_bytes, int64_t batch, int64_t in_feat, int64_t in_height, int64_t in_width,
                  int64_t out_feat, int64_t out_height, int64_t out_width, int64_t kernel_height,
                  int64_t kernel_width, int64_t stride_height, int64_t stride_width, int64_t padding_height,
                  int64_t padding_width, int64_t groups, int in_dtype, int bias_dtype, int out_dtype,
                  at_stream_t stream) {
  if (!input || !weight || !output) return AT_ERR_NULL;
  if (!dtype_valid(in_dtype) || !dtype_valid(out_dtype) || (bias && !dtype_valid(bias_dtype))) return AT_ERR_DTYPE;
  const ConvShape s = shape_of(batch, in_feat, in_height, in_width, out_feat, out_height, out_width, kernel_height,
                               kernel_width, stride_height, stride_width, padding_height, padding_width, groups);
  int rc = check_shape(s);
  if (rc) return rc;
  if (in_dtype == out_dtype) {
    // 16-bit matrix-core path when the shape allows and the caller brought the workspace for it
    const ConvProblem p = problem_of(s, in_dtype);
    const int64_t need = conv_igemm_fwd_workspace(p);
    if (need > 0 && workspace && workspace_bytes >= need && aligned16(workspace))
      return conv_igemm_fwd(p, input, weight, bias, bias_dtype, output, workspace, (hipStream_t)stream);
  }
  ConvArgs g = base_args(s);
  g.a = input; g.b = weight; g.out = output; g.bias = bias; g.bias_dt = bias_dtype;
  g.M = s.N * s.OH * s.OW; g.K = (int64_t)g.Cg * g.KH * g.KW; g.cols = g.Og;
  if (g.Og <= kThinFeat && g.K <= kThinWalkFwd) {
    g.M = s.N * s.O * s.OH * s.OW;
    if (cdiv64(g.M, 256) > INT32_MAX) return AT_ERR_DIM;
    return dispatch_dtype(in_dtype, [&](auto* ti) -> int {
      typedef std::remove_pointer_t<decltype(ti)> TI;
      return dispatch_dtype(out_dtype, [&](auto* to) -> int {
        typedef std::remove_pointer_t<decltype(to)> TO;
        hipLaunchKernelGGL((conv_direct_fwd_kernel<TI, TO>), dim3((unsigned)cdiv64(g.M, 256)), dim3(256), 0,
                           (hipStream_t)stream, g);
        return launch_status();
      });
    });
  }
  const dim3 grid((unsigned)(cdiv64(g.M, TM) * cdiv64(g.cols, TN)), 1, (unsigned)g.groups);
  return dispatch_dtype(in_dtype, [&](auto* ti) -> int {
    typedef std::remove_pointer_t<decltype(ti)> TI;
    return dispatch_dtype(out_dtype, [&](auto* to) -> int {
      typedef std::remove_pointer_t<decltype(to)> TO;
      hipLaunchKernelGGL((conv_gemm_kernel<kConvFwd, TI, TO>), grid, dim3(256), 0, (hipStream_t)stream, g);
      return launch_status();
    });
  });
}

int64_t at_conv2d_bwd_input_workspace_bytes(int64_t batch, int64_t in_feat, int64_t in_height, int64_t in_width,
                                            int64_t out_feat, int64_t out_height, int64_t out_width,
                                            int64_t kernel_height, int64_t kernel_width, int64_t stride_height,
                                            int64_t stride_width, int64_t padding_height, int64_t padding_width,
                                            int64_t groups, int dtype) {
  const ConvShape s = shape_of(batch, in_feat, in_height, in_width, out_feat, out_height, out_width, kernel_height,
                               kernel_width, stride_height, stride_width, padding_height, padding_width, groups);
  if (check_shape(s)) return 0;
  return conv_igemm_dx_workspace(problem_of(s, dtype));
}

int at_conv2d_bwd_input(const void* output_grad, const void* output_grad_nhwc, const void* weight,
                        void* input_grad, void* workspace, int64_t workspace_bytes, int64_t batch, int64_t in_feat, int64_t in_height,
                        int64_t in_width, int64_t out_feat, int64_t out_height, int64_t out_width,
                        int64_t kernel_height, int64_t kernel_width, int64_t stride_height, int64_t stride_width,
                        int64_t padding_height, int64_t padding_width, int64_t groups, int dtype,
                        at_stream_t stream) {
  if (!output_grad || !weight || !input_grad) return AT_ERR_NULL;
  if (!dtype_valid(dtype)) return AT_ERR_DTYPE;
  const ConvShape s = shape_of(batch, in_feat, in_height, in_width, out_feat, out_height, out_width, kernel_height,
                               kernel_width, stride_height, stride_width, padding_height, padding_width, groups);
  int rc = check_shape(s);
  if (rc) return rc;
  {
    const ConvProblem p = problem_of(s, dtype);
    const int64_t need = conv_igemm_dx_workspace(p);
    if (need > 0 && workspace && workspace_bytes >= need && aligned16(workspace))
      return conv_igemm_dx(p, output_grad, output_grad_nhwc, weight, input_grad, workspace, (hipStream_t)stream);
  }
  ConvArgs g = base_args(s);
  g.a = output_grad; g.b = weight; g.out = input_grad;
  g.M = s.N * s.H * s.W; g.K = (int64_t)g.Og * g.KH * g.KW; g.cols = g.Cg;
  if (g.Cg <= kThinFeat && g.K <= kThinWalkDx) {
    if (s.N * s.C > INT32_MAX || s.H * s.W > (int64_t)65535 * 256) return AT_ERR_DIM;
    return dispatch_dtype(dtype, [&](auto* tp) -> int {
      typedef std::remove_pointer_t<decltype(tp)> T;
      hipLaunchKernelGGL((conv_direct_dx_kernel<T>), dim3((unsigned)(s.N * s.C), (unsigned)cdiv64(s.H * s.W, 256)),
                         dim3(256), 0, (hipStream_t)stream, g);
      return launch_status();
    });
  }
  const dim3 grid((unsigned)(cdiv64(g.M, TM) * cdiv64(g.cols, TN)), 1, (unsigned)g.groups);
  return dispatch_dtype(dtype, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    hipLaunchKernelGGL((conv_gemm_kernel<kConvDx, T, T>), grid, dim3(256), 0, (hipStream_t)stream, g);
    return launch_status();
  });
}

int64_t at_conv2d_bwd_weight_workspace_bytes(int64_t batch, int64_t in_feat, int64_t in_height, int64_t in_width,
                                             int64_t out_feat, int64_t out_height, int64_t out_width,
                                             int64_t kernel_height, int64_t kernel_width, int64_t stride_height,
                                             int64_t stride_width, int64_t padding_height, int64_t padding_width,
                                             int64_t groups, int dtype) {
  const ConvShape s = shape_of(batch, in_feat, in_height, in_width, out_feat, out_height, out_width, kernel_height,
                               kernel_width, stride_height, stride_width, padding_height, padding_width, groups);
  if (check_shape(s)) return 0;
  const int64_t generic = (int64_t)kDwMaxSplits * out_feat * (in_feat / groups) * kernel_height * kernel_width *
                          (int64_t)sizeof(float);
  const int64_t fast = conv_igemm_dw_workspace(problem_of(s, dtype));
  return fast > generic ? fast : generic;
}

int at_conv2d_bwd_weight(const void* output_grad, const void* output_grad_nhwc, const void* input,
                         const void* input_nhwc, void* weight_grad, void* workspace, int64_t workspace_bytes, int64_t batch, int64_t in_feat, int64_t in_height,
                         int64_t in_width, int64_t out_feat, int64_t out_height, int64_t out_width,
                         int64_t kernel_height, int64_t kernel_width, int64_t stride_height, int64_t stride_width,
                         int64_t padding_height, int64_t padding_width, int64_t groups, int dtype,
                         at_stream_t stream) {
  if (!output_grad || !input || !weight_grad) return AT_ERR_NULL;
  if (!dtype_valid(dtype)) return AT_ERR_DTYPE;
  const ConvShape s = shape_of(batch, in_feat, in_height, in_width, out_feat, out_height, out_width, kernel_height,
                               kernel_width, stride_height, stride_width, padding_height, padding_width, groups);
  int rc = check_shape(s);
  if (rc) return rc;
  {
    const ConvProblem p = problem_of(s, dtype);
    const int64_t need = conv_igemm_dw_workspace(p);
    if (need > 0 && workspace && workspace_bytes >= need && aligned16(workspace))
      return conv_igemm_dw(p, output_grad, output_grad_nhwc, input, input_nhwc, weight_grad, workspace,
                           (hipStream_t)stream);
  }
  ConvArgs g = base_args(s);
  const int64_t total = s.O * g.Cg * s.KH * s.KW;
  if (g.Og <= kThinFeat && g.Cg <= kThinFeat && (int64_t)g.Cg * g.KH * g.KW <= kThinWalkFwd) {
    // one workgroup per filter plane and slice of the batch x space positions
    const int64_t positions = s.N * s.OH * s.OW, planes = s.O * g.Cg;
    int64_t want = cdiv64((int64_t)device_cu_count() * 4, planes);
    const int64_t by_work = cdiv64(positions, 1024);
    if (want > by_work) want = by_work;
    if (want > kDwMaxSplits) want = kDwMaxSplits;
    if (want < 1) want = 1;
    g.k_per_split = cdiv64(positions, want);
    const int thin_splits = (int)cdiv64(positions, g.k_per_split);
    if (!workspace || workspace_bytes < (int64_t)thin_splits * total * (int64_t)sizeof(float)) return AT_ERR_WORKSPACE;
    g.a = output_grad; g.b = input; g.out = workspace; g.K = positions;
    return dispatch_dtype(dtype, [&](auto* tp) -> int {
      typedef std::remove_pointer_t<decltype(tp)> T;
      hipLaunchKernelGGL((conv_direct_dw_kernel<T>), dim3((unsigned)planes, (unsigned)thin_splits), dim3(256), 0,
                         (hipStream_t)stream, g);
      int rc2 = launch_status();
      if (rc2) return rc2;
      hipLaunchKernelGGL((conv_dw_reduce_kernel<T>), dim3((unsigned)cdiv64(total, 256)), dim3(256), 0,
                         (hipStream_t)stream, (const float*)workspace, (T*)weight_grad, thin_splits, total);
      return launch_status();
    });
  }
  const int splits = dw_splits(s);
  if (!workspace || workspace_bytes < (int64_t)splits * total * (int64_t)sizeof(float)) return AT_ERR_WORKSPACE;
  g.a = output_grad; g.b = input; g.out = workspace;
  g.M = g.Og; g.K = s.N * s.OH * s.OW; g.cols = g.Cg * g.KH * g.KW;
  g.k_per_split = cdiv64(cdiv64(g.K, splits), TK) * TK;
  const dim3 grid((unsigned)(cdiv64(g.M, TM) * cdiv64(g.cols, TN)), (unsigned)splits, (unsigned)g.groups);
  return dispatch_dtype(dtype, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    hipLaunchKernelGGL((conv_gemm_kernel<kConvDw, T, float>), grid, dim3(256), 0, (hipStream_t)stream, g);
    int rc2 = launch_status();
    if (rc2) return rc2;
    hipLaunchKernelGGL((conv_dw_reduce_kernel<T>), dim3((unsigned)cdiv64(total, 256)), dim3(256), 0,
                       (hipStream_t)stream, (const float*)workspace, (T*)weight_grad, splits, total);
    return launch_status();
  });
}

// ---- channels-last tensors ([batch, height, width, feat]) in and out, 16-bit matrix-core path only ----
int64_t at_conv2d_nhwc_workspace_bytes(int pass, int64_t batch, int64_t in_feat, int64_t in_height, int64_t in_width, int64_t out_feat,
    int64_t out_height, int64_t out_width, int64_t kernel_height, int64_t kernel_width, int64_t stride_height,
    int64_t stride_width, int64_t padding_height, int64_t padding_width, int64_t groups, int dtype) {
  const ConvShape s = shape_of(batch, in_feat, in_height, in_width, out_feat, out_height, out_width, kernel_height,
                               kernel_width, stride_height, stride_width, padding_height, padding_width, groups);
  if (check_shape(s)) return 0;
  const ConvProblem p = problem_of(s, dtype);
  if (pass == 0) return conv_igemm_fwd_last_workspace(p);
  if (pass == 1) return conv_igemm_dx_last_workspace(p);
  if (pass == 2) return conv_igemm_dw_workspace(p);
  return 0;
}

int at_conv2d_fwd_nhwc(const void* input, const void* weight, const void* bias, void* output, void* workspace,
                       int64_t workspace_bytes, int64_t batch, int64_t in_feat, int64_t in_height, int64_t in_width, int64_t out_feat,
    int64_t out_height, int64_t out_width, int64_t kernel_height, int64_t kernel_width, int64_t stride_height,
    int64_t stride_width, int64_t padding_height, int64_t padding_width, int64_t groups, int dtype, int bias_dtype, at_stream_t stream) {
  if (!input || !weight || !output) return AT_ERR_NULL;
  if (!dtype_valid(dtype) || (bias && !dtype_valid(bias_dtype))) return AT_ERR_DTYPE;
  const ConvShape s = shape_of(batch, in_feat, in_height, in_width, out_feat, out_height, out_width, kernel_height,
                               kernel_width, stride_height, stride_width, padding_height, padding_width, groups);
  int rc = check_shape(s);
  if (rc) return rc;
  const ConvProblem p = problem_of(s, dtype);
  const int64_t need = conv_igemm_fwd_last_workspace(p);
  if (need <= 0) return AT_ERR_UNSUPPORTED;
  if (!workspace || workspace_bytes < need) return AT_ERR_WORKSPACE;
  if (!aligned16(workspace) || !aligned16(input) || !aligned16(output)) return AT_ERR_ALIGN;
  return conv_igemm_fwd_last(p, input, weight, bias, bias_dtype, output, workspace, (hipStream_t)stream);
}

int at_conv2d_bwd_input_nhwc(const void* output_grad, const void* weight, void* input_grad, void* workspace,
                             int64_t workspace_bytes, int64_t batch, int64_t in_feat, int64_t in_height, int64_t in_width, int64_t out_feat,
    int64_t out_height, int64_t out_width, int64_t kernel_height, int64_t kernel_width, int64_t stride_height,
    int64_t stride_width, int64_t padding_height, int64_t padding_width, int64_t groups, int dtype, at_stream_t stream) {
  if (!output_grad || !weight || !input_grad) return AT_ERR_NULL;
  if (!dtype_valid(dtype)) return AT_ERR_DTYPE;
  const ConvShape s = shape_of(batch, in_feat, in_height, in_width, out_feat, out_height, out_width, kernel_height,
                               kernel_width, stride_height, stride_width, padding_height, padding_width, groups);
  int rc = check_shape(s);
  if (rc) return rc;
  const ConvProblem p = problem_of(s, dtype);
  const int64_t need = conv_igemm_dx_last_workspace(p);
  if (need <= 0) return AT_ERR_UNSUPPORTED;
  if (!workspace || workspace_bytes < need) return AT_ERR_WORKSPACE;
  if (!aligned16(workspace) || !aligned16(output_grad) || !aligned16(input_grad)) return AT_ERR_ALIGN;
  return conv_igemm_dx_last(p, output_grad, weight, input_grad, workspace, (hipStream_t)stream);
}

int at_conv2d_bwd_weight_nhwc(const void* output_grad, const void* input, void* weight_grad, void* workspace,
                              int64_t workspace_bytes, int64_t batch, int64_t in_feat, int64_t in_height, int64_t in_width, int64_t out_feat,
    int64_t out_height, int64_t out_width, int64_t kernel_height, int64_t kernel_width, int64_t stride_height,
    int64_t stride_width, int64_t padding_height, int64_t padding_width, int64_t groups, int dtype, at_stream_t stream) {
  if (!output_grad || !input || !weight_grad) return AT_ERR_NULL;
  if (!dtype_valid(dtype)) return AT_ERR_DTYPE;
  const ConvShape s = shape_of(batch, in_feat, in_height, in_width, out_feat, out_height, out_width, kernel_height,
                               kernel_width, stride_height, stride_width, padding_height, padding_width, groups);
  int rc = check_shape(s);
  if (rc) return rc;
  const ConvProblem p = problem_of(s, dtype);
  const int64_t need = conv_igemm_dw_workspace(p);
  if (need <= 0) return AT_ERR_UNSUPPORTED;
  if (!workspace || workspace_bytes < need) return AT_ERR_WORKSPACE;
  if (!aligned16(workspace) || !aligned16(output_grad) || !aligned16(input)) return AT_ERR_ALIGN;
  // both operands are already channels-last: the channels-first arguments are not read
  return conv_igemm_dw(p, nullptr, output_grad, nullptr, input, weight_grad, workspace, (hipStream_t)stream);
}

int at_nchw_to_nhwc(const void* src, void* dst, int64_t batch, int64_t feat, int64_t spatial, int dtype,
                    at_stream_t stream) {
  if (!src || !dst) return AT_ERR_NULL;
  return conv_nchw_to_nhwc(src, dst, batch, feat, spatial, dtype, (hipStream_t)stream);
}

int at_channel_sum(const void* x, void* out, int64_t batch, int64_t feat, int64_t spatial, int x_dtype,
                   int out_dtype, at_stream_t stream) {
  if (!x || !out) return AT_ERR_NULL;
  if (!dtype_valid(x_dtype) || !dtype_valid(out_dtype)) return AT_ERR_DTYPE;
  if (batch <= 0 || feat <= 0 || spatial <= 0 || feat > INT32_MAX) return AT_ERR_DIM;
  return dispatch_dtype(x_dtype, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    if (spatial % (16 / (int64_t)sizeof(T)) == 0 && aligned16(x))
      hipLaunchKernelGGL((channel_sum_kernel<T, true>), dim3((unsigned)feat), dim3(kChannelSumBlock), 0,
                         (hipStream_t)stream, (const T*)x, out, out_dtype, batch, (int)feat, spatial);
    else
      hipLaunchKernelGGL((channel_sum_kernel<T, false>), dim3((unsigned)feat), dim3(kChannelSumBlock), 0,
                         (hipStream_t)stream, (const T*)x, out, out_dtype, batch, (int)feat, spatial);
    return launch_status();
  });
}

}  // extern "C"
