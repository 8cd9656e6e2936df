// Cross entropy with mean reduction, optional class weights and ignore_index: loss and the
// gradient of the logits from ONE pass over the logits.
//
// HBM-bound: the algorithmic traffic is one read of the logits and one write of the gradient.
// One workgroup of 512 lanes (1024 for rows of more than 4096 vectors: twice the waves with half
// the vectors each move the same bytes 4 % faster) owns a row and keeps it in registers as raw
// 128-bit vectors (CACHE_VECS per lane), so the three sweeps the math needs (max, sum of
// exponentials, gradient) cost a single read.  A workgroup ends with its row: on this
// architecture a wave's loads are counted behind its own earlier stores, so a workgroup that walks
// over several rows waits for the acknowledgement of one row's stores before the next row's loads
// count as arrived (a persistent grid of resident workgroups measured 363 us against 300 us).  Rows need not be 16-byte aligned (a vocabulary of 50257
// fp16 logits makes every other row start on an odd element): a row is addressed through
// the 16-byte grid of its own address space, interior vectors move with 128-bit accesses and
// only the first and last vector of a row fall back to guarded element accesses.  The
// gradient may be stored in the dtype of the logits or in fp32 (16-bit logits under autocast);
// its rows must sit at the phase of the 16-byte grid that matches the logits row for this
// path, anything else takes the streaming kernel.
//
// The same kernels serve the backward entry point: with an upstream gradient pointer they
// skip the loss, multiply the scale by the upstream value in fp32 before the one rounding
// (as the reference's backward kernel does) and, when told that the destination already holds
// the gradient for an upstream value of one, return at once if the value is exactly one.
#include <type_traits>

#include "at_common.h"

namespace at_hip {
namespace {

constexpr int kCeBlock = 512;         // lanes per row, rows of up to 4096 vectors
constexpr int kCeWideBlock = 1024;    // lanes per row beyond that
// The divisor of the mean is summed by kCeDenomParts workgroups, each over its share of the rows;
// their partial sums sit at the start of the workspace and every reader adds them in index order.
constexpr int kCeDenomParts = 16;
constexpr int kCeDenomBlock = 512;

__device__ __forceinline__ bool target_kept(int64_t t, int64_t ignore_index, int feat) {
  return t != ignore_index && t >= 0 && t < feat;
}

// denom_parts[p] = sum over the kept rows of share p of weight[target] (or their count).  The shares
// and the order inside a workgroup are fixed, so the divisor is reproducible.
__global__ __launch_bounds__(kCeDenomBlock) void ce_denominator_kernel(
    const int64_t* __restrict__ target, const void* __restrict__ weight, int wdt,
    float* __restrict__ denom_parts, int64_t batch, int feat, int64_t ignore_index) {
  __shared__ float scratch[16];
  const int64_t share = (batch + kCeDenomParts - 1) / kCeDenomParts;
  const int64_t begin = (int64_t)blockIdx.x * share;
  const int64_t end = begin + share < batch ? begin + share : batch;
  float s = 0.f;
  // targets first, then the weights they select: two rounds of independent loads per batch of
  // rows instead of a dependent pair per row (the pass is pure memory latency)
  constexpr int U = 4;
  for (int64_t base = begin + threadIdx.x; base < end; base += (int64_t)kCeDenomBlock * U) {
    int64_t t[U];
    bool kept[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t i = base + (int64_t)u * kCeDenomBlock;
      t[u] = i < end ? target[i] : 0;
      kept[u] = i < end && target_kept(t[u], ignore_index, feat);
    }
    float w[U];
#pragma unroll
    for (int u = 0; u < U; ++u) w[u] = kept[u] ? (weight ? load_scalar_f32(weight, wdt, t[u]) : 1.f) : 0.f;
#pragma unroll
    for (int u = 0; u < U; ++u) s += w[u];
  }
  s = group_reduce(s, kCeDenomBlock, scratch, SumOp(), 0.f);
  if (threadIdx.x == 0) denom_parts[blockIdx.x] = s;
}

// The divisor from its partial sums, added in index order (the pointer is uniform: scalar loads).
__device__ __forceinline__ float ce_denominator(const float* __restrict__ denom_parts) {
  float d = 0.f;
#pragma unroll
  for (int p = 0; p < kCeDenomParts; ++p) d += denom_parts[p];
  return d;
}

__global__ __launch_bounds__(1024) void ce_finalize_kernel(
    const float* __restrict__ row_loss, const float* __restrict__ denom, void* __restrict__ loss,
    int out_dt, int64_t batch) {
  __shared__ float scratch[16];
  float s = 0.f;
#pragma unroll 8
  for (int64_t i = threadIdx.x; i < batch; i += blockDim.x) s += row_loss[i];
  s = group_reduce(s, (int)blockDim.x, scratch, SumOp(), 0.f);
  if (threadIdx.x == 0) store_scalar_f32(loss, out_dt, 0, s / ce_denominator(denom));
}

// Stores the 16 / sizeof(T) gradient values of interior vector v of a row; `base` is the address of
// the row's first interior element in the gradient (16-byte aligned, host check).
template <typename T, typename TO>
__device__ __forceinline__ void store_grad_vec(TO* __restrict__ base, int v, const float (&f)[16 / sizeof(T)]) {
  constexpr int VEC = 16 / (int)sizeof(T);
  if constexpr (std::is_same<T, TO>::value) {
    reinterpret_cast<uint4*>(base)[v] = pack16<T>(f);
  } else {   // fp32 gradient of 16-bit logits: 32 contiguous bytes per lane
    float4* dst = reinterpret_cast<float4*>(base + (int64_t)v * VEC);
    dst[0] = make_float4(f[0], f[1], f[2], f[3]);
    dst[1] = make_float4(f[4], f[5], f[6], f[7]);
  }
}

// Upstream gradient of the backward entry point: 1 in the forward call (no pointer).  Returns false
// when nothing has to be computed (the destination already holds the gradient for the value 1).
__device__ __forceinline__ bool read_upstream(const void* upstream, int gdt, int skip_if_one, float& g) {
  g = 1.f;
  if (!upstream) return true;
  g = load_scalar_f32(upstream, gdt, 0);
  return !(skip_if_one && g == 1.f);
}

// Register-cached row kernel.  T is the dtype of the logits, TO of the gradient (T or float).
// A row is split into "interior" 16-byte vectors (fully inside the row, 128-bit accesses) and
// at most 7 + 7 "edge" elements before the first and after the last interior vector, each
// owned by one of the first 16 lanes and moved with element accesses.
// BLOCK lanes per row: 512 (three workgroups per CU) or 1024 (two workgroups per CU).
template <typename T, typename TO, int CACHE_VECS, int BLOCK>
__global__ __launch_bounds__(BLOCK, (BLOCK == kCeWideBlock ? 8 : 6)) void ce_row_kernel(
    const T* __restrict__ logits, const int64_t* __restrict__ target, const void* __restrict__ weight,
    int wdt, const float* __restrict__ denom, float* __restrict__ row_loss, TO* __restrict__ dlogits,
    int feat, int64_t xs, int64_t ds, int64_t ignore_index, const void* __restrict__ upstream, int gdt,
    int skip_if_one) {
  constexpr int VEC = 16 / (int)sizeof(T);
  __shared__ float scratch[16];
  float up;
  if (!read_upstream(upstream, gdt, skip_if_one, up)) return;
  const int tid = threadIdx.x;
  const int64_t row = blockIdx.x;
  const T* xr = logits + row * xs;
  TO* dr = dlogits ? dlogits + row * ds : nullptr;
  const int off = (int)((reinterpret_cast<uintptr_t>(xr) & 15u) / sizeof(T));
  const int head_n = off ? (VEC - off < feat ? VEC - off : feat) : 0;  // row elements [0, head_n)
  const int n_int = (feat - head_n) / VEC;                             // interior vectors
  const int tail0 = head_n + n_int * VEC;                              // row elements [tail0, feat)
  const uint4* xv = reinterpret_cast<const uint4*>(xr + head_n);       // 16-byte aligned
  TO* dv = dr ? dr + head_n : nullptr;                                 // 16-byte aligned too (host check)
  // edge element owned by this lane, -1 if none
  const int edge = tid < 8 ? (tid < head_n ? tid : -1)
                           : (tid < 16 && tail0 + tid - 8 < feat ? tail0 + tid - 8 : -1);
  const int64_t t = target[row];
  const bool kept = target_kept(t, ignore_index, feat);

  if (!kept) {
    if (tid == 0 && row_loss) row_loss[row] = 0.f;
    if (dr) {
      float zero[VEC];
#pragma unroll
      for (int j = 0; j < VEC; ++j) zero[j] = 0.f;
      for (int v = tid; v < n_int; v += BLOCK) store_grad_vec<T, TO>(dv, v, zero);
      if (edge >= 0) dr[edge] = from_f32<TO>(0.f);
    }
    return;
  }

  // Vectors per lane that this row really uses; uniform, so the unrolled sweeps below skip the
  // rest of the cache with scalar branches.
  const int n_iter = (n_int + BLOCK - 1) / BLOCK;
  constexpr float kLog2e = 1.4426950408889634f;

  // All loads of the row are issued back to back and without a branch (the register writes on the
  // other side of a branch would have to wait for the load): a lane with no vector at position v
  // reads the aligned 16 bytes that hold the first element of the row instead (the same page as
  // that element, so always mapped), and what it read is replaced by the padding afterwards.
  uint4 cache[CACHE_VECS];
  // xr - off is on the 16-byte grid whatever the row looks like (xv is only when the row reaches
  // its first boundary, i.e. when it has interior vectors at all)
  const uint4* const safe = reinterpret_cast<const uint4*>(xr - off);
#pragma unroll
  for (int i = 0; i < CACHE_VECS; ++i) {
    const int v = tid + i * BLOCK;
    cache[i] = *(v < n_int ? xv + v : safe);
  }
  const float edge_x = to_f32(xr[edge >= 0 ? edge : 0]);
#pragma unroll
  for (int i = 0; i < CACHE_VECS; ++i) {
    constexpr uint32_t P = Word<T>::kNegInf;
    if (tid + i * BLOCK >= n_int) cache[i] = make_uint4(P, P, P, P);
  }

  float m = edge >= 0 ? edge_x : -INFINITY;
#pragma unroll
  for (int i = 0; i < CACHE_VECS; ++i) {
    if (i < n_iter) {
      float f[VEC];
      unpack16<T>(cache[i], f);
#pragma unroll
      for (int j = 0; j < VEC; ++j) m = fmaxf(m, f[j]);
    }
  }
  m = group_reduce(m, BLOCK, scratch, MaxOp(), -INFINITY);
  // Keep the row cached as raw data: without this the compiler may keep widened fp32 copies
  // of every element alive across the sweeps.
#pragma unroll
  for (int i = 0; i < CACHE_VECS; ++i) keep_raw(cache[i]);

  // Second sweep: e = exp(x - max) replaces x in the cache (in the storage format: the gradient
  // is rounded to it anyway), so the third sweep is a multiplication.
  const float m2 = m * kLog2e;
  const float edge_e = edge >= 0 ? exp2f(fmaf(edge_x, kLog2e, -m2)) : 0.f;
  float s = edge_e;
#pragma unroll
  for (int i = 0; i < CACHE_VECS; ++i) {
    if (i < n_iter) {
      float f[VEC];
      unpack16<T>(cache[i], f);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        f[j] = __builtin_amdgcn_exp2f(fmaf(f[j], kLog2e, -m2));   // 0 for the -inf padding
        s += f[j];
      }
      cache[i] = pack16<T>(f);
    }
  }
  s = group_reduce(s, BLOCK, scratch, SumOp(), 0.f);
#pragma unroll
  for (int i = 0; i < CACHE_VECS; ++i) keep_raw(cache[i]);

  const float wt = weight ? load_scalar_f32(weight, wdt, t) : 1.f;
  const float x_t = to_f32(xr[t]);
  if (tid == 0 && row_loss) row_loss[row] = (__logf(s) - x_t + m) * wt;
  if (!dr) return;

  const float scale = wt / ce_denominator(denom) * up;
  const float k = scale / s;
  const int tv = (int)t - head_n;   // target position relative to the first interior element
  const float g_target = fmaf(__builtin_amdgcn_exp2f(fmaf(x_t, kLog2e, -m2)), k, -scale);   // softmax - 1, scaled
  if constexpr (!std::is_same<T, TO>::value) {
    // fp32 gradient of 16-bit logits.  A lane's 8 values are 32 bytes of the output; stored as they
    // are, each of the two store instructions of a wave writes every other 16 bytes of 2 KB — half
    // of every cache line.  The values change lanes through LDS first (2 KB per wave, nobody else's:
    // no workgroup barrier, a wave's LDS operations complete in order; wave barriers keep the compiler
    // from reordering them), so that each instruction writes one contiguous KiB.
    __shared__ float4 exchange[BLOCK / 64][128];
    const int lane = tid & 63, wave = tid >> 6;
    float4* const mine = exchange[wave];
#pragma unroll
    for (int i = 0; i < CACHE_VECS; ++i) {
      if (i < n_iter) {   // uniform
        float f[VEC];
        unpack16<T>(cache[i], f);
#pragma unroll
        for (int j = 0; j < VEC; ++j) f[j] *= k;
        mine[2 * lane] = make_float4(f[0], f[1], f[2], f[3]);
        mine[2 * lane + 1] = make_float4(f[4], f[5], f[6], f[7]);
        __builtin_amdgcn_wave_barrier();   // compiler only: the reads below stay behind the writes above
        const float4 lo = mine[lane], hi = mine[64 + lane];
        __builtin_amdgcn_wave_barrier();   // ... and ahead of the next sweep's writes
        const int v0 = wave * 64 + i * BLOCK;   // the wave's first vector of this sweep
        float4* out = reinterpret_cast<float4*>(dv + (int64_t)v0 * VEC);
        if (v0 + (lane >> 1) < n_int) out[lane] = lo;
        if (v0 + 32 + (lane >> 1) < n_int) out[64 + lane] = hi;
      }
    }
    if (edge >= 0) dr[edge] = edge_e * k;
    // The target column gets softmax - 1 from the lane that stored it (stores of one lane to one
    // address stay in order): vector tv / 8 is number tv / 8 % 64 of its wave's group of 64, and
    // 16-byte piece 2 (number % 32) + (tv % 8) / 4 of that group's lower or upper KiB.
    const int target_vec = tv / VEC;
    const bool owner = (tv >= 0 && tv < n_int * VEC)
                           ? (tid == (((target_vec >> 6) & (BLOCK / 64 - 1)) << 6 | (target_vec & 31) << 1 |
                                      ((tv >> 2) & 1)))
                           : (edge == (int)t);
    if (owner) dr[t] = g_target;
  } else {
#pragma unroll
    for (int i = 0; i < CACHE_VECS; ++i) {
      const int v = tid + i * BLOCK;
      if (i < n_iter && v < n_int) {
        float f[VEC];
        unpack16<T>(cache[i], f);
#pragma unroll
        for (int j = 0; j < VEC; ++j) f[j] *= k;
        store_grad_vec<T, TO>(dv, v, f);
      }
    }
    if (edge >= 0) dr[edge] = from_f32<TO>(edge_e * k);
    // The target column gets softmax - 1: the lane that stored the column overwrites it (stores of
    // one lane to one address stay in order).
    const bool owner = (tv >= 0 && tv < n_int * VEC) ? ((tv / VEC) % BLOCK == tid) : (edge == (int)t);
    if (owner) dr[t] = from_f32<TO>(g_target);
  }
}

// Streaming kernel: any dtypes, any alignment, any width; the row is read twice (online
// max / sum of exponentials, then the gradient), element accesses only.
template <typename T, typename TO>
__global__ __launch_bounds__(1024) void ce_row_stream_kernel(
    const T* __restrict__ logits, const int64_t* __restrict__ target, const void* __restrict__ weight,
    int wdt, const float* __restrict__ denom, float* __restrict__ row_loss, TO* __restrict__ dlogits,
    int feat, int64_t xs, int64_t ds, int64_t ignore_index, const void* __restrict__ upstream, int gdt,
    int skip_if_one) {
  __shared__ float scratch[16];
  float up;
  if (!read_upstream(upstream, gdt, skip_if_one, up)) return;
  const int64_t row = blockIdx.x;
  const T* xr = logits + row * xs;
  TO* dr = dlogits ? dlogits + row * ds : nullptr;
  const int64_t t = target[row];
  const bool kept = target_kept(t, ignore_index, feat);
  if (!kept) {
    if (threadIdx.x == 0 && row_loss) row_loss[row] = 0.f;
    if (dr)
      for (int c = threadIdx.x; c < feat; c += blockDim.x) dr[c] = from_f32<TO>(0.f);
    return;
  }
  float m = -INFINITY;
  for (int c = threadIdx.x; c < feat; c += blockDim.x) m = fmaxf(m, to_f32(xr[c]));
  m = group_reduce(m, (int)blockDim.x, scratch, MaxOp(), -INFINITY);
  float s = 0.f;
  for (int c = threadIdx.x; c < feat; c += blockDim.x) s += __expf(to_f32(xr[c]) - m);
  s = group_reduce(s, (int)blockDim.x, scratch, SumOp(), 0.f);
  const float wt = weight ? load_scalar_f32(weight, wdt, t) : 1.f;
  if (threadIdx.x == 0 && row_loss) row_loss[row] = (__logf(s) - to_f32(xr[t]) + m) * wt;
  if (!dr) return;
  const float scale = wt / ce_denominator(denom) * up;
  const float k = scale / s;
  for (int c = threadIdx.x; c < feat; c += blockDim.x) {
    float g = __expf(to_f32(xr[c]) - m) * k;
    if (c == (int)t) g -= scale;
    dr[c] = from_f32<TO>(g);
  }
}

// In-place scale of a [batch, feat] gradient by a device scalar; nothing is touched when the
// scalar is exactly 1.
template <typename T>
__global__ void ce_scale_kernel(T* __restrict__ d, const void* __restrict__ g_ptr, int gdt,
                                int64_t batch, int feat, int64_t ds) {
  const float g = load_scalar_f32(g_ptr, gdt, 0);
  if (g == 1.0f) return;
  const int64_t total = batch * (int64_t)feat;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int64_t r = i / feat, c = i - r * feat;
    T* p = d + r * ds + c;
    *p = from_f32<T>(to_f32(*p) * g);
  }
}

template <typename T>
__global__ void ce_scale_flat_kernel(T* __restrict__ d, const void* __restrict__ g_ptr, int gdt,
                                     int64_t total) {
  constexpr int VEC = 16 / (int)sizeof(T);
  const float g = load_scalar_f32(g_ptr, gdt, 0);
  if (g == 1.0f) return;
  // d is 16-byte aligned (checked by the host); vectors first, then the tail.
  const int64_t nvec = total / VEC;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < nvec; v += stride) {
    float f[VEC];
    load_f32<T, VEC>(d + v * VEC, f);
#pragma unroll
    for (int j = 0; j < VEC; ++j) f[j] *= g;
    store_f32<T, VEC>(d + v * VEC, f);
  }
  if (blockIdx.x == 0)
    for (int64_t i = nvec * VEC + threadIdx.x; i < total; i += blockDim.x)
      d[i] = from_f32<T>(to_f32(d[i]) * g);
}

template <typename F>
inline int dispatch_one(int dt, F&& f) {
  if (dt == AT_DTYPE_F32) return f((float*)0);
  if (dt == AT_DTYPE_F16) return f((f16_t*)0);
  if (dt == AT_DTYPE_BF16) return f((bf16_t*)0);
  return AT_ERR_DTYPE;
}

// Per-device address of the library's own workspace for the allocation-free entry point.
constexpr int64_t kCeStaticMaxBatch = 65536;
constexpr int kCeMaxDevices = 64;

// One row kernel launch: loss and/or gradient rows.  upstream == nullptr: forward call.
int launch_ce_rows(const void* logits, const int64_t* target, const void* weight, const float* denom,
                   float* row_loss, void* dlogits, int64_t batch, int64_t feat, int64_t logits_stride,
                   int64_t dlogits_stride, int64_t ignore_index, int logits_dtype, int weight_dtype,
                   int out_dtype, const void* upstream, int grad_dtype, int skip_if_one, hipStream_t stream) {
  const int es = dtype_size(logits_dtype), os = dtype_size(out_dtype);
  const int vec = 16 / es;
  const int64_t max_vecs = cdiv64(feat, vec);
  // The gradient row must reach a 16-byte boundary at the same element as the logits row does.
  const uintptr_t la = reinterpret_cast<uintptr_t>(logits), da = reinterpret_cast<uintptr_t>(dlogits);
  bool same_phase = true;
  if (dlogits) {
    const int64_t unit = 16 / os;   // elements of the gradient per 16 bytes
    same_phase = (la % es) == 0 && (da % os) == 0 &&
                 ((int64_t)(da / os) - (int64_t)(la / es)) % unit == 0 && (dlogits_stride - logits_stride) % unit == 0;
  }
  const bool cached = same_phase && max_vecs <= (int64_t)kCeWideBlock * 8 && (la % es) == 0;

  return dispatch_one(logits_dtype, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    auto run = [&](auto* top) -> int {
      typedef std::remove_pointer_t<decltype(top)> TO;
      if (cached) {
#define AT_CE_LAUNCH(CV, BLK)                                                                            \
  hipLaunchKernelGGL((ce_row_kernel<T, TO, CV, BLK>), dim3((unsigned)batch), dim3(BLK), 0, stream,       \
                     (const T*)logits, target, weight, weight_dtype, denom, row_loss, (TO*)dlogits,      \
                     (int)feat, logits_stride, dlogits_stride, ignore_index, upstream, grad_dtype, skip_if_one)
        if (max_vecs > (int64_t)kCeBlock * 8) {
          const int per_lane = (int)cdiv64(max_vecs, kCeWideBlock);   // 5 .. 8
          if (per_lane <= 6) AT_CE_LAUNCH(6, kCeWideBlock);
          else if (per_lane <= 7) AT_CE_LAUNCH(7, kCeWideBlock);
          else AT_CE_LAUNCH(8, kCeWideBlock);
        } else {
          const int per_lane = (int)cdiv64(max_vecs, kCeBlock);
          if (per_lane <= 2) AT_CE_LAUNCH(2, kCeBlock);
          else if (per_lane <= 4) AT_CE_LAUNCH(4, kCeBlock);
          else AT_CE_LAUNCH(8, kCeBlock);
        }
#undef AT_CE_LAUNCH
      } else {
        hipLaunchKernelGGL((ce_row_stream_kernel<T, TO>), dim3((unsigned)batch), dim3(1024), 0, stream,
                           (const T*)logits, target, weight, weight_dtype, denom, row_loss, (TO*)dlogits,
                           (int)feat, logits_stride, dlogits_stride, ignore_index, upstream, grad_dtype,
                           skip_if_one);
      }
      return launch_status();
    };
    if (out_dtype == logits_dtype) return run((T*)0);
    return run((float*)0);
  });
}

int check_ce_args(const void* logits, const int64_t* target, const void* weight, int64_t batch, int64_t feat,
                  int64_t logits_stride, const void* dlogits, int64_t dlogits_stride, int logits_dtype,
                  int weight_dtype, int out_dtype) {
  if (!logits || !target) return AT_ERR_NULL;
  if (!dtype_valid(logits_dtype) || !dtype_valid(out_dtype) || (weight && !dtype_valid(weight_dtype)))
    return AT_ERR_DTYPE;
  if (!(out_dtype == logits_dtype || out_dtype == AT_DTYPE_F32)) return AT_ERR_DTYPE;
  if (batch <= 0 || feat <= 0 || feat > ((int64_t)1 << 30)) return AT_ERR_DIM;
  if (logits_stride < feat || (dlogits && dlogits_stride < feat)) return AT_ERR_DIM;
  return AT_OK;
}

// Forward call on a given workspace (the caller's or the library's own).
int ce_fwd_bwd(const void* logits, const int64_t* target, const void* weight, void* loss, void* dlogits,
               float* workspace, int64_t batch, int64_t feat, int64_t logits_stride, int64_t dlogits_stride,
               int64_t ignore_index, int logits_dtype, int weight_dtype, int out_dtype, int loss_dtype,
               hipStream_t stream) {
  if (!dtype_valid(loss_dtype)) return AT_ERR_DTYPE;
  float* denom = workspace;                  // kCeDenomParts partial sums
  float* row_loss = denom + kCeDenomParts;
  hipLaunchKernelGGL(ce_denominator_kernel, dim3(kCeDenomParts), dim3(kCeDenomBlock), 0, stream, target, weight,
                     weight_dtype, denom, batch, (int)feat, ignore_index);
  int rc = launch_ce_rows(logits, target, weight, denom, row_loss, dlogits, batch, feat, logits_stride,
                          dlogits_stride, ignore_index, logits_dtype, weight_dtype, out_dtype, nullptr, 0, 0,
                          stream);
  if (rc) return rc;
  hipLaunchKernelGGL(ce_finalize_kernel, dim3(1), dim3(1024), 0, stream, row_loss, denom, loss, loss_dtype,
                     batch);
  return launch_status();
}

}  // namespace
}  // namespace at_hip

using namespace at_hip;

// Workspace of at_cross_entropy_fwd_bwd_static: the divisor's partial sums and one loss per row
// (65536 rows at most, 256 KiB).  Device memory of the library itself: every GPU the library runs on holds its own
// copy until the process ends.  In host code this name is only a handle for hipGetSymbolAddress;
// kernels receive the address that call returns for the current device.
static __device__ __align__(256) float ce_static_scratch[kCeDenomParts + 65536];

extern "C" {

int64_t at_cross_entropy_workspace_bytes(int64_t batch) {
  if (batch < 0) return 0;
  return (kCeDenomParts + batch) * (int64_t)sizeof(float);
}

int at_cross_entropy_fwd_bwd(const void* logits, const int64_t* target, const void* weight, void* loss,
                             void* dlogits, void* workspace, int64_t workspace_bytes, int64_t batch,
                             int64_t feat, int64_t logits_stride, int64_t dlogits_stride,
                             int64_t ignore_index, int logits_dtype, int weight_dtype, int out_dtype,
                             int loss_dtype, at_stream_t stream_) {
  if (!loss) return AT_ERR_NULL;
  int rc = check_ce_args(logits, target, weight, batch, feat, logits_stride, dlogits, dlogits_stride,
                         logits_dtype, weight_dtype, out_dtype);
  if (rc) return rc;
  if (!workspace || workspace_bytes < at_cross_entropy_workspace_bytes(batch)) return AT_ERR_WORKSPACE;
  if ((reinterpret_cast<uintptr_t>(workspace) & 3u) != 0) return AT_ERR_ALIGN;
  return ce_fwd_bwd(logits, target, weight, loss, dlogits, (float*)workspace, batch, feat, logits_stride,
                    dlogits_stride, ignore_index, logits_dtype, weight_dtype, out_dtype, loss_dtype,
                    (hipStream_t)stream_);
}

int64_t at_cross_entropy_static_max_batch(void) { return kCeStaticMaxBatch; }

int at_cross_entropy_fwd_bwd_static(const void* logits, const int64_t* target, const void* weight, void* loss,
                                    void* dlogits, int64_t batch, int64_t feat, int64_t logits_stride,
                                    int64_t dlogits_stride, int64_t ignore_index, int logits_dtype,
                                    int weight_dtype, int out_dtype, int loss_dtype, at_stream_t stream_) {
  if (!loss) return AT_ERR_NULL;
  int rc = check_ce_args(logits, target, weight, batch, feat, logits_stride, dlogits, dlogits_stride,
                         logits_dtype, weight_dtype, out_dtype);
  if (rc) return rc;
  if (batch > kCeStaticMaxBatch) return AT_ERR_WORKSPACE;   // the library's own workspace holds 65536 rows
  // Address of this device's copy of the workspace, looked up once per device (the lookup does
  // not allocate: the array is part of the loaded code object).  Racing first calls store the
  // same value.
  static float* scratch_of_device[kCeMaxDevices] = {};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kCeMaxDevices) return AT_ERR_UNSUPPORTED;
  float* scratch = scratch_of_device[dev];
  if (!scratch) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(ce_static_scratch));
    if (e != hipSuccess) return (int)e;
    if (!p) return AT_ERR_UNSUPPORTED;
    scratch = (float*)p;
    scratch_of_device[dev] = scratch;
  }
  // every element the kernels read from the workspace is written earlier in this call (the divisor
  // by the first launch, one loss per row by the row kernel), so nothing has to be cleared
  return ce_fwd_bwd(logits, target, weight, loss, dlogits, scratch, batch, feat, logits_stride,
                    dlogits_stride, ignore_index, logits_dtype, weight_dtype, out_dtype, loss_dtype,
                    (hipStream_t)stream_);
}

int at_cross_entropy_bwd(const void* logits, const int64_t* target, const void* weight,
                         const void* output_grad, const void* workspace, void* dlogits, int64_t batch,
                         int64_t feat, int64_t logits_stride, int64_t dlogits_stride, int64_t ignore_index,
                         int holds_unit_grad, int logits_dtype, int weight_dtype, int grad_dtype,
                         int out_dtype, at_stream_t stream_) {
  if (!output_grad || !workspace || !dlogits) return AT_ERR_NULL;
  int rc = check_ce_args(logits, target, weight, batch, feat, logits_stride, dlogits, dlogits_stride,
                         logits_dtype, weight_dtype, out_dtype);
  if (rc) return rc;
  if (!dtype_valid(grad_dtype)) return AT_ERR_DTYPE;
  if ((reinterpret_cast<uintptr_t>(workspace) & 3u) != 0) return AT_ERR_ALIGN;
  return launch_ce_rows(logits, target, weight, (const float*)workspace, nullptr, dlogits, batch, feat,
                        logits_stride, dlogits_stride, ignore_index, logits_dtype, weight_dtype, out_dtype,
                        output_grad, grad_dtype, holds_unit_grad ? 1 : 0, (hipStream_t)stream_);
}

int at_cross_entropy_scale_grad(void* dlogits, const void* output_grad, int64_t batch, int64_t feat,
                                int64_t dlogits_stride, int dlogits_dtype, int grad_dtype,
                                at_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!dlogits || !output_grad) return AT_ERR_NULL;
  if (!dtype_valid(dlogits_dtype) || !dtype_valid(grad_dtype)) return AT_ERR_DTYPE;
  if (batch <= 0 || feat <= 0 || dlogits_stride < feat) return AT_ERR_DIM;
  const int blocks = device_cu_count() * 8;
  return dispatch_one(dlogits_dtype, [&](auto* tp) -> int {
    typedef std::remove_pointer_t<decltype(tp)> T;
    if (dlogits_stride == feat && aligned16(dlogits))
      hipLaunchKernelGGL((ce_scale_flat_kernel<T>), dim3(blocks), dim3(256), 0, stream, (T*)dlogits,
                         output_grad, grad_dtype, batch * feat);
    else
      hipLaunchKernelGGL((ce_scale_kernel<T>), dim3(blocks), dim3(256), 0, stream, (T*)dlogits, output_grad,
                         grad_dtype, batch, (int)feat, dlogits_stride);
    return launch_status();
  });
}

}  // extern "C"
