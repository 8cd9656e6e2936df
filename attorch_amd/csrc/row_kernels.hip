// Row-reduction kernels: RMSNorm, LayerNorm, Softmax/LogSoftmax/Softmin, forward and backward.
//
// These are HBM-bound: every element is read once and written once per pass.  A row is owned
// by a "group" of 2^k consecutive lanes (a fraction of a wave for narrow rows, one wave, or
// several waves of one workgroup for wide rows).  Each lane keeps its chunks of the row in
// registers (ITERS chunks of VEC elements, 128-bit accesses on the vector path), so the row is
// read from memory exactly once even though the math needs two or three sweeps.  Rows wider
// than the register budget use the streaming kernels, which give a row to one workgroup and
// re-read it from cache for every sweep.  Parameter gradients of the norms are accumulated per lane across a
// persistent grid, reduced across the workgroup through LDS, written as one partial row per
// workgroup and summed by a second launch in fixed order (deterministic, no atomics).
#include <map>
#include <mutex>
#include <tuple>
#include <type_traits>

#include "at_common.h"

namespace at_hip {
namespace {

// Makes an index opaque to the optimiser.  Parameter vectors do not depend on the row, so inside
// a row loop the compiler would hoist their loads out of the loop and keep them (widened to
// fp32) in registers for the whole kernel; an opaque index ties each load to its iteration.
__device__ __forceinline__ int64_t opaque_index(int64_t i) {
  int lo = (int)i;
  asm volatile("" : "+v"(lo));
  return (int64_t)lo;
}

// One chunk of a row as a lane keeps it between the sweeps of a kernel.  When the chunk is
// exactly 128 bits of storage it stays packed (4 registers for 8 bf16 / fp16 values) and is
// widened on use; otherwise it is kept as fp32.
template <typename T, int VEC, bool PACKED = (sizeof(T) * VEC == 16)>
struct Chunk;

template <typename T, int VEC>
struct Chunk<T, VEC, true> {
  uint4 raw;
  __device__ __forceinline__ void load(const T* p) { raw = *reinterpret_cast<const uint4*>(p); }
  __device__ __forceinline__ void fill(float v) {
    float f[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) f[j] = v;
    raw = pack16<T>(f);
  }
  __device__ __forceinline__ void get(float (&f)[VEC]) const { unpack16<T>(raw, f); }
  __device__ __forceinline__ void pin() { keep_raw(raw); }
};

template <typename T, int VEC>
struct Chunk<T, VEC, false> {
  float v[VEC];
  __device__ __forceinline__ void load(const T* p) { load_f32<T, VEC>(p, v); }
  __device__ __forceinline__ void fill(float x) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) v[j] = x;
  }
  __device__ __forceinline__ void get(float (&f)[VEC]) const {
#pragma unroll
    for (int j = 0; j < VEC; ++j) f[j] = v[j];
  }
  __device__ __forceinline__ void pin() {}
};

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

// group_reduce at the cost of one workgroup barrier instead of two: the slot row alternates with
// `parity`, which the caller flips after every call.  A wave writes a slot row again only after
// the barrier of the call in between, which every wave reaches after its reads of that row.
template <typename Op>
__device__ __forceinline__ float group_reduce_alt(float v, int group, float (*slots)[16], int& parity,
                                                  Op op, float identity) {
  if (group <= kWave) return wave_reduce(v, group, op);
  v = wave_reduce(v, kWave, op);
  const int wave = threadIdx.x / kWave;
  const int waves_per_group = group / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) slots[parity][wave] = v;
  __syncthreads();
  const int first = (wave / waves_per_group) * waves_per_group;
  float r = identity;
  for (int i = 0; i < waves_per_group; ++i) r = op(r, slots[parity][first + i]);
  parity ^= 1;
  return r;
}

// Sums two values over the group at the cost of one workgroup barrier.  `slots` alternates with
// `parity` from call to call: a wave can only write a slot again after passing the barrier of
// the call in between, which every wave reaches only after its reads of that slot.
__device__ __forceinline__ void group_sum2(float& a, float& b, int group, float (*slots)[16][2],
                                           int parity) {
  a = wave_reduce(a, group < kWave ? group : kWave, SumOp());
  b = wave_reduce(b, group < kWave ? group : kWave, SumOp());
  if (group <= kWave) return;
  const int wave = threadIdx.x / kWave;
  const int waves_per_group = group / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) {
    slots[parity][wave][0] = a;
    slots[parity][wave][1] = b;
  }
  __syncthreads();
  const int first = (wave / waves_per_group) * waves_per_group;
  a = 0.f;
  b = 0.f;
  for (int i = 0; i < waves_per_group; ++i) {
    a += slots[parity][first + i][0];
    b += slots[parity][first + i][1];
  }
}

// The chunks one lane holds of one row of one tensor: ITERS chunks, `group` lanes apart.
template <typename T, int VEC, int ITERS>
struct RowCache {
  Chunk<T, VEC> ch[ITERS];
  // Issues the loads of this lane's chunks of `row`, without a branch: an invalid row reads row 0
  // and a chunk past the end of the row reads chunk 0 (both exist), and mask() replaces what
  // they brought by the padding value once the row is about to be used.  A load inside a
  // divergent branch would be waited for at the end of that branch, i.e. before the next load is
  // even issued.
  __device__ __forceinline__ void load(const T* __restrict__ base, int64_t row, int64_t stride,
                                       bool valid, int lane, int group, int chunks) {
    const T* r = base + (valid ? row : 0) * stride;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int c = lane + it * group;
      ch[it].load(r + (int64_t)(c < chunks ? c : 0) * VEC);
    }
  }
  __device__ __forceinline__ void mask(bool valid, int lane, int group, int chunks, float pad) {
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int c = lane + it * group;
      if (!(valid && c < chunks)) ch[it].fill(pad);
    }
  }
  __device__ __forceinline__ void pin() {
#pragma unroll
    for (int it = 0; it < ITERS; ++it) ch[it].pin();
  }
};

// The register-cached kernels below are persistent: the grid is sized to what the machine keeps
// resident and every workgroup walks its row-blocks with a grid stride.  A row must be complete
// before any of its output can be written, so a wave that handled one row at a time would
// alternate between waiting on reads and issuing writes; instead the loads of the next row-block
// are issued before the current one is reduced and written, which keeps reads and writes of
// different rows in flight together.  Memory operations retire in order per wave, so nothing
// that the current row waits on may be issued after the prefetch: parameters are held in
// registers (packed) and per-row statistics travel with the prefetch.  The two row-blocks live
// in two register sets that swap roles from one iteration to the next (the loop body exists
// twice): copying the prefetched set into the current one would have to wait for its loads.

// ------------------------------------------------------------------------------------------
// Norm forward.  LAYER = true: LayerNorm (mean subtracted, optional bias); false: RMSNorm.
// ------------------------------------------------------------------------------------------
// PERSIST: the workgroup walks over row-blocks and requests the next one ahead; !PERSIST: one
// row-block per workgroup, nothing requested ahead (see one_shot).
template <bool LAYER, typename TX, typename TY, typename TW, int VEC, int ITERS, bool PERSIST>
__global__ __launch_bounds__(512) void norm_fwd_kernel(
    const TX* __restrict__ x, const TW* __restrict__ w, const TW* __restrict__ b,
    float* __restrict__ mean_out, float* __restrict__ rstd_out, TY* __restrict__ y,
    int64_t batch, int feat, int64_t xs, int64_t ys, float eps, int group_log2) {
  static_assert(ITERS > 0, "rows are cached in registers");
  // parameters stay in registers when a chunk of them is one 128-bit word
  constexpr bool HOIST = sizeof(TW) * VEC == 16;
  __shared__ float slots[2][16];
  int parity = 0;
  const int group = 1 << group_log2;
  const int lane = threadIdx.x & (group - 1);
  const int rpb = blockDim.x >> group_log2;
  const int rib = threadIdx.x >> group_log2;
  const int chunks = feat / VEC;
  const float inv_feat = 1.0f / (float)feat;
  const int64_t row_blocks = (batch + rpb - 1) / rpb;
  const int64_t row_step = (int64_t)gridDim.x * rpb;

  Chunk<TW, VEC> pw[HOIST ? ITERS : 1], pb[(HOIST && LAYER) ? ITERS : 1];
  if (HOIST) {
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int c = lane + it * group;
      if (w && c < chunks) pw[HOIST ? it : 0].load(w + (int64_t)c * VEC);
      else pw[HOIST ? it : 0].fill(1.f);
      if (LAYER) {
        if (w && b && c < chunks) pb[(HOIST && LAYER) ? it : 0].load(b + (int64_t)c * VEC);
        else pb[(HOIST && LAYER) ? it : 0].fill(0.f);
      }
    }
  }

  RowCache<TX, VEC, ITERS> set_a, set_b;
  {
    const int64_t row0 = (int64_t)blockIdx.x * rpb + rib;
    set_a.load(x, row0, xs, row0 < batch, lane, group, chunks);
  }
  auto step = [&](int64_t rb, RowCache<TX, VEC, ITERS>& cur, RowCache<TX, VEC, ITERS>& nxt) {
    const int64_t row = rb * rpb + rib;
    const bool valid = row < batch;
    if (PERSIST) nxt.load(x, row + row_step, xs, row + row_step < batch, lane, group, chunks);
    cur.mask(valid, lane, group, chunks, 0.f);
    if (HOIST) {   // opaque per iteration: otherwise their widening to fp32 is hoisted out of the loop
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        pw[HOIST ? it : 0].pin();
        if (LAYER) pb[(HOIST && LAYER) ? it : 0].pin();
      }
    }
    __builtin_amdgcn_sched_barrier(0);

    float s = 0.f;
    if (LAYER) {
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        float v[VEC];
        cur.ch[it].get(v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) s += v[j];
      }
    }
    const float mean = LAYER ? group_reduce_alt(s, group, slots, parity, SumOp(), 0.f) * inv_feat : 0.f;
    if (LAYER) cur.pin();   // re-widen per sweep instead of keeping the row as fp32

    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int c = lane + it * group;
      if (!LAYER || c < chunks) {   // padding is zero: harmless without a mean
        float v[VEC];
        cur.ch[it].get(v);
#pragma unroll
        for (int j = 0; j < VEC; ++j) {
          const float d = v[j] - mean;
          ss += d * d;
        }
      }
    }
    ss = group_reduce_alt(ss, group, slots, parity, SumOp(), 0.f);
    const float rstd = rsqrtf(ss * inv_feat + eps);
    cur.pin();

    if (valid && lane == 0) {
      if (LAYER && mean_out) mean_out[row] = mean;
      if (rstd_out) rstd_out[row] = rstd;
    }
    if (valid) {
      TY* yr = y + row * ys;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int c = lane + it * group;
        if (c < chunks) {
          float v[VEC];
          cur.ch[it].get(v);
#pragma unroll
          for (int j = 0; j < VEC; ++j) v[j] = (v[j] - mean) * rstd;
          if (w) {
            float wv[VEC];
            if (HOIST) pw[HOIST ? it : 0].get(wv);
            else load_f32<TW, VEC>(w + opaque_index((int64_t)c * VEC), wv);
#pragma unroll
            for (int j = 0; j < VEC; ++j) v[j] *= wv[j];
            if (LAYER && b) {
              float bv[VEC];
              if (HOIST) pb[(HOIST && LAYER) ? it : 0].get(bv);
              else load_f32<TW, VEC>(b + opaque_index((int64_t)c * VEC), bv);
#pragma unroll
              for (int j = 0; j < VEC; ++j) v[j] += bv[j];
            }
          }
          store_f32<TY, VEC>(yr + (int64_t)c * VEC, v);
        }
      }
    }
  };
  if (!PERSIST) {
    step(blockIdx.x, set_a, set_b);
    return;
  }
#pragma unroll 1
  for (int64_t rb = blockIdx.x; rb < row_blocks; rb += 2 * (int64_t)gridDim.x) {
    step(rb, set_a, set_b);
    if (rb + gridDim.x < row_blocks) step(rb + gridDim.x, set_b, set_a);
  }
}

// Streaming forward for rows too wide for the register cache: one row per workgroup, the row is
// re-read (from cache) for each sweep.
template <bool LAYER, typename TX, typename TY, int VEC>
__global__ __launch_bounds__(1024) void norm_fwd_stream_kernel(
    const TX* __restrict__ x, const void* __restrict__ w, const void* __restrict__ b,
    float* __restrict__ mean_out, float* __restrict__ rstd_out, TY* __restrict__ y, int feat,
    int64_t xs, int64_t ys, float eps, int wdt) {
  __shared__ float scratch[16];
  const int group = blockDim.x;
  const int lane = threadIdx.x;
  const int64_t row = blockIdx.x;
  const int chunks = feat / VEC;
  const float inv_feat = 1.0f / (float)feat;
  const TX* xr = x + row * xs;
  TY* yr = y + row * ys;
  float s = 0.f;
  if (LAYER) {
    for (int c = lane; c < chunks; c += group) {
      float v[VEC];
      load_f32<TX, VEC>(xr + (int64_t)c * VEC, v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) s += v[j];
    }
  }
  const float mean = LAYER ? group_reduce(s, group, scratch, SumOp(), 0.f) * inv_feat : 0.f;
  float ss = 0.f;
  for (int c = lane; c < chunks; c += group) {
    float v[VEC];
    load_f32<TX, VEC>(xr + (int64_t)c * VEC, v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float d = v[j] - mean;
      ss += d * d;
    }
  }
  ss = group_reduce(ss, group, scratch, SumOp(), 0.f);
  const float rstd = rsqrtf(ss * inv_feat + eps);
  if (lane == 0) {
    if (LAYER && mean_out) mean_out[row] = mean;
    if (rstd_out) rstd_out[row] = rstd;
  }
  for (int c = lane; c < chunks; c += group) {
    float v[VEC];
    load_f32<TX, VEC>(xr + (int64_t)c * VEC, v);
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

// ------------------------------------------------------------------------------------------
// Norm backward over a persistent grid.  Each workgroup walks row-blocks with a grid stride;
// each lane accumulates the parameter gradients of the columns it owns.
//   part_w / part_b: [gridDim.x, feat] fp32 partial rows (null when not wanted).
// Dynamic LDS: (blockDim.x - lanes per row) * VEC * ITERS floats per parameter gradient (only used
// when a workgroup holds several rows; at most 57 KB: rows of more than two chunks per lane take
// the whole workgroup).
// ------------------------------------------------------------------------------------------
constexpr bool norm_bwd_fused_tail(bool layer, int iters) { return layer || iters > 2; }

template <bool LAYER, typename TDY, typename TX, typename TDX, typename TW, int VEC, int ITERS>
// RMSNorm with at most two chunks per lane fits 128 registers, i.e. two workgroups per CU; the
// LayerNorm instance (bias gradient accumulators on top) would spill there and runs one per CU.
__global__ __launch_bounds__(512, (ITERS <= 2 && !LAYER ? 4 : 1)) void norm_bwd_kernel(
    const TDY* __restrict__ dy, const TX* __restrict__ x, const float* __restrict__ mean_in,
    const float* __restrict__ rstd_in, const TW* __restrict__ w, TDX* __restrict__ dx,
    float* __restrict__ part_w, float* __restrict__ part_b, int64_t batch, int feat,
    int64_t dys, int64_t xs, int64_t dxs, int group_log2) {
  static_assert(ITERS > 0, "rows are cached in registers");
  constexpr bool HOIST = sizeof(TW) * VEC == 16;
  // With few chunks per lane the normalised input and the scaled gradient of the first sweep stay
  // in registers as fp32 for the second; otherwise the second sweep recomputes them.
  constexpr bool KEEP = ITERS * VEC <= 16;
  // Whether the parameter gradients leave inside the workgroup's last row-block (see `step`) or
  // behind the loop.  The instances held to 128 registers (two workgroups per CU) spill in their
  // main loop with the former and keep the latter.
  constexpr bool FUSED_TAIL = norm_bwd_fused_tail(LAYER, ITERS);
  __shared__ float slots[2][16][2];
  extern __shared__ float red[];
  const int group = 1 << group_log2;
  const int lane = threadIdx.x & (group - 1);
  const int rpb = blockDim.x >> group_log2;
  const int rib = threadIdx.x >> group_log2;
  const int chunks = feat / VEC;
  const float inv_feat = 1.0f / (float)feat;
  const int64_t row_blocks = (batch + rpb - 1) / rpb;
  const int64_t row_step = (int64_t)gridDim.x * rpb;

  float acc_w[ITERS][VEC], acc_b[LAYER ? ITERS : 1][VEC];
  Chunk<TW, VEC> pw[HOIST ? ITERS : 1];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      acc_w[it][j] = 0.f;
      if (LAYER) acc_b[LAYER ? it : 0][j] = 0.f;
    }
    if (HOIST) {
      const int c = lane + it * group;
      if (w && c < chunks) pw[HOIST ? it : 0].load(w + (int64_t)c * VEC);
      else pw[HOIST ? it : 0].fill(1.f);
    }
  }

  // the row stays in registers in its storage format between the two sweeps
  struct RowSet {
    RowCache<TDY, VEC, ITERS> dy;
    RowCache<TX, VEC, ITERS> x;
    float mean, rstd;   // of an invalid row: those of row 0 (finite; its dy is masked to zero)
  };
  RowSet set_a, set_b;
  int parity = 0;
  auto fetch = [&](RowSet& t, int64_t row) {
    const bool v = row < batch;
    t.mean = LAYER ? mean_in[v ? row : 0] : 0.f;
    t.rstd = rstd_in[v ? row : 0];
    t.dy.load(dy, row, dys, v, lane, group, chunks);
    t.x.load(x, row, xs, v, lane, group, chunks);
  };
  fetch(set_a, (int64_t)blockIdx.x * rpb + rib);
  // LAST: the workgroup's last row-block.  Nothing is requested ahead, and the parameter gradients,
  // complete after its first sweep, leave in front of its stores instead of behind the loop: a
  // barrier at the end of the kernel would first wait for the acknowledgement of the last stores.
  // The row-groups after the first hand their sums over through LDS as red[value][thread - group]
  // (consecutive lanes, consecutive banks), published by the barrier of the row sums; the first
  // row-group adds them up in a fixed order and writes the workgroup's partial row.
  auto step = [&](int64_t rb, RowSet& cur, RowSet& nxt, auto last_tag) {
    constexpr bool LAST = decltype(last_tag)::value;
    const int64_t row = rb * rpb + rib;
    const bool valid = row < batch;
    if (!LAST) fetch(nxt, row + row_step);
    RowCache<TDY, VEC, ITERS>& cdy = cur.dy;
    RowCache<TX, VEC, ITERS>& cx = cur.x;
    const float mean = cur.mean, rstd = cur.rstd;
    const float shift = -mean * rstd;
    cdy.mask(valid, lane, group, chunks, 0.f);
    if (HOIST) {   // opaque per iteration: otherwise their widening to fp32 is hoisted out of the loop
#pragma unroll
      for (int it = 0; it < ITERS; ++it) pw[HOIST ? it : 0].pin();
    }
    __builtin_amdgcn_sched_barrier(0);

    // padding chunks and invalid rows hold dy = 0, so every product below vanishes for them
    float s1 = 0.f, s2 = 0.f;
    float keep_h[KEEP ? ITERS : 1][VEC], keep_g[KEEP ? ITERS : 1][VEC];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int c = lane + it * group;
      float dv[VEC], xv[VEC], wv[VEC];
      cdy.ch[it].get(dv);
      cx.ch[it].get(xv);
      if (HOIST) pw[HOIST ? it : 0].get(wv);
      else if (w && c < chunks) load_f32<TW, VEC>(w + opaque_index((int64_t)c * VEC), wv);
      else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) wv[j] = 1.f;
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        // (x - mean) * rstd; one fma where the input has 16 bits anyway (the rounded product
        // mean * rstd costs accuracy when |mean| is large next to the spread of the row)
        const float h = sizeof(TX) == 2 ? fmaf(xv[j], rstd, shift) : (xv[j] - mean) * rstd;
        const float gg = dv[j] * wv[j];
        s1 += h * gg;
        s2 += gg;
        acc_w[it][j] += dv[j] * h;
        if (LAYER) acc_b[LAYER ? it : 0][j] += dv[j];
        // Accumulate here and now: left alone, the compiler sinks these updates to the end of
        // the iteration and keeps every widened operand alive until then.
        asm volatile("" : "+v"(acc_w[it][j]));
        if (LAYER) asm volatile("" : "+v"(acc_b[LAYER ? it : 0][j]));
        if (KEEP) {
          keep_h[KEEP ? it : 0][j] = h;
          keep_g[KEEP ? it : 0][j] = gg;
        }
      }
      // one chunk at a time: keeps the widened temporaries of a single chunk live, not of all
      __builtin_amdgcn_sched_barrier(0);
    }
    const int n_out = (part_w ? 1 : 0) + ((LAYER && part_b) ? 1 : 0);
    const int others = blockDim.x - group;   // lanes of the row-groups 1 .. rpb - 1
    if (LAST && FUSED_TAIL && rib > 0) {
      for (int which = 0; which < n_out; ++which) {
        const bool is_w = (which == 0 && part_w);
#pragma unroll
        for (int it = 0; it < ITERS; ++it)
#pragma unroll
          for (int j = 0; j < VEC; ++j)
            red[((which * ITERS + it) * VEC + j) * others + (threadIdx.x - group)] =
                (is_w || !LAYER) ? acc_w[it][j] : acc_b[LAYER ? it : 0][j];
      }
    }
    group_sum2(s1, s2, group, slots, parity);
    parity ^= 1;
    if (LAST && FUSED_TAIL && n_out > 0) {
      if (rpb > 1 && group <= kWave) __syncthreads();   // the row sums of such groups pass no barrier of their own
      if (rib == 0) {
        for (int which = 0; which < n_out; ++which) {
          const bool is_w = (which == 0 && part_w);
          float* part = (is_w ? part_w : part_b) + (int64_t)blockIdx.x * feat;
#pragma unroll
          for (int it = 0; it < ITERS; ++it) {
            const int c = lane + it * group;
            float v[VEC];
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
              float sum = (is_w || !LAYER) ? acc_w[it][j] : acc_b[LAYER ? it : 0][j];
              const float* col = red + ((which * ITERS + it) * VEC + j) * others + lane;
              for (int r = 1; r < rpb; ++r) sum += col[(r - 1) * group];
              v[j] = sum;
            }
            if (c < chunks) {
#pragma unroll
              for (int j = 0; j < VEC; ++j) part[(int64_t)c * VEC + j] = v[j];
            }
          }
        }
      }
    }
    // the input gradient is rstd * (g - (h * s1 + s2) / feat); rstd / feat folded into the sums
    s1 *= inv_feat * rstd;
    s2 = LAYER ? s2 * inv_feat * rstd : 0.f;
    if (!KEEP) {
      cdy.pin();
      cx.pin();
    }

    if (valid) {
      TDX* dxr = dx + row * dxs;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int c = lane + it * group;
        if (c < chunks) {
          float o[VEC];
          if (KEEP) {
#pragma unroll
            for (int j = 0; j < VEC; ++j)
              o[j] = fmaf(keep_g[KEEP ? it : 0][j], rstd, -fmaf(keep_h[KEEP ? it : 0][j], s1, s2));
          } else {
            float dv[VEC], xv[VEC], wv[VEC];
            cdy.ch[it].get(dv);
            cx.ch[it].get(xv);
            if (HOIST) pw[HOIST ? it : 0].get(wv);
            else if (w) load_f32<TW, VEC>(w + opaque_index((int64_t)c * VEC), wv);
            else {
#pragma unroll
              for (int j = 0; j < VEC; ++j) wv[j] = 1.f;
            }
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
              const float h = sizeof(TX) == 2 ? fmaf(xv[j], rstd, shift) : (xv[j] - mean) * rstd;
              o[j] = fmaf(dv[j] * wv[j], rstd, -fmaf(h, s1, s2));
            }
          }
          store_f32<TDX, VEC>(dxr + (int64_t)c * VEC, o);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  const int64_t stride = gridDim.x;
  if constexpr (FUSED_TAIL) {
    // every workgroup has at least one row-block (the grid is no larger than their number)
#pragma unroll 1
    for (int64_t rb = blockIdx.x;; rb += 2 * stride) {
      if (rb + stride >= row_blocks) {
        step(rb, set_a, set_b, std::true_type());
        break;
      }
      step(rb, set_a, set_b, std::false_type());
      if (rb + 2 * stride >= row_blocks) {
        step(rb + stride, set_b, set_a, std::true_type());
        break;
      }
      step(rb + stride, set_b, set_a, std::false_type());
    }
  } else {
#pragma unroll 1
    for (int64_t rb = blockIdx.x; rb < row_blocks; rb += 2 * stride) {
      step(rb, set_a, set_b, std::false_type());
      if (rb + stride < row_blocks) step(rb + stride, set_b, set_a, std::false_type());
    }
  }

  if (FUSED_TAIL || (!part_w && !part_b)) return;
  // Behind the loop: fold the row-groups of this workgroup together, then emit one partial row.
  // Same hand-over through LDS, with a pair of barriers of its own.
  {
    const int n_out = (part_w ? 1 : 0) + ((LAYER && part_b) ? 1 : 0);
    const int others = blockDim.x - group;
    if (rpb > 1) {
      __syncthreads();
      if (rib > 0) {
        for (int which = 0; which < n_out; ++which) {
          const bool is_w = (which == 0 && part_w);
#pragma unroll
          for (int it = 0; it < ITERS; ++it)
#pragma unroll
            for (int j = 0; j < VEC; ++j)
              red[((which * ITERS + it) * VEC + j) * others + (threadIdx.x - group)] =
                  (is_w || !LAYER) ? acc_w[it][j] : acc_b[LAYER ? it : 0][j];
        }
      }
      __syncthreads();
    }
    if (rib == 0) {
      for (int which = 0; which < n_out; ++which) {
        const bool is_w = (which == 0 && part_w);
        float* part = (is_w ? part_w : part_b) + (int64_t)blockIdx.x * feat;
#pragma unroll
        for (int it = 0; it < ITERS; ++it) {
          const int c = lane + it * group;
          float v[VEC];
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            float sum = (is_w || !LAYER) ? acc_w[it][j] : acc_b[LAYER ? it : 0][j];
            const float* col = red + ((which * ITERS + it) * VEC + j) * others + lane;
            for (int r = 1; r < rpb; ++r) sum += col[(r - 1) * group];
            v[j] = sum;
          }
          if (c < chunks) {
#pragma unroll
            for (int j = 0; j < VEC; ++j) part[(int64_t)c * VEC + j] = v[j];
          }
        }
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
    if (w) load_param_f32<VEC>(w, wdt, opaque_index((int64_t)c * VEC), wv);
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
    if (w) load_param_f32<VEC>(w, wdt, opaque_index((int64_t)c * VEC), wv);
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

// out[f] = sum over p of part[p, f], in a fixed order.  A workgroup owns 16 columns: 4 column
// quads x 64 row slices; grid.x covers the columns in steps of 16, grid.y selects the gradient.
constexpr int kReduceCols = 16;
__global__ __launch_bounds__(256) void reduce_partials_kernel(
    const float* __restrict__ part0, float* __restrict__ out0, const float* __restrict__ part1,
    float* __restrict__ out1, int parts, int feat) {
  __shared__ float sm[64][kReduceCols + 1];
  const float* part = blockIdx.y == 0 ? part0 : part1;
  float* out = blockIdx.y == 0 ? out0 : out1;
  if (!part || !out) return;
  const int cq = threadIdx.x & 3, slice = threadIdx.x >> 2;
  const int col = blockIdx.x * kReduceCols + cq * 4;
  float a[4] = {0.f, 0.f, 0.f, 0.f};
  if (col + 3 < feat && (feat & 3) == 0 && (reinterpret_cast<uintptr_t>(part) & 15) == 0) {
#pragma unroll 4
    for (int p = slice; p < parts; p += 64) {
      const float4 v = *reinterpret_cast<const float4*>(part + (int64_t)p * feat + col);
      a[0] += v.x; a[1] += v.y; a[2] += v.z; a[3] += v.w;
    }
  } else {
    for (int p = slice; p < parts; p += 64) {
      const float* src = part + (int64_t)p * feat + col;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (col + j < feat) a[j] += src[j];
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) sm[slice][cq * 4 + j] = a[j];
  __syncthreads();
  if (threadIdx.x < kReduceCols) {
    float s = 0.f;
#pragma unroll
    for (int r = 0; r < 64; ++r) s += sm[r][threadIdx.x];
    const int c = blockIdx.x * kReduceCols + threadIdx.x;
    if (c < feat) out[c] = s;
  }
}

// ------------------------------------------------------------------------------------------
// Softmax family.
// ------------------------------------------------------------------------------------------
// MAXB: largest workgroup the instance is launched with (256 leaves the compiler 256 registers per lane).
// PERSIST as in softmax_bwd_kernel: false = one row-block per workgroup, nothing requested ahead.
template <typename TX, typename TY, int VEC, int ITERS, int MAXB, bool PERSIST>
__global__ __launch_bounds__(MAXB) void softmax_fwd_kernel(
    const TX* __restrict__ x, TY* __restrict__ y, int64_t batch, int feat, int64_t xs, int64_t ys,
    int neg, int log, int group_log2) {
  static_assert(ITERS > 0, "rows are cached in registers");
  // With few enough elements per lane the exponentials of the second sweep (the shifted logits for
  // log-softmax) stay in registers as fp32 and the third sweep is one multiplication per element;
  // otherwise the third sweep computes them again from the cached row.
  constexpr bool KEEP = ITERS * VEC <= (MAXB <= 256 ? 64 : 16);
  constexpr float kLog2e = 1.4426950408889634f, kLn2 = 0.6931471805599453f;
  __shared__ float slots[2][16];
  int parity = 0;
  const int group = 1 << group_log2;
  const int lane = threadIdx.x & (group - 1);
  const int rpb = blockDim.x >> group_log2;
  const int rib = threadIdx.x >> group_log2;
  const int chunks = feat / VEC;
  const float sign = neg ? -1.f : 1.f;
  const float scale = sign * kLog2e;    // exponentials in base 2: exp(s x - m) = exp2(x * scale - m * log2(e))
  const float pad = -sign * INFINITY;   // padding never wins the max and adds exp(-inf) = 0
  const int64_t row_blocks = (batch + rpb - 1) / rpb;
  const int64_t row_step = (int64_t)gridDim.x * rpb;

  RowCache<TX, VEC, ITERS> set_a, set_b;
  {
    const int64_t row0 = (int64_t)blockIdx.x * rpb + rib;
    set_a.load(x, row0, xs, row0 < batch, lane, group, chunks);
  }
  auto step = [&](int64_t rb, RowCache<TX, VEC, ITERS>& cur, RowCache<TX, VEC, ITERS>& nxt) {
    const int64_t row = rb * rpb + rib;
    const bool valid = row < batch;
    if (PERSIST) nxt.load(x, row + row_step, xs, row + row_step < batch, lane, group, chunks);
    cur.mask(valid, lane, group, chunks, pad);
    __builtin_amdgcn_sched_barrier(0);

    float m = -INFINITY;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      float v[VEC];
      cur.ch[it].get(v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) m = fmaxf(m, v[j] * sign);
    }
    m = group_reduce_alt(m, group, slots, parity, MaxOp(), -INFINITY);
    if (!valid) m = 0.f;   // an invalid row is all padding: keep its arithmetic finite
    cur.pin();

    const float m2 = m * kLog2e;
    float s = 0.f;
    float kept[KEEP ? ITERS : 1][VEC];
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      float v[VEC];
      cur.ch[it].get(v);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        const float t = fmaf(v[j], scale, -m2);          // (s x - m) * log2(e); -inf for padding
        const float e = __builtin_amdgcn_exp2f(t);
        s += e;
        if (KEEP) kept[KEEP ? it : 0][j] = log ? t : e;
      }
    }
    s = group_reduce_alt(s, group, slots, parity, SumOp(), 0.f);
    if (!KEEP) cur.pin();

    if (valid) {
      const float inv = 1.0f / s;
      const float lg = __logf(s);
      TY* yr = y + row * ys;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int c = lane + it * group;
        if (c < chunks) {
          float v[VEC];
          if (KEEP) {
#pragma unroll
            for (int j = 0; j < VEC; ++j)
              v[j] = log ? fmaf(kept[KEEP ? it : 0][j], kLn2, -lg) : kept[KEEP ? it : 0][j] * inv;
          } else {
            cur.ch[it].get(v);
#pragma unroll
            for (int j = 0; j < VEC; ++j) {
              const float t = fmaf(v[j], scale, -m2);
              v[j] = log ? fmaf(t, kLn2, -lg) : __builtin_amdgcn_exp2f(t) * inv;
            }
          }
          store_f32<TY, VEC>(yr + (int64_t)c * VEC, v);
        }
      }
    }
  };
  if (!PERSIST) {
    step(blockIdx.x, set_a, set_b);
    return;
  }
#pragma unroll 1
  for (int64_t rb = blockIdx.x; rb < row_blocks; rb += 2 * (int64_t)gridDim.x) {
    step(rb, set_a, set_b);
    if (rb + gridDim.x < row_blocks) step(rb + gridDim.x, set_b, set_a);
  }
}

// Streaming forward for rows too wide for the register cache: one row per workgroup.
template <typename TX, typename TY, int VEC>
__global__ __launch_bounds__(1024) void softmax_fwd_stream_kernel(
    const TX* __restrict__ x, TY* __restrict__ y, int feat, int64_t xs, int64_t ys, int neg, int log) {
  __shared__ float scratch[16];
  const int group = blockDim.x;
  const int lane = threadIdx.x;
  const int chunks = feat / VEC;
  const float sign = neg ? -1.f : 1.f;
  const TX* xr = x + (int64_t)blockIdx.x * xs;
  TY* yr = y + (int64_t)blockIdx.x * ys;
  float m = -INFINITY;
  for (int c = lane; c < chunks; c += group) {
    float v[VEC];
    load_f32<TX, VEC>(xr + (int64_t)c * VEC, v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) m = fmaxf(m, v[j] * sign);
  }
  m = group_reduce(m, group, scratch, MaxOp(), -INFINITY);
  float s = 0.f;
  for (int c = lane; c < chunks; c += group) {
    float v[VEC];
    load_f32<TX, VEC>(xr + (int64_t)c * VEC, v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) s += __expf(v[j] * sign - m);
  }
  s = group_reduce(s, group, scratch, SumOp(), 0.f);
  const float inv = 1.0f / s;
  const float lg = __logf(s);
  for (int c = lane; c < chunks; c += group) {
    float v[VEC];
    load_f32<TX, VEC>(xr + (int64_t)c * VEC, v);
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      const float d = v[j] * sign - m;
      v[j] = log ? d - lg : __expf(d) * inv;
    }
    store_f32<TY, VEC>(yr + (int64_t)c * VEC, v);
  }
}

// PERSIST: the workgroup walks over row-blocks (grid sized to the chip) and requests the next
// row-block before it reduces and stores the current one.  !PERSIST: one row-block per workgroup
// and nothing requested ahead; the grid covers the rows.
template <typename TDY, typename TY, typename TDX, int VEC, int ITERS, bool PERSIST>
__global__ __launch_bounds__(1024) void softmax_bwd_kernel(
    const TDY* __restrict__ dy, const TY* __restrict__ y, TDX* __restrict__ dx, int64_t batch,
    int feat, int64_t dys, int64_t ys, int64_t dxs, int neg, int log, int group_log2) {
  static_assert(ITERS > 0, "rows are cached in registers");
  __shared__ float slots[2][16];
  int parity = 0;
  const int group = 1 << group_log2;
  const int lane = threadIdx.x & (group - 1);
  const int rpb = blockDim.x >> group_log2;
  const int rib = threadIdx.x >> group_log2;
  const int chunks = feat / VEC;
  const float sign = neg ? -1.f : 1.f;
  const int64_t row_blocks = (batch + rpb - 1) / rpb;
  const int64_t row_step = (int64_t)gridDim.x * rpb;

  struct RowSet {
    RowCache<TDY, VEC, ITERS> dy;
    RowCache<TY, VEC, ITERS> y;
  };
  RowSet set_a, set_b;
  {
    const int64_t row0 = (int64_t)blockIdx.x * rpb + rib;
    set_a.dy.load(dy, row0, dys, row0 < batch, lane, group, chunks);
    set_a.y.load(y, row0, ys, row0 < batch, lane, group, chunks);
  }
  auto step = [&](int64_t rb, RowSet& cur, RowSet& nxt) {
    const int64_t row = rb * rpb + rib;
    const bool valid = row < batch;
    if (PERSIST) {
      nxt.dy.load(dy, row + row_step, dys, row + row_step < batch, lane, group, chunks);
      nxt.y.load(y, row + row_step, ys, row + row_step < batch, lane, group, chunks);
    }
    RowCache<TDY, VEC, ITERS>& cdy = cur.dy;
    RowCache<TY, VEC, ITERS>& cy = cur.y;
    cdy.mask(valid, lane, group, chunks, 0.f);   // dy = 0 makes every product of the padding vanish
    cy.mask(valid, lane, group, chunks, 0.f);
    __builtin_amdgcn_sched_barrier(0);

    float s = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      float dv[VEC], yv[VEC];
      cdy.ch[it].get(dv);
      cy.ch[it].get(yv);
#pragma unroll
      for (int j = 0; j < VEC; ++j) s += log ? dv[j] : dv[j] * yv[j];
    }
    s = group_reduce_alt(s, group, slots, parity, SumOp(), 0.f);
    cdy.pin();
    cy.pin();

    if (valid) {
      TDX* dxr = dx + row * dxs;
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int c = lane + it * group;
        if (c < chunks) {
          float dv[VEC], yv[VEC], o[VEC];
          cdy.ch[it].get(dv);
          cy.ch[it].get(yv);
#pragma unroll
          for (int j = 0; j < VEC; ++j)
            o[j] = sign * (log ? dv[j] - __expf(yv[j]) * s : yv[j] * (dv[j] - s));
          store_f32<TDX, VEC>(dxr + (int64_t)c * VEC, o);
        }
      }
    }
  };
  if (!PERSIST) {
    step(blockIdx.x, set_a, set_b);
    return;
  }
#pragma unroll 1
  for (int64_t rb = blockIdx.x; rb < row_blocks; rb += 2 * (int64_t)gridDim.x) {
    step(rb, set_a, set_b);
    if (rb + gridDim.x < row_blocks) step(rb + gridDim.x, set_b, set_a);
  }
}

// Streaming backward for rows too wide for the register cache: one row per workgroup.
template <typename TDY, typename TY, typename TDX, int VEC>
__global__ __launch_bounds__(1024) void softmax_bwd_stream_kernel(
    const TDY* __restrict__ dy, const TY* __restrict__ y, TDX* __restrict__ dx, int feat,
    int64_t dys, int64_t ys, int64_t dxs, int neg, int log) {
  __shared__ float scratch[16];
  const int group = blockDim.x;
  const int lane = threadIdx.x;
  const int chunks = feat / VEC;
  const float sign = neg ? -1.f : 1.f;
  const TDY* dyr = dy + (int64_t)blockIdx.x * dys;
  const TY* yr = y + (int64_t)blockIdx.x * ys;
  TDX* dxr = dx + (int64_t)blockIdx.x * dxs;
  float s = 0.f;
  for (int c = lane; c < chunks; c += group) {
    float dv[VEC], yv[VEC];
    load_f32<TDY, VEC>(dyr + (int64_t)c * VEC, dv);
    load_f32<TY, VEC>(yr + (int64_t)c * VEC, yv);
#pragma unroll
    for (int j = 0; j < VEC; ++j) s += log ? dv[j] : dv[j] * yv[j];
  }
  s = group_reduce(s, group, scratch, SumOp(), 0.f);
  for (int c = lane; c < chunks; c += group) {
    float dv[VEC], yv[VEC], o[VEC];
    load_f32<TDY, VEC>(dyr + (int64_t)c * VEC, dv);
    load_f32<TY, VEC>(yr + (int64_t)c * VEC, yv);
#pragma unroll
    for (int j = 0; j < VEC; ++j)
      o[j] = sign * (log ? dv[j] - __expf(yv[j]) * s : yv[j] * (dv[j] - s));
    store_f32<TDX, VEC>(dxr + (int64_t)c * VEC, o);
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
    default: { constexpr int ITERS = 8; __VA_ARGS__; break; }      \
  }

#define AT_DISPATCH_ITERS4(ITERS_VALUE, ...)                      \
  switch (ITERS_VALUE) {                                           \
    case 1: { constexpr int ITERS = 1; __VA_ARGS__; break; }       \
    case 2: { constexpr int ITERS = 2; __VA_ARGS__; break; }       \
    default: { constexpr int ITERS = 4; __VA_ARGS__; break; }      \
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
  if (batch > (int64_t)0x7fffffff) return AT_ERR_DIM;  // one workgroup per row on the streaming path
  if (s0 < feat || s1 < feat || s2 < feat) return AT_ERR_DIM;
  return AT_OK;
}

// Workgroups of `fn` one CU keeps resident at this block size (asked once per kernel).
inline int resident_blocks(const void* fn, int block, size_t lds) {
  static std::mutex mu;
  static std::map<std::tuple<const void*, int, size_t>, int> known;
  std::lock_guard<std::mutex> lock(mu);
  const auto key = std::make_tuple(fn, block, lds);
  auto it = known.find(key);
  if (it != known.end()) return it->second;
  int n = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, fn, block, lds) != hipSuccess || n <= 0) {
    (void)hipGetLastError();
    n = 1;
  }
  known.emplace(key, n);
  return n;
}

// Whether a backward pass that holds two tensors per row runs one row-block per workgroup instead
// of the persistent grid: when there is work for many rounds of workgroups, a workgroup that ends
// behind its stores does better than one that loops (its next loads count as arrived only after
// its own stores are acknowledged); with few row-blocks per resident workgroup the ramp of short
// workgroups costs more than that.
inline bool one_shot(int64_t row_blocks, unsigned persistent) {
  return row_blocks >= (int64_t)persistent * 4 && row_blocks <= (int64_t)INT32_MAX;
}

// Grid of a persistent row kernel: no more workgroups than stay resident at once, and as even a
// number of row-blocks per workgroup as that allows.  max_blocks > 0 caps the grid further.
inline unsigned persistent_grid(const void* fn, int block, size_t lds, int64_t row_blocks,
                                int64_t max_blocks) {
  int64_t cap = (int64_t)device_cu_count() * resident_blocks(fn, block, lds);
  if (max_blocks > 0 && cap > max_blocks) cap = max_blocks;
  if (row_blocks <= cap) return (unsigned)row_blocks;
  const int64_t rounds = cdiv64(row_blocks, cap);
  return (unsigned)cdiv64(row_blocks, rounds);
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
  if (weight && wdt != xdt && wdt != AT_DTYPE_F32) return AT_ERR_DTYPE;  // parameters: input dtype or fp32
  int vec = narrow_vec(xdt, ydt, AT_DTYPE_F32);
  const bool vector_ok = feat % vec == 0 && rows_vectorizable(x, xs, xdt) &&
                         rows_vectorizable(y, ys, ydt) && (!weight || aligned16(weight)) &&
                         (!bias || aligned16(bias));
  if (!vector_ok) vec = 1;
  // up to four chunks per lane before a row spreads over more than one wave: fewer waves share
  // each reduction, and enough of them stay resident to hide its latency
  const RowPlan p = plan_rows(feat, vec, 256, 4, 512);
  return dispatch_pair(xdt, ydt, [&](auto* tx, auto* ty) -> int {
    typedef std::remove_pointer_t<decltype(tx)> TX;
    typedef std::remove_pointer_t<decltype(ty)> TY;
    constexpr int VECW = sizeof(TX) == 4 && sizeof(TY) == 4 ? 4 : 8;
    if (p.iters == 0) {
      if (vec != 1)
        hipLaunchKernelGGL((norm_fwd_stream_kernel<LAYER, TX, TY, VECW>), dim3((unsigned)batch), dim3(1024),
                           0, stream, (const TX*)x, weight, bias, mean, rstd, (TY*)y, (int)feat, xs, ys,
                           eps, wdt);
      else
        hipLaunchKernelGGL((norm_fwd_stream_kernel<LAYER, TX, TY, 1>), dim3((unsigned)batch), dim3(1024), 0,
                           stream, (const TX*)x, weight, bias, mean, rstd, (TY*)y, (int)feat, xs, ys, eps,
                           wdt);
      return launch_status();
    }
    const int64_t row_blocks = cdiv64(batch, p.block >> p.group_log2);
#define AT_NORM_FWD_LAUNCH(TW, VV)                                                                       \
  AT_DISPATCH_ITERS(p.iters, {                                                                           \
    auto kernel = norm_fwd_kernel<LAYER, TX, TY, TW, VV, ITERS, true>;                                   \
    const unsigned grid = persistent_grid((const void*)kernel, p.block, 0, row_blocks, 0);               \
    /* measured: fp32 rows gain 5-13 % without the second register set, 16-bit rows lose up to 15 % */ \
    if (sizeof(TX) == 4 && one_shot(row_blocks, grid))                                                   \
      hipLaunchKernelGGL((norm_fwd_kernel<LAYER, TX, TY, TW, VV, ITERS, false>),                         \
                         dim3((unsigned)row_blocks), dim3(p.block), 0, stream, (const TX*)x,             \
                         (const TW*)weight, (const TW*)bias, mean, rstd, (TY*)y, batch, (int)feat, xs,   \
                         ys, eps, p.group_log2);                                                         \
    else                                                                                                 \
      hipLaunchKernelGGL(kernel, dim3(grid), dim3(p.block), 0, stream, (const TX*)x, (const TW*)weight,  \
                         (const TW*)bias, mean, rstd, (TY*)y, batch, (int)feat, xs, ys, eps,             \
                         p.group_log2);                                                                  \
  })
    // parameters are stored either like the input or in fp32
    if (weight && wdt == AT_DTYPE_F32 && xdt != AT_DTYPE_F32) {
      if (vec != 1) { AT_NORM_FWD_LAUNCH(float, VECW); } else { AT_NORM_FWD_LAUNCH(float, 1); }
    } else {
      if (vec != 1) { AT_NORM_FWD_LAUNCH(TX, VECW); } else { AT_NORM_FWD_LAUNCH(TX, 1); }
    }
#undef AT_NORM_FWD_LAUNCH
    return launch_status();
  });
}

constexpr int kBwdBlock = 512;        // 8 waves: room for 256 VGPRs per lane
constexpr int kStreamSlices = 256;    // row slices of the column kernel in the streaming fallback
constexpr int kMaxPartialRows = 1024; // upper bound on partial rows (grid size or kStreamSlices)

template <bool LAYER>
int norm_bwd(const void* dy, const void* x, const float* mean, const float* rstd, const void* weight,
             void* dx, float* weight_grad, float* bias_grad, void* workspace, int64_t workspace_bytes,
             int64_t batch, int64_t feat, int64_t dys, int64_t xs, int64_t dxs, int dydt, int xdt,
             int wdt, int dxdt, hipStream_t stream) {
  if (!dy || !x || !rstd || !dx || (LAYER && !mean)) return AT_ERR_NULL;
  if (!dtype_valid(dydt) || !dtype_valid(xdt) || !dtype_valid(dxdt) || (weight && !dtype_valid(wdt)))
    return AT_ERR_DTYPE;
  if (dxdt != dydt) return AT_ERR_DTYPE;  // the input gradient is produced in the output dtype
  if (weight && wdt != xdt && wdt != AT_DTYPE_F32) return AT_ERR_DTYPE;  // parameters: input dtype or fp32
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
      hipLaunchKernelGGL(reduce_partials_kernel, dim3((unsigned)cdiv64(feat, kReduceCols), bias_grad ? 2 : 1),
                         dim3(256), 0, stream, (const float*)workspace, weight_grad,
                         (const float*)workspace, bias_grad, 0, (int)feat);
    return launch_status();
  }
  int vec = narrow_vec(dydt, xdt, dxdt);
  const bool vector_ok = feat % vec == 0 && rows_vectorizable(dy, dys, dydt) &&
                         rows_vectorizable(x, xs, xdt) && rows_vectorizable(dx, dxs, dxdt) &&
                         (!weight || aligned16(weight));
  if (!vector_ok) vec = 1;
  // The backward kernel keeps ITERS * VEC fp32 column accumulators per parameter gradient next
  // to two rows of both cached tensors: it prefers two chunks per lane (rows spread over more
  // waves) and stops at four; wider rows stream.
  RowPlan p = plan_rows(feat, vec, kBwdBlock, 2, kBwdBlock);
  if (p.iters > 4) p.iters = 0;
  float* part_w = weight_grad ? (float*)workspace : nullptr;
  int parts = 0;

  rc = dispatch_pair(xdt, dydt, [&](auto* tx, auto* tdy) -> int {
    typedef std::remove_pointer_t<decltype(tx)> TX;
    typedef std::remove_pointer_t<decltype(tdy)> TDY;
    constexpr int VECW = sizeof(TX) == 4 && sizeof(TDY) == 4 ? 4 : 8;
    if (p.iters != 0) {
      const int rpb = p.block >> p.group_log2;
      const int64_t row_blocks = cdiv64(batch, rpb);
#define AT_NORM_BWD_LAUNCH(TW, VV)                                                                       \
  {                                                                                                      \
    AT_DISPATCH_ITERS4(p.iters, {                                                                        \
      const size_t lds = rpb > 1 ? (size_t)(p.block - (1 << p.group_log2)) * VV * ITERS * n_grads * sizeof(float) : 0; \
      auto kernel = norm_bwd_kernel<LAYER, TDY, TX, TDY, TW, VV, ITERS>;                                 \
      parts = (int)persistent_grid((const void*)kernel, p.block, lds, row_blocks, kMaxPartialRows);      \
      float* part_b = bias_grad ? part_w + (int64_t)parts * feat : nullptr;                              \
      hipLaunchKernelGGL(kernel, dim3(parts), dim3(p.block), lds, stream, (const TDY*)dy, (const TX*)x,  \
                         mean, rstd, (const TW*)weight, (TDY*)dx, part_w, part_b, batch, (int)feat, dys, \
                         xs, dxs, p.group_log2);                                                         \
    });                                                                                                  \
  }
      if (weight && wdt == AT_DTYPE_F32 && xdt != AT_DTYPE_F32) {
        if (vec != 1) AT_NORM_BWD_LAUNCH(float, VECW) else AT_NORM_BWD_LAUNCH(float, 1)
      } else {
        if (vec != 1) AT_NORM_BWD_LAUNCH(TX, VECW) else AT_NORM_BWD_LAUNCH(TX, 1)
      }
#undef AT_NORM_BWD_LAUNCH
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
    hipLaunchKernelGGL(reduce_partials_kernel, dim3((unsigned)cdiv64(feat, kReduceCols), bias_grad ? 2 : 1),
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
                   int64_t y_stride, int neg, int log, int x_dtype, int y_dtype, at_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  if (!x || !y) return AT_ERR_NULL;
  if (!dtype_valid(x_dtype) || !dtype_valid(y_dtype)) return AT_ERR_DTYPE;
  int rc = check_rows(batch, feat, x_stride, y_stride, feat);
  if (rc) return rc;
  if (batch == 0) return AT_OK;
  int vec = narrow_vec(x_dtype, y_dtype, AT_DTYPE_F32);
  if (!(feat % vec == 0 && rows_vectorizable(x, x_stride, x_dtype) && rows_vectorizable(y, y_stride, y_dtype)))
    vec = 1;
  // one wave per row up to eight chunks per lane (no workgroup barrier in the reductions)
  const RowPlan p = plan_rows(feat, vec, 256, 8, 1024);
  return dispatch_pair(x_dtype, y_dtype, [&](auto* tx, auto* ty) -> int {
    typedef std::remove_pointer_t<decltype(tx)> TX;
    typedef std::remove_pointer_t<decltype(ty)> TY;
    constexpr int VECW = sizeof(TX) == 4 && sizeof(TY) == 4 ? 4 : 8;
    if (p.iters == 0) {
      if (vec != 1)
        hipLaunchKernelGGL((softmax_fwd_stream_kernel<TX, TY, VECW>), dim3((unsigned)batch), dim3(1024), 0,
                           stream, (const TX*)x, (TY*)y, (int)feat, x_stride, y_stride, neg, log);
      else
        hipLaunchKernelGGL((softmax_fwd_stream_kernel<TX, TY, 1>), dim3((unsigned)batch), dim3(1024), 0,
                           stream, (const TX*)x, (TY*)y, (int)feat, x_stride, y_stride, neg, log);
      return launch_status();
    }
    const int64_t row_blocks = cdiv64(batch, p.block >> p.group_log2);
#define AT_SOFTMAX_FWD_LAUNCH(VV, MAXB)                                                                  \
  AT_DISPATCH_ITERS(p.iters, {                                                                           \
    auto kernel = softmax_fwd_kernel<TX, TY, VV, ITERS, MAXB, true>;                                     \
    const unsigned grid = persistent_grid((const void*)kernel, p.block, 0, row_blocks, 0);               \
    /* eight chunks per lane (one wave per wide row) do slightly better with the look-ahead */          \
    if (ITERS < 8 && one_shot(row_blocks, grid))                                                         \
      hipLaunchKernelGGL((softmax_fwd_kernel<TX, TY, VV, ITERS, MAXB, false>), dim3((unsigned)row_blocks), \
                         dim3(p.block), 0, stream, (const TX*)x, (TY*)y, batch, (int)feat, x_stride,     \
                         y_stride, neg, log, p.group_log2);                                              \
    else                                                                                                 \
      hipLaunchKernelGGL(kernel, dim3(grid), dim3(p.block), 0, stream, (const TX*)x, (TY*)y, batch,      \
                         (int)feat, x_stride, y_stride, neg, log, p.group_log2);                         \
  })
    if (p.block <= 256) {
      if (vec != 1) { AT_SOFTMAX_FWD_LAUNCH(VECW, 256); } else { AT_SOFTMAX_FWD_LAUNCH(1, 256); }
    } else {
      if (vec != 1) { AT_SOFTMAX_FWD_LAUNCH(VECW, 1024); } else { AT_SOFTMAX_FWD_LAUNCH(1, 1024); }
    }
#undef AT_SOFTMAX_FWD_LAUNCH
    return launch_status();
  });
}

int at_softmax_bwd(const void* dy, const void* y, void* dx, int64_t batch, int64_t feat,
                   int64_t dy_stride, int64_t y_stride, int64_t dx_stride, int neg, int log,
                   int dy_dtype, int y_dtype, int dx_dtype, at_stream_t stream_) {
  hipStream_t stream = (hipStream_t)stream_;
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
  // two rows of two tensors are held at once: four chunks per lane and tensor at most
  RowPlan p = plan_rows(feat, vec, 256, 2, 1024);
  if (p.iters > 4) p.iters = 0;
  return dispatch_pair(dy_dtype, y_dtype, [&](auto* tdy, auto* ty) -> int {
    typedef std::remove_pointer_t<decltype(tdy)> TDY;
    typedef std::remove_pointer_t<decltype(ty)> TY;
    constexpr int VECW = sizeof(TDY) == 4 && sizeof(TY) == 4 ? 4 : 8;
    if (p.iters == 0) {
      if (vec != 1)
        hipLaunchKernelGGL((softmax_bwd_stream_kernel<TDY, TY, TY, VECW>), dim3((unsigned)batch), dim3(1024),
                           0, stream, (const TDY*)dy, (const TY*)y, (TY*)dx, (int)feat, dy_stride, y_stride,
                           dx_stride, neg, log);
      else
        hipLaunchKernelGGL((softmax_bwd_stream_kernel<TDY, TY, TY, 1>), dim3((unsigned)batch), dim3(1024), 0,
                           stream, (const TDY*)dy, (const TY*)y, (TY*)dx, (int)feat, dy_stride, y_stride,
                           dx_stride, neg, log);
      return launch_status();
    }
    const int64_t row_blocks = cdiv64(batch, p.block >> p.group_log2);
#define AT_SOFTMAX_BWD_LAUNCH(VV)                                                                        \
  AT_DISPATCH_ITERS4(p.iters, {                                                                          \
    auto kernel = softmax_bwd_kernel<TDY, TY, TY, VV, ITERS, true>;                                      \
    const unsigned grid = persistent_grid((const void*)kernel, p.block, 0, row_blocks, 0);               \
    if (one_shot(row_blocks, grid))                                                                      \
      hipLaunchKernelGGL((softmax_bwd_kernel<TDY, TY, TY, VV, ITERS, false>), dim3((unsigned)row_blocks), \
                         dim3(p.block), 0, stream, (const TDY*)dy, (const TY*)y, (TY*)dx, batch,         \
                         (int)feat, dy_stride, y_stride, dx_stride, neg, log, p.group_log2);             \
    else                                                                                                 \
      hipLaunchKernelGGL(kernel, dim3(grid), dim3(p.block), 0, stream, (const TDY*)dy, (const TY*)y,     \
                         (TY*)dx, batch, (int)feat, dy_stride, y_stride, dx_stride, neg, log,            \
                         p.group_log2);                                                                  \
  })
    if (vec != 1) { AT_SOFTMAX_BWD_LAUNCH(VECW); } else { AT_SOFTMAX_BWD_LAUNCH(1); }
#undef AT_SOFTMAX_BWD_LAUNCH
    return launch_status();
  });
}

}  // extern "C"
