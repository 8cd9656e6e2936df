// Version and error-string entry points of libattorch_hip, and the matrix-core probe.
#include "at_common.h"
#include "at_mfma.h"

namespace at_hip {
namespace {

// v_mfma_f32_32x32x16_bf16 back to back, operands and accumulators in registers, no memory
// traffic: what the matrix cores sustain by themselves.  RANDOM: eight register sets of
// pseudo-random values in [-1, 1) that change from one MFMA to the next, as the operands of a
// real product do; otherwise one pair of small integers throughout.
template <bool RANDOM>
__global__ __launch_bounds__(256) void mfma_probe_kernel(int iters, float* sink) {
  f32x16 acc[4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[a][e] = 0.f;
  constexpr int SETS = RANDOM ? 8 : 1;
  bf16x8 x[SETS], y[SETS];
  unsigned s = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
#pragma unroll
  for (int r = 0; r < SETS; ++r)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (RANDOM) {
        s = s * 1664525u + 1013904223u;
        x[r][e] = (__bf16)(((int)(s >> 16) & 0xfff) * (1.f / 2048.f) - 1.f);
        s = s * 1664525u + 1013904223u;
        y[r][e] = (__bf16)(((int)(s >> 16) & 0xfff) * (1.f / 2048.f) - 1.f);
      } else {
        x[r][e] = (__bf16)(float)((threadIdx.x + e) & 7);
        y[r][e] = (__bf16)(float)((blockIdx.x + e) & 7);
      }
    }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int u = 0; u < 16; ++u)
#pragma unroll
      for (int a = 0; a < 4; ++a)
        acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x[(u + a) % SETS], y[(u * 3 + a) % SETS], acc[a], 0, 0, 0);
  }
  float t = 0.f;
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int e = 0; e < 16; ++e) t += acc[a][e];
  if (t == 12345.678f) sink[0] = t;   // keeps the accumulators alive; never true for these operands' sums in practice
}

}  // namespace
}  // namespace at_hip

extern "C" {

int at_version(void) { return 100; }

const char* at_error_string(int code) {
  switch (code) {
    case AT_OK: return "success";
    case AT_ERR_NULL: return "a required pointer is null";
    case AT_ERR_DIM: return "a dimension or stride is out of range";
    case AT_ERR_DTYPE: return "unknown dtype or unsupported dtype combination";
    case AT_ERR_ACT: return "unknown activation id";
    case AT_ERR_WORKSPACE: return "workspace missing or too small";
    case AT_ERR_ALIGN: return "pointer or stride alignment the kernel cannot serve";
    case AT_ERR_UNSUPPORTED: return "configuration not implemented";
    default: return code > 0 ? "HIP runtime error (hipError_t)" : "unknown error code";
  }
}

int64_t at_mfma_probe_flop(int64_t iters) {
  if (iters <= 0) return 0;
  // 2 workgroups of 4 waves per CU, 64 MFMAs of 32 x 32 x 16 per iteration and wave
  return (int64_t)at_hip::device_cu_count() * 2 * 4 * iters * 64 * (2LL * 32 * 32 * 16);
}

int at_mfma_probe(int64_t iters, int random_operands, void* scratch4, at_stream_t stream) {
  if (!scratch4) return AT_ERR_NULL;
  if (iters <= 0 || iters > (1 << 24)) return AT_ERR_DIM;
  const dim3 grid((unsigned)at_hip::device_cu_count() * 2);
  if (random_operands)
    hipLaunchKernelGGL((at_hip::mfma_probe_kernel<true>), grid, dim3(256), 0, (hipStream_t)stream, (int)iters, (float*)scratch4);
  else
    hipLaunchKernelGGL((at_hip::mfma_probe_kernel<false>), grid, dim3(256), 0, (hipStream_t)stream, (int)iters, (float*)scratch4);
  return at_hip::launch_status();
}

}  // extern "C"
