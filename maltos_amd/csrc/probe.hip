// Measurement aid: the rate at which this chip's matrix cores run v_mfma_f32_32x32x16_bf16 and nothing else, on operands
// the caller chooses.  The cores' power, and with it the clock the chip holds, depends on the operand values (zeros run
// at the nominal 2.5 PFLOP/s, normally distributed values well below), so the figure says how much of the nominal peak
// a given GPU sustains on data like a workload's; the attention kernels' rates are read against it.
#include "common.hpp"

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kProbeThreads = 512;  // two wavefronts per SIMD
constexpr int kProbeFrags = 8;      // four A and four B fragments of eight bf16 per lane

__global__ __launch_bounds__(kProbeThreads) void mfma_probe_kernel(const __bf16* __restrict__ operands, float* __restrict__ out,
                                                                   int iters) {
  probe_bf16x8 a[4], b[4];
  const __bf16* src = operands + static_cast<int64_t>(threadIdx.x) * (kProbeFrags * 8);
#pragma unroll
  for (int f = 0; f < 4; ++f) {
    a[f] = *reinterpret_cast<const probe_bf16x8*>(src + f * 8);
    b[f] = *reinterpret_cast<const probe_bf16x8*>(src + 32 + f * 8);
  }
  f32x16 acc[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[c][e] = 0.f;
  for (int it = 0; it < iters; ++it) {
    // sixteen MFMAs over all (A, B) pairs; four independent accumulators, so consecutive MFMAs never wait for each other
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(u + c) & 3], b[c], acc[c], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < 4; ++c)
#pragma unroll
    for (int e = 0; e < 16; ++e) s += acc[c][e];
  out[static_cast<int64_t>(blockIdx.x) * kProbeThreads + threadIdx.x] = s;
}

}  // namespace

extern "C" int64_t mlts_mfma_probe_flops(int32_t blocks, int32_t iters) {
  return static_cast<int64_t>(blocks) * (kProbeThreads / 64) * iters * 16 * (2LL * 32 * 32 * 16);
}

extern "C" int mlts_mfma_probe(const void* operands, int64_t n_operands, float* out, int32_t blocks, int32_t iters,
                               mlts_stream_t stream) {
  MLTS_REQUIRE(operands && out, "mlts_mfma_probe: null pointer");
  MLTS_REQUIRE(n_operands >= kProbeThreads * kProbeFrags * 8, "mlts_mfma_probe: needs %d bf16 operands", kProbeThreads * kProbeFrags * 8);
  MLTS_REQUIRE(mlts_aligned16(operands), "mlts_mfma_probe: operands must be 16-byte aligned");
  MLTS_REQUIRE(blocks > 0 && iters >= 0, "mlts_mfma_probe: blocks must be > 0 and iters >= 0");
  hipStream_t st = static_cast<hipStream_t>(stream);
  {
    MltsKernelTimer timer("mfma_probe", st);
    hipLaunchKernelGGL(mfma_probe_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kProbeThreads), 0, st,
                       static_cast<const __bf16*>(operands), out, iters);
  }
  return mlts_check_launch("mlts_mfma_probe");
}
