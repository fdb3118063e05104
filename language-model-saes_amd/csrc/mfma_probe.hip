// Matrix-core rate probe: v_mfma_f32_16x16x32_bf16 issued back to back from registers, no memory traffic inside
// the loop.  It measures what the matrix cores deliver on this card at the clock the power management grants, the
// ceiling the encoder GEMM is to be read against next to the published peak.  Not part of the train step.
#include "common.h"

namespace sae {

typedef __attribute__((ext_vector_type(8))) __bf16 probe_bf16x8;
typedef __attribute__((ext_vector_type(4))) float probe_f32x4;

constexpr int PROBE_THREADS = 256;   // 4 waves per workgroup, one per SIMD
constexpr int PROBE_ACC = 8;         // independent accumulators per wave (covers the MFMA's result latency)

__global__ __launch_bounds__(PROBE_THREADS) void mfma_probe_kernel(float *__restrict__ out, int iters) {
  const int tid = threadIdx.x;
  // four operand pairs of hashed values in (-1, 1), used in turn, so that the operand lines toggle as they do
  // on real data (the power drawn, and with it the clock, depends on that)
  probe_bf16x8 a[4], b[4];
  uint32_t h = 0x9e3779b9u * (uint32_t)(blockIdx.x * PROBE_THREADS + tid + 1);
  for (int r = 0; r < 4; ++r)
    for (int i = 0; i < 8; ++i) {
      h = h * 1664525u + 1013904223u;
      a[r][i] = (__bf16)((float)(int32_t)h * (1.0f / 2147483648.0f));
      h = h * 1664525u + 1013904223u;
      b[r][i] = (__bf16)((float)(int32_t)h * (1.0f / 2147483648.0f));
    }
  probe_f32x4 acc[PROBE_ACC];
  for (int j = 0; j < PROBE_ACC; ++j) acc[j] = probe_f32x4{0.f, 0.f, 0.f, 0.f};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int j = 0; j < PROBE_ACC; ++j) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[r], b[r], acc[j], 0, 0, 0);
  }
  float s = 0.f;
  for (int j = 0; j < PROBE_ACC; ++j) s += acc[j][0] + acc[j][1] + acc[j][2] + acc[j][3];
  out[(size_t)blockIdx.x * PROBE_THREADS + tid] = s;
}

}  // namespace sae

extern "C" int sae_mfma_probe(float *out, int64_t n_workgroups, int64_t iters, double *flop_out, void *stream) {
  using namespace sae;
  SAE_REQUIRE(out, SAE_ERR_INVALID_ARG, "mfma_probe: null output");
  SAE_REQUIRE(n_workgroups > 0 && n_workgroups <= 65536 && iters > 0 && iters <= (1 << 24), SAE_ERR_INVALID_ARG,
              "mfma_probe: n_workgroups in [1, 65536], iters in [1, 2^24]");
  hipLaunchKernelGGL(mfma_probe_kernel, dim3((unsigned)n_workgroups), dim3(PROBE_THREADS), 0, (hipStream_t)stream, out,
                     (int)iters);
  // 16 x 16 x 32 multiply-adds per instruction, 4 x PROBE_ACC instructions per iteration and wave
  if (flop_out)
    *flop_out = 2.0 * 16 * 16 * 32 * 4.0 * PROBE_ACC * (double)iters * (PROBE_THREADS / 64) * (double)n_workgroups;
  return check_launch("mfma_probe");
}
