// Training metrics computed from the sparse code and the two [B, d] tensors of a step, so that logging
// never forms a dense [B, F] activation matrix.
#include "common.h"

namespace sae {

// One wave per token.  freq[f] += w_b for every kept slot with a positive value (w_b = 1 without a mask),
// l0_tok[b] = number of such slots, totals += (sum of all kept values, #positive, sum_b w_b #positive_b).
// Counts and 0/1 weights are integers well below 2^24, so the float atomics are exact and the result does
// not depend on their order.
__global__ __launch_bounds__(256) void code_stats_kernel(const int32_t *__restrict__ idx, const float *__restrict__ val,
                                                         const int64_t *__restrict__ row_off,
                                                         const int32_t *__restrict__ row_nnz,
                                                         const float *__restrict__ tok_w, int64_t B, int64_t F,
                                                         float *__restrict__ freq, float *__restrict__ l0_tok,
                                                         double *__restrict__ totals) {
  __shared__ double red[12];
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int64_t b = (int64_t)blockIdx.x * 4 + w;
  double s_val = 0.0, s_cnt = 0.0, s_wcnt = 0.0;
  if (b < B) {
    const int64_t off = row_off[b];
    const int n = row_nnz[b];
    const float wb = tok_w ? tok_w[b] : 1.f;
    float sum = 0.f;
    int cnt = 0;
    for (int i = lane; i < n; i += 64) {
      const float v = val[off + i];
      sum += v;
      if (v > 0.f) {
        ++cnt;
        const int32_t f = idx[off + i];
        if (freq && wb != 0.f && f >= 0 && f < F) atomicAdd(&freq[f], wb);
      }
    }
    sum = wave_sum(sum);
    cnt = wave_sum_i(cnt);
    if (lane == 0) {
      if (l0_tok) l0_tok[b] = (float)cnt;
      s_val = (double)sum;
      s_cnt = (double)cnt;
      s_wcnt = (double)wb * (double)cnt;
    }
  }
  if (lane == 0) { red[w] = s_val; red[4 + w] = s_cnt; red[8 + w] = s_wcnt; }
  __syncthreads();
  if (threadIdx.x == 0 && totals) {
    atomicAdd(&totals[0], red[0] + red[1] + red[2] + red[3]);
    atomicAdd(&totals[1], red[4] + red[5] + red[6] + red[7]);
    atomicAdd(&totals[2], red[8] + red[9] + red[10] + red[11]);
  }
}

// One workgroup per token: tok[b] = (sum (recon - label)^2, sum (label - mean)^2, sum label^2).
__global__ __launch_bounds__(256) void recon_stats_kernel(const float *__restrict__ label, const float *__restrict__ recon,
                                                          const float *__restrict__ mean, int d,
                                                          float *__restrict__ tok) {
  __shared__ float red[4];
  const int64_t b = blockIdx.x;
  const float *lr = label + b * d, *rr = recon + b * d;
  float se = 0.f, var = 0.f, l2 = 0.f;
  if ((d & 3) == 0) {
    for (int i = threadIdx.x; i < (d >> 2); i += 256) {
      const float4 l = reinterpret_cast<const float4 *>(lr)[i];
      const float4 r = reinterpret_cast<const float4 *>(rr)[i];
      const float4 m = reinterpret_cast<const float4 *>(mean)[i];
      float e;
      e = r.x - l.x; se = fmaf(e, e, se); e = r.y - l.y; se = fmaf(e, e, se);
      e = r.z - l.z; se = fmaf(e, e, se); e = r.w - l.w; se = fmaf(e, e, se);
      e = l.x - m.x; var = fmaf(e, e, var); e = l.y - m.y; var = fmaf(e, e, var);
      e = l.z - m.z; var = fmaf(e, e, var); e = l.w - m.w; var = fmaf(e, e, var);
      l2 = fmaf(l.x, l.x, l2); l2 = fmaf(l.y, l.y, l2); l2 = fmaf(l.z, l.z, l2); l2 = fmaf(l.w, l.w, l2);
    }
  } else {
    for (int i = threadIdx.x; i < d; i += 256) {
      const float l = lr[i];
      float e = rr[i] - l; se = fmaf(e, e, se);
      e = l - mean[i]; var = fmaf(e, e, var);
      l2 = fmaf(l, l, l2);
    }
  }
  se = block_sum<4>(se, red);
  var = block_sum<4>(var, red);
  l2 = block_sum<4>(l2, red);
  if (threadIdx.x == 0) { tok[3 * b] = se; tok[3 * b + 1] = var; tok[3 * b + 2] = l2; }
}

// One workgroup, fixed order: the masked token means behind the explained-variance and L2-error metrics,
//   acc[0] += 1 - mean(se) / mean(var)          acc[1] += mean(1 - se / var)
//   acc[2] += mean(sqrt(se))                    acc[3] += mean(sqrt(se)) / mean(sqrt(l2))
// mean = sum_b w_b (.) / sum_b w_b; step_out (nullable) receives this step's four values.
__global__ __launch_bounds__(1024) void recon_stats_finish_kernel(const float *__restrict__ tok, const float *__restrict__ tok_w,
                                                                  int64_t B, double *__restrict__ acc,
                                                                  float *__restrict__ step_out) {
  __shared__ double red[6][16];
  double s[6] = {0, 0, 0, 0, 0, 0};
  for (int64_t b = threadIdx.x; b < B; b += 1024) {
    const double w = tok_w ? (double)tok_w[b] : 1.0;
    if (w == 0.0) continue;  // a masked token contributes nothing (not even a NaN from 0 / 0)
    const float se = tok[3 * b], var = tok[3 * b + 1], l2 = tok[3 * b + 2];
    s[0] += w;
    s[1] += w * (double)se;
    s[2] += w * (double)var;
    s[3] += w * (double)(1.f - se / var);
    s[4] += w * (double)sqrtf(se);
    s[5] += w * (double)sqrtf(l2);
  }
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
#pragma unroll
  for (int q = 0; q < 6; ++q) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) s[q] += __shfl_xor(s[q], o, 64);
    if (lane == 0) red[q][wv] = s[q];
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    double t[6];
    for (int q = 0; q < 6; ++q) {
      t[q] = 0.0;
      for (int i = 0; i < 16; ++i) t[q] += red[q][i];
    }
    const double n = t[0];
    const double ev = 1.0 - (t[1] / n) / (t[2] / n), legacy = t[3] / n, err = t[4] / n, ratio = err / (t[5] / n);
    acc[0] += ev; acc[1] += legacy; acc[2] += err; acc[3] += ratio;
    if (step_out) { step_out[0] = (float)ev; step_out[1] = (float)legacy; step_out[2] = (float)err; step_out[3] = (float)ratio; }
  }
}

}  // namespace sae

extern "C" int sae_code_stats(const int32_t *idx, const float *val, const int64_t *row_off, const int32_t *row_nnz,
                              const float *tok_w, int64_t B, int64_t F, float *freq_acc, float *l0_tok, double *totals,
                              void *stream) {
  using namespace sae;
  SAE_REQUIRE(idx && val && row_off && row_nnz, SAE_ERR_INVALID_ARG, "code_stats: null pointer");
  SAE_REQUIRE(B > 0 && F > 0, SAE_ERR_INVALID_ARG, "code_stats: bad sizes");
  hipLaunchKernelGGL(code_stats_kernel, dim3((unsigned)((B + 3) / 4)), dim3(256), 0, (hipStream_t)stream, idx, val, row_off,
                     row_nnz, tok_w, B, F, freq_acc, l0_tok, totals);
  return check_launch("code_stats");
}

extern "C" int sae_recon_stats(const float *label, const float *recon, const float *label_mean, const float *tok_w,
                               int64_t B, int64_t d, float *tok_workspace, double *acc, float *step_out, void *stream) {
  using namespace sae;
  SAE_REQUIRE(label && recon && label_mean && tok_workspace && acc, SAE_ERR_INVALID_ARG, "recon_stats: null pointer");
  SAE_REQUIRE(B > 0 && d > 0 && d < (1LL << 31) && B < (1LL << 31), SAE_ERR_INVALID_ARG, "recon_stats: bad sizes");
  SAE_REQUIRE(d % 4 != 0 || (((uintptr_t)label | (uintptr_t)recon | (uintptr_t)label_mean) & 15) == 0, SAE_ERR_INVALID_ARG,
              "recon_stats: 16-byte alignment required");
  hipStream_t st = (hipStream_t)stream;
  hipLaunchKernelGGL(recon_stats_kernel, dim3((unsigned)B), dim3(256), 0, st, label, recon, label_mean, (int)d, tok_workspace);
  hipLaunchKernelGGL(recon_stats_finish_kernel, dim3(1), dim3(1024), 0, st, tok_workspace, tok_w, B, acc, step_out);
  return check_launch("recon_stats");
}
