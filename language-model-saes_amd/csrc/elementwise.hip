// Small streaming kernels around the hot path: casts, row norms, transposes, column sums.
// All are HBM-bound single passes with 16-byte accesses where the shape allows.
#include "common.h"

namespace sae {

__global__ void zero_fill_kernel(uint32_t *p, size_t n_words) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n_words; i += stride) p[i] = 0u;
}

int zero_fill(void *p, size_t bytes, hipStream_t st) {
  if (bytes == 0) return SAE_OK;
  const size_t n_words = bytes / 4;
  size_t blocks = (n_words + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(zero_fill_kernel, dim3((unsigned)blocks), dim3(256), 0, st, reinterpret_cast<uint32_t *>(p), n_words);
  return check_launch("zero_fill");
}

__global__ __launch_bounds__(256) void cast_f32_bf16_kernel(const float *__restrict__ src, uint16_t *__restrict__ dst,
                                                            int64_t n) {
  const int64_t n8 = n >> 3;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += stride) {
    const float4 a = reinterpret_cast<const float4 *>(src)[2 * i];
    const float4 b = reinterpret_cast<const float4 *>(src)[2 * i + 1];
    u32x4 o;
    o.x = (uint32_t)f32_to_bf16_bits(a.x) | ((uint32_t)f32_to_bf16_bits(a.y) << 16);
    o.y = (uint32_t)f32_to_bf16_bits(a.z) | ((uint32_t)f32_to_bf16_bits(a.w) << 16);
    o.z = (uint32_t)f32_to_bf16_bits(b.x) | ((uint32_t)f32_to_bf16_bits(b.y) << 16);
    o.w = (uint32_t)f32_to_bf16_bits(b.z) | ((uint32_t)f32_to_bf16_bits(b.w) << 16);
    reinterpret_cast<u32x4 *>(dst)[i] = o;
  }
  // tail (n not a multiple of 8)
  const int64_t t = (n8 << 3) + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n) dst[t] = f32_to_bf16_bits(src[t]);
}

// one wave per row
__global__ __launch_bounds__(256) void row_norm_kernel(const float *__restrict__ w, float *__restrict__ out, int64_t F,
                                                       int d) {
  const int64_t f = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (f >= F) return;
  const int lane = threadIdx.x & 63;
  const float *row = w + f * d;
  float s = 0.f;
  if ((d & 3) == 0) {
    for (int i = lane; i < (d >> 2); i += 64) {
      const float4 v = reinterpret_cast<const float4 *>(row)[i];
      s = fmaf(v.x, v.x, s); s = fmaf(v.y, v.y, s); s = fmaf(v.z, v.z, s); s = fmaf(v.w, v.w, s);
    }
  } else {
    for (int i = lane; i < d; i += 64) s = fmaf(row[i], row[i], s);
  }
  s = wave_sum(s);
  if (lane == 0) out[f] = sqrtf(s);
}

// 64 x 64 tile transpose through LDS (padded to dodge bank conflicts)
__global__ __launch_bounds__(256) void transpose_kernel(const float *__restrict__ src, float *__restrict__ dst,
                                                        int64_t rows, int64_t cols) {
  __shared__ float tile[64][65];
  const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    const int64_t r = r0 + i, c = c0 + tx;
    tile[i][tx] = (r < rows && c < cols) ? src[r * cols + c] : 0.f;
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int64_t c = c0 + i, r = r0 + tx;
    if (c < cols && r < rows) dst[c * rows + r] = tile[tx][i];
  }
}

// Column sums of src [B, n].  Grid (ceil(n/256), chunks); every block sums `rows_per` rows of
// 256 columns in a fixed order and the chunk partials are combined in a second kernel, so the
// result does not depend on scheduling.
__global__ __launch_bounds__(256) void col_sum_partial_kernel(const float *__restrict__ src, float *__restrict__ part,
                                                              int64_t B, int64_t n, int rows_per) {
  const int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (j >= n) return;
  const int64_t b0 = (int64_t)blockIdx.y * rows_per, b1 = min(B, b0 + rows_per);
  float s = 0.f;
  for (int64_t b = b0; b < b1; ++b) s += src[b * n + j];
  part[(int64_t)blockIdx.y * n + j] = s;
}

__global__ __launch_bounds__(256) void col_sum_final_kernel(const float *__restrict__ part, float *__restrict__ out,
                                                            int64_t n, int chunks, int accumulate) {
  const int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (j >= n) return;
  float s = 0.f;
  for (int c = 0; c < chunks; ++c) s += part[(int64_t)c * n + j];
  out[j] = accumulate ? out[j] + s : s;
}

}  // namespace sae

extern "C" int sae_cast_f32_to_bf16(const float *src, void *dst, int64_t n, void *stream) {
  using namespace sae;
  SAE_REQUIRE(src && dst, SAE_ERR_INVALID_ARG, "cast_f32_to_bf16: null pointer");
  SAE_REQUIRE(n > 0, SAE_ERR_INVALID_ARG, "cast_f32_to_bf16: n must be positive");
  SAE_REQUIRE((((uintptr_t)src | (uintptr_t)dst) & 15) == 0, SAE_ERR_INVALID_ARG, "cast_f32_to_bf16: 16-byte alignment required");
  int64_t blocks = ((n >> 3) + 255) / 256;
  if (blocks < 1) blocks = 1;
  if (blocks > 16384) blocks = 16384;
  hipLaunchKernelGGL(cast_f32_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, src,
                     reinterpret_cast<uint16_t *>(dst), n);
  return check_launch("cast_f32_to_bf16");
}

extern "C" int sae_row_norm(const float *w, float *out, int64_t F, int64_t d, void *stream) {
  using namespace sae;
  SAE_REQUIRE(w && out, SAE_ERR_INVALID_ARG, "row_norm: null pointer");
  SAE_REQUIRE(F > 0 && d > 0 && d < (1LL << 31), SAE_ERR_INVALID_ARG, "row_norm: bad shape");
  SAE_REQUIRE((d & 3) != 0 || (((uintptr_t)w) & 15) == 0, SAE_ERR_INVALID_ARG, "row_norm: 16-byte alignment required");
  hipLaunchKernelGGL(row_norm_kernel, dim3((unsigned)((F + 3) / 4)), dim3(256), 0, (hipStream_t)stream, w, out, F, (int)d);
  return check_launch("row_norm");
}

extern "C" int sae_transpose_f32(const float *src, float *dst, int64_t rows, int64_t cols, void *stream) {
  using namespace sae;
  SAE_REQUIRE(src && dst, SAE_ERR_INVALID_ARG, "transpose_f32: null pointer");
  SAE_REQUIRE(rows > 0 && cols > 0, SAE_ERR_INVALID_ARG, "transpose_f32: bad shape");
  const int64_t gx = (cols + 63) / 64, gy = (rows + 63) / 64;
  SAE_REQUIRE(gy <= 65535, SAE_ERR_UNSUPPORTED, "transpose_f32: rows=%lld above %d", (long long)rows, 65535 * 64);
  hipLaunchKernelGGL(transpose_kernel, dim3((unsigned)gx, (unsigned)gy), dim3(256), 0, (hipStream_t)stream, src, dst, rows, cols);
  return check_launch("transpose_f32");
}

extern "C" int64_t sae_col_sum_workspace_bytes(int64_t B, int64_t n) {
  if (B <= 0 || n <= 0) return 0;
  return 64 * n * (int64_t)sizeof(float);
}

extern "C" int sae_col_sum(const float *src, float *out, int64_t B, int64_t n, int accumulate, void *workspace,
                           int64_t workspace_bytes, void *stream) {
  using namespace sae;
  SAE_REQUIRE(src && out, SAE_ERR_INVALID_ARG, "col_sum: null pointer");
  SAE_REQUIRE(B > 0 && n > 0, SAE_ERR_INVALID_ARG, "col_sum: bad shape");
  SAE_REQUIRE(workspace && workspace_bytes >= sae_col_sum_workspace_bytes(B, n), SAE_ERR_WORKSPACE,
              "col_sum: workspace of %lld bytes needed", (long long)sae_col_sum_workspace_bytes(B, n));
  const int chunks = (int)(B < 64 ? B : 64);
  const int rows_per = (int)((B + chunks - 1) / chunks);
  const unsigned gx = (unsigned)((n + 255) / 256);
  float *part = reinterpret_cast<float *>(workspace);
  hipLaunchKernelGGL(col_sum_partial_kernel, dim3(gx, (unsigned)chunks), dim3(256), 0, (hipStream_t)stream, src, part, B, n, rows_per);
  hipLaunchKernelGGL(col_sum_final_kernel, dim3(gx), dim3(256), 0, (hipStream_t)stream, part, out, n, chunks, accumulate);
  return check_launch("col_sum");
}
