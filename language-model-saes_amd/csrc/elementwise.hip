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

// dst[i, :] = cast(scale * src[row_idx[i], :]).  One workgroup per output row, 8 elements per thread per
// trip (16-byte loads from bf16 rows, 2 x 16 from fp32 rows); rows whose byte length is not a multiple of
// 16 take the element-wise tail path for the whole row.
template <bool SRC_BF16, bool DST_BF16>
__global__ __launch_bounds__(256) void gather_rows_kernel(const void *__restrict__ src, const int64_t *__restrict__ row_idx,
                                                          int64_t n_src_rows, int d, void *__restrict__ dst, float scale) {
  const int64_t i = blockIdx.x;
  const int64_t r = row_idx[i];
  if (r < 0 || r >= n_src_rows) return;   // the host validates indices it generated; a foreign index writes nothing
  const size_t s_es = SRC_BF16 ? 2 : 4, d_es = DST_BF16 ? 2 : 4;
  const char *srow = reinterpret_cast<const char *>(src) + (size_t)r * d * s_es;
  char *drow = reinterpret_cast<char *>(dst) + (size_t)i * d * d_es;
  const bool vec = (d & 7) == 0 && ((reinterpret_cast<uintptr_t>(srow) | reinterpret_cast<uintptr_t>(drow)) & 15) == 0;
  if (vec) {
    for (int c = threadIdx.x; c < (d >> 3); c += 256) {
      float v[8];
      if constexpr (SRC_BF16) {
        const u32x4 q = reinterpret_cast<const u32x4 *>(srow)[c];
        v[0] = __uint_as_float(q.x << 16); v[1] = __uint_as_float(q.x & 0xffff0000u);
        v[2] = __uint_as_float(q.y << 16); v[3] = __uint_as_float(q.y & 0xffff0000u);
        v[4] = __uint_as_float(q.z << 16); v[5] = __uint_as_float(q.z & 0xffff0000u);
        v[6] = __uint_as_float(q.w << 16); v[7] = __uint_as_float(q.w & 0xffff0000u);
      } else {
        const float4 a = reinterpret_cast<const float4 *>(srow)[2 * c], b = reinterpret_cast<const float4 *>(srow)[2 * c + 1];
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
      }
      if (scale != 1.f) {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] *= scale;
      }
      if constexpr (DST_BF16) {
        u32x4 o;
        o.x = (uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
        o.y = (uint32_t)f32_to_bf16_bits(v[2]) | ((uint32_t)f32_to_bf16_bits(v[3]) << 16);
        o.z = (uint32_t)f32_to_bf16_bits(v[4]) | ((uint32_t)f32_to_bf16_bits(v[5]) << 16);
        o.w = (uint32_t)f32_to_bf16_bits(v[6]) | ((uint32_t)f32_to_bf16_bits(v[7]) << 16);
        reinterpret_cast<u32x4 *>(drow)[c] = o;
      } else {
        reinterpret_cast<float4 *>(drow)[2 * c] = make_float4(v[0], v[1], v[2], v[3]);
        reinterpret_cast<float4 *>(drow)[2 * c + 1] = make_float4(v[4], v[5], v[6], v[7]);
      }
    }
  } else {
    for (int c = threadIdx.x; c < d; c += 256) {
      float x = SRC_BF16 ? bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(srow)[c]) : reinterpret_cast<const float *>(srow)[c];
      if (scale != 1.f) x *= scale;
      if constexpr (DST_BF16) reinterpret_cast<uint16_t *>(drow)[c] = f32_to_bf16_bits(x);
      else reinterpret_cast<float *>(drow)[c] = x;
    }
  }
}

}  // namespace sae

extern "C" int sae_gather_rows(const void *src, int src_dtype, const int64_t *row_idx, int64_t n_src_rows, int64_t n_rows,
                               int64_t d, void *dst, int dst_dtype, double scale, void *stream) {
  using namespace sae;
  SAE_REQUIRE(src && row_idx && dst, SAE_ERR_INVALID_ARG, "gather_rows: null pointer");
  SAE_REQUIRE(n_rows > 0 && d > 0 && n_src_rows > 0 && d < (1LL << 31) && n_rows < (1LL << 31), SAE_ERR_INVALID_ARG,
              "gather_rows: bad sizes");
  SAE_REQUIRE((src_dtype == SAE_F32 || src_dtype == SAE_BF16) && (dst_dtype == SAE_F32 || dst_dtype == SAE_BF16),
              SAE_ERR_INVALID_ARG, "gather_rows: bad dtype %d -> %d", src_dtype, dst_dtype);
  hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)n_rows), block(256);
  const float sc = (float)scale;
  if (src_dtype == SAE_BF16 && dst_dtype == SAE_BF16)
    hipLaunchKernelGGL((gather_rows_kernel<true, true>), grid, block, 0, st, src, row_idx, n_src_rows, (int)d, dst, sc);
  else if (src_dtype == SAE_BF16)
    hipLaunchKernelGGL((gather_rows_kernel<true, false>), grid, block, 0, st, src, row_idx, n_src_rows, (int)d, dst, sc);
  else if (dst_dtype == SAE_BF16)
    hipLaunchKernelGGL((gather_rows_kernel<false, true>), grid, block, 0, st, src, row_idx, n_src_rows, (int)d, dst, sc);
  else
    hipLaunchKernelGGL((gather_rows_kernel<false, false>), grid, block, 0, st, src, row_idx, n_src_rows, (int)d, dst, sc);
  return check_launch("gather_rows");
}

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
