// Small streaming kernels around the hot path: casts, row norms, transposes, column sums.
// All are HBM-bound single passes with 16-byte accesses where the shape allows.
#include "common.h"

#include <mutex>

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
  // eight loads are issued before their sums (same order of additions): the loop is otherwise one load latency per row
  float s = 0.f;
  int64_t b = b0;
  for (; b + 8 <= b1; b += 8) {
    float t[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) t[q] = src[(b + q) * n + j];
#pragma unroll
    for (int q = 0; q < 8; ++q) s += t[q];
  }
  for (; b < b1; ++b) s += src[b * n + j];
  part[(int64_t)blockIdx.y * n + j] = s;
}

__global__ __launch_bounds__(256) void col_sum_final_kernel(const float *__restrict__ part, float *__restrict__ out,
                                                            int64_t n, int chunks, int accumulate) {
  const int64_t j = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (j >= n) return;
  float s = 0.f;
  int c = 0;
  for (; c + 8 <= chunks; c += 8) {
    float t[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) t[q] = part[(int64_t)(c + q) * n + j];
#pragma unroll
    for (int q = 0; q < 8; ++q) s += t[q];
  }
  for (; c < chunks; ++c) s += part[(int64_t)c * n + j];
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

// [rows, cols] fp32 or bf16 -> bf16 [cols, rows] through a 64 x 64 LDS tile.  With `mask` (fp32 [rows, cols]) an
// entry whose mask is not positive is written as 0.  With `col_part` the tile's column sums of the (masked)
// fp32 values go to col_part[tile_row, col]: summing those rows gives the column sums in a fixed order.
// VEC: rows and cols are multiples of 8 and the pointers 16-byte aligned, so every access is a whole vector.
template <bool SRC_BF16, bool VEC>
__global__ __launch_bounds__(256) void transpose_to_bf16_kernel(const void *__restrict__ src, const float *__restrict__ mask,
                                                                int64_t rows, int64_t cols, uint16_t *__restrict__ dst,
                                                                float *__restrict__ col_part) {
  __shared__ float tile[64][65];
  const int64_t r0 = (int64_t)blockIdx.y * 64, c0 = (int64_t)blockIdx.x * 64;
  const int tid = threadIdx.x;
  if constexpr (VEC) {
    constexpr int W = SRC_BF16 ? 8 : 4;          // elements per 16-byte load
    constexpr int TX = 64 / W, RP = 256 / TX;    // threads across a tile row, tile rows per pass
    const int tx = tid % TX, ty = tid / TX;
#pragma unroll
    for (int p = 0; p < 64 / RP; ++p) {
      const int i = ty + p * RP;
      const int64_t r = r0 + i, c = c0 + tx * W;
      float v[W];
#pragma unroll
      for (int e = 0; e < W; ++e) v[e] = 0.f;
      if (r < rows && c < cols) {
        const u32x4 raw = *reinterpret_cast<const u32x4 *>(reinterpret_cast<const char *>(src) + (r * cols + c) * (SRC_BF16 ? 2 : 4));
        if constexpr (SRC_BF16) {
          const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
          for (int q = 0; q < 4; ++q) { v[2 * q] = __uint_as_float(w[q] << 16); v[2 * q + 1] = __uint_as_float(w[q] & 0xffff0000u); }
        } else {
          v[0] = __uint_as_float(raw.x); v[1] = __uint_as_float(raw.y); v[2] = __uint_as_float(raw.z); v[3] = __uint_as_float(raw.w);
        }
        if (mask) {
#pragma unroll
          for (int q = 0; q < W / 4; ++q) {
            const float4 m = *reinterpret_cast<const float4 *>(mask + r * cols + c + 4 * q);
            if (!(m.x > 0.f)) v[4 * q] = 0.f;
            if (!(m.y > 0.f)) v[4 * q + 1] = 0.f;
            if (!(m.z > 0.f)) v[4 * q + 2] = 0.f;
            if (!(m.w > 0.f)) v[4 * q + 3] = 0.f;
          }
        }
      }
#pragma unroll
      for (int e = 0; e < W; ++e) tile[i][tx * W + e] = v[e];
    }
  } else {
    const int tx = tid & 63, ty = tid >> 6;
    for (int i = ty; i < 64; i += 4) {
      const int64_t r = r0 + i, c = c0 + tx;
      float v = 0.f;
      if (r < rows && c < cols) {
        if constexpr (SRC_BF16) v = bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(src)[r * cols + c]);
        else v = reinterpret_cast<const float *>(src)[r * cols + c];
        if (mask && !(mask[r * cols + c] > 0.f)) v = 0.f;
      }
      tile[i][tx] = v;
    }
  }
  __syncthreads();
  if (col_part && tid < 64 && c0 + tid < cols) {
    float s = 0.f;
#pragma unroll 8
    for (int i = 0; i < 64; ++i) s += tile[i][tid];   // rows past the matrix hold 0
    col_part[(int64_t)blockIdx.y * cols + c0 + tid] = s;
  }
  if constexpr (VEC) {
    const int tx = tid & 7, ty = tid >> 3;   // 8 threads write the 64 bf16 of one output row
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      const int cc = ty + 32 * p;
      const int64_t c = c0 + cc, r = r0 + tx * 8;
      if (c < cols && r < rows) {
        u32x4 o;
        o.x = ((uint32_t)f32_to_bf16_bits(tile[tx * 8 + 0][cc]) | ((uint32_t)f32_to_bf16_bits(tile[tx * 8 + 1][cc]) << 16));
        o.y = ((uint32_t)f32_to_bf16_bits(tile[tx * 8 + 2][cc]) | ((uint32_t)f32_to_bf16_bits(tile[tx * 8 + 3][cc]) << 16));
        o.z = ((uint32_t)f32_to_bf16_bits(tile[tx * 8 + 4][cc]) | ((uint32_t)f32_to_bf16_bits(tile[tx * 8 + 5][cc]) << 16));
        o.w = ((uint32_t)f32_to_bf16_bits(tile[tx * 8 + 6][cc]) | ((uint32_t)f32_to_bf16_bits(tile[tx * 8 + 7][cc]) << 16));
        *reinterpret_cast<u32x4 *>(dst + c * rows + r) = o;
      }
    }
  } else {
    const int tx = tid & 63, ty = tid >> 6;
    for (int i = ty; i < 64; i += 4) {
      const int64_t c = c0 + i, r = r0 + tx;
      if (c < cols && r < rows) dst[c * rows + r] = f32_to_bf16_bits(tile[tx][i]);
    }
  }
}

// One workgroup per token: the token's sparse row (idx, val in slots row_off[b] .. + row_nnz[b]) written out as a
// dense row of n_cols entries, in fp32 and / or bf16.  The row is assembled in LDS 8192 columns at a time, so every
// global write is coalesced (16 bytes per lane where the row length and the outputs' alignment allow it); indices outside
// [0, n_cols) are dropped.
constexpr int C2D_CHUNK = 8192;
__global__ __launch_bounds__(256) void code_to_dense_kernel(const int32_t *__restrict__ idx, const float *__restrict__ val,
                                                            const int64_t *__restrict__ row_off,
                                                            const int32_t *__restrict__ row_nnz, int64_t n_cols,
                                                            float *__restrict__ out_f32, uint16_t *__restrict__ out_bf16) {
  __shared__ __attribute__((aligned(16))) float row[C2D_CHUNK];
  const int64_t b = blockIdx.x;
  const int64_t off = row_off[b];
  const int n = row_nnz[b], tid = threadIdx.x;
  const bool vec = (n_cols & 7) == 0 && ((((uintptr_t)out_f32) | ((uintptr_t)out_bf16)) & 15) == 0;
  for (int64_t c0 = 0; c0 < n_cols; c0 += C2D_CHUNK) {
    const int w = (int)(n_cols - c0 < C2D_CHUNK ? n_cols - c0 : C2D_CHUNK);
    if (vec) {
      const float4 z = {0.f, 0.f, 0.f, 0.f};
      for (int i = tid * 4; i < w; i += 1024) *reinterpret_cast<float4 *>(row + i) = z;
    } else {
      for (int i = tid; i < w; i += 256) row[i] = 0.f;
    }
    __syncthreads();
    for (int s = tid; s < n; s += 256) {
      const int64_t j = (int64_t)idx[off + s] - c0;
      if (j >= 0 && j < w) row[j] = val[off + s];   // a token's indices are distinct
    }
    __syncthreads();
    if (vec) {   // 16-byte stores: rows of a multiple of 8 columns from 16-byte aligned outputs
      if (out_f32)
        for (int i = tid * 4; i < w; i += 1024)
          *reinterpret_cast<float4 *>(out_f32 + b * n_cols + c0 + i) = *reinterpret_cast<const float4 *>(row + i);
      if (out_bf16)
        for (int i = tid * 8; i < w; i += 2048) {
          const float4 lo = *reinterpret_cast<const float4 *>(row + i), hi = *reinterpret_cast<const float4 *>(row + i + 4);
          u32x4 o;
          o.x = (uint32_t)f32_to_bf16_bits(lo.x) | ((uint32_t)f32_to_bf16_bits(lo.y) << 16);
          o.y = (uint32_t)f32_to_bf16_bits(lo.z) | ((uint32_t)f32_to_bf16_bits(lo.w) << 16);
          o.z = (uint32_t)f32_to_bf16_bits(hi.x) | ((uint32_t)f32_to_bf16_bits(hi.y) << 16);
          o.w = (uint32_t)f32_to_bf16_bits(hi.z) | ((uint32_t)f32_to_bf16_bits(hi.w) << 16);
          *reinterpret_cast<u32x4 *>(out_bf16 + b * n_cols + c0 + i) = o;
        }
    } else {
      if (out_f32) for (int i = tid; i < w; i += 256) out_f32[b * n_cols + c0 + i] = row[i];
      if (out_bf16) for (int i = tid; i < w; i += 256) out_bf16[b * n_cols + c0 + i] = f32_to_bf16_bits(row[i]);
    }
    __syncthreads();
  }
}

// The same matrix transposed, [n_cols, B] in bf16 (cleared beforehand): one wave per token scatters the token's entries
// down its column.  The left operand of a product over the token axis (a dense weight gradient acts^T g).
__global__ __launch_bounds__(64) void code_to_dense_t_kernel(const int32_t *__restrict__ idx, const float *__restrict__ val,
                                                             const int64_t *__restrict__ row_off,
                                                             const int32_t *__restrict__ row_nnz, int64_t B, int64_t n_cols,
                                                             uint16_t *__restrict__ out_t) {
  const int64_t b = blockIdx.x;
  const int64_t off = row_off[b];
  const int n = row_nnz[b];
  for (int s = threadIdx.x; s < n; s += 64) {
    const int64_t j = idx[off + s];
    if (j >= 0 && j < n_cols) out_t[j * B + b] = f32_to_bf16_bits(val[off + s]);
  }
}

// One workgroup per token: squared error, aux-k residual and both output gradients in one pass over the row.
//   diff = recon - label            rec_tok[b] = w_b * sum diff^2
//   r = (label - recon) - aux       aux_tok[b] = w_b * sum r^2                       (aux given)
//   g_aux = (-2 alpha w_b) r        grad_recon = (2 w_b) diff + g_aux                (g_aux = 0 without aux)
// grad_recon is also written as bf16 when asked (the operand of the decoder's factored gradient under autocast).
__global__ __launch_bounds__(256) void mse_auxk_kernel(const float *__restrict__ recon, const float *__restrict__ label,
                                                       const float *__restrict__ aux, const float *__restrict__ tok_w,
                                                       float alpha, int d, float *__restrict__ rec_tok,
                                                       float *__restrict__ aux_tok, float *__restrict__ g_aux,
                                                       float *__restrict__ grad_recon, uint16_t *__restrict__ grad_bf16) {
  __shared__ float red[4];
  const int64_t b = blockIdx.x;
  const int tid = threadIdx.x, n4 = d >> 2;
  const float w = tok_w ? tok_w[b] : 1.f;
  const float ca = mul_rn(-2.f * alpha, w), cr = mul_rn(2.f, w);
  const float4 *rp = reinterpret_cast<const float4 *>(recon + b * d), *lp = reinterpret_cast<const float4 *>(label + b * d);
  const float4 *ap = aux ? reinterpret_cast<const float4 *>(aux + b * d) : nullptr;
  float sq_rec = 0.f, sq_aux = 0.f;
  for (int i = tid; i < n4; i += 256) {
    const float4 rc = rp[i], lb = lp[i];
    const float4 ax = ap ? ap[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    const float rv[4] = {rc.x, rc.y, rc.z, rc.w}, lv[4] = {lb.x, lb.y, lb.z, lb.w}, av[4] = {ax.x, ax.y, ax.z, ax.w};
    float go[4], ga[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float diff = sub_rn(rv[e], lv[e]);
      sq_rec = fmaf(diff, diff, sq_rec);
      ga[e] = 0.f;
      if (ap) {
        const float r = sub_rn(sub_rn(lv[e], rv[e]), av[e]);
        sq_aux = fmaf(r, r, sq_aux);
        ga[e] = mul_rn(ca, r);
      }
      go[e] = add_rn(mul_rn(cr, diff), ga[e]);
    }
    reinterpret_cast<float4 *>(grad_recon + b * d)[i] = make_float4(go[0], go[1], go[2], go[3]);
    if (ap && g_aux) reinterpret_cast<float4 *>(g_aux + b * d)[i] = make_float4(ga[0], ga[1], ga[2], ga[3]);
    if (grad_bf16) {
      uint2 o;
      o.x = (uint32_t)f32_to_bf16_bits(go[0]) | ((uint32_t)f32_to_bf16_bits(go[1]) << 16);
      o.y = (uint32_t)f32_to_bf16_bits(go[2]) | ((uint32_t)f32_to_bf16_bits(go[3]) << 16);
      reinterpret_cast<uint2 *>(grad_bf16 + b * d)[i] = o;
    }
  }
  const float tr = block_sum<4>(sq_rec, red);
  __syncthreads();
  const float ta = block_sum<4>(sq_aux, red);
  if (tid == 0) {
    rec_tok[b] = w * tr;
    if (aux_tok) aux_tok[b] = w * ta;
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

extern "C" int sae_transpose_to_bf16(const void *src, int src_dtype, const float *mask, int64_t rows, int64_t cols,
                                     void *dst, float *col_part, void *stream) {
  using namespace sae;
  SAE_REQUIRE(src && dst, SAE_ERR_INVALID_ARG, "transpose_to_bf16: null pointer");
  SAE_REQUIRE(rows > 0 && cols > 0, SAE_ERR_INVALID_ARG, "transpose_to_bf16: bad shape");
  SAE_REQUIRE(src_dtype == SAE_F32 || src_dtype == SAE_BF16, SAE_ERR_INVALID_ARG, "transpose_to_bf16: bad dtype %d", src_dtype);
  const int64_t gx = (cols + 63) / 64, gy = (rows + 63) / 64;
  SAE_REQUIRE(gy <= 65535, SAE_ERR_UNSUPPORTED, "transpose_to_bf16: rows=%lld above %d", (long long)rows, 65535 * 64);
  const bool vec = rows % 8 == 0 && cols % 8 == 0 &&
                   ((((uintptr_t)src | (uintptr_t)dst | (uintptr_t)mask) & 15) == 0);
  const dim3 grid((unsigned)gx, (unsigned)gy), block(256);
  hipStream_t st = (hipStream_t)stream;
  uint16_t *out = reinterpret_cast<uint16_t *>(dst);
  if (src_dtype == SAE_BF16) {
    if (vec) hipLaunchKernelGGL((transpose_to_bf16_kernel<true, true>), grid, block, 0, st, src, mask, rows, cols, out, col_part);
    else hipLaunchKernelGGL((transpose_to_bf16_kernel<true, false>), grid, block, 0, st, src, mask, rows, cols, out, col_part);
  } else {
    if (vec) hipLaunchKernelGGL((transpose_to_bf16_kernel<false, true>), grid, block, 0, st, src, mask, rows, cols, out, col_part);
    else hipLaunchKernelGGL((transpose_to_bf16_kernel<false, false>), grid, block, 0, st, src, mask, rows, cols, out, col_part);
  }
  return check_launch("transpose_to_bf16");
}

extern "C" int sae_code_to_dense(const int32_t *idx, const float *val, const int64_t *row_off, const int32_t *row_nnz,
                                 int64_t B, int64_t n_cols, float *dense_f32, void *dense_bf16, void *stream) {
  using namespace sae;
  SAE_REQUIRE(idx && val && row_off && row_nnz, SAE_ERR_INVALID_ARG, "code_to_dense: null pointer");
  SAE_REQUIRE(dense_f32 || dense_bf16, SAE_ERR_INVALID_ARG, "code_to_dense: no output");
  SAE_REQUIRE(B > 0 && n_cols > 0 && B < (1LL << 31), SAE_ERR_INVALID_ARG, "code_to_dense: bad shape");
  hipLaunchKernelGGL(code_to_dense_kernel, dim3((unsigned)B), dim3(256), 0, (hipStream_t)stream, idx, val, row_off, row_nnz,
                     n_cols, dense_f32, reinterpret_cast<uint16_t *>(dense_bf16));
  return check_launch("code_to_dense");
}

extern "C" int sae_code_to_dense_t(const int32_t *idx, const float *val, const int64_t *row_off, const int32_t *row_nnz,
                                   int64_t B, int64_t n_cols, void *dense_t_bf16, void *stream) {
  using namespace sae;
  SAE_REQUIRE(idx && val && row_off && row_nnz && dense_t_bf16, SAE_ERR_INVALID_ARG, "code_to_dense_t: null pointer");
  SAE_REQUIRE(B > 0 && n_cols > 0 && B < (1LL << 31), SAE_ERR_INVALID_ARG, "code_to_dense_t: bad shape");
  const int rc = zero_fill(dense_t_bf16, (size_t)B * (size_t)n_cols * 2, (hipStream_t)stream);
  if (rc) return rc;
  hipLaunchKernelGGL(code_to_dense_t_kernel, dim3((unsigned)B), dim3(64), 0, (hipStream_t)stream, idx, val, row_off, row_nnz, B,
                     n_cols, reinterpret_cast<uint16_t *>(dense_t_bf16));
  return check_launch("code_to_dense_t");
}

extern "C" int sae_mse_auxk_fused(const float *recon, const float *label, const float *aux_recon, const float *tok_w,
                                  double alpha, int64_t B, int64_t d, float *rec_tok, float *aux_tok, float *g_aux,
                                  float *grad_recon, void *grad_recon_bf16, void *stream) {
  using namespace sae;
  SAE_REQUIRE(recon && label && rec_tok && grad_recon, SAE_ERR_INVALID_ARG, "mse_auxk_fused: null pointer");
  SAE_REQUIRE(!aux_recon || (aux_tok && g_aux), SAE_ERR_INVALID_ARG, "mse_auxk_fused: aux_tok and g_aux go with aux_recon");
  SAE_REQUIRE(B > 0 && d > 0 && d % 4 == 0 && d < (1LL << 31) && B < (1LL << 31), SAE_ERR_INVALID_ARG,
              "mse_auxk_fused: bad shape (d must be a multiple of 4)");
  SAE_REQUIRE((((uintptr_t)recon | (uintptr_t)label | (uintptr_t)aux_recon | (uintptr_t)g_aux | (uintptr_t)grad_recon |
                (uintptr_t)grad_recon_bf16) & 15) == 0, SAE_ERR_INVALID_ARG, "mse_auxk_fused: 16-byte alignment required");
  hipLaunchKernelGGL(mse_auxk_kernel, dim3((unsigned)B), dim3(256), 0, (hipStream_t)stream, recon, label, aux_recon, tok_w,
                     (float)alpha, (int)d, rec_tok, aux_recon ? aux_tok : nullptr, g_aux, grad_recon,
                     reinterpret_cast<uint16_t *>(grad_recon_bf16));
  return check_launch("mse_auxk_fused");
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

// ---- column sums with the partial sums in a fixed device array --------------------------------------
// The partial sums of sae_col_sum live in caller-supplied workspace.  Callers that cannot allocate one
// (code under graph capture, serving loops) use this array instead: 64 chunks x SAE_COL_SUM_STATIC_MAX_N
// floats = 4 MiB, held by every device the library runs on until the process ends.
static __device__ __align__(256) float scratch[64 * SAE_COL_SUM_STATIC_MAX_N];

namespace {
constexpr int kMaxDevices = 64;
float *g_scratch_ptr[kMaxDevices] = {nullptr};   // device address of `scratch`, one per device
std::mutex g_scratch_mutex;

// Device address of this device's copy of `scratch` (the array's name is a host-side handle, not an address).
int scratch_address(float **out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return sae::fail(SAE_ERR_LAUNCH, "col_sum_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return sae::fail(SAE_ERR_UNSUPPORTED, "col_sum_static: device %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    float *ptr = nullptr;
    e = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return sae::fail(SAE_ERR_LAUNCH, "col_sum_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return SAE_OK;
}
}  // namespace

extern "C" int sae_col_sum_static(const float *src, float *out, int64_t B, int64_t n, int accumulate, void *stream) {
  using namespace sae;
  SAE_REQUIRE(src && out, SAE_ERR_INVALID_ARG, "col_sum_static: null pointer");
  SAE_REQUIRE(B > 0 && n > 0, SAE_ERR_INVALID_ARG, "col_sum_static: bad shape");
  SAE_REQUIRE(n <= SAE_COL_SUM_STATIC_MAX_N, SAE_ERR_UNSUPPORTED,
              "col_sum_static: n = %lld exceeds the fixed scratch array's %d columns; use sae_col_sum with a workspace",
              (long long)n, (int)SAE_COL_SUM_STATIC_MAX_N);
  float *part = nullptr;
  const int rc = scratch_address(&part);
  if (rc != SAE_OK) return rc;
  // Same grid, chunking and order of additions as sae_col_sum, so the bits are the same.  Every partial the
  // second kernel reads (chunks x n) is written by the first, so nothing left by an earlier call is seen.
  const int chunks = (int)(B < 64 ? B : 64);
  const int rows_per = (int)((B + chunks - 1) / chunks);
  const unsigned gx = (unsigned)((n + 255) / 256);
  hipLaunchKernelGGL(col_sum_partial_kernel, dim3(gx, (unsigned)chunks), dim3(256), 0, (hipStream_t)stream, src, part, B, n, rows_per);
  hipLaunchKernelGGL(col_sum_final_kernel, dim3(gx), dim3(256), 0, (hipStream_t)stream, part, out, n, chunks, accumulate);
  return check_launch("col_sum_static");
}
