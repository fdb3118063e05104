// Dense [B, F] feature activations -> sparse code (the layout the select kernels emit), in two passes:
// count the non-zeros of every token, then, given the row offsets, write each token's (feature, value) pairs in
// ascending feature order.  What get_sparse_representation does with nonzero / bincount / cumsum / scatter
// (kernels/kernels.py:14-58) before the sparse decoder kernels can run on a dense activation matrix.
#include "common.h"

namespace sae {

template <bool BF16>
__device__ __forceinline__ void load8(const void *__restrict__ row, int64_t col, int64_t F, float (&x)[8]) {
  if constexpr (BF16) {
    const uint16_t *r = reinterpret_cast<const uint16_t *>(row);
    if (col + 8 <= F && ((F & 7) == 0)) {
      const u32x4 v = *reinterpret_cast<const u32x4 *>(r + col);
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x[2 * j] = __uint_as_float(w[j] << 16);
        x[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] = col + j < F ? bf16_bits_to_f32(r[col + j]) : 0.f;
    }
  } else {
    const float *r = reinterpret_cast<const float *>(row);
    if (col + 8 <= F && ((F & 3) == 0)) {
      const float4 a = *reinterpret_cast<const float4 *>(r + col), b = *reinterpret_cast<const float4 *>(r + col + 4);
      x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w; x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] = col + j < F ? r[col + j] : 0.f;
    }
  }
}

// one workgroup per token: row_nnz[b] = #{f : dense[b, f] != 0}
template <bool BF16>
__global__ __launch_bounds__(256) void dense_row_nnz_kernel(const void *__restrict__ dense, int64_t F, int32_t *__restrict__ row_nnz) {
  __shared__ float red[4];
  const int64_t b = blockIdx.x;
  const char *row = reinterpret_cast<const char *>(dense) + b * F * (BF16 ? 2 : 4);
  int cnt = 0;
  for (int64_t col = (int64_t)threadIdx.x * 8; col < F; col += 256 * 8) {
    float x[8];
    load8<BF16>(row, col, F, x);
#pragma unroll
    for (int j = 0; j < 8; ++j) cnt += x[j] != 0.f;
  }
  const float total = block_sum<4>((float)cnt, red);     // exact: at most 2^24 non-zeros per row are countable this way
  if (threadIdx.x == 0) row_nnz[b] = (int32_t)total;
}

// one workgroup per token: the non-zeros of the row, in ascending feature order, to idx / val from row_off[b] on; entries
// that would land at or past `capacity` are not written, and `row_nnz` (optional) is cut to the entries that were, so
// that no consumer of the code walks past the arrays
template <bool BF16>
__global__ __launch_bounds__(256) void dense_to_code_kernel(const void *__restrict__ dense, int64_t F, const int64_t *__restrict__ row_off,
                                                            int32_t *__restrict__ idx, float *__restrict__ val, int64_t capacity,
                                                            int32_t *__restrict__ row_nnz) {
  __shared__ int wave_tot[4];
  const int64_t b = blockIdx.x;
  const char *row = reinterpret_cast<const char *>(dense) + b * F * (BF16 ? 2 : 4);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int64_t run = row_off[b];
  for (int64_t base = 0; base < F; base += 256 * 8) {
    const int64_t col = base + (int64_t)threadIdx.x * 8;
    float x[8];
    if (col < F) {
      load8<BF16>(row, col, F, x);
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] = 0.f;
    }
    int cnt = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) cnt += x[j] != 0.f;
    int incl = cnt;                                   // inclusive prefix over the wave's lanes
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int t = __shfl_up(incl, o, 64);
      if (lane >= o) incl += t;
    }
    __syncthreads();                                  // the previous chunk's totals have been read
    if (lane == 63) wave_tot[wave] = incl;
    __syncthreads();
    int before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const int t = wave_tot[w];
      before += w < wave ? t : 0;
      total += t;
    }
    int64_t pos = run + before + incl - cnt;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (x[j] != 0.f) {
        if (pos < capacity) {
          idx[pos] = (int32_t)(col + j);
          val[pos] = x[j];
        }
        ++pos;
      }
    }
    run += total;
  }
  if (row_nnz && threadIdx.x == 0) {
    const int64_t first = row_off[b], room = capacity > first ? capacity - first : 0, found = run - first;
    row_nnz[b] = (int32_t)(found < room ? found : room);
  }
}


// Per-layer codes of one shape, stacked layer after layer (row l * B + b holds at most k entries of layer l for token b,
// ascending features, in slots [row * k, row * k + row_nnz)), -> one code over L * F features (feature l * F + f) with
// L * k slots per token: a token's entries are its layers' entries one layer after the other, which is ascending order of
// l * F + f.  One thread per slot: it moves its own entry (if its slot holds one) and zeroes the output slot of the same
// number if that lies past the token's entries, so every output slot is written exactly once.
__global__ __launch_bounds__(256) void merge_layer_codes_kernel(const int32_t *__restrict__ idx, const float *__restrict__ val,
                                                                const int32_t *__restrict__ row_nnz, int L, int B, int k, int F,
                                                                int32_t *__restrict__ out_idx, float *__restrict__ out_val,
                                                                int64_t *__restrict__ out_row_off, int32_t *__restrict__ out_row_nnz,
                                                                int32_t *__restrict__ layer_cnt) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int per_tok = L * k;
  if (t >= (int64_t)B * per_tok) return;
  const int b = (int)(t / per_tok), s = (int)(t % per_tok), l = s / k, j = s % k;
  int before = 0, total = 0, mine = 0;
  for (int q = 0; q < L; ++q) {
    const int n = row_nnz[(size_t)q * B + b];
    before += q < l ? n : 0;
    mine = q == l ? n : mine;
    total += n;
  }
  const size_t base = (size_t)b * per_tok;
  if (j < mine) {
    const size_t src = ((size_t)l * B + b) * k + j;
    out_idx[base + before + j] = idx[src] + l * F;
    out_val[base + before + j] = val[src];
  }
  if (s >= total) { out_idx[base + s] = 0; out_val[base + s] = 0.f; }
  if (j == 0) layer_cnt[(size_t)b * L + l] = mine;
  if (s == 0) { out_row_off[b] = (int64_t)base; out_row_nnz[b] = total; }
}


// Codes of G groups over the same tokens and features, stacked group after group (row g * B + b: group g, token b, at most k
// entries in slots [row * k, row * k + row_nnz)) -> one code with every (token, feature) once: token b's entries are the
// distinct features of its G rows, in order of first appearance (group 0's entries first), each with the sum of the values
// that feature carries in the token's rows, added in group order.  One wave per token; the token's G * k entries sit in
// LDS.  Rows whose features ascend (what the select kernels write) are searched by bisection, one search per entry and
// other group; a token with a row that does not ascend has every entry compared with all of them instead (G * k <= 1024:
// at most 16 passes of 1024 broadcast reads per lane).  Same result either way.
constexpr int UNION_MAX = 1024;
__global__ __launch_bounds__(256) void union_group_codes_kernel(const int32_t *__restrict__ idx, const float *__restrict__ val,
                                                                const int32_t *__restrict__ row_nnz, int G, int B, int k,
                                                                int32_t *__restrict__ out_idx, float *__restrict__ out_val,
                                                                int64_t *__restrict__ out_row_off, int32_t *__restrict__ out_row_nnz) {
  __shared__ int32_t s_idx[4][UNION_MAX];
  __shared__ float s_val[4][UNION_MAX];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int b = blockIdx.x * 4 + wave;
  const int per_tok = b < B ? G * k : 0;   // a wave past the last token does nothing but meet the barrier
  int32_t *si = s_idx[wave];
  float *sv = s_val[wave];
  // slot s = g * k + j holds group g's j-th entry, or feature -1 past that row's entries
  for (int s = lane; s < per_tok; s += 64) {
    const int g = s / k, j = s - g * k;
    const size_t row = (size_t)g * B + b;
    const bool live = j < row_nnz[row];
    si[s] = live ? idx[row * k + j] : -1;
    sv[s] = live ? val[row * k + j] : 0.f;
  }
  __syncthreads();
  if (b >= B) return;
  const size_t base = (size_t)b * per_tok;
  // do the live entries of every row ascend?  (dead slots hold -1 and follow the live ones)
  bool bad = false;
  for (int s = lane; s < per_tok; s += 64) {
    const int j = s % k;
    bad = bad || (j > 0 && si[s] >= 0 && si[s - 1] >= si[s]);
  }
  const bool ascending = __ballot(bad) == 0ull;
  int written = 0;
  for (int s0 = 0; s0 < per_tok; s0 += 64) {
    const int s = s0 + lane;
    const int mine = s < per_tok ? si[s] : -1;
    float sum = 0.f;
    bool first = mine >= 0;
    if (ascending) {
      const int g = s / k;
      if (mine >= 0) {
        for (int q = 0; q < G; ++q) {
          if (q == g) { sum += sv[s]; continue; }
          // first slot of row q that is dead or holds a feature >= mine
          int lo = q * k, hi = lo + k;
          while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            const int v = si[mid];
            if (v >= 0 && v < mine) lo = mid + 1; else hi = mid;
          }
          if (lo < (q + 1) * k && si[lo] == mine) {
            sum += sv[lo];
            first = first && q > g;
          }
        }
      }
    } else {
      for (int q = 0; q < per_tok; ++q) {
        const bool same = si[q] == mine;
        sum += same ? sv[q] : 0.f;
        first = first && !(same && q < s);
      }
    }
    const unsigned long long keep = __ballot(first);
    if (first) {
      const int pos = written + __popcll(keep & ((1ull << lane) - 1ull));
      out_idx[base + pos] = mine;
      out_val[base + pos] = sum;
    }
    written += __popcll(keep);
  }
  for (int s = written + lane; s < per_tok; s += 64) { out_idx[base + s] = 0; out_val[base + s] = 0.f; }
  if (lane == 0) { out_row_off[b] = (int64_t)base; out_row_nnz[b] = written; }
}

}  // namespace sae

extern "C" int sae_dense_row_nnz(const void *dense, int dtype, int64_t B, int64_t F, int32_t *row_nnz, void *stream) {
  using namespace sae;
  SAE_REQUIRE(dense && row_nnz, SAE_ERR_INVALID_ARG, "dense_row_nnz: null pointer");
  SAE_REQUIRE(B > 0 && F > 0 && B < ((int64_t)1 << 31) && F < ((int64_t)1 << 31), SAE_ERR_INVALID_ARG, "dense_row_nnz: bad shape");
  SAE_REQUIRE(dtype == SAE_F32 || dtype == SAE_BF16, SAE_ERR_INVALID_ARG, "dense_row_nnz: bad dtype");
  if (dtype == SAE_BF16)
    hipLaunchKernelGGL(dense_row_nnz_kernel<true>, dim3((unsigned)B), dim3(256), 0, (hipStream_t)stream, dense, F, row_nnz);
  else
    hipLaunchKernelGGL(dense_row_nnz_kernel<false>, dim3((unsigned)B), dim3(256), 0, (hipStream_t)stream, dense, F, row_nnz);
  return check_launch("dense_row_nnz");
}

extern "C" int sae_dense_to_code(const void *dense, int dtype, int64_t B, int64_t F, const int64_t *row_off, int32_t *idx,
                                 float *val, int64_t capacity, int32_t *row_nnz, void *stream) {
  using namespace sae;
  SAE_REQUIRE(dense && row_off && idx && val, SAE_ERR_INVALID_ARG, "dense_to_code: null pointer");
  SAE_REQUIRE(B > 0 && F > 0 && B < ((int64_t)1 << 31) && F < ((int64_t)1 << 31) && capacity >= 0, SAE_ERR_INVALID_ARG,
              "dense_to_code: bad shape");
  SAE_REQUIRE(dtype == SAE_F32 || dtype == SAE_BF16, SAE_ERR_INVALID_ARG, "dense_to_code: bad dtype");
  if (dtype == SAE_BF16)
    hipLaunchKernelGGL(dense_to_code_kernel<true>, dim3((unsigned)B), dim3(256), 0, (hipStream_t)stream, dense, F, row_off, idx, val, capacity, row_nnz);
  else
    hipLaunchKernelGGL(dense_to_code_kernel<false>, dim3((unsigned)B), dim3(256), 0, (hipStream_t)stream, dense, F, row_off, idx, val, capacity, row_nnz);
  return check_launch("dense_to_code");
}

extern "C" int sae_merge_layer_codes(const int32_t *idx, const float *val, const int32_t *row_nnz, int64_t L, int64_t B, int64_t k,
                                     int64_t F, int32_t *out_idx, float *out_val, int64_t *out_row_off, int32_t *out_row_nnz,
                                     int32_t *layer_cnt, void *stream) {
  using namespace sae;
  SAE_REQUIRE(idx && val && row_nnz && out_idx && out_val && out_row_off && out_row_nnz && layer_cnt, SAE_ERR_INVALID_ARG,
              "merge_layer_codes: null pointer");
  SAE_REQUIRE(L > 0 && B > 0 && k > 0 && F > 0, SAE_ERR_INVALID_ARG, "merge_layer_codes: sizes must be positive");
  SAE_REQUIRE(L * F < ((int64_t)1 << 31) && L * k < ((int64_t)1 << 31) && B < ((int64_t)1 << 31) &&
                  B * L * k < ((int64_t)1 << 39), SAE_ERR_UNSUPPORTED, "merge_layer_codes: too large");
  const int64_t n = B * L * k;
  hipLaunchKernelGGL(merge_layer_codes_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, idx, val, row_nnz,
                     (int)L, (int)B, (int)k, (int)F, out_idx, out_val, out_row_off, out_row_nnz, layer_cnt);
  return check_launch("merge_layer_codes");
}

extern "C" int sae_union_group_codes(const int32_t *idx, const float *val, const int32_t *row_nnz, int64_t G, int64_t B, int64_t k,
                                     int32_t *out_idx, float *out_val, int64_t *out_row_off, int32_t *out_row_nnz, void *stream) {
  using namespace sae;
  SAE_REQUIRE(idx && val && row_nnz && out_idx && out_val && out_row_off && out_row_nnz, SAE_ERR_INVALID_ARG,
              "union_group_codes: null pointer");
  SAE_REQUIRE(G > 0 && B > 0 && k > 0, SAE_ERR_INVALID_ARG, "union_group_codes: sizes must be positive");
  SAE_REQUIRE(G * k <= UNION_MAX, SAE_ERR_UNSUPPORTED, "union_group_codes: more than 1024 entries per token");
  SAE_REQUIRE(B < ((int64_t)1 << 31) && G * B < ((int64_t)1 << 31), SAE_ERR_UNSUPPORTED, "union_group_codes: too many rows");
  hipLaunchKernelGGL(union_group_codes_kernel, dim3((unsigned)((B + 3) / 4)), dim3(256), 0, (hipStream_t)stream, idx, val, row_nnz,
                     (int)G, (int)B, (int)k, out_idx, out_val, out_row_off, out_row_nnz);
  return check_launch("union_group_codes");
}
