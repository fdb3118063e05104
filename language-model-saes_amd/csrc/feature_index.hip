// Feature-major index of a sparse code, and the weight-gradient rows built from it (gfx950).
//
// The select kernels emit the code token-major (slots of token 0, then token 1, ...).  The
// weight gradients need the transpose: for every feature, the slots that name it.
//
//   count   one global atomic per valid slot into counts[F]; also records slot -> token
//   scan    exclusive prefix sum over counts -> feat_ptr[F + 1] (tile sums, scan of sums, finish)
//   fill    slot ids dropped into their feature's segment through a per-feature cursor
//   order   every segment is put into ascending slot order, so the result (and every sum
//           taken over a segment afterwards) is independent of the order in which the
//           atomics of `fill` landed: short segments by a rank count inside one wave, long
//           ones by a bitmap counting sort over the token range.
//
// The gradient kernel then owns one feature per workgroup and writes the whole [d] row:
// sum over the segment of coef[slot] * dense[token(slot), :].  Features with an empty
// segment get zeros, so no clearing pass over the [F, d] gradient is needed, and no atomics
// touch it.
#include "common.h"

namespace sae {

constexpr int FI_THREADS = 256;

__global__ void fi_zero_kernel(int32_t *p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

// one wave per token; lanes stride over its slots
__global__ __launch_bounds__(FI_THREADS) void fi_count_kernel(const int32_t *__restrict__ idx,
                                                              const int64_t *__restrict__ row_off,
                                                              const int32_t *__restrict__ row_nnz, int B, int F,
                                                              int32_t *__restrict__ counts,
                                                              int32_t *__restrict__ slot_tok) {
  const int b = blockIdx.x * (FI_THREADS / 64) + (threadIdx.x >> 6);
  if (b >= B) return;
  const int lane = threadIdx.x & 63;
  const int64_t off = row_off[b];
  const int nnz = row_nnz[b];
  for (int j = lane; j < nnz; j += 64) {
    const int f = idx[off + j];
    if ((unsigned)f < (unsigned)F) atomicAdd(&counts[f], 1);
    slot_tok[off + j] = b;
  }
}

// Exclusive scan of counts[F] in three small launches: per-tile sums (1024 counters per
// workgroup, coalesced), a one-workgroup scan of the tile sums, per-tile scan + tile offset.
constexpr int SCAN_TILE = 1024;  // counters per workgroup (256 threads x 4)

__device__ __forceinline__ int block_excl_scan_256(int v, int *lds_wave, int &total) {
  // exclusive scan over 256 threads; lds_wave holds 4 ints
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  int incl = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int t = __shfl_up(incl, o, 64);
    if (lane >= o) incl += t;
  }
  __syncthreads();
  if (lane == 63) lds_wave[w] = incl;
  __syncthreads();
  int base = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) base += (i < w) ? lds_wave[i] : 0;
  total = lds_wave[0] + lds_wave[1] + lds_wave[2] + lds_wave[3];
  return base + incl - v;
}

__global__ __launch_bounds__(256) void fi_tile_sum_kernel(const int32_t *__restrict__ counts, int F,
                                                          int32_t *__restrict__ tile_sums) {
  __shared__ int lds_wave[4];
  const int base = blockIdx.x * SCAN_TILE + threadIdx.x * 4;
  int s = 0;
#pragma unroll
  for (int e = 0; e < 4; ++e) s += (base + e < F) ? counts[base + e] : 0;
  int total;
  block_excl_scan_256(s, lds_wave, total);
  if (threadIdx.x == 0) tile_sums[blockIdx.x] = total;
}

// one workgroup; n_tiles is small (F / 1024), handled in chunks of 256
__global__ __launch_bounds__(256) void fi_tile_scan_kernel(int32_t *__restrict__ tile_sums, int n_tiles,
                                                           int32_t *__restrict__ feat_ptr, int F) {
  __shared__ int lds_wave[4];
  int carry = 0;
  for (int c0 = 0; c0 < n_tiles; c0 += 256) {
    const int i = c0 + threadIdx.x;
    const int v = i < n_tiles ? tile_sums[i] : 0;
    int total;
    const int ex = block_excl_scan_256(v, lds_wave, total);
    if (i < n_tiles) tile_sums[i] = carry + ex;
    carry += total;
    __syncthreads();
  }
  if (threadIdx.x == 0) feat_ptr[F] = carry;
}

__global__ __launch_bounds__(256) void fi_tile_finish_kernel(const int32_t *__restrict__ counts, int F,
                                                             const int32_t *__restrict__ tile_offsets,
                                                             int32_t *__restrict__ feat_ptr,
                                                             int32_t *__restrict__ cursor) {
  __shared__ int lds_wave[4];
  const int base = blockIdx.x * SCAN_TILE + threadIdx.x * 4;
  int c[4];
  int s = 0;
#pragma unroll
  for (int e = 0; e < 4; ++e) { c[e] = (base + e < F) ? counts[base + e] : 0; s += c[e]; }
  int total;
  int run = tile_offsets[blockIdx.x] + block_excl_scan_256(s, lds_wave, total);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (base + e < F) { feat_ptr[base + e] = run; cursor[base + e] = run; }
    run += c[e];
  }
}

__global__ __launch_bounds__(FI_THREADS) void fi_fill_kernel(const int32_t *__restrict__ idx,
                                                             const int64_t *__restrict__ row_off,
                                                             const int32_t *__restrict__ row_nnz, int B, int F,
                                                             int32_t *__restrict__ cursor,
                                                             int32_t *__restrict__ feat_slot) {
  const int b = blockIdx.x * (FI_THREADS / 64) + (threadIdx.x >> 6);
  if (b >= B) return;
  const int lane = threadIdx.x & 63;
  const int64_t off = row_off[b];
  const int nnz = row_nnz[b];
  for (int j = lane; j < nnz; j += 64) {
    const int f = idx[off + j];
    if ((unsigned)f < (unsigned)F) {
      const int pos = atomicAdd(&cursor[f], 1);
      feat_slot[pos] = (int32_t)(off + j);
    }
  }
}

// Put every segment into ascending slot order (out of place: `unordered` -> feat_slot).
// One wave per feature handles segments of up to 64 slots with a rank count across lanes.
__global__ __launch_bounds__(FI_THREADS) void fi_order_kernel(const int32_t *__restrict__ feat_ptr, int F,
                                                              const int32_t *__restrict__ unordered,
                                                              int32_t *__restrict__ feat_slot) {
  const int f = blockIdx.x * (FI_THREADS / 64) + (threadIdx.x >> 6);
  if (f >= F) return;
  const int lane = threadIdx.x & 63;
  const int lo = feat_ptr[f], hi = feat_ptr[f + 1];
  const int len = hi - lo;
  if (len == 0 || len > 64) return;
  const int mine = lane < len ? unordered[lo + lane] : 0x7fffffff;
  int rank = 0;
  for (int j = 0; j < len; ++j) rank += __shfl(mine, j, 64) < mine;
  if (lane < len) feat_slot[lo + rank] = mine;
}

// Segments longer than 64 slots: a workgroup runs a counting sort keyed by token.  A feature occurs at most once
// per token, so a bitmap over the B tokens plus a prefix popcount gives every slot its rank.
// LDS: bitmap[ceil(B/32)] + prefix[ceil(B/32)].  Workgroup w looks at features w, w + gridDim.x, ... (FI_THREADS
// of them per round, one per thread), lists the long ones in LDS and sorts them one after another: a sparse code
// has few long segments, and a grid of one workgroup per feature spent its time starting workgroups that left
// at once.
constexpr int FI_LONG_GRID = 16384;
__global__ __launch_bounds__(FI_THREADS) void fi_order_long_kernel(const int32_t *__restrict__ feat_ptr, int F,
                                                                   const int32_t *__restrict__ unordered,
                                                                   const int32_t *__restrict__ slot_tok, int B,
                                                                   int32_t *__restrict__ feat_slot) {
  extern __shared__ uint32_t fi_lds[];
  __shared__ int32_t part[FI_THREADS / 64];
  __shared__ int32_t long_list[FI_THREADS];
  __shared__ int32_t n_long;
  const int tid = threadIdx.x;
  const int W = (B + 31) >> 5;
  uint32_t *bitmap = fi_lds;
  uint32_t *prefix = fi_lds + W;
  for (int64_t first = blockIdx.x; first < F; first += (int64_t)gridDim.x * FI_THREADS) {
    if (tid == 0) n_long = 0;
    __syncthreads();
    const int64_t mine = first + (int64_t)tid * gridDim.x;
    if (mine < F && feat_ptr[mine + 1] - feat_ptr[mine] > 64) long_list[atomicAdd(&n_long, 1)] = (int32_t)mine;
    __syncthreads();
    const int nl = n_long;
    for (int q = 0; q < nl; ++q) {
      const int f = long_list[q];
      const int lo = feat_ptr[f], hi = feat_ptr[f + 1];
      for (int w = tid; w < W; w += FI_THREADS) bitmap[w] = 0u;
      __syncthreads();
      for (int i = lo + tid; i < hi; i += FI_THREADS) {
        const int t = slot_tok[unordered[i]];
        atomicOr(&bitmap[t >> 5], 1u << (t & 31));
      }
      __syncthreads();
      const int per = (W + FI_THREADS - 1) / FI_THREADS;
      const int wlo = tid * per, whi = min(W, wlo + per);
      int s = 0;
      for (int w = wlo; w < whi; ++w) s += __popc(bitmap[w]);
      int incl = s;   // inclusive scan inside the wave, then the waves' totals through LDS
      for (int o = 1; o < 64; o <<= 1) {
        const int v = __shfl_up(incl, o);
        if ((tid & 63) >= o) incl += v;
      }
      if ((tid & 63) == 63) part[tid >> 6] = incl;
      __syncthreads();
      int run = incl - s;
      for (int w = 0; w < (tid >> 6); ++w) run += part[w];
      for (int w = wlo; w < whi; ++w) {
        prefix[w] = (uint32_t)run;
        run += __popc(bitmap[w]);
      }
      __syncthreads();
      for (int i = lo + tid; i < hi; i += FI_THREADS) {
        const int slot = unordered[i];
        const int t = slot_tok[slot];
        const int rank = (int)prefix[t >> 5] + __popc(bitmap[t >> 5] & ((1u << (t & 31)) - 1u));
        feat_slot[lo + rank] = slot;
      }
      __syncthreads();   // the bitmap is cleared again for the next feature
    }
  }
}

// out[f, :] = sum_{s in segment f} coef[s] * dense[slot_tok[s], :]
template <bool DENSE_BF16>
__global__ __launch_bounds__(FI_THREADS) void sparse_grad_rows_kernel(
    const int32_t *__restrict__ feat_ptr, const int32_t *__restrict__ feat_slot,
    const int32_t *__restrict__ slot_tok, const float *__restrict__ coef, const void *__restrict__ dense,
    float *__restrict__ out, float *__restrict__ bias_out, int d) {
  const int f = blockIdx.x, tid = threadIdx.x;
  const int lo = feat_ptr[f], hi = feat_ptr[f + 1];
  const int n_seg = d >> 2;  // float4 segments of the output row
  const size_t row_bytes = (size_t)d * (DENSE_BF16 ? 2 : 4);
  const char *dbase = reinterpret_cast<const char *>(dense);
  float *orow = out + (size_t)f * d;

  if (bias_out && tid < 64) {
    float s = 0.f;
    for (int i = lo + tid; i < hi; i += 64) s += coef[feat_slot[i]];
    s = wave_sum(s);
    if (tid == 0) bias_out[f] = s;
  }
  for (int seg0 = tid; seg0 < n_seg; seg0 += FI_THREADS * 4) {
    float4 acc[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) acc[u] = make_float4(0.f, 0.f, 0.f, 0.f);
    gather_rows_fma<DENSE_BF16, FI_THREADS>(acc, lo, hi, feat_slot, slot_tok, coef, dbase, row_bytes, seg0, n_seg);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int seg = seg0 + u * FI_THREADS;
      if (seg < n_seg) reinterpret_cast<float4 *>(orow)[seg] = acc[u];
    }
  }
}

}  // namespace sae

extern "C" int64_t sae_feature_index_workspace_bytes(int64_t B, int64_t F, int64_t n_slots) {
  (void)B;
  if (F <= 0 || n_slots <= 0) return 0;
  // counts[F] + cursor[F] + unordered slots[n_slots] + scan tile sums[ceil(F / 1024)]
  return (int64_t)sizeof(int32_t) * (2 * F + n_slots + (F + 1023) / 1024) + 256;
}

extern "C" int sae_build_feature_index(const int32_t *idx, const int64_t *row_off, const int32_t *row_nnz, int64_t B,
                                       int64_t F, int64_t n_slots, int32_t *feat_ptr, int32_t *feat_slot,
                                       int32_t *slot_tok, void *workspace, int64_t workspace_bytes, void *stream) {
  using namespace sae;
  SAE_REQUIRE(idx && row_off && row_nnz && feat_ptr && feat_slot && slot_tok, SAE_ERR_INVALID_ARG,
              "build_feature_index: null pointer");
  SAE_REQUIRE(B > 0 && F > 0 && n_slots > 0, SAE_ERR_INVALID_ARG, "build_feature_index: sizes must be positive");
  SAE_REQUIRE(B < (1LL << 31) && F < (1LL << 31) - 1 && n_slots < (1LL << 31), SAE_ERR_UNSUPPORTED,
              "build_feature_index: size too large for 32-bit slots");
  SAE_REQUIRE(B <= 131072, SAE_ERR_UNSUPPORTED, "build_feature_index: B=%lld above 131072 tokens per call", (long long)B);
  SAE_REQUIRE(workspace && workspace_bytes >= sae_feature_index_workspace_bytes(B, F, n_slots), SAE_ERR_WORKSPACE,
              "build_feature_index: workspace of %lld bytes needed", (long long)sae_feature_index_workspace_bytes(B, F, n_slots));
  hipStream_t st = (hipStream_t)stream;
  int32_t *counts = reinterpret_cast<int32_t *>(workspace);
  int32_t *cursor = counts + F;
  int32_t *unordered = cursor + F;
  int32_t *tile_sums = unordered + n_slots;
  hipLaunchKernelGGL(fi_zero_kernel, dim3((unsigned)((F + 255) / 256)), dim3(256), 0, st, counts, F);
  const unsigned tok_blocks = (unsigned)((B + (FI_THREADS / 64) - 1) / (FI_THREADS / 64));
  hipLaunchKernelGGL(fi_count_kernel, dim3(tok_blocks), dim3(FI_THREADS), 0, st, idx, row_off, row_nnz, (int)B, (int)F,
                     counts, slot_tok);
  const int n_tiles = (int)((F + SCAN_TILE - 1) / SCAN_TILE);
  hipLaunchKernelGGL(fi_tile_sum_kernel, dim3(n_tiles), dim3(256), 0, st, counts, (int)F, tile_sums);
  hipLaunchKernelGGL(fi_tile_scan_kernel, dim3(1), dim3(256), 0, st, tile_sums, n_tiles, feat_ptr, (int)F);
  hipLaunchKernelGGL(fi_tile_finish_kernel, dim3(n_tiles), dim3(256), 0, st, counts, (int)F, tile_sums, feat_ptr, cursor);
  hipLaunchKernelGGL(fi_fill_kernel, dim3(tok_blocks), dim3(FI_THREADS), 0, st, idx, row_off, row_nnz, (int)B, (int)F,
                     cursor, unordered);
  const unsigned feat_blocks = (unsigned)((F + (FI_THREADS / 64) - 1) / (FI_THREADS / 64));
  hipLaunchKernelGGL(fi_order_kernel, dim3(feat_blocks), dim3(FI_THREADS), 0, st, feat_ptr, (int)F, unordered, feat_slot);
  const size_t bitmap_lds = (size_t)2 * ((B + 31) / 32) * sizeof(uint32_t);
  hipLaunchKernelGGL(fi_order_long_kernel, dim3((unsigned)(F < FI_LONG_GRID ? F : FI_LONG_GRID)), dim3(FI_THREADS), bitmap_lds,
                     st, feat_ptr, (int)F, unordered, slot_tok, (int)B, feat_slot);
  return check_launch("build_feature_index");
}

extern "C" int sae_sparse_grad_rows(const int32_t *feat_ptr, const int32_t *feat_slot, const int32_t *slot_tok,
                                    const float *coef, const void *dense, int dense_dtype, float *out, float *bias_out,
                                    int64_t F, int64_t d, void *stream) {
  using namespace sae;
  SAE_REQUIRE(feat_ptr && feat_slot && slot_tok && coef && dense && out, SAE_ERR_INVALID_ARG,
              "sparse_grad_rows: null pointer");
  SAE_REQUIRE(F > 0 && d > 0, SAE_ERR_INVALID_ARG, "sparse_grad_rows: F and d must be positive");
  SAE_REQUIRE(dense_dtype == SAE_F32 || dense_dtype == SAE_BF16, SAE_ERR_INVALID_ARG, "sparse_grad_rows: bad dtype %d", dense_dtype);
  SAE_REQUIRE(d % 4 == 0, SAE_ERR_UNSUPPORTED, "sparse_grad_rows: d_model=%lld must be a multiple of 4", (long long)d);
  SAE_REQUIRE(F < (1LL << 31), SAE_ERR_UNSUPPORTED, "sparse_grad_rows: F too large");
  hipStream_t st = (hipStream_t)stream;
  if (dense_dtype == SAE_BF16)
    hipLaunchKernelGGL(sparse_grad_rows_kernel<true>, dim3((unsigned)F), dim3(FI_THREADS), 0, st, feat_ptr, feat_slot,
                       slot_tok, coef, dense, out, bias_out, (int)d);
  else
    hipLaunchKernelGGL(sparse_grad_rows_kernel<false>, dim3((unsigned)F), dim3(FI_THREADS), 0, st, feat_ptr, feat_slot,
                       slot_tok, coef, dense, out, bias_out, (int)d);
  return check_launch("sparse_grad_rows");
}

namespace sae {

// out_x[f] = sum over feature f's slots of x[slot], for up to two per-slot arrays at once; one wave per feature,
// lane-strided partial sums added in a fixed order.
__global__ __launch_bounds__(256) void fi_segment_sums_kernel(const int32_t *__restrict__ feat_ptr, const int32_t *__restrict__ feat_slot,
                                                              const float *__restrict__ a, const float *__restrict__ b, int F,
                                                              float *__restrict__ out_a, float *__restrict__ out_b) {
  const int f = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (f >= F) return;
  const int lo = feat_ptr[f], hi = feat_ptr[f + 1];
  float sa = 0.f, sb = 0.f;
  for (int i = lo + lane; i < hi; i += 64) {
    const int sl = feat_slot[i];
    sa += a[sl];
    if (b) sb += b[sl];
  }
  sa = wave_sum(sa);
  if (b) sb = wave_sum(sb);
  if (lane == 0) {
    out_a[f] = sa;
    if (b) out_b[f] = sb;
  }
}

}  // namespace sae

extern "C" int sae_feature_segment_sums(const int32_t *feat_ptr, const int32_t *feat_slot, const float *a, const float *b, int64_t F,
                                        float *out_a, float *out_b, void *stream) {
  using namespace sae;
  SAE_REQUIRE(feat_ptr && feat_slot && a && out_a && (!b || out_b), SAE_ERR_INVALID_ARG, "feature_segment_sums: null pointer");
  SAE_REQUIRE(F > 0 && F < (1LL << 31), SAE_ERR_INVALID_ARG, "feature_segment_sums: bad F");
  hipLaunchKernelGGL(fi_segment_sums_kernel, dim3((unsigned)((F + 3) / 4)), dim3(256), 0, (hipStream_t)stream, feat_ptr, feat_slot, a, b,
                     (int)F, out_a, out_b);
  return check_launch("feature_segment_sums");
}
