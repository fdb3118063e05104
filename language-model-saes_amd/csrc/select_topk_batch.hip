// Batch-global TopK select (BatchTopK) with fused encoder bias and decoder-norm scale (gfx950).
//
// Keeps the k_total largest positive h1 = (pre + b_enc) * scale over the WHOLE [B, F] batch
// (ties at the threshold: lowest flattened index b * F + f first) and emits the survivors as a
// sparse code with one variable-length row per token, indices ascending.
//
//   hist x3   exact radix select of the k_total-th largest key over all B * F keys: three
//             streaming passes build 11 + 11 + 9-bit digit histograms (per-wave private
//             histograms in LDS, merged with one global atomic per bin and workgroup); a
//             one-workgroup kernel after each pass picks the digit and narrows the prefix
//   count     one workgroup per token: number of keys above the threshold and equal to it
//   plan      one workgroup: prefix sums over tokens -> row offsets, and how many of each token's
//             threshold ties are kept (the first `need` ties in flattened order)
//   emit      one workgroup per token walks its row in index order and compacts the kept
//             elements with a block-wide prefix sum, so indices ascend without a sort
//
// Keys are the bit patterns of positive floats (unsigned order == float order); non-positive
// entries have key 0 and are never kept, which is the reference's relu mask.  k_total may be
// given as a host value or read from device memory (aux-k: k' * B with k' = min(k_aux, #dead)
// known only on the device).
#include "common.h"

namespace sae {

constexpr int BT_THREADS = 1024;
constexpr int BT_WAVES = BT_THREADS / 64;
constexpr int BT_BINS = 2048;

struct BatchSelState {      // lives in the workspace, one per call
  uint32_t prefix;          // bits of the threshold key decided so far
  uint32_t mask;            // which bits those are
  int64_t remaining;        // rank still to resolve inside the current prefix
  int64_t k_total;          // resolved k (min(k_total, #positives))
  int64_t n_positive;
  int32_t done;             // 1 when the threshold needs no (further) search
  uint32_t threshold;       // final: keep key > threshold, plus the first `remaining` keys == threshold
};

__device__ __forceinline__ uint32_t bt_key(float pre, float b, float s, float fm, bool has_mask) {
  float h1 = (pre + b) * s;
  if (has_mask) h1 = ((h1 / s) * fm) * s;   // aux-k: hidden_pre * dead * scale, op for op
  return h1 > 0.f ? __float_as_uint(h1) : 0u;
}

template <bool BF16>
struct BatchReader {
  const void *pre;
  const float *b_enc, *scale, *fmask;
  int F;
  // fn(f, key) for every element of row b, in any order
  template <typename Fn>
  __device__ __forceinline__ void row_for_each(int b, Fn fn) const {
    const char *row = reinterpret_cast<const char *>(pre) + (size_t)b * F * (BF16 ? 2 : 4);
    constexpr int V = BF16 ? 8 : 4;
    const bool vec_ok = (F % V == 0) && ((((uintptr_t)row | (uintptr_t)b_enc | (uintptr_t)scale | (uintptr_t)fmask) & 15) == 0);
    if (vec_ok) {
      for (int c = threadIdx.x; c < F / V; c += blockDim.x) chunk(row, c, fn);
    } else {
      for (int i = threadIdx.x; i < F; i += blockDim.x) fn(i, scalar_key(row, i));
    }
  }
  __device__ __forceinline__ uint32_t scalar_key(const char *row, int i) const {
    float p;
    if constexpr (BF16) p = bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(row)[i]);
    else p = reinterpret_cast<const float *>(row)[i];
    return bt_key(p, b_enc ? b_enc[i] : 0.f, scale ? scale[i] : 1.f, fmask ? fmask[i] : 1.f, fmask != nullptr);
  }
  template <typename Fn>
  __device__ __forceinline__ void chunk(const char *row, int c, Fn fn) const {
    constexpr int V = BF16 ? 8 : 4;
    const u32x4 raw = reinterpret_cast<const u32x4 *>(row)[c];
    float p[V], bb[V], ss[V], mm[V];
    if constexpr (BF16) {
      const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int q = 0; q < 4; ++q) { p[2 * q] = __uint_as_float(w[q] << 16); p[2 * q + 1] = __uint_as_float(w[q] & 0xffff0000u); }
    } else {
      p[0] = __uint_as_float(raw.x); p[1] = __uint_as_float(raw.y); p[2] = __uint_as_float(raw.z); p[3] = __uint_as_float(raw.w);
    }
    const int base = c * V;
    auto load = [&](const float *src, float (&dst)[V], float dflt) {
      if (src) {
#pragma unroll
        for (int q = 0; q < V / 4; ++q) {
          const float4 t = reinterpret_cast<const float4 *>(src + base)[q];
          dst[4 * q] = t.x; dst[4 * q + 1] = t.y; dst[4 * q + 2] = t.z; dst[4 * q + 3] = t.w;
        }
      } else {
#pragma unroll
        for (int e = 0; e < V; ++e) dst[e] = dflt;
      }
    };
    load(b_enc, bb, 0.f); load(scale, ss, 1.f); load(fmask, mm, 1.f);
#pragma unroll
    for (int e = 0; e < V; ++e) fn(base + e, bt_key(p[e], bb[e], ss[e], mm[e], fmask != nullptr));
  }
};

__global__ void bt_init_kernel(BatchSelState *st, uint32_t *hist, int64_t k_host, const int64_t *k_dev) {
  for (int i = threadIdx.x; i < BT_BINS; i += blockDim.x) hist[i] = 0u;
  if (threadIdx.x == 0) {
    st->prefix = 0u; st->mask = 0u; st->done = 0; st->n_positive = 0; st->threshold = 0u;
    st->k_total = k_dev ? *k_dev : k_host;
    st->remaining = st->k_total;
    if (st->k_total <= 0) { st->done = 1; st->k_total = 0; st->remaining = 0; st->threshold = 0xffffffffu; }  // keep nothing
  }
}

// digit histogram of keys matching the current prefix; grid-stride over rows
template <bool BF16>
__global__ __launch_bounds__(BT_THREADS) void bt_hist_kernel(BatchReader<BF16> rd, int B, const BatchSelState *st,
                                                             uint32_t *__restrict__ hist, int shift, int bits) {
  extern __shared__ uint32_t bt_lds[];  // BT_WAVES private histograms of (1 << bits) bins
  const int nb = 1 << bits;
  if (st->done) return;
  for (int i = threadIdx.x; i < nb * BT_WAVES; i += BT_THREADS) bt_lds[i] = 0u;
  __syncthreads();
  uint32_t *mine = bt_lds + (threadIdx.x >> 6) * nb;
  const uint32_t prefix = st->prefix, mask = st->mask, dm = (uint32_t)nb - 1u;
  for (int b = blockIdx.x; b < B; b += gridDim.x) {
    rd.row_for_each(b, [&](int, uint32_t key) {
      if (key != 0u && (key & mask) == prefix) atomicAdd(&mine[(key >> shift) & dm], 1u);
    });
  }
  __syncthreads();
  for (int i = threadIdx.x; i < nb; i += BT_THREADS) {
    uint32_t s = 0;
#pragma unroll
    for (int w = 0; w < BT_WAVES; ++w) s += bt_lds[w * nb + i];
    if (s) atomicAdd(&hist[i], s);
  }
}

// one workgroup: choose the digit in which the running count (from the top bin down) reaches `remaining`
__global__ __launch_bounds__(1024) void bt_pick_kernel(BatchSelState *st, uint32_t *hist, int shift, int bits, int first) {
  __shared__ int64_t part[1024];
  __shared__ int chosen;
  const int nb = 1 << bits, tid = threadIdx.x;
  if (st->done) { for (int i = tid; i < BT_BINS; i += 1024) hist[i] = 0u; return; }
  // thread t owns bins [hi - 2t - 1 ... ] from the top: with 2048 bins and 1024 threads, 2 bins each
  const int per = (nb + 1023) / 1024;
  int64_t local = 0;
  for (int e = 0; e < per; ++e) { const int bin = nb - 1 - (tid * per + e); if (bin >= 0) local += hist[bin]; }
  part[tid] = local;
  __syncthreads();
  for (int o = 1; o < 1024; o <<= 1) {
    const int64_t v = tid >= o ? part[tid - o] : 0;
    __syncthreads();
    part[tid] += v;
    __syncthreads();
  }
  const int64_t total = part[1023];
  if (tid == 0) chosen = -1;
  __syncthreads();
  // decisions taken by thread 0 travel through LDS (a global flag re-read by the other waves could come
  // from a stale scalar-cache line)
  __shared__ int sh_done;
  __shared__ int64_t sh_remaining;
  if (tid == 0) {
    int done = 0;
    if (first) {
      st->n_positive = total;
      if (total <= st->k_total) {  // fewer positives than k: keep every positive
        st->done = 1; st->k_total = total; st->prefix = 0u; st->mask = 0u; st->remaining = 0; st->threshold = 0u;
        done = 1;
      }
    }
    sh_done = done;
    sh_remaining = st->remaining;
  }
  __syncthreads();
  if (!sh_done) {
    const int64_t remaining = sh_remaining;
    const int64_t excl = part[tid] - local;
    if (excl < remaining && part[tid] >= remaining) {
      int64_t need = remaining - excl;
      for (int e = 0; e < per; ++e) {
        const int bin = nb - 1 - (tid * per + e);
        if (bin < 0) break;
        const int64_t h = hist[bin];
        if (h >= need) { chosen = bin; st->remaining = need; break; }
        need -= h;
      }
    }
  }
  __syncthreads();
  if (tid == 0 && chosen >= 0) {
    st->prefix |= ((uint32_t)chosen) << shift;
    st->mask |= ((uint32_t)(nb - 1)) << shift;
    if (shift == 0) st->threshold = st->prefix;
  }
  __syncthreads();
  for (int i = tid; i < BT_BINS; i += 1024) hist[i] = 0u;  // ready for the next pass
}

// per token: how many keys are above the threshold, how many equal it
template <bool BF16>
__global__ __launch_bounds__(BT_THREADS) void bt_count_kernel(BatchReader<BF16> rd, const BatchSelState *st,
                                                              int32_t *__restrict__ n_gt, int32_t *__restrict__ n_tie) {
  __shared__ int red[2 * BT_WAVES];
  const int b = blockIdx.x;
  const uint32_t T = st->threshold;
  int gt = 0, tie = 0;
  rd.row_for_each(b, [&](int, uint32_t key) { gt += key > T; tie += (key == T) && key != 0u; });
  gt = wave_sum_i(gt); tie = wave_sum_i(tie);
  if ((threadIdx.x & 63) == 0) { red[threadIdx.x >> 6] = gt; red[BT_WAVES + (threadIdx.x >> 6)] = tie; }
  __syncthreads();
  if (threadIdx.x == 0) {
    int a = 0, c = 0;
    for (int w = 0; w < BT_WAVES; ++w) { a += red[w]; c += red[BT_WAVES + w]; }
    n_gt[b] = a; n_tie[b] = c;
  }
}

// one workgroup: row offsets and per-token tie allowance (first `need` ties in flattened order)
__global__ __launch_bounds__(1024) void bt_plan_kernel(const BatchSelState *st, const int32_t *__restrict__ n_gt,
                                                       const int32_t *__restrict__ n_tie, int B,
                                                       int32_t *__restrict__ tie_keep, int64_t *__restrict__ row_off,
                                                       int32_t *__restrict__ row_nnz, int64_t *__restrict__ total_out) {
  __shared__ int64_t part[1024];
  __shared__ int64_t carry_tie, carry_off;
  const int tid = threadIdx.x;
  const int64_t need = st->done ? 0 : st->remaining;  // threshold ties that belong to the top k_total
  if (tid == 0) { carry_tie = 0; carry_off = 0; }
  __syncthreads();
  for (int b0 = 0; b0 < B; b0 += 1024) {
    const int b = b0 + tid;
    // exclusive scan of tie counts over this chunk of tokens
    const int64_t t = b < B ? n_tie[b] : 0;
    part[tid] = t;
    __syncthreads();
    for (int o = 1; o < 1024; o <<= 1) { const int64_t v = tid >= o ? part[tid - o] : 0; __syncthreads(); part[tid] += v; __syncthreads(); }
    const int64_t ties_before = carry_tie + part[tid] - t;
    const int64_t chunk_ties = part[1023];
    __syncthreads();
    int64_t keep = need - ties_before;
    keep = keep < 0 ? 0 : (keep > t ? t : keep);
    const int64_t nnz = b < B ? (int64_t)n_gt[b] + keep : 0;
    part[tid] = nnz;
    __syncthreads();
    for (int o = 1; o < 1024; o <<= 1) { const int64_t v = tid >= o ? part[tid - o] : 0; __syncthreads(); part[tid] += v; __syncthreads(); }
    if (b < B) { tie_keep[b] = (int32_t)keep; row_nnz[b] = (int32_t)nnz; row_off[b] = carry_off + part[tid] - nnz; }
    const int64_t chunk_nnz = part[1023];
    __syncthreads();
    if (tid == 0) { carry_tie += chunk_ties; carry_off += chunk_nnz; }
    __syncthreads();
  }
  if (tid == 0 && total_out) *total_out = carry_off;
}

// per token: ordered compaction of the kept elements
template <bool BF16>
__global__ __launch_bounds__(BT_THREADS) void bt_emit_kernel(BatchReader<BF16> rd, const BatchSelState *st,
                                                             const int32_t *__restrict__ tie_keep,
                                                             const int64_t *__restrict__ row_off,
                                                             int32_t *__restrict__ idx_out, float *__restrict__ val_out,
                                                             int64_t capacity) {
  __shared__ int wsum_sel[BT_WAVES], wsum_tie[BT_WAVES];
  __shared__ int run_sel, run_tie;
  const int b = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t T = st->threshold;
  const int keep_ties = tie_keep[b];
  const int64_t off = row_off[b];
  const char *row = reinterpret_cast<const char *>(rd.pre) + (size_t)b * rd.F * (BF16 ? 2 : 4);
  if (tid == 0) { run_sel = 0; run_tie = 0; }
  __syncthreads();
  constexpr int V = BF16 ? 8 : 4;
  const int F = rd.F;
  const bool vec_ok = (F % V == 0) && ((((uintptr_t)row | (uintptr_t)rd.b_enc | (uintptr_t)rd.scale | (uintptr_t)rd.fmask) & 15) == 0);
  const int per_thread = vec_ok ? V : 1;
  const int chunk_elems = BT_THREADS * per_thread;
  for (int c0 = 0; c0 < F; c0 += chunk_elems) {
    // thread tid owns elements [c0 + tid * per_thread, + per_thread): contiguous, so thread order == index order
    uint32_t keys[V];
    int n_mine = 0;
    const int base = c0 + tid * per_thread;
    if (vec_ok) {
      if (base < F) { rd.chunk(row, base / V, [&](int i, uint32_t k) { keys[i - base] = k; }); n_mine = V; }
    } else if (base < F) { keys[0] = rd.scalar_key(row, base); n_mine = 1; }
    int my_gt_or_tie = 0, my_tie = 0;
    for (int e = 0; e < n_mine; ++e) { my_tie += keys[e] == T && keys[e] != 0u; my_gt_or_tie += keys[e] > T; }
    // block-wide exclusive scans (ties, and strictly-greater) in thread order
    int inc_t = my_tie, inc_g = my_gt_or_tie;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int a = __shfl_up(inc_t, o, 64), g = __shfl_up(inc_g, o, 64);
      if (lane >= o) { inc_t += a; inc_g += g; }
    }
    if (lane == 63) { wsum_tie[wave] = inc_t; wsum_sel[wave] = inc_g; }
    __syncthreads();
    int base_t = run_tie, base_g = 0, tot_t = 0, tot_g = 0;
#pragma unroll
    for (int w = 0; w < BT_WAVES; ++w) {
      if (w < wave) { base_t += wsum_tie[w]; base_g += wsum_sel[w]; }
      tot_t += wsum_tie[w]; tot_g += wsum_sel[w];
    }
    int tie_rank = base_t + inc_t - my_tie;   // ties of this token seen before my first element
    // position among kept elements = kept greater-than before me + kept ties before me (+ row running total)
    int gt_before = base_g + inc_g - my_gt_or_tie;
    const int ties_kept_before = tie_rank < keep_ties ? tie_rank : keep_ties;
    int pos = run_sel + gt_before + (ties_kept_before - (run_tie < keep_ties ? run_tie : keep_ties));
    for (int e = 0; e < n_mine; ++e) {
      const uint32_t k = keys[e];
      bool keep = k > T;
      if (k == T && k != 0u) { keep = tie_rank < keep_ties; ++tie_rank; }
      if (keep) {
        const int64_t o = off + pos;
        if (o < capacity) {
          const int f = base + e;
          const float h1 = __uint_as_float(k);
          idx_out[o] = f;
          val_out[o] = rd.scale ? h1 / rd.scale[f] : h1;
        }
        ++pos;
      }
    }
    __syncthreads();
    if (tid == 0) {
      const int kept_t_before = run_tie < keep_ties ? run_tie : keep_ties;
      const int new_tie = run_tie + tot_t;
      const int kept_t_after = new_tie < keep_ties ? new_tie : keep_ties;
      run_sel += tot_g + (kept_t_after - kept_t_before);
      run_tie = new_tie;
    }
    __syncthreads();
  }
}

template <bool BF16>
static int run_batch_select(const void *pre, const float *b_enc, const float *scale, const float *fmask, int64_t B,
                            int64_t F, int64_t k_total, const int64_t *k_total_dev, int32_t *idx, float *val,
                            int64_t capacity, int64_t *row_off, int32_t *row_nnz, int64_t *total_out, void *workspace,
                            hipStream_t st) {
  char *ws = reinterpret_cast<char *>(workspace);
  BatchSelState *state = reinterpret_cast<BatchSelState *>(ws);
  uint32_t *hist = reinterpret_cast<uint32_t *>(ws + 256);
  int32_t *n_gt = reinterpret_cast<int32_t *>(ws + 256 + BT_BINS * 4);
  int32_t *n_tie = n_gt + B;
  int32_t *tie_keep = n_tie + B;
  BatchReader<BF16> rd{pre, b_enc, scale, fmask, (int)F};
  hipLaunchKernelGGL(bt_init_kernel, dim3(1), dim3(256), 0, st, state, hist, k_total, k_total_dev);
  const unsigned hist_grid = (unsigned)(B < 1024 ? B : 1024);
  const int shifts[3] = {20, 9, 0}, bits[3] = {11, 11, 9};  // bits 30..20, 19..9, 8..0 (bit 31 is the sign: always 0)
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(bt_hist_kernel<BF16>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (BT_WAVES << 11) * 4);
    if (e != hipSuccess) return fail(SAE_ERR_LAUNCH, "select_topk_batch: LDS reservation failed: %s", hipGetErrorString(e));
    attr_set = true;
  }
  for (int p = 0; p < 3; ++p) {
    hipLaunchKernelGGL(bt_hist_kernel<BF16>, dim3(hist_grid), dim3(BT_THREADS), (size_t)(BT_WAVES << bits[p]) * 4, st, rd,
                       (int)B, state, hist, shifts[p], bits[p]);
    hipLaunchKernelGGL(bt_pick_kernel, dim3(1), dim3(1024), 0, st, state, hist, shifts[p], bits[p], p == 0 ? 1 : 0);
  }
  hipLaunchKernelGGL(bt_count_kernel<BF16>, dim3((unsigned)B), dim3(BT_THREADS), 0, st, rd, state, n_gt, n_tie);
  hipLaunchKernelGGL(bt_plan_kernel, dim3(1), dim3(1024), 0, st, state, n_gt, n_tie, (int)B, tie_keep, row_off, row_nnz,
                     total_out);
  hipLaunchKernelGGL(bt_emit_kernel<BF16>, dim3((unsigned)B), dim3(BT_THREADS), 0, st, rd, state, tie_keep, row_off, idx,
                     val, capacity);
  return check_launch("select_topk_batch");
}

}  // namespace sae

extern "C" int64_t sae_select_topk_batch_workspace_bytes(int64_t B, int64_t F) {
  (void)F;
  if (B <= 0) return 0;
  return 256 + sae::BT_BINS * 4 + 3 * B * (int64_t)sizeof(int32_t) + 256;
}

extern "C" int sae_select_topk_batch(const void *pre, int pre_dtype, const float *b_enc, const float *scale,
                                     const float *feat_mask, int64_t B, int64_t F, int64_t k_total,
                                     const int64_t *k_total_dev, int32_t *idx, float *val, int64_t capacity,
                                     int64_t *row_off, int32_t *row_nnz, int64_t *total_out, void *workspace,
                                     int64_t workspace_bytes, void *stream) {
  using namespace sae;
  SAE_REQUIRE(pre && idx && val && row_off && row_nnz, SAE_ERR_INVALID_ARG, "select_topk_batch: null pointer");
  SAE_REQUIRE(B > 0 && F > 0 && B < (1LL << 31) && F < (1LL << 31), SAE_ERR_INVALID_ARG, "select_topk_batch: bad shape");
  SAE_REQUIRE(pre_dtype == SAE_F32 || pre_dtype == SAE_BF16, SAE_ERR_INVALID_ARG, "select_topk_batch: bad dtype %d", pre_dtype);
  SAE_REQUIRE(k_total_dev || k_total >= 0, SAE_ERR_INVALID_ARG, "select_topk_batch: k_total must be >= 0");
  SAE_REQUIRE(capacity > 0, SAE_ERR_INVALID_ARG, "select_topk_batch: capacity must be positive");
  SAE_REQUIRE(workspace && workspace_bytes >= sae_select_topk_batch_workspace_bytes(B, F), SAE_ERR_WORKSPACE,
              "select_topk_batch: workspace of %lld bytes needed", (long long)sae_select_topk_batch_workspace_bytes(B, F));
  SAE_REQUIRE((((uintptr_t)workspace) & 255) == 0, SAE_ERR_INVALID_ARG, "select_topk_batch: workspace must be 256-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (pre_dtype == SAE_BF16)
    return run_batch_select<true>(pre, b_enc, scale, feat_mask, B, F, k_total, k_total_dev, idx, val, capacity, row_off,
                                  row_nnz, total_out, workspace, st);
  return run_batch_select<false>(pre, b_enc, scale, feat_mask, B, F, k_total, k_total_dev, idx, val, capacity, row_off,
                                 row_nnz, total_out, workspace, st);
}
