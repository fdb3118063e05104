// Per-token TopK select with fused encoder bias and decoder-norm scale (gfx950).
//
// One workgroup of 1024 threads owns one token's row of F pre-activations.  The key of an
// element is the bit pattern of h1 = (pre + b_enc) * scale when h1 > 0 and 0 otherwise: for
// positive floats unsigned-integer order equals float order, and non-positive entries can
// never be kept (the reference applies a relu mask before the top-k).
//
// Fast path (two streaming reads of the row, no histogram over the row):
//   1. every thread takes the maximum key of the elements it owns; the k-th largest of those
//      1024 maxima is a lower bound L of the k-th largest key of the row, because k distinct
//      elements are >= L;
//   2. every element with key >= L is appended to a candidate list in LDS -- for i.i.d. data about
//      k + a few elements.  Rows of up to 131072 elements are not read again for this: pass 1 keeps
//      the largest key of every 16-byte chunk in registers, which is enough to rule out all but a
//      handful of chunks, and only those are re-formed from memory (the bias and scale vectors
//      cost four times the row's own bytes per pass, so a second pass over memory is what the
//      kernel's time would otherwise go to).  Longer rows are read a second time;
//   3. an exact radix select over the candidates in LDS yields the threshold key T; among
//      the candidates with key == T the lowest indices win (a second radix select over the
//      indices); the kept elements are ranked by index and written in ascending order.
// General path (any row, any k <= 4096): the same exact select, but with the 8-bit-digit
// histograms taken over the whole row in global memory.  It is used when the candidate list
// would overflow (massive ties, k above the thread count) and by the tests, which check both
// paths against each other.
#include "common.h"

namespace sae {

constexpr int SEL_THREADS = 1024;
constexpr int SEL_WAVES = SEL_THREADS / 64;
constexpr int SEL_CAP = 4096;      // candidate capacity == largest supported k
constexpr int SEL_MAX_K = 4096;
constexpr int SEL_ROW_FLAG = -1;   // row_nnz of a row the granule kernel left to the general kernel

struct SelShared {
  uint32_t cand_key[SEL_CAP];
  int32_t cand_idx[SEL_CAP];
  uint32_t tmax[SEL_THREADS];
  uint32_t hist[256];
  int32_t count;        // candidates appended
  uint32_t prefix;      // radix-select state
  int32_t remaining;
  int32_t digit_found;
};

// LOWP: the arithmetic of a dictionary whose parameters are bf16 tensors -- the sum with the bias and the product
// with the norm are each rounded to bf16, as the tensors `x @ W_E + b_E` and `hidden_pre * decoder_norm()` are
// (models/sae.py:324-335 with cfg.dtype = bfloat16); the bias and scale arrive as fp32 copies of bf16 values.
__device__ __forceinline__ float sel_bf16_round(float x) { return bf16_round(x); }
// ARITH selects the arithmetic at compile time: the masked (aux-k) form costs registers that the plain form,
// which runs every step, should not pay for (with one kernel for both, 14 registers per lane were spilled).
// LOWP_MASKED: the aux-k keys of such a dictionary, `hidden_pre * is_dead * decoder_norm` with hidden_pre the bf16
// quotient the encoder returned (models/sparse_dictionary.py:958-966): one more rounding after each operation.
constexpr int SEL_PLAIN = 0, SEL_LOWP = 1, SEL_MASKED = 2, SEL_LOWP_MASKED = 3;
constexpr bool sel_has_mask(int arith) { return arith == SEL_MASKED || arith == SEL_LOWP_MASKED; }
constexpr bool sel_is_lowp(int arith) { return arith == SEL_LOWP || arith == SEL_LOWP_MASKED; }
template <int ARITH>
__device__ __forceinline__ uint32_t key_of(float pre, float b, float s, float fm) {
  if constexpr (ARITH == SEL_PLAIN) return select_key_plain(pre, b, s);
  float h1;
  if constexpr (ARITH == SEL_LOWP) {
    h1 = sel_bf16_round(mul_rn(sel_bf16_round(add_rn(pre, b)), s));
  } else if constexpr (ARITH == SEL_LOWP_MASKED) {
    h1 = sel_bf16_round(mul_rn(sel_bf16_round(add_rn(pre, b)), s));
    h1 = sel_bf16_round(h1 / s);
    h1 = sel_bf16_round(mul_rn(sel_bf16_round(mul_rn(h1, fm)), s));
  } else {
    h1 = (pre + b) * s;
    h1 = ((h1 / s) * fm) * s;  // aux-k: hidden_pre * dead * scale, op for op
  }
  return h1 > 0.f ? __float_as_uint(h1) : 0u;
}

// Scan hist[255..0] from the top and find the bin where the running count reaches
// `remaining`.  Executed by wave 0; results go to sh->prefix / sh->remaining.
template <typename SH>
__device__ __forceinline__ void pick_digit(SH *sh, int shift) {
  if (threadIdx.x < 64) {
    const int lane = threadIdx.x;
    // lane 0 owns the top four bins (255..252), lane 63 the bottom four
    const int top = 255 - 4 * lane;
    const uint32_t h0 = sh->hist[top], h1 = sh->hist[top - 1], h2 = sh->hist[top - 2], h3 = sh->hist[top - 3];
    const int local = (int)(h0 + h1 + h2 + h3);
    int incl = local;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int t = __shfl_up(incl, o, 64);
      if (lane >= o) incl += t;
    }
    const int excl = incl - local;
    const int remaining = sh->remaining;
    if (excl < remaining && incl >= remaining) {
      int need = remaining - excl;  // still to take inside my four bins
      int bin;
      if ((int)h0 >= need) bin = top;
      else if ((int)(h0 + h1) >= need) { bin = top - 1; need -= (int)h0; }
      else if ((int)(h0 + h1 + h2) >= need) { bin = top - 2; need -= (int)(h0 + h1); }
      else { bin = top - 3; need -= (int)(h0 + h1 + h2); }
      sh->prefix |= ((uint32_t)bin) << shift;
      sh->remaining = need;
      sh->digit_found = 1;
    }
  }
}

// Exact k-th largest of `n` keys held in LDS (n >= k >= 1).  On return (after the final
// barrier) sh->prefix is that key and sh->remaining the number of elements equal to it that
// belong to the top k.  `xform` maps a stored key to the ordering key.
template <int THREADS = SEL_THREADS, typename SH, typename KeyAt>
__device__ __forceinline__ void lds_kth_largest(SH *sh, int n, int k, KeyAt key_at) {
  if (threadIdx.x == 0) { sh->prefix = 0u; sh->remaining = k; }
  uint32_t mask = 0u;
#pragma unroll 1
  for (int shift = 24; shift >= 0; shift -= 8) {
    if (threadIdx.x < 256) sh->hist[threadIdx.x] = 0u;
    __syncthreads();
    const uint32_t prefix = sh->prefix;
    for (int i = threadIdx.x; i < n; i += THREADS) {
      const uint32_t key = key_at(i);
      if ((key & mask) == prefix) atomicAdd(&sh->hist[(key >> shift) & 255u], 1u);
    }
    __syncthreads();
    pick_digit(sh, shift);
    mask |= 255u << shift;
    __syncthreads();
  }
}

template <bool BF16, int ARITH = SEL_PLAIN>
struct RowReader {
  const void *row;
  const float *b_enc;
  const float *scale;
  const float *fmask;
  int F;
  static constexpr int V = BF16 ? 8 : 4;  // elements per 16-byte load
  __device__ __forceinline__ bool vec_ok() const {
    return (F % V == 0) && (((((uintptr_t)row) | (uintptr_t)b_enc | (uintptr_t)scale | (uintptr_t)fmask) & 15) == 0);
  }
  // keys of the V elements of 16-byte chunk c
  __device__ __forceinline__ u32x4 load_raw(int c) const { return reinterpret_cast<const u32x4 *>(row)[c]; }
  __device__ __forceinline__ void chunk_keys(int c, uint32_t (&keys)[V]) const { keys_from_raw(c, load_raw(c), keys); }
  __device__ __forceinline__ void keys_from_raw(int c, const u32x4 &raw, uint32_t (&keys)[V]) const {
    float pre[V];
    if constexpr (BF16) {
      const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        pre[2 * q] = __uint_as_float(w[q] << 16);
        pre[2 * q + 1] = __uint_as_float(w[q] & 0xffff0000u);
      }
    } else {
      pre[0] = __uint_as_float(raw.x); pre[1] = __uint_as_float(raw.y);
      pre[2] = __uint_as_float(raw.z); pre[3] = __uint_as_float(raw.w);
    }
    const int base = c * V;
    float bb[V], ss[V], mm[V];
    if constexpr (sel_has_mask(ARITH)) {
#pragma unroll
      for (int q = 0; q < V / 4; ++q) {
        const float4 t = reinterpret_cast<const float4 *>(fmask + base)[q];
        mm[4 * q] = t.x; mm[4 * q + 1] = t.y; mm[4 * q + 2] = t.z; mm[4 * q + 3] = t.w;
      }
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) mm[e] = 1.f;
    }
    if (b_enc) {
#pragma unroll
      for (int q = 0; q < V / 4; ++q) {
        const float4 t = reinterpret_cast<const float4 *>(b_enc + base)[q];
        bb[4 * q] = t.x; bb[4 * q + 1] = t.y; bb[4 * q + 2] = t.z; bb[4 * q + 3] = t.w;
      }
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) bb[e] = 0.f;
    }
    if (scale) {
#pragma unroll
      for (int q = 0; q < V / 4; ++q) {
        const float4 t = reinterpret_cast<const float4 *>(scale + base)[q];
        ss[4 * q] = t.x; ss[4 * q + 1] = t.y; ss[4 * q + 2] = t.z; ss[4 * q + 3] = t.w;
      }
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) ss[e] = 1.f;
    }
#pragma unroll
    for (int e = 0; e < V; ++e) keys[e] = key_of<ARITH>(pre[e], bb[e], ss[e], mm[e]);
  }
  // key of one element
  __device__ __forceinline__ uint32_t key_at(int i) const {
    float pre;
    if constexpr (BF16) pre = bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(row)[i]);
    else pre = reinterpret_cast<const float *>(row)[i];
    return key_of<ARITH>(pre, b_enc ? b_enc[i] : 0.f, scale ? scale[i] : 1.f, sel_has_mask(ARITH) ? fmask[i] : 1.f);
  }
  // calls fn(index, key) for every element of the row, vectorised when the row allows it
  template <typename Fn>
  __device__ __forceinline__ void for_each(Fn fn) const {
    if (vec_ok()) {
      const int n_chunks = F / V;
      for (int c = threadIdx.x; c < n_chunks; c += SEL_THREADS) {
        uint32_t keys[V];
        chunk_keys(c, keys);
#pragma unroll
        for (int e = 0; e < V; ++e) fn(c * V + e, keys[e]);
      }
    } else {
      for (int i = threadIdx.x; i < F; i += SEL_THREADS) fn(i, key_at(i));
    }
  }
};

// Exact k-th largest over the whole row in global memory (general path).
template <bool BF16, int ARITH>
__device__ __forceinline__ void row_kth_largest(SelShared *sh, const RowReader<BF16, ARITH> &rr, int k) {
  if (threadIdx.x == 0) { sh->prefix = 0u; sh->remaining = k; }
  uint32_t mask = 0u;
#pragma unroll 1
  for (int shift = 24; shift >= 0; shift -= 8) {
    if (threadIdx.x < 256) sh->hist[threadIdx.x] = 0u;
    __syncthreads();
    const uint32_t prefix = sh->prefix;
    rr.for_each([&](int, uint32_t key) {
      if (key != 0u && (key & mask) == prefix) atomicAdd(&sh->hist[(key >> shift) & 255u], 1u);
    });
    __syncthreads();
    pick_digit(sh, shift);
    mask |= 255u << shift;
    __syncthreads();
  }
}

// STASH: the row has at most SEL_STASH_ELEMS elements per thread and is 16-byte addressable.  Pass 1 then
// keeps the largest key of every 16-byte chunk it reads in a register (16 or 32 per thread), and pass 2
// walks those registers instead of reading the row, its bias and its scale a second time: a chunk can only
// contribute to the candidate list if its largest key is >= the bound, and only those chunks (k plus a
// handful per row) are formed again from memory.
constexpr int SEL_STASH_ELEMS = 128;  // per thread: rows up to 131072 elements

template <bool BF16, bool STASH, int ARITH = SEL_PLAIN>
__global__ __launch_bounds__(SEL_THREADS, 8) void select_topk_row_kernel(
    const void *__restrict__ pre, const float *__restrict__ b_enc, const float *__restrict__ scale,
    const float *__restrict__ fmask, int F, int k,
    int32_t *__restrict__ idx_out, float *__restrict__ val_out, int64_t *__restrict__ row_off,
    int32_t *__restrict__ row_nnz, int cand_cap, int only_flagged, int rows_per_group, int pre_rows) {
  __shared__ SelShared sh;
  const int b = blockIdx.x;
  const int tid = threadIdx.x;
  int src_row = b;
  if (only_flagged) {     // the pass after the granule kernel: the rows it gave up on, with their group's bias / scale
    if (row_nnz[b] != SEL_ROW_FLAG) return;
    const size_t grp = (size_t)(b / rows_per_group);
    if (b_enc) b_enc += grp * F;
    if (scale) scale += grp * F;
    src_row = b % pre_rows;  // groups that share one matrix of pre_rows rows
  }
  RowReader<BF16, ARITH> rr;
  rr.row = reinterpret_cast<const char *>(pre) + (size_t)src_row * F * (BF16 ? 2 : 4);
  rr.b_enc = b_enc;
  rr.scale = scale;
  rr.fmask = fmask;
  rr.F = F;

  // ---- pass 1: per-thread maximum key and number of positive elements ----
  uint32_t my_max = 0u;
  int my_pos = 0;
  constexpr int V = RowReader<BF16, ARITH>::V;
  constexpr int NCH = SEL_STASH_ELEMS / V;            // chunks per thread when stashing
  uint32_t cmax[STASH ? NCH : 1];                     // largest key of each of this thread's chunks
  if constexpr (STASH) {
    const int n_chunks = F / V;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int c = tid + j * SEL_THREADS;
      uint32_t m = 0u;
      if (c < n_chunks) {
        uint32_t keys[V];
        rr.chunk_keys(c, keys);
#pragma unroll
        for (int e = 0; e < V; ++e) {
          m = keys[e] > m ? keys[e] : m;
          my_pos += keys[e] != 0u;
        }
      }
      cmax[j] = m;
      my_max = m > my_max ? m : my_max;
    }
  } else {
    rr.for_each([&](int, uint32_t key) {
      my_max = key > my_max ? key : my_max;
      my_pos += key != 0u;
    });
  }
  sh.tmax[tid] = my_max;
  if (tid == 0) sh.count = 0;
  // total positives in the row
  int pos = wave_sum_i(my_pos);
  __syncthreads();
  if ((tid & 63) == 0) sh.hist[tid >> 6] = (uint32_t)pos;
  __syncthreads();
  int n_pos = 0;
#pragma unroll
  for (int w = 0; w < SEL_WAVES; ++w) n_pos += (int)sh.hist[w];
  __syncthreads();

  const int k_eff = n_pos < k ? n_pos : k;  // how many elements will be kept
  bool general = false;
  uint32_t T = 0u;       // threshold key: keep key > T and `need` lowest-index elements with key == T
  int need = 0;
  int n_cand = 0;

  if (k_eff == 0) {
    if (tid == 0) { row_off[b] = (int64_t)b * k; row_nnz[b] = 0; }
    for (int i = tid; i < k; i += SEL_THREADS) { idx_out[(size_t)b * k + i] = 0; val_out[(size_t)b * k + i] = 0.f; }
    return;
  }

  if (n_pos <= k) {
    // fewer positives than k: everything positive is kept
    if (n_pos > cand_cap) general = true;  // cannot happen for k <= cand_cap; kept for safety
    T = 0u; need = 0;
  } else if (k <= SEL_THREADS) {
    // ---- lower bound L from the per-thread maxima ----
    lds_kth_largest(&sh, SEL_THREADS, k, [&](int i) { return sh.tmax[i]; });
    T = sh.prefix;  // = L for now (may be 0 when fewer than k threads saw a positive)
    __syncthreads();
  } else {
    general = true;
  }

  if (!general) {
    // ---- pass 2: gather candidates with key >= L (and key > 0) into LDS ----
    const uint32_t L = (n_pos <= k) ? 1u : (T == 0u ? 1u : T);
    auto consider = [&](int i, uint32_t key) {
      if (key >= L) {
        const int slot = atomicAdd(&sh.count, 1);
        if (slot < cand_cap) { sh.cand_key[slot] = key; sh.cand_idx[slot] = i; }
      }
    };
    if constexpr (STASH) {
      // only chunks whose largest key reaches L can contribute: k plus a handful per row; those are read again
#pragma unroll
      for (int j = 0; j < NCH; ++j) {
        if (cmax[j] >= L) {
          const int c = tid + j * SEL_THREADS;
          uint32_t keys[V];
          rr.chunk_keys(c, keys);
#pragma unroll
          for (int e = 0; e < V; ++e) consider(c * V + e, keys[e]);
        }
      }
    } else {
      rr.for_each(consider);
    }
    __syncthreads();
    n_cand = sh.count;
    if (n_cand > cand_cap) general = true;
  }

  if (general) {
    // ---- general path: exact threshold over the whole row ----
    __syncthreads();
    row_kth_largest<BF16, ARITH>(&sh, rr, k_eff);
    T = sh.prefix;
    need = sh.remaining;  // elements equal to T that are kept
    __syncthreads();
    // lowest `need` indices among the ties: radix select over ~idx restricted to key == T.
    // Count ties first; if all ties are kept no index threshold is needed.
    if (tid == 0) sh.count = 0;
    __syncthreads();
    int my_ties = 0;
    rr.for_each([&](int, uint32_t key) { my_ties += key == T; });
    my_ties = wave_sum_i(my_ties);
    if ((tid & 63) == 0 && my_ties) atomicAdd(&sh.count, my_ties);
    __syncthreads();
    const int n_ties = sh.count;
    uint32_t idx_limit = 0xffffffffu;  // keep ties with idx <= idx_limit
    __syncthreads();
    if (n_ties > need) {
      if (tid == 0) { sh.prefix = 0u; sh.remaining = need; }
      uint32_t mask = 0u;
#pragma unroll 1
      for (int shift = 24; shift >= 0; shift -= 8) {
        if (tid < 256) sh.hist[tid] = 0u;
        __syncthreads();
        const uint32_t prefix = sh.prefix;
        rr.for_each([&](int i, uint32_t key) {
          const uint32_t ik = ~(uint32_t)i;
          if (key == T && (ik & mask) == prefix) atomicAdd(&sh.hist[(ik >> shift) & 255u], 1u);
        });
        __syncthreads();
        pick_digit(&sh, shift);
        mask |= 255u << shift;
        __syncthreads();
      }
      idx_limit = ~sh.prefix;
      __syncthreads();
    }
    // emit the kept elements into the candidate arrays (exactly k_eff of them)
    if (tid == 0) sh.count = 0;
    __syncthreads();
    rr.for_each([&](int i, uint32_t key) {
      if (key > T || (key == T && key != 0u && (uint32_t)i <= idx_limit)) {
        const int slot = atomicAdd(&sh.count, 1);
        if (slot < SEL_CAP) { sh.cand_key[slot] = key; sh.cand_idx[slot] = i; }
      }
    });
    __syncthreads();
    n_cand = sh.count < SEL_CAP ? sh.count : SEL_CAP;  // == k_eff
  } else if (n_cand > k_eff) {
    // ---- exact threshold among the candidates ----
    lds_kth_largest(&sh, n_cand, k_eff, [&](int i) { return sh.cand_key[i]; });
    T = sh.prefix;
    need = sh.remaining;
    __syncthreads();
    // ties: keep the `need` lowest indices among candidates with key == T
    int my_ties = 0;
    for (int i = tid; i < n_cand; i += SEL_THREADS) my_ties += sh.cand_key[i] == T;
    if (tid == 0) sh.count = 0;
    __syncthreads();
    my_ties = wave_sum_i(my_ties);
    if ((tid & 63) == 0 && my_ties) atomicAdd(&sh.count, my_ties);
    __syncthreads();
    const int n_ties = sh.count;
    __syncthreads();
    uint32_t idx_limit = 0xffffffffu;
    if (n_ties > need) {
      lds_kth_largest(&sh, n_cand, need, [&](int i) { return sh.cand_key[i] == T ? ~(uint32_t)sh.cand_idx[i] : 0u; });
      idx_limit = ~sh.prefix;
      __syncthreads();
    }
    // mark dropped candidates by clearing their key
    for (int i = tid; i < n_cand; i += SEL_THREADS) {
      const uint32_t key = sh.cand_key[i];
      const bool keep = key > T || (key == T && (uint32_t)sh.cand_idx[i] <= idx_limit);
      if (!keep) sh.cand_key[i] = 0u;
    }
    __syncthreads();
  }

  // ---- rank the kept candidates by index and write them out in ascending order ----
  for (int i = tid; i < n_cand; i += SEL_THREADS) {
    const uint32_t key = sh.cand_key[i];
    if (key == 0u) continue;
    const int my_idx = sh.cand_idx[i];
    int rank = 0;
    for (int j = 0; j < n_cand; ++j) rank += (sh.cand_key[j] != 0u) && (sh.cand_idx[j] < my_idx);
    const float h1 = __uint_as_float(key);
    const float s = scale ? scale[my_idx] : 1.f;
    if (rank < k) {
      idx_out[(size_t)b * k + rank] = my_idx;
      val_out[(size_t)b * k + rank] = scale ? (sel_is_lowp(ARITH) ? sel_bf16_round(h1 / s) : h1 / s) : h1;
    }
  }
  for (int i = k_eff + tid; i < k; i += SEL_THREADS) { idx_out[(size_t)b * k + i] = 0; val_out[(size_t)b * k + i] = 0.f; }
  if (tid == 0) { row_off[b] = (int64_t)b * k; row_nnz[b] = k_eff; }
}

}  // namespace sae

namespace sae {
static int select_topk_row_impl(bool lowp, const void *pre, int pre_dtype, const float *b_enc, const float *scale,
                                const float *feat_mask, int64_t B, int64_t F, int k, int32_t *idx, float *val,
                                int64_t *row_off, int32_t *row_nnz, int cand_cap, void *stream, int only_flagged = 0,
                                int rows_per_group = 1, int pre_rows = 1) {
  SAE_REQUIRE(pre && idx && val && row_off && row_nnz, SAE_ERR_INVALID_ARG, "select_topk_row: null pointer");
  SAE_REQUIRE(B > 0 && F > 0, SAE_ERR_INVALID_ARG, "select_topk_row: B and F must be positive");
  SAE_REQUIRE(pre_dtype == SAE_F32 || pre_dtype == SAE_BF16, SAE_ERR_INVALID_ARG, "select_topk_row: bad dtype %d", pre_dtype);
  SAE_REQUIRE(k >= 1 && k <= SEL_MAX_K, SAE_ERR_UNSUPPORTED, "select_topk_row: k=%d outside [1, %d]", k, SEL_MAX_K);
  SAE_REQUIRE(F < (1LL << 31) && B < (1LL << 31), SAE_ERR_UNSUPPORTED, "select_topk_row: size too large");
  SAE_REQUIRE(cand_cap >= 0 && cand_cap <= SEL_CAP, SAE_ERR_INVALID_ARG, "select_topk_row: cand_cap outside [0, %d]", SEL_CAP);
  hipStream_t st = (hipStream_t)stream;
  const int V = pre_dtype == SAE_BF16 ? 8 : 4;
  const size_t row_bytes = (size_t)F * (pre_dtype == SAE_BF16 ? 2 : 4);
  // every row 16-byte addressable and short enough for the register stash
  const bool stash = (F % V == 0) && F <= (int64_t)SEL_STASH_ELEMS * SEL_THREADS && (row_bytes % 16 == 0) &&
                     (((((uintptr_t)pre) | (uintptr_t)b_enc | (uintptr_t)scale | (uintptr_t)feat_mask) & 15) == 0);
#define SAE_LAUNCH_SELECT(BF, ST, ...)                                                                                     \
  hipLaunchKernelGGL((select_topk_row_kernel<BF, ST, ##__VA_ARGS__>), dim3((unsigned)B), dim3(SEL_THREADS), 0, st, pre, b_enc, \
                     scale, feat_mask, (int)F, k, idx, val, row_off, row_nnz, cand_cap, only_flagged, rows_per_group, pre_rows)
  if (lowp && feat_mask) {
    if (stash) SAE_LAUNCH_SELECT(true, true, SEL_LOWP_MASKED); else SAE_LAUNCH_SELECT(true, false, SEL_LOWP_MASKED);
  } else if (lowp) {
    if (stash) SAE_LAUNCH_SELECT(true, true, SEL_LOWP); else SAE_LAUNCH_SELECT(true, false, SEL_LOWP);
  } else if (feat_mask) {
    if (pre_dtype == SAE_BF16) {
      if (stash) SAE_LAUNCH_SELECT(true, true, SEL_MASKED); else SAE_LAUNCH_SELECT(true, false, SEL_MASKED);
    } else {
      if (stash) SAE_LAUNCH_SELECT(false, true, SEL_MASKED); else SAE_LAUNCH_SELECT(false, false, SEL_MASKED);
    }
  } else if (pre_dtype == SAE_BF16) {
    if (stash) SAE_LAUNCH_SELECT(true, true); else SAE_LAUNCH_SELECT(true, false);
  } else {
    if (stash) SAE_LAUNCH_SELECT(false, true); else SAE_LAUNCH_SELECT(false, false);
  }
#undef SAE_LAUNCH_SELECT
  return check_launch("select_topk_row");
}
// ---- select from per-granule maxima -----------------------------------------------------------------------------
// The encoder GEMM can leave, next to pre [B, F] (bf16), the largest key of every aligned granule of 64 features
// (gmax [B, F / 64]).  The k-th largest granule maximum is a lower bound L of the row's k-th largest key (k distinct
// elements reach it), and only granules whose maximum reaches L can hold a kept element: about k of them.  One
// workgroup of 256 threads per token reads the granule maxima (F / 16 bytes instead of the row's 2 F), radix-selects
// L among them in LDS, re-forms the keys of the qualifying granules from memory and finishes like the kernel above:
// exact threshold among the candidates, lowest indices among ties, ascending order.  Rows whose candidates do not fit
// (mass ties) are flagged in row_nnz and redone by the general kernel in a second launch that skips every other row.
constexpr int GS_THREADS = 256;
constexpr int GS_CAP = 1024;            // candidates per row
constexpr int GS_QCAP = 1024;           // qualifying granules per row
constexpr int GS_MAX_K = 512;
constexpr int GS_MAX_GRANULES = 4096;   // F <= 262144

struct GsShared {
  uint32_t cand_key[GS_CAP];
  int32_t cand_idx[GS_CAP];
  uint16_t q[GS_QCAP];
  uint32_t hist[256];
  int32_t count, qcount, gpos;
  uint32_t prefix;
  int32_t remaining, digit_found;
};

// ARITH: SEL_PLAIN, or SEL_LOWP for maxima and keys in the bf16 arithmetic of a dictionary held in bf16
template <int ARITH>
__global__ __launch_bounds__(GS_THREADS) void select_topk_row_granule_kernel(
    const uint16_t *__restrict__ pre, const uint32_t *__restrict__ gmax, const float *__restrict__ b_enc,
    const float *__restrict__ scale, int F, int k, int32_t *__restrict__ idx_out, float *__restrict__ val_out,
    int64_t *__restrict__ row_off, int32_t *__restrict__ row_nnz, int rows_per_group, int pre_rows) {
  __shared__ GsShared sh;
  extern __shared__ __attribute__((aligned(16))) uint32_t gk[];   // the row's granule maxima
  const int b = blockIdx.x, tid = threadIdx.x, ng = F >> 6;
  {   // rows are stacked group after group, each group with a bias / scale vector of its own
    const size_t grp = (size_t)(b / rows_per_group);
    if (b_enc) b_enc += grp * F;
    if (scale) scale += grp * F;
  }
  RowReader<true, ARITH> rr;
  rr.row = pre + (size_t)(b % pre_rows) * F;     // pre_rows < number of rows: the groups share one matrix of pre_rows rows
  rr.b_enc = b_enc;
  rr.scale = scale;
  rr.fmask = nullptr;
  rr.F = F;
  if (tid == 0) { sh.count = 0; sh.qcount = 0; sh.gpos = 0; }
  __syncthreads();
  int my_pos = 0;
  const uint32_t *grow = gmax + (size_t)b * ng;
  for (int g = tid; g < ng; g += GS_THREADS) {
    const uint32_t key = grow[g];
    gk[g] = key;
    my_pos += key != 0u;
  }
  my_pos = wave_sum_i(my_pos);
  if ((tid & 63) == 0 && my_pos) atomicAdd(&sh.gpos, my_pos);
  __syncthreads();
  const int n_gpos = sh.gpos;
  if (n_gpos == 0) {        // no positive element in the row
    if (tid == 0) { row_off[b] = (int64_t)b * k; row_nnz[b] = 0; }
    for (int i = tid; i < k; i += GS_THREADS) { idx_out[(size_t)b * k + i] = 0; val_out[(size_t)b * k + i] = 0.f; }
    return;
  }
  // with fewer than k positive granules every positive element is a candidate (their count decides how many are kept)
  uint32_t L = 1u;
  if (n_gpos >= k) {
    lds_kth_largest<GS_THREADS>(&sh, ng, k, [&](int i) { return gk[i]; });
    L = sh.prefix;
    __syncthreads();
  }
  for (int g = tid; g < ng; g += GS_THREADS) {
    if (gk[g] >= L) {
      const int slot = atomicAdd(&sh.qcount, 1);
      if (slot < GS_QCAP) sh.q[slot] = (uint16_t)g;
    }
  }
  __syncthreads();
  const int nq = sh.qcount;
  bool give_up = nq > GS_QCAP;
  if (!give_up) {
    for (int p = tid; p < nq * 8; p += GS_THREADS) {     // one 16-byte chunk of a qualifying granule per thread and round
      const int c = (int)sh.q[p >> 3] * 8 + (p & 7);
      uint32_t keys[8];
      rr.chunk_keys(c, keys);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (keys[e] >= L) {
          const int slot = atomicAdd(&sh.count, 1);
          if (slot < GS_CAP) { sh.cand_key[slot] = keys[e]; sh.cand_idx[slot] = c * 8 + e; }
        }
      }
    }
    __syncthreads();
    give_up = sh.count > GS_CAP;
  }
  if (give_up) {
    if (tid == 0) row_nnz[b] = SEL_ROW_FLAG;
    return;
  }
  const int n_cand = sh.count;
  const int k_eff = n_cand < k ? n_cand : k;
  if (n_cand > k_eff) {
    // ---- exact threshold among the candidates ----
    lds_kth_largest<GS_THREADS>(&sh, n_cand, k_eff, [&](int i) { return sh.cand_key[i]; });
    const uint32_t T = sh.prefix;
    const int need = sh.remaining;
    __syncthreads();
    int my_ties = 0;
    for (int i = tid; i < n_cand; i += GS_THREADS) my_ties += sh.cand_key[i] == T;
    if (tid == 0) sh.count = 0;
    __syncthreads();
    my_ties = wave_sum_i(my_ties);
    if ((tid & 63) == 0 && my_ties) atomicAdd(&sh.count, my_ties);
    __syncthreads();
    const int n_ties = sh.count;
    __syncthreads();
    uint32_t idx_limit = 0xffffffffu;
    if (n_ties > need) {     // ties at the threshold: the lowest indices are kept
      lds_kth_largest<GS_THREADS>(&sh, n_cand, need, [&](int i) { return sh.cand_key[i] == T ? ~(uint32_t)sh.cand_idx[i] : 0u; });
      idx_limit = ~sh.prefix;
      __syncthreads();
    }
    for (int i = tid; i < n_cand; i += GS_THREADS) {
      const uint32_t key = sh.cand_key[i];
      const bool keep = key > T || (key == T && (uint32_t)sh.cand_idx[i] <= idx_limit);
      if (!keep) sh.cand_key[i] = 0u;
    }
    __syncthreads();
  }
  // ---- rank the kept candidates by index and write them out in ascending order ----
  for (int i = tid; i < n_cand; i += GS_THREADS) {
    const uint32_t key = sh.cand_key[i];
    if (key == 0u) continue;
    const int my_idx = sh.cand_idx[i];
    int rank = 0;
    for (int j = 0; j < n_cand; ++j) rank += (sh.cand_key[j] != 0u) && (sh.cand_idx[j] < my_idx);
    const float h1 = __uint_as_float(key);
    if (rank < k) {
      idx_out[(size_t)b * k + rank] = my_idx;
      float v = h1;
      if (scale) { v = h1 / scale[my_idx]; if (sel_is_lowp(ARITH)) v = sel_bf16_round(v); }
      val_out[(size_t)b * k + rank] = v;
    }
  }
  for (int i = k_eff + tid; i < k; i += GS_THREADS) { idx_out[(size_t)b * k + i] = 0; val_out[(size_t)b * k + i] = 0.f; }
  if (tid == 0) { row_off[b] = (int64_t)b * k; row_nnz[b] = k_eff; }
}

// Granule maxima of rows that no GEMM epilogue left them for: eight lanes per granule (one 16-byte chunk each), eight
// granules per wave.  A lane keeps its chunk of bias and scale (64 bytes) for R consecutive rows of one group, so a row
// costs its own 16 bytes of pre; the launch uses R = 8 when the groups are multiples of 8 rows and R = 1 otherwise.
// With `groups` > 1 the rows are `groups` repeats of the same pre rows, one repeat per group of bias and scale (row
// g * n_rows + r reads pre row r): the lane keeps its R chunks of pre and walks the groups, so pre is read once.
template <int R>
__global__ __launch_bounds__(256) void granule_max_kernel(const uint16_t *__restrict__ pre, const float *__restrict__ b_enc,
                                                          const float *__restrict__ scale, int F, int64_t n_rows, int64_t n_items,
                                                          int rows_per_group, int pre_rows, int groups,
                                                          uint32_t *__restrict__ gmax) {
  const int64_t item = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 3;   // (block of R rows, granule)
  if (item >= n_items) return;            // the eight lanes of an item leave together
  const int part = threadIdx.x & 7, ng = F >> 6;
  const int64_t row0 = (item / ng) * R;
  const int gi = (int)(item % ng);
  const int c = gi * 8 + part;
  u32x4 raw[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int64_t row = row0 + r < n_rows ? row0 + r : n_rows - 1;
    raw[r] = reinterpret_cast<const u32x4 *>(pre + (size_t)(row % pre_rows) * F)[c];
  }
  for (int g = 0; g < groups; ++g) {
  const size_t grp = groups > 1 ? (size_t)g : (size_t)(row0 / rows_per_group);
  uint32_t *gout = gmax + (size_t)g * n_rows * ng;
  float bb[8], ss[8];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const float4 zb = {0.f, 0.f, 0.f, 0.f}, os = {1.f, 1.f, 1.f, 1.f};
    const float4 t = b_enc ? reinterpret_cast<const float4 *>(b_enc + grp * F + (size_t)c * 8)[q] : zb;
    const float4 u = scale ? reinterpret_cast<const float4 *>(scale + grp * F + (size_t)c * 8)[q] : os;
    bb[4 * q] = t.x; bb[4 * q + 1] = t.y; bb[4 * q + 2] = t.z; bb[4 * q + 3] = t.w;
    ss[4 * q] = u.x; ss[4 * q + 1] = u.y; ss[4 * q + 2] = u.z; ss[4 * q + 3] = u.w;
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const uint32_t w[4] = {raw[r].x, raw[r].y, raw[r].z, raw[r].w};
    uint32_t m = 0u;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint32_t k0 = key_of<SEL_PLAIN>(__uint_as_float(w[q] << 16), bb[2 * q], ss[2 * q], 1.f);
      const uint32_t k1 = key_of<SEL_PLAIN>(__uint_as_float(w[q] & 0xffff0000u), bb[2 * q + 1], ss[2 * q + 1], 1.f);
      m = k0 > m ? k0 : m;
      m = k1 > m ? k1 : m;
    }
#pragma unroll
    for (int o = 1; o < 8; o <<= 1) {
      const uint32_t t = (uint32_t)__shfl_xor((int)m, o, 64);
      m = t > m ? t : m;
    }
    if (part == 0 && row0 + r < n_rows) gout[(size_t)(row0 + r) * ng + gi] = m;
  }
  }
}

}  // namespace sae

namespace sae {
static int select_topk_row_granule_impl(bool lowp, const void *pre_bf16, const uint32_t *granule_max, const float *b_enc,
                                        const float *scale, int64_t B, int64_t F, int k, int64_t rows_per_group, int64_t pre_rows,
                                        int32_t *idx, float *val, int64_t *row_off, int32_t *row_nnz, void *stream) {
  SAE_REQUIRE(pre_bf16 && granule_max && idx && val && row_off && row_nnz, SAE_ERR_INVALID_ARG, "select_topk_row_granule: null pointer");
  SAE_REQUIRE(B > 0 && F > 0 && B < (1LL << 31), SAE_ERR_INVALID_ARG, "select_topk_row_granule: bad sizes");
  if (rows_per_group <= 0) rows_per_group = B;
  if (pre_rows <= 0) pre_rows = B;
  SAE_REQUIRE(pre_rows <= B && B % pre_rows == 0, SAE_ERR_INVALID_ARG, "select_topk_row_granule: B=%lld is not a multiple of pre_rows=%lld",
              (long long)B, (long long)pre_rows);
  SAE_REQUIRE(B % rows_per_group == 0, SAE_ERR_INVALID_ARG, "select_topk_row_granule: B=%lld is not a multiple of rows_per_group=%lld",
              (long long)B, (long long)rows_per_group);
  SAE_REQUIRE(F % 64 == 0 && F / 64 <= GS_MAX_GRANULES, SAE_ERR_UNSUPPORTED,
              "select_topk_row_granule: F=%lld must be a multiple of 64, at most %d", (long long)F, 64 * GS_MAX_GRANULES);
  SAE_REQUIRE(k >= 1 && k <= GS_MAX_K, SAE_ERR_UNSUPPORTED, "select_topk_row_granule: k=%d outside [1, %d]", k, GS_MAX_K);
  SAE_REQUIRE((((uintptr_t)pre_bf16 | (uintptr_t)b_enc | (uintptr_t)scale) & 15) == 0, SAE_ERR_INVALID_ARG,
              "select_topk_row_granule: pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (lowp)
    hipLaunchKernelGGL(select_topk_row_granule_kernel<SEL_LOWP>, dim3((unsigned)B), dim3(GS_THREADS), (size_t)(F / 64) * 4, st,
                       (const uint16_t *)pre_bf16, granule_max, b_enc, scale, (int)F, k, idx, val, row_off, row_nnz, (int)rows_per_group,
                       (int)pre_rows);
  else
    hipLaunchKernelGGL(select_topk_row_granule_kernel<SEL_PLAIN>, dim3((unsigned)B), dim3(GS_THREADS), (size_t)(F / 64) * 4, st,
                       (const uint16_t *)pre_bf16, granule_max, b_enc, scale, (int)F, k, idx, val, row_off, row_nnz, (int)rows_per_group,
                       (int)pre_rows);
  const int rc = check_launch("select_topk_row_granule");
  if (rc != SAE_OK) return rc;
  // rows the granule kernel flagged (mass ties) are redone from the whole row; every other workgroup leaves at once
  return select_topk_row_impl(lowp, pre_bf16, SAE_BF16, b_enc, scale, nullptr, B, F, k, idx, val, row_off, row_nnz, SEL_CAP, stream, 1,
                              (int)rows_per_group, (int)pre_rows);
}
}  // namespace sae

extern "C" int sae_select_topk_row_granule(const void *pre_bf16, const uint32_t *granule_max, const float *b_enc,
                                           const float *scale, int64_t B, int64_t F, int k, int64_t rows_per_group, int64_t pre_rows,
                                           int32_t *idx, float *val, int64_t *row_off, int32_t *row_nnz, void *stream) {
  return sae::select_topk_row_granule_impl(false, pre_bf16, granule_max, b_enc, scale, B, F, k, rows_per_group, pre_rows, idx, val,
                                           row_off, row_nnz, stream);
}

extern "C" int sae_select_topk_row_granule_lowp(const void *pre_bf16, const uint32_t *granule_max, const float *b_enc,
                                                const float *scale, int64_t B, int64_t F, int k, int64_t rows_per_group, int64_t pre_rows,
                                                int32_t *idx, float *val, int64_t *row_off, int32_t *row_nnz, void *stream) {
  return sae::select_topk_row_granule_impl(true, pre_bf16, granule_max, b_enc, scale, B, F, k, rows_per_group, pre_rows, idx, val,
                                           row_off, row_nnz, stream);
}

extern "C" int sae_select_topk_row_ex(const void *pre, int pre_dtype, const float *b_enc, const float *scale,
                                      const float *feat_mask, int64_t B, int64_t F, int k, int32_t *idx, float *val,
                                      int64_t *row_off, int32_t *row_nnz, int cand_cap, void *stream) {
  return sae::select_topk_row_impl(false, pre, pre_dtype, b_enc, scale, feat_mask, B, F, k, idx, val, row_off, row_nnz, cand_cap,
                                   stream);
}

extern "C" int sae_select_topk_row_lowp(const void *pre_bf16, const float *b_enc, const float *scale, const float *feat_mask,
                                        int64_t B, int64_t F, int k, int32_t *idx, float *val, int64_t *row_off,
                                        int32_t *row_nnz, void *stream) {
  return sae::select_topk_row_impl(true, pre_bf16, SAE_BF16, b_enc, scale, feat_mask, B, F, k, idx, val, row_off, row_nnz,
                                   sae::SEL_CAP, stream);
}

extern "C" int sae_select_topk_row(const void *pre, int pre_dtype, const float *b_enc, const float *scale, int64_t B,
                                   int64_t F, int k, int32_t *idx, float *val, int64_t *row_off, int32_t *row_nnz,
                                   void *stream) {
  return sae_select_topk_row_ex(pre, pre_dtype, b_enc, scale, nullptr, B, F, k, idx, val, row_off, row_nnz, sae::SEL_CAP, stream);
}

extern "C" int sae_granule_max(const void *pre_bf16, const float *b_enc, const float *scale, int64_t B, int64_t F,
                               int64_t rows_per_group, int64_t pre_rows, uint32_t *granule_max, void *stream) {
  using namespace sae;
  SAE_REQUIRE(pre_bf16 && granule_max, SAE_ERR_INVALID_ARG, "granule_max: null pointer");
  SAE_REQUIRE(B > 0 && F > 0 && B < (1LL << 31) && F < (1LL << 31), SAE_ERR_INVALID_ARG, "granule_max: bad sizes");
  SAE_REQUIRE(F % 64 == 0, SAE_ERR_UNSUPPORTED, "granule_max: F=%lld must be a multiple of 64", (long long)F);
  if (rows_per_group <= 0) rows_per_group = B;
  SAE_REQUIRE(B % rows_per_group == 0, SAE_ERR_INVALID_ARG, "granule_max: B=%lld is not a multiple of rows_per_group=%lld",
              (long long)B, (long long)rows_per_group);
  if (pre_rows <= 0) pre_rows = B;
  SAE_REQUIRE(pre_rows <= B && B % pre_rows == 0, SAE_ERR_INVALID_ARG, "granule_max: B=%lld is not a multiple of pre_rows=%lld",
              (long long)B, (long long)pre_rows);
  SAE_REQUIRE((((uintptr_t)pre_bf16 | (uintptr_t)b_enc | (uintptr_t)scale) & 15) == 0, SAE_ERR_INVALID_ARG,
              "granule_max: pointers must be 16-byte aligned");
  // rows of one block share a group's bias and scale: blocks of 8 rows when no block straddles two groups; groups that
  // are repeats of the same pre rows are walked inside the kernel, over those rows once
  const int R = rows_per_group % 8 == 0 ? 8 : 1;
  const bool repeats = pre_rows < B && rows_per_group == pre_rows;
  const int64_t rows = repeats ? pre_rows : B;
  const int groups = repeats ? (int)(B / pre_rows) : 1;
  const int64_t n = ((rows + R - 1) / R) * (F / 64);
  SAE_REQUIRE((n * 8 + 255) / 256 < (1LL << 31), SAE_ERR_UNSUPPORTED, "granule_max: too large");
  if (R == 8)
    hipLaunchKernelGGL(granule_max_kernel<8>, dim3((unsigned)((n * 8 + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t *)pre_bf16, b_enc, scale, (int)F, rows, n, (int)rows_per_group, (int)pre_rows, groups,
                       granule_max);
  else
    hipLaunchKernelGGL(granule_max_kernel<1>, dim3((unsigned)((n * 8 + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const uint16_t *)pre_bf16, b_enc, scale, (int)F, rows, n, (int)rows_per_group, (int)pre_rows, groups,
                       granule_max);
  return check_launch("granule_max");
}
