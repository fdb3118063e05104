// Batch-global TopK select (BatchTopK) with fused encoder bias and decoder-norm scale (gfx950).
//
// Keeps the k_total largest positive h1 = (pre + b_enc) * scale over the WHOLE [B, F] batch
// (ties at the threshold: lowest flattened index b * F + f first) and emits the survivors as a
// sparse code with one variable-length row per token, indices ascending.
//
// The [B, F] matrix is read in full ONCE.  A row is cut into granules of 8 * V consecutive
// elements (V = 8 bf16 / 4 fp32: the 128 bytes eight lanes read with one 16-byte load each).
//
//   first     the one full pass: the largest key of every granule, kept in the workspace, and the
//             histogram of the top 11 bits of those maxima
//   bound     one workgroup: at least as many keys as granule maxima reach any value, so the
//             k_total-th largest maximum (rounded down to its histogram bin) is a lower bound on the
//             threshold
//   gather    per token: the keys at or above the lower bound (the candidates: about 1.5 k_total of
//             them) with their features, token by token and in feature order, into a list; only
//             granules whose largest key reaches the bound are read
//   next x3   exact radix select of the k_total-th largest key: digit histograms of bits 30..20,
//             19..9 and 8..0 of the candidates that match the prefix so far
//   pick      after each: one workgroup picks the digit in which the running count from the top
//             reaches the wanted rank (fewer positives than k_total: keep every positive, no search)
//   count     per token: candidates above the threshold and equal to it
//   plan      one workgroup: prefix sums over tokens -> row offsets, and how many of each token's
//             threshold ties are kept (the first `need` ties in flattened order)
//   emit      per token: walks the token's candidates in feature order and places the kept ones
//             with an in-wave prefix sum, so indices ascend without a sort
//
// The candidate list holds B * F / 64 + 1024 entries.  When more keys reach the lower bound (a matrix
// of few distinct values, or k_total itself beyond the list: then gather is skipped), next, count and
// emit read the matrix again instead, granule by granule as gather does: same results, about twice
// the time.
//
// gather, next, count and emit give one WAVE to each token: it reads the token's granule maxima
// 256 at a time, packs the surviving granules' numbers into a list, and reads them 32 at a time
// (four loads in flight, each covering eight granules), with no workgroup barrier.
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
constexpr uint32_t BT_KEEP_NOTHING = 0xffffffffu;
constexpr int BT_GL = 8;                  // lanes that read one granule
constexpr int BT_GPW = 64 / BT_GL;        // granules one wave-wide load covers
constexpr int BT_LIVE = 256;              // granule maxima a wave examines at a time

struct BatchSelState {      // lives in the workspace, one per call
  uint32_t prefix;          // bits of the threshold key decided so far
  uint32_t mask;            // which bits those are
  int64_t remaining;        // rank still to resolve inside the current prefix
  int64_t k_total;          // resolved k (min(k_total, #positives))
  int64_t n_positive;       // number of positive keys when every one of them is a candidate, else -1
  int32_t done;             // 1 when the threshold needs no (further) search
  uint32_t threshold;       // final: keep key > threshold, plus the first `remaining` keys == threshold
  uint32_t lower;           // a lower bound on the threshold, found from the granule maxima
  unsigned long long cand_count;  // keys >= lower that the gather pass met (may exceed the list's capacity)
  int32_t overflow;         // 1: they did not fit; the later passes read the matrix again instead
};

constexpr int BT_STASH = 512;   // candidates of one token a wave collects in LDS before it reserves their place

// capacity of the candidate list for a [B, F] matrix: k_total is B * F / 512 for k = F / 512 per token, and about
// twice k_total keys reach the lower bound, so this leaves a wide margin at 1/8 of a bf16 matrix's bytes
__host__ __device__ inline int64_t bt_candidate_capacity(int64_t B, int64_t F) {
  const int64_t c = B * F / 64 + 1024;
  return c < 0x7fffffffLL ? c : 0x7fffffffLL;
}

// lowp: the arithmetic of a dictionary whose parameters are bf16 tensors -- the sum with the bias and the product with
// the norm are each rounded to bf16, as the tensors `x @ W_E + b_E` and `hidden_pre * decoder_norm()` are
// (models/sae.py:324-335 with cfg.dtype = bfloat16); the bias and scale arrive as fp32 copies of bf16 values.  The flag
// is the same for every lane of a launch.
__device__ __forceinline__ uint32_t bt_key(float pre, float b, float s, float fm, bool has_mask, bool lowp) {
  float h1;
  if (lowp) {
    h1 = bf16_round(mul_rn(bf16_round(add_rn(pre, b)), s));
    if (has_mask) {   // aux-k: the bf16 quotient the encoder returned, times the mask, times the norm, each a bf16 tensor
      h1 = bf16_round(h1 / s);
      h1 = bf16_round(mul_rn(bf16_round(mul_rn(h1, fm)), s));
    }
  } else {
    h1 = (pre + b) * s;
    if (has_mask) h1 = ((h1 / s) * fm) * s;   // aux-k: hidden_pre * dead * scale, op for op
  }
  return h1 > 0.f ? __float_as_uint(h1) : 0u;
}

template <bool BF16>
struct BatchReader {
  static constexpr int V = BF16 ? 8 : 4;
  const void *pre;
  const float *b_enc, *scale, *fmask;
  int F;
  int vec;    // rows, bias, scale and mask can be read as 16-byte vectors
  int nseg;   // 64-lane segments per row (the full pass walks these)
  int ngran;  // granules per row, rounded up to a multiple of 4 (the maxima past the row's end are 0)
  int lowp;   // keys and values in bf16 arithmetic (see bt_key)
  __device__ __forceinline__ const char *row_ptr(int b) const {
    return reinterpret_cast<const char *>(pre) + (size_t)b * F * (BF16 ? 2 : 4);
  }
  // feature index of the first of this lane's V consecutive elements when its quarter wave reads granule g
  __device__ __forceinline__ int lane_base(int g) const { return (g * BT_GL + (int)(threadIdx.x & (BT_GL - 1))) * V; }
  // Loads under a per-lane condition are each followed by a wait for memory; the loads below are therefore
  // issued by every lane, a lane with nothing to read (base < 0 or past the row's end) reading the row's first
  // bytes instead, and its result is discarded when the keys are formed.
  __device__ __forceinline__ int safe_base(int base) const { return (base >= 0 && base < F) ? base : 0; }
  // the 16 bytes of row b at feature `base` (vector layout only)
  __device__ __forceinline__ u32x4 load_raw(int b, int base) const {
    u32x4 raw = {0u, 0u, 0u, 0u};
    if (vec) raw = reinterpret_cast<const u32x4 *>(row_ptr(b))[safe_base(base) / V];
    return raw;
  }
  struct Params { float bb[V], ss[V], mm[V]; };  // bias, scale and mask of V consecutive features
  __device__ __forceinline__ void load_params(int base, Params &pr) const {
    auto load_vec = [&](const float *src, float (&dst)[V], float dflt) {
#pragma unroll
      for (int e = 0; e < V; ++e) dst[e] = dflt;
      if (!src) return;
      if (vec) {
        const int sb = safe_base(base);
#pragma unroll
        for (int q = 0; q < V / 4; ++q) {
          const float4 t = reinterpret_cast<const float4 *>(src + sb)[q];
          dst[4 * q] = t.x; dst[4 * q + 1] = t.y; dst[4 * q + 2] = t.z; dst[4 * q + 3] = t.w;
        }
      } else if (base >= 0) {
#pragma unroll
        for (int e = 0; e < V; ++e) if (base + e < F) dst[e] = src[base + e];
      }
    };
    load_vec(b_enc, pr.bb, 0.f); load_vec(scale, pr.ss, 1.f); load_vec(fmask, pr.mm, 1.f);
  }
  // keys of the V elements of row b from `base` on, with their bias, scale and mask already in registers
  __device__ __forceinline__ void keys_with(int b, int base, const u32x4 &raw, const Params &pr, uint32_t (&keys)[V]) const {
    float p[V];
    if (vec) {
      if constexpr (BF16) {
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int q = 0; q < 4; ++q) { p[2 * q] = __uint_as_float(w[q] << 16); p[2 * q + 1] = __uint_as_float(w[q] & 0xffff0000u); }
      } else {
        p[0] = __uint_as_float(raw.x); p[1] = __uint_as_float(raw.y); p[2] = __uint_as_float(raw.z); p[3] = __uint_as_float(raw.w);
      }
    } else {
      const char *row = row_ptr(b);
#pragma unroll
      for (int e = 0; e < V; ++e) {
        p[e] = 0.f;
        if (base >= 0 && base + e < F) {
          if constexpr (BF16) p[e] = bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(row)[base + e]);
          else p[e] = reinterpret_cast<const float *>(row)[base + e];
        }
      }
    }
    const bool inside = base >= 0 && base < F;
#pragma unroll
    for (int e = 0; e < V; ++e)
      keys[e] = (inside && base + e < F) ? bt_key(p[e], pr.bb[e], pr.ss[e], pr.mm[e], fmask != nullptr, lowp != 0) : 0u;
  }
  // the same, fetching bias, scale and mask
  __device__ __forceinline__ void keys_of(int b, int base, const u32x4 &raw, uint32_t (&keys)[V]) const {
    Params pr;
    load_params(base, pr);
    keys_with(b, base, raw, pr, keys);
  }
  // fn(base, keys) over the granules of row b whose largest key is >= bound, run by ONE wave: each call hands
  // every lane the V keys from feature `base` on (base < 0: none, keys are 0) with bases ascending over the
  // lanes and over the calls, and every lane takes part in every call, so fn may use cross-lane operations.
  // `live` is BT_LIVE ints of LDS private to the wave.
  template <typename Fn>
  __device__ __forceinline__ void for_live_granules(int b, const uint32_t *__restrict__ gran_max_row, uint32_t bound,
                                                    int *live, Fn fn) const {
    const int lane = threadIdx.x & 63, part = lane / BT_GL;
    for (int g0 = 0; g0 < ngran; g0 += BT_LIVE) {
      // a lane looks at four consecutive granules; the list keeps them in ascending order
      const int gl = g0 + lane * 4;
      u32x4 mx = {0u, 0u, 0u, 0u};
      if (gl < ngran) mx = *reinterpret_cast<const u32x4 *>(gran_max_row + gl);   // ngran is a multiple of 4
      const bool a0 = mx.x >= bound, a1 = mx.y >= bound, a2 = mx.z >= bound, a3 = mx.w >= bound;   // bound >= 1
      const unsigned long long m0 = __ballot(a0), m1 = __ballot(a1), m2 = __ballot(a2), m3 = __ballot(a3);
      const unsigned long long below = (1ull << lane) - 1ull;
      int r = __popcll(m0 & below) + __popcll(m1 & below) + __popcll(m2 & below) + __popcll(m3 & below);
      if (a0) live[r++] = gl;
      if (a1) live[r++] = gl + 1;
      if (a2) live[r++] = gl + 2;
      if (a3) live[r++] = gl + 3;   // same wave: LDS operations complete in order
      const int n = __popcll(m0) + __popcll(m1) + __popcll(m2) + __popcll(m3);
      __builtin_amdgcn_wave_barrier();
      for (int i = 0; i < n; i += 4 * BT_GPW) {
        int base[4];
        u32x4 raw[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int j = i + BT_GPW * q + part;
          base[q] = j < n ? lane_base(live[j]) : -1;
          raw[q] = load_raw(b, base[q]);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          if (i + BT_GPW * q < n) {
            uint32_t keys[V];
            keys_of(b, base[q], raw[q], keys);
            fn(base[q], keys);
          }
        }
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
};

__global__ void bt_init_kernel(BatchSelState *st, uint32_t *hist, int64_t k_host, const int64_t *k_dev, int64_t cand_cap) {
  for (int i = threadIdx.x; i < BT_BINS; i += blockDim.x) hist[i] = 0u;
  if (threadIdx.x == 0) {
    st->prefix = 0u; st->mask = 0u; st->done = 0; st->n_positive = 0; st->threshold = 0u; st->lower = 1u;
    st->cand_count = 0ull;
    st->k_total = k_dev ? *k_dev : k_host;
    st->remaining = st->k_total;
    // k_total keys or more reach the lower bound (or every positive key does): a list shorter than k_total is
    // not worth trying, and the gather pass is skipped
    st->overflow = st->k_total > cand_cap;
    if (st->k_total <= 0) { st->done = 1; st->k_total = 0; st->remaining = 0; st->threshold = BT_KEEP_NOTHING; }
  }
}

// The full pass: every granule's largest key and the histogram of the top 11 bits of those maxima.  At least as
// many keys as granule maxima reach any given value, so the k_total-th largest maximum is a lower bound on the
// k_total-th largest key.
template <bool BF16>
__global__ __launch_bounds__(BT_THREADS) void bt_first_kernel(BatchReader<BF16> rd, int B, int rows_per_wg, const BatchSelState *st,
                                                              uint32_t *__restrict__ hist, uint32_t *__restrict__ gran_max) {
  __shared__ uint32_t h[BT_BINS];
  constexpr int V = BatchReader<BF16>::V;
  if (st->done) return;  // k_total <= 0: nothing is kept and the maxima are never read
  for (int i = threadIdx.x; i < BT_BINS; i += BT_THREADS) h[i] = 0u;
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // A wave owns ONE 64-lane segment of the columns and walks rows_per_wg rows of it, so bias, scale and mask
  // are fetched once and stay in registers; four rows' loads are in flight at a time.
  const int s = blockIdx.x * BT_WAVES + wave;
  const int r0 = blockIdx.y * rows_per_wg, r1 = r0 + rows_per_wg < B ? r0 + rows_per_wg : B;
  if (s < rd.nseg) {
    const int base = (s * 64 + lane) * V;
    const int g = s * BT_GPW + lane / BT_GL;
    typename BatchReader<BF16>::Params pr;
    rd.load_params(base, pr);
    for (int r = r0; r < r1; r += 4) {
      u32x4 raw[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) raw[q] = rd.load_raw(r + q < r1 ? r + q : r, base);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (r + q < r1) {
          uint32_t keys[V];
          rd.keys_with(r + q, base, raw[q], pr, keys);
          uint32_t mx = 0u;
#pragma unroll
          for (int e = 0; e < V; ++e) mx = keys[e] > mx ? keys[e] : mx;
#pragma unroll
          for (int o = BT_GL / 2; o > 0; o >>= 1) { const uint32_t t = (uint32_t)__shfl_xor((int)mx, o, 64); mx = t > mx ? t : mx; }
          if ((lane & (BT_GL - 1)) == 0 && g < rd.ngran) {
            gran_max[(size_t)(r + q) * rd.ngran + g] = mx;
            if (mx) atomicAdd(&h[mx >> 20], 1u);
          }
        }
      }
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < BT_BINS; i += BT_THREADS)
    if (h[i]) atomicAdd(&hist[i], h[i]);
}

// The full pass when the granule maxima already exist (the encoder GEMM's epilogue leaves them): only their histogram.
__global__ __launch_bounds__(BT_THREADS) void bt_hist_kernel(const uint32_t *__restrict__ gran_max, int64_t n, const BatchSelState *st,
                                                             uint32_t *__restrict__ hist) {
  __shared__ uint32_t h[BT_BINS];
  if (st->done) return;
  for (int i = threadIdx.x; i < BT_BINS; i += BT_THREADS) h[i] = 0u;
  __syncthreads();
  for (int64_t i = ((int64_t)blockIdx.x * BT_THREADS + threadIdx.x) * 4; i < n; i += (int64_t)gridDim.x * BT_THREADS * 4) {
    const u32x4 m = *reinterpret_cast<const u32x4 *>(gran_max + i);      // n is a multiple of 4
    if (m.x) atomicAdd(&h[m.x >> 20], 1u);
    if (m.y) atomicAdd(&h[m.y >> 20], 1u);
    if (m.z) atomicAdd(&h[m.z >> 20], 1u);
    if (m.w) atomicAdd(&h[m.w >> 20], 1u);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < BT_BINS; i += BT_THREADS)
    if (h[i]) atomicAdd(&hist[i], h[i]);
}

constexpr int BT_TOKENS_PER_WG = 4;  // gather, next, count, emit: one wave per token

struct BatchCandidates {     // the keys >= lower, token by token, each token's in ascending feature order
  uint32_t *key;
  int32_t *feat;
  uint32_t *tok_start;       // where token b's candidates begin
  int32_t *tok_cnt;
  int64_t cap;
};

// per token: the keys that reach the lower bound, with their features, appended to the candidate list.  The wave
// collects them in LDS, reserves their place with one atomic and copies them out; a token with more than
// BT_STASH of them walks its granules a second time and writes directly.
template <bool BF16>
__global__ __launch_bounds__(BT_TOKENS_PER_WG * 64) void bt_gather_kernel(BatchReader<BF16> rd, int B, BatchSelState *st,
                                                                          const uint32_t *__restrict__ gran_max,
                                                                          BatchCandidates cd) {
  __shared__ int live[BT_TOKENS_PER_WG * BT_LIVE];
  __shared__ uint32_t stash_key[BT_TOKENS_PER_WG * BT_STASH];
  __shared__ int32_t stash_feat[BT_TOKENS_PER_WG * BT_STASH];
  constexpr int V = BatchReader<BF16>::V;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int b = blockIdx.x * BT_TOKENS_PER_WG + wave;
  if (b >= B) return;
  if (st->threshold == BT_KEEP_NOTHING) return;
  if (st->overflow) return;           // known beforehand (k_total beyond the list), or found by a token before this one
  const uint32_t lower = st->lower;   // 1 when every positive key is kept
  uint32_t *my_key = stash_key + wave * BT_STASH;
  int32_t *my_feat = stash_feat + wave * BT_STASH;
  unsigned long long start = 0;
  int n = 0;
  for (int pass = 0; pass < 2; ++pass) {
    n = 0;   // candidates of this token before the current call; the same in every lane
    rd.for_live_granules(b, gran_max + (size_t)b * rd.ngran, lower, live + wave * BT_LIVE, [&](int base, const uint32_t (&keys)[V]) {
      int mine = 0;
#pragma unroll
      for (int e = 0; e < V; ++e) mine += keys[e] >= lower;
      int inc = mine;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const int t = __shfl_up(inc, o, 64);
        if (lane >= o) inc += t;
      }
      int pos = n + inc - mine;
      if (mine) {
#pragma unroll
        for (int e = 0; e < V; ++e) {
          if (keys[e] >= lower) {
            if (pass == 0) {
              if (pos < BT_STASH) { my_key[pos] = keys[e]; my_feat[pos] = base + e; }
            } else {
              cd.key[start + pos] = keys[e]; cd.feat[start + pos] = base + e;
            }
            ++pos;
          }
        }
      }
      n += __shfl(inc, 63, 64);
    });
    if (pass == 1) break;
    if (lane == 0) start = atomicAdd(&st->cand_count, (unsigned long long)n);
    start = __shfl((long long)start, 0, 64);
    const bool fits = start + (unsigned long long)n <= (unsigned long long)cd.cap;
    if (lane == 0) {
      cd.tok_start[b] = fits ? (uint32_t)start : 0u;
      cd.tok_cnt[b] = fits ? n : 0;
      if (!fits) st->overflow = 1;
    }
    if (!fits) break;
    if (n <= BT_STASH) {
      __builtin_amdgcn_wave_barrier();
      for (int i = lane; i < n; i += 64) { cd.key[start + i] = my_key[i]; cd.feat[start + i] = my_feat[i]; }
      break;
    }
  }
}

// digit histogram of the keys matching the prefix found so far: over the candidate list, or, when that
// overflowed, over the granules of the matrix that can hold such a key
template <bool BF16>
__global__ __launch_bounds__(BT_TOKENS_PER_WG * 64) void bt_next_kernel(BatchReader<BF16> rd, int B, const BatchSelState *st,
                                                                        uint32_t *__restrict__ hist,
                                                                        const uint32_t *__restrict__ gran_max,
                                                                        BatchCandidates cd, int shift, int bits) {
  __shared__ uint32_t h[BT_BINS];
  __shared__ int live[BT_TOKENS_PER_WG * BT_LIVE];
  constexpr int V = BatchReader<BF16>::V;
  if (st->done) return;
  const int nb = 1 << bits;
  for (int i = threadIdx.x; i < nb; i += blockDim.x) h[i] = 0u;
  __syncthreads();
  const uint32_t prefix = st->prefix, mask = st->mask, dm = (uint32_t)nb - 1u, lower = st->lower;
  if (!st->overflow) {
    // the list is short: a few workgroups read it (four keys in flight per thread), so that few partial
    // histograms reach the global one
    constexpr int LIST_WGS = 128;
    if (blockIdx.x >= LIST_WGS) return;
    const int64_t n = (int64_t)st->cand_count;
    const int64_t stride = (int64_t)(gridDim.x < LIST_WGS ? gridDim.x : LIST_WGS) * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += 4 * stride) {
      uint32_t key[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) key[q] = cd.key[i + q * stride < n ? i + q * stride : n - 1];   // unconditional loads
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (i + q * stride < n && (key[q] & mask) == prefix) atomicAdd(&h[(key[q] >> shift) & dm], 1u);
    }
  } else {
    // every key that matches is >= prefix (its undecided bits are >= 0); keys below `lower` cannot be the threshold
    const uint32_t bound = prefix > lower ? prefix : lower;
    const int b = blockIdx.x * BT_TOKENS_PER_WG + (threadIdx.x >> 6);
    if (b < B) {
      rd.for_live_granules(b, gran_max + (size_t)b * rd.ngran, bound, live + (threadIdx.x >> 6) * BT_LIVE, [&](int, const uint32_t (&keys)[V]) {
#pragma unroll
        for (int e = 0; e < V; ++e)
          if (keys[e] >= lower && (keys[e] & mask) == prefix) atomicAdd(&h[(keys[e] >> shift) & dm], 1u);
      });
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < nb; i += blockDim.x)
    if (h[i]) atomicAdd(&hist[i], h[i]);
}

// inclusive prefix sum over the 1024 threads of a workgroup (wsum: BT_WAVES values of LDS)
__device__ __forceinline__ int64_t bt_block_scan(int64_t v, int64_t *wsum) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int64_t t = __shfl_up((long long)v, o, 64);
    if (lane >= o) v += t;
  }
  if (lane == 63) wsum[wave] = v;
  __syncthreads();
  int64_t base = 0;
  for (int w = 0; w < wave; ++w) base += wsum[w];
  __syncthreads();
  return v + base;
}

// Walking the nb bins from the top down, the bin in which the running count reaches `target` (> 0), and the rank
// wanted inside that bin; *bin stays -1 when the histogram holds fewer than `target`; *total_out is the
// histogram's total.  One workgroup of 1024; the results (in LDS) are visible to every thread on return.
__device__ __forceinline__ void bt_find_from_top(const uint32_t *hist, int nb, int64_t target, int64_t *wsum, int *bin,
                                                 int64_t *need_out, int64_t *total_out) {
  const int tid = threadIdx.x;
  if (tid == 0) *bin = -1;
  const int per = (nb + 1023) / 1024;  // thread t owns the bins nb - 1 - (t * per + e)
  int64_t local = 0;
  for (int e = 0; e < per; ++e) { const int i = nb - 1 - (tid * per + e); if (i >= 0) local += hist[i]; }
  const int64_t incl = bt_block_scan(local, wsum);  // its barriers also order the write of *bin above
  const int64_t excl = incl - local;
  if (tid == 1023) *total_out = incl;
  if (excl < target && incl >= target) {
    int64_t need = target - excl;
    for (int e = 0; e < per; ++e) {
      const int i = nb - 1 - (tid * per + e);
      if (i < 0) break;
      const int64_t c = hist[i];
      if (c >= need) { *bin = i; *need_out = need; break; }
      need -= c;
    }
  }
  __syncthreads();
}

// one workgroup, after the full pass: the key from which the search starts
__global__ __launch_bounds__(1024) void bt_bound_kernel(BatchSelState *st, uint32_t *hist) {
  __shared__ int64_t wsum[BT_WAVES];
  __shared__ int bin;
  __shared__ int64_t need, total;
  const int tid = threadIdx.x;
  if (st->done) { for (int i = tid; i < BT_BINS; i += 1024) hist[i] = 0u; return; }
  bt_find_from_top(hist, BT_BINS, st->k_total, wsum, &bin, &need, &total);
  // k_total granules have a maximum in this bin or above, so the threshold is at least the bin's lower edge;
  // with fewer positive maxima than k_total (bin < 0) every positive key is a candidate
  if (tid == 0) st->lower = bin > 0 ? ((uint32_t)bin) << 20 : 1u;
  for (int i = tid; i < BT_BINS; i += 1024) hist[i] = 0u;  // the key histograms start from zero
}

// one workgroup: choose the digit in which the running count (from the top bin down) reaches `remaining`.
// The first of the three also settles the case of fewer positives than k_total: then the lower bound is 1, the
// first histogram holds every positive key, and all of them are kept.
__global__ __launch_bounds__(1024) void bt_pick_kernel(BatchSelState *st, uint32_t *hist, int shift, int bits, int first) {
  __shared__ int64_t wsum[BT_WAVES];
  __shared__ int bin;
  __shared__ int64_t need, total;
  const int nb = 1 << bits, tid = threadIdx.x;
  if (st->done) { for (int i = tid; i < BT_BINS; i += 1024) hist[i] = 0u; return; }
  bt_find_from_top(hist, nb, st->remaining, wsum, &bin, &need, &total);
  if (tid == 0) {
    const bool all_counted = first && st->lower == 1u;   // the histogram's total is the number of positive keys
    if (first) st->n_positive = all_counted ? total : -1;
    if (all_counted && total <= st->k_total) {
      st->done = 1; st->k_total = total; st->prefix = 0u; st->mask = 0u; st->remaining = 0; st->threshold = 0u;
    } else if (bin >= 0) {
      st->remaining = need;
      st->prefix |= ((uint32_t)bin) << shift;
      st->mask |= ((uint32_t)(nb - 1)) << shift;
      if (shift == 0) st->threshold = st->prefix;
    }
  }
  for (int i = tid; i < BT_BINS; i += 1024) hist[i] = 0u;  // ready for the next pass
}

// per token: how many keys are above the threshold, how many equal it
template <bool BF16>
__global__ __launch_bounds__(BT_TOKENS_PER_WG * 64) void bt_count_kernel(BatchReader<BF16> rd, int B, const BatchSelState *st,
                                                                         const uint32_t *__restrict__ gran_max,
                                                                         BatchCandidates cd, int32_t *__restrict__ n_gt,
                                                                         int32_t *__restrict__ n_tie) {
  __shared__ int live[BT_TOKENS_PER_WG * BT_LIVE];
  constexpr int V = BatchReader<BF16>::V;
  const int b = blockIdx.x * BT_TOKENS_PER_WG + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (b >= B) return;
  const uint32_t T = st->threshold;
  int gt = 0, tie = 0;
  if (T == BT_KEEP_NOTHING) {
  } else if (!st->overflow) {
    const uint32_t *keys = cd.key + cd.tok_start[b];
    const int n = cd.tok_cnt[b];
    for (int i = lane; i < n; i += 64) { const uint32_t k = keys[i]; gt += k > T; tie += k == T; }
  } else {
    rd.for_live_granules(b, gran_max + (size_t)b * rd.ngran, T ? T : 1u, live + (threadIdx.x >> 6) * BT_LIVE, [&](int, const uint32_t (&keys)[V]) {
#pragma unroll
      for (int e = 0; e < V; ++e) { gt += keys[e] > T; tie += (keys[e] == T) && keys[e] != 0u; }
    });
  }
  gt = wave_sum_i(gt); tie = wave_sum_i(tie);
  if (lane == 0) { n_gt[b] = gt; n_tie[b] = tie; }
}

// one workgroup: row offsets and per-token tie allowance (first `need` ties in flattened order).
// Thread t owns the tokens [t * per, (t + 1) * per).
__global__ __launch_bounds__(1024) void bt_plan_kernel(const BatchSelState *st, const int32_t *__restrict__ n_gt,
                                                       const int32_t *__restrict__ n_tie, int B,
                                                       int32_t *__restrict__ tie_keep, int64_t *__restrict__ row_off,
                                                       int32_t *__restrict__ row_nnz, int64_t *__restrict__ total_out) {
  __shared__ int64_t wsum[BT_WAVES];
  const int tid = threadIdx.x;
  const int64_t need = st->done ? 0 : st->remaining;  // threshold ties that belong to the top k_total
  const int64_t per = ((int64_t)B + 1023) / 1024;
  const int lo = (int)(tid * per < B ? tid * per : B), hi = (int)(lo + per < B ? lo + per : B);
  // The three walks below take a thread's tokens eight at a time.  Their loads are unconditional (a slot past
  // the thread's range re-reads its last token and is masked afterwards): loads under a per-lane condition
  // would each be followed by a wait for memory.
  const int last = hi > lo ? hi - 1 : 0;   // B >= 1, so token 0 exists
  int64_t ties = 0;
  for (int c = lo; c < hi; c += 8) {
    int32_t t[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) t[j] = n_tie[c + j < hi ? c + j : last];
#pragma unroll
    for (int j = 0; j < 8; ++j) ties += c + j < hi ? t[j] : 0;
  }
  int64_t ties_before = bt_block_scan(ties, wsum) - ties;
  int64_t nnz_sum = 0;
  for (int c = lo; c < hi; c += 8) {
    int32_t t[8], g[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) { const int b = c + j < hi ? c + j : last; t[j] = n_tie[b]; g[j] = n_gt[b]; }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (c + j < hi) {
        int64_t keep = need - ties_before;
        keep = keep < 0 ? 0 : (keep > t[j] ? t[j] : keep);
        ties_before += t[j];
        const int64_t nnz = (int64_t)g[j] + keep;
        tie_keep[c + j] = (int32_t)keep; row_nnz[c + j] = (int32_t)nnz;
        nnz_sum += nnz;
      }
    }
  }
  const int64_t incl = bt_block_scan(nnz_sum, wsum);
  int64_t off = incl - nnz_sum;
  for (int c = lo; c < hi; c += 8) {
    int32_t z[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) z[j] = row_nnz[c + j < hi ? c + j : last];   // this thread's own stores above
#pragma unroll
    for (int j = 0; j < 8; ++j) { if (c + j < hi) { row_off[c + j] = off; off += z[j]; } }
  }
  if (tid == 1023 && total_out) *total_out = incl;
}

// per token: ordered compaction of the kept elements
template <bool BF16>
__global__ __launch_bounds__(BT_TOKENS_PER_WG * 64) void bt_emit_kernel(BatchReader<BF16> rd, int B, const BatchSelState *st,
                                                                        const uint32_t *__restrict__ gran_max,
                                                                        BatchCandidates cd,
                                                                        const int32_t *__restrict__ tie_keep,
                                                                        const int64_t *__restrict__ row_off,
                                                                        int32_t *__restrict__ idx_out,
                                                                        float *__restrict__ val_out, int64_t capacity) {
  __shared__ int live[BT_TOKENS_PER_WG * BT_LIVE];
  constexpr int V = BatchReader<BF16>::V;
  const int b = blockIdx.x * BT_TOKENS_PER_WG + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (b >= B) return;
  const uint32_t T = st->threshold;
  if (T == BT_KEEP_NOTHING) return;
  const int keep_ties = tie_keep[b];
  const int64_t off = row_off[b];
  int run_gt = 0, run_tie = 0;  // of this token, before the elements of the current call
  // One call places up to 64 * N keys; lane l holds keys[e] with features feat0 + e, ascending over e, lanes and calls.
  auto place = [&](int feat0, const auto &keys, auto n_const) {
    constexpr int N = decltype(n_const)::value;
    int mine = 0;  // keys above the threshold in the low half, ties in the high half (one call holds <= 512 keys)
#pragma unroll
    for (int e = 0; e < N; ++e) mine += (int)(keys[e] > T) + ((int)(keys[e] == T && keys[e] != 0u) << 16);
    int inc = mine;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int a = __shfl_up(inc, o, 64);
      if (lane >= o) inc += a;
    }
    const int total = __shfl(inc, 63, 64);
    const int before = inc - mine;
    int tie_rank = run_tie + (before >> 16);  // ties of this token before my first element
    // kept elements before my first one: every greater key, and the first keep_ties ties
    int pos = run_gt + (before & 0xffff) + (tie_rank < keep_ties ? tie_rank : keep_ties);
    if (mine) {
#pragma unroll
      for (int e = 0; e < N; ++e) {
        const uint32_t k = keys[e];
        bool keep = k > T;
        if (k == T && k != 0u) { keep = tie_rank < keep_ties; ++tie_rank; }
        if (keep) {
          const int64_t o = off + pos;
          if (o < capacity) {
            const int f = feat0 + e;
            const float h1 = __uint_as_float(k);
            idx_out[o] = f;
            float v = h1;
            if (rd.scale) { v = h1 / rd.scale[f]; if (rd.lowp) v = bf16_round(v); }   // the quotient is a bf16 tensor too
            val_out[o] = v;
          }
          ++pos;
        }
      }
    }
    run_gt += total & 0xffff;
    run_tie += total >> 16;
  };
  if (!st->overflow) {
    const uint32_t *ck = cd.key + cd.tok_start[b];
    const int32_t *cf = cd.feat + cd.tok_start[b];
    const int n = cd.tok_cnt[b];
    for (int i0 = 0; i0 < n; i0 += 64) {
      const int i = i0 + lane;
      const uint32_t one[1] = {i < n ? ck[i] : 0u};
      place(i < n ? cf[i] : 0, one, std::integral_constant<int, 1>{});
    }
  } else {
    rd.for_live_granules(b, gran_max + (size_t)b * rd.ngran, T ? T : 1u, live + (threadIdx.x >> 6) * BT_LIVE,
                         [&](int base, const uint32_t (&keys)[V]) { place(base, keys, std::integral_constant<int, V>{}); });
  }
}

template <bool BF16>
static int run_batch_select(const void *pre, const float *b_enc, const float *scale, const float *fmask, int64_t B,
                            int64_t F, int64_t k_total, const int64_t *k_total_dev, int32_t *idx, float *val,
                            int64_t capacity, int64_t *row_off, int32_t *row_nnz, int64_t *total_out, void *workspace,
                            hipStream_t st, const uint32_t *gran_max_given = nullptr, bool lowp = false) {
  constexpr int V = BatchReader<BF16>::V;
  char *ws = reinterpret_cast<char *>(workspace);
  BatchSelState *state = reinterpret_cast<BatchSelState *>(ws);
  const bool vec = (F % V == 0) &&
                   ((((uintptr_t)pre | (uintptr_t)b_enc | (uintptr_t)scale | (uintptr_t)fmask) & 15) == 0);
  const int nseg = (int)((F + 64 * V - 1) / (64 * V)), ngran = (int)((F + BT_GL * V - 1) / (BT_GL * V) + 3) / 4 * 4;
  uint32_t *hist = reinterpret_cast<uint32_t *>(ws + 256);
  uint32_t *gran_ws = reinterpret_cast<uint32_t *>(ws + 256 + BT_BINS * 4);   // 16-byte aligned rows
  // maxima handed in (same granules, same keys: [B, F / 64] with F / 64 a multiple of 4) are read where they lie
  const uint32_t *gran_max = gran_max_given ? gran_max_given : gran_ws;
  int32_t *n_gt = reinterpret_cast<int32_t *>(gran_ws + B * ngran);
  int32_t *n_tie = n_gt + B;
  int32_t *tie_keep = n_tie + B;
  BatchCandidates cd;
  cd.tok_start = reinterpret_cast<uint32_t *>(tie_keep + B);
  cd.tok_cnt = reinterpret_cast<int32_t *>(cd.tok_start + B);
  cd.cap = bt_candidate_capacity(B, F);
  cd.key = reinterpret_cast<uint32_t *>(cd.tok_cnt + B);
  cd.feat = reinterpret_cast<int32_t *>(cd.key + cd.cap);
  BatchReader<BF16> rd{pre, b_enc, scale, fmask, (int)F, vec ? 1 : 0, nseg, ngran, lowp ? 1 : 0};
  hipLaunchKernelGGL(bt_init_kernel, dim3(1), dim3(256), 0, st, state, hist, k_total, k_total_dev, bt_candidate_capacity(B, F));
  const int rows_per_wg = (int)(B / 65535 > 16 ? B / 65535 + 1 : 16);
  if (gran_max_given) {
    const int64_t n = B * ngran;
    const int64_t blocks = (n / 4 + BT_THREADS - 1) / BT_THREADS;
    hipLaunchKernelGGL(bt_hist_kernel, dim3((unsigned)(blocks < 2048 ? blocks : 2048)), dim3(BT_THREADS), 0, st, gran_max, n, state, hist);
  } else {
    hipLaunchKernelGGL(bt_first_kernel<BF16>, dim3((unsigned)((nseg + BT_WAVES - 1) / BT_WAVES), (unsigned)((B + rows_per_wg - 1) / rows_per_wg)),
                       dim3(BT_THREADS), 0, st, rd, (int)B, rows_per_wg, state, hist, gran_ws);
  }
  hipLaunchKernelGGL(bt_bound_kernel, dim3(1), dim3(1024), 0, st, state, hist);
  const unsigned token_grid = (unsigned)((B + BT_TOKENS_PER_WG - 1) / BT_TOKENS_PER_WG);
  const dim3 token_block(BT_TOKENS_PER_WG * 64);
  hipLaunchKernelGGL(bt_gather_kernel<BF16>, dim3(token_grid), token_block, 0, st, rd, (int)B, state, gran_max, cd);
  const int shifts[3] = {20, 9, 0}, bits[3] = {11, 11, 9};  // bits 30..20, 19..9, 8..0 (bit 31 is the sign: always 0)
  for (int p = 0; p < 3; ++p) {
    hipLaunchKernelGGL(bt_next_kernel<BF16>, dim3(token_grid), token_block, 0, st, rd, (int)B, state, hist, gran_max, cd,
                       shifts[p], bits[p]);
    hipLaunchKernelGGL(bt_pick_kernel, dim3(1), dim3(1024), 0, st, state, hist, shifts[p], bits[p], p == 0 ? 1 : 0);
  }
  hipLaunchKernelGGL(bt_count_kernel<BF16>, dim3(token_grid), token_block, 0, st, rd, (int)B, state, gran_max, cd, n_gt, n_tie);
  hipLaunchKernelGGL(bt_plan_kernel, dim3(1), dim3(1024), 0, st, state, n_gt, n_tie, (int)B, tie_keep, row_off, row_nnz,
                     total_out);
  hipLaunchKernelGGL(bt_emit_kernel<BF16>, dim3(token_grid), token_block, 0, st, rd, (int)B, state, gran_max, cd, tie_keep,
                     row_off, idx, val, capacity);
  return check_launch("select_topk_batch");
}

}  // namespace sae

extern "C" int64_t sae_select_topk_batch_workspace_bytes(int64_t B, int64_t F) {
  if (B <= 0 || F <= 0) return 0;
  // state, histogram, 5 per-token counters, the candidate list (key and feature), and one largest key per 256
  // bytes of a row (sized for the shorter fp32 granules of 64 elements)
  const int64_t ngran = ((F + sae::BT_GL * 4 - 1) / (sae::BT_GL * 4) + 3) / 4 * 4;
  return 256 + sae::BT_BINS * 4 + 5 * B * (int64_t)sizeof(int32_t) + 8 * sae::bt_candidate_capacity(B, F) +
         B * ngran * 4 + 256;
}

extern "C" int sae_select_topk_batch(const void *pre, int pre_dtype, const float *b_enc, const float *scale,
                                     const float *feat_mask, int64_t B, int64_t F, int64_t k_total,
                                     const int64_t *k_total_dev, int32_t *idx, float *val, int64_t capacity,
                                     int64_t *row_off, int32_t *row_nnz, int64_t *total_out, void *workspace,
                                     int64_t workspace_bytes, void *stream) {
  using namespace sae;
  SAE_REQUIRE(pre && idx && val && row_off && row_nnz, SAE_ERR_INVALID_ARG, "select_topk_batch: null pointer");
  SAE_REQUIRE(B > 0 && F > 0 && B < (1LL << 31) && F <= (1LL << 30), SAE_ERR_INVALID_ARG, "select_topk_batch: bad shape");
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

extern "C" int sae_select_topk_batch_lowp(const void *pre_bf16, const uint32_t *granule_max, const float *b_enc,
                                          const float *scale, const float *feat_mask, int64_t B, int64_t F, int64_t k_total,
                                          const int64_t *k_total_dev, int32_t *idx, float *val, int64_t capacity,
                                          int64_t *row_off, int32_t *row_nnz, int64_t *total_out, void *workspace,
                                          int64_t workspace_bytes, void *stream) {
  using namespace sae;
  SAE_REQUIRE(pre_bf16 && idx && val && row_off && row_nnz, SAE_ERR_INVALID_ARG, "select_topk_batch_lowp: null pointer");
  SAE_REQUIRE(B > 0 && F > 0 && B < (1LL << 31) && F <= (1LL << 30), SAE_ERR_INVALID_ARG, "select_topk_batch_lowp: bad shape");
  SAE_REQUIRE(k_total_dev || k_total >= 0, SAE_ERR_INVALID_ARG, "select_topk_batch_lowp: k_total must be >= 0");
  SAE_REQUIRE(capacity > 0, SAE_ERR_INVALID_ARG, "select_topk_batch_lowp: capacity must be positive");
  SAE_REQUIRE(workspace && workspace_bytes >= sae_select_topk_batch_workspace_bytes(B, F), SAE_ERR_WORKSPACE,
              "select_topk_batch_lowp: workspace of %lld bytes needed", (long long)sae_select_topk_batch_workspace_bytes(B, F));
  SAE_REQUIRE((((uintptr_t)workspace) & 255) == 0, SAE_ERR_INVALID_ARG, "select_topk_batch_lowp: workspace must be 256-byte aligned");
  SAE_REQUIRE(!granule_max || (!feat_mask && F % 256 == 0 &&
                               (((uintptr_t)granule_max | (uintptr_t)pre_bf16 | (uintptr_t)b_enc | (uintptr_t)scale) & 15) == 0),
              SAE_ERR_UNSUPPORTED, "select_topk_batch_lowp: granule maxima need F a multiple of 256, 16-byte aligned pointers and no feat_mask");
  return run_batch_select<true>(pre_bf16, b_enc, scale, feat_mask, B, F, k_total, k_total_dev, idx, val, capacity, row_off,
                                row_nnz, total_out, workspace, (hipStream_t)stream, granule_max, true);
}

extern "C" int sae_select_topk_batch_granule(const void *pre_bf16, const uint32_t *granule_max, const float *b_enc,
                                             const float *scale, int64_t B, int64_t F, int64_t k_total, const int64_t *k_total_dev,
                                             int32_t *idx, float *val, int64_t capacity, int64_t *row_off, int32_t *row_nnz,
                                             int64_t *total_out, void *workspace, int64_t workspace_bytes, void *stream) {
  using namespace sae;
  SAE_REQUIRE(pre_bf16 && granule_max && idx && val && row_off && row_nnz, SAE_ERR_INVALID_ARG, "select_topk_batch_granule: null pointer");
  SAE_REQUIRE(B > 0 && F > 0 && B < (1LL << 31) && F <= (1LL << 30), SAE_ERR_INVALID_ARG, "select_topk_batch_granule: bad shape");
  SAE_REQUIRE(F % 256 == 0, SAE_ERR_UNSUPPORTED, "select_topk_batch_granule: F=%lld must be a multiple of 256", (long long)F);
  SAE_REQUIRE(k_total_dev || k_total >= 0, SAE_ERR_INVALID_ARG, "select_topk_batch_granule: k_total must be >= 0");
  SAE_REQUIRE(capacity > 0, SAE_ERR_INVALID_ARG, "select_topk_batch_granule: capacity must be positive");
  SAE_REQUIRE(workspace && workspace_bytes >= sae_select_topk_batch_workspace_bytes(B, F), SAE_ERR_WORKSPACE,
              "select_topk_batch_granule: workspace of %lld bytes needed", (long long)sae_select_topk_batch_workspace_bytes(B, F));
  SAE_REQUIRE((((uintptr_t)workspace) & 255) == 0 && (((uintptr_t)granule_max | (uintptr_t)pre_bf16 | (uintptr_t)b_enc | (uintptr_t)scale) & 15) == 0,
              SAE_ERR_INVALID_ARG, "select_topk_batch_granule: workspace must be 256-byte, the other pointers 16-byte aligned");
  return run_batch_select<true>(pre_bf16, b_enc, scale, nullptr, B, F, k_total, k_total_dev, idx, val, capacity, row_off, row_nnz,
                                total_out, workspace, (hipStream_t)stream, granule_max);
}
