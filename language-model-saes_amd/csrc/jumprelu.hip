// JumpReLU activation with its straight-through threshold gradient and the sparsity penalties that read
// the same [B, F] data, as two streaming passes (forward, backward).  Each element is read and written once, but at
// bf16 the passes run at about half the memory system's rate: two dozen vector instructions per element (a division,
// a tanh, conversions) and, in the forward, the per-feature vectors re-read from L2 set the pace.  The forward
// reads the pre-activation and writes the activation once; the backward reads the pre-activation and
// the incoming gradient once, writes the pre-activation gradient once, and reduces three per-feature
// sums (bias, threshold, decoder-norm gradients) through per-row-group partials that a second kernel
// adds in a fixed order, so results do not depend on scheduling.
//
// Per element, with h = pre + b_enc, s = scale (decoder norm, 1 when absent), u = h * s:
//   keep = u > theta                      activation  a = keep ? h : 0   ( = jumprelu(u) / s )
// and with n = pen_norm (the decoder norm the penalties weigh by, 1 when absent; it is the same vector as
// `scale` when the activation includes the decoder norm, but the penalties use it either way):
//   tanh term   t = tanh(c * a * n)       lp term  relu(theta - h) * n
// and for the backward, with ga = d_acts + g_tanh[b] * c * n * (1 - t^2):
//   d_pre    = keep ? ga : 0   - (theta > h ? g_lp[b] * n : 0)
//   d_theta += (|u - theta| < window/2 and u > 0) ? (ga / s) * (-theta / window) : 0   + (theta > h ? g_lp[b] * n : 0)
//   d_pen_norm += g_tanh[b] * c * a * (1 - t^2) + g_lp[b] * relu(theta - h)
//   d_bias  += d_pre
// (the two derivative terms of a = jumprelu(h s) / s with respect to s cancel exactly).
#include "common.h"

namespace sae {

constexpr int JR_THREADS = 256;
constexpr int JR_ROWS = 64;  // rows per block of the backward pass (one partial per row group and feature)

// STREAM: non-temporal access for [B, F] data that is touched once per pass
typedef __attribute__((ext_vector_type(4))) unsigned nt_u32x4;

template <bool BF16, bool STREAM = false>
__device__ __forceinline__ void load8(const void *__restrict__ p, int64_t g, float (&v)[8]) {
  if constexpr (BF16) {
    u32x4 r;
    if constexpr (STREAM) {
      const nt_u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const nt_u32x4 *>(p) + g);
      r.x = t[0]; r.y = t[1]; r.z = t[2]; r.w = t[3];
    } else {
      r = reinterpret_cast<const u32x4 *>(p)[g];
    }
    v[0] = bf16_bits_to_f32((uint16_t)(r.x & 0xffffu)); v[1] = bf16_bits_to_f32((uint16_t)(r.x >> 16));
    v[2] = bf16_bits_to_f32((uint16_t)(r.y & 0xffffu)); v[3] = bf16_bits_to_f32((uint16_t)(r.y >> 16));
    v[4] = bf16_bits_to_f32((uint16_t)(r.z & 0xffffu)); v[5] = bf16_bits_to_f32((uint16_t)(r.z >> 16));
    v[6] = bf16_bits_to_f32((uint16_t)(r.w & 0xffffu)); v[7] = bf16_bits_to_f32((uint16_t)(r.w >> 16));
  } else {
    float4 a, b;
    if constexpr (STREAM) {
      a = load_stream(reinterpret_cast<const float *>(p), 2 * g);
      b = load_stream(reinterpret_cast<const float *>(p), 2 * g + 1);
    } else {
      a = reinterpret_cast<const float4 *>(p)[2 * g];
      b = reinterpret_cast<const float4 *>(p)[2 * g + 1];
    }
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
}

template <bool BF16, bool STREAM = false>
__device__ __forceinline__ void store8(void *__restrict__ p, int64_t g, const float (&v)[8]) {
  if constexpr (BF16) {
    u32x4 o;
    o.x = pack_bf16x2(v[0], v[1]);
    o.y = pack_bf16x2(v[2], v[3]);
    o.z = pack_bf16x2(v[4], v[5]);
    o.w = pack_bf16x2(v[6], v[7]);
    if constexpr (STREAM) {
      const nt_u32x4 t = {o.x, o.y, o.z, o.w};
      __builtin_nontemporal_store(t, reinterpret_cast<nt_u32x4 *>(p) + g);
    } else {
      reinterpret_cast<u32x4 *>(p)[g] = o;
    }
  } else if constexpr (STREAM) {
    store_stream(reinterpret_cast<float *>(p), 2 * g, make_float4(v[0], v[1], v[2], v[3]));
    store_stream(reinterpret_cast<float *>(p), 2 * g + 1, make_float4(v[4], v[5], v[6], v[7]));
  } else {
    reinterpret_cast<float4 *>(p)[2 * g] = make_float4(v[0], v[1], v[2], v[3]);
    reinterpret_cast<float4 *>(p)[2 * g + 1] = make_float4(v[4], v[5], v[6], v[7]);
  }
}

__device__ __forceinline__ void load8_f32_or(const float *__restrict__ p, int64_t g, float fill, float (&v)[8]) {
  if (p) {
    load8<false>(p, g, v);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = fill;
  }
}

// tanh for x >= 0 through one hardware exponential: 1 - 2 / (e^{2x} + 1); below 0.04 the cancellation in that form
// would cost more than the 1e-7 relative error of the odd series x - x^3/3 + 2 x^5 / 15
__device__ __forceinline__ float tanh_pos(float x) {
  if (x < 0.04f) {
    const float x2 = x * x;
    return x * (1.f - x2 * (0.33333334f - 0.13333334f * x2));
  }
  const float e = __expf(2.f * x);
  return 1.f - 2.f * __builtin_amdgcn_rcpf(e + 1.f);   // the reciprocal's 1 ulp is 1e-7 of the result at most
}

// u / s.  The fp32 instantiations keep the correctly rounded quotient; the bf16 ones, whose result is rounded to 8 bits
// of mantissa right away, take the hardware reciprocal with one correction step (the passes are bound by their
// arithmetic, and the IEEE sequence is a quarter of it).
template <bool BF16>
__device__ __forceinline__ float jr_div(float u, float s) {
  if constexpr (BF16) {
    const float r = __builtin_amdgcn_rcpf(s);
    const float q = u * r;
    return fmaf(fmaf(-q, s, u), r, q);
  } else {
    return u / s;
  }
}

// one block per JR_FWD_ROWS token rows: the per-feature vectors (bias, scale, penalty norm, threshold: 128 bytes per
// lane and step against 16 bytes of a bf16 row) are fetched once for all of them
constexpr int JR_FWD_ROWS = 4;
template <bool BF16>
__global__ __launch_bounds__(JR_THREADS) void jumprelu_fwd_kernel(
    const void *__restrict__ pre, const float *__restrict__ b_enc, const float *__restrict__ scale,
    const float *__restrict__ pen, const float *__restrict__ theta, int64_t B, int64_t F, float tanh_c,
    void *__restrict__ acts, float *__restrict__ tanh_tok, float *__restrict__ lp_tok, float *__restrict__ l0_tok) {
  __shared__ float red[JR_THREADS / 64];
  constexpr int R = JR_FWD_ROWS;
  const int64_t row0 = (int64_t)blockIdx.x * R;
  const int n_rows = (int)((B - row0) < R ? (B - row0) : R);
  const int64_t groups = F >> 3;
  float tsum[R], lpsum[R], cnt[R];
#pragma unroll
  for (int r = 0; r < R; ++r) tsum[r] = lpsum[r] = cnt[r] = 0.f;
  for (int64_t g = threadIdx.x; g < groups; g += JR_THREADS) {
    float p[R][8], b[8], s[8], np[8], th[8];
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (r < n_rows) load8<BF16, true>(pre, (row0 + r) * groups + g, p[r]);
    load8_f32_or(b_enc, g, 0.f, b);
    load8_f32_or(scale, g, 1.f, s);
    load8_f32_or(pen, g, 1.f, np);
    load8<false>(theta, g, th);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (r < n_rows) {
        float a[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float h = p[r][i] + b[i];
          const float u = mul_rn(h, s[i]);
          const bool keep = u > th[i];
          a[i] = keep ? (scale ? jr_div<BF16>(u, s[i]) : h) : 0.f;
          cnt[r] += keep ? 1.f : 0.f;
          if (tanh_tok && keep) tsum[r] += tanh_pos(tanh_c * a[i] * np[i]);
          if (lp_tok) lpsum[r] += fmaxf(th[i] - h, 0.f) * np[i];
        }
        store8<BF16, true>(acts, (row0 + r) * groups + g, a);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    if (r < n_rows) {   // uniform over the block
      if (tanh_tok) {
        const float t = block_sum<JR_THREADS / 64>(tsum[r], red);
        if (threadIdx.x == 0) tanh_tok[row0 + r] = t;
      }
      if (lp_tok) {
        const float t = block_sum<JR_THREADS / 64>(lpsum[r], red);
        if (threadIdx.x == 0) lp_tok[row0 + r] = t;
      }
      if (l0_tok) {
        const float t = block_sum<JR_THREADS / 64>(cnt[r], red);
        if (threadIdx.x == 0) l0_tok[row0 + r] = t;
      }
    }
  }
}

// grid (ceil(F / 2048), ceil(B / JR_ROWS)); a thread owns 8 adjacent features for JR_ROWS rows
template <bool BF16>
__global__ __launch_bounds__(JR_THREADS) void jumprelu_bwd_kernel(
    const void *__restrict__ pre, const float *__restrict__ b_enc, const float *__restrict__ scale,
    const float *__restrict__ pen, const float *__restrict__ theta, const void *__restrict__ d_acts,
    const float *__restrict__ g_tanh, float tanh_c,
    const float *__restrict__ g_lp, float window, int64_t B, int64_t F, void *__restrict__ d_pre,
    float *__restrict__ part_bias, float *__restrict__ part_theta, float *__restrict__ part_scale) {
  const int64_t groups = F >> 3;
  const int64_t g = (int64_t)blockIdx.x * JR_THREADS + threadIdx.x;
  if (g >= groups) return;
  float b[8], s[8], np[8], th[8];
  load8_f32_or(b_enc, g, 0.f, b);
  load8_f32_or(scale, g, 1.f, s);
  load8_f32_or(pen, g, 1.f, np);
  load8<false>(theta, g, th);
  float acc_b[8], acc_t[8], acc_s[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc_b[i] = acc_t[i] = acc_s[i] = 0.f;
  const float half_w = 0.5f * window;
  const int64_t r0 = (int64_t)blockIdx.y * JR_ROWS;
  const int64_t r1 = (r0 + JR_ROWS < B) ? r0 + JR_ROWS : B;
#pragma unroll 2
  for (int64_t r = r0; r < r1; ++r) {
    float p[8], ga[8], dp[8];
    load8<BF16, true>(pre, r * groups + g, p);
    load8<BF16, true>(d_acts, r * groups + g, ga);
    const float gt = g_tanh ? g_tanh[r] * tanh_c : 0.f;
    const float gl = g_lp ? g_lp[r] : 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const float h = p[i] + b[i];
      const float u = mul_rn(h, s[i]);
      const bool keep = u > th[i];
      float gtot = ga[i];
      if (g_tanh) {
        const float a = keep ? (scale ? jr_div<BF16>(u, s[i]) : h) : 0.f;
        const float t = keep ? tanh_pos(tanh_c * a * np[i]) : 0.f;
        const float sech2 = 1.f - t * t;
        gtot += gt * np[i] * sech2;
        acc_s[i] += gt * a * sech2;
      }
      float d = keep ? gtot : 0.f;
      const bool in_window = (fabsf(sub_rn(u, th[i])) < half_w) && (u > 0.f);
      if (in_window) acc_t[i] += (gtot / s[i]) * (-th[i] / window);
      if (g_lp && th[i] > h) {
        d -= gl * np[i];
        acc_t[i] += gl * np[i];
        acc_s[i] += gl * (th[i] - h);
      }
      dp[i] = d;
      acc_b[i] += d;
    }
    store8<BF16, true>(d_pre, r * groups + g, dp);
  }
  const int64_t off = (int64_t)blockIdx.y * groups + g;
  store8<false>(part_bias, off, acc_b);
  store8<false>(part_theta, off, acc_t);
  if (part_scale) store8<false>(part_scale, off, acc_s);
}

// out[f] = sum over row groups of part[group][f], in group order
__global__ __launch_bounds__(256) void jumprelu_reduce_kernel(const float *__restrict__ part, int n_groups, int64_t F,
                                                              float *__restrict__ out) {
  const int64_t f = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (f >= F) return;
  float s = 0.f;
  for (int j = 0; j < n_groups; ++j) s += part[(int64_t)j * F + f];
  out[f] = s;
}

static int check_shape(const char *who, const void *pre, int dtype, const float *theta, const float *b_enc,
                       const float *scale, int64_t B, int64_t F) {
  SAE_REQUIRE(pre && theta, SAE_ERR_INVALID_ARG, "%s: null pointer", who);
  SAE_REQUIRE(B > 0 && F > 0 && B < (1LL << 31) && F < (1LL << 31), SAE_ERR_INVALID_ARG, "%s: bad shape", who);
  SAE_REQUIRE(dtype == SAE_F32 || dtype == SAE_BF16, SAE_ERR_INVALID_ARG, "%s: bad dtype %d", who, dtype);
  SAE_REQUIRE(F % 8 == 0, SAE_ERR_UNSUPPORTED, "%s: d_sae=%lld must be a multiple of 8", who, (long long)F);
  SAE_REQUIRE(((((uintptr_t)pre) | ((uintptr_t)theta) | ((uintptr_t)b_enc) | ((uintptr_t)scale)) & 15) == 0,
              SAE_ERR_INVALID_ARG, "%s: pre, theta, b_enc and scale must be 16-byte aligned", who);
  return SAE_OK;
}

}  // namespace sae

using namespace sae;

namespace sae {

// ---- the sparse route: threshold select -> sparse code --------------------------------------------------------
// A trained JumpReLU dictionary keeps a few dozen of its features per token.  The step then needs, per token, the
// kept features (u > theta: value u / s) and the features inside the straight-through window that are not kept
// (|u - theta| < window / 2, u > 0: value 0, flagged): the former carry the reconstruction, both carry a threshold
// gradient.  Two passes over the pre-activation (count, then emit in ascending feature order at the row offsets the
// caller derives from the counts) give a sparse code in the layout the TopK select emits, which the sparse decoder,
// the feature index and the factored optimizer pass consume as they are.  Same arithmetic per element as the dense
// kernels above.
template <bool BF16>
__device__ __forceinline__ void jr_classify(const void *__restrict__ pre, const float *__restrict__ b_enc,
                                            const float *__restrict__ scale, const float *__restrict__ theta, int64_t rbase,
                                            int64_t g, float half_w, float (&a)[8], bool (&keep)[8], bool (&win)[8]) {
  float p[8], b[8], s[8], th[8];
  load8<BF16, false>(pre, rbase + g, p);
  load8_f32_or(b_enc, g, 0.f, b);
  load8_f32_or(scale, g, 1.f, s);
  load8<false>(theta, g, th);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float h = p[i] + b[i];
    const float u = mul_rn(h, s[i]);      // a rounded product, as the tensor h * norm is: never fused into u - theta
    keep[i] = u > th[i];
    win[i] = (fabsf(sub_rn(u, th[i])) < half_w) && (u > 0.f);
    a[i] = keep[i] ? (scale ? u / s[i] : h) : 0.f;
  }
}

// With the per-granule margins of the encoder product's epilogue (margin[row][F / 64] = the largest (h s - theta) of
// the granule) only granules whose margin reaches -window / 2 can hold an entry: their numbers, ascending, are listed
// in LDS and the kernels below walk the 16-byte chunks of those granules instead of the whole row.  Returns the number
// of listed granules (the same in every thread).  `tot` is JR_THREADS / 64 ints of LDS.
constexpr int JR_MAX_GRANULES = 4096;
__device__ __forceinline__ int jr_live_granules(const float *__restrict__ margin_row, int n_gran, float half_w,
                                                uint16_t *__restrict__ live, int *__restrict__ tot) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int run = 0;
  for (int g0 = 0; g0 < n_gran; g0 += JR_THREADS) {
    const int g = g0 + threadIdx.x;
    const bool on = g < n_gran && margin_row[g] > -half_w;
    const unsigned long long m = __ballot(on);
    __syncthreads();                                  // the previous round's totals have been read
    if (lane == 0) tot[wave] = __popcll(m);
    __syncthreads();
    int before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < JR_THREADS / 64; ++w) {
      const int t = tot[w];
      before += w < wave ? t : 0;
      total += t;
    }
    if (on) live[run + before + __popcll(m & ((1ull << lane) - 1ull))] = (uint16_t)g;
    run += total;
  }
  __syncthreads();
  return run;
}

template <bool BF16>
__global__ __launch_bounds__(JR_THREADS) void jumprelu_select_count_kernel(
    const void *__restrict__ pre, const float *__restrict__ b_enc, const float *__restrict__ scale,
    const float *__restrict__ theta, int64_t F, float half_w, int32_t *__restrict__ row_nnz, const float *__restrict__ margin) {
  __shared__ float red[JR_THREADS / 64];
  __shared__ uint16_t live[JR_MAX_GRANULES];
  __shared__ int tot[JR_THREADS / 64];
  const int64_t row = blockIdx.x;
  int64_t groups = F >> 3;
  const int64_t rbase = row * groups;
  if (margin) groups = 8 * (int64_t)jr_live_granules(margin + row * (F >> 6), (int)(F >> 6), half_w, live, tot);
  int cnt = 0;
  for (int64_t c = threadIdx.x; c < groups; c += JR_THREADS) {
    const int64_t g = margin ? (int64_t)live[c >> 3] * 8 + (c & 7) : c;
    float a[8];
    bool keep[8], win[8];
    jr_classify<BF16>(pre, b_enc, scale, theta, rbase, g, half_w, a, keep, win);
#pragma unroll
    for (int i = 0; i < 8; ++i) cnt += (keep[i] || win[i]) ? 1 : 0;
  }
  const float t = block_sum<JR_THREADS / 64>((float)cnt, red);
  if (threadIdx.x == 0) row_nnz[row] = (int32_t)t;
}

template <bool BF16>
__global__ __launch_bounds__(JR_THREADS) void jumprelu_select_emit_kernel(
    const void *__restrict__ pre, const float *__restrict__ b_enc, const float *__restrict__ scale,
    const float *__restrict__ pen, const float *__restrict__ theta, int64_t F, float half_w, float tanh_c,
    const int64_t *__restrict__ row_off, int32_t *__restrict__ idx, float *__restrict__ val, float *__restrict__ in_window,
    int64_t capacity, float *__restrict__ tanh_tok, float *__restrict__ l0_tok, const float *__restrict__ margin) {
  __shared__ float red[JR_THREADS / 64];
  __shared__ int wave_tot[JR_THREADS / 64];
  __shared__ uint16_t live[JR_MAX_GRANULES];
  const int64_t row = blockIdx.x;
  int64_t groups = F >> 3;
  const int64_t rbase = row * groups;
  if (margin) groups = 8 * (int64_t)jr_live_granules(margin + row * (F >> 6), (int)(F >> 6), half_w, live, wave_tot);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int64_t run = row_off[row];
  float tsum = 0.f, kept = 0.f;
  for (int64_t g0 = 0; g0 < groups; g0 += JR_THREADS) {
    const int64_t c = g0 + threadIdx.x;
    // chunk c of the walk: of the row, or of the listed granules (ascending either way, so the entries come out in
    // ascending feature order)
    const int64_t g = (margin && c < groups) ? (int64_t)live[c >> 3] * 8 + (c & 7) : c;
    float a[8];
    bool keep[8], win[8];
    int cnt = 0;
    if (c < groups) {
      jr_classify<BF16>(pre, b_enc, scale, theta, rbase, g, half_w, a, keep, win);
#pragma unroll
      for (int i = 0; i < 8; ++i) cnt += (keep[i] || win[i]) ? 1 : 0;
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) { a[i] = 0.f; keep[i] = win[i] = false; }
    }
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
    for (int w = 0; w < JR_THREADS / 64; ++w) {
      const int t = wave_tot[w];
      before += w < wave ? t : 0;
      total += t;
    }
    int64_t pos = run + before + incl - cnt;
    if (cnt) {
      float np[8];
      load8_f32_or(pen, g, 1.f, np);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (keep[i] || win[i]) {
          if (pos < capacity) {
            idx[pos] = (int32_t)(g * 8 + i);
            val[pos] = a[i];
            in_window[pos] = win[i] ? 1.f : 0.f;
          }
          ++pos;
        }
        if (keep[i]) {
          kept += 1.f;
          if (tanh_tok) tsum += tanh_pos(tanh_c * a[i] * np[i]);
        }
      }
    }
    run += total;
  }
  if (tanh_tok) {
    const float t = block_sum<JR_THREADS / 64>(tsum, red);
    if (threadIdx.x == 0) tanh_tok[row] = t;
  }
  if (l0_tok) {
    const float t = block_sum<JR_THREADS / 64>(kept, red);
    if (threadIdx.x == 0) l0_tok[row] = t;
  }
}

}  // namespace sae

extern "C" int sae_jumprelu_select_count(const void *pre, int dtype, const float *b_enc, const float *scale, const float *theta,
                                         const float *granule_margin, double window, int64_t B, int64_t F, int32_t *row_nnz,
                                         void *stream) {
  using namespace sae;
  SAE_REQUIRE(pre && theta && row_nnz, SAE_ERR_INVALID_ARG, "jumprelu_select_count: null pointer");
  SAE_REQUIRE(!granule_margin || (F % 64 == 0 && F / 64 <= JR_MAX_GRANULES), SAE_ERR_UNSUPPORTED,
              "jumprelu_select_count: granule margins need F a multiple of 64, at most %d", 64 * JR_MAX_GRANULES);
  SAE_REQUIRE(B > 0 && F > 0 && (F & 7) == 0 && B < ((int64_t)1 << 31), SAE_ERR_INVALID_ARG,
              "jumprelu_select_count: B > 0 and F a positive multiple of 8 expected");
  SAE_REQUIRE(dtype == SAE_F32 || dtype == SAE_BF16, SAE_ERR_INVALID_ARG, "jumprelu_select_count: bad dtype");
  const float hw = 0.5f * (float)window;
  if (dtype == SAE_BF16)
    hipLaunchKernelGGL(jumprelu_select_count_kernel<true>, dim3((unsigned)B), dim3(JR_THREADS), 0, (hipStream_t)stream, pre, b_enc,
                       scale, theta, F, hw, row_nnz, granule_margin);
  else
    hipLaunchKernelGGL(jumprelu_select_count_kernel<false>, dim3((unsigned)B), dim3(JR_THREADS), 0, (hipStream_t)stream, pre, b_enc,
                       scale, theta, F, hw, row_nnz, granule_margin);
  return check_launch("jumprelu_select_count");
}

extern "C" int sae_jumprelu_select_emit(const void *pre, int dtype, const float *b_enc, const float *scale, const float *pen_norm,
                                        const float *theta, const float *granule_margin, double window, double tanh_c, int64_t B,
                                        int64_t F,
                                        const int64_t *row_off, int32_t *idx, float *val, float *in_window, int64_t capacity,
                                        float *tanh_tok, float *l0_tok, void *stream) {
  using namespace sae;
  SAE_REQUIRE(pre && theta && row_off && idx && val && in_window, SAE_ERR_INVALID_ARG, "jumprelu_select_emit: null pointer");
  SAE_REQUIRE(!granule_margin || (F % 64 == 0 && F / 64 <= JR_MAX_GRANULES), SAE_ERR_UNSUPPORTED,
              "jumprelu_select_emit: granule margins need F a multiple of 64, at most %d", 64 * JR_MAX_GRANULES);
  SAE_REQUIRE(B > 0 && F > 0 && (F & 7) == 0 && B < ((int64_t)1 << 31) && capacity >= 0, SAE_ERR_INVALID_ARG,
              "jumprelu_select_emit: B > 0 and F a positive multiple of 8 expected");
  SAE_REQUIRE(dtype == SAE_F32 || dtype == SAE_BF16, SAE_ERR_INVALID_ARG, "jumprelu_select_emit: bad dtype");
  const float hw = 0.5f * (float)window;
  if (dtype == SAE_BF16)
    hipLaunchKernelGGL(jumprelu_select_emit_kernel<true>, dim3((unsigned)B), dim3(JR_THREADS), 0, (hipStream_t)stream, pre, b_enc,
                       scale, pen_norm, theta, F, hw, (float)tanh_c, row_off, idx, val, in_window, capacity, tanh_tok, l0_tok, granule_margin);
  else
    hipLaunchKernelGGL(jumprelu_select_emit_kernel<false>, dim3((unsigned)B), dim3(JR_THREADS), 0, (hipStream_t)stream, pre, b_enc,
                       scale, pen_norm, theta, F, hw, (float)tanh_c, row_off, idx, val, in_window, capacity, tanh_tok, l0_tok, granule_margin);
  return check_launch("jumprelu_select_emit");
}

extern "C" int sae_jumprelu_fwd(const void *pre, int dtype, const float *b_enc, const float *scale,
                                const float *pen_norm, const float *theta, int64_t B, int64_t F, double tanh_c_d, void *acts, float *tanh_tok, float *lp_tok,
                                float *l0_tok, void *stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  const float tanh_c = (float)tanh_c_d;
  int rc = check_shape("jumprelu_fwd", pre, dtype, theta, b_enc, scale, B, F);
  if (rc) return rc;
  SAE_REQUIRE(acts && (((uintptr_t)acts) & 15) == 0, SAE_ERR_INVALID_ARG, "jumprelu_fwd: acts must be a 16-byte aligned buffer");
  const unsigned fwd_blocks = (unsigned)((B + JR_FWD_ROWS - 1) / JR_FWD_ROWS);
  if (dtype == SAE_BF16)
    hipLaunchKernelGGL(jumprelu_fwd_kernel<true>, dim3(fwd_blocks), dim3(JR_THREADS), 0, st, pre, b_enc, scale, pen_norm,
                       theta, B, F, tanh_c, acts, tanh_tok, lp_tok, l0_tok);
  else
    hipLaunchKernelGGL(jumprelu_fwd_kernel<false>, dim3(fwd_blocks), dim3(JR_THREADS), 0, st, pre, b_enc, scale, pen_norm,
                       theta, B, F, tanh_c, acts, tanh_tok, lp_tok, l0_tok);
  return check_launch("jumprelu_fwd");
}

extern "C" int64_t sae_jumprelu_bwd_workspace_bytes(int64_t B, int64_t F) {
  const int64_t n_groups = (B + JR_ROWS - 1) / JR_ROWS;
  return 3 * n_groups * F * (int64_t)sizeof(float);
}

extern "C" int sae_jumprelu_bwd(const void *pre, int dtype, const float *b_enc, const float *scale,
                                const float *pen_norm, const float *theta, const void *d_acts, const float *g_tanh, double tanh_c_d, const float *g_lp,
                                double window_d, int64_t B, int64_t F, void *d_pre, float *d_bias, float *d_theta,
                                float *d_pen_norm, void *workspace, int64_t workspace_bytes, void *stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  const float tanh_c = (float)tanh_c_d, window = (float)window_d;
  int rc = check_shape("jumprelu_bwd", pre, dtype, theta, b_enc, scale, B, F);
  if (rc) return rc;
  SAE_REQUIRE(d_acts && d_pre && d_bias && d_theta, SAE_ERR_INVALID_ARG, "jumprelu_bwd: null pointer");
  SAE_REQUIRE(((((uintptr_t)d_acts) | ((uintptr_t)d_pre)) & 15) == 0, SAE_ERR_INVALID_ARG,
              "jumprelu_bwd: d_acts and d_pre must be 16-byte aligned");
  SAE_REQUIRE(window > 0.f, SAE_ERR_INVALID_ARG, "jumprelu_bwd: window must be positive");
  SAE_REQUIRE(!d_pen_norm || pen_norm, SAE_ERR_INVALID_ARG, "jumprelu_bwd: d_pen_norm needs pen_norm");
  SAE_REQUIRE((((uintptr_t)pen_norm) & 15) == 0, SAE_ERR_INVALID_ARG, "jumprelu_bwd: pen_norm must be 16-byte aligned");
  SAE_REQUIRE(workspace && workspace_bytes >= sae_jumprelu_bwd_workspace_bytes(B, F) && (((uintptr_t)workspace) & 15) == 0,
              SAE_ERR_WORKSPACE, "jumprelu_bwd: workspace too small or misaligned");
  const int64_t n_groups = (B + JR_ROWS - 1) / JR_ROWS;
  float *part_bias = reinterpret_cast<float *>(workspace);
  float *part_theta = part_bias + n_groups * F;
  float *part_scale = d_pen_norm ? part_theta + n_groups * F : nullptr;
  const int64_t groups = F >> 3;
  const dim3 grid((unsigned)((groups + JR_THREADS - 1) / JR_THREADS), (unsigned)n_groups);
  if (dtype == SAE_BF16)
    hipLaunchKernelGGL(jumprelu_bwd_kernel<true>, grid, dim3(JR_THREADS), 0, st, pre, b_enc, scale, pen_norm, theta, d_acts, g_tanh,
                       tanh_c, g_lp, window, B, F, d_pre, part_bias, part_theta, part_scale);
  else
    hipLaunchKernelGGL(jumprelu_bwd_kernel<false>, grid, dim3(JR_THREADS), 0, st, pre, b_enc, scale, pen_norm, theta, d_acts, g_tanh,
                       tanh_c, g_lp, window, B, F, d_pre, part_bias, part_theta, part_scale);
  rc = check_launch("jumprelu_bwd");
  if (rc) return rc;
  const unsigned rb = (unsigned)((F + 255) / 256);
  hipLaunchKernelGGL(jumprelu_reduce_kernel, dim3(rb), dim3(256), 0, st, part_bias, (int)n_groups, F, d_bias);
  hipLaunchKernelGGL(jumprelu_reduce_kernel, dim3(rb), dim3(256), 0, st, part_theta, (int)n_groups, F, d_theta);
  if (d_pen_norm)
    hipLaunchKernelGGL(jumprelu_reduce_kernel, dim3(rb), dim3(256), 0, st, part_scale, (int)n_groups, F, d_pen_norm);
  return check_launch("jumprelu_bwd(reduce)");
}
