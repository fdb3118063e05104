// Sparse decoder for gfx950: a token's reconstruction is the weighted sum of the few W_D
// rows its sparse code names.  Bandwidth-bound: every active (token, feature) pair costs one
// row of d_model weights, fetched with 16-byte loads that a workgroup issues fully coalesced
// (256 lanes x 16 bytes = 4 KiB of one row per instruction).
//
// One workgroup of 256 threads per token.
//   phase 1 (gather-accumulate): thread t owns the 8-element segments t, t+256, ... of the
//     row and keeps them in registers while the workgroup walks the token's slots, four rows
//     in flight at a time.
//   phase 2 (optional, fused loss): recon - label, the token's squared error, and
//     grad_recon = 2 * tok_w * (recon - label), written out and parked in LDS.
//   phase 3 (optional, d val): wave w takes slots w, w+4, ...; it streams the row again (it
//     was just read, so it comes from L2 / Infinity Cache) against the LDS copy of
//     grad_recon and reduces across its 64 lanes.  No workgroup barrier per slot.
#include "common.h"

namespace sae {

constexpr int DEC_THREADS = 256;
constexpr int DEC_WAVES = DEC_THREADS / 64;

template <bool W_BF16>
__device__ __forceinline__ void load8(const void *row, int seg, float (&o)[8]) {
  if constexpr (W_BF16) {
    const u32x4 r = reinterpret_cast<const u32x4 *>(row)[seg];
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      o[2 * q] = __uint_as_float(w[q] << 16);
      o[2 * q + 1] = __uint_as_float(w[q] & 0xffff0000u);
    }
  } else {
    const float4 a = reinterpret_cast<const float4 *>(row)[2 * seg];
    const float4 b = reinterpret_cast<const float4 *>(row)[2 * seg + 1];
    o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
    o[4] = b.x; o[5] = b.y; o[6] = b.z; o[7] = b.w;
  }
}

// FWD: compute recon.  LOSS: also loss / grad_recon (implies FWD).  DVAL: compute dval from
// grad_recon (own, when LOSS; read from memory otherwise).
template <bool W_BF16, int SEGS, bool FWD, bool LOSS, bool DVAL, int THREADS = DEC_THREADS, bool SHORT_LISTS = false>
__global__ __launch_bounds__(THREADS) void sparse_decode_kernel(
    const int32_t *__restrict__ idx, const float *__restrict__ val, const int64_t *__restrict__ row_off,
    const int32_t *__restrict__ row_nnz, const void *__restrict__ w_dec, const float *__restrict__ b_dec,
    const float *__restrict__ label, const float *__restrict__ tok_w, float *__restrict__ recon,
    float *__restrict__ loss_tok, float *__restrict__ grad_recon, float *__restrict__ dval, int d, int acc_dval) {
  extern __shared__ __attribute__((aligned(16))) float g_lds[];  // [d] when DVAL
  constexpr int WAVES = THREADS / 64;
  __shared__ float red[WAVES];
  const int b = blockIdx.x, tid = threadIdx.x;
  const int64_t off = row_off[b];
  const int nnz = row_nnz[b];
  const int n_seg = d >> 3;
  const size_t row_bytes = (size_t)d * (W_BF16 ? 2 : 4);
  const char *wbase = reinterpret_cast<const char *>(w_dec);

  float acc[SEGS][8];
  if constexpr (FWD) {
#pragma unroll
    for (int s = 0; s < SEGS; ++s)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[s][e] = 0.f;

    // rows in flight per step.  Few: what hides the gathers' latency is the number of tokens resident on a CU, and
    // the staging registers decide that (d = 4096: two rows, 8 waves per SIMD, 0.59 ms; four rows, 5 waves, 0.72 ms)
    constexpr int U = SEGS == 1 ? 4 : (SEGS <= 4 ? 2 : 1);
    int j = 0;
    for (; j + U <= nnz; j += U) {
      float w[U][SEGS][8];
      float v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int f = idx[off + j + u];
        v[u] = val[off + j + u];
        const char *row = wbase + (size_t)f * row_bytes;
#pragma unroll
        for (int s = 0; s < SEGS; ++s) {
          const int seg = tid + s * THREADS;
          if (seg < n_seg) load8<W_BF16>(row, seg, w[u][s]);
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int s = 0; s < SEGS; ++s)
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[s][e] = fmaf(v[u], w[u][s][e], acc[s][e]);
    }
    for (; j < nnz; ++j) {
      const int f = idx[off + j];
      const float v = val[off + j];
      const char *row = wbase + (size_t)f * row_bytes;
#pragma unroll
      for (int s = 0; s < SEGS; ++s) {
        const int seg = tid + s * THREADS;
        if (seg < n_seg) {
          float w[8];
          load8<W_BF16>(row, seg, w);
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[s][e] = fmaf(v, w[e], acc[s][e]);
        }
      }
    }

    float sq = 0.f;
    const float tw = LOSS ? (tok_w ? tok_w[b] : 1.f) : 0.f;
#pragma unroll
    for (int s = 0; s < SEGS; ++s) {
      const int seg = tid + s * THREADS;
      if (seg < n_seg) {
        const size_t o = (size_t)b * d + (size_t)seg * 8;
        float r[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) r[e] = acc[s][e];
        if (b_dec) {
          float bd[8];
          load8<false>(b_dec, seg, bd);
#pragma unroll
          for (int e = 0; e < 8; ++e) r[e] += bd[e];
        }
        if (recon) {
          reinterpret_cast<float4 *>(recon + o)[0] = make_float4(r[0], r[1], r[2], r[3]);
          reinterpret_cast<float4 *>(recon + o)[1] = make_float4(r[4], r[5], r[6], r[7]);
        }
        if constexpr (LOSS) {
          float y[8], g[8];
          load8<false>(label + (size_t)b * d, seg, y);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float df = r[e] - y[e];
            sq = fmaf(df, df, sq);
            g[e] = 2.f * tw * df;
          }
          reinterpret_cast<float4 *>(grad_recon + o)[0] = make_float4(g[0], g[1], g[2], g[3]);
          reinterpret_cast<float4 *>(grad_recon + o)[1] = make_float4(g[4], g[5], g[6], g[7]);
          if constexpr (DVAL) {
            reinterpret_cast<float4 *>(g_lds + seg * 8)[0] = make_float4(g[0], g[1], g[2], g[3]);
            reinterpret_cast<float4 *>(g_lds + seg * 8)[1] = make_float4(g[4], g[5], g[6], g[7]);
          }
        }
      }
    }
    if constexpr (LOSS) {
      const float tot = block_sum<WAVES>(sq, red);
      if (tid == 0) loss_tok[b] = tw * tot;
    }
  }

  if constexpr (DVAL) {
    if constexpr (!LOSS) {
      // grad_recon comes from memory
      for (int seg = tid; seg < n_seg; seg += THREADS) {
        const float4 a = reinterpret_cast<const float4 *>(grad_recon + (size_t)b * d)[2 * seg];
        const float4 c = reinterpret_cast<const float4 *>(grad_recon + (size_t)b * d)[2 * seg + 1];
        reinterpret_cast<float4 *>(g_lds + seg * 8)[0] = a;
        reinterpret_cast<float4 *>(g_lds + seg * 8)[1] = c;
      }
    }
    __syncthreads();
    const int lane = tid & 63, wave = tid >> 6;
    if constexpr (SHORT_LISTS) {
      // short rows (n_seg <= 128) and short row lists: a wave takes two rows at a time (four 16-byte loads in flight
      // per lane instead of two); a lane's products run over its segments in ascending order as below, so a row's
      // dot product has the same bits.  A separate instantiation: with long lists (the CLT's prefix codes) this
      // path is slower (4.7 -> 6.4 ms), and its registers alone cost the other path residency (4.7 -> 7.2 ms).
      for (int j0 = wave * 2; j0 < nnz; j0 += WAVES * 2) {
        const bool two = j0 + 1 < nnz;
        const int f0 = idx[off + j0], f1 = idx[off + (two ? j0 + 1 : j0)];
        // the running sums these two results are added to, asked for together with the rows
        const float prev0 = (acc_dval && lane == 0) ? dval[off + j0] : 0.f;
        const float prev1 = (acc_dval && lane == 0 && two) ? dval[off + j0 + 1] : 0.f;
        const char *row0 = wbase + (size_t)f0 * row_bytes, *row1 = wbase + (size_t)f1 * row_bytes;
        float w0[2][8], w1[2][8];
#pragma unroll
        for (int l = 0; l < 2; ++l) {
          const int sg = lane + 64 * l;
          if (sg < n_seg) { load8<W_BF16>(row0, sg, w0[l]); load8<W_BF16>(row1, sg, w1[l]); }
        }
        float d0 = 0.f, d1 = 0.f;
#pragma unroll
        for (int l = 0; l < 2; ++l) {
          const int sg = lane + 64 * l;
          if (sg < n_seg) {
            const float4 g0 = reinterpret_cast<const float4 *>(g_lds + sg * 8)[0];
            const float4 g1 = reinterpret_cast<const float4 *>(g_lds + sg * 8)[1];
            d0 = fmaf(g0.x, w0[l][0], d0); d0 = fmaf(g0.y, w0[l][1], d0); d0 = fmaf(g0.z, w0[l][2], d0); d0 = fmaf(g0.w, w0[l][3], d0);
            d0 = fmaf(g1.x, w0[l][4], d0); d0 = fmaf(g1.y, w0[l][5], d0); d0 = fmaf(g1.z, w0[l][6], d0); d0 = fmaf(g1.w, w0[l][7], d0);
            d1 = fmaf(g0.x, w1[l][0], d1); d1 = fmaf(g0.y, w1[l][1], d1); d1 = fmaf(g0.z, w1[l][2], d1); d1 = fmaf(g0.w, w1[l][3], d1);
            d1 = fmaf(g1.x, w1[l][4], d1); d1 = fmaf(g1.y, w1[l][5], d1); d1 = fmaf(g1.z, w1[l][6], d1); d1 = fmaf(g1.w, w1[l][7], d1);
          }
        }
        d0 = wave_sum(d0); d1 = wave_sum(d1);
        if (lane == 0) {
          dval[off + j0] = acc_dval ? prev0 + d0 : d0;
          if (two) dval[off + j0 + 1] = acc_dval ? prev1 + d1 : d1;
        }
      }
      return;
    }
    for (int j = wave; j < nnz; j += WAVES) {
      const int f = idx[off + j];
      const char *row = wbase + (size_t)f * row_bytes;
      const float prev = (acc_dval && lane == 0) ? dval[off + j] : 0.f;   // asked for together with the row
      float dot = 0.f;
      for (int seg = lane; seg < n_seg; seg += 64 * 4) {
        float w[4][8];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int sg = seg + 64 * u;
          if (sg < n_seg) load8<W_BF16>(row, sg, w[u]);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int sg = seg + 64 * u;
          if (sg < n_seg) {
            const float4 g0 = reinterpret_cast<const float4 *>(g_lds + sg * 8)[0];
            const float4 g1 = reinterpret_cast<const float4 *>(g_lds + sg * 8)[1];
            dot = fmaf(g0.x, w[u][0], dot); dot = fmaf(g0.y, w[u][1], dot);
            dot = fmaf(g0.z, w[u][2], dot); dot = fmaf(g0.w, w[u][3], dot);
            dot = fmaf(g1.x, w[u][4], dot); dot = fmaf(g1.y, w[u][5], dot);
            dot = fmaf(g1.z, w[u][6], dot); dot = fmaf(g1.w, w[u][7], dot);
          }
        }
      }
      dot = wave_sum(dot);
      if (lane == 0) dval[off + j] = acc_dval ? prev + dot : dot;
    }
  }
}

template <bool W_BF16, bool FWD, bool LOSS, bool DVAL>
static int launch_decode(const int32_t *idx, const float *val, const int64_t *row_off, const int32_t *row_nnz,
                         const void *w_dec, const float *b_dec, const float *label, const float *tok_w, float *recon,
                         float *loss_tok, float *grad_recon, float *dval, int64_t B, int64_t d, hipStream_t st,
                         int64_t n_slots = 0, int acc_dval = 0) {
  const int n_seg = (int)(d / 8);
  const size_t lds = DVAL ? (size_t)d * sizeof(float) : 0;
  const int segs = (n_seg + DEC_THREADS - 1) / DEC_THREADS;
#define SAE_DEC_LAUNCH(S)                                                                                         \
  do {                                                                                                            \
    auto kern = sparse_decode_kernel<W_BF16, S, FWD, LOSS, DVAL>;                                                 \
    if (lds > 48 * 1024) {                                                                                        \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                                    \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);                   \
      if (e != hipSuccess) return fail(SAE_ERR_LAUNCH, "sparse_decode: LDS reservation failed: %s", hipGetErrorString(e)); \
    }                                                                                                             \
    hipLaunchKernelGGL(kern, dim3((unsigned)B), dim3(DEC_THREADS), lds, st, idx, val, row_off, row_nnz, w_dec,    \
                       b_dec, label, tok_w, recon, loss_tok, grad_recon, dval, (int)d, acc_dval);                 \
  } while (0)
  // Short rows (d <= 1024): two waves per token, so that most lanes own a segment and twice as many tokens are
  // resident per CU (the gathers' latency is hidden by resident tokens).  Not when the d val phase has long row
  // lists to walk (more than 128 slots per token on average): there each wave takes one row at a time and four
  // waves per token finish sooner (Lorsa's 64-row tokens 0.43 -> 0.30 ms with two waves, the CLT's up to 768-row
  // prefix codes 4.7 -> 6.1 ms).
  const bool short_lists = n_slots <= 128 * B;   // also when the caller gave no slot count (forward only)
  if (n_seg <= 128 && (!DVAL || short_lists)) {
    auto kern = sparse_decode_kernel<W_BF16, 1, FWD, LOSS, DVAL, 128, true>;
    hipLaunchKernelGGL(kern, dim3((unsigned)B), dim3(128), lds, st, idx, val, row_off, row_nnz, w_dec, b_dec, label,
                       tok_w, recon, loss_tok, grad_recon, dval, (int)d, acc_dval);
  } else if (!FWD) SAE_DEC_LAUNCH(1);
  else if (segs <= 1) SAE_DEC_LAUNCH(1);
  else if (segs <= 2) SAE_DEC_LAUNCH(2);
  else if (segs <= 4) SAE_DEC_LAUNCH(4);
  else SAE_DEC_LAUNCH(8);
#undef SAE_DEC_LAUNCH
  return check_launch("sparse_decode");
}

static int check_common(const char *who, const void *idx, const void *row_off, const void *row_nnz, const void *w_dec,
                        int w_dtype, int64_t B, int64_t d, int64_t F) {
  SAE_REQUIRE(idx && row_off && row_nnz && w_dec, SAE_ERR_INVALID_ARG, "%s: null pointer", who);
  SAE_REQUIRE(B > 0 && d > 0 && F > 0, SAE_ERR_INVALID_ARG, "%s: B, d, F must be positive", who);
  SAE_REQUIRE(w_dtype == SAE_F32 || w_dtype == SAE_BF16, SAE_ERR_INVALID_ARG, "%s: bad w_dtype %d", who, w_dtype);
  SAE_REQUIRE(d % 8 == 0, SAE_ERR_UNSUPPORTED, "%s: d_model=%lld must be a multiple of 8", who, (long long)d);
  SAE_REQUIRE(d <= 8LL * 8 * DEC_THREADS, SAE_ERR_UNSUPPORTED, "%s: d_model=%lld above %d", who, (long long)d,
              8 * 8 * DEC_THREADS);
  SAE_REQUIRE((((uintptr_t)w_dec) & 15) == 0, SAE_ERR_INVALID_ARG, "%s: w_dec must be 16-byte aligned", who);
  return SAE_OK;
}

}  // namespace sae

extern "C" int sae_sparse_decode_fwd(const int32_t *idx, const float *val, const int64_t *row_off,
                                     const int32_t *row_nnz, const void *w_dec, int w_dtype, const float *b_dec,
                                     float *recon, int64_t B, int64_t d, int64_t F, void *stream) {
  using namespace sae;
  int rc = check_common("sparse_decode_fwd", idx, row_off, row_nnz, w_dec, w_dtype, B, d, F);
  if (rc) return rc;
  SAE_REQUIRE(val && recon, SAE_ERR_INVALID_ARG, "sparse_decode_fwd: null pointer");
  hipStream_t st = (hipStream_t)stream;
  if (w_dtype == SAE_BF16)
    return launch_decode<true, true, false, false>(idx, val, row_off, row_nnz, w_dec, b_dec, nullptr, nullptr, recon,
                                                   nullptr, nullptr, nullptr, B, d, st);
  return launch_decode<false, true, false, false>(idx, val, row_off, row_nnz, w_dec, b_dec, nullptr, nullptr, recon,
                                                  nullptr, nullptr, nullptr, B, d, st);
}

extern "C" int sae_sparse_decode_bwd_dval(const int32_t *idx, const int64_t *row_off, const int32_t *row_nnz,
                                          const float *grad_recon, const void *w_dec, int w_dtype, float *dval,
                                          int64_t B, int64_t d, int64_t F, int64_t n_slots, void *stream) {
  using namespace sae;
  int rc = check_common("sparse_decode_bwd_dval", idx, row_off, row_nnz, w_dec, w_dtype, B, d, F);
  if (rc) return rc;
  SAE_REQUIRE(grad_recon && dval && n_slots > 0, SAE_ERR_INVALID_ARG, "sparse_decode_bwd_dval: null pointer / n_slots");
  hipStream_t st = (hipStream_t)stream;
  rc = zero_fill(dval, (size_t)n_slots * sizeof(float), st);
  if (rc) return rc;
  if (w_dtype == SAE_BF16)
    return launch_decode<true, false, false, true>(idx, nullptr, row_off, row_nnz, w_dec, nullptr, nullptr, nullptr,
                                                   nullptr, nullptr, const_cast<float *>(grad_recon), dval, B, d, st, n_slots);
  return launch_decode<false, false, false, true>(idx, nullptr, row_off, row_nnz, w_dec, nullptr, nullptr, nullptr,
                                                  nullptr, nullptr, const_cast<float *>(grad_recon), dval, B, d, st, n_slots);
}

extern "C" int sae_sparse_decode_mse_fused(const int32_t *idx, const float *val, const int64_t *row_off,
                                           const int32_t *row_nnz, const void *w_dec, int w_dtype, const float *b_dec,
                                           const float *label, const float *tok_w, float *recon, float *loss_tok,
                                           float *grad_recon, float *dval, int64_t B, int64_t d, int64_t F,
                                           int64_t n_slots, void *stream) {
  using namespace sae;
  int rc = check_common("sparse_decode_mse_fused", idx, row_off, row_nnz, w_dec, w_dtype, B, d, F);
  if (rc) return rc;
  SAE_REQUIRE(val && label && loss_tok && grad_recon && dval && n_slots > 0, SAE_ERR_INVALID_ARG,
              "sparse_decode_mse_fused: null pointer / n_slots");
  hipStream_t st = (hipStream_t)stream;
  rc = zero_fill(dval, (size_t)n_slots * sizeof(float), st);
  if (rc) return rc;
  if (w_dtype == SAE_BF16)
    return launch_decode<true, true, true, true>(idx, val, row_off, row_nnz, w_dec, b_dec, label, tok_w, recon,
                                                 loss_tok, grad_recon, dval, B, d, st, n_slots);
  return launch_decode<false, true, true, true>(idx, val, row_off, row_nnz, w_dec, b_dec, label, tok_w, recon,
                                                loss_tok, grad_recon, dval, B, d, st, n_slots);
}

extern "C" int sae_sparse_decode_mse_fused_acc(const int32_t *idx, const float *val, const int64_t *row_off,
                                               const int32_t *row_nnz, const void *w_dec, int w_dtype, const float *b_dec,
                                               const float *label, const float *tok_w, float *recon, float *loss_tok,
                                               float *grad_recon, float *dval_acc, int64_t B, int64_t d, int64_t F,
                                               int64_t n_slots, void *stream) {
  using namespace sae;
  int rc = check_common("sparse_decode_mse_fused_acc", idx, row_off, row_nnz, w_dec, w_dtype, B, d, F);
  if (rc) return rc;
  SAE_REQUIRE(val && label && loss_tok && grad_recon && dval_acc && n_slots > 0, SAE_ERR_INVALID_ARG,
              "sparse_decode_mse_fused_acc: null pointer / n_slots");
  hipStream_t st = (hipStream_t)stream;
  if (w_dtype == SAE_BF16)
    return launch_decode<true, true, true, true>(idx, val, row_off, row_nnz, w_dec, b_dec, label, tok_w, recon,
                                                 loss_tok, grad_recon, dval_acc, B, d, st, n_slots, 1);
  return launch_decode<false, true, true, true>(idx, val, row_off, row_nnz, w_dec, b_dec, label, tok_w, recon,
                                                loss_tok, grad_recon, dval_acc, B, d, st, n_slots, 1);
}
