// Fused Adam for gfx950: one streaming pass that reads g, p, m, v and writes p, m, v
// (28 bytes per parameter), optionally the bf16 shadow of p that the next step's GEMM and
// row gathers read (+2 bytes) and the L2 norm of every updated row (the next step's
// decoder_norm(), free because the row is in registers anyway).
#include "common.h"

namespace sae {

struct AdamScalars {
  float beta1, beta2, one_minus_beta1, one_minus_beta2, step_size, inv_bc2_sqrt, eps, bc2_sqrt;
};

// Every multiply-add is written out as a fused one, so that no kernel that inlines this leaves the choice of
// what to fuse to the compiler: the kernels that promise identical bits (the plain passes, the passes that rebuild
// the gradient rows) then really compute the same thing.
__device__ __forceinline__ float adam_one(float &p, float g, float &m, float &v, const AdamScalars &a) {
  m = fmaf(a.one_minus_beta1, sub_rn(g, m), m);   // lerp, as torch does
  v = fmaf(a.beta2, v, mul_rn(mul_rn(a.one_minus_beta2, g), g));
  const float denom = fmaf(sqrtf(v), a.inv_bc2_sqrt, a.eps);
  p = fmaf(-a.step_size, m / denom, p);
  return p;
}

// The update of a parameter held in bf16 with bf16 moments, as torch's multi-tensor Adam computes it on such
// tensors (the reference's optimizer when the dictionary's dtype is bfloat16, trainer.py:375-390): every
// element-wise operation works in fp32 and rounds its result to bf16 -- lerp for m; mul then addcmul for v;
// sqrt, division by sqrt(bias correction 2) and the addition of eps for the denominator; addcdiv for p.  (With
// beta2 = 0.999 the product v * beta2 mostly rounds back to v: that is what the reference's arithmetic does.)
// Rounding goes through the hardware's packed conversion (two values per instruction); the square root, the
// division by sqrt(bias correction 2) and the quotient m / denominator use the single-instruction forms (1 ulp in
// fp32), whose error disappears in the rounding to bf16 that follows each of them except on rare boundary cases:
// with IEEE division and square root sequences the pass is bound by its arithmetic, not by memory.
// two elements at a time; both lanes of a pair see exactly the scalar sequence
__device__ __forceinline__ void adam_two_lowp(float &p0, float &p1, float g0, float g1, float &m0, float &m1, float &v0,
                                              float &v1, const AdamScalars &a) {
  bf16_round2(g0, g1);
  m0 = fmaf(a.one_minus_beta1, sub_rn(g0, m0), m0); m1 = fmaf(a.one_minus_beta1, sub_rn(g1, m1), m1);
  bf16_round2(m0, m1);
  v0 = mul_rn(v0, a.beta2); v1 = mul_rn(v1, a.beta2);
  bf16_round2(v0, v1);
  v0 = fmaf(mul_rn(a.one_minus_beta2, g0), g0, v0); v1 = fmaf(mul_rn(a.one_minus_beta2, g1), g1, v1);
  bf16_round2(v0, v1);
  float d0 = __builtin_amdgcn_sqrtf(v0), d1 = __builtin_amdgcn_sqrtf(v1);
  bf16_round2(d0, d1);
  d0 = mul_rn(d0, a.inv_bc2_sqrt); d1 = mul_rn(d1, a.inv_bc2_sqrt);
  bf16_round2(d0, d1);
  d0 = add_rn(d0, a.eps); d1 = add_rn(d1, a.eps);
  bf16_round2(d0, d1);
  p0 = fmaf(-a.step_size, mul_rn(m0, __builtin_amdgcn_rcpf(d0)), p0);
  p1 = fmaf(-a.step_size, mul_rn(m1, __builtin_amdgcn_rcpf(d1)), p1);
  bf16_round2(p0, p1);
}
template <bool S_BF16>
__device__ __forceinline__ void adam_any(float &p, float g, float &m, float &v, const AdamScalars &a) {
  if constexpr (S_BF16) {
    float p1 = p, m1 = m, v1 = v;
    adam_two_lowp(p, p1, g, g, m, m1, v, v1, a);
  } else {
    adam_one(p, g, m, v, a);
  }
}
template <bool S_BF16>
__device__ __forceinline__ void adam_any4(float4 &p, const float4 &g, float4 &m, float4 &v, const AdamScalars &a) {
  if constexpr (S_BF16) {
    adam_two_lowp(p.x, p.y, g.x, g.y, m.x, m.y, v.x, v.y, a);
    adam_two_lowp(p.z, p.w, g.z, g.w, m.z, m.w, v.z, v.w, a);
  } else {
    adam_one(p.x, g.x, m.x, v.x, a); adam_one(p.y, g.y, m.y, v.y, a);
    adam_one(p.z, g.z, m.z, v.z, a); adam_one(p.w, g.w, m.w, v.w, a);
  }
}

// four elements of group q of a parameter or moment array: fp32, or bf16 (widened exactly / rounded on the way out)
template <bool S_BF16>
__device__ __forceinline__ float4 load_state4(const float *base, int64_t q) {
  if constexpr (S_BF16) {
    const nt_u32x2 t = __builtin_nontemporal_load(reinterpret_cast<const nt_u32x2 *>(base) + q);
    return make_float4(__uint_as_float(t[0] << 16), __uint_as_float(t[0] & 0xffff0000u), __uint_as_float(t[1] << 16),
                       __uint_as_float(t[1] & 0xffff0000u));
  } else {
    return load_stream(base, q);
  }
}
template <bool S_BF16>
__device__ __forceinline__ void store_state4(float *base, int64_t q, const float4 &x) {
  if constexpr (S_BF16) {
    uint2 o;   // the values are bf16-representable already
    o.x = (__float_as_uint(x.x) >> 16) | (__float_as_uint(x.y) & 0xffff0000u);
    o.y = (__float_as_uint(x.z) >> 16) | (__float_as_uint(x.w) & 0xffff0000u);
    store_stream(reinterpret_cast<uint16_t *>(base), q, o);
  } else {
    store_stream(base, q, x);
  }
}
template <bool S_BF16>
__device__ __forceinline__ float load_state1(const float *base, int64_t i) {
  if constexpr (S_BF16) return bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(base)[i]);
  else return base[i];
}
template <bool S_BF16>
__device__ __forceinline__ void store_state1(float *base, int64_t i, float x) {
  if constexpr (S_BF16) reinterpret_cast<uint16_t *>(base)[i] = (uint16_t)(__float_as_uint(x) >> 16);
  else base[i] = x;
}

// four gradient elements from group q of an fp32 or a bf16 gradient (a bf16 value widens exactly)
template <bool G_BF16>
__device__ __forceinline__ float4 load_grad4(const void *g, int64_t q) {
  if constexpr (G_BF16) {
    const nt_u32x2 t = __builtin_nontemporal_load(reinterpret_cast<const nt_u32x2 *>(g) + q);
    return make_float4(__uint_as_float(t[0] << 16), __uint_as_float(t[0] & 0xffff0000u), __uint_as_float(t[1] << 16),
                       __uint_as_float(t[1] & 0xffff0000u));
  } else {
    return load_stream(reinterpret_cast<const float *>(g), q);
  }
}
template <bool G_BF16>
__device__ __forceinline__ float load_grad1(const void *g, int64_t i) {
  if constexpr (G_BF16) return bf16_bits_to_f32(reinterpret_cast<const uint16_t *>(g)[i]);
  else return reinterpret_cast<const float *>(g)[i];
}

// flat: a workgroup owns ADAM_FLAT_CHUNK consecutive groups of four elements (16 KB of each fp32 array: with a stride of
// the whole grid between a thread's groups the same update ran 15 % slower on 537 M elements).  S_BF16: p, m, v point to
// bf16 arrays (the pointer type is nominal) and the update is the low-precision one above.
constexpr int ADAM_FLAT_CHUNK = 1024;
template <bool G_BF16, bool S_BF16 = false>
__global__ __launch_bounds__(256) void adam_flat_kernel(float *__restrict__ p, const void *__restrict__ g,
                                                        float *__restrict__ m, float *__restrict__ v, int64_t n,
                                                        AdamScalars a, uint16_t *__restrict__ shadow) {
  const int64_t n4 = n >> 2;
  const int64_t first = (int64_t)blockIdx.x * ADAM_FLAT_CHUNK, last = first + ADAM_FLAT_CHUNK < n4 ? first + ADAM_FLAT_CHUNK : n4;
  for (int64_t i = first + threadIdx.x; i < last; i += 256) {
    float4 pp = load_state4<S_BF16>(p, i);
    const float4 gg = load_grad4<G_BF16>(g, i);
    float4 mm = load_state4<S_BF16>(m, i);
    float4 vv = load_state4<S_BF16>(v, i);
    adam_any4<S_BF16>(pp, gg, mm, vv, a);
    store_state4<S_BF16>(p, i, pp);
    store_state4<S_BF16>(m, i, mm);
    store_state4<S_BF16>(v, i, vv);
    if (shadow) {
      uint2 o;
      o.x = (uint32_t)f32_to_bf16_bits(pp.x) | ((uint32_t)f32_to_bf16_bits(pp.y) << 16);
      o.y = (uint32_t)f32_to_bf16_bits(pp.z) | ((uint32_t)f32_to_bf16_bits(pp.w) << 16);
      store_stream(shadow, i, o);
    }
  }
  const int64_t t = (n4 << 2) + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n) {
    float pp = load_state1<S_BF16>(p, t), mm = load_state1<S_BF16>(m, t), vv = load_state1<S_BF16>(v, t);
    adam_any<S_BF16>(pp, load_grad1<G_BF16>(g, t), mm, vv, a);
    store_state1<S_BF16>(p, t, pp); store_state1<S_BF16>(m, t, mm); store_state1<S_BF16>(v, t, vv);
    if (shadow) shadow[t] = f32_to_bf16_bits(pp);
  }
}

// row-wise: one workgroup per row of row_len (a multiple of 4) elements; also emits the row norm.  With row_coef
// the gradient of row r is g + row_coef[r] * p (product and sum rounded separately, as when that term is added to
// the gradient tensor beforehand): the gradient that reaches a weight through its row norms, d n / n times the row.
template <bool G_BF16, bool S_BF16 = false>
__global__ __launch_bounds__(256) void adam_rows_kernel(float *__restrict__ p, const void *__restrict__ g,
                                                        float *__restrict__ m, float *__restrict__ v, int row_len,
                                                        AdamScalars a, uint16_t *__restrict__ shadow,
                                                        float *__restrict__ row_norm, const float *__restrict__ row_coef) {
  __shared__ float red[4];
  const int64_t base4 = (int64_t)blockIdx.x * (row_len >> 2);
  const float rc = row_coef ? row_coef[blockIdx.x] : 0.f;
  float sq = 0.f;
  for (int i = threadIdx.x; i < (row_len >> 2); i += 256) {
    const int64_t q = base4 + i;
    float4 pp = load_state4<S_BF16>(p, q);
    float4 gg = load_grad4<G_BF16>(g, q);
    float4 mm = load_state4<S_BF16>(m, q);
    float4 vv = load_state4<S_BF16>(v, q);
    if (row_coef) {
      if constexpr (S_BF16) {   // both gradient terms exist as bf16 tensors before they are added
        gg.x = add_rn(bf16_round(gg.x), bf16_round(mul_rn(rc, pp.x))); gg.y = add_rn(bf16_round(gg.y), bf16_round(mul_rn(rc, pp.y)));
        gg.z = add_rn(bf16_round(gg.z), bf16_round(mul_rn(rc, pp.z))); gg.w = add_rn(bf16_round(gg.w), bf16_round(mul_rn(rc, pp.w)));
      } else {
        gg.x = add_rn(gg.x, mul_rn(rc, pp.x)); gg.y = add_rn(gg.y, mul_rn(rc, pp.y));
        gg.z = add_rn(gg.z, mul_rn(rc, pp.z)); gg.w = add_rn(gg.w, mul_rn(rc, pp.w));
      }
    }
    adam_any4<S_BF16>(pp, gg, mm, vv, a);
    store_state4<S_BF16>(p, q, pp);
    store_state4<S_BF16>(m, q, mm);
    store_state4<S_BF16>(v, q, vv);
    sq = fmaf(pp.x, pp.x, sq); sq = fmaf(pp.y, pp.y, sq); sq = fmaf(pp.z, pp.z, sq); sq = fmaf(pp.w, pp.w, sq);
    if (shadow) {
      uint2 o;
      o.x = (uint32_t)f32_to_bf16_bits(pp.x) | ((uint32_t)f32_to_bf16_bits(pp.y) << 16);
      o.y = (uint32_t)f32_to_bf16_bits(pp.z) | ((uint32_t)f32_to_bf16_bits(pp.w) << 16);
      store_stream(shadow, q, o);
    }
  }
  if (row_norm) {
    const float tot = block_sum<4>(sq, red);
    if (threadIdx.x == 0) row_norm[blockIdx.x] = sqrtf(tot);
  }
}

}  // namespace sae

namespace sae {
static int adam_step_impl(bool lowp, float *p, const void *g, int g_dtype, float *m, float *v, int64_t n, double lr,
                          double beta1, double beta2, double eps, int64_t step, void *shadow_bf16,
                          float *row_norm_out, int64_t row_len, const float *row_grad_coef, void *stream) {
  SAE_REQUIRE(p && g && m && v, SAE_ERR_INVALID_ARG, "adam_step: null pointer");
  SAE_REQUIRE(g_dtype == SAE_F32 || g_dtype == SAE_BF16, SAE_ERR_INVALID_ARG, "adam_step: bad gradient dtype %d", g_dtype);
  SAE_REQUIRE(n > 0 && step >= 1, SAE_ERR_INVALID_ARG, "adam_step: n must be positive and step >= 1");
  SAE_REQUIRE((((uintptr_t)p | (uintptr_t)g | (uintptr_t)m | (uintptr_t)v) & 15) == 0, SAE_ERR_INVALID_ARG,
              "adam_step: 16-byte alignment required");
  AdamScalars a;
  // scalars are formed in double on the host, as the Python optimiser does, then narrowed once
  a.beta1 = (float)beta1; a.beta2 = (float)beta2;
  a.one_minus_beta1 = (float)(1.0 - beta1);
  a.one_minus_beta2 = (float)(1.0 - beta2);
  const double bc1 = 1.0 - pow(beta1, (double)step);
  const double bc2 = 1.0 - pow(beta2, (double)step);
  a.step_size = (float)(lr / bc1);
  a.inv_bc2_sqrt = (float)(1.0 / sqrt(bc2));
  a.bc2_sqrt = (float)sqrt(bc2);
  a.eps = (float)eps;
  hipStream_t st = (hipStream_t)stream;
  if (row_norm_out || row_grad_coef) {
    SAE_REQUIRE(row_len > 0 && row_len % 4 == 0 && n % row_len == 0 && row_len < (1LL << 31), SAE_ERR_INVALID_ARG,
                "adam_step: row_norm_out / row_grad_coef need row_len %% 4 == 0 dividing n");
    const int64_t rows = n / row_len;
    SAE_REQUIRE(rows < (1LL << 31), SAE_ERR_UNSUPPORTED, "adam_step: too many rows");
#define SAE_ADAM_DENSE_ROWS(GB, SB)                                                                                  \
  hipLaunchKernelGGL((adam_rows_kernel<GB, SB>), dim3((unsigned)rows), dim3(256), 0, st, p, g, m, v, (int)row_len, a, \
                     reinterpret_cast<uint16_t *>(shadow_bf16), row_norm_out, row_grad_coef)
    if (lowp) { if (g_dtype == SAE_BF16) SAE_ADAM_DENSE_ROWS(true, true); else SAE_ADAM_DENSE_ROWS(false, true); }
    else { if (g_dtype == SAE_BF16) SAE_ADAM_DENSE_ROWS(true, false); else SAE_ADAM_DENSE_ROWS(false, false); }
#undef SAE_ADAM_DENSE_ROWS
  } else {
    int64_t blocks = ((n >> 2) + ADAM_FLAT_CHUNK - 1) / ADAM_FLAT_CHUNK;
    if (blocks < 1) blocks = 1;
    SAE_REQUIRE(blocks < (1LL << 31), SAE_ERR_UNSUPPORTED, "adam_step: too many elements");
#define SAE_ADAM_FLAT(GB, SB)                                                                                 \
  hipLaunchKernelGGL((adam_flat_kernel<GB, SB>), dim3((unsigned)blocks), dim3(256), 0, st, p, g, m, v, n, a, \
                     reinterpret_cast<uint16_t *>(shadow_bf16))
    if (lowp) { if (g_dtype == SAE_BF16) SAE_ADAM_FLAT(true, true); else SAE_ADAM_FLAT(false, true); }
    else { if (g_dtype == SAE_BF16) SAE_ADAM_FLAT(true, false); else SAE_ADAM_FLAT(false, false); }
#undef SAE_ADAM_FLAT
  }
  return check_launch("adam_step");
}
}  // namespace sae

extern "C" int sae_adam_step(float *p, const void *g, int g_dtype, float *m, float *v, int64_t n, double lr,
                             double beta1, double beta2, double eps, int64_t step, void *shadow_bf16,
                             float *row_norm_out, int64_t row_len, const float *row_grad_coef, void *stream) {
  return sae::adam_step_impl(false, p, g, g_dtype, m, v, n, lr, beta1, beta2, eps, step, shadow_bf16, row_norm_out, row_len,
                             row_grad_coef, stream);
}

extern "C" int sae_adam_step_lowp(void *p_bf16, const void *g, int g_dtype, void *m_bf16, void *v_bf16, int64_t n, double lr,
                                  double beta1, double beta2, double eps, int64_t step, float *row_norm_out,
                                  int64_t row_len, const float *row_grad_coef, void *stream) {
  return sae::adam_step_impl(true, reinterpret_cast<float *>(p_bf16), g, g_dtype, reinterpret_cast<float *>(m_bf16),
                             reinterpret_cast<float *>(v_bf16), n, lr, beta1, beta2, eps, step, nullptr, row_norm_out,
                             row_len, row_grad_coef, stream);
}

// ---------------------------------------------------------------------------------------------
// Adam with the gradient row rebuilt on the fly from the sparse code.
//
// For the two weight matrices the gradient of feature f is a short sum,
//   g[f, :] = sum_{slot in segment f} coef[slot] * dense[token(slot), :],
// (dW_D: coef = feature activation, dense = grad_recon; dW_E^T: coef = d pre-activation, dense = x).
// One workgroup owns a feature: it forms g[f, :] in registers from the feature index (the dense
// operand rows come from L2 / Infinity Cache: 64 MB and 32 MB at the headline shape), and applies
// the Adam update to that row at once.  The dense [F, d] gradient never exists in HBM: per
// parameter the pass moves 12 B in + 12 B out (+ 2 B bf16 shadow) instead of 4 B gradient write +
// 16 B in + 12 B out (+ 2 B).  The summation order inside a segment is the feature index's
// (ascending token), the same as sae_sparse_grad_rows, so both routes give identical bits.
// ---------------------------------------------------------------------------------------------
namespace sae {

__global__ void sq_nnz_finish_kernel(const double *__restrict__ partial, int64_t F, double *acc);  // defined below

// NT threads: 256, or fewer for rows whose pieces do not fill four waves (a row of 768 elements has 192 pieces: a fourth
// wave would hold a place on its SIMD and do nothing but help staging; a wave that owns no piece adds nothing to any sum,
// so the results are the same bits)
template <bool DENSE_BF16, int U, int NT = 256>
__global__ __launch_bounds__(NT) void adam_sparse_rows_kernel(
    const int32_t *__restrict__ feat_ptr, const int32_t *__restrict__ feat_slot,
    const int32_t *__restrict__ slot_tok, const float *__restrict__ coef, const void *__restrict__ dense,
    float *__restrict__ p, float *__restrict__ m, float *__restrict__ v, int d, AdamScalars a,
    uint16_t *__restrict__ shadow, float *__restrict__ row_norm, float *__restrict__ bias_grad,
    const float *__restrict__ grad_scale, double *__restrict__ sq_nnz_partial,
    const int32_t *__restrict__ extra_map, const float *__restrict__ extra_rows, const float *__restrict__ extra_bias,
    const float *__restrict__ row_grad_coef) {
  __shared__ float red[4];
  __shared__ double red_d[8];
  __shared__ float s_coef[NT];
  __shared__ int32_t s_tok[NT];
  const int f = blockIdx.x, tid = threadIdx.x;
  const float gs = grad_scale ? grad_scale[0] : 1.f;
  const float rc = row_grad_coef ? row_grad_coef[f] : 0.f;   // the row's gradient through its L2 norm: rc * p[f, :]
  const int xo = extra_map ? extra_map[f] : -1;   // row of the dense gradient block that adds to this feature, or -1
  const int lo = feat_ptr[f], hi = feat_ptr[f + 1];
  const int n_seg = d >> 2;
  const size_t row_bytes = (size_t)d * (DENSE_BF16 ? 2 : 4);
  const char *dbase = reinterpret_cast<const char *>(dense);
  const int64_t base4 = (int64_t)f * n_seg;

  if (bias_grad && tid < 64) {
    float s = 0.f;
    for (int i = lo + tid; i < hi; i += 64) s += coef[feat_slot[i]];
    s = wave_sum(s);
    if (xo >= 0 && extra_bias) s += extra_bias[xo];
    if (tid == 0) bias_grad[f] = grad_scale ? s * gs : s;
  }

  float sq = 0.f;
  double g_sq = 0.0;
  int g_nz = 0;
  // U pieces of 4 elements per thread and pass: a row of up to 1024 U elements takes one pass (the same for every
  // thread of the workgroup, which gathers the gradient row together)
  for (int seg_base = 0; seg_base < n_seg; seg_base += NT * U) {
    const int seg0 = seg_base + tid;
    // issue the streaming reads of p, m, v first: they are the HBM traffic; the gradient operands hit cache
    float4 pp[U], mm[U], vv[U], g[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int seg = seg0 + u * NT;
      if (seg < n_seg) {
        pp[u] = load_state4<false>(p, base4 + seg);
        mm[u] = load_state4<false>(m, base4 + seg);
        vv[u] = load_state4<false>(v, base4 + seg);
      }
      g[u] = (xo >= 0 && seg < n_seg) ? reinterpret_cast<const float4 *>(extra_rows)[(int64_t)xo * n_seg + seg]
                                      : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    gather_rows_staged<DENSE_BF16, NT, U>(g, lo, hi, feat_slot, slot_tok, coef, dbase, row_bytes, seg0, n_seg, s_coef, s_tok);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int seg = seg0 + u * NT;
      if (seg < n_seg) {
        if (row_grad_coef) {   // product and sum rounded separately, as when the term is added to a stored gradient
          g[u].x = add_rn(g[u].x, mul_rn(rc, pp[u].x)); g[u].y = add_rn(g[u].y, mul_rn(rc, pp[u].y));
          g[u].z = add_rn(g[u].z, mul_rn(rc, pp[u].z)); g[u].w = add_rn(g[u].w, mul_rn(rc, pp[u].w));
        }
        if (grad_scale) {   // rounded products, as when the scaled gradient is written out before the step
          g[u].x = mul_rn(g[u].x, gs); g[u].y = mul_rn(g[u].y, gs);
          g[u].z = mul_rn(g[u].z, gs); g[u].w = mul_rn(g[u].w, gs);
        }
        if (sq_nnz_partial) {  // the same 4-element fp32 partials as sparse_rows_sq_nnz_kernel
          float s4 = g[u].x * g[u].x;
          s4 = fmaf(g[u].y, g[u].y, s4); s4 = fmaf(g[u].z, g[u].z, s4); s4 = fmaf(g[u].w, g[u].w, s4);
          g_sq += (double)s4;
          g_nz += (g[u].x != 0.f) + (g[u].y != 0.f) + (g[u].z != 0.f) + (g[u].w != 0.f);
        }
        adam_any4<false>(pp[u], g[u], mm[u], vv[u], a);
        store_state4<false>(p, base4 + seg, pp[u]);
        store_state4<false>(m, base4 + seg, mm[u]);
        store_state4<false>(v, base4 + seg, vv[u]);
        sq = fmaf(pp[u].x, pp[u].x, sq); sq = fmaf(pp[u].y, pp[u].y, sq);
        sq = fmaf(pp[u].z, pp[u].z, sq); sq = fmaf(pp[u].w, pp[u].w, sq);
        if (shadow) {
          uint2 o;
          o.x = (uint32_t)f32_to_bf16_bits(pp[u].x) | ((uint32_t)f32_to_bf16_bits(pp[u].y) << 16);
          o.y = (uint32_t)f32_to_bf16_bits(pp[u].z) | ((uint32_t)f32_to_bf16_bits(pp[u].w) << 16);
          store_stream(shadow, base4 + seg, o);
        }
      }
    }
  }
  if (row_norm) {
    const float tot = block_sum<NT / 64>(sq, red);
    if (tid == 0) row_norm[f] = sqrtf(tot);
  }
  if (sq_nnz_partial) {
    double cnt = (double)g_nz;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) { g_sq += __shfl_xor(g_sq, o, 64); cnt += __shfl_xor(cnt, o, 64); }
    const int lane = tid & 63, w = tid >> 6;
    if (lane == 0) { red_d[w] = g_sq; red_d[4 + w] = cnt; }
    __syncthreads();
    if (tid == 0) {
      double s = red_d[0], c = red_d[4];
#pragma unroll
      for (int w2 = 1; w2 < NT / 64; ++w2) { s += red_d[w2]; c += red_d[4 + w2]; }
      sq_nnz_partial[2 * (size_t)f] = s;
      sq_nnz_partial[2 * (size_t)f + 1] = c;
    }
  }
}

}  // namespace sae

namespace sae {

// The same pass in persistent form, used for bf16 p, m, v.  A row is 6 bytes per parameter there, so a workgroup
// per row keeps too few bytes in flight to fill the memory system while it waits for its index loads and gathers
// (3.3 TB/s).  Here a workgroup walks rows blockIdx.x, blockIdx.x + gridDim.x, ... in units of 256 U pieces, and
// requests the next unit's p, m, v (as they lie in memory: 6 registers per piece) before it gathers and updates
// the current one: 4.4 TB/s.  Arithmetic and summation order are those of the kernel above, so the dense route
// over rounded gradient rows gives the same bits.  For fp32 state (S_BF16 = false compiles, and passes the same
// tests) this form is slower than a workgroup per row, 2.86 against 2.51 ms at the headline shape and 6.3 against
// 4.9 ms over a cross-layer transcoder's rows of 768, whatever the grid: it is not dispatched.  Five waves per SIMD are asked for: at 98 registers (104 allocated) only four fit,
// and the pass falls from 1.46 to 1.69 ms.
template <bool DENSE_BF16, int U, bool S_BF16>
__global__ __launch_bounds__(256, 5) void adam_sparse_rows_persistent_kernel(
    const int32_t *__restrict__ feat_ptr, const int32_t *__restrict__ feat_slot,
    const int32_t *__restrict__ slot_tok, const float *__restrict__ coef, const void *__restrict__ dense,
    float *__restrict__ p, float *__restrict__ m, float *__restrict__ v, int F, int d, AdamScalars a,
    uint16_t *__restrict__ shadow, float *__restrict__ row_norm, float *__restrict__ bias_grad,
    const float *__restrict__ grad_scale, double *__restrict__ sq_nnz_partial,
    const int32_t *__restrict__ extra_map, const float *__restrict__ extra_rows, const float *__restrict__ extra_bias) {
  __shared__ float red[4];
  __shared__ double red_d[8];
  __shared__ float s_coef[256];
  __shared__ int32_t s_tok[256];
  const int tid = threadIdx.x;
  const float gs = grad_scale ? grad_scale[0] : 1.f;
  const int n_seg = d >> 2;
  const int passes = (n_seg + 256 * U - 1) / (256 * U);
  const size_t row_bytes = (size_t)d * (DENSE_BF16 ? 2 : 4);
  const char *dbase = reinterpret_cast<const char *>(dense);
  typedef typename std::conditional<S_BF16, nt_u32x2, nt_f32x4>::type raw_t;   // four elements as they lie in memory
  struct Raw { raw_t p[U], m[U], v[U]; };
  auto request = [&](Raw &r, int row, int pass) {
    const int64_t base4 = (int64_t)row * n_seg;
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int seg = pass * 256 * U + tid + u * 256;
      if (seg < n_seg) {
        r.p[u] = __builtin_nontemporal_load(reinterpret_cast<const raw_t *>(p) + base4 + seg);
        r.m[u] = __builtin_nontemporal_load(reinterpret_cast<const raw_t *>(m) + base4 + seg);
        r.v[u] = __builtin_nontemporal_load(reinterpret_cast<const raw_t *>(v) + base4 + seg);
      }
    }
  };
  auto widen = [](const raw_t &t) {
    if constexpr (S_BF16)
      return make_float4(__uint_as_float(t[0] << 16), __uint_as_float(t[0] & 0xffff0000u), __uint_as_float(t[1] << 16),
                         __uint_as_float(t[1] & 0xffff0000u));
    else
      return make_float4(t[0], t[1], t[2], t[3]);
  };
  Raw next;
  if ((int)blockIdx.x < F) request(next, blockIdx.x, 0);
  for (int f = blockIdx.x; f < F; f += gridDim.x) {
    const int lo = feat_ptr[f], hi = feat_ptr[f + 1];
    const int xo = extra_map ? extra_map[f] : -1;   // row of the dense gradient block that adds to this feature, or -1
    const int64_t base4 = (int64_t)f * n_seg;
    if (bias_grad && tid < 64) {
      float s = 0.f;
      for (int i = lo + tid; i < hi; i += 64) s += coef[feat_slot[i]];
      s = wave_sum(s);
      if (xo >= 0 && extra_bias) s += extra_bias[xo];
      if (tid == 0) bias_grad[f] = grad_scale ? s * gs : s;
    }
    float sq = 0.f;
    double g_sq = 0.0;
    int g_nz = 0;
    for (int pass = 0; pass < passes; ++pass) {
      const Raw cur = next;
      if (pass + 1 < passes) request(next, f, pass + 1);
      else if (f + (int)gridDim.x < F) request(next, f + gridDim.x, 0);
      const int seg0 = pass * 256 * U + tid;
      float4 g[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int seg = seg0 + u * 256;
        g[u] = (xo >= 0 && seg < n_seg) ? reinterpret_cast<const float4 *>(extra_rows)[(int64_t)xo * n_seg + seg]
                                        : make_float4(0.f, 0.f, 0.f, 0.f);
      }
      gather_rows_staged<DENSE_BF16, 256, U>(g, lo, hi, feat_slot, slot_tok, coef, dbase, row_bytes, seg0, n_seg, s_coef, s_tok);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int seg = seg0 + u * 256;
        if (seg < n_seg) {
          if constexpr (S_BF16) {   // the gradient is a bf16 tensor before anything reads it
            g[u].x = bf16_round(g[u].x); g[u].y = bf16_round(g[u].y); g[u].z = bf16_round(g[u].z); g[u].w = bf16_round(g[u].w);
          }
          if (grad_scale) {
            g[u].x = mul_rn(g[u].x, gs); g[u].y = mul_rn(g[u].y, gs);
            g[u].z = mul_rn(g[u].z, gs); g[u].w = mul_rn(g[u].w, gs);
          }
          if (sq_nnz_partial) {
            float s4 = g[u].x * g[u].x;
            s4 = fmaf(g[u].y, g[u].y, s4); s4 = fmaf(g[u].z, g[u].z, s4); s4 = fmaf(g[u].w, g[u].w, s4);
            g_sq += (double)s4;
            g_nz += (g[u].x != 0.f) + (g[u].y != 0.f) + (g[u].z != 0.f) + (g[u].w != 0.f);
          }
          float4 pp = widen(cur.p[u]), mm = widen(cur.m[u]), vv = widen(cur.v[u]);
          adam_any4<S_BF16>(pp, g[u], mm, vv, a);
          store_state4<S_BF16>(p, base4 + seg, pp);
          store_state4<S_BF16>(m, base4 + seg, mm);
          store_state4<S_BF16>(v, base4 + seg, vv);
          if (!S_BF16 && shadow) {
            uint2 o;
            o.x = (uint32_t)f32_to_bf16_bits(pp.x) | ((uint32_t)f32_to_bf16_bits(pp.y) << 16);
            o.y = (uint32_t)f32_to_bf16_bits(pp.z) | ((uint32_t)f32_to_bf16_bits(pp.w) << 16);
            store_stream(shadow, base4 + seg, o);
          }
          sq = fmaf(pp.x, pp.x, sq); sq = fmaf(pp.y, pp.y, sq);
          sq = fmaf(pp.z, pp.z, sq); sq = fmaf(pp.w, pp.w, sq);
        }
      }
    }
    if (row_norm) {
      const float tot = block_sum<4>(sq, red);
      if (tid == 0) row_norm[f] = sqrtf(tot);
    }
    if (sq_nnz_partial) {
      double cnt = (double)g_nz;
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) { g_sq += __shfl_xor(g_sq, o, 64); cnt += __shfl_xor(cnt, o, 64); }
      const int lane = tid & 63, w = tid >> 6;
      __syncthreads();   // red_d of the previous row has been read
      if (lane == 0) { red_d[w] = g_sq; red_d[4 + w] = cnt; }
      __syncthreads();
      if (tid == 0) {
        sq_nnz_partial[2 * (size_t)f] = red_d[0] + red_d[1] + red_d[2] + red_d[3];
        sq_nnz_partial[2 * (size_t)f + 1] = red_d[4] + red_d[5] + red_d[6] + red_d[7];
      }
    }
  }
}

}  // namespace sae

namespace sae {
static int adam_step_sparse_rows_impl(bool lowp, const int32_t *feat_ptr, const int32_t *feat_slot, const int32_t *slot_tok,
                                      const float *coef, const void *dense, int dense_dtype, float *p, float *m,
                                      float *v, int64_t F, int64_t d, double lr, double beta1, double beta2,
                                      double eps, int64_t step, void *shadow_bf16, float *row_norm_out,
                                      float *bias_grad_out, const float *grad_scale, double *grad_sq_nnz_acc,
                                      void *workspace, int64_t workspace_bytes, const int32_t *extra_map,
                                      const float *extra_rows, const float *extra_bias, const float *row_grad_coef,
                                      void *stream) {
  SAE_REQUIRE(feat_ptr && feat_slot && slot_tok && coef && dense && p && m && v, SAE_ERR_INVALID_ARG,
              "adam_step_sparse_rows: null pointer");
  SAE_REQUIRE(!(lowp && row_grad_coef), SAE_ERR_UNSUPPORTED, "adam_step_sparse_rows_lowp: no row_grad_coef for bf16 state");
  SAE_REQUIRE((extra_map == nullptr) == (extra_rows == nullptr) && (((uintptr_t)extra_rows) & 15) == 0, SAE_ERR_INVALID_ARG,
              "adam_step_sparse_rows: extra_map and extra_rows go together (extra_rows 16-byte aligned)");
  SAE_REQUIRE(!grad_sq_nnz_acc || (workspace && workspace_bytes >= 16 * F && ((uintptr_t)workspace & 15) == 0),
              SAE_ERR_WORKSPACE, "adam_step_sparse_rows: the gradient sums need an aligned workspace of %lld bytes",
              (long long)(16 * F));
  SAE_REQUIRE(F > 0 && d > 0 && step >= 1, SAE_ERR_INVALID_ARG, "adam_step_sparse_rows: bad sizes / step");
  SAE_REQUIRE(dense_dtype == SAE_F32 || dense_dtype == SAE_BF16, SAE_ERR_INVALID_ARG, "adam_step_sparse_rows: bad dtype %d", dense_dtype);
  SAE_REQUIRE(d % 4 == 0 && F < (1LL << 31) && d < (1LL << 31), SAE_ERR_UNSUPPORTED,
              "adam_step_sparse_rows: d_model=%lld must be a multiple of 4", (long long)d);
  SAE_REQUIRE((((uintptr_t)p | (uintptr_t)m | (uintptr_t)v | (uintptr_t)dense) & 15) == 0, SAE_ERR_INVALID_ARG,
              "adam_step_sparse_rows: 16-byte alignment required");
  AdamScalars a;
  a.beta1 = (float)beta1; a.beta2 = (float)beta2;
  a.one_minus_beta1 = (float)(1.0 - beta1);
  a.one_minus_beta2 = (float)(1.0 - beta2);
  a.step_size = (float)(lr / (1.0 - pow(beta1, (double)step)));
  a.inv_bc2_sqrt = (float)(1.0 / sqrt(1.0 - pow(beta2, (double)step)));
  a.bc2_sqrt = (float)sqrt(1.0 - pow(beta2, (double)step));
  a.eps = (float)eps;
  hipStream_t st = (hipStream_t)stream;
  double *partial = grad_sq_nnz_acc ? reinterpret_cast<double *>(workspace) : nullptr;
  {
#define SAE_ADAM_ROWS(BF, UU)                                                                                              \
  hipLaunchKernelGGL((adam_sparse_rows_kernel<BF, UU>), dim3((unsigned)F), dim3(256), 0, st, feat_ptr, feat_slot, slot_tok, \
                     coef, dense, p, m, v, (int)d, a, reinterpret_cast<uint16_t *>(shadow_bf16), row_norm_out,            \
                     bias_grad_out, grad_scale, partial, extra_map, extra_rows, extra_bias, row_grad_coef)
    // pieces of 4 elements per thread: short rows keep fewer registers, so more rows are in flight per CU
    const int u = d <= 1024 ? 1 : (d <= 2048 ? 2 : 4);
    if (lowp) {
      SAE_REQUIRE(F < (1LL << 31) - (1 << 20), SAE_ERR_UNSUPPORTED, "adam_step_sparse_rows_lowp: F too large");
      // persistent form: at most two pieces per thread and unit (95-102 registers: five workgroups per CU), and two
      // rounds of resident workgroups -- a grid that is not a multiple of what is resident leaves a tail
      // (1536 workgroups on 256 CUs: 1.84 ms against 1.47 ms with 1280 or 2560)
      int dev = 0, cus = 256;
      if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
      const int64_t gmax = (int64_t)(cus > 0 ? cus : 256) * (d <= 1024 ? 14 : 10);   // 7 resident per CU at 66 registers
      const unsigned grid = (unsigned)(F < gmax ? F : gmax);
#define SAE_ADAM_ROWS_LOWP(BF, UU)                                                                                      \
  hipLaunchKernelGGL((adam_sparse_rows_persistent_kernel<BF, UU, true>), dim3(grid), dim3(256), 0, st, feat_ptr, feat_slot, \
                     slot_tok, coef, dense, p, m, v, (int)F, (int)d, a, nullptr, row_norm_out, bias_grad_out, grad_scale,  \
                     partial, extra_map, extra_rows, extra_bias)
      if (dense_dtype == SAE_BF16) {
        if (d <= 1024) SAE_ADAM_ROWS_LOWP(true, 1); else SAE_ADAM_ROWS_LOWP(true, 2);
      } else {
        if (d <= 1024) SAE_ADAM_ROWS_LOWP(false, 1); else SAE_ADAM_ROWS_LOWP(false, 2);
      }
#undef SAE_ADAM_ROWS_LOWP
    } else if (u == 1 && d <= 768 && d > 512) {   // 129-192 pieces: three waves
#define SAE_ADAM_ROWS_192(BF)                                                                                              \
  hipLaunchKernelGGL((adam_sparse_rows_kernel<BF, 1, 192>), dim3((unsigned)F), dim3(192), 0, st, feat_ptr, feat_slot, slot_tok, \
                     coef, dense, p, m, v, (int)d, a, reinterpret_cast<uint16_t *>(shadow_bf16), row_norm_out,            \
                     bias_grad_out, grad_scale, partial, extra_map, extra_rows, extra_bias, row_grad_coef)
      if (dense_dtype == SAE_BF16) SAE_ADAM_ROWS_192(true); else SAE_ADAM_ROWS_192(false);
#undef SAE_ADAM_ROWS_192
    } else if (dense_dtype == SAE_BF16) {
      if (u == 1) SAE_ADAM_ROWS(true, 1); else if (u == 2) SAE_ADAM_ROWS(true, 2); else SAE_ADAM_ROWS(true, 4);
    } else {
      if (u == 1) SAE_ADAM_ROWS(false, 1); else if (u == 2) SAE_ADAM_ROWS(false, 2); else SAE_ADAM_ROWS(false, 4);
    }
#undef SAE_ADAM_ROWS
  }
  if (partial) hipLaunchKernelGGL(sq_nnz_finish_kernel, dim3(1), dim3(1024), 0, st, partial, F, grad_sq_nnz_acc);
  return check_launch("adam_step_sparse_rows");
}
}  // namespace sae

extern "C" int sae_adam_step_sparse_rows(const int32_t *feat_ptr, const int32_t *feat_slot, const int32_t *slot_tok,
                                         const float *coef, const void *dense, int dense_dtype, float *p, float *m,
                                         float *v, int64_t F, int64_t d, double lr, double beta1, double beta2,
                                         double eps, int64_t step, void *shadow_bf16, float *row_norm_out,
                                         float *bias_grad_out, const float *grad_scale, double *grad_sq_nnz_acc,
                                         void *workspace, int64_t workspace_bytes, const int32_t *extra_map,
                                         const float *extra_rows, const float *extra_bias, const float *row_grad_coef,
                                         void *stream) {
  return sae::adam_step_sparse_rows_impl(false, feat_ptr, feat_slot, slot_tok, coef, dense, dense_dtype, p, m, v, F, d, lr,
                                         beta1, beta2, eps, step, shadow_bf16, row_norm_out, bias_grad_out, grad_scale,
                                         grad_sq_nnz_acc, workspace, workspace_bytes, extra_map, extra_rows, extra_bias,
                                         row_grad_coef, stream);
}

extern "C" int sae_adam_step_sparse_rows_lowp(const int32_t *feat_ptr, const int32_t *feat_slot, const int32_t *slot_tok,
                                              const float *coef, const void *dense, int dense_dtype, void *p_bf16,
                                              void *m_bf16, void *v_bf16, int64_t F, int64_t d, double lr, double beta1,
                                              double beta2, double eps, int64_t step, float *row_norm_out,
                                              float *bias_grad_out, const float *grad_scale, double *grad_sq_nnz_acc,
                                              void *workspace, int64_t workspace_bytes, const int32_t *extra_map,
                                              const float *extra_rows, const float *extra_bias, void *stream) {
  return sae::adam_step_sparse_rows_impl(true, feat_ptr, feat_slot, slot_tok, coef, dense, dense_dtype,
                                         reinterpret_cast<float *>(p_bf16), reinterpret_cast<float *>(m_bf16),
                                         reinterpret_cast<float *>(v_bf16), F, d, lr, beta1, beta2, eps, step, nullptr,
                                         row_norm_out, bias_grad_out, grad_scale, grad_sq_nnz_acc, workspace,
                                         workspace_bytes, extra_map, extra_rows, extra_bias, nullptr, stream);
}

// ---------------------------------------------------------------------------------------------
// SparseAdam (masked-momentum Adam) and the gradient-norm diagnostic.
// ---------------------------------------------------------------------------------------------
namespace sae {

__global__ __launch_bounds__(256) void any_nonzero_kernel(const float *__restrict__ g, int64_t n, int32_t *flag) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  int hit = 0;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) hit |= g[i] != 0.f;
  hit = wave_sum_i(hit);
  if ((threadIdx.x & 63) == 0 && hit) atomicOr(flag, 1);
}

// moments decay everywhere; gradient contributions and the parameter move only where g != 0;
// nothing at all happens (and the step counter stays) when the whole gradient is zero
__global__ __launch_bounds__(256) void sparse_adam_kernel(float *__restrict__ p, const float *__restrict__ g,
                                                          float *__restrict__ m, float *__restrict__ v, int64_t n,
                                                          double lr, double beta1, double beta2, float eps,
                                                          const float *__restrict__ step_state,
                                                          const int32_t *__restrict__ flag, uint16_t *__restrict__ shadow) {
  if (*flag == 0) return;
  const double t = (double)step_state[0] + 1.0;
  const float step_size = (float)(lr * sqrt(1.0 - pow(beta2, t)) / (1.0 - pow(beta1, t)));
  const float b1 = (float)beta1, b2 = (float)beta2, omb1 = (float)(1.0 - beta1), omb2 = (float)(1.0 - beta2);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const float gg = g[i];
    float mm = m[i] * b1, vv = v[i] * b2, pp = p[i];
    if (gg != 0.f) {
      mm = mm + omb1 * gg;
      vv = vv + omb2 * gg * gg;
      pp = pp - step_size * mm / (sqrtf(vv) + eps);
      p[i] = pp;
    }
    m[i] = mm;
    v[i] = vv;
    if (shadow) shadow[i] = f32_to_bf16_bits(pp);
  }
}

__global__ void sparse_adam_advance_kernel(float *step_state, const int32_t *flag) {
  if (threadIdx.x == 0 && blockIdx.x == 0 && *flag) step_state[0] += 1.f;
}

// acc[0] += sum g^2 (fp64), acc[1] += #(g != 0) (fp64 count)
__global__ __launch_bounds__(256) void grad_sq_nnz_kernel(const float *__restrict__ g, int64_t n, double *acc) {
  __shared__ double red[8];
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  double sq = 0.0;
  int nz = 0;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const float x = g[i];
    sq += (double)x * (double)x;
    nz += x != 0.f;
  }
  double cnt = (double)nz;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) { sq += __shfl_xor(sq, o, 64); cnt += __shfl_xor(cnt, o, 64); }
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  if (lane == 0) { red[w] = sq; red[4 + w] = cnt; }
  __syncthreads();
  if (threadIdx.x == 0) {
    atomicAdd(&acc[0], red[0] + red[1] + red[2] + red[3]);
    atomicAdd(&acc[1], red[4] + red[5] + red[6] + red[7]);
  }
}

}  // namespace sae

extern "C" int sae_sparse_adam_step(float *p, const float *g, float *m, float *v, int64_t n, double lr, double beta1,
                                    double beta2, double eps, float *step_state, int32_t *flag_workspace,
                                    void *shadow_bf16, void *stream) {
  using namespace sae;
  SAE_REQUIRE(p && g && m && v && step_state && flag_workspace, SAE_ERR_INVALID_ARG, "sparse_adam_step: null pointer");
  SAE_REQUIRE(n > 0, SAE_ERR_INVALID_ARG, "sparse_adam_step: n must be positive");
  hipStream_t st = (hipStream_t)stream;
  int rc = zero_fill(flag_workspace, 4, st);
  if (rc) return rc;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 32768) blocks = 32768;
  hipLaunchKernelGGL(any_nonzero_kernel, dim3((unsigned)blocks), dim3(256), 0, st, g, n, flag_workspace);
  hipLaunchKernelGGL(sparse_adam_kernel, dim3((unsigned)blocks), dim3(256), 0, st, p, g, m, v, n, lr, beta1, beta2,
                     (float)eps, step_state, flag_workspace, reinterpret_cast<uint16_t *>(shadow_bf16));
  hipLaunchKernelGGL(sparse_adam_advance_kernel, dim3(1), dim3(64), 0, st, step_state, flag_workspace);
  return check_launch("sparse_adam_step");
}

namespace sae {

// One workgroup per feature: rebuilds the feature's gradient row exactly as adam_sparse_rows_kernel does
// (same accumulation order, so the same bits) and reduces sum g^2 and #(g != 0) into partial[2 f], partial[2 f + 1].
template <bool DENSE_BF16>
__global__ __launch_bounds__(256) void sparse_rows_sq_nnz_kernel(
    const int32_t *__restrict__ feat_ptr, const int32_t *__restrict__ feat_slot, const int32_t *__restrict__ slot_tok,
    const float *__restrict__ coef, const void *__restrict__ dense, int d, double *__restrict__ partial,
    float *__restrict__ bias_grad, const int32_t *__restrict__ extra_map, const float *__restrict__ extra_rows,
    const float *__restrict__ extra_bias) {
  __shared__ double red[8];
  const int f = blockIdx.x, tid = threadIdx.x;
  const int lo = feat_ptr[f], hi = feat_ptr[f + 1];
  const int xo = extra_map ? extra_map[f] : -1;
  if (bias_grad && tid < 64) {
    float s = 0.f;
    for (int i = lo + tid; i < hi; i += 64) s += coef[feat_slot[i]];
    s = wave_sum(s);
    if (xo >= 0 && extra_bias) s += extra_bias[xo];
    if (tid == 0) bias_grad[f] = s;
  }
  if (lo == hi && xo < 0) {  // no token used this feature: the row gradient is exactly zero
    if (tid == 0) { partial[2 * (size_t)f] = 0.0; partial[2 * (size_t)f + 1] = 0.0; }
    return;
  }
  const int n_seg = d >> 2;
  const size_t row_bytes = (size_t)d * (DENSE_BF16 ? 2 : 4);
  const char *dbase = reinterpret_cast<const char *>(dense);
  double sq = 0.0;
  int nz = 0;
  for (int seg0 = tid; seg0 < n_seg; seg0 += 256 * 4) {
    float4 g[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int seg = seg0 + u * 256;
      g[u] = (xo >= 0 && seg < n_seg) ? reinterpret_cast<const float4 *>(extra_rows)[(int64_t)xo * n_seg + seg]
                                      : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    gather_rows_fma<DENSE_BF16>(g, lo, hi, feat_slot, slot_tok, coef, dbase, row_bytes, seg0, n_seg);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      float s4 = g[u].x * g[u].x;   // a 4-element fp32 partial keeps the fp64 adds off the critical path
      s4 = fmaf(g[u].y, g[u].y, s4); s4 = fmaf(g[u].z, g[u].z, s4); s4 = fmaf(g[u].w, g[u].w, s4);
      sq += (double)s4;
      nz += (g[u].x != 0.f) + (g[u].y != 0.f) + (g[u].z != 0.f) + (g[u].w != 0.f);
    }
  }
  double cnt = (double)nz;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) { sq += __shfl_xor(sq, o, 64); cnt += __shfl_xor(cnt, o, 64); }
  const int lane = tid & 63, w = tid >> 6;
  if (lane == 0) { red[w] = sq; red[4 + w] = cnt; }
  __syncthreads();
  if (tid == 0) {
    partial[2 * (size_t)f] = red[0] + red[1] + red[2] + red[3];
    partial[2 * (size_t)f + 1] = red[4] + red[5] + red[6] + red[7];
  }
}

// acc[0] += sum of partial[2 f], acc[1] += sum of partial[2 f + 1], in a fixed order (one workgroup)
__global__ __launch_bounds__(1024) void sq_nnz_finish_kernel(const double *__restrict__ partial, int64_t F, double *acc) {
  __shared__ double red[32];
  double sq = 0.0, cnt = 0.0;
  // four independent 16-byte loads in flight per thread; the order of the additions is fixed by the indexing
  typedef __attribute__((ext_vector_type(2))) double f64x2;
  const f64x2 *pairs = reinterpret_cast<const f64x2 *>(partial);
  int64_t f = threadIdx.x;
  for (; f + 3 * 1024 < F; f += 4 * 1024) {
    const f64x2 a = pairs[f], b = pairs[f + 1024], c = pairs[f + 2048], d = pairs[f + 3072];
    sq += (a[0] + b[0]) + (c[0] + d[0]);
    cnt += (a[1] + b[1]) + (c[1] + d[1]);
  }
  for (; f < F; f += 1024) { const f64x2 a = pairs[f]; sq += a[0]; cnt += a[1]; }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) { sq += __shfl_xor(sq, o, 64); cnt += __shfl_xor(cnt, o, 64); }
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  if (lane == 0) { red[w] = sq; red[16 + w] = cnt; }
  __syncthreads();
  if (threadIdx.x == 0) {
    double a = 0.0, b = 0.0;
    for (int i = 0; i < 16; ++i) { a += red[i]; b += red[16 + i]; }
    acc[0] += a;
    acc[1] += b;
  }
}

}  // namespace sae

extern "C" int64_t sae_sparse_rows_grad_sq_nnz_workspace_bytes(int64_t F) { return F > 0 ? 16 * F : 0; }

extern "C" int sae_sparse_rows_grad_sq_nnz(const int32_t *feat_ptr, const int32_t *feat_slot, const int32_t *slot_tok,
                                           const float *coef, const void *dense, int dense_dtype, int64_t F, int64_t d,
                                           double *acc, float *bias_grad_out, void *workspace, int64_t workspace_bytes,
                                           const int32_t *extra_map, const float *extra_rows, const float *extra_bias,
                                           void *stream) {
  using namespace sae;
  SAE_REQUIRE(feat_ptr && feat_slot && slot_tok && coef && dense && acc && workspace, SAE_ERR_INVALID_ARG,
              "sparse_rows_grad_sq_nnz: null pointer");
  SAE_REQUIRE(F > 0 && d > 0, SAE_ERR_INVALID_ARG, "sparse_rows_grad_sq_nnz: bad sizes");
  SAE_REQUIRE(dense_dtype == SAE_F32 || dense_dtype == SAE_BF16, SAE_ERR_INVALID_ARG, "sparse_rows_grad_sq_nnz: bad dtype %d", dense_dtype);
  SAE_REQUIRE(d % 4 == 0 && F < (1LL << 31) && d < (1LL << 31), SAE_ERR_UNSUPPORTED,
              "sparse_rows_grad_sq_nnz: d_model=%lld must be a multiple of 4", (long long)d);
  SAE_REQUIRE((((uintptr_t)dense | (uintptr_t)workspace) & 15) == 0, SAE_ERR_INVALID_ARG,
              "sparse_rows_grad_sq_nnz: 16-byte alignment required");
  SAE_REQUIRE(workspace_bytes >= 16 * F, SAE_ERR_INVALID_ARG, "sparse_rows_grad_sq_nnz: workspace of %lld bytes, %lld needed",
              (long long)workspace_bytes, (long long)(16 * F));
  hipStream_t st = (hipStream_t)stream;
  double *partial = reinterpret_cast<double *>(workspace);
  if (dense_dtype == SAE_BF16)
    hipLaunchKernelGGL(sparse_rows_sq_nnz_kernel<true>, dim3((unsigned)F), dim3(256), 0, st, feat_ptr, feat_slot, slot_tok, coef,
                       dense, (int)d, partial, bias_grad_out, extra_map, extra_rows, extra_bias);
  else
    hipLaunchKernelGGL(sparse_rows_sq_nnz_kernel<false>, dim3((unsigned)F), dim3(256), 0, st, feat_ptr, feat_slot, slot_tok, coef,
                       dense, (int)d, partial, bias_grad_out, extra_map, extra_rows, extra_bias);
  hipLaunchKernelGGL(sq_nnz_finish_kernel, dim3(1), dim3(1024), 0, st, partial, F, acc);
  return check_launch("sparse_rows_grad_sq_nnz");
}

extern "C" int sae_grad_sq_nnz(const float *g, int64_t n, double *acc, void *stream) {
  using namespace sae;
  SAE_REQUIRE(g && acc, SAE_ERR_INVALID_ARG, "grad_sq_nnz: null pointer");
  SAE_REQUIRE(n > 0, SAE_ERR_INVALID_ARG, "grad_sq_nnz: n must be positive");
  int64_t blocks = (n + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  hipLaunchKernelGGL(grad_sq_nnz_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, g, n, acc);
  return check_launch("grad_sq_nnz");
}
