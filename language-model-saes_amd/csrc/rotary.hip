// Rotary positional embedding around the attention kernels (gfx950): Lorsa rotates its queries and keys between the
// projection and the scores (models/lorsa.py:821-824, 864-904).
//
// The reference rotates x [b, s, h, dq] per head: the first `rotary_dim` elements pair up (adjacent elements, or element j
// with j + rotary_dim / 2) and
//     y[j] = x[j] * cos[pos, j] + flip(x)[j] * sin[pos, j],   flip(x)[a] = -x[b], flip(x)[b] = x[a] for a pair (a, b),
// elements from rotary_dim on pass through; pos is the position inside the sequence.  Under bf16 autocast x is
// `bf16 product + fp32 bias`, an fp32 tensor, the rotation runs in fp32 and the attention rounds its operands to bf16.
//
//   forward   out = bf16(rotate(float(bf16(acc)) + bias)) from the projection's fp32 accumulators: the bias and the one
//             rounding of the attention's operand happen here, so the rotation sees the values the reference's sees
//   backward  the attention's backward leaves d q^T, d k^T [h dq, T] (bf16, one row per head element); the transpose of
//             the rotation is applied in place, rows in pairs, so the buffer stays the operand of the weight-gradient
//             product:  dx[a] = dy[a] cos[a] + dy[b] sin[b],  dx[b] = dy[b] cos[b] - dy[a] sin[a]
// Each product is rounded before the sum, as the framework's element-wise kernels leave it.
#include "common.h"

namespace sae {

// one thread: 8 consecutive elements of one head of one token
__global__ __launch_bounds__(256) void rotary_fwd_kernel(const float *__restrict__ acc, const float *__restrict__ bias,
                                                         const float *__restrict__ cos_tab, const float *__restrict__ sin_tab,
                                                         int64_t T, int seq, int width, int d_head, int rotary_dim,
                                                         int adjacent, uint16_t *__restrict__ out) {
  const int chunks = width >> 3;
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= T * chunks) return;
  const int64_t t = gid / chunks;
  const int c0 = (int)(gid - t * chunks) * 8;   // first column of this thread's chunk
  const int j0 = c0 % d_head;                   // and its place inside the head
  const int pos = (int)(t % seq);
  auto load8v = [&](int col, float (&v)[8]) {
    const float4 a = *reinterpret_cast<const float4 *>(acc + t * width + col);
    const float4 b = *reinterpret_cast<const float4 *>(acc + t * width + col + 4);
    const float raw[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = add_rn(bf16_round(raw[e]), bias ? bias[col + e] : 0.f);
  };
  float x[8], y[8];
  load8v(c0, x);
  if (j0 >= rotary_dim) {
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = x[e];
  } else {
    // rotary_dim is a multiple of 16 here, so a chunk lies wholly inside the rotated part
    float cs[8], sn[8], flip[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      cs[e] = cos_tab[(int64_t)pos * rotary_dim + j0 + e];
      sn[e] = sin_tab[(int64_t)pos * rotary_dim + j0 + e];
    }
    if (adjacent) {
#pragma unroll
      for (int e = 0; e < 8; e += 2) { flip[e] = -x[e + 1]; flip[e + 1] = x[e]; }
    } else {
      const int n = rotary_dim >> 1;
      float partner[8];
      const bool first = j0 < n;
      load8v(first ? c0 + n : c0 - n, partner);
#pragma unroll
      for (int e = 0; e < 8; ++e) flip[e] = first ? -partner[e] : partner[e];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = add_rn(mul_rn(x[e], cs[e]), mul_rn(flip[e], sn[e]));
  }
  uint4 o;
  o.x = pack_bf16x2(y[0], y[1]); o.y = pack_bf16x2(y[2], y[3]); o.z = pack_bf16x2(y[4], y[5]); o.w = pack_bf16x2(y[6], y[7]);
  *reinterpret_cast<uint4 *>(out + t * width + c0) = o;
}

// one thread: one pair of rows (a, b) of one head, 8 consecutive tokens; cos_t / sin_t are [rotary_dim, n_ctx]
__global__ __launch_bounds__(256) void rotary_bwd_t_kernel(uint16_t *__restrict__ g, int64_t T, const float *__restrict__ cos_t,
                                                           const float *__restrict__ sin_t, int n_ctx, int seq, int n_heads,
                                                           int d_head, int rotary_dim, int adjacent) {
  const int half = rotary_dim >> 1;
  const int64_t tchunks = T >> 3;
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (gid >= (int64_t)n_heads * half * tchunks) return;
  const int64_t tc = gid % tchunks;
  const int pr = (int)((gid / tchunks) % half), hh = (int)(gid / (tchunks * half));
  const int ja = adjacent ? 2 * pr : pr, jb = adjacent ? 2 * pr + 1 : pr + half;
  const int64_t t0 = tc * 8;
  const int pos0 = (int)(t0 % seq);   // seq is a multiple of 8: the eight tokens share a sequence
  uint16_t *ra = g + ((int64_t)hh * d_head + ja) * T + t0, *rb = g + ((int64_t)hh * d_head + jb) * T + t0;
  const uint4 va = *reinterpret_cast<const uint4 *>(ra), vb = *reinterpret_cast<const uint4 *>(rb);
  const uint32_t wa[4] = {va.x, va.y, va.z, va.w}, wb[4] = {vb.x, vb.y, vb.z, vb.w};
  float da[8], db[8], oa[8], ob[8];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    da[2 * q] = __uint_as_float(wa[q] << 16); da[2 * q + 1] = __uint_as_float(wa[q] & 0xffff0000u);
    db[2 * q] = __uint_as_float(wb[q] << 16); db[2 * q + 1] = __uint_as_float(wb[q] & 0xffff0000u);
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float ca = cos_t[(int64_t)ja * n_ctx + pos0 + e], sa = sin_t[(int64_t)ja * n_ctx + pos0 + e];
    const float cb = cos_t[(int64_t)jb * n_ctx + pos0 + e], sb = sin_t[(int64_t)jb * n_ctx + pos0 + e];
    oa[e] = add_rn(mul_rn(da[e], ca), mul_rn(db[e], sb));
    ob[e] = sub_rn(mul_rn(db[e], cb), mul_rn(da[e], sa));
  }
  uint4 pa, pb;
  pa.x = pack_bf16x2(oa[0], oa[1]); pa.y = pack_bf16x2(oa[2], oa[3]); pa.z = pack_bf16x2(oa[4], oa[5]); pa.w = pack_bf16x2(oa[6], oa[7]);
  pb.x = pack_bf16x2(ob[0], ob[1]); pb.y = pack_bf16x2(ob[2], ob[3]); pb.z = pack_bf16x2(ob[4], ob[5]); pb.w = pack_bf16x2(ob[6], ob[7]);
  *reinterpret_cast<uint4 *>(ra) = pa;
  *reinterpret_cast<uint4 *>(rb) = pb;
}

static int check_rotary(const char *what, int64_t T, int64_t seq, int64_t n_heads, int64_t d_head, int64_t rotary_dim,
                        int64_t n_ctx) {
  SAE_REQUIRE(T > 0 && seq > 0 && T % seq == 0 && seq % 8 == 0, SAE_ERR_INVALID_ARG,
              "%s: T=%lld must be a multiple of seq=%lld, seq a multiple of 8", what, (long long)T, (long long)seq);
  SAE_REQUIRE(n_heads > 0 && d_head > 0 && d_head % 8 == 0 && n_heads * d_head < (1LL << 24), SAE_ERR_INVALID_ARG,
              "%s: bad head shape %lld x %lld", what, (long long)n_heads, (long long)d_head);
  SAE_REQUIRE(rotary_dim > 0 && rotary_dim <= d_head && rotary_dim % 16 == 0, SAE_ERR_UNSUPPORTED,
              "%s: rotary_dim=%lld must be a multiple of 16, at most d_head=%lld", what, (long long)rotary_dim, (long long)d_head);
  SAE_REQUIRE(seq <= n_ctx, SAE_ERR_INVALID_ARG, "%s: the tables hold %lld positions, the sequences %lld", what,
              (long long)n_ctx, (long long)seq);
  SAE_REQUIRE(T * n_heads * d_head < (1LL << 40), SAE_ERR_UNSUPPORTED, "%s: too large", what);
  return SAE_OK;
}

}  // namespace sae

extern "C" int sae_rotary_fwd(const float *acc, const float *bias, const float *cos_tab, const float *sin_tab, int64_t n_ctx,
                              int64_t T, int64_t seq, int64_t n_heads, int64_t d_head, int64_t rotary_dim, int adjacent_pairs,
                              void *out_bf16, void *stream) {
  using namespace sae;
  SAE_REQUIRE(acc && cos_tab && sin_tab && out_bf16, SAE_ERR_INVALID_ARG, "rotary_fwd: null pointer");
  SAE_REQUIRE((((uintptr_t)acc | (uintptr_t)out_bf16) & 15) == 0, SAE_ERR_INVALID_ARG, "rotary_fwd: 16-byte alignment required");
  const int rc = check_rotary("rotary_fwd", T, seq, n_heads, d_head, rotary_dim, n_ctx);
  if (rc) return rc;
  const int64_t width = n_heads * d_head, n = T * (width / 8);
  hipLaunchKernelGGL(rotary_fwd_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, acc, bias, cos_tab,
                     sin_tab, T, (int)seq, (int)width, (int)d_head, (int)rotary_dim, adjacent_pairs ? 1 : 0,
                     reinterpret_cast<uint16_t *>(out_bf16));
  return check_launch("rotary_fwd");
}

extern "C" int sae_rotary_bwd_t(void *grad_t_bf16, const float *cos_t, const float *sin_t, int64_t n_ctx, int64_t T, int64_t seq,
                                int64_t n_heads, int64_t d_head, int64_t rotary_dim, int adjacent_pairs, void *stream) {
  using namespace sae;
  SAE_REQUIRE(grad_t_bf16 && cos_t && sin_t, SAE_ERR_INVALID_ARG, "rotary_bwd_t: null pointer");
  SAE_REQUIRE((((uintptr_t)grad_t_bf16) & 15) == 0, SAE_ERR_INVALID_ARG, "rotary_bwd_t: 16-byte alignment required");
  const int rc = check_rotary("rotary_bwd_t", T, seq, n_heads, d_head, rotary_dim, n_ctx);
  if (rc) return rc;
  const int64_t n = n_heads * (rotary_dim / 2) * (T / 8);
  hipLaunchKernelGGL(rotary_bwd_t_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     reinterpret_cast<uint16_t *>(grad_t_bf16), T, cos_t, sin_t, (int)n_ctx, (int)seq, (int)n_heads, (int)d_head,
                     (int)rotary_dim, adjacent_pairs ? 1 : 0);
  return check_launch("rotary_bwd_t");
}
