// Shared helpers for the gfx950 kernels of libsae_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include <type_traits>

#include "../../include/sae_hip.h"

namespace sae {

// ---- error reporting ----------------------------------------------------------------
char *error_buffer();            // thread-local, 512 bytes (defined in capi.hip)
int fail(int code, const char *fmt, ...);

#define SAE_REQUIRE(cond, code, ...)                 \
  do {                                               \
    if (!(cond)) return ::sae::fail((code), __VA_ARGS__); \
  } while (0)

inline int check_launch(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(SAE_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return SAE_OK;
}

// Clears `bytes` bytes (a multiple of 4) with a fill kernel; safe under HIP graph capture,
// where a memset node is not.  Defined in elementwise.hip.
int zero_fill(void *p, size_t bytes, hipStream_t st);

// ---- bf16 <-> fp32 (bit level, round-to-nearest-even like torch) ---------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);  // quiet NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float round_to_bf16(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

// Round-to-nearest-even to bf16 precision through the packed hardware conversion (two values per instruction).
typedef __attribute__((ext_vector_type(2))) float cvt_f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 cvt_bf16x2;
__device__ __forceinline__ void bf16_round2(float &x, float &y) {
  const cvt_f32x2 in = {x, y};
  const uint32_t packed = __builtin_bit_cast(uint32_t, __builtin_convertvector(in, cvt_bf16x2));
  x = __uint_as_float(packed << 16);
  y = __uint_as_float(packed & 0xffff0000u);
}
// two fp32 values rounded to bf16 (round-to-nearest-even) and packed, `lo` in the low half
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const cvt_f32x2 in = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(in, cvt_bf16x2));
}
__device__ __forceinline__ float bf16_round(float x) {
  float y = x;
  bf16_round2(x, y);
  return x;
}

// ---- single operations that stay single ----------------------------------------------------
// The compiler may fuse a product with a following sum into one fused multiply-add (and HIP's __fmul_rn /
// __fadd_rn are plain operators, so they do not prevent it).  Where a result has to have the bits of two
// separately rounded operations (kernels that promise the same bits as another route, or as the framework's
// element-wise kernels), the operations go through these: an operation compiled with contraction off is never
// fused, also after inlining.
__device__ __forceinline__ float mul_rn(float a, float b) {
#pragma clang fp contract(off)
  return a * b;
}
__device__ __forceinline__ float add_rn(float a, float b) {
#pragma clang fp contract(off)
  return a + b;
}
__device__ __forceinline__ float sub_rn(float a, float b) {
#pragma clang fp contract(off)
  return a - b;
}

// ---- wave (64 lanes) and block reductions ---------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Ordering key of one pre-activation in the TopK selects: the bit pattern of h1 = (pre + b_enc) * scale when h1 > 0 and
// 0 otherwise (for positive floats unsigned-integer order equals float order; non-positive entries are never kept).
// One definition for the select kernels and for the GEMM epilogue that emits per-granule maxima of these keys.
__device__ __forceinline__ uint32_t select_key_plain(float pre, float b, float s) {
  const float h1 = (pre + b) * s;
  return h1 > 0.f ? __float_as_uint(h1) : 0u;
}

__device__ __forceinline__ int wave_sum_i(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Sum over a block of NW waves; every thread gets the result.  `red` holds >= NW floats.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float *red) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) red[w] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NW; ++i) t += red[i];
  return t;
}

// Streaming (non-temporal) 16- and 8-byte accesses for data that is touched once per pass:
// measured +7 % on the 26 B/parameter Adam stream (5.3 -> 5.7 TB/s).
typedef __attribute__((ext_vector_type(4))) float nt_f32x4;
typedef __attribute__((ext_vector_type(2))) unsigned nt_u32x2;
__device__ __forceinline__ float4 load_stream(const float *base, int64_t q) {
  const nt_f32x4 t = __builtin_nontemporal_load(reinterpret_cast<const nt_f32x4 *>(base) + q);
  return make_float4(t[0], t[1], t[2], t[3]);
}
__device__ __forceinline__ void store_stream(float *base, int64_t q, const float4 &x) {
  const nt_f32x4 t = {x.x, x.y, x.z, x.w};
  __builtin_nontemporal_store(t, reinterpret_cast<nt_f32x4 *>(base) + q);
}
__device__ __forceinline__ void store_stream(uint16_t *base, int64_t q, const uint2 &x) {
  const nt_u32x2 t = {x.x, x.y};
  __builtin_nontemporal_store(t, reinterpret_cast<nt_u32x2 *>(base) + q);
}

// 16-byte vector of raw bits
struct __attribute__((aligned(16))) u32x4 {
  uint32_t x, y, z, w;
};

// g[u] += sum over the segment's (slot, token) pairs of coef[slot] * dense[token, 4-element piece seg0 + ROW_THREADS u], pairs
// in ascending order (the order every route to these gradient rows uses, so all of them give the same bits).
// A pair costs three dependent loads (slot, then coefficient and token, then the row): pairs are taken in groups
// whose index and row loads are all issued before the first multiply-add, which hides that chain on long segments.
template <bool DENSE_BF16, int ROW_THREADS = 256>
__device__ __forceinline__ void gather_rows_fma(float4 (&g)[4], int lo, int hi, const int32_t *__restrict__ feat_slot,
                                                const int32_t *__restrict__ slot_tok, const float *__restrict__ coef,
                                                const char *dbase, size_t row_bytes, int seg0, int n_seg) {
  constexpr int C = DENSE_BF16 ? 4 : 2;
  typedef typename std::conditional<DENSE_BF16, uint2, float4>::type piece_t;
  auto fma_piece = [&](float4 &acc, float c, const piece_t &r) {
    float4 x;
    if constexpr (DENSE_BF16) {
      x.x = __uint_as_float(r.x << 16); x.y = __uint_as_float(r.x & 0xffff0000u);
      x.z = __uint_as_float(r.y << 16); x.w = __uint_as_float(r.y & 0xffff0000u);
    } else {
      x = r;
    }
    acc.x = fmaf(c, x.x, acc.x); acc.y = fmaf(c, x.y, acc.y);
    acc.z = fmaf(c, x.z, acc.z); acc.w = fmaf(c, x.w, acc.w);
  };
  int i = lo;
  for (; i + C <= hi; i += C) {
    int sl[C];
#pragma unroll
    for (int j = 0; j < C; ++j) sl[j] = feat_slot[i + j];
    float c[C];
    const piece_t *row[C];
#pragma unroll
    for (int j = 0; j < C; ++j) {
      c[j] = coef[sl[j]];
      row[j] = reinterpret_cast<const piece_t *>(dbase + (size_t)slot_tok[sl[j]] * row_bytes);
    }
    piece_t r[C][4];
#pragma unroll
    for (int j = 0; j < C; ++j)
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int seg = seg0 + u * ROW_THREADS;
        if (seg < n_seg) r[j][u] = row[j][seg];
      }
#pragma unroll
    for (int j = 0; j < C; ++j)
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (seg0 + u * ROW_THREADS < n_seg) fma_piece(g[u], c[j], r[j][u]);
  }
  for (; i < hi; ++i) {
    const int sl = feat_slot[i];
    const float c = coef[sl];
    const piece_t *row = reinterpret_cast<const piece_t *>(dbase + (size_t)slot_tok[sl] * row_bytes);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int seg = seg0 + u * ROW_THREADS;
      if (seg < n_seg) fma_piece(g[u], c, row[seg]);
    }
  }
}

// The same sum, computed by a whole workgroup of ROW_THREADS threads for ONE segment (every thread calls it; a
// thread whose pieces lie past the row passes seg0 >= n_seg and only helps).  The segment's coefficients and
// tokens are first staged in LDS, ROW_THREADS pairs at a time and one pair per thread, so the two dependent
// index loads are paid once per chunk instead of once per group of pairs; the rows of a group of pairs are then
// all requested before the first multiply-add.  U pieces per thread (piece u at seg0 + ROW_THREADS u); pairs in
// ascending order as above, so the bits are the same.  s_coef / s_tok: ROW_THREADS entries of LDS each.
template <bool DENSE_BF16, int ROW_THREADS, int U>
__device__ __forceinline__ void gather_rows_staged(float4 (&g)[U], int lo, int hi, const int32_t *__restrict__ feat_slot,
                                                   const int32_t *__restrict__ slot_tok, const float *__restrict__ coef,
                                                   const char *dbase, size_t row_bytes, int seg0, int n_seg,
                                                   float *s_coef, int32_t *s_tok) {
  constexpr int C = (DENSE_BF16 ? 8 : 4) / (U == 4 ? 2 : 1);   // pairs whose rows are in flight together
  typedef typename std::conditional<DENSE_BF16, uint2, float4>::type piece_t;
  auto fma_piece = [&](float4 &acc, float c, const piece_t &r) {
    float4 x;
    if constexpr (DENSE_BF16) {
      x.x = __uint_as_float(r.x << 16); x.y = __uint_as_float(r.x & 0xffff0000u);
      x.z = __uint_as_float(r.y << 16); x.w = __uint_as_float(r.y & 0xffff0000u);
    } else {
      x = r;
    }
    acc.x = fmaf(c, x.x, acc.x); acc.y = fmaf(c, x.y, acc.y);
    acc.z = fmaf(c, x.z, acc.z); acc.w = fmaf(c, x.w, acc.w);
  };
  const int tid = threadIdx.x;
  for (int c0 = lo; c0 < hi; c0 += ROW_THREADS) {
    const int n = hi - c0 < ROW_THREADS ? hi - c0 : ROW_THREADS;
    __syncthreads();   // the previous chunk (or the previous call) has been consumed
    if (tid < n) {
      const int sl = feat_slot[c0 + tid];
      s_coef[tid] = coef[sl];
      s_tok[tid] = slot_tok[sl];
    }
    __syncthreads();
    int i = 0;
    for (; i + C <= n; i += C) {
      piece_t r[C][U];
#pragma unroll
      for (int j = 0; j < C; ++j) {
        const piece_t *row = reinterpret_cast<const piece_t *>(dbase + (size_t)s_tok[i + j] * row_bytes);
#pragma unroll
        for (int u = 0; u < U; ++u)
          if (seg0 + u * ROW_THREADS < n_seg) r[j][u] = row[seg0 + u * ROW_THREADS];
      }
#pragma unroll
      for (int j = 0; j < C; ++j) {
        const float c = s_coef[i + j];
#pragma unroll
        for (int u = 0; u < U; ++u)
          if (seg0 + u * ROW_THREADS < n_seg) fma_piece(g[u], c, r[j][u]);
      }
    }
    for (; i < n; ++i) {
      const float c = s_coef[i];
      const piece_t *row = reinterpret_cast<const piece_t *>(dbase + (size_t)s_tok[i] * row_bytes);
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (seg0 + u * ROW_THREADS < n_seg) fma_piece(g[u], c, row[seg0 + u * ROW_THREADS]);
    }
  }
}

}  // namespace sae
