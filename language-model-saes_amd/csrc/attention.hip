// Causal softmax attention with grouped value heads for gfx950 (bf16 operands, fp32 accumulation), forward and
// backward, on the matrix cores (v_mfma_f32_16x16x32_bf16).
//
// The mixing step of low-rank sparse attention: every query/key head h has d_qk-wide queries and keys and a
// d_v-wide value whose columns are d_v separate rank-1 value heads (dictionary features h * d_v .. (h + 1) * d_v - 1)
// that share head h's attention pattern.  out[b, s, h, :] = sum_{s' <= s} softmax_s'(scale * q[b,s,h] . k[b,s',h]) v[b,s',h,:].
//
// Layouts (bf16 unless noted; T = n_batch * seq tokens, token t = b * seq + s):
//   "natural"     [T, n_heads * width]   one token's heads side by side (what the projections x @ W produce),
//   "transposed"  [n_heads * width, T]   the same matrix transposed (what the projections W @ x^T produce).
// A matrix-core operand needs its contraction index contiguous in memory.  The scores contract over the head
// width (natural q, k), the mixing contracts over key positions (transposed v), and the backward products
// contract over positions or over widths in turn, so each kernel takes every operand in the layout(s) its
// products need; the transposed copies come for free from the projection GEMM with its operands swapped, or
// from the cast-transpose kernel.
//
// Fragment convention of the instruction (D = A B, 16 x 16 x 32): lane l supplies A[m = l % 16][8 consecutive k of
// group l / 16] and B[same k][n = l % 16], and receives D[m = 4 (l / 16) + i][n = l % 16], i < 4.  The contraction
// slots of a lane group only have to mean the same index in A and B: a probability tile leaves the score product
// as D (4 consecutive positions per lane), is packed to bf16 in registers and used as the B operand of the next
// product with slots {4g + i} of one 16-position tile and {4g + i} of the next; the A operand is read from LDS
// with the same two 8-byte pieces.  No probability ever goes through LDS or HBM.
//
// Forward: one workgroup = 64 queries of one (batch, head); wave w owns queries 16 w .. 16 w + 15 and walks the
// key blocks 0 .. diagonal with the online softmax (running maximum and sum per query in fp32, log2 domain).
// Backward: D[q] = sum_dv dout * out (one small kernel); dV and dK each by a workgroup per 64 keys that walks the
// query blocks diagonal .. last; dQ by a workgroup per 64 queries that walks the key blocks 0 .. diagonal.  All three
// recompute the probabilities from q, k and the saved log-sum-exp.  No atomics: results are reproducible.
#include "common.h"

namespace sae {

typedef __attribute__((ext_vector_type(8))) __bf16 att_bf16x8;
typedef __attribute__((ext_vector_type(4))) float att_f32x4;

constexpr int ATT_BLOCK = 64;       // positions per workgroup and per inner iteration
constexpr int ATT_THREADS = 256;
constexpr int ATT_TPITCH = 144;     // bytes per LDS row of a transposed tile: 64 positions * 2 + 16 (bank spread)
constexpr float ATT_LOG2E = 1.4426950408889634f;

__device__ __forceinline__ constexpr int att_nat_pitch(int cols) { return cols * 2 + 16; }

__device__ __forceinline__ uint32_t att_pack2(float a, float b) {
  const cvt_f32x2 in = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(in, cvt_bf16x2));
}

__device__ __forceinline__ att_bf16x8 att_pack8(const att_f32x4 &lo, const att_f32x4 &hi) {
  u32x4 r;
  r.x = att_pack2(lo[0], lo[1]); r.y = att_pack2(lo[2], lo[3]);
  r.z = att_pack2(hi[0], hi[1]); r.w = att_pack2(hi[2], hi[3]);
  return __builtin_bit_cast(att_bf16x8, r);
}

// 8 bf16 + 8 fp32 biases -> 8 bf16 (each sum rounded to nearest even: what `bf16_tensor + fp32_bias` cast back gives)
__device__ __forceinline__ u32x4 att_add_bias8(const u32x4 &v, const float *__restrict__ bias) {
  const float4 b0 = *reinterpret_cast<const float4 *>(bias), b1 = *reinterpret_cast<const float4 *>(bias + 4);
  u32x4 r;
  r.x = att_pack2(__uint_as_float(v.x << 16) + b0.x, __uint_as_float(v.x & 0xffff0000u) + b0.y);
  r.y = att_pack2(__uint_as_float(v.y << 16) + b0.z, __uint_as_float(v.y & 0xffff0000u) + b0.w);
  r.z = att_pack2(__uint_as_float(v.z << 16) + b1.x, __uint_as_float(v.z & 0xffff0000u) + b1.y);
  r.w = att_pack2(__uint_as_float(v.w << 16) + b1.z, __uint_as_float(v.w & 0xffff0000u) + b1.w);
  return r;
}

__device__ __forceinline__ u32x4 att_add_bias1(const u32x4 &v, float b) {
  u32x4 r;
  r.x = att_pack2(__uint_as_float(v.x << 16) + b, __uint_as_float(v.x & 0xffff0000u) + b);
  r.y = att_pack2(__uint_as_float(v.y << 16) + b, __uint_as_float(v.y & 0xffff0000u) + b);
  r.z = att_pack2(__uint_as_float(v.z << 16) + b, __uint_as_float(v.z & 0xffff0000u) + b);
  r.w = att_pack2(__uint_as_float(v.w << 16) + b, __uint_as_float(v.w & 0xffff0000u) + b);
  return r;
}

// Tiles travel global -> registers -> LDS in two halves, so that the loads of the next tile are in flight while the
// current one is consumed: att_load_* issues the 16-byte loads of a thread's pieces, att_store_* (an iteration later)
// adds the bias, if any, and writes them to LDS.
//
// Natural layout: 64 consecutive tokens x COLS columns -> LDS rows of att_nat_pitch(COLS) bytes.  Rows at or past
// `rows_valid` are zero.  `bias` (nullable) is indexed by absolute column.
template <int COLS>
__device__ __forceinline__ void att_load_nat(u32x4 (&regs)[COLS / 32], const uint16_t *__restrict__ g, int64_t ld, int64_t tok0,
                                             int rows_valid, int col0) {
  constexpr int CH = COLS / 8;
#pragma unroll
  for (int j = 0; j < COLS / 32; ++j) {
    const int c = threadIdx.x + j * ATT_THREADS;
    const int r = c / CH, cc = c % CH;
    regs[j] = u32x4{0u, 0u, 0u, 0u};
    if (r < rows_valid) regs[j] = *reinterpret_cast<const u32x4 *>(g + (tok0 + r) * ld + col0 + cc * 8);
  }
}

template <int COLS>
__device__ __forceinline__ void att_store_nat(char *lds, const u32x4 (&regs)[COLS / 32], int rows_valid, int col0,
                                              const float *__restrict__ bias) {
  constexpr int CH = COLS / 8, PITCH = att_nat_pitch(COLS);
#pragma unroll
  for (int j = 0; j < COLS / 32; ++j) {
    const int c = threadIdx.x + j * ATT_THREADS;
    const int r = c / CH, cc = c % CH;
    u32x4 v = regs[j];
    if (bias && r < rows_valid) v = att_add_bias8(v, bias + col0 + cc * 8);
    *reinterpret_cast<u32x4 *>(lds + r * PITCH + cc * 16) = v;
  }
}

// Transposed layout: ROWS rows x 64 consecutive tokens -> LDS rows of ATT_TPITCH bytes.  Columns at or past
// `cols_valid` (a multiple of 8) are zero.  `bias` (nullable) is indexed by absolute row.
template <int ROWS>
__device__ __forceinline__ void att_load_tr(u32x4 (&regs)[ROWS / 32], const uint16_t *__restrict__ gt, int64_t ld, int row0,
                                            int64_t tok0, int cols_valid) {
#pragma unroll
  for (int j = 0; j < ROWS / 32; ++j) {
    const int c = threadIdx.x + j * ATT_THREADS;
    const int r = c >> 3, cc = c & 7;
    regs[j] = u32x4{0u, 0u, 0u, 0u};
    if (cc * 8 < cols_valid) regs[j] = *reinterpret_cast<const u32x4 *>(gt + (int64_t)(row0 + r) * ld + tok0 + cc * 8);
  }
}

template <int ROWS>
__device__ __forceinline__ void att_store_tr(char *lds, const u32x4 (&regs)[ROWS / 32], int row0, int cols_valid,
                                             const float *__restrict__ bias) {
#pragma unroll
  for (int j = 0; j < ROWS / 32; ++j) {
    const int c = threadIdx.x + j * ATT_THREADS;
    const int r = c >> 3, cc = c & 7;
    u32x4 v = regs[j];
    if (bias && cc * 8 < cols_valid) v = att_add_bias1(v, bias[row0 + r]);
    *reinterpret_cast<u32x4 *>(lds + r * ATT_TPITCH + cc * 16) = v;
  }
}

// One token's row of a natural-layout matrix as the register fragments of a lane (8 columns of group g per 32-column step).
template <int COLS>
__device__ __forceinline__ void att_row_frags(att_bf16x8 (&f)[COLS / 32], const uint16_t *__restrict__ g, int64_t ld,
                                              int64_t tok, bool valid, int col0, int grp, const float *__restrict__ bias) {
#pragma unroll
  for (int kk = 0; kk < COLS / 32; ++kk) {
    u32x4 v = {0u, 0u, 0u, 0u};
    if (valid) {
      v = *reinterpret_cast<const u32x4 *>(g + tok * ld + col0 + kk * 32 + grp * 8);
      if (bias) v = att_add_bias8(v, bias + col0 + kk * 32 + grp * 8);
    }
    f[kk] = __builtin_bit_cast(att_bf16x8, v);
  }
}

__device__ __forceinline__ att_bf16x8 att_nat_frag(const char *lds, int pitch, int row, int kk, int grp) {
  return *reinterpret_cast<const att_bf16x8 *>(lds + row * pitch + (kk * 32 + grp * 8) * 2);
}

// positions {32 u + 4 g + i} and {32 u + 16 + 4 g + i}, i < 4, of one row of a transposed tile
__device__ __forceinline__ att_bf16x8 att_tr_frag(const char *lds, int row, int u, int grp) {
  const uint2 lo = *reinterpret_cast<const uint2 *>(lds + row * ATT_TPITCH + (32 * u + 4 * grp) * 2);
  const uint2 hi = *reinterpret_cast<const uint2 *>(lds + row * ATT_TPITCH + (32 * u + 16 + 4 * grp) * 2);
  u32x4 r;
  r.x = lo.x; r.y = lo.y; r.z = hi.x; r.w = hi.y;
  return __builtin_bit_cast(att_bf16x8, r);
}

// Workgroup id -> (position block, head, sequence).  The hardware deals consecutive workgroup ids round-robin to the 8
// XCDs, each with an L2 of its own; all position blocks of one (sequence, head) re-read the same keys / values (or
// queries), so they are placed on ONE XCD: id = 8 * slot + xcd, and inside an XCD the slots walk the blocks of head
// group xcd, 8 + xcd, ...  Within a head the block with the most work comes first (`reverse`).
__device__ __forceinline__ void att_block_coords(int n_blocks, int n_heads, int n_batch, bool reverse, int &blk, int &h, int &b) {
  const int id = blockIdx.x, nh = n_heads * n_batch;
  int bh, x;
  if ((nh & 7) == 0) {
    const int xcd = id & 7, slot = id >> 3;
    bh = (slot / n_blocks) * 8 + xcd;
    x = slot % n_blocks;
  } else {
    bh = id / n_blocks;
    x = id % n_blocks;
  }
  blk = reverse ? n_blocks - 1 - x : x;
  h = bh % n_heads;
  b = bh / n_heads;
}

__device__ __forceinline__ att_f32x4 att_mfma(const att_bf16x8 &a, const att_bf16x8 &b, const att_f32x4 &c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ float att_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ---- forward ---------------------------------------------------------------------------------------------
template <int DQK, int DV>
__global__ __launch_bounds__(ATT_THREADS) void attn_fwd_kernel(
    const uint16_t *__restrict__ q, const uint16_t *__restrict__ k, const uint16_t *__restrict__ vt,
    const float *__restrict__ bq, const float *__restrict__ bk, const float *__restrict__ bv, uint16_t *__restrict__ out,
    float *__restrict__ lse, int seq, int n_heads, int n_batch, int64_t T, float sc2) {
  constexpr int KP = att_nat_pitch(DQK);
  __shared__ __attribute__((aligned(16))) char s_k[ATT_BLOCK * KP];
  __shared__ __attribute__((aligned(16))) char s_vt[DV * ATT_TPITCH];
  int qb, h, b;
  att_block_coords((seq + ATT_BLOCK - 1) / ATT_BLOCK, n_heads, n_batch, true, qb, h, b);     // long rows of work first
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, lr = lane & 15, grp = lane >> 4;
  const int64_t tok0 = (int64_t)b * seq;
  const int64_t ldq = (int64_t)n_heads * DQK, ldv = (int64_t)n_heads * DV;
  const int q_row = qb * ATT_BLOCK + wave * 16 + lr;

  att_bf16x8 qf[DQK / 32];
  att_row_frags<DQK>(qf, q, ldq, tok0 + q_row, q_row < seq, h * DQK, grp, bq);
  att_f32x4 o[DV / 16];
#pragma unroll
  for (int n = 0; n < DV / 16; ++n) o[n] = att_f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  u32x4 rk[DQK / 32], rvt[DV / 32];
  att_load_nat<DQK>(rk, k, ldq, tok0, min(ATT_BLOCK, seq), h * DQK);
  att_load_tr<DV>(rvt, vt, T, h * DV, tok0, min(ATT_BLOCK, seq));
  for (int kb = 0; kb <= qb; ++kb) {
    const int valid = min(ATT_BLOCK, seq - kb * ATT_BLOCK);
    __syncthreads();                       // every wave is done with the previous tile
    att_store_nat<DQK>(s_k, rk, valid, h * DQK, bk);
    att_store_tr<DV>(s_vt, rvt, h * DV, valid, bv);
    __syncthreads();
    if (kb < qb) {                         // the next tile's loads fly while this one is consumed
      const int nvalid = min(ATT_BLOCK, seq - (kb + 1) * ATT_BLOCK);
      att_load_nat<DQK>(rk, k, ldq, tok0 + (kb + 1) * ATT_BLOCK, nvalid, h * DQK);
      att_load_tr<DV>(rvt, vt, T, h * DV, tok0 + (kb + 1) * ATT_BLOCK, nvalid);
    }
    att_f32x4 s[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      s[t] = att_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < DQK / 32; ++kk) s[t] = att_mfma(att_nat_frag(s_k, KP, t * 16 + lr, kk, grp), qf[kk], s[t]);
    }
    if (kb == qb) {                       // only the diagonal block has keys after the query
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (kb * ATT_BLOCK + t * 16 + 4 * grp + i > q_row) s[t][i] = -INFINITY;
    }
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) mx = fmaxf(mx, s[t][i]);
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    // every row meets at least one unmasked key in every block it visits, so m_new is finite; the scale is positive,
    // so the maximum is taken over the raw scores and scaled once
    const float m_new = fmaxf(m, mx * sc2);
    if (__any(m_new > m)) {               // a running maximum that did not move leaves the sums as they are
      const float alpha = att_exp2(m - m_new);      // exp2(-inf) = 0 on the first block
      l *= alpha;
#pragma unroll
      for (int n = 0; n < DV / 16; ++n)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[n][i] *= alpha;
      m = m_new;
    }
    float rs = 0.f;
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = att_exp2(fmaf(s[t][i], sc2, -m));
        s[t][i] = p;
        rs += p;
      }
    l += rs;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const att_bf16x8 pf = att_pack8(s[2 * u], s[2 * u + 1]);
#pragma unroll
      for (int n = 0; n < DV / 16; ++n) o[n] = att_mfma(att_tr_frag(s_vt, n * 16 + lr, u, grp), pf, o[n]);
    }
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (q_row < seq) {
    const float inv = 1.f / l;
    uint16_t *orow = out + (tok0 + q_row) * ldv + h * DV + 4 * grp;
#pragma unroll
    for (int n = 0; n < DV / 16; ++n) {
      uint2 pk;
      pk.x = att_pack2(o[n][0] * inv, o[n][1] * inv);
      pk.y = att_pack2(o[n][2] * inv, o[n][3] * inv);
      *reinterpret_cast<uint2 *>(orow + n * 16) = pk;
    }
    if (grp == 0) lse[((int64_t)b * n_heads + h) * seq + q_row] = (m + __log2f(l)) * 0.6931471805599453f;
  }
}

// ---- backward: D[b, h, s] = sum_dv dout[t, h, dv] * out[t, h, dv] ---------------------------------------------
template <int DV>
__global__ __launch_bounds__(256) void attn_bwd_prep_kernel(const uint16_t *__restrict__ dout, const uint16_t *__restrict__ out,
                                                            float *__restrict__ dvec, int seq, int n_heads, int64_t T) {
  // 16 lanes per (token, head); a lane covers 8 columns per trip
  const int64_t pair = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 4;
  const int sub = threadIdx.x & 15;
  const int64_t n_pairs = T * n_heads;
  float acc = 0.f;
  if (pair < n_pairs) {
    const int64_t t = pair / n_heads;
    const int h = (int)(pair % n_heads);
    const int64_t base = t * ((int64_t)n_heads * DV) + (int64_t)h * DV;
    for (int c = sub * 8; c < DV; c += 128) {
      const u32x4 a = *reinterpret_cast<const u32x4 *>(dout + base + c), o = *reinterpret_cast<const u32x4 *>(out + base + c);
      const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, ow[4] = {o.x, o.y, o.z, o.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc = fmaf(__uint_as_float(aw[j] << 16), __uint_as_float(ow[j] << 16), acc);
        acc = fmaf(__uint_as_float(aw[j] & 0xffff0000u), __uint_as_float(ow[j] & 0xffff0000u), acc);
      }
    }
  }
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
  if (pair < n_pairs && sub == 0) {
    const int64_t t = pair / n_heads;
    const int h = (int)(pair % n_heads);
    dvec[((t / seq) * n_heads + h) * seq + (t % seq)] = acc;
  }
}

// ---- backward: dV^T (one workgroup per 64 keys) ------------------------------------------------------------------
// dV^T[dv, key] = sum_q dout^T[dv, q] P[q, key].  (dK lives in a kernel of its own: fused, the two accumulators, the
// four operand tiles and their fragments leave one wave per SIMD, and the kernel waits on its own barriers.)
template <int DQK, int DV>
__global__ __launch_bounds__(ATT_THREADS) void attn_bwd_dv_kernel(
    const uint16_t *__restrict__ q, const uint16_t *__restrict__ k, const uint16_t *__restrict__ doutt,
    const float *__restrict__ bq, const float *__restrict__ bk, const float *__restrict__ lse, uint16_t *__restrict__ dvt,
    int seq, int n_heads, int n_batch, int64_t T, float sc2) {
  constexpr int QP = att_nat_pitch(DQK);
  __shared__ __attribute__((aligned(16))) char s_q[ATT_BLOCK * QP];
  __shared__ __attribute__((aligned(16))) char s_dot[DV * ATT_TPITCH];
  __shared__ float s_lse[ATT_BLOCK];
  const int nqb = (seq + ATT_BLOCK - 1) / ATT_BLOCK;
  int kb, h, b;
  att_block_coords(nqb, n_heads, n_batch, false, kb, h, b);     // key block 0 walks every query block: first
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, lr = lane & 15, grp = lane >> 4;
  const int64_t tok0 = (int64_t)b * seq;
  const int64_t ldq = (int64_t)n_heads * DQK;
  const int key_col = kb * ATT_BLOCK + wave * 16 + lr;

  att_bf16x8 kf[DQK / 32];
  att_row_frags<DQK>(kf, k, ldq, tok0 + key_col, key_col < seq, h * DQK, grp, bk);
  att_f32x4 dv[DV / 16];
#pragma unroll
  for (int n = 0; n < DV / 16; ++n) dv[n] = att_f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 rq[DQK / 32], rdot[DV / 32];
  float r_lse = INFINITY;                  // threads 0..63: one query's log-sum-exp in the log2 domain
  auto load_tiles = [&](int qb) {
    const int valid = min(ATT_BLOCK, seq - qb * ATT_BLOCK);
    att_load_nat<DQK>(rq, q, ldq, tok0 + qb * ATT_BLOCK, valid, h * DQK);
    att_load_tr<DV>(rdot, doutt, T, h * DV, tok0 + qb * ATT_BLOCK, valid);
    if (threadIdx.x < ATT_BLOCK) {
      const int qq = qb * ATT_BLOCK + threadIdx.x;
      r_lse = qq < seq ? lse[((int64_t)b * n_heads + h) * seq + qq] * ATT_LOG2E : INFINITY;   // +inf: p = 0 past the sequence
    }
  };
  load_tiles(kb);
  for (int qb = kb; qb < nqb; ++qb) {
    const int valid = min(ATT_BLOCK, seq - qb * ATT_BLOCK);
    __syncthreads();
    att_store_nat<DQK>(s_q, rq, valid, h * DQK, bq);
    att_store_tr<DV>(s_dot, rdot, h * DV, valid, nullptr);
    if (threadIdx.x < ATT_BLOCK) s_lse[threadIdx.x] = r_lse;
    __syncthreads();
    if (qb + 1 < nqb) load_tiles(qb + 1);
    att_f32x4 p[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      att_f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < DQK / 32; ++kk) s = att_mfma(att_nat_frag(s_q, QP, t * 16 + lr, kk, grp), kf[kk], s);
      const att_f32x4 l4 = *reinterpret_cast<const att_f32x4 *>(s_lse + t * 16 + 4 * grp);
#pragma unroll
      for (int i = 0; i < 4; ++i) p[t][i] = att_exp2(fmaf(s[i], sc2, -l4[i]));
    }
    if (qb == kb) {                        // the diagonal block: queries before the key do not see it
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (key_col > qb * ATT_BLOCK + t * 16 + 4 * grp + i) p[t][i] = 0.f;
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const att_bf16x8 pf = att_pack8(p[2 * u], p[2 * u + 1]);
#pragma unroll
      for (int n = 0; n < DV / 16; ++n) dv[n] = att_mfma(att_tr_frag(s_dot, n * 16 + lr, u, grp), pf, dv[n]);
    }
  }
  if (key_col < seq) {
#pragma unroll
    for (int n = 0; n < DV / 16; ++n)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        dvt[(int64_t)(h * DV + n * 16 + 4 * grp + i) * T + tok0 + key_col] = (uint16_t)(att_pack2(dv[n][i], 0.f) & 0xffffu);
  }
}

// ---- backward: dK^T (one workgroup per 64 keys) ------------------------------------------------------------------
// dK^T[dqk, key] = sum_q q^T[dqk, q] dS[q, key],  dS = P (dP - D) scale,  dP[q, key] = dout[q, :] . v[key, :].
template <int DQK, int DV>
__global__ __launch_bounds__(ATT_THREADS) void attn_bwd_dk_kernel(
    const uint16_t *__restrict__ q, const uint16_t *__restrict__ qt, const uint16_t *__restrict__ k,
    const uint16_t *__restrict__ v, const uint16_t *__restrict__ dout, const float *__restrict__ bq,
    const float *__restrict__ bk, const float *__restrict__ bv, const float *__restrict__ lse,
    const float *__restrict__ dvec, uint16_t *__restrict__ dkt, int seq, int n_heads, int n_batch, int64_t T, float sc2,
    float scale) {
  constexpr int QP = att_nat_pitch(DQK), OP = att_nat_pitch(DV);
  __shared__ __attribute__((aligned(16))) char s_q[ATT_BLOCK * QP];
  __shared__ __attribute__((aligned(16))) char s_qt[DQK * ATT_TPITCH];
  __shared__ __attribute__((aligned(16))) char s_do[ATT_BLOCK * OP];
  __shared__ float s_lse[ATT_BLOCK], s_d[ATT_BLOCK];
  const int nqb = (seq + ATT_BLOCK - 1) / ATT_BLOCK;
  int kb, h, b;
  att_block_coords(nqb, n_heads, n_batch, false, kb, h, b);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, lr = lane & 15, grp = lane >> 4;
  const int64_t tok0 = (int64_t)b * seq;
  const int64_t ldq = (int64_t)n_heads * DQK, ldv = (int64_t)n_heads * DV;
  const int key_col = kb * ATT_BLOCK + wave * 16 + lr;

  att_bf16x8 kf[DQK / 32], vf[DV / 32];
  att_row_frags<DQK>(kf, k, ldq, tok0 + key_col, key_col < seq, h * DQK, grp, bk);
  att_row_frags<DV>(vf, v, ldv, tok0 + key_col, key_col < seq, h * DV, grp, bv);
  att_f32x4 dk[DQK / 16];
#pragma unroll
  for (int n = 0; n < DQK / 16; ++n) dk[n] = att_f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 rq[DQK / 32], rqt[DQK / 32], rdo[DV / 32];
  float r_lse = INFINITY, r_d = 0.f;       // threads 0..63: one query's log-sum-exp (log2 domain) and D
  auto load_tiles = [&](int qb) {
    const int valid = min(ATT_BLOCK, seq - qb * ATT_BLOCK);
    att_load_nat<DQK>(rq, q, ldq, tok0 + qb * ATT_BLOCK, valid, h * DQK);
    att_load_tr<DQK>(rqt, qt, T, h * DQK, tok0 + qb * ATT_BLOCK, valid);
    att_load_nat<DV>(rdo, dout, ldv, tok0 + qb * ATT_BLOCK, valid, h * DV);
    if (threadIdx.x < ATT_BLOCK) {
      const int qq = qb * ATT_BLOCK + threadIdx.x;
      const int64_t at = ((int64_t)b * n_heads + h) * seq + qq;
      r_lse = qq < seq ? lse[at] * ATT_LOG2E : INFINITY;   // +inf: a row past the sequence gets p = 0
      r_d = qq < seq ? dvec[at] : 0.f;
    }
  };
  load_tiles(kb);
  for (int qb = kb; qb < nqb; ++qb) {
    const int valid = min(ATT_BLOCK, seq - qb * ATT_BLOCK);
    __syncthreads();
    att_store_nat<DQK>(s_q, rq, valid, h * DQK, bq);
    att_store_tr<DQK>(s_qt, rqt, h * DQK, valid, bq);
    att_store_nat<DV>(s_do, rdo, valid, h * DV, nullptr);
    if (threadIdx.x < ATT_BLOCK) {
      s_lse[threadIdx.x] = r_lse;
      s_d[threadIdx.x] = r_d;
    }
    __syncthreads();
    if (qb + 1 < nqb) load_tiles(qb + 1);
    att_f32x4 ds[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      att_f32x4 s = {0.f, 0.f, 0.f, 0.f}, dp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < DQK / 32; ++kk) s = att_mfma(att_nat_frag(s_q, QP, t * 16 + lr, kk, grp), kf[kk], s);
#pragma unroll
      for (int kk = 0; kk < DV / 32; ++kk) dp = att_mfma(att_nat_frag(s_do, OP, t * 16 + lr, kk, grp), vf[kk], dp);
      const att_f32x4 l4 = *reinterpret_cast<const att_f32x4 *>(s_lse + t * 16 + 4 * grp);
      const att_f32x4 d4 = *reinterpret_cast<const att_f32x4 *>(s_d + t * 16 + 4 * grp);
#pragma unroll
      for (int i = 0; i < 4; ++i) ds[t][i] = att_exp2(fmaf(s[i], sc2, -l4[i])) * ((dp[i] - d4[i]) * scale);
    }
    if (qb == kb) {
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (key_col > qb * ATT_BLOCK + t * 16 + 4 * grp + i) ds[t][i] = 0.f;
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const att_bf16x8 dsf = att_pack8(ds[2 * u], ds[2 * u + 1]);
#pragma unroll
      for (int n = 0; n < DQK / 16; ++n) dk[n] = att_mfma(att_tr_frag(s_qt, n * 16 + lr, u, grp), dsf, dk[n]);
    }
  }
  if (key_col < seq) {
#pragma unroll
    for (int n = 0; n < DQK / 16; ++n)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        dkt[(int64_t)(h * DQK + n * 16 + 4 * grp + i) * T + tok0 + key_col] = (uint16_t)(att_pack2(dk[n][i], 0.f) & 0xffffu);
  }
}

// ---- backward: dQ^T (one workgroup per 64 queries) -------------------------------------------------------------
template <int DQK, int DV>
__global__ __launch_bounds__(ATT_THREADS) void attn_bwd_dq_kernel(
    const uint16_t *__restrict__ q, const uint16_t *__restrict__ k, const uint16_t *__restrict__ kt,
    const uint16_t *__restrict__ v, const uint16_t *__restrict__ dout, const float *__restrict__ bq,
    const float *__restrict__ bk, const float *__restrict__ bv, const float *__restrict__ lse,
    const float *__restrict__ dvec, uint16_t *__restrict__ dqt, int seq, int n_heads, int n_batch, int64_t T, float sc2,
    float scale) {
  constexpr int KP = att_nat_pitch(DQK), VP = att_nat_pitch(DV);
  __shared__ __attribute__((aligned(16))) char s_k[ATT_BLOCK * KP];
  __shared__ __attribute__((aligned(16))) char s_kt[DQK * ATT_TPITCH];
  __shared__ __attribute__((aligned(16))) char s_v[ATT_BLOCK * VP];
  int qb, h, b;
  att_block_coords((seq + ATT_BLOCK - 1) / ATT_BLOCK, n_heads, n_batch, true, qb, h, b);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, lr = lane & 15, grp = lane >> 4;
  const int64_t tok0 = (int64_t)b * seq;
  const int64_t ldq = (int64_t)n_heads * DQK, ldv = (int64_t)n_heads * DV;
  const int q_row = qb * ATT_BLOCK + wave * 16 + lr;
  const bool q_ok = q_row < seq;

  att_bf16x8 qf[DQK / 32], dof[DV / 32];
  att_row_frags<DQK>(qf, q, ldq, tok0 + q_row, q_ok, h * DQK, grp, bq);
  att_row_frags<DV>(dof, dout, ldv, tok0 + q_row, q_ok, h * DV, grp, nullptr);
  const int64_t at = ((int64_t)b * n_heads + h) * seq + q_row;
  const float lse2 = q_ok ? lse[at] * ATT_LOG2E : INFINITY;
  const float dq_sum = q_ok ? dvec[at] : 0.f;
  att_f32x4 dq[DQK / 16];
#pragma unroll
  for (int n = 0; n < DQK / 16; ++n) dq[n] = att_f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 rk[DQK / 32], rkt[DQK / 32], rv[DV / 32];
  auto load_tiles = [&](int kb) {
    const int valid = min(ATT_BLOCK, seq - kb * ATT_BLOCK);
    att_load_nat<DQK>(rk, k, ldq, tok0 + kb * ATT_BLOCK, valid, h * DQK);
    att_load_tr<DQK>(rkt, kt, T, h * DQK, tok0 + kb * ATT_BLOCK, valid);
    att_load_nat<DV>(rv, v, ldv, tok0 + kb * ATT_BLOCK, valid, h * DV);
  };
  load_tiles(0);
  for (int kb = 0; kb <= qb; ++kb) {
    const int valid = min(ATT_BLOCK, seq - kb * ATT_BLOCK);
    __syncthreads();
    att_store_nat<DQK>(s_k, rk, valid, h * DQK, bk);
    att_store_tr<DQK>(s_kt, rkt, h * DQK, valid, bk);
    att_store_nat<DV>(s_v, rv, valid, h * DV, bv);
    __syncthreads();
    if (kb < qb) load_tiles(kb + 1);
    att_f32x4 ds[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      att_f32x4 s = {0.f, 0.f, 0.f, 0.f}, dp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < DQK / 32; ++kk) s = att_mfma(att_nat_frag(s_k, KP, t * 16 + lr, kk, grp), qf[kk], s);
#pragma unroll
      for (int kk = 0; kk < DV / 32; ++kk) dp = att_mfma(att_nat_frag(s_v, VP, t * 16 + lr, kk, grp), dof[kk], dp);
#pragma unroll
      for (int i = 0; i < 4; ++i) ds[t][i] = att_exp2(fmaf(s[i], sc2, -lse2)) * ((dp[i] - dq_sum) * scale);
    }
    if (kb == qb) {                        // only the diagonal block has keys after the query
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (kb * ATT_BLOCK + t * 16 + 4 * grp + i > q_row) ds[t][i] = 0.f;
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const att_bf16x8 dsf = att_pack8(ds[2 * u], ds[2 * u + 1]);
#pragma unroll
      for (int n = 0; n < DQK / 16; ++n) dq[n] = att_mfma(att_tr_frag(s_kt, n * 16 + lr, u, grp), dsf, dq[n]);
    }
  }
  if (q_ok) {
#pragma unroll
    for (int n = 0; n < DQK / 16; ++n)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        dqt[(int64_t)(h * DQK + n * 16 + 4 * grp + i) * T + tok0 + q_row] = (uint16_t)(att_pack2(dq[n][i], 0.f) & 0xffffu);
  }
}

// out[r] = sum_c src[r, c] in fp32 for a bf16 or fp32 matrix [rows, cols]; one wave per row, fixed order; 16-byte
// loads when the rows allow it (cols a multiple of 8 / 4: every row then starts 16-byte aligned).
template <bool SRC_BF16>
__global__ __launch_bounds__(256) void row_sum_kernel(const void *__restrict__ src, float *__restrict__ out, int64_t rows, int64_t cols) {
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (r >= rows) return;
  float acc = 0.f;
  if constexpr (SRC_BF16) {
    const uint16_t *row = reinterpret_cast<const uint16_t *>(src) + r * cols;
    if ((cols & 7) == 0) {
      const u32x4 *row16 = reinterpret_cast<const u32x4 *>(row);
      const int64_t n16 = cols >> 3;
      for (int64_t c = lane; c < n16; c += 64) {
        const u32x4 v = row16[c];
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) acc += __uint_as_float(w[j] << 16) + __uint_as_float(w[j] & 0xffff0000u);
      }
    } else {
      for (int64_t c = lane; c < cols; c += 64) acc += bf16_bits_to_f32(row[c]);
    }
  } else {
    const float *row = reinterpret_cast<const float *>(src) + r * cols;
    if ((cols & 3) == 0) {
      const float4 *row16 = reinterpret_cast<const float4 *>(row);
      const int64_t n16 = cols >> 2;
      for (int64_t c = lane; c < n16; c += 64) {
        const float4 v = row16[c];
        acc += (v.x + v.y) + (v.z + v.w);
      }
    } else {
      for (int64_t c = lane; c < cols; c += 64) acc += row[c];
    }
  }
  acc = wave_sum(acc);
  if (lane == 0) out[r] = acc;
}

template <int DQK, int DV>
static int launch_fwd(const void *q, const void *k, const void *vt, const float *bq, const float *bk, const float *bv,
                      int64_t n_batch, int64_t seq, int64_t n_heads, double scale, void *out, float *lse, hipStream_t st) {
  const dim3 grid((unsigned)(((seq + ATT_BLOCK - 1) / ATT_BLOCK) * n_heads * n_batch));
  hipLaunchKernelGGL((attn_fwd_kernel<DQK, DV>), grid, dim3(ATT_THREADS), 0, st, (const uint16_t *)q, (const uint16_t *)k,
                     (const uint16_t *)vt, bq, bk, bv, (uint16_t *)out, lse, (int)seq, (int)n_heads, (int)n_batch, n_batch * seq,
                     (float)(scale * 1.4426950408889634));
  return check_launch("attention_fwd");
}

template <int DQK, int DV>
static int launch_bwd(const void *q, const void *qt, const void *k, const void *kt, const void *v, const void *out,
                      const void *dout, const void *doutt, const float *bq, const float *bk, const float *bv, const float *lse,
                      int64_t n_batch, int64_t seq, int64_t n_heads, double scale, float *dvec, void *dqt, void *dkt, void *dvt,
                      hipStream_t st) {
  const int64_t T = n_batch * seq;
  const dim3 grid((unsigned)(((seq + ATT_BLOCK - 1) / ATT_BLOCK) * n_heads * n_batch));
  const float sc2 = (float)(scale * 1.4426950408889634);
  const int64_t prep_blocks = (T * n_heads * 16 + 255) / 256;
  hipLaunchKernelGGL((attn_bwd_prep_kernel<DV>), dim3((unsigned)prep_blocks), dim3(256), 0, st, (const uint16_t *)dout,
                     (const uint16_t *)out, dvec, (int)seq, (int)n_heads, T);
  hipLaunchKernelGGL((attn_bwd_dv_kernel<DQK, DV>), grid, dim3(ATT_THREADS), 0, st, (const uint16_t *)q, (const uint16_t *)k,
                     (const uint16_t *)doutt, bq, bk, lse, (uint16_t *)dvt, (int)seq, (int)n_heads, (int)n_batch, T, sc2);
  hipLaunchKernelGGL((attn_bwd_dk_kernel<DQK, DV>), grid, dim3(ATT_THREADS), 0, st, (const uint16_t *)q, (const uint16_t *)qt,
                     (const uint16_t *)k, (const uint16_t *)v, (const uint16_t *)dout, bq, bk, bv, lse, dvec, (uint16_t *)dkt,
                     (int)seq, (int)n_heads, (int)n_batch, T, sc2, (float)scale);
  hipLaunchKernelGGL((attn_bwd_dq_kernel<DQK, DV>), grid, dim3(ATT_THREADS), 0, st, (const uint16_t *)q, (const uint16_t *)k,
                     (const uint16_t *)kt, (const uint16_t *)v, (const uint16_t *)dout, bq, bk, bv, lse, dvec, (uint16_t *)dqt,
                     (int)seq, (int)n_heads, (int)n_batch, T, sc2, (float)scale);
  return check_launch("attention_bwd");
}

static int check_shapes(const char *what, int64_t n_batch, int64_t seq, int64_t n_heads, int64_t d_qk, int64_t d_v) {
  SAE_REQUIRE(n_batch > 0 && seq > 0 && n_heads > 0, SAE_ERR_INVALID_ARG, "%s: sizes must be positive", what);
  SAE_REQUIRE(((seq + ATT_BLOCK - 1) / ATT_BLOCK) * n_heads * n_batch < ((int64_t)1 << 31), SAE_ERR_UNSUPPORTED,
              "%s: too many (block, head, sequence) workgroups", what);
  SAE_REQUIRE(seq % 8 == 0, SAE_ERR_UNSUPPORTED, "%s: seq = %lld must be a multiple of 8 (16-byte pieces of the transposed operands)",
              what, (long long)seq);
  SAE_REQUIRE((d_qk == 32 || d_qk == 64) && (d_v == 32 || d_v == 64 || d_v == 128), SAE_ERR_UNSUPPORTED,
              "%s: built for d_qk in {32, 64} and d_v in {32, 64, 128}, got %lld / %lld", what, (long long)d_qk, (long long)d_v);
  SAE_REQUIRE(n_batch * seq * n_heads * (d_v > d_qk ? d_v : d_qk) < (int64_t)1 << 40, SAE_ERR_UNSUPPORTED, "%s: too large", what);
  return SAE_OK;
}

}  // namespace sae

#define ATT_DISPATCH(CALL)                                                      \
  if (d_qk == 32 && d_v == 32) return CALL(32, 32);                             \
  if (d_qk == 32 && d_v == 64) return CALL(32, 64);                             \
  if (d_qk == 32 && d_v == 128) return CALL(32, 128);                           \
  if (d_qk == 64 && d_v == 32) return CALL(64, 32);                             \
  if (d_qk == 64 && d_v == 64) return CALL(64, 64);                             \
  return CALL(64, 128);

extern "C" int sae_attention_fwd(const void *q, const void *k, const void *vt, const float *q_bias, const float *k_bias,
                                 const float *v_bias, int64_t n_batch, int64_t seq, int64_t n_heads, int64_t d_qk, int64_t d_v,
                                 double scale, void *out, float *lse, void *stream) {
  using namespace sae;
  SAE_REQUIRE(q && k && vt && out && lse, SAE_ERR_INVALID_ARG, "attention_fwd: null pointer");
  const int rc = check_shapes("attention_fwd", n_batch, seq, n_heads, d_qk, d_v);
  if (rc != SAE_OK) return rc;
#define ATT_FWD(A, B) launch_fwd<A, B>(q, k, vt, q_bias, k_bias, v_bias, n_batch, seq, n_heads, scale, out, lse, (hipStream_t)stream)
  ATT_DISPATCH(ATT_FWD)
#undef ATT_FWD
}

extern "C" int sae_attention_bwd(const void *q, const void *qt, const void *k, const void *kt, const void *v, const void *out,
                                 const void *dout, const void *doutt, const float *q_bias, const float *k_bias,
                                 const float *v_bias, const float *lse, int64_t n_batch, int64_t seq, int64_t n_heads,
                                 int64_t d_qk, int64_t d_v, double scale, float *dvec_workspace, void *dqt, void *dkt, void *dvt,
                                 void *stream) {
  using namespace sae;
  SAE_REQUIRE(q && qt && k && kt && v && out && dout && doutt && lse && dvec_workspace && dqt && dkt && dvt,
              SAE_ERR_INVALID_ARG, "attention_bwd: null pointer");
  const int rc = check_shapes("attention_bwd", n_batch, seq, n_heads, d_qk, d_v);
  if (rc != SAE_OK) return rc;
#define ATT_BWD(A, B)                                                                                                        \
  launch_bwd<A, B>(q, qt, k, kt, v, out, dout, doutt, q_bias, k_bias, v_bias, lse, n_batch, seq, n_heads, scale, dvec_workspace, \
                   dqt, dkt, dvt, (hipStream_t)stream)
  ATT_DISPATCH(ATT_BWD)
#undef ATT_BWD
}

extern "C" int sae_row_sum(const void *src, int src_dtype, int64_t rows, int64_t cols, float *out, void *stream) {
  using namespace sae;
  SAE_REQUIRE(src && out, SAE_ERR_INVALID_ARG, "row_sum: null pointer");
  SAE_REQUIRE(rows > 0 && cols > 0, SAE_ERR_INVALID_ARG, "row_sum: bad shape");
  SAE_REQUIRE(src_dtype == SAE_F32 || src_dtype == SAE_BF16, SAE_ERR_INVALID_ARG, "row_sum: bad dtype");
  const unsigned blocks = (unsigned)((rows + 3) / 4);
  if (src_dtype == SAE_BF16)
    hipLaunchKernelGGL(row_sum_kernel<true>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, src, out, rows, cols);
  else
    hipLaunchKernelGGL(row_sum_kernel<false>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, src, out, rows, cols);
  return check_launch("row_sum");
}
