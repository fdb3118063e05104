// Causal softmax attention with grouped value heads for gfx950 (bf16 operands, fp32 accumulation), forward and
// backward, on the matrix cores (v_mfma_f32_32x32x16_bf16).
//
// The mixing step of low-rank sparse attention: every query/key head h has d_qk-wide queries and keys and a
// d_v-wide value whose columns are d_v separate rank-1 value heads (dictionary features h * d_v .. (h + 1) * d_v - 1)
// that share head h's attention pattern.  out[b, s, h, :] = sum_{s' <= s} softmax_s'(scale * q[b,s,h] . k[b,s',h]) v[b,s',h,:].
//
// Layouts (bf16 unless noted; T = n_batch * seq tokens, token t = b * seq + s):
//   "natural"     [T, n_heads * width]   one token's heads side by side (what the projections x @ W produce),
//   "transposed"  [n_heads * width, T]   the same matrix transposed.
// Every operand is taken natural.  A matrix-core operand needs its contraction index in a lane's registers: the
// scores contract over the head width (a row of a q / k tile: an ordinary 16-byte LDS read), the mixing and the
// backward's accumulating products contract over positions (a column of a v / dout / q / k tile: ds_read_b64_tr_b16,
// the LDS read that hands a lane 4 consecutive rows of one column).  The gradients leave transposed, which is the
// layout in which they are the left operand of the weight-gradient product over the token axis.
//
// Fragment convention of the instruction (D = A B, 32 x 32 x 16): lane l supplies A[m = l % 32][8 consecutive k of
// half l / 32] and B[same k][n = l % 32], and receives D[m = 8 j + 4 (l / 32) + i][n = l % 32] in register 4 j + i
// (i, j < 4).  A workgroup is 4 waves; a wave owns 32 positions (queries in the forward and dQ kernels, keys in the
// dV and dK kernels) as the n index of every product, so that everything kept per position (running maximum and sum,
// log-sum-exp, the accumulators' rescaling) is per lane.  A 32 x 32 tile of probabilities leaves the score product as
// D (lane halves hold alternate groups of 4 positions of the contraction index of the next product); packed to bf16,
// two v_permlane32_swap per 16 positions hand each half the 8 consecutive positions the B operand wants.  No
// probability ever goes through LDS or HBM.
//
// Tiles of the streamed operand (64 positions per iteration) go from global memory straight into LDS
// (global_load_lds_dwordx4, two buffers: the loads of tile i + 1 are in flight while tile i is consumed; one
// workgroup barrier per tile).  Such a load writes 1 KiB linearly (lane l -> base + 16 l), so the bank swizzle is
// applied on the global side: a tile row holds its 16-byte chunk c at physical chunk c ^ key(row), with a key such that
// both access patterns cover 256 distinct bytes: 16 consecutive rows x one chunk (a fragment read along rows) and 4
// consecutive rows x 4 consecutive chunks (a transposing read across rows).
//
// Forward: one workgroup = 128 queries of one (batch, head), walking the key blocks 0 .. diagonal with the online
// softmax (running maximum and sum per query in fp32, log2 domain; the accumulators are rescaled only when some
// row's maximum has grown by more than 2^8, so probabilities are formed relative to a reference at most that far
// below the true maximum: exact in real arithmetic, and bf16 keeps its relative precision at any magnitude).
// Backward: dQ by a workgroup per 128 queries that walks the key blocks 0 .. diagonal; it is launched first and also
// leaves, for its own queries, D[q] = sum_dv dout * out and the log-sum-exp in the log2 domain, which dV and dK (each by
// a workgroup per 128 keys that walks the query blocks diagonal .. last) read per query.  All three recompute the
// probabilities from q, k and the saved log-sum-exp.  No atomics: results are reproducible.
//
// In the forward kernel a wave runs its score products and its exponentials / value products at raised priority
// (s_setprio) and its masking, running maximum and address arithmetic at the base one: of the waves that share a
// SIMD the one that can feed the matrix cores goes first (1-2 % in alternating runs; nothing measurable in the
// backward kernels, which do without).
//
// Positions past the end of a sequence (seq not a multiple of the block sizes): loads repeat the last valid row or
// 8-position piece, so every operand stays finite; their scores are masked (keys), zeroed (queries of the dV / dK
// kernels) or never stored.
#include "common.h"

namespace sae {

typedef __attribute__((ext_vector_type(8))) __bf16 att_bf16x8;
typedef __attribute__((ext_vector_type(16))) float att_f32x16;

constexpr int ATT_THREADS = 256;
constexpr int ATT_OWN = 128;        // positions owned by a workgroup: 4 waves of 32
constexpr int ATT_STEP = 64;        // positions of the streamed operand per iteration
constexpr float ATT_LOG2E = 1.4426950408889634f;
constexpr float ATT_RESCALE_STEP = 8.f;

#define ATT_WAITCNT_VM(N) (((N) & 0xf) | (0x7 << 4) | (0xf << 8) | (((N) >> 4) << 14))
#if defined(__HIP_DEVICE_COMPILE__)
// LDS[LDSADDR + 16 lane] = 16 bytes at SBASE + VOFF (scalar base, per-lane byte offset); LDSADDR is wave-uniform
#define ATT_DMA16(SBASE, VOFF, LDSADDR)                                                                        \
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(__builtin_amdgcn_readfirstlane(LDSADDR)), \
               "v"(VOFF), "s"(SBASE)                                                                           \
               : "memory")
#define ATT_DMA4(SBASE, VOFF, LDSADDR)                                                                         \
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(__builtin_amdgcn_readfirstlane(LDSADDR)),   \
               "v"(VOFF), "s"(SBASE)                                                                           \
               : "memory")
#else
#define ATT_DMA16(SBASE, VOFF, LDSADDR) ((void)0)
#define ATT_DMA4(SBASE, VOFF, LDSADDR) ((void)0)
#endif

__device__ __forceinline__ uint32_t att_pack2(float a, float b) {
  const cvt_f32x2 in = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(in, cvt_bf16x2));
}

// byte offset of logical chunk `chunk` of row `row` in a tile whose rows are RB bytes
// chunk permutation of a row: any 16 consecutive rows x one chunk, and any 4 consecutive rows (from a multiple of 4) x 4
// consecutive chunks (from a multiple of 4), cover 256 distinct bytes
template <int RB>
__device__ __forceinline__ int att_swz_key(int row) {
  if constexpr (RB == 64) return (row >> 2) & 3;
  else if constexpr (RB == 128) return (((row >> 1) & 1) << 2) | ((row >> 2) & 3);
  else return ((row & 3) << 2) | ((row >> 2) & 3);
}
template <int RB>
__device__ __forceinline__ int att_swz(int row, int chunk) {
  return row * RB + ((chunk ^ att_swz_key<RB>(row)) << 4);
}

// A operand: row `row` of a tile, contraction positions 16 st + 8 g .. + 7
template <int RB>
__device__ __forceinline__ att_bf16x8 att_frag(const char *tile, int row, int st, int g) {
  return *reinterpret_cast<const att_bf16x8 *>(tile + att_swz<RB>(row, 2 * st + g));
}

// A operand read ACROSS the rows of a natural tile: m = column col0 + lane % 32, contraction positions = rows
// 16 st + 8 g .. + 7.  ds_read_b64_tr_b16 hands lane j of a group of 16 element j % 4 of the 8-byte pieces that lanes
// 4 e + j / 4 (e < 4) point at; lane i therefore points at row 8 g + 4 hh + i / 4, columns 16 (group % 2) + 4 (i % 4) .. + 3.
// att_tr_addr gives the per-lane byte offset for (col0, hh) at st = 0; a step adds 16 RB bytes (the permutation key of
// a row does not depend on st).
typedef __attribute__((ext_vector_type(4))) short att_i16x4;
template <int RB>
__device__ __forceinline__ int att_tr_addr(int lane, int col0, int hh) {
  const int i = lane & 15, grp = lane >> 4;
  const int row = 8 * (grp >> 1) + 4 * hh + (i >> 2), col = col0 + 16 * (grp & 1) + 4 * (i & 3);
  return att_swz<RB>(row, col >> 3) + (col & 7) * 2;
}
__device__ __forceinline__ att_bf16x8 att_frag_tr(const char *tile, int addr0, int addr1, int step_bytes) {
  typedef __attribute__((address_space(3))) att_i16x4 *lds_i16x4;
  const att_i16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4)(tile + addr0 + step_bytes));
  const att_i16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4)(tile + addr1 + step_bytes));
  typedef __attribute__((ext_vector_type(8))) short i16x8;
  const i16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(att_bf16x8, v);
}

// Per-lane byte offsets of a wave's NL loads of a tile (wave-load wl = wave * NL + i covers 1 KiB of it).
// Natural tile: rows are consecutive tokens of a matrix with `ld` elements per token, RB bytes of each are taken;
// rows at or past `rows_valid` repeat row rows_valid - 1.
template <int RB, int NL>
__device__ __forceinline__ void att_nat_offsets(uint32_t (&off)[NL], int wave, int lane, int ld, int rows_valid) {
  constexpr int CPR = RB / 16, RPL = 1024 / RB;
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const int row = (wave * NL + i) * RPL + lane / CPR, ch = (lane % CPR) ^ att_swz_key<RB>(row);
    off[i] = (uint32_t)(min(row, rows_valid - 1) * ld + ch * 8) * 2u;
  }
}
template <int NL>
__device__ __forceinline__ void att_dma(const void *sbase, const uint32_t (&off)[NL], uint32_t lds_addr) {
#pragma unroll
  for (int i = 0; i < NL; ++i) ATT_DMA16(sbase, off[i], lds_addr + i * 1024);
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

__device__ __forceinline__ att_f32x16 att_mfma(const att_bf16x8 &a, const att_bf16x8 &b, const att_f32x16 &c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ att_f32x16 att_zero16() {
  att_f32x16 z;
#pragma unroll
  for (int i = 0; i < 16; ++i) z[i] = 0.f;
  return z;
}

__device__ __forceinline__ float att_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// both halves of the wave get max / sum of lane l and lane l ^ 32
__device__ __forceinline__ float att_half_max(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float att_half_sum(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// A lane's 16 values of a 32 x 32 tile (positions 8 j + 4 g + i of the tile's m index) -> the B operands of the two
// 16-position steps of a product that contracts over m: half g of step c gets positions 16 c + 8 g .. + 7.  The swap
// exchanges the upper half of its first operand with the lower half of its second.
__device__ __forceinline__ void att_to_b_operands(const uint32_t (&pk)[8], att_bf16x8 (&b)[2]) {
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    const auto w0 = __builtin_amdgcn_permlane32_swap(pk[4 * c], pk[4 * c + 2], false, false);
    const auto w1 = __builtin_amdgcn_permlane32_swap(pk[4 * c + 1], pk[4 * c + 3], false, false);
    u32x4 w;
    w.x = w0[0]; w.y = w1[0]; w.z = w0[1]; w.w = w1[1];
    b[c] = __builtin_bit_cast(att_bf16x8, w);
  }
}
__device__ __forceinline__ void att_pack16(const att_f32x16 &x, uint32_t (&pk)[8]) {
#pragma unroll
  for (int r = 0; r < 8; ++r) pk[r] = att_pack2(x[2 * r], x[2 * r + 1]);
}

// One token's row of a natural-layout matrix as the B operands of a lane (8 columns of half g per 16-column step).
template <int COLS>
__device__ __forceinline__ void att_row_operands(att_bf16x8 (&f)[COLS / 16], const uint16_t *__restrict__ row, int g) {
#pragma unroll
  for (int st = 0; st < COLS / 16; ++st) f[st] = *reinterpret_cast<const att_bf16x8 *>(row + st * 16 + g * 8);
}

// A wave's 32 x ROWS accumulator tile set (acc[n] = rows 32 n .. 32 n + 31, this lane's token) -> transposed layout
// dst[(row0 + row) * T + tok]
template <int ROWS>
__device__ __forceinline__ void att_store_transposed(uint16_t *__restrict__ dst, const att_f32x16 (&acc)[ROWS / 32], int row0, int64_t T,
                                                     int64_t tok, int g) {
#pragma unroll
  for (int n = 0; n < ROWS / 32; ++n)
#pragma unroll
    for (int r = 0; r < 16; ++r)
      dst[(int64_t)(row0 + n * 32 + 8 * (r >> 2) + 4 * g + (r & 3)) * T + tok] = (uint16_t)(att_pack2(acc[n][r], 0.f) & 0xffffu);
}

// ---- forward ---------------------------------------------------------------------------------------------
template <int DQK, int DV>
__global__ __launch_bounds__(ATT_THREADS, 3) void attn_fwd_kernel(
    const uint16_t *__restrict__ q, const uint16_t *__restrict__ k, const uint16_t *__restrict__ v, uint16_t *__restrict__ out,
    float *__restrict__ lse, int seq, int n_heads, int n_batch, float sc2) {
  constexpr int KRB = DQK * 2;                                    // bytes of a key row
  constexpr int VRB = DV * 2;
  constexpr int K_BYTES = ATT_STEP * KRB, V_BYTES = ATT_STEP * VRB, BUF = K_BYTES + V_BYTES;
  constexpr int KNL = K_BYTES / 4096, VNL = V_BYTES / 4096;      // loads per wave and tile
  constexpr int OP = DV * 2 + 16;                                 // staging row pitch of the epilogue
  constexpr int LDS_BYTES = 2 * BUF > 4 * 32 * OP ? 2 * BUF : 4 * 32 * OP;
  __shared__ __attribute__((aligned(1024))) char lds[LDS_BYTES];
  int qb, h, b;
  att_block_coords((seq + ATT_OWN - 1) / ATT_OWN, n_heads, n_batch, true, qb, h, b);     // long rows of work first
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), r32 = lane & 31, g = lane >> 5;
  const int64_t tok0 = (int64_t)b * seq;
  const int ldq = n_heads * DQK, ldv = n_heads * DV;
  const int wq0 = qb * ATT_OWN + wave * 32, q_row = wq0 + r32;

  att_bf16x8 qf[DQK / 16];
  att_row_operands<DQK>(qf, q + (tok0 + min(q_row, seq - 1)) * ldq + h * DQK, g);
  att_f32x16 o[DV / 32];
#pragma unroll
  for (int n = 0; n < DV / 32; ++n) o[n] = att_zero16();
  float m = -INFINITY, l = 0.f;

  typedef __attribute__((address_space(3))) void *lds_ptr_t;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
  const int n_kb = (min(seq, (qb + 1) * ATT_OWN) + ATT_STEP - 1) / ATT_STEP;
  uint32_t koff[KNL], voff[VNL];
  att_nat_offsets<KRB, KNL>(koff, wave, lane, ldq, ATT_STEP);
  att_nat_offsets<VRB, VNL>(voff, wave, lane, ldv, ATT_STEP);
  const uint16_t *kbase = k + tok0 * ldq + h * DQK, *vbase = v + tok0 * ldv + h * DV;
  auto issue = [&](int kb) {
    const uint32_t buf = lds_base + (uint32_t)(kb & 1) * BUF;
    const uint16_t *k_ = kbase + (int64_t)kb * ATT_STEP * ldq, *v_ = vbase + (int64_t)kb * ATT_STEP * ldv;
    const int rem = seq - kb * ATT_STEP;
    if (rem >= ATT_STEP) {
      att_dma<KNL>(k_, koff, buf + wave * KNL * 1024);
      att_dma<VNL>(v_, voff, buf + K_BYTES + wave * VNL * 1024);
    } else {
      uint32_t ko[KNL], vo[VNL];
      att_nat_offsets<KRB, KNL>(ko, wave, lane, ldq, rem);
      att_nat_offsets<VRB, VNL>(vo, wave, lane, ldv, rem);
      att_dma<KNL>(k_, ko, buf + wave * KNL * 1024);
      att_dma<VNL>(v_, vo, buf + K_BYTES + wave * VNL * 1024);
    }
  };
  int vaddr[DV / 32][2];
#pragma unroll
  for (int n = 0; n < DV / 32; ++n)
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) vaddr[n][hh] = att_tr_addr<VRB>(lane, n * 32, hh);
  issue(0);
  for (int kb = 0; kb < n_kb; ++kb) {
    __builtin_amdgcn_s_waitcnt(ATT_WAITCNT_VM(0));
    __syncthreads();                       // tile kb is in LDS; every wave is done with the other buffer
    if (kb + 1 < n_kb) issue(kb + 1);
    const int key0 = kb * ATT_STEP;
    if (key0 > wq0 + 31) continue;         // every key of this block lies after every query of this wave
    const char *sk = lds + (kb & 1) * BUF, *sv = sk + K_BYTES;
    att_f32x16 s[2];
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      s[t] = att_zero16();
#pragma unroll
      for (int st = 0; st < DQK / 16; ++st) s[t] = att_mfma(att_frag<KRB>(sk, t * 32 + r32, st, g), qf[st], s[t]);
    }
    __builtin_amdgcn_s_setprio(0);
    if (key0 + ATT_STEP - 1 > wq0) {       // some key of the block lies after some query of the wave
      const int thr = q_row - key0 - 4 * g;      // the lane's element at key offset 32 t + 8 j + i above this is masked
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[t][r] = (t * 32 + 8 * (r >> 2) + (r & 3) > thr) ? -INFINITY : s[t][r];
    }
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[t][r]);
    mx = att_half_max(mx);
    // key0 <= wq0 here (both are multiples of 32), so every row sees at least one key of the block and m_new is finite;
    // the scale is positive, so the maximum is taken over the raw scores and scaled once
    const float m_new = fmaxf(m, mx * sc2);
    if (__any(m_new > m + ATT_RESCALE_STEP)) {
      const float alpha = att_exp2(m - m_new);      // exp2(-inf) = 0 on the first block
      l *= alpha;
#pragma unroll
      for (int n = 0; n < DV / 32; ++n)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[n][r] *= alpha;
      m = m_new;
    }
    float rs = 0.f;
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      uint32_t pk[8];
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        const float p0 = att_exp2(fmaf(s[t][2 * r], sc2, -m)), p1 = att_exp2(fmaf(s[t][2 * r + 1], sc2, -m));
        rs += p0 + p1;
        pk[r] = att_pack2(p0, p1);
      }
      att_bf16x8 pb[2];
      att_to_b_operands(pk, pb);
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int n = 0; n < DV / 32; ++n) o[n] = att_mfma(att_frag_tr(sv, vaddr[n][0], vaddr[n][1], (2 * t + c) * 16 * VRB), pb[c], o[n]);
    }
    l += rs;
    __builtin_amdgcn_s_setprio(0);
  }
  l = att_half_sum(l);
  __syncthreads();                         // the tile buffers become the staging area of the epilogue
  const float inv = 1.f / l;
  char *so = lds + wave * 32 * OP;
#pragma unroll
  for (int n = 0; n < DV / 32; ++n)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint2 pkv;
      pkv.x = att_pack2(o[n][4 * j] * inv, o[n][4 * j + 1] * inv);
      pkv.y = att_pack2(o[n][4 * j + 2] * inv, o[n][4 * j + 3] * inv);
      *reinterpret_cast<uint2 *>(so + r32 * OP + (n * 32 + 8 * j + 4 * g) * 2) = pkv;
    }
  constexpr int CH = DV / 8, ROWS_PER_PASS = 64 / CH;   // whole rows of the output leave as 16-byte pieces
#pragma unroll
  for (int ps = 0; ps < 32 / ROWS_PER_PASS; ++ps) {
    const int row = ps * ROWS_PER_PASS + lane / CH, cc = lane % CH;
    const u32x4 v = *reinterpret_cast<const u32x4 *>(so + row * OP + cc * 16);
    if (wq0 + row < seq) *reinterpret_cast<u32x4 *>(out + (tok0 + wq0 + row) * ldv + h * DV + cc * 8) = v;
  }
  if (q_row < seq && g == 0) lse[((int64_t)b * n_heads + h) * seq + q_row] = (m + __log2f(l)) * 0.6931471805599453f;
}

// ---- backward: dV^T and dK^T (one workgroup per 128 keys, a wave per 32) -----------------------------------------------
// P[q, key] = exp2(sc2 * q . k - lse2[q]) for q >= key.
// WHAT = 0: dV^T[dv, key] = sum_q dout^T[dv, q] P[q, key].
// WHAT = 1: dK^T[c, key] = sum_q q^T[c, q] dS[q, key],  dS = P (dP - D) scale,  dP[q, key] = dout[q, :] . v[key, :].
// (One kernel for both would hold both accumulators, both register-resident rows and four streamed tiles: one wave per
// SIMD, which waits on its own barriers.)
template <int DQK, int DV, int WHAT>
__global__ __launch_bounds__(ATT_THREADS, WHAT == 0 ? 3 : 2) void attn_bwd_dkv_kernel(
    const uint16_t *__restrict__ q, const uint16_t *__restrict__ k, const uint16_t *__restrict__ v,
    const uint16_t *__restrict__ dout, const float *__restrict__ lse2,
    const float *__restrict__ dvec, uint16_t *__restrict__ dst, int seq, int n_heads, int n_batch, int64_t T, float sc2, float scale) {
  constexpr bool DK = WHAT == 1;
  constexpr int QRB = DQK * 2, ORB = DV * 2;
  constexpr int Q_BYTES = ATT_STEP * QRB, O_BYTES = ATT_STEP * ORB;    // the streamed tiles: 64 queries' q and dout rows
  constexpr int VEC_BYTES = 512;                                       // 64 x (lse2, D)
  constexpr int BUF = Q_BYTES + O_BYTES + VEC_BYTES;
  constexpr int QNL = Q_BYTES / 4096, ONL = O_BYTES / 4096;
  constexpr int ACC = DK ? DQK : DV;                                   // rows of the accumulated matrix
  constexpr int ARB = DK ? QRB : ORB;                                  // row bytes of the tile the accumulating product reads across
  __shared__ __attribute__((aligned(1024))) char lds[2 * BUF];
  const int n_qb = (seq + ATT_STEP - 1) / ATT_STEP;
  int kb, h, b;
  att_block_coords((seq + ATT_OWN - 1) / ATT_OWN, n_heads, n_batch, false, kb, h, b);     // key block 0 walks every query block: first
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), r32 = lane & 31, g = lane >> 5;
  const int64_t tok0 = (int64_t)b * seq;
  const int ldq = n_heads * DQK, ldv = n_heads * DV;
  const int wk0 = kb * ATT_OWN + wave * 32, key = wk0 + r32;

  att_bf16x8 kf[DQK / 16], vf[DK ? DV / 16 : 1];
  att_row_operands<DQK>(kf, k + (tok0 + min(key, seq - 1)) * ldq + h * DQK, g);
  if constexpr (DK) att_row_operands<DV>(vf, v + (tok0 + min(key, seq - 1)) * ldv + h * DV, g);
  att_f32x16 acc[ACC / 32];
#pragma unroll
  for (int n = 0; n < ACC / 32; ++n) acc[n] = att_zero16();

  typedef __attribute__((address_space(3))) void *lds_ptr_t;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
  uint32_t qoff[QNL], ooff[ONL];
  att_nat_offsets<QRB, QNL>(qoff, wave, lane, ldq, ATT_STEP);
  att_nat_offsets<ORB, ONL>(ooff, wave, lane, ldv, ATT_STEP);
  int aaddr[ACC / 32][2];
#pragma unroll
  for (int n = 0; n < ACC / 32; ++n)
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) aaddr[n][hh] = att_tr_addr<ARB>(lane, n * 32, hh);
  const uint16_t *qbase = q + tok0 * ldq + h * DQK;
  const uint16_t *obase = dout + tok0 * ldv + h * DV;
  const float *lbase = lse2 + ((int64_t)b * n_heads + h) * seq, *dbase = dvec + ((int64_t)b * n_heads + h) * seq;
  auto issue = [&](int qb, int slot) {
    const uint32_t buf = lds_base + (uint32_t)slot * BUF;
    const int q0 = qb * ATT_STEP, rem = seq - q0;
    const uint16_t *q_ = qbase + (int64_t)q0 * ldq, *o_ = obase + (int64_t)q0 * ldv;
    if (rem >= ATT_STEP) {
      att_dma<QNL>(q_, qoff, buf + wave * QNL * 1024);
      att_dma<ONL>(o_, ooff, buf + Q_BYTES + wave * ONL * 1024);
    } else {
      uint32_t qo[QNL], oo[ONL];
      att_nat_offsets<QRB, QNL>(qo, wave, lane, ldq, rem);
      att_nat_offsets<ORB, ONL>(oo, wave, lane, ldv, rem);
      att_dma<QNL>(q_, qo, buf + wave * QNL * 1024);
      att_dma<ONL>(o_, oo, buf + Q_BYTES + wave * ONL * 1024);
    }
    // the 64 queries' log-sum-exp (wave 0) and D (wave 1, dK only): 4 bytes per lane
    const uint32_t voff = (uint32_t)min(lane, rem - 1) * 4u;
    if (wave == 0) ATT_DMA4(lbase + q0, voff, buf + Q_BYTES + O_BYTES);
    if (DK && wave == 1) ATT_DMA4(dbase + q0, voff, buf + Q_BYTES + O_BYTES + 256);
  };
  const int qb0 = kb * (ATT_OWN / ATT_STEP);
  if (qb0 < n_qb) issue(qb0, 0);
  for (int qb = qb0; qb < n_qb; ++qb) {
    const int slot = (qb - qb0) & 1;
    __builtin_amdgcn_s_waitcnt(ATT_WAITCNT_VM(0));
    __syncthreads();                       // tile qb is in LDS; every wave is done with the other buffer
    if (qb + 1 < n_qb) issue(qb + 1, slot ^ 1);
    const int q0 = qb * ATT_STEP;
    if (q0 + ATT_STEP - 1 < wk0) continue; // every query of this block lies before every key of this wave
    const char *sq = lds + slot * BUF, *so = sq + Q_BYTES, *sa = DK ? sq : so;
    const float *svec = reinterpret_cast<const float *>(so + O_BYTES);
    const bool diag = q0 < wk0 + 31;       // some query of the block lies before some key of the wave
    const bool tail = q0 + ATT_STEP > seq; // some query of the block lies past the sequence
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      att_f32x16 s = att_zero16();
#pragma unroll
      for (int st = 0; st < DQK / 16; ++st) s = att_mfma(att_frag<QRB>(sq, t * 32 + r32, st, g), kf[st], s);
      att_f32x16 x;                        // P (dV) or dS (dK) of this lane's key and 16 of the tile's queries
      if constexpr (DK) {
        att_f32x16 dp = att_zero16();
#pragma unroll
        for (int st = 0; st < DV / 16; ++st) dp = att_mfma(att_frag<ORB>(so, t * 32 + r32, st, g), vf[st], dp);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float4 l4 = *reinterpret_cast<const float4 *>(svec + t * 32 + 8 * j + 4 * g);
          const float4 d4 = *reinterpret_cast<const float4 *>(svec + 64 + t * 32 + 8 * j + 4 * g);
          const float lj[4] = {l4.x, l4.y, l4.z, l4.w}, dj[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
          for (int i = 0; i < 4; ++i) x[4 * j + i] = att_exp2(fmaf(s[4 * j + i], sc2, -lj[i])) * ((dp[4 * j + i] - dj[i]) * scale);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float4 l4 = *reinterpret_cast<const float4 *>(svec + t * 32 + 8 * j + 4 * g);
          const float lj[4] = {l4.x, l4.y, l4.z, l4.w};
#pragma unroll
          for (int i = 0; i < 4; ++i) x[4 * j + i] = att_exp2(fmaf(s[4 * j + i], sc2, -lj[i]));
        }
      }
      if (diag || tail) {
        // query offset 32 t + 8 j + 4 g + i: before the key -> 0; at or past the end of the sequence -> 0
        const int lo = key - q0 - 4 * g, hi = seq - q0 - 4 * g;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int qo = t * 32 + 8 * (r >> 2) + (r & 3);
          x[r] = (qo < lo || qo >= hi) ? 0.f : x[r];
        }
      }
      uint32_t pk[8];
      att_pack16(x, pk);
      att_bf16x8 xb[2];
      att_to_b_operands(pk, xb);
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int n = 0; n < ACC / 32; ++n) acc[n] = att_mfma(att_frag_tr(sa, aaddr[n][0], aaddr[n][1], (2 * t + c) * 16 * ARB), xb[c], acc[n]);
    }
  }
  if (key < seq) att_store_transposed<ACC>(dst, acc, h * ACC, T, tok0 + key, g);
}

// ---- backward: dQ^T (one workgroup per 128 queries, a wave per 32) -------------------------------------------------------
// dQ^T[c, q] = sum_key k^T[c, key] dS[q, key] over key <= q.
// The kernel also forms, for its own queries, what the other two backward kernels read per query: D = sum_dv dout * out (from
// the rows it holds anyway: each half of the wave has half of a row) and the log-sum-exp in the log2 domain, written to
// dvec / lse2 [n_batch, n_heads, seq].  It is therefore launched first.
template <int DQK, int DV>
__global__ __launch_bounds__(ATT_THREADS, 2) void attn_bwd_dq_kernel(
    const uint16_t *__restrict__ q, const uint16_t *__restrict__ k, const uint16_t *__restrict__ v,
    const uint16_t *__restrict__ out, const uint16_t *__restrict__ dout, const float *__restrict__ lse, float *__restrict__ lse2,
    float *__restrict__ dvec, uint16_t *__restrict__ dqt, int seq, int n_heads, int n_batch, int64_t T, float sc2, float scale) {
  constexpr int KRB = DQK * 2, VRB = DV * 2;
  constexpr int K_BYTES = ATT_STEP * KRB, V_BYTES = ATT_STEP * VRB, BUF = K_BYTES + V_BYTES;
  constexpr int KNL = K_BYTES / 4096, VNL = V_BYTES / 4096;
  __shared__ __attribute__((aligned(1024))) char lds[2 * BUF];
  int qb, h, b;
  att_block_coords((seq + ATT_OWN - 1) / ATT_OWN, n_heads, n_batch, true, qb, h, b);
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), r32 = lane & 31, g = lane >> 5;
  const int64_t tok0 = (int64_t)b * seq;
  const int ldq = n_heads * DQK, ldv = n_heads * DV;
  const int wq0 = qb * ATT_OWN + wave * 32, q_row = wq0 + r32, q_ld = min(q_row, seq - 1);

  att_bf16x8 qf[DQK / 16], dof[DV / 16];
  att_row_operands<DQK>(qf, q + (tok0 + q_ld) * ldq + h * DQK, g);
  att_row_operands<DV>(dof, dout + (tok0 + q_ld) * ldv + h * DV, g);
  const int64_t at = ((int64_t)b * n_heads + h) * seq + q_ld;
  const float l2 = lse[at] * ATT_LOG2E;
  float dsum = 0.f;
  {
    const uint16_t *orow = out + (tok0 + q_ld) * ldv + h * DV;
#pragma unroll
    for (int st = 0; st < DV / 16; ++st) {
      const u32x4 o4 = *reinterpret_cast<const u32x4 *>(orow + st * 16 + g * 8), a4 = __builtin_bit_cast(u32x4, dof[st]);
      const uint32_t ow[4] = {o4.x, o4.y, o4.z, o4.w}, aw[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        dsum = fmaf(__uint_as_float(aw[j] << 16), __uint_as_float(ow[j] << 16), dsum);
        dsum = fmaf(__uint_as_float(aw[j] & 0xffff0000u), __uint_as_float(ow[j] & 0xffff0000u), dsum);
      }
    }
    dsum = att_half_sum(dsum);
    if (q_row < seq && g == 0) {
      lse2[at] = l2;
      dvec[at] = dsum;
    }
  }
  att_f32x16 dq[DQK / 32];
#pragma unroll
  for (int n = 0; n < DQK / 32; ++n) dq[n] = att_zero16();

  typedef __attribute__((address_space(3))) void *lds_ptr_t;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
  const int n_kb = (min(seq, (qb + 1) * ATT_OWN) + ATT_STEP - 1) / ATT_STEP;
  uint32_t koff[KNL], voff[VNL];
  att_nat_offsets<KRB, KNL>(koff, wave, lane, ldq, ATT_STEP);
  att_nat_offsets<VRB, VNL>(voff, wave, lane, ldv, ATT_STEP);
  int kaddr[DQK / 32][2];
#pragma unroll
  for (int n = 0; n < DQK / 32; ++n)
#pragma unroll
    for (int hh = 0; hh < 2; ++hh) kaddr[n][hh] = att_tr_addr<KRB>(lane, n * 32, hh);
  const uint16_t *kbase = k + tok0 * ldq + h * DQK, *vbase = v + tok0 * ldv + h * DV;
  auto issue = [&](int kb) {
    const uint32_t buf = lds_base + (uint32_t)(kb & 1) * BUF;
    const int key0 = kb * ATT_STEP, rem = seq - key0;
    const uint16_t *k_ = kbase + (int64_t)key0 * ldq, *v_ = vbase + (int64_t)key0 * ldv;
    if (rem >= ATT_STEP) {
      att_dma<KNL>(k_, koff, buf + wave * KNL * 1024);
      att_dma<VNL>(v_, voff, buf + K_BYTES + wave * VNL * 1024);
    } else {
      uint32_t ko[KNL], vo[VNL];
      att_nat_offsets<KRB, KNL>(ko, wave, lane, ldq, rem);
      att_nat_offsets<VRB, VNL>(vo, wave, lane, ldv, rem);
      att_dma<KNL>(k_, ko, buf + wave * KNL * 1024);
      att_dma<VNL>(v_, vo, buf + K_BYTES + wave * VNL * 1024);
    }
  };
  issue(0);
  for (int kb = 0; kb < n_kb; ++kb) {
    __builtin_amdgcn_s_waitcnt(ATT_WAITCNT_VM(0));
    __syncthreads();
    if (kb + 1 < n_kb) issue(kb + 1);
    const int key0 = kb * ATT_STEP;
    if (key0 > wq0 + 31) continue;         // every key of this block lies after every query of this wave
    const char *sk = lds + (kb & 1) * BUF, *sv = sk + K_BYTES;
    const bool diag = key0 + ATT_STEP - 1 > wq0;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      att_f32x16 s = att_zero16(), dp = att_zero16();
#pragma unroll
      for (int st = 0; st < DQK / 16; ++st) s = att_mfma(att_frag<KRB>(sk, t * 32 + r32, st, g), qf[st], s);
#pragma unroll
      for (int st = 0; st < DV / 16; ++st) dp = att_mfma(att_frag<VRB>(sv, t * 32 + r32, st, g), dof[st], dp);
      att_f32x16 ds;
#pragma unroll
      for (int r = 0; r < 16; ++r) ds[r] = att_exp2(fmaf(s[r], sc2, -l2)) * ((dp[r] - dsum) * scale);
      if (diag) {
        const int thr = q_row - key0 - 4 * g;
#pragma unroll
        for (int r = 0; r < 16; ++r) ds[r] = (t * 32 + 8 * (r >> 2) + (r & 3) > thr) ? 0.f : ds[r];
      }
      uint32_t pk[8];
      att_pack16(ds, pk);
      att_bf16x8 db[2];
      att_to_b_operands(pk, db);
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int n = 0; n < DQK / 32; ++n) dq[n] = att_mfma(att_frag_tr(sk, kaddr[n][0], kaddr[n][1], (2 * t + c) * 16 * KRB), db[c], dq[n]);
    }
  }
  if (q_row < seq) att_store_transposed<DQK>(dqt, dq, h * DQK, T, tok0 + q_row, g);
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
static int launch_fwd(const void *q, const void *k, const void *v, int64_t n_batch, int64_t seq, int64_t n_heads, double scale,
                      void *out, float *lse, hipStream_t st) {
  const dim3 grid((unsigned)(((seq + ATT_OWN - 1) / ATT_OWN) * n_heads * n_batch));
  hipLaunchKernelGGL((attn_fwd_kernel<DQK, DV>), grid, dim3(ATT_THREADS), 0, st, (const uint16_t *)q, (const uint16_t *)k,
                     (const uint16_t *)v, (uint16_t *)out, lse, (int)seq, (int)n_heads, (int)n_batch,
                     (float)(scale * 1.4426950408889634));
  return check_launch("attention_fwd");
}

template <int DQK, int DV>
static int launch_bwd(const void *q, const void *k, const void *v, const void *out, const void *dout, const float *lse,
                      int64_t n_batch, int64_t seq, int64_t n_heads, double scale, float *workspace, void *dqt, void *dkt,
                      void *dvt, hipStream_t st) {
  const int64_t T = n_batch * seq;
  const dim3 grid((unsigned)(((seq + ATT_OWN - 1) / ATT_OWN) * n_heads * n_batch));
  const float sc2 = (float)(scale * 1.4426950408889634);
  float *dvec = workspace, *lse2 = workspace + n_batch * n_heads * seq;
  // dQ first: it leaves D and the log2-domain log-sum-exp of every query for the two key-side kernels
  hipLaunchKernelGGL((attn_bwd_dq_kernel<DQK, DV>), grid, dim3(ATT_THREADS), 0, st, (const uint16_t *)q, (const uint16_t *)k,
                     (const uint16_t *)v, (const uint16_t *)out, (const uint16_t *)dout, lse, lse2, dvec, (uint16_t *)dqt, (int)seq,
                     (int)n_heads, (int)n_batch, T, sc2, (float)scale);
  hipLaunchKernelGGL((attn_bwd_dkv_kernel<DQK, DV, 0>), grid, dim3(ATT_THREADS), 0, st, (const uint16_t *)q, (const uint16_t *)k,
                     (const uint16_t *)v, (const uint16_t *)dout, lse2, dvec, (uint16_t *)dvt, (int)seq, (int)n_heads,
                     (int)n_batch, T, sc2, (float)scale);
  hipLaunchKernelGGL((attn_bwd_dkv_kernel<DQK, DV, 1>), grid, dim3(ATT_THREADS), 0, st, (const uint16_t *)q, (const uint16_t *)k,
                     (const uint16_t *)v, (const uint16_t *)dout, lse2, dvec, (uint16_t *)dkt, (int)seq, (int)n_heads,
                     (int)n_batch, T, sc2, (float)scale);
  return check_launch("attention_bwd");
}

static int check_shapes(const char *what, int64_t n_batch, int64_t seq, int64_t n_heads, int64_t d_qk, int64_t d_v) {
  SAE_REQUIRE(n_batch > 0 && seq > 0 && n_heads > 0, SAE_ERR_INVALID_ARG, "%s: sizes must be positive", what);
  SAE_REQUIRE(((seq + ATT_OWN - 1) / ATT_OWN) * n_heads * n_batch < ((int64_t)1 << 31), SAE_ERR_UNSUPPORTED,
              "%s: too many (block, head, sequence) workgroups", what);
  SAE_REQUIRE(seq % 8 == 0, SAE_ERR_UNSUPPORTED, "%s: seq = %lld must be a multiple of 8 (16-byte pieces of the transposed operands)",
              what, (long long)seq);
  SAE_REQUIRE((d_qk == 32 || d_qk == 64) && (d_v == 32 || d_v == 64 || d_v == 128), SAE_ERR_UNSUPPORTED,
              "%s: built for d_qk in {32, 64} and d_v in {32, 64, 128}, got %lld / %lld", what, (long long)d_qk, (long long)d_v);
  // a tile's per-lane offsets are 32-bit byte offsets from the tile's first element
  SAE_REQUIRE(n_batch * seq * 128 * 2 < ((int64_t)1 << 32) && n_heads * 128 * 64 * 2 < ((int64_t)1 << 32), SAE_ERR_UNSUPPORTED,
              "%s: more than 2^24 tokens or 2^18 heads", what);
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

extern "C" int sae_attention_fwd(const void *q, const void *k, const void *v, int64_t n_batch, int64_t seq, int64_t n_heads,
                                 int64_t d_qk, int64_t d_v, double scale, void *out, float *lse, void *stream) {
  using namespace sae;
  SAE_REQUIRE(q && k && v && out && lse, SAE_ERR_INVALID_ARG, "attention_fwd: null pointer");
  const int rc = check_shapes("attention_fwd", n_batch, seq, n_heads, d_qk, d_v);
  if (rc != SAE_OK) return rc;
#define ATT_FWD(A, B) launch_fwd<A, B>(q, k, v, n_batch, seq, n_heads, scale, out, lse, (hipStream_t)stream)
  ATT_DISPATCH(ATT_FWD)
#undef ATT_FWD
}

extern "C" int sae_attention_bwd(const void *q, const void *k, const void *v, const void *out, const void *dout, const float *lse,
                                 int64_t n_batch, int64_t seq, int64_t n_heads, int64_t d_qk, int64_t d_v, double scale,
                                 float *workspace, void *dqt, void *dkt, void *dvt, void *stream) {
  using namespace sae;
  SAE_REQUIRE(q && k && v && out && dout && lse && workspace && dqt && dkt && dvt, SAE_ERR_INVALID_ARG,
              "attention_bwd: null pointer");
  const int rc = check_shapes("attention_bwd", n_batch, seq, n_heads, d_qk, d_v);
  if (rc != SAE_OK) return rc;
#define ATT_BWD(A, B) \
  launch_bwd<A, B>(q, k, v, out, dout, lse, n_batch, seq, n_heads, scale, workspace, dqt, dkt, dvt, (hipStream_t)stream)
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
