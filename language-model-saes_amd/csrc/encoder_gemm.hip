// Encoder pre-activation GEMM for gfx950:  pre[B, F] = x[B, d] * W_E^T[F, d]^T.
//
// Both operands are K-contiguous ("NT" GEMM), so a 16-byte piece of a row is exactly the 8 bf16
// (or 4 fp32) one lane feeds to a matrix-core instruction.
//
// Tiling: one workgroup of 512 threads (8 waves of 64, two per SIMD) owns a 256-token x 256-feature tile and
// walks K in slabs of 128 bytes per row (64 bf16 / 32 fp32): a full cache line per row, which the
// L2 serves at twice the rate of half lines (measured 27 vs 13 TB/s aggregate L2->LDS).  Waves are
// arranged 2 x 4: each owns 128 tokens x 64 features (128 fp32 accumulators per lane): 8 x 4 tiles of
// v_mfma_f32_16x16x32_bf16 for bf16 operands (two k-steps of 64 bytes per slab, a quarter wave per
// 16-byte chunk), 4 x 2 tiles of v_mfma_f32_32x32x2f32 for fp32 operands.
//
// LDS (all 160 KiB of the CU) is a ring of five 32 KiB slots; a slot holds one operand's
// slab (256 rows x 128 bytes).  Load units alternate W slab j, x slab j, W slab j+1, ...; unit t
// lives in slot t % 5.  Slots are filled by LDS-direct loads (global_load_lds_dwordx4: the data
// never passes through VGPRs), issued through inline assembly so that the compiler's wait-count
// insertion does not serialise them against LDS reads of other slots.  While slab j is consumed, x slab j+1
// and W slab j+2 are in flight: the weights, which come from HBM, get the longer lead; the activations
// mostly hit L2 / Infinity Cache.
//
// bf16 operands, the schedule ("ping-pong"): the four waves that own tokens 0-127 of the tile (one per SIMD) and
// the four that own tokens 128-255 alternate between a memory phase -- the 12 fragment reads of one k-step from
// LDS plus 4 LDS-direct loads of 1 KiB -- and a matrix-core phase -- the k-step's 32 instructions.  A workgroup
// barrier ends every phase and the second group runs one phase behind the first, so on every SIMD one wave
// feeds the matrix cores while the other waits on LDS.  With all eight waves in the same phase (one barrier per
// slab, loads and fragment reads interleaved with the matrix-core instructions by the compiler) the matrix cores
// were busy 60 % of the cycles and each ingredient added its own time; with the phases they are busy 77 %
// (3.49 -> 3.05 ms at B = d = 4096, F = 131072 on random operands).  What remains is the engine clock: it falls
// as the matrix cores get busier (2.0 -> 1.8 GHz), the card is at its power limit.
// A slab is read in phases 4j .. 4j+3 (phase numbers of the early group; the late group's step s runs in phase
// 4j+s+1).  Early waves issue their quarter of x slab j+1 in phase 4j and of W slab j+2 in phase 4j+2, late
// waves theirs in phases 4j+1 and 4j+3, into the slots slab j-1 left; every wave waits for all but its 4
// youngest loads at the end of phase 4j+3, and the barrier that ends that phase publishes slab j+1.
// fp32 operands keep the older schedule (one barrier per slab, four sub-phases, all waves in step): their
// matrix-core time per byte is 16 times longer and hides everything else.
//
// LDS layout: row r of a slot is 128 bytes = 8 chunks of 16 bytes; chunk c is stored at physical
// chunk c ^ ((r >> 1) & 7).  A group of 16 lanes then covers 256 distinct bytes when MFMA
// fragments are read (16 rows, one logical chunk): no bank conflicts (SQ_LDS_BANK_CONFLICT = 0).
// An LDS-direct load writes 1 KiB linearly (lane l -> base + 16 l), so the swizzle is applied on
// the global side: lane l fetches the logical chunk that belongs at its physical slot.
//
// The matrix cores compute D = Wtile * xtile^T (features along the "rows" of the instruction),
// which leaves every lane holding 4 consecutive features of one token.  For bf16 output a full tile is
// transposed through LDS, wave by wave, and leaves as whole 128-byte lines; edge tiles and fp32 output
// store each lane's 4 features directly (8 or 16 bytes).
//
// Workgroup order: consecutive ids land on the 8 XCDs round-robin; within an XCD, 32 consecutive
// workgroups (one per CU) cover RM token tiles x 32 / RM feature tiles, so every slab in an XCD's L2 is
// shared by the resident workgroups (bf16: RM = 8 when there are at least 8 token tiles, 3.05 against 3.09 ms
// for RM = 4 and 3.3 for RM = 2; fp32: RM = 4).  The feature tiles are the dimension dealt to the XCDs, unless there are
// fewer than 8 of them and more token tiles than that: then the token tiles are dealt and an XCD's 32 workgroups cover
// all feature tiles of 32 / (feature tiles) token tiles (a 768-feature product would otherwise run on 3 XCDs).
//
// Rows beyond B or F are clamped to the last valid row when loading (their products land in
// accumulators that the epilogue never stores), so the main loop has no bounds checks.
#include "common.h"

namespace sae {

#define WAITCNT_VM4 ((4 & 0xf) | (0x7 << 4) | (0xf << 8) | ((4 >> 4) << 14))

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

constexpr int GEMM_BM = 256;       // tokens per workgroup tile
constexpr int GEMM_BN = 256;       // features per workgroup tile
constexpr int GEMM_SLAB = 128;     // bytes of K per row per slab
constexpr int GEMM_SLOTS = 5;      // ring of 32 KiB slots, each holding one operand's slab
constexpr int GEMM_THREADS = 512;
constexpr int GEMM_SLOT_BYTES = 256 * GEMM_SLAB;
constexpr int GEMM_LDS_BYTES = GEMM_SLOTS * GEMM_SLOT_BYTES;

__device__ __forceinline__ int swz(int row, int chunk) { return row * GEMM_SLAB + ((chunk ^ ((row >> 1) & 7)) << 4); }

// one 16-byte chunk of K (4 fp32) of a 32 x 32 tile
__device__ __forceinline__ void mma_chunk_f32(const u32x4 &wf, const u32x4 &xf, f32x16_t &acc) {
  f32x4_t a = __builtin_bit_cast(f32x4_t, wf);
  f32x4_t b = __builtin_bit_cast(f32x4_t, xf);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[0], b[0], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[1], b[1], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[2], b[2], acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[3], b[3], acc, 0, 0, 0);
}

// ---- fp32 operands ---------------------------------------------------------------------------------------------
template <bool BF16_OUT>
__global__ __launch_bounds__(GEMM_THREADS) void encoder_gemm_f32_kernel(
    const char *__restrict__ x, const char *__restrict__ w, void *__restrict__ out, int M, int N,
    int row_bytes /* d * 4 */, int tiles_m, int tiles_n) {
  extern __shared__ __attribute__((aligned(16))) char lds[];   // the ring of GEMM_SLOTS operand slabs

  // ---- XCD-aware tile assignment ----
  const int bid = blockIdx.x;
  int tile_m, tile_n;
  {
    const int xcd = bid & 7, slot = bid >> 3;
    // per XCD: groups of 32 consecutive workgroups cover 4 token tiles x 8 feature tiles
    const int grp = slot >> 5, in = slot & 31;
    const int m_groups = (tiles_m + 3) >> 2;           // groups of 4 token tiles (last one may be partial)
    const int n_grp = grp / m_groups, m_half = grp % m_groups;
    tile_m = m_half * 4 + (in & 3);
    tile_n = (n_grp * 8 + (in >> 2)) * 8 + xcd;
    if (tile_n >= tiles_n || tile_m >= tiles_m) return;
  }
  const int m0 = tile_m * GEMM_BM, n0 = tile_n * GEMM_BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 2, wn = wave & 3;

  // ---- global -> LDS staging assignment: 8 lanes cover one 128-byte row slab ----
  const int ld_phys = lane & 7;  // physical 16-byte chunk this lane fills
  const char *xg[4];
  const char *wg[4];
  bool xok[4], wok[4];
  int lds_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = wave * 32 + i * 8 + (lane >> 3);
    const int ld_chunk = ld_phys ^ ((r >> 1) & 7);  // logical chunk that lives at this physical slot
    xok[i] = (m0 + r) < M;
    wok[i] = (n0 + r) < N;
    xg[i] = x + (size_t)(xok[i] ? (m0 + r) : (M - 1)) * row_bytes + ld_chunk * 16;
    wg[i] = w + (size_t)(wok[i] ? (n0 + r) : (N - 1)) * row_bytes + ld_chunk * 16;
    lds_off[i] = (wave * 32 + i * 8) * GEMM_SLAB;  // wave-uniform base of the 1 KiB this load fills
  }

  f32x16_t acc[2][4];  // [feature sub-tile of 32][token sub-tile of 32]
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int n_slabs = row_bytes / GEMM_SLAB;
  typedef __attribute__((address_space(3))) void *lds_ptr_t;
  typedef const __attribute__((address_space(1))) void *glb_ptr_t;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
#if defined(__HIP_DEVICE_COMPILE__)
#define LDS_DMA16(GPTR, LDSADDR)                                                          \
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(__builtin_amdgcn_readfirstlane(LDSADDR)), "v"(GPTR) : "memory")
#else
#define LDS_DMA16(GPTR, LDSADDR) ((void)0)
#endif
  // unit t of the load sequence: t even -> W slab t/2, t odd -> x slab (t-1)/2; it lives in slot t % 5
#define LOAD_UNIT(T)                                                                                     \
  {                                                                                                      \
    const int t_ = (T);                                                                                  \
    int slab_ = t_ >> 1;                                                                                 \
    slab_ = slab_ < n_slabs ? slab_ : n_slabs - 1; /* tail: harmless re-read */                          \
    const uint32_t slot_ = lds_base + (uint32_t)(t_ % GEMM_SLOTS) * GEMM_SLOT_BYTES;                     \
    if (t_ & 1) {                                                                                        \
      _Pragma("unroll") for (int i = 0; i < 4; ++i) LDS_DMA16(xg[i] + (size_t)slab_ * GEMM_SLAB, slot_ + lds_off[i]); \
    } else {                                                                                             \
      _Pragma("unroll") for (int i = 0; i < 4; ++i) LDS_DMA16(wg[i] + (size_t)slab_ * GEMM_SLAB, slot_ + lds_off[i]); \
    }                                                                                                    \
  }
  // prologue: W0 x0 W1 x1 W2 in flight
  LOAD_UNIT(0) LOAD_UNIT(1) LOAD_UNIT(2) LOAD_UNIT(3) LOAD_UNIT(4)

  const int frag_row = lane & 31, frag_half = lane >> 5;
  for (int slab = 0; slab < n_slabs; ++slab) {
    // units 2*slab and 2*slab+1 must have landed; at most one younger unit (4 loads) may be outstanding
    __builtin_amdgcn_s_waitcnt(WAITCNT_VM4);
    __builtin_amdgcn_s_barrier();  // everyone's part landed; everyone is done with the previous slab's two slots
    // units issued while this slab is consumed: x slab+1 -> slot freed by W slab-1, W slab+2 -> slot freed by
    // x slab-1.  Two of the eight loads per phase, so that requests trickle instead of bursting.
    const int tA = 2 * slab + 3, tB = 2 * slab + 4;
    int sA = tA >> 1; sA = sA < n_slabs ? sA : n_slabs - 1;
    int sB = tB >> 1; sB = sB < n_slabs ? sB : n_slabs - 1;
    const uint32_t slotA = lds_base + (uint32_t)(tA % GEMM_SLOTS) * GEMM_SLOT_BYTES;
    const uint32_t slotB = lds_base + (uint32_t)(tB % GEMM_SLOTS) * GEMM_SLOT_BYTES;
    __builtin_amdgcn_sched_barrier(0);
    const char *lw = lds + ((2 * slab) % GEMM_SLOTS) * GEMM_SLOT_BYTES;
    const char *lx = lds + ((2 * slab + 1) % GEMM_SLOTS) * GEMM_SLOT_BYTES;
#pragma unroll
    for (int s = 0; s < 4; ++s) {  // 4 phases per slab, each with a quarter of the slab's loads and matrix-core work
      const int chunk = 2 * s + frag_half;
      if (slab >= 1) {
        // x unit in phases 0-1, W unit in phases 2-3: the W loads stay the four youngest, which is what
        // the vmcnt(4) at the top of the next slab relies on
        if (s < 2) {
          LDS_DMA16(xg[2 * s] + (size_t)sA * GEMM_SLAB, slotA + lds_off[2 * s]);
          LDS_DMA16(xg[2 * s + 1] + (size_t)sA * GEMM_SLAB, slotA + lds_off[2 * s + 1]);
        } else {
          LDS_DMA16(wg[2 * s - 4] + (size_t)sB * GEMM_SLAB, slotB + lds_off[2 * s - 4]);
          LDS_DMA16(wg[2 * s - 3] + (size_t)sB * GEMM_SLAB, slotB + lds_off[2 * s - 3]);
        }
      }
      // 32x32x2 fp32 instructions: phase s covers 32 bytes of K (two chunks, one per half wave)
      u32x4 wf[2], xf[4];
#pragma unroll
      for (int i = 0; i < 2; ++i) wf[i] = *reinterpret_cast<const u32x4 *>(lw + swz(wn * 64 + i * 32 + frag_row, chunk));
#pragma unroll
      for (int j = 0; j < 4; ++j) xf[j] = *reinterpret_cast<const u32x4 *>(lx + swz(wm * 128 + j * 32 + frag_row, chunk));
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) mma_chunk_f32(wf[i], xf[j], acc[i][j]);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  __builtin_amdgcn_s_waitcnt(0);

  // ---- epilogue: lane holds, per (i, j, g): 4 consecutive features of one token ----
  // D[row = feature, col = token]: token = lane % 32, feature = 8*g + 4*(lane/32) + r
  if constexpr (BF16_OUT) {
    // Full tiles go through LDS (free now) so that global stores are whole 128-byte lines: every wave transposes
    // its own 128-token x 64-feature block in a private region, rows padded to 136 bytes (the 8-byte writes of a
    // half-wave then fall on 64 distinct banks), and writes it out 8 token rows per instruction.
    if (m0 + GEMM_BM <= M && n0 + GEMM_BN <= N && (N & 63) == 0) {
      constexpr int PITCH = 136;
      __builtin_amdgcn_s_barrier();  // every wave is done reading operand slabs (and its own loads have landed)
      char *stage = lds + wave * (128 * PITCH);
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            uint2 pk;
            pk.x = pack_bf16x2(acc[i][j][4 * g + 0], acc[i][j][4 * g + 1]);
            pk.y = pack_bf16x2(acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]);
            *reinterpret_cast<uint2 *>(stage + (j * 32 + frag_row) * PITCH + (i * 32 + 8 * g + 4 * frag_half) * 2) = pk;
          }
      // the region is private to the wave: no barrier, the compiler's wait on the LDS writes is enough
      uint16_t *obase = reinterpret_cast<uint16_t *>(out) + (size_t)(m0 + wm * 128) * N + n0 + wn * 64;
      const int r_in = lane >> 3, c16 = lane & 7;
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int row = q * 8 + r_in;
        const char *src = stage + row * PITCH + c16 * 16;
        const uint2 lo = *reinterpret_cast<const uint2 *>(src), hi = *reinterpret_cast<const uint2 *>(src + 8);
        u32x4 v;
        v.x = lo.x; v.y = lo.y; v.z = hi.x; v.w = hi.y;
        *reinterpret_cast<u32x4 *>(obase + (size_t)row * N + c16 * 8) = v;
      }
      return;
    }
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int tok = m0 + wm * 128 + j * 32 + frag_row;
    if (tok >= M) continue;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int f = n0 + wn * 64 + i * 32 + 8 * g + 4 * frag_half;
        const float v0 = acc[i][j][4 * g + 0], v1 = acc[i][j][4 * g + 1], v2 = acc[i][j][4 * g + 2], v3 = acc[i][j][4 * g + 3];
        if constexpr (BF16_OUT) {
          uint16_t *o = reinterpret_cast<uint16_t *>(out) + (size_t)tok * N + f;
          if (f + 3 < N && (N & 3) == 0) {
            uint2 pk;
            pk.x = (uint32_t)f32_to_bf16_bits(v0) | ((uint32_t)f32_to_bf16_bits(v1) << 16);
            pk.y = (uint32_t)f32_to_bf16_bits(v2) | ((uint32_t)f32_to_bf16_bits(v3) << 16);
            *reinterpret_cast<uint2 *>(o) = pk;
          } else {
            if (f + 0 < N) o[0] = f32_to_bf16_bits(v0);
            if (f + 1 < N) o[1] = f32_to_bf16_bits(v1);
            if (f + 2 < N) o[2] = f32_to_bf16_bits(v2);
            if (f + 3 < N) o[3] = f32_to_bf16_bits(v3);
          }
        } else {
          float *o = reinterpret_cast<float *>(out) + (size_t)tok * N + f;
          if (f + 3 < N && (N & 3) == 0) {
            *reinterpret_cast<float4 *>(o) = make_float4(v0, v1, v2, v3);
          } else {
            if (f + 0 < N) o[0] = v0;
            if (f + 1 < N) o[1] = v1;
            if (f + 2 < N) o[2] = v2;
            if (f + 3 < N) o[3] = v3;
          }
        }
      }
    }
  }
}

// ---- bf16 operands ---------------------------------------------------------------------------------------------
#define WAITCNT_VM(N) (((N) & 0xf) | (0x7 << 4) | (0xf << 8) | (((N) >> 4) << 14))
#define WAITCNT_LGKM0 (0xf | (0x7 << 4) | (0x0 << 8) | (0x3 << 14))
#define PHASE_BARRIER()                   \
  __builtin_amdgcn_sched_barrier(0);      \
  __builtin_amdgcn_s_barrier();           \
  __builtin_amdgcn_sched_barrier(0)

// EPI_GMAX (bf16 output, N a multiple of 64): the epilogue also writes, for every token and every aligned granule of 64
// features, the largest select key of the granule's rounded outputs to gmax[token][N / 64]; the wave's 64 features are
// one granule.
// EPI_BIAS (bf16 output): out = bf16(float(bf16(acc)) + bias), the value of `(x @ w) + bias` when the product is a bf16
// tensor and the bias an fp32 one; `b_enc` then holds a bias per output column (nullable), `scale` one per output row
// (nullable).
// EPI_MARGIN (bf16 output, N a multiple of 64): like EPI_GMAX, but what is written per token and granule is the largest
// JumpReLU margin (out + bias) * scale - theta of the granule's rounded outputs (a float, each operation rounded on its
// own as the activation kernels do): a granule holds an active or in-window entry only if that reaches -window / 2.
// EPI_GMAX_LOWP: EPI_GMAX with the keys in the bf16 arithmetic of a dictionary held in bf16 (the sum with the bias and the
// product with the scale each rounded to bf16: what sae_select_topk_row_lowp / sae_select_topk_batch_lowp form).
constexpr int EPI_NONE = 0, EPI_GMAX = 1, EPI_BIAS = 2, EPI_MARGIN = 3, EPI_GMAX_LOWP = 4;

// Operand layouts.  The default is K-contiguous: row r of the operand (a token of x, a feature of w) holds its K values
// side by side.  XT / WT say that the operand is stored the other way round, [K, rows] with the rows side by side (what a
// product over the token axis finds: dW = d(pre)^T x reads d(pre) [tokens, features] and x [tokens, d_model] as they
// are; acts @ W_D reads W_D [features, d_model] as it is).  A slab of such an operand is 64 K-rows of 256 values
// (512 bytes each): the same 32 KiB slot, filled by the same 1 KiB LDS-direct loads (two K-rows per load), and its
// matrix-core fragments (8 consecutive K values of one row) are read ACROSS the K-rows with ds_read_b64_tr_b16, two per
// fragment: lane i of a group of 16 points at K-row 4 hh + i / 4, values 4 (i % 4) .. + 3 and receives the four K values
// of value i.  Chunk c (16 bytes) of K-row r sits at chunk c ^ tkey(r), tkey(r) = 2 ((r & 3) | ((r >> 3) & 1) << 2): the
// eight K-rows x 32 bytes that half a wave reads at once then fall on 256 distinct bytes.
__device__ __forceinline__ int gemm_tkey(int krow) { return ((krow & 3) | (((krow >> 3) & 1) << 2)) << 1; }

template <bool BF16_OUT, int EPI, bool XT = false, bool WT = false>
__global__ __launch_bounds__(GEMM_THREADS) void encoder_gemm_bf16_kernel(
    const char *__restrict__ x, const char *__restrict__ w, void *__restrict__ out, int M, int N,
    int row_bytes /* contraction length * 2 */, int pitch_x, int pitch_w /* bytes between stored rows of x / w */,
    int tiles_m, int tiles_n, int rm_log2, const float *__restrict__ b_enc,
    const float *__restrict__ scale, uint32_t *__restrict__ gmax, const float *__restrict__ theta) {
  extern __shared__ __attribute__((aligned(16))) char lds[];   // the ring of GEMM_SLOTS operand slabs
  if (blockIdx.y) {
    // group g of a batch of independent products of one shape, each operand stacked group after group; or, when the rows
    // are longer than the contraction (or an operand is stored [K, rows]), slice g of the contraction axis (split-K: the
    // caller sums the groups' outputs)
    const size_t g = blockIdx.y;
    if (XT || WT || pitch_x != row_bytes) {
      x += XT ? g * (size_t)(row_bytes >> 1) * pitch_x : g * (size_t)row_bytes;
      w += WT ? g * (size_t)(row_bytes >> 1) * pitch_w : g * (size_t)row_bytes;
    } else {
      x += g * (size_t)M * row_bytes;
      w += g * (size_t)N * row_bytes;
    }
    out = reinterpret_cast<char *>(out) + g * (size_t)M * N * (BF16_OUT ? 2 : 4);
    if constexpr (EPI == EPI_GMAX || EPI == EPI_MARGIN || EPI == EPI_GMAX_LOWP) {
      if (b_enc) b_enc += g * (size_t)N;
      if (scale) scale += g * (size_t)N;
      gmax += g * (size_t)M * (N >> 6);
    }
  }

  // ---- XCD-aware tile assignment.  One tile dimension is dealt round-robin to the 8 XCDs (the feature tiles, or, when
  // there are fewer than 8 of those, the token tiles: rm_log2 < 0 says so and -rm_log2 - 1 takes its place); 32 consecutive
  // workgroups of an XCD cover 2^rm_log2 tiles of the other dimension x the rest in tiles of the dealt one.
  int tile_m, tile_n;
  {
    const int bid = blockIdx.x, xcd = bid & 7, slot = bid >> 3;
    const int grp = slot >> 5, in = slot & 31;
    const bool deal_m = rm_log2 < 0;
    const int ro_log2 = deal_m ? -rm_log2 - 1 : rm_log2;
    const int tiles_o = deal_m ? tiles_n : tiles_m;        // the dimension kept whole inside an XCD
    const int ro = 1 << ro_log2, rs = 32 >> ro_log2;
    const int o_groups = (tiles_o + ro - 1) >> ro_log2;
    const int s_grp = grp / o_groups, o_part = grp % o_groups;
    const int tile_o = o_part * ro + (in & (ro - 1));
    const int tile_s = (s_grp * rs + (in >> ro_log2)) * 8 + xcd;
    tile_m = deal_m ? tile_s : tile_o;
    tile_n = deal_m ? tile_o : tile_s;
    if (tile_n >= tiles_n || tile_m >= tiles_m) return;     // the whole workgroup leaves: no barrier is left short
  }
  const int m0 = tile_m * GEMM_BM, n0 = tile_n * GEMM_BN;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;
  const bool late = wm != 0;          // the group that runs one phase behind

  // ---- global -> LDS: every wave fills 32 rows of each operand slab with 4 loads of 1 KiB (8 lanes per 128-byte row,
  // the chunk swizzle applied on the global side)
  const char *xg[4], *wg[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = wave * 32 + i * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((r >> 1) & 7);
    // stored [K, rows]: this load fills K-rows 8 wave + 2 i and + 1 of the slab, 32 chunks of 8 values each; values past
    // the operand's last row repeat its last 8 (their products land in accumulators that are never stored)
    const int kr = wave * 8 + i * 2 + (lane >> 5), tc = (lane & 31) ^ gemm_tkey(kr);
    if constexpr (XT) {
      const int m = m0 + tc * 8;
      xg[i] = x + (size_t)kr * pitch_x + (size_t)(m + 8 <= M ? m : M - 8) * 2;
    } else {
      xg[i] = x + (size_t)(m0 + r < M ? m0 + r : M - 1) * pitch_x + chunk * 16;
    }
    if constexpr (WT) {
      const int n = n0 + tc * 8;
      wg[i] = w + (size_t)kr * pitch_w + (size_t)(n + 8 <= N ? n : N - 8) * 2;
    } else {
      wg[i] = w + (size_t)(n0 + r < N ? n0 + r : N - 1) * pitch_w + chunk * 16;
    }
  }
  const size_t x_adv = XT ? (size_t)64 * pitch_x : (size_t)GEMM_SLAB, w_adv = WT ? (size_t)64 * pitch_w : (size_t)GEMM_SLAB;
  const uint32_t ld_base = (uint32_t)(wave * 32) * GEMM_SLAB;

  f32x4_t acc[4][8];   // [feature sub-tile of 16][token sub-tile of 16]
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.f;

  const int n_slabs = row_bytes / GEMM_SLAB;
  typedef __attribute__((address_space(3))) void *lds_ptr_t;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
  // unit t of the load sequence: t even -> W slab t / 2, t odd -> x slab (t - 1) / 2; it lives in slot t % 5
#define ISSUE_UNIT(UNIT, SLAB)                                                                                      \
  {                                                                                                                 \
    const uint32_t slot_ = lds_base + (uint32_t)((UNIT) % GEMM_SLOTS) * GEMM_SLOT_BYTES + ld_base;                  \
    _Pragma("unroll") for (int i = 0; i < 4; ++i)                                                                   \
        LDS_DMA16(((UNIT) & 1 ? xg[i] + (size_t)(SLAB) * x_adv : wg[i] + (size_t)(SLAB) * w_adv), slot_ + i * 1024); \
  }
  // at the end of the phase in which the last fragments of a slab are read, the next slab (x issued this slab, W a
  // slab ago) must be in LDS: everything but this wave's 4 youngest loads (W two slabs ahead, if there is one)
#define WAIT_NEXT_SLAB()                                                                 \
  if (slab + 2 < n_slabs) __builtin_amdgcn_s_waitcnt(WAITCNT_VM(4));                     \
  else __builtin_amdgcn_s_waitcnt(WAITCNT_VM(0))
  ISSUE_UNIT(0, 0)
  ISSUE_UNIT(1, 0)
  if (n_slabs > 1) {
    ISSUE_UNIT(2, 1)
    __builtin_amdgcn_s_waitcnt(WAITCNT_VM(4));
  } else {
    __builtin_amdgcn_s_waitcnt(WAITCNT_VM(0));
  }
  PHASE_BARRIER();                      // slab 0 is in LDS
  if (late) { PHASE_BARRIER(); }        // the late group sits out the first phase (the early group the last one)

  const int frow = lane & 15, fq = lane >> 4;
  u32x4 wf[4], xf[8];
  // stored [K, rows]: the lane's byte offset inside a slab for k-step 0, hh = 0 of every sub-tile (a k-step adds 32 K-rows =
  // 16384 bytes, hh = 1 four K-rows = 2048 bytes; the chunk key depends on neither)
  int xt_off[XT ? 8 : 1], wt_off[WT ? 4 : 1];
  if constexpr (XT || WT) {
    const int krow = 8 * fq + (frow >> 2), key = gemm_tkey(krow), sub = (frow & 3) >> 1, byte = (frow & 1) * 8;
    if constexpr (XT) {
#pragma unroll
      for (int j = 0; j < 8; ++j) xt_off[j] = krow * 512 + (((wm * 16 + 2 * j + sub) ^ key) << 4) + byte;
    }
    if constexpr (WT) {
#pragma unroll
      for (int i = 0; i < 4; ++i) wt_off[i] = krow * 512 + (((wn * 8 + 2 * i + sub) ^ key) << 4) + byte;
    }
  }
  typedef __attribute__((ext_vector_type(4))) short gemm_i16x4;
  typedef __attribute__((address_space(3))) gemm_i16x4 *gemm_lds_i16x4;
#define READ_TR(DST, BASE, OFF)                                                                                     \
  {                                                                                                                 \
    const gemm_i16x4 lo_ = __builtin_amdgcn_ds_read_tr16_b64_v4i16((gemm_lds_i16x4)((BASE) + (OFF)));               \
    const gemm_i16x4 hi_ = __builtin_amdgcn_ds_read_tr16_b64_v4i16((gemm_lds_i16x4)((BASE) + (OFF) + 2048));        \
    typedef __attribute__((ext_vector_type(8))) short i16x8_;                                                       \
    DST = __builtin_bit_cast(u32x4, (i16x8_)__builtin_shufflevector(lo_, hi_, 0, 1, 2, 3, 4, 5, 6, 7));             \
  }
  // a k-step is 64 bytes of K: 4 chunks, one per quarter wave
#define READ_FRAGS(KS)                                                                                              \
  {                                                                                                                 \
    const int c16_ = 4 * (KS) + fq;                                                                                 \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                                                 \
      if constexpr (WT) READ_TR(wf[i], lw, wt_off[i] + (KS) * 16384)                                                \
      else wf[i] = *reinterpret_cast<const u32x4 *>(lw + swz(wn * 64 + i * 16 + frow, c16_));                       \
    }                                                                                                               \
    _Pragma("unroll") for (int j = 0; j < 8; ++j) {                                                                 \
      if constexpr (XT) READ_TR(xf[j], lx, xt_off[j] + (KS) * 16384)                                                \
      else xf[j] = *reinterpret_cast<const u32x4 *>(lx + swz(wm * 128 + j * 16 + frow, c16_));                      \
    }                                                                                                               \
  }
#define MMA_STEP()                                                                                                  \
  _Pragma("unroll") for (int j = 0; j < 8; ++j)                                                                     \
  _Pragma("unroll") for (int i = 0; i < 4; ++i)                                                                     \
      acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, wf[i]),                      \
                                                          __builtin_bit_cast(bf16x8_t, xf[j]), acc[i][j], 0, 0, 0);

  // EPI_GMAX: this lane's 16 bias and 16 scale values; EPI_BIAS: its 16 column biases and 8 row biases.  Asked for here
  // so that the epilogue does not wait for them.
  constexpr bool MARGIN = EPI == EPI_MARGIN, LOWPK = EPI == EPI_GMAX_LOWP, GMAX = EPI == EPI_GMAX || MARGIN || LOWPK, BIAS = EPI == EPI_BIAS;
  float bb[EPI != EPI_NONE ? 4 : 1][4], ss[GMAX ? 4 : 1][4], rb[BIAS ? 8 : 1];
  if constexpr (EPI != EPI_NONE) {
    const int f0 = n0 + wn * 64;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int f = f0 + i * 16 + 4 * fq;
      float4 b4 = make_float4(0.f, 0.f, 0.f, 0.f), s4 = make_float4(1.f, 1.f, 1.f, 1.f);
      if (GMAX || (N & 3) == 0) {
        if (b_enc && f + 3 < N) b4 = *reinterpret_cast<const float4 *>(b_enc + f);
      } else if (b_enc) {     // a bias vector that is not 16-byte addressable at every f
        b4.x = f < N ? b_enc[f] : 0.f; b4.y = f + 1 < N ? b_enc[f + 1] : 0.f;
        b4.z = f + 2 < N ? b_enc[f + 2] : 0.f; b4.w = f + 3 < N ? b_enc[f + 3] : 0.f;
      }
      bb[i][0] = b4.x; bb[i][1] = b4.y; bb[i][2] = b4.z; bb[i][3] = b4.w;
      if constexpr (GMAX) {
        if (scale && f0 < N) s4 = *reinterpret_cast<const float4 *>(scale + f);
        ss[i][0] = s4.x; ss[i][1] = s4.y; ss[i][2] = s4.z; ss[i][3] = s4.w;
      }
    }
    if constexpr (BIAS) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int tok = m0 + wm * 128 + j * 16 + frow;
        rb[j] = scale && tok < M ? scale[tok] : 0.f;
      }
    }
  }
  for (int slab = 0; slab < n_slabs; ++slab) {
    const char *lw = lds + ((2 * slab) % GEMM_SLOTS) * GEMM_SLOT_BYTES;
    const char *lx = lds + ((2 * slab + 1) % GEMM_SLOTS) * GEMM_SLOT_BYTES;
    // memory phase, k-step 0; x of the next slab goes into the slot the previous slab's W left
    READ_FRAGS(0)
    if (slab + 1 < n_slabs) ISSUE_UNIT(2 * slab + 3, slab + 1)
    __builtin_amdgcn_s_waitcnt(WAITCNT_LGKM0);
    PHASE_BARRIER();
    MMA_STEP()
    PHASE_BARRIER();
    // memory phase, k-step 1; W two slabs ahead goes into the slot the previous slab's x left
    READ_FRAGS(1)
    if (slab + 2 < n_slabs) ISSUE_UNIT(2 * slab + 4, slab + 2)
    if (late) { WAIT_NEXT_SLAB(); }     // the late group's last reads of the slab: the phase the early group computes in
    __builtin_amdgcn_s_waitcnt(WAITCNT_LGKM0);
    PHASE_BARRIER();
    MMA_STEP()
    if (!late) { WAIT_NEXT_SLAB(); }
    PHASE_BARRIER();
  }
#undef ISSUE_UNIT
#undef WAIT_NEXT_SLAB
#undef READ_FRAGS
#undef READ_TR
#undef MMA_STEP
  // The early group has one barrier to go (the late group's last matrix-core phase).  No wave reads operand slabs any
  // more and every load has landed, so LDS is free: the early waves stage and store their output under that phase.

  // ---- epilogue: lane holds, per (i, j): features 4 (lane / 16) .. + 3 of sub-tile i for token lane % 16 of sub-tile j
  if constexpr (BIAS) {
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t lo = pack_bf16x2(acc[i][j][0], acc[i][j][1]), hi = pack_bf16x2(acc[i][j][2], acc[i][j][3]);
        acc[i][j][0] = (__uint_as_float(lo << 16) + bb[i][0]) + rb[j];
        acc[i][j][1] = (__uint_as_float(lo & 0xffff0000u) + bb[i][1]) + rb[j];
        acc[i][j][2] = (__uint_as_float(hi << 16) + bb[i][2]) + rb[j];
        acc[i][j][3] = (__uint_as_float(hi & 0xffff0000u) + bb[i][3]) + rb[j];
      }
  }
  if constexpr (GMAX) {
    const int f0 = n0 + wn * 64;
    if (f0 < N) {
      const int ng = N >> 6;
      float th[MARGIN ? 4 : 1][4];
      if constexpr (MARGIN) {     // the thresholds are asked for here: the main loop's fragment registers are free now
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float4 t4 = *reinterpret_cast<const float4 *>(theta + f0 + i * 16 + 4 * fq);
          th[i][0] = t4.x; th[i][1] = t4.y; th[i][2] = t4.z; th[i][3] = t4.w;
        }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        // positive floats order like their bit patterns, so the largest key is the key of the largest h1; the maximum
        // starts at 0 and v_max ignores NaN operands, as the key of a NaN (0) is ignored
        float hmax = MARGIN ? -INFINITY : 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // the accumulators take their rounded values here, so the stores below write exactly what the keys were formed from
          const uint32_t lo = pack_bf16x2(acc[i][j][0], acc[i][j][1]), hi = pack_bf16x2(acc[i][j][2], acc[i][j][3]);
          acc[i][j][0] = __uint_as_float(lo << 16); acc[i][j][1] = __uint_as_float(lo & 0xffff0000u);
          acc[i][j][2] = __uint_as_float(hi << 16); acc[i][j][3] = __uint_as_float(hi & 0xffff0000u);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            if constexpr (MARGIN) hmax = fmaxf(hmax, sub_rn(mul_rn(acc[i][j][r] + bb[i][r], ss[i][r]), th[i][r]));
            else if constexpr (LOWPK) hmax = fmaxf(hmax, bf16_round(mul_rn(bf16_round(add_rn(acc[i][j][r], bb[i][r])), ss[i][r])));
            else hmax = fmaxf(hmax, (acc[i][j][r] + bb[i][r]) * ss[i][r]);   // h1 of select_key_plain
          }
        }
        hmax = fmaxf(hmax, __shfl_xor(hmax, 16, 64));
        hmax = fmaxf(hmax, __shfl_xor(hmax, 32, 64));
        const int tok = m0 + wm * 128 + j * 16 + frow;
        if (fq == 0 && tok < M)
          gmax[(size_t)tok * ng + (f0 >> 6)] = MARGIN ? __float_as_uint(hmax) : (hmax > 0.f ? __float_as_uint(hmax) : 0u);
      }
    }
  }
  bool stored = false;
  if constexpr (BF16_OUT) {
    // Full tiles go through LDS so that global stores are whole 128-byte lines: every wave transposes its own
    // 128-token x 64-feature block in a private region, rows padded to 136 bytes (the 8-byte writes of a quarter
    // wave pair then fall on distinct banks), and writes it out 8 token rows per instruction.
    if (m0 + GEMM_BM <= M && n0 + GEMM_BN <= N && (N & 63) == 0) {
      constexpr int PITCH = 136;
      char *stage = lds + wave * (128 * PITCH);
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          uint2 pk;
          pk.x = pack_bf16x2(acc[i][j][0], acc[i][j][1]);
          pk.y = pack_bf16x2(acc[i][j][2], acc[i][j][3]);
          *reinterpret_cast<uint2 *>(stage + (j * 16 + frow) * PITCH + (i * 16 + 4 * fq) * 2) = pk;
        }
      // the region is private to the wave: no barrier, the compiler's wait on the LDS writes is enough
      uint16_t *obase = reinterpret_cast<uint16_t *>(out) + (size_t)(m0 + wm * 128) * N + n0 + wn * 64;
      const int r_in = lane >> 3, c16 = lane & 7;
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int row = q * 8 + r_in;
        const char *src = stage + row * PITCH + c16 * 16;
        const uint2 lo = *reinterpret_cast<const uint2 *>(src), hi = *reinterpret_cast<const uint2 *>(src + 8);
        u32x4 v;
        v.x = lo.x; v.y = lo.y; v.z = hi.x; v.w = hi.y;
        *reinterpret_cast<u32x4 *>(obase + (size_t)row * N + c16 * 8) = v;
      }
      stored = true;
    }
  }
  if (!stored) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int tok = m0 + wm * 128 + j * 16 + frow;
      if (tok >= M) continue;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int f = n0 + wn * 64 + i * 16 + 4 * fq;
        const float v0 = acc[i][j][0], v1 = acc[i][j][1], v2 = acc[i][j][2], v3 = acc[i][j][3];
        if constexpr (BF16_OUT) {
          uint16_t *o = reinterpret_cast<uint16_t *>(out) + (size_t)tok * N + f;
          if (f + 3 < N && (N & 3) == 0) {
            uint2 pk;
            pk.x = (uint32_t)f32_to_bf16_bits(v0) | ((uint32_t)f32_to_bf16_bits(v1) << 16);
            pk.y = (uint32_t)f32_to_bf16_bits(v2) | ((uint32_t)f32_to_bf16_bits(v3) << 16);
            *reinterpret_cast<uint2 *>(o) = pk;
          } else {
            if (f + 0 < N) o[0] = f32_to_bf16_bits(v0);
            if (f + 1 < N) o[1] = f32_to_bf16_bits(v1);
            if (f + 2 < N) o[2] = f32_to_bf16_bits(v2);
            if (f + 3 < N) o[3] = f32_to_bf16_bits(v3);
          }
        } else {
          float *o = reinterpret_cast<float *>(out) + (size_t)tok * N + f;
          if (f + 3 < N && (N & 3) == 0) {
            *reinterpret_cast<float4 *>(o) = make_float4(v0, v1, v2, v3);
          } else {
            if (f + 0 < N) o[0] = v0;
            if (f + 1 < N) o[1] = v1;
            if (f + 2 < N) o[2] = v2;
            if (f + 3 < N) o[3] = v3;
          }
        }
      }
    }
  }
  if (!late) { PHASE_BARRIER(); }       // pairs with the late group's last phase
}

// grid: 8 XCDs x (token tiles padded to rm) x (feature tiles per XCD padded to 32 / rm); padding workgroups exit at once
static int reserve_lds(const void *kern) {
  // asked for on every launch (a host-side table lookup): the attribute belongs to the kernel on the current device, and
  // a cached "done" flag would be neither per device nor safe between threads
  hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS_BYTES);
  if (e != hipSuccess) return fail(SAE_ERR_LAUNCH, "encoder_gemm: cannot reserve %d bytes of LDS: %s", GEMM_LDS_BYTES,
                                   hipGetErrorString(e));
  return SAE_OK;
}

template <bool BF16_OUT>
static int launch_gemm_f32(const void *x, const void *w, void *out, int64_t B, int64_t d, int64_t F, hipStream_t st) {
  const int tiles_m = (int)((B + GEMM_BM - 1) / GEMM_BM), tiles_n = (int)((F + GEMM_BN - 1) / GEMM_BN);
  auto kern = encoder_gemm_f32_kernel<BF16_OUT>;
  const int rc = reserve_lds(reinterpret_cast<const void *>(kern));
  if (rc != SAE_OK) return rc;
  const int m_pad = (tiles_m + 3) / 4 * 4, n_local_pad = ((tiles_n + 7) / 8 + 7) / 8 * 8;
  hipLaunchKernelGGL(kern, dim3(8 * m_pad * n_local_pad), dim3(GEMM_THREADS), GEMM_LDS_BYTES, st, (const char *)x,
                     (const char *)w, out, (int)B, (int)F, (int)(d * 4), tiles_m, tiles_n);
  return check_launch("encoder_gemm");
}

template <bool BF16_OUT, int EPI, bool XT = false, bool WT = false>
static int launch_gemm_bf16(const void *x, const void *w, void *out, int64_t B, int64_t d, int64_t F, const float *b_enc,
                            const float *scale, uint32_t *gmax, hipStream_t st, int64_t n_groups = 1,
                            const float *theta = nullptr, int64_t split_k = 1) {
  // split_k > 1: d is the length of one slice of a contraction that is split_k * d long; the slices are the launch's groups
  const int tiles_m = (int)((B + GEMM_BM - 1) / GEMM_BM), tiles_n = (int)((F + GEMM_BN - 1) / GEMM_BN);
  auto kern = encoder_gemm_bf16_kernel<BF16_OUT, EPI, XT, WT>;
  const int rc = reserve_lds(reinterpret_cast<const void *>(kern));
  if (rc != SAE_OK) return rc;
  // with fewer than 8 feature tiles most XCDs would sit idle if those were what is dealt to them: deal the token tiles
  const bool deal_m = tiles_n < 8 && tiles_m > tiles_n;
  const int tiles_o = deal_m ? tiles_n : tiles_m, tiles_s = deal_m ? tiles_m : tiles_n;
  const int ro_log2 = tiles_o >= 8 ? 3 : (tiles_o > 2 ? 2 : (tiles_o > 1 ? 1 : 0)), ro = 1 << ro_log2, rs = 32 >> ro_log2;
  const int rm_log2 = deal_m ? -ro_log2 - 1 : ro_log2;
  const int m_pad = (tiles_o + ro - 1) / ro * ro, n_local_pad = ((tiles_s + 7) / 8 + rs - 1) / rs * rs;
  // bytes between stored rows: an operand stored [K, rows] has rows of `rows` values; a K-contiguous one rows of the whole
  // contraction
  const int64_t k_total = d * (split_k > 1 ? split_k : 1);
  const int pitch_x = (int)((XT ? B : k_total) * 2), pitch_w = (int)((WT ? F : k_total) * 2);
  hipLaunchKernelGGL(kern, dim3(8 * m_pad * n_local_pad, (unsigned)(split_k > 1 ? split_k : n_groups)), dim3(GEMM_THREADS),
                     GEMM_LDS_BYTES, st, (const char *)x, (const char *)w, out, (int)B, (int)F, (int)(d * 2), pitch_x, pitch_w,
                     tiles_m, tiles_n, rm_log2, b_enc, scale, gmax, theta);
  return check_launch("encoder_gemm");
}

}  // namespace sae

extern "C" int sae_encoder_gemm(const void *x, const void *w_enc_t, void *pre, int64_t B, int64_t d, int64_t F,
                                int in_dtype, int out_dtype, void *stream) {
  using namespace sae;
  SAE_REQUIRE(x && w_enc_t && pre, SAE_ERR_INVALID_ARG, "encoder_gemm: null pointer");
  SAE_REQUIRE(B > 0 && d > 0 && F > 0, SAE_ERR_INVALID_ARG, "encoder_gemm: B, d, F must be positive");
  SAE_REQUIRE(in_dtype == SAE_F32 || in_dtype == SAE_BF16, SAE_ERR_INVALID_ARG, "encoder_gemm: bad in_dtype %d", in_dtype);
  SAE_REQUIRE(out_dtype == SAE_F32 || out_dtype == SAE_BF16, SAE_ERR_INVALID_ARG, "encoder_gemm: bad out_dtype %d", out_dtype);
  SAE_REQUIRE(B < (1LL << 31) && F < (1LL << 31) && d < (1LL << 28), SAE_ERR_UNSUPPORTED, "encoder_gemm: size too large");
  const int64_t per_slab = in_dtype == SAE_BF16 ? 64 : 32;
  SAE_REQUIRE(d % per_slab == 0, SAE_ERR_UNSUPPORTED, "encoder_gemm: d_model=%lld must be a multiple of %lld",
              (long long)d, (long long)per_slab);
  SAE_REQUIRE((((uintptr_t)x | (uintptr_t)w_enc_t | (uintptr_t)pre) & 15) == 0, SAE_ERR_INVALID_ARG,
              "encoder_gemm: pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (in_dtype == SAE_BF16) {
    return out_dtype == SAE_BF16 ? launch_gemm_bf16<true, EPI_NONE>(x, w_enc_t, pre, B, d, F, nullptr, nullptr, nullptr, st)
                                 : launch_gemm_bf16<false, EPI_NONE>(x, w_enc_t, pre, B, d, F, nullptr, nullptr, nullptr, st);
  }
  return out_dtype == SAE_BF16 ? launch_gemm_f32<true>(x, w_enc_t, pre, B, d, F, st)
                               : launch_gemm_f32<false>(x, w_enc_t, pre, B, d, F, st);
}

extern "C" int sae_encoder_gemm_split_k(const void *x_bf16, const void *w_t_bf16, float *partials, int64_t n_splits, int64_t B,
                                        int64_t d, int64_t F, void *stream) {
  using namespace sae;
  SAE_REQUIRE(x_bf16 && w_t_bf16 && partials, SAE_ERR_INVALID_ARG, "encoder_gemm_split_k: null pointer");
  SAE_REQUIRE(B > 0 && d > 0 && F > 0 && n_splits > 1, SAE_ERR_INVALID_ARG, "encoder_gemm_split_k: sizes must be positive, n_splits > 1");
  SAE_REQUIRE(B < (1LL << 31) && F < (1LL << 31) && d < (1LL << 28) && n_splits <= 64, SAE_ERR_UNSUPPORTED,
              "encoder_gemm_split_k: size too large");
  SAE_REQUIRE(d % (64 * n_splits) == 0, SAE_ERR_UNSUPPORTED, "encoder_gemm_split_k: d=%lld must be a multiple of 64 * n_splits",
              (long long)d);
  SAE_REQUIRE((B * F * 4) % 16 == 0, SAE_ERR_UNSUPPORTED, "encoder_gemm_split_k: a slice's output must be a multiple of 16 bytes");
  SAE_REQUIRE((((uintptr_t)x_bf16 | (uintptr_t)w_t_bf16 | (uintptr_t)partials) & 15) == 0, SAE_ERR_INVALID_ARG,
              "encoder_gemm_split_k: pointers must be 16-byte aligned");
  return launch_gemm_bf16<false, EPI_NONE>(x_bf16, w_t_bf16, partials, B, d / n_splits, F, nullptr, nullptr, nullptr,
                                           (hipStream_t)stream, 1, nullptr, n_splits);
}

extern "C" int sae_gemm_bf16(const void *a, int a_k_major, const void *b, int b_k_major, void *out, int out_dtype, int64_t M,
                             int64_t N, int64_t K, int64_t n_splits, void *stream) {
  using namespace sae;
  SAE_REQUIRE(a && b && out, SAE_ERR_INVALID_ARG, "gemm_bf16: null pointer");
  SAE_REQUIRE(M > 0 && N > 0 && K > 0 && n_splits >= 1, SAE_ERR_INVALID_ARG, "gemm_bf16: sizes must be positive");
  SAE_REQUIRE(out_dtype == SAE_F32 || out_dtype == SAE_BF16, SAE_ERR_INVALID_ARG, "gemm_bf16: bad out_dtype %d", out_dtype);
  SAE_REQUIRE(M < (1LL << 30) && N < (1LL << 30) && K < (1LL << 28) && n_splits <= 64, SAE_ERR_UNSUPPORTED, "gemm_bf16: size too large");
  SAE_REQUIRE(K % (64 * n_splits) == 0, SAE_ERR_UNSUPPORTED, "gemm_bf16: K=%lld must be a multiple of 64 * n_splits", (long long)K);
  SAE_REQUIRE(n_splits == 1 || (out_dtype == SAE_F32 && (M * N * 4) % 16 == 0), SAE_ERR_UNSUPPORTED,
              "gemm_bf16: split products write fp32 partial results of a multiple of 16 bytes each");
  SAE_REQUIRE(!a_k_major || (M % 8 == 0), SAE_ERR_UNSUPPORTED, "gemm_bf16: an operand stored [K, M] needs M=%lld to be a multiple of 8",
              (long long)M);
  SAE_REQUIRE(!b_k_major || (N % 8 == 0), SAE_ERR_UNSUPPORTED, "gemm_bf16: an operand stored [K, N] needs N=%lld to be a multiple of 8",
              (long long)N);
  SAE_REQUIRE((((uintptr_t)a | (uintptr_t)b | (uintptr_t)out) & 15) == 0, SAE_ERR_INVALID_ARG, "gemm_bf16: pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  const int64_t ks = K / n_splits;
#define SAE_GEMM_CASE(XT, WT)                                                                                                 \
  return out_dtype == SAE_BF16                                                                                                \
             ? launch_gemm_bf16<true, EPI_NONE, XT, WT>(a, b, out, M, ks, N, nullptr, nullptr, nullptr, st, 1, nullptr, n_splits) \
             : launch_gemm_bf16<false, EPI_NONE, XT, WT>(a, b, out, M, ks, N, nullptr, nullptr, nullptr, st, 1, nullptr, n_splits)
  if (a_k_major && b_k_major) { SAE_GEMM_CASE(true, true); }
  if (a_k_major) { SAE_GEMM_CASE(true, false); }
  if (b_k_major) { SAE_GEMM_CASE(false, true); }
  SAE_GEMM_CASE(false, false);
#undef SAE_GEMM_CASE
}

extern "C" int sae_encoder_gemm_granule_max(const void *x_bf16, const void *w_enc_t_bf16, void *pre_bf16, int64_t n_groups,
                                            int64_t B, int64_t d, int64_t F, const float *b_enc, const float *scale,
                                            uint32_t *granule_max, void *stream) {
  using namespace sae;
  SAE_REQUIRE(x_bf16 && w_enc_t_bf16 && pre_bf16 && granule_max, SAE_ERR_INVALID_ARG, "encoder_gemm_granule_max: null pointer");
  SAE_REQUIRE(B > 0 && d > 0 && F > 0 && n_groups > 0, SAE_ERR_INVALID_ARG, "encoder_gemm_granule_max: sizes must be positive");
  SAE_REQUIRE(B < (1LL << 31) && F < (1LL << 31) && d < (1LL << 28) && n_groups <= 65535, SAE_ERR_UNSUPPORTED,
              "encoder_gemm_granule_max: size too large");
  SAE_REQUIRE(d % 64 == 0, SAE_ERR_UNSUPPORTED, "encoder_gemm_granule_max: d_model=%lld must be a multiple of 64", (long long)d);
  SAE_REQUIRE(F % 64 == 0, SAE_ERR_UNSUPPORTED, "encoder_gemm_granule_max: F=%lld must be a multiple of 64 (whole granules)",
              (long long)F);
  SAE_REQUIRE((((uintptr_t)x_bf16 | (uintptr_t)w_enc_t_bf16 | (uintptr_t)pre_bf16 | (uintptr_t)b_enc | (uintptr_t)scale) & 15) == 0,
              SAE_ERR_INVALID_ARG, "encoder_gemm_granule_max: pointers must be 16-byte aligned");
  return launch_gemm_bf16<true, EPI_GMAX>(x_bf16, w_enc_t_bf16, pre_bf16, B, d, F, b_enc, scale, granule_max, (hipStream_t)stream,
                                      n_groups);
}

extern "C" int sae_encoder_gemm_granule_max_lowp(const void *x_bf16, const void *w_enc_t_bf16, void *pre_bf16, int64_t n_groups,
                                                 int64_t B, int64_t d, int64_t F, const float *b_enc, const float *scale,
                                                 uint32_t *granule_max, void *stream) {
  using namespace sae;
  SAE_REQUIRE(x_bf16 && w_enc_t_bf16 && pre_bf16 && granule_max, SAE_ERR_INVALID_ARG, "encoder_gemm_granule_max_lowp: null pointer");
  SAE_REQUIRE(B > 0 && d > 0 && F > 0 && n_groups > 0, SAE_ERR_INVALID_ARG, "encoder_gemm_granule_max_lowp: sizes must be positive");
  SAE_REQUIRE(B < (1LL << 31) && F < (1LL << 31) && d < (1LL << 28) && n_groups <= 65535, SAE_ERR_UNSUPPORTED,
              "encoder_gemm_granule_max_lowp: size too large");
  SAE_REQUIRE(d % 64 == 0 && F % 64 == 0, SAE_ERR_UNSUPPORTED,
              "encoder_gemm_granule_max_lowp: d_model=%lld and F=%lld must be multiples of 64", (long long)d, (long long)F);
  SAE_REQUIRE((((uintptr_t)x_bf16 | (uintptr_t)w_enc_t_bf16 | (uintptr_t)pre_bf16 | (uintptr_t)b_enc | (uintptr_t)scale) & 15) == 0,
              SAE_ERR_INVALID_ARG, "encoder_gemm_granule_max_lowp: pointers must be 16-byte aligned");
  return launch_gemm_bf16<true, EPI_GMAX_LOWP>(x_bf16, w_enc_t_bf16, pre_bf16, B, d, F, b_enc, scale, granule_max,
                                           (hipStream_t)stream, n_groups);
}

extern "C" int sae_encoder_gemm_bias(const void *x_bf16, const void *w_t_bf16, void *out_bf16, int64_t B, int64_t d, int64_t F,
                                     const float *col_bias, const float *row_bias, void *stream) {
  using namespace sae;
  SAE_REQUIRE(x_bf16 && w_t_bf16 && out_bf16, SAE_ERR_INVALID_ARG, "encoder_gemm_bias: null pointer");
  SAE_REQUIRE(B > 0 && d > 0 && F > 0, SAE_ERR_INVALID_ARG, "encoder_gemm_bias: sizes must be positive");
  SAE_REQUIRE(B < (1LL << 31) && F < (1LL << 31) && d < (1LL << 28), SAE_ERR_UNSUPPORTED, "encoder_gemm_bias: size too large");
  SAE_REQUIRE(d % 64 == 0, SAE_ERR_UNSUPPORTED, "encoder_gemm_bias: d=%lld must be a multiple of 64", (long long)d);
  SAE_REQUIRE((((uintptr_t)x_bf16 | (uintptr_t)w_t_bf16 | (uintptr_t)out_bf16 | (uintptr_t)col_bias) & 15) == 0, SAE_ERR_INVALID_ARG,
              "encoder_gemm_bias: pointers must be 16-byte aligned");
  return launch_gemm_bf16<true, EPI_BIAS>(x_bf16, w_t_bf16, out_bf16, B, d, F, col_bias, row_bias, nullptr, (hipStream_t)stream);
}

extern "C" int sae_encoder_gemm_jumprelu_margin(const void *x_bf16, const void *w_enc_t_bf16, void *pre_bf16, int64_t B, int64_t d,
                                                int64_t F, const float *b_enc, const float *scale, const float *theta,
                                                float *granule_margin, void *stream) {
  using namespace sae;
  SAE_REQUIRE(x_bf16 && w_enc_t_bf16 && pre_bf16 && theta && granule_margin, SAE_ERR_INVALID_ARG,
              "encoder_gemm_jumprelu_margin: null pointer");
  SAE_REQUIRE(B > 0 && d > 0 && F > 0, SAE_ERR_INVALID_ARG, "encoder_gemm_jumprelu_margin: sizes must be positive");
  SAE_REQUIRE(B < (1LL << 31) && F < (1LL << 31) && d < (1LL << 28), SAE_ERR_UNSUPPORTED, "encoder_gemm_jumprelu_margin: size too large");
  SAE_REQUIRE(d % 64 == 0 && F % 64 == 0, SAE_ERR_UNSUPPORTED, "encoder_gemm_jumprelu_margin: d=%lld and F=%lld must be multiples of 64",
              (long long)d, (long long)F);
  SAE_REQUIRE((((uintptr_t)x_bf16 | (uintptr_t)w_enc_t_bf16 | (uintptr_t)pre_bf16 | (uintptr_t)b_enc | (uintptr_t)scale |
                (uintptr_t)theta) & 15) == 0, SAE_ERR_INVALID_ARG, "encoder_gemm_jumprelu_margin: pointers must be 16-byte aligned");
  return launch_gemm_bf16<true, EPI_MARGIN>(x_bf16, w_enc_t_bf16, pre_bf16, B, d, F, b_enc, scale,
                                            reinterpret_cast<uint32_t *>(granule_margin), (hipStream_t)stream, 1, theta);
}
