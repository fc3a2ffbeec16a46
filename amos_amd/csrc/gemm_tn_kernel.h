// GEMM / batched GEMM with both operands K-contiguous ("ntn": A[M,K], B stored [N,K]),
// the layout v_mfma wants: every lane's operand fragment is 16 contiguous bytes of K.
//
// Block tile BI x BJ (256x256 for large problems; 128x128, 128x256, 256x128 where those fill
// the chip better), K step 128 bytes per row (64 halves / 128 int8), NS LDS stages of
// (BI + BJ) * 128 bytes (two for 256x256; the smaller tiles, whose workgroups are often alone on
// a CU, keep three or four tiles in flight).  Differences to the generic implicit-GEMM kernel:
//   * global -> LDS copies are direct (global_load_lds_dwordx4): no staging
//     registers, no ds_write; the XOR swizzle of the LDS layout is applied on the
//     global-address side (a wave instruction fills 1 KB of LDS linearly, lane l
//     fetches the 16-byte chunk that belongs at that position);
//   * operand fragments are double buffered in registers: the ds_reads of the next half
//     sub-step are in flight while the MFMAs (16x16x32, int8 16x16x64) of this one issue;
//   * one barrier per K step; the copies for step kt+NS are issued right after it and
//     have NS-1 steps to land.  Every step issues a tile (steps past the end fetch the last
//     one again), so that the number of copies in flight behind the tile a step waits for
//     is the same at every step.
// Rows beyond M / N are clamped to the last valid row on load (their products only
// reach outputs that are never stored); K must be a multiple of the K step.
//
// Role in the reference: the "kernel2" main loop that
// python/tvm/auto_tensorize/tensorization_phases/schedulers/cuda_v2.py:582-825
// schedules (cache_read to shared, load_matrix_sync, mma_sync, store_matrix_sync;
// README.md:369-424) -- there with synchronous copies and no double buffering.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "igemm_kernel.h"

namespace amos {

struct GemmTnParams {
  const char* a;   // row operand, [I][lda] elements, K contiguous
  const char* b;   // column operand, [J][ldb]
  char* c;         // [I][ldc] fp32 / int32
  int I, J, K;
  int64_t lda, ldb, ldc;
  int64_t batch_a, batch_b, batch_c;  // elements between batches
  int tiles_i, tiles_j;
  int kt_per_split;       // split-K: blockIdx.y takes the K tiles [y * kt_per_split, (y + 1) * kt_per_split) ...
  int64_t split_stride;   // ... and stores its partial sums at c + y * split_stride (0: no split)
  EpiParams epi;   // fused tail: C = acc + cast(D), D[i][j] at i*epi.si + j
#if AMOS_SPLIT_IN_KERNEL
  SplitFinish fin; // split-K: the last workgroup of a tile adds the slices
#endif
};

#define AMOS_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define AMOS_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

// The 16x16 matrix-core shapes (v_mfma_f32_16x16x32_f16 / _bf16, v_mfma_i32_16x16x64_i8): the same
// flops per LDS byte as 32x32x16 on the same wave tile, and measured 3-8 % faster at every tile here
// (on random operands the chip sustains a higher clock under them).  An operand fragment is
// row = lane % 16 and one 16-byte chunk of a 64-byte K sub-step per lane group lane / 16.
template <int DT>
struct Mfma16;
template <>
struct Mfma16<DT_F16> {
  typedef float acc_t __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ acc_t run(v4i a, v4i b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
};
template <>
struct Mfma16<DT_BF16> {
  typedef float acc_t __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ acc_t run(v4i a, v4i b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  }
};
template <>
struct Mfma16<DT_I8> {
  typedef int acc_t __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ acc_t run(v4i a, v4i b, acc_t c) {
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
  }
};

// A K step (128 bytes per row) is two sub-steps of 64 bytes; each is issued in two halves over the
// wave tile's rows, so that the fragment registers in flight stay at two half-sets of A and two
// sets of B while the reads of the next half are in flight behind the MFMAs of this one.
template <int DT, int WI, int WJ, int BI = 256, int BJ = 256, int NS = 2>
__global__ __launch_bounds__(64 * WI * WJ) void amos_gemm_tn(const GemmTnParams p) {
  typedef Mfma16<DT> MM;
  typedef typename MM::acc_t acc_t;
  typedef typename Mfma<DT>::out_t out_t;
  constexpr int ES = Mfma<DT>::ES;
  constexpr int BKE = 128 / ES;
  constexpr int NW = WI * WJ;
  constexpr int TI = BI / (16 * WI), TJ = BJ / (16 * WJ);   // 16x16 blocks of the wave tile
  constexpr int HA = TI / 2;                                // A blocks per half
  static_assert(TI % 2 == 0 && TI * WI * 16 == BI && TJ * WJ * 16 == BJ && TJ >= 1, "wave tile");
  // the swizzle term of a fragment offset repeats every 64 rows: offsets of up to four blocks are
  // kept, the others are those plus whole 64-row strides
  constexpr int AO = TI < 4 ? TI : 4, BO = TJ < 4 ? TJ : 4;
  static_assert((TI <= 4 || (TI * 16) % 64 == 0) && (TJ <= 4 || (TJ * 16) % 64 == 0), "offset reuse");
  constexpr int OPER = BI * 128;
  constexpr int STAGE = (BI + BJ) * 128;
  constexpr int QA = BI / 8;
  constexpr int CH = (BI + BJ) / 8 / NW;
  static_assert(CH >= 1 && CH * NW * 8 == BI + BJ, "copy chunks");

  extern __shared__ __attribute__((aligned(16))) char smem[];

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wi = wave / WJ, wj = wave % WJ;

  int tile_i, tile_j;
  int64_t batch = blockIdx.z;
  // A batch of small products (its tiles fewer than the chip's workgroup slots): workgroups are
  // dealt round-robin to the 8 XCDs in launch order (x fastest, then z), which spreads the tiles
  // of one batch over all XCDs -- every L2 then fetches that batch's row and column panels.  Where
  // the counts allow it, XCD x takes whole batches x, x + 8, ...: its s-th workgroup is tile
  // s % T of batch x + 8 * (s / T), and a batch's panels are fetched by one L2 only.
  if (gridDim.z > 1 && gridDim.y == 1 && (gridDim.z & 7) == 0) {
    const unsigned T = gridDim.x, L = blockIdx.x + T * blockIdx.z;
    const unsigned xcd = L & 7, sq = L >> 3;
    const unsigned tile = sq % T;
    batch = xcd + 8 * (sq / T);
    const int per_group = 8 * p.tiles_j;   // (the walk of block_to_tile without its own XCD permutation)
    const int gidx = (int)tile / per_group, first_i = gidx * 8;
    const int rows_here = p.tiles_i - first_i < 8 ? p.tiles_i - first_i : 8;
    const int in_group = (int)tile - gidx * per_group;
    tile_i = first_i + in_group % rows_here;
    tile_j = in_group / rows_here;
  } else {
    block_to_tile(blockIdx.x, gridDim.x, p.tiles_i, p.tiles_j, tile_i, tile_j);
  }
  const int bi0 = tile_i * BI, bj0 = tile_j * BJ;
  const char* const abase = p.a + (batch * p.batch_a + (int64_t)bi0 * p.lda) * ES;
  const char* const bbase = p.b + (batch * p.batch_b + (int64_t)bj0 * p.ldb) * ES;

  unsigned g_off[CH];
#pragma unroll
  for (int u = 0; u < CH; ++u) {
    const int q = wave + NW * u;
    const int qq = q < QA ? q : q - QA;
    const int row = qq * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row ^ (row >> 3)) & 7);
    if (q < QA) {
      int r = bi0 + row < p.I ? row : p.I - 1 - bi0;
      g_off[u] = (unsigned)r * (unsigned)(p.lda * ES) + chunk * 16;
    } else {
      int r = bj0 + row < p.J ? row : p.J - 1 - bj0;
      g_off[u] = (unsigned)r * (unsigned)(p.ldb * ES) + chunk * 16;
    }
  }

  // this block's K tiles: all of them, or blockIdx.y's share of a split-K launch
  const int kt0 = p.kt_per_split ? (int)blockIdx.y * p.kt_per_split : 0;
  auto issue_copies = [&](int kt, int stage) {
    const char* ak = abase + (int64_t)(kt0 + kt) * 128;
    const char* bk = bbase + (int64_t)(kt0 + kt) * 128;
    char* s = smem + stage * STAGE;
#pragma unroll
    for (int u = 0; u < CH; ++u) {
      const int q = wave + NW * u;
      const char* src = (q < QA ? ak : bk) + g_off[u];
      __builtin_amdgcn_global_load_lds(AMOS_GLOBAL_PTR(src), AMOS_LDS_PTR(s + q * 1024), 16, 0, 0);
    }
  };

  // Lane group q = lane / 16 feeds the matrix core's K positions [8q, 8q + 8) of a sub-step; which
  // 16-byte chunk of the tile it takes them from is free as long as both operands agree (a dot
  // product does not care about the order of K).  A 16-byte LDS read serves lanes l and l + 32 in
  // the same cycle, so groups q and q + 2 take chunks that differ in the lowest bit, which the
  // swizzle maps to different banks: chunks 0, 2, 1, 3 for q = 0..3.  (With chunk = q the
  // conflict counter read half of all LDS cycles.)
  const int frag_row = lane & 15, frag_q = lane >> 4;
  const int frag_chunk = (frag_q >> 1) | ((frag_q & 1) << 1);
  int a_off[AO][2], b_off[BO][2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
    for (int a = 0; a < AO; ++a)
      a_off[a][ks] = lds_chunk_offset(wi * TI * 16 + a * 16 + frag_row, ks * 4 + frag_chunk);
#pragma unroll
    for (int b = 0; b < BO; ++b)
      b_off[b][ks] = OPER + lds_chunk_offset(wj * TJ * 16 + b * 16 + frag_row, ks * 4 + frag_chunk);
  }

  acc_t acc[TI][TJ];
#pragma unroll
  for (int a = 0; a < TI; ++a)
#pragma unroll
    for (int b = 0; b < TJ; ++b)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[a][b][r] = 0;

  v4i af[2][HA], bf[2][TJ];
  auto read_a = [&](int stage, int ks, int h, int slot) {
    const char* s = smem + stage * STAGE;
#pragma unroll
    for (int a = 0; a < HA; ++a) {
      const int ab = h * HA + a;
      af[slot][a] = *(const v4i*)(s + a_off[ab & 3][ks] + (ab >> 2) * (64 * 128));
    }
  };
  auto read_b = [&](int stage, int ks, int slot) {
    const char* s = smem + stage * STAGE;
#pragma unroll
    for (int b = 0; b < TJ; ++b) bf[slot][b] = *(const v4i*)(s + b_off[b & 3][ks] + (b >> 2) * (64 * 128));
  };
  auto mma = [&](int h, int sa, int sb) {   // (B fragment outermost: measured 1 % ahead of A outermost)
#pragma unroll
    for (int b = 0; b < TJ; ++b)
#pragma unroll
      for (int a = 0; a < HA; ++a) acc[h * HA + a][b] = MM::run(af[sa][a], bf[sb][b], acc[h * HA + a][b]);
  };

  int KT = p.K / BKE - kt0;
  if (p.kt_per_split && KT > p.kt_per_split) KT = p.kt_per_split;
  static_assert(NS >= 2 && (NS - 1) * CH <= 63, "stages");
#pragma unroll
  for (int s = 0; s < NS; ++s) issue_copies(s < KT ? s : KT - 1, s);
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((NS - 1) * CH) : "memory");
  read_a(0, 0, 0, 0);
  read_b(0, 0, 0);

  int st = 0;
  for (int kt = 0; kt < KT; ++kt) {
    const int st_next = st + 1 == NS ? 0 : st + 1;
    read_a(st, 0, 1, 1);
    mma(0, 0, 0);
    read_a(st, 1, 0, 0);
    read_b(st, 1, 1);
    mma(1, 1, 0);
    read_a(st, 1, 1, 1);
    mma(0, 0, 1);
    // every ds_read of this stage has been issued; once they and this wave's copies of the
    // next tile are complete (the NS-2 tiles behind it may still be in flight), meet the other
    // waves: after the barrier the next stage is fully written and this stage is free to be
    // overwritten
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"((NS - 2) * CH) : "memory");
    issue_copies(kt + NS < KT ? kt + NS : KT - 1, st);
    if (kt + 1 < KT) {
      read_a(st_next, 0, 0, 0);
      read_b(st_next, 0, 0);
    }
    mma(1, 1, 1);
    st = st_next;
  }

  // ---- epilogue: lane holds column j = lane % 16 of rows 4 * (lane / 16) + r of every block
  // Where C's rows are 16-byte aligned a row block goes through a private LDS strip of the wave
  // (16 rows x the wave tile's width) and leaves as 16-byte stores that cover whole rows of the
  // wave tile: 64 / (4 TJ) rows x 64 TJ bytes per instruction instead of four rows x 64 bytes.
  // LDS operations of one wave complete in issue order, so the strip needs no barrier of its own.
  out_t* const out = (out_t*)p.c + batch * p.batch_c + (int64_t)blockIdx.y * p.split_stride;
  constexpr int SP = TJ * 16 + 4;          // strip row pitch in elements
  constexpr int CPR = TJ * 4, RPI = 64 / CPR;   // 16-byte chunks per row, rows per store instruction
  static_assert(TJ <= 16 && (TJ & (TJ - 1)) == 0 && NW * 16 * SP * 4 <= NS * STAGE, "output strip");
  // (measured: the 64- and 128-column wave tiles 4-5 % faster through the strip; the 32-column
  // tile of the store-bound 192 x (512x512x64) batched product 2 % faster once an XCD's workgroups
  // write one batch's rows instead of eight batches')
  const bool vec_out = TJ >= 2 && ((((uintptr_t)out) & 15) | (uintptr_t)(p.ldc & 3) | (uintptr_t)(p.J & 3)) == 0;
  out_t* const strip = (out_t*)(smem + wave * (16 * SP * 4));
  // the last K steps re-issue copies of the final tile: they (any wave's) must have landed, and
  // every wave must be done with its fragment reads, before the stages are reused
  if (vec_out) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
  for (int a = 0; a < TI; ++a) {
    const int i0 = bi0 + (wi * TI + a) * 16 + 4 * frag_q;
    if (p.epi.dt != EPI_NONE && blockIdx.y == 0) {   // (one K split adds D) the row block's loads in flight before the first addition
      out_t dv[TJ][4];
#pragma unroll
      for (int b = 0; b < TJ; ++b) {
        const int j = bj0 + (wj * TJ + b) * 16 + frag_row;
        const int jc = j < p.J ? j : p.J - 1;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int i = i0 + r;
          dv[b][r] = epi_value<out_t>(p.epi, batch * p.epi.batch + (int64_t)(i < p.I ? i : p.I - 1) * p.epi.si + jc);
        }
      }
#pragma unroll
      for (int b = 0; b < TJ; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[a][b][r] += dv[b][r];
    }
    if (vec_out) {
#pragma unroll
      for (int b = 0; b < TJ; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) strip[(4 * frag_q + r) * SP + b * 16 + frag_row] = acc[a][b][r];
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      acc_t v[TJ];
#pragma unroll
      for (int n = 0; n < TJ; ++n) v[n] = *(const acc_t*)(strip + (n * RPI + lane / CPR) * SP + (lane % CPR) * 4);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      const int j = bj0 + wj * TJ * 16 + (lane % CPR) * 4;
#pragma unroll
      for (int n = 0; n < TJ; ++n) {
        const int i = bi0 + (wi * TI + a) * 16 + n * RPI + lane / CPR;
        if (i < p.I && j < p.J) *(acc_t*)(out + (int64_t)i * p.ldc + j) = v[n];
      }
      continue;
    }
#pragma unroll
    for (int b = 0; b < TJ; ++b) {
      const int j = bj0 + (wj * TJ + b) * 16 + frag_row;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = i0 + r;
        if (i < p.I && j < p.J) out[(int64_t)i * p.ldc + j] = acc[a][b][r];
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#if AMOS_SPLIT_IN_KERNEL
  if (p.fin.tickets) {
    // (the tile index is taken from the launch grid, whatever walk mapped it to (tile_i, tile_j))
    split_finish<out_t>(p.fin, (unsigned)(blockIdx.z * gridDim.x + blockIdx.x), (const out_t*)p.c, t, 64 * NW, BI, BJ,
                        (lds_flag_t)smem, [&](int r, int c) -> int64_t {
                          const int i = bi0 + r, j = bj0 + c;
                          return i < p.I && j < p.J ? batch * p.batch_c + (int64_t)i * p.ldc + j : (int64_t)-1;
                        });
  }
#endif
}

}  // namespace amos
