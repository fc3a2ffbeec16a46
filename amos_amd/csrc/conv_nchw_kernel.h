// Implicit-GEMM forward convolution (3x3 windows, conv2d / conv3d) that reads the tensors as the
// caller holds them -- NCDHW activations, KCTRS weights -- in ONE launch and without a workspace:
//
//   Out(i = output channel, j = (image, od, op, oq)) = sum_k W(i, k) * Col(j, k),  k = (t, c, r, s)
//
// The matrix core wants, per lane, 16 contiguous bytes of K of one row / column.  Neither tensor
// offers that (in NCDHW the positions are contiguous, in KCTRS the window taps), so both operands
// are transposed in registers on their way from global memory to LDS:
//   * activations: a thread fetches, for one 16-byte chunk of channels, one 8-byte run of input
//     positions per channel (coalesced: 16 lanes cover 128 contiguous bytes of a channel plane),
//     turns them with byte permutes into one 16-byte vector of channels per position and stores
//     those into the zero-padded patch [position][64 bytes of channels] of the tile;
//   * weights: a thread fetches the nine taps of a chunk of channels of one output channel (144
//     contiguous bytes in 2-d; per channel an unaligned 18 / 9 byte run in 3-d), and writes one
//     16-byte vector of channels per tap into that tap's weight tile [row][64 bytes].
// A macro step is (depth tap, 64 bytes of channels): its patch serves all nine taps (a tap only
// shifts the position a lane reads) and its nine weight tiles are resident together, both double
// buffered, so a workgroup meets at ONE barrier per macro step = per nine K steps; the loads of
// macro step m+2 and the transposition of m+1 run under the matrix-core work of m.
//
// What the reference does here: separate kernels write the padded tensor, the im2col matrix and
// the reordered weights to memory before its "kernel2" (README.md:344-424,
// src/auto_tensorize/compute_transform.cc:181-293), and one more scatters the result
// (compute_transform.cc:439-497); its main loop copies synchronously between two barriers per
// step (python/tvm/auto_tensorize/tensorization_phases/schedulers/cuda_v2.py:582-825).
#pragma once
#define AMOS_CONV_NCHW_KERNEL_INCLUDED 1
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "conv_nchw_geom.h"
#include "gemm_tn_kernel.h"
#include "igemm_kernel.h"

namespace amos {

struct ConvNchwParams {
  const char* x;   // [N][C][D][H][W]
  const char* w;   // [K][C][T][3][3]
  char* y;         // [N][K][OD][OP][OQ] fp32 / int32
  NchwShape s;
  int c_chunks;          // C * esize / 64
  int macro_steps;       // T * c_chunks; macro step m = (depth tap m / c_chunks, chunk m % c_chunks)
  int macro_per_split;   // macro steps of one blockIdx.y
  int tiles_i, tiles_j;
  int max_pos;           // LDS positions of one patch buffer (multiple of 4)
  int64_t split_stride;  // elements between the partial outputs of the split-K blocks
  NchwDiv div_cc, div_odpq;
  EpiParams epi;         // fused tail: Y = acc + cast(D), D laid out like Y
  long long* dbg;        // DEBUG: per-workgroup timestamps
  int dbg_flags;         // DEBUG: 1 = no staging stores, 2 = no global loads after the prologue
};

#define AMOS_LDS_ADDR(off) ((__attribute__((address_space(3))) char*)(size_t)(off))
enum { NCHW_W_KCTRS = 0, NCHW_W_KCRS = 1, NCHW_W_PACKED = 2 };
template <int N> struct NchwSet { static constexpr int value = N; };
// f(NchwSet<B>{}), ..., f(NchwSet<E - 1>{}): a loop whose counter is a constant in every iteration
template <int B, int E, typename F>
__device__ __forceinline__ void nchw_static_for(F&& f) {
  if constexpr (B < E) {
    f(NchwSet<B>{});
    nchw_static_for<B + 1, E>(f);
  }
}
struct __attribute__((packed, aligned(2))) NchwUnaligned16 { v4i v; };
struct __attribute__((packed, aligned(1))) NchwUnaligned8 { uint2 v; };

// one dword of a transposed vector: its four bytes are bytes B0..B3 of `raw` seen as a byte array
// (all indices are constants once the callers' loops are unrolled)
template <int ES>
__device__ __forceinline__ unsigned nchw_gather(const unsigned* raw, int B0, int B1, int B2, int B3) {
  if (ES == 2) {   // B1 = B0 + 1 and B3 = B2 + 1 inside one dword each: a single permute
    const unsigned sel = (unsigned)(B0 & 3) | ((unsigned)((B0 & 3) + 1) << 8) | ((unsigned)(4 + (B2 & 3)) << 16) |
                         ((unsigned)(5 + (B2 & 3)) << 24);
    return __builtin_amdgcn_perm(raw[B2 >> 2], raw[B0 >> 2], sel);
  }
  const unsigned lo = __builtin_amdgcn_perm(raw[B1 >> 2], raw[B0 >> 2], (unsigned)(B0 & 3) | ((unsigned)(4 + (B1 & 3)) << 8));
  const unsigned hi = __builtin_amdgcn_perm(raw[B3 >> 2], raw[B2 >> 2], (unsigned)(B2 & 3) | ((unsigned)(4 + (B3 & 3)) << 8));
  return __builtin_amdgcn_perm(hi, lo, 0x05040100u);
}

// Weights KCTRS -> [K][T*R*S][C]: with the channels innermost a (row, tap)'s chunk of channels is
// one contiguous 64-byte run, which the convolution kernel copies as it is.  One thread per 16
// bytes of the result.  (The reference's counterpart is the stage that materialises the reordered
// weight operand in front of its main kernel, src/auto_tensorize/compute_transform.cc:181-293.)
template <typename T>
__global__ __launch_bounds__(256) void amos_conv_pack_weights_kernel(const T* __restrict__ w, T* __restrict__ out,
                                                                     int K, int C, int TRS, NchwDiv div_chunks,
                                                                     NchwDiv div_trs) {
  constexpr int CE = 16 / (int)sizeof(T);
  const int chunks = C / CE;
  const int total = K * TRS * chunks;   // (the host keeps the tensor below 4 GiB)
  for (int idx = (int)(blockIdx.x * 256 + threadIdx.x); idx < total; idx += (int)(gridDim.x * 256)) {
    const int r = nchw_div(idx, div_chunks), cc = idx - r * chunks;
    const int k = nchw_div(r, div_trs), tap = r - k * TRS;
    const T* src = w + ((int64_t)k * C + cc * CE) * TRS + tap;
    T v[CE];
#pragma unroll
    for (int e = 0; e < CE; ++e) v[e] = src[(int64_t)e * TRS];
    *(uint4*)(out + ((int64_t)r * C + cc * CE)) = *(const uint4*)v;
  }
}

// bytes of one patch buffer: a constant of the tile, so that the second buffer is an immediate
// offset of every LDS access; the last 1 KB of a buffer is a dump line for stores that have no
// position to go to (one 16-byte slot per lane)
constexpr int nchw_patch_buffer_bytes(int bj) { return bj <= 128 ? 32 * 1024 : 40 * 1024; }
constexpr int nchw_max_positions(int bj) { return nchw_patch_buffer_bytes(bj) / kNchwPosBytes - 16; }

// BI x BJ: output channels x output positions of a workgroup; WI x WJ: its wave grid; PT: load
// groups a thread may own per macro step; WMODE: where the weights come from -- NCHW_W_KCTRS: the
// caller's tensor, per channel an unaligned run of nine taps; NCHW_W_KCRS: the same where a chunk
// of channels is one contiguous, 16-byte aligned run (conv2d with aligned weights);
// NCHW_W_PACKED: [K][T*9][C], written by amos_conv_pack_weights (into the workspace by the same
// call, or once by the owner of the weights): 16-byte loads that four lanes per row make
// contiguous, no transposition; DEPTH: macro steps a global load
// has to land (1 or 2 sets of staging registers); OCC: waves per SIMD the compiler leaves room for
// (the register budget of a wave is 512 / OCC)
template <int DT, int BI, int BJ, int WI, int WJ, int PT, int WMODE, int DEPTH, int OCC>
__global__ __launch_bounds__(64 * WI * WJ, OCC) void amos_conv_nchw(const ConvNchwParams p) {
  typedef Mfma16<DT> MM;
  typedef typename MM::acc_t acc_t;
  typedef typename Mfma<DT>::out_t out_t;
  constexpr int ES = Mfma<DT>::ES;
  constexpr int NW = WI * WJ, NT = 64 * NW;
  constexpr int TI = BI / (16 * WI), TJ = BJ / (16 * WJ);
  static_assert(TI >= 1 && TJ >= 1 && TI * WI * 16 == BI && TJ * WJ * 16 == BJ, "wave tile");
  constexpr int PG = 8 / ES;      // input positions per 8-byte load
  constexpr int CG = 16 / ES;     // channels per 16-byte chunk
  constexpr int CK = 64 / ES;     // channels per macro step
  constexpr int RS = 9;
  constexpr int WTILE = BI * 64;  // one tap's weight tile
  constexpr int WBUF = RS * WTILE;
  constexpr int PBUF = nchw_patch_buffer_bytes(BJ);
  constexpr int UNITS = BI * 4;   // (row, chunk of channels) pairs of a macro step's weights
  constexpr int WU = (UNITS + NT - 1) / NT;
  constexpr bool T1 = WMODE == NCHW_W_KCRS, PACKED = WMODE == NCHW_W_PACKED;
  constexpr int CHW = T1 ? 0 : (ES == 2 ? 5 : 3);       // dwords of one channel's taps (3-d path)
  constexpr int WRAW = T1 ? 36 : CG * CHW;              // dwords of a unit's raw weights
  // packed weights: a thread copies one 16-byte chunk of one row of one tap per item; the taps of
  // a macro step are 9 * BI * 4 items = 4.5 per thread (taps 2v and 2v + 1 for the lower / upper
  // half of the threads)
  static_assert(BI * 8 == NT, "a tap's weight tile is half a round of the threads' chunks");
  constexpr int WITEMS = 5;
  static_assert(DEPTH == 1 || DEPTH == 2, "one or two sets of staging registers");
  // LDS, by byte offset from 0 (the kernel has no static LDS; the host checks that):
  //   [2][9][BI * 64] weight tiles | [2][PBUF] patches, the last 1 KB of each a dump line
  constexpr unsigned PBASE = 2 * WBUF;
  constexpr unsigned DUMP = PBUF - 1024;

  const NchwShape& s = p.s;
  const int t = threadIdx.x;
  int dbg_k = 0;
  auto stamp = [&]() __attribute__((always_inline)) { if (p.dbg && t == 0 && dbg_k < 16) p.dbg[blockIdx.x * 16 + dbg_k++] = clock64(); };
  stamp();
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wi = wave / WJ, wj = wave % WJ;
  const int frag_row = lane & 15, frag_q = lane >> 4;

  // Workgroups are dealt round-robin to the 8 XCDs: give each XCD a contiguous run of tiles, the
  // tiles of one patch (tile_i fastest) next to each other, so that an XCD's L2 sees a patch once
  int logical;
  {
    const int n_wg = (int)gridDim.x, wg = (int)blockIdx.x;
    const int x = wg & 7, per = n_wg >> 3, rem = n_wg & 7;
    logical = x * per + (x < rem ? x : rem) + (wg >> 3);
  }
  const int tile_j = logical / p.tiles_i, tile_i = logical - tile_j * p.tiles_i;
  const int bi0 = tile_i * BI, bj0 = tile_j * BJ;
  const int HW = s.H * s.W;
  const int64_t DHW = (int64_t)s.D * HW;
  // ---- this thread's share of the weights ----------------------------------------------------------
  unsigned w_src[WU];   // byte offset of (row, first channel of the chunk): below 4 GiB
  unsigned w_dst[WU];   // LDS address inside a tap's tile of the first buffer
  bool w_on[WU];
  const int TRS = s.T * RS;
  const int upper = __builtin_amdgcn_readfirstlane(t >= NT / 2 ? 1 : 0);   // packed: which of a pair of taps
#pragma unroll
  for (int v = 0; v < WU; ++v) {
    // (with fewer units than threads they go to the last waves: the first ones own the patch's
    // load groups, and a macro step waits for the wave with the most staging work)
    const int u = PACKED ? (t & (NT / 2 - 1)) : UNITS < NT ? t - (NT - UNITS) : t + NT * v;
    // (lanes 4x .. 4x+3 of a wave take row nchw_row_of_slot(x) of their sixteen: no bank conflicts)
    const int cq = u & 3, row = ((u >> 6) * 16 + nchw_row_of_slot((u >> 2) & 15)) & (BI - 1);
    w_on[v] = u >= 0 && u < UNITS;
    const int k = bi0 + row < s.K ? bi0 + row : s.K - 1;
    if (PACKED) {
      w_src[v] = (unsigned)(((int64_t)k * TRS * s.C) * ES + cq * 16);
      w_dst[v] = (unsigned)(nchw_position_offset(row, cq) + upper * WTILE);
    } else {
      w_src[v] = (unsigned)((((int64_t)k * s.C + cq * CG) * TRS) * ES);
      w_dst[v] = (unsigned)nchw_position_offset(row, cq);
    }
  }
  const int m_begin = blockIdx.y * p.macro_per_split;
  int m_end = m_begin + p.macro_per_split;
  if (m_end > p.macro_steps) m_end = p.macro_steps;

  unsigned wraw[DEPTH][WU][PACKED ? WITEMS * 4 : WRAW];
  unsigned praw[DEPTH][PT][CG][2];

  auto load_weights = [&](auto set_c, int m) __attribute__((always_inline)) {
    constexpr int SET = decltype(set_c)::value;
    const int tt = nchw_div(m, p.div_cc), cc = m - tt * p.c_chunks;
    // (a wave-uniform base plus a 32-bit lane offset: one address register per load, not two)
    if constexpr (PACKED) {
      // tap 2v + upper of this macro step: row k's 64 bytes of the chunk at [k][tt * 9 + tap][cc * CK]
      const char* const wm = p.w + (((int64_t)tt * RS + upper) * s.C + (int64_t)cc * CK) * ES;
#pragma unroll
      for (int v = 0; v < WITEMS; ++v) {
        if (2 * v + upper < RS) {
          const v4i x = *(const v4i*)(wm + (int64_t)(2 * v) * s.C * ES + w_src[0]);
          wraw[SET][0][4 * v] = x.x; wraw[SET][0][4 * v + 1] = x.y; wraw[SET][0][4 * v + 2] = x.z; wraw[SET][0][4 * v + 3] = x.w;
        }
      }
      return;
    }
    const char* const wm = p.w + ((int64_t)cc * CK * TRS + tt * RS) * ES;
#pragma unroll
    for (int v = 0; v < WU; ++v) {
      if (!w_on[v]) continue;
      const char* src = wm + w_src[v];
      if (T1) {
#pragma unroll
        for (int i = 0; i < 9; ++i) {
          const v4i x = *(const v4i*)(src + i * 16);
          wraw[SET][v][4 * i] = x.x; wraw[SET][v][4 * i + 1] = x.y; wraw[SET][v][4 * i + 2] = x.z; wraw[SET][v][4 * i + 3] = x.w;
        }
      } else {
#pragma unroll
        for (int ci = 0; ci < CG; ++ci) {
          const char* sc = src + (int64_t)ci * TRS * ES;
          if (ES == 2) {
            const v4i x = ((const NchwUnaligned16*)sc)->v;
            wraw[SET][v][ci * CHW] = x.x; wraw[SET][v][ci * CHW + 1] = x.y; wraw[SET][v][ci * CHW + 2] = x.z; wraw[SET][v][ci * CHW + 3] = x.w;
            wraw[SET][v][ci * CHW + 4] = *(const unsigned short*)(sc + 16);
          } else {
            const uint2 x = ((const NchwUnaligned8*)sc)->v;
            wraw[SET][v][ci * CHW] = x.x; wraw[SET][v][ci * CHW + 1] = x.y;
            wraw[SET][v][ci * CHW + 2] = *(const unsigned char*)(sc + 8);
          }
        }
      }
    }
  };
  // the first weights go out before the tile's geometry is worked out
  if (m_begin < m_end) load_weights(NchwSet<0>{}, m_begin);

  const NchwTile tile = nchw_tile(s, bj0, BJ);

  // ---- this thread's load groups of the patch ------------------------------------------------
  unsigned p_src[PT];      // byte offset of (image, first channel of the chunk, depth 0, group): below 4 GiB
  int p_d0[PT];            // input depth at depth tap 0
  bool p_on[PT];
  unsigned p_dst[PT][PG];  // LDS addresses (first buffer) of the group's positions; the dump line
                           // for positions that are not part of the window
#pragma unroll
  for (int v = 0; v < PT; ++v) {
    const int q = t + NT * v;
    const int cg = q & 3, grp = q >> 2;
    p_on[v] = grp < tile.ngroups;
    int f = 0;
    const NchwSeg seg = nchw_group(s, tile, p_on[v] ? grp : 0, &f);
    p_src[v] = (unsigned)((((int64_t)seg.n * s.C + cg * CG) * DHW + f) * ES);
    p_d0[v] = seg.d0;
#pragma unroll
    for (int i = 0; i < PG; ++i) {
      // (the upper half of a wave stores its positions in the order 1, 0, 3, 2, ...: see the bank
      // conflict notes of the geometry header)
      const int off = p_on[v] ? nchw_writer_offset(s, seg, f + (i ^ (lane >> 5)), cg) : -1;
      p_dst[v][i] = PBASE + (off >= 0 ? (unsigned)off : DUMP + (unsigned)lane * 16);
    }
  }
  // byte selectors that pick position i (lower half of the wave) or i ^ 1 (upper half) out of a
  // staging dword: 16-bit types hold two positions per dword, int8 four
  unsigned p_sel[ES == 2 ? 2 : 4];
#pragma unroll
  for (int i = 0; i < (ES == 2 ? 2 : 4); ++i) {
    const int pos = i ^ (lane >> 5);
    p_sel[i] = ES == 2 ? (pos ? 0x07060302u : 0x05040100u) : ((unsigned)pos | ((unsigned)(4 + pos) << 8));
  }
  // ---- fragment addresses: all of them are computed here, the loop only adds immediates ----------
  // weights: [buffer][16-row block]; patch: [tap][16-position block], first buffer
  unsigned a_addr[2][TI];
#pragma unroll
  for (int a = 0; a < TI; ++a) {
    const int row = (wi * TI + a) * 16 + frag_row;
    a_addr[0][a] = (unsigned)nchw_position_offset(row, nchw_frag_chunk(frag_q));
    a_addr[1][a] = a_addr[0][a] + WBUF;
  }
  unsigned b_addr[RS][TJ];
#pragma unroll
  for (int b = 0; b < TJ; ++b) {
    int j = bj0 + (wj * TJ + b) * 16 + frag_row;
    if (j > tile.j_last) j = tile.j_last;
    const int column = nchw_column(s, tile, j);
#pragma unroll
    for (int tap = 0; tap < RS; ++tap)
      b_addr[tap][b] = PBASE + (unsigned)nchw_reader_offset(s, column, tap / 3, tap % 3, nchw_frag_chunk(frag_q));
  }

  auto load_patch = [&](auto set_c, int m) __attribute__((always_inline)) {
    constexpr int SET = decltype(set_c)::value;
    const int tt = nchw_div(m, p.div_cc), cc = m - tt * p.c_chunks;
#pragma unroll
    for (int v = 0; v < PT; ++v) {
      const int d = p_d0[v] + tt * s.dd;
      if (p_on[v] && (unsigned)d < (unsigned)s.D) {
        // (the depth is the lane's own: its offset stays below 4 GiB like the rest of the tensor)
        const unsigned off = p_src[v] + (unsigned)d * (unsigned)(HW * ES);
#pragma unroll
        for (int ci = 0; ci < CG; ++ci) {
          const char* const xm = p.x + ((int64_t)cc * CK + ci) * DHW * ES;
          const uint2 x = *(const uint2*)(xm + off);
          praw[SET][v][ci][0] = x.x; praw[SET][v][ci][1] = x.y;
        }
      } else {
#pragma unroll
        for (int ci = 0; ci < CG; ++ci) { praw[SET][v][ci][0] = 0; praw[SET][v][ci][1] = 0; }
      }
    }
  };
  auto load_both = [&](auto set_c, int m) __attribute__((always_inline)) {
    if (m < m_end) {
      load_weights(set_c, m);
      load_patch(set_c, m);
    }
  };
  // raw byte index of byte bb of channel ci at tap tap
  auto wbyte = [](int ci, int tap, int bb) __attribute__((always_inline)) {
    return T1 ? (ci * 9 + tap) * ES + bb : ci * CHW * 4 + tap * ES + bb;
  };
  // tap `tap` of this thread's weight units of the next macro step: one 16-byte vector of channels
  auto stage_weights_tap = [&](auto set_c, auto buf_c, auto tap_c) __attribute__((always_inline)) {
    constexpr int SET = decltype(set_c)::value;
    constexpr int tap = decltype(tap_c)::value;
    constexpr unsigned OFF = decltype(buf_c)::value * WBUF + tap * WTILE;
    if constexpr (PACKED) {
      // item `tap` (of five) is the chunk of tap 2 * tap + upper: stored as it came
      if constexpr (tap < WITEMS) {
        if (2 * tap + upper < RS) {
          const v4i o = {(int)wraw[SET][0][4 * tap], (int)wraw[SET][0][4 * tap + 1], (int)wraw[SET][0][4 * tap + 2],
                         (int)wraw[SET][0][4 * tap + 3]};
          *(v4i*)AMOS_LDS_ADDR(w_dst[0] + decltype(buf_c)::value * WBUF + 2 * tap * WTILE) = o;
        }
      }
      return;
    }
#pragma unroll
    for (int v = 0; v < WU; ++v) {
      if (!w_on[v]) continue;
      v4i o;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (ES == 2)
          o[j] = (int)nchw_gather<ES>(wraw[SET][v], wbyte(2 * j, tap, 0), wbyte(2 * j, tap, 1), wbyte(2 * j + 1, tap, 0),
                                      wbyte(2 * j + 1, tap, 1));
        else
          o[j] = (int)nchw_gather<ES>(wraw[SET][v], wbyte(4 * j, tap, 0), wbyte(4 * j + 1, tap, 0), wbyte(4 * j + 2, tap, 0),
                                      wbyte(4 * j + 3, tap, 0));
      }
      *(v4i*)AMOS_LDS_ADDR(w_dst[v] + OFF) = o;
    }
  };
  // position i of load group v of the next macro step's patch: one 16-byte vector of channels
  auto stage_patch_pos = [&](auto set_c, auto buf_c, auto e_c) __attribute__((always_inline)) {
    constexpr int SET = decltype(set_c)::value;
    constexpr int v = decltype(e_c)::value / PG, i = decltype(e_c)::value % PG;
    v4i o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if constexpr (ES == 2) {
        o[j] = (int)__builtin_amdgcn_perm(praw[SET][v][2 * j + 1][i >> 1], praw[SET][v][2 * j][i >> 1], p_sel[i & 1]);
      } else {
        const unsigned sel = p_sel[i & 3];
        const unsigned lo = __builtin_amdgcn_perm(praw[SET][v][4 * j + 1][i >> 2], praw[SET][v][4 * j][i >> 2], sel);
        const unsigned hi = __builtin_amdgcn_perm(praw[SET][v][4 * j + 3][i >> 2], praw[SET][v][4 * j + 2][i >> 2], sel);
        o[j] = (int)__builtin_amdgcn_perm(hi, lo, 0x05040100u);
      }
    }
    *(v4i*)AMOS_LDS_ADDR(p_dst[v][i] + decltype(buf_c)::value * PBUF) = o;
  };
  // the staging work of a macro step in RS slices, one per tap of the macro step it runs under
  constexpr int PVEC = PT * PG;                       // patch vectors per thread
  constexpr int PPER = (PVEC + RS - 1) / RS;          // ... per slice
  auto stage_slice = [&](auto set_c, auto buf_c, auto tap_c) __attribute__((always_inline)) {
    constexpr int tap = decltype(tap_c)::value;
    stage_weights_tap(set_c, buf_c, tap_c);
    constexpr int E0 = tap * PPER < PVEC ? tap * PPER : PVEC, E1 = (tap + 1) * PPER < PVEC ? (tap + 1) * PPER : PVEC;
    nchw_static_for<E0, E1>([&](auto e_c) { stage_patch_pos(set_c, buf_c, e_c); });
  };

  acc_t acc[TI][TJ];
#pragma unroll
  for (int a = 0; a < TI; ++a)
#pragma unroll
    for (int b = 0; b < TJ; ++b)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[a][b][r] = 0;

  // operand fragments are read NF - 1 taps ahead: a batch of LDS reads takes some 200 cycles to
  // come back, a tap's matrix-core work of a wave 64
  constexpr int NF = TI * TJ >= 8 ? 2 : 3;
  v4i af[NF][TI], bf[NF][TJ];
  auto read_frags = [&](auto buf_c, auto tap_c) __attribute__((always_inline)) {
    constexpr int BUF = decltype(buf_c)::value, tap = decltype(tap_c)::value, slot = tap % NF;
#pragma unroll
    for (int a = 0; a < TI; ++a) af[slot][a] = *(const v4i*)AMOS_LDS_ADDR(a_addr[BUF][a] + tap * WTILE);
#pragma unroll
    for (int b = 0; b < TJ; ++b) bf[slot][b] = *(const v4i*)AMOS_LDS_ADDR(b_addr[tap][b] + BUF * PBUF);
  };
  auto mma = [&](int slot) __attribute__((always_inline)) {
#pragma unroll
    for (int b = 0; b < TJ; ++b)
#pragma unroll
      for (int a = 0; a < TI; ++a) acc[a][b] = MM::run(af[slot][a], bf[slot][b], acc[a][b]);
  };

  stamp();
  // ---- prologue -------------------------------------------------------------------------------------
  // the first loads go out before anything else; the patch buffers are cleared under their latency
  // (padding positions are never written, so both buffers start as zeros)
  if (m_begin < m_end) load_patch(NchwSet<0>{}, m_begin);
  if (DEPTH == 2) load_both(NchwSet<DEPTH - 1>{}, m_begin + 1);
  for (int i = t; i < p.max_pos * 4; i += NT) {
    *(v4i*)AMOS_LDS_ADDR(PBASE + i * 16) = v4i{0, 0, 0, 0};
    *(v4i*)AMOS_LDS_ADDR(PBASE + PBUF + i * 16) = v4i{0, 0, 0, 0};
  }
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  if (m_begin < m_end) {
    nchw_static_for<0, RS>([&](auto tap_c) { stage_slice(NchwSet<0>{}, NchwSet<0>{}, tap_c); });
    load_both(NchwSet<0>{}, m_begin + DEPTH);
  }
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

  stamp();
  // One macro step: nine taps out of buffer BUF; under them the next macro step is transposed
  // from staging set SET into the other buffer (last read a macro step ago) and the set refilled
  // with the loads of the macro step DEPTH further on.
  auto macro_body = [&](auto set_c, auto next_c, auto buf_c, int m) __attribute__((always_inline)) {
    constexpr bool NEXT = decltype(next_c)::value != 0;
    constexpr int BUF = decltype(buf_c)::value;
    read_frags(buf_c, NchwSet<0>{});
    if (NF > 2) read_frags(buf_c, NchwSet<1>{});
    __builtin_amdgcn_sched_barrier(0);
    nchw_static_for<0, RS>([&](auto tap_c) {
      constexpr int tap = decltype(tap_c)::value;
      // (the order below is pinned: left to itself the scheduler moves a tap's fragment reads next
      // to its matrix-core instructions, and every tap then waits for LDS)
      if constexpr (tap + NF - 1 < RS) read_frags(buf_c, NchwSet<tap + NF - 1>{});
      __builtin_amdgcn_sched_barrier(0);
      mma(tap % NF);
      __builtin_amdgcn_sched_barrier(0);
      if (NEXT) {
        if (!(p.dbg_flags & 1)) stage_slice(set_c, NchwSet<BUF ^ 1>{}, tap_c);
        if (tap == RS - 1 && !(p.dbg_flags & 2)) load_both(set_c, m + 1 + DEPTH);
        __builtin_amdgcn_sched_barrier(0);
      }
    });
    // own LDS writes done, every wave through with this macro step's buffers
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    stamp();
  };
  auto macro_step = [&](auto set_c, auto buf_c, int m) __attribute__((always_inline)) {
    if (m + 1 < m_end) macro_body(set_c, NchwSet<1>{}, buf_c, m);
    else macro_body(set_c, NchwSet<0>{}, buf_c, m);
  };
  // macro step m_begin + r computes from buffer r & 1 and stages m + 1 from set (r + 1) % DEPTH
  for (int m = m_begin; m < m_end; m += 2) {
    macro_step(NchwSet<DEPTH == 2 ? 1 : 0>{}, NchwSet<0>{}, m);
    if (m + 1 < m_end) macro_step(NchwSet<0>{}, NchwSet<1>{}, m + 1);
  }

  // ---- epilogue: Y[(n * K + i) * ODPQ + s], a lane holds column j of rows 4 * frag_q + r ----------
  out_t* const out = (out_t*)p.y + (int64_t)blockIdx.y * p.split_stride;
  const int ODPQ = s.OD * s.OP * s.OQ;
  const bool add_d = p.epi.dt != EPI_NONE && blockIdx.y == 0;
#pragma unroll
  for (int b = 0; b < TJ; ++b) {
    const int j = bj0 + (wj * TJ + b) * 16 + frag_row;
    const int jc = j < s.J ? j : s.J - 1;
    const int n = nchw_div(jc, p.div_odpq);
    const int64_t coff = (int64_t)n * s.K * ODPQ + (jc - n * ODPQ);
#pragma unroll
    for (int a = 0; a < TI; ++a) {
      const int i0 = bi0 + (wi * TI + a) * 16 + 4 * frag_q;
      if (add_d) {
        out_t dv[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) dv[r] = epi_value<out_t>(p.epi, coff + (int64_t)(i0 + r < s.K ? i0 + r : s.K - 1) * ODPQ);
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[a][b][r] += dv[r];
      }
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (i0 + r < s.K && j < s.J) out[coff + (int64_t)(i0 + r) * ODPQ] = acc[a][b][r];
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  stamp();
}

}  // namespace amos
