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
};

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

// BI x BJ: output channels x output positions of a workgroup; WI x WJ: its wave grid; PT: load
// groups a thread may own per macro step; T1: the weights of a chunk of channels are one
// contiguous, 16-byte aligned run (conv2d with aligned weights)
template <int DT, int BI, int BJ, int WI, int WJ, int PT, bool T1>
__global__ __launch_bounds__(64 * WI * WJ) void amos_conv_nchw(const ConvNchwParams p) {
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
  constexpr int UNITS = BI * 4;   // (row, chunk of channels) pairs of a macro step's weights
  constexpr int WU = (UNITS + NT - 1) / NT;
  constexpr int CHW = T1 ? 0 : (ES == 2 ? 5 : 3);       // dwords of one channel's taps (3-d path)
  constexpr int WRAW = T1 ? 36 : CG * CHW;              // dwords of a unit's raw weights

  extern __shared__ __attribute__((aligned(16))) char smem[];
  const NchwShape& s = p.s;
  const int t = threadIdx.x;
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
  const NchwTile tile = nchw_tile(s, bj0, BJ);
  const int HW = s.H * s.W;
  const int64_t DHW = (int64_t)s.D * HW;

  // ---- this thread's load groups of the patch ------------------------------------------------
  int64_t p_src[PT];    // element offset of (image, first channel of the chunk, depth 0, group)
  int p_d0[PT];         // input depth at depth tap 0
  bool p_on[PT];
  int p_dst[PT][PG];    // LDS byte offsets of the group's positions, -1 = not part of the window
#pragma unroll
  for (int v = 0; v < PT; ++v) {
    const int q = t + NT * v;
    const int cg = q & 3, grp = q >> 2;
    p_on[v] = grp < tile.ngroups;
    int f = 0;
    const NchwSeg seg = nchw_group(s, tile, p_on[v] ? grp : 0, &f);
    p_src[v] = ((int64_t)seg.n * s.C + cg * CG) * DHW + f;
    p_d0[v] = seg.d0;
#pragma unroll
    for (int i = 0; i < PG; ++i) p_dst[v][i] = p_on[v] ? nchw_writer_offset(s, seg, f + i, cg) : -1;
  }
  // ---- this thread's weight units -------------------------------------------------------------
  int64_t w_src[WU];
  int w_dst[WU];
  bool w_on[WU];
  const int TRS = s.T * RS;
#pragma unroll
  for (int v = 0; v < WU; ++v) {
    const int u = t + NT * v;
    const int cq = u & 3, row = u >> 2;
    w_on[v] = u < UNITS;
    const int k = bi0 + row < s.K ? bi0 + row : s.K - 1;
    w_src[v] = ((int64_t)k * s.C + cq * CG) * TRS;
    w_dst[v] = row * 64 + (((cq ^ (row >> 2)) & 3) << 4);
  }
  // ---- fragment addresses -----------------------------------------------------------------------
  int colP[TJ], colK[TJ];
#pragma unroll
  for (int b = 0; b < TJ; ++b) {
    int j = bj0 + (wj * TJ + b) * 16 + frag_row;
    if (j > tile.j_last) j = tile.j_last;
    const NchwColumn c = nchw_column(s, tile, j);
    colP[b] = c.P;
    colK[b] = c.key;
  }
  int a_off[TI];
#pragma unroll
  for (int a = 0; a < TI; ++a) {
    const int row = (wi * TI + a) * 16 + frag_row;
    a_off[a] = row * 64 + (((frag_q ^ (row >> 2)) & 3) << 4);
  }
  const int rowP = s.dh * s.Wp, rowK = s.dh * s.key_pitch;

  char* const wbase = smem;
  char* const pbase = smem + 2 * WBUF;
  const int PBUF = p.max_pos * kNchwPosBytes;

  // ---- both patch buffers start as zeros: padding positions are never written ---------------------
  for (int i = t; i < 2 * p.max_pos * 4; i += NT) *(v4i*)(pbase + i * 16) = v4i{0, 0, 0, 0};
  __syncthreads();

  const int m_begin = blockIdx.y * p.macro_per_split;
  int m_end = m_begin + p.macro_per_split;
  if (m_end > p.macro_steps) m_end = p.macro_steps;

  unsigned wraw[WU][WRAW];
  unsigned praw[PT][CG][2];

  auto load_weights = [&](int m) {
    const int tt = nchw_div(m, p.div_cc), cc = m - tt * p.c_chunks;
#pragma unroll
    for (int v = 0; v < WU; ++v) {
      if (!w_on[v]) continue;
      const char* src = p.w + (w_src[v] + (int64_t)cc * CK * TRS + tt * RS) * ES;
      if (T1) {
#pragma unroll
        for (int i = 0; i < 9; ++i) {
          const v4i x = *(const v4i*)(src + i * 16);
          wraw[v][4 * i] = x.x; wraw[v][4 * i + 1] = x.y; wraw[v][4 * i + 2] = x.z; wraw[v][4 * i + 3] = x.w;
        }
      } else {
#pragma unroll
        for (int ci = 0; ci < CG; ++ci) {
          const char* sc = src + (int64_t)ci * TRS * ES;
          if (ES == 2) {
            const v4i x = ((const NchwUnaligned16*)sc)->v;
            wraw[v][ci * CHW] = x.x; wraw[v][ci * CHW + 1] = x.y; wraw[v][ci * CHW + 2] = x.z; wraw[v][ci * CHW + 3] = x.w;
            wraw[v][ci * CHW + 4] = *(const unsigned short*)(sc + 16);
          } else {
            const uint2 x = ((const NchwUnaligned8*)sc)->v;
            wraw[v][ci * CHW] = x.x; wraw[v][ci * CHW + 1] = x.y;
            wraw[v][ci * CHW + 2] = *(const unsigned char*)(sc + 8);
          }
        }
      }
    }
  };
  auto load_patch = [&](int m) {
    const int tt = nchw_div(m, p.div_cc), cc = m - tt * p.c_chunks;
#pragma unroll
    for (int v = 0; v < PT; ++v) {
      const int d = p_d0[v] + tt * s.dd;
      if (p_on[v] && (unsigned)d < (unsigned)s.D) {
        const char* src = p.x + (p_src[v] + (int64_t)cc * CK * DHW + (int64_t)d * HW) * ES;
#pragma unroll
        for (int ci = 0; ci < CG; ++ci) {
          const uint2 x = *(const uint2*)(src + (int64_t)ci * DHW * ES);
          praw[v][ci][0] = x.x; praw[v][ci][1] = x.y;
        }
      } else {
#pragma unroll
        for (int ci = 0; ci < CG; ++ci) { praw[v][ci][0] = 0; praw[v][ci][1] = 0; }
      }
    }
  };
  // raw byte index of byte bb of channel ci at tap tap
  auto wbyte = [](int ci, int tap, int bb) {
    return T1 ? (ci * 9 + tap) * ES + bb : ci * CHW * 4 + tap * ES + bb;
  };
  auto stage_weights = [&](int buf) {
    char* const wb = wbase + buf * WBUF;
#pragma unroll
    for (int v = 0; v < WU; ++v) {
      if (!w_on[v]) continue;
#pragma unroll
      for (int tap = 0; tap < RS; ++tap) {
        v4i o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (ES == 2)
            o[j] = (int)nchw_gather<ES>(wraw[v], wbyte(2 * j, tap, 0), wbyte(2 * j, tap, 1), wbyte(2 * j + 1, tap, 0),
                                        wbyte(2 * j + 1, tap, 1));
          else
            o[j] = (int)nchw_gather<ES>(wraw[v], wbyte(4 * j, tap, 0), wbyte(4 * j + 1, tap, 0), wbyte(4 * j + 2, tap, 0),
                                        wbyte(4 * j + 3, tap, 0));
        }
        *(v4i*)(wb + tap * WTILE + w_dst[v]) = o;
      }
    }
  };
  auto stage_patch = [&](int buf) {
    char* const pb = pbase + buf * PBUF;
#pragma unroll
    for (int v = 0; v < PT; ++v) {
#pragma unroll
      for (int i = 0; i < PG; ++i) {
        v4i o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (ES == 2) {
            const unsigned sel = (i & 1) ? 0x07060302u : 0x05040100u;
            o[j] = (int)__builtin_amdgcn_perm(praw[v][2 * j + 1][i >> 1], praw[v][2 * j][i >> 1], sel);
          } else {
            const unsigned sel = (unsigned)(i & 3) | ((unsigned)(4 + (i & 3)) << 8);
            const unsigned lo = __builtin_amdgcn_perm(praw[v][4 * j + 1][i >> 2], praw[v][4 * j][i >> 2], sel);
            const unsigned hi = __builtin_amdgcn_perm(praw[v][4 * j + 3][i >> 2], praw[v][4 * j + 2][i >> 2], sel);
            o[j] = (int)__builtin_amdgcn_perm(hi, lo, 0x05040100u);
          }
        }
        if (p_dst[v][i] >= 0) *(v4i*)(pb + p_dst[v][i]) = o;
      }
    }
  };

  acc_t acc[TI][TJ];
#pragma unroll
  for (int a = 0; a < TI; ++a)
#pragma unroll
    for (int b = 0; b < TJ; ++b)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[a][b][r] = 0;

  v4i af[2][TI], bf[2][TJ];
  auto read_frags = [&](int slot, int tap, const char* wb, const char* pb) {
    const int tr = tap / 3, ts = tap - 3 * tr;
#pragma unroll
    for (int a = 0; a < TI; ++a) af[slot][a] = *(const v4i*)(wb + tap * WTILE + a_off[a]);
#pragma unroll
    for (int b = 0; b < TJ; ++b) {
      const int P = colP[b] + tr * rowP + ts * s.dw;
      const int key = colK[b] + tr * rowK + ts * s.dw;
      bf[slot][b] = *(const v4i*)(pb + P * kNchwPosBytes + (((frag_q ^ (key >> 2)) & 3) << 4));
    }
  };
  auto mma = [&](int slot) {
#pragma unroll
    for (int b = 0; b < TJ; ++b)
#pragma unroll
      for (int a = 0; a < TI; ++a) acc[a][b] = MM::run(af[slot][a], bf[slot][b], acc[a][b]);
  };

  // ---- prologue: macro step m_begin into buffer 0, the loads of m_begin + 1 in flight -------------
  if (m_begin < m_end) {
    load_weights(m_begin);
    load_patch(m_begin);
    stage_weights(0);
    stage_patch(0);
    if (m_begin + 1 < m_end) {
      load_weights(m_begin + 1);
      load_patch(m_begin + 1);
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

  for (int m = m_begin; m < m_end; ++m) {
    const int buf = (m - m_begin) & 1;
    const char* const wb = wbase + buf * WBUF;
    const char* const pb = pbase + buf * PBUF;
    read_frags(0, 0, wb, pb);
#pragma unroll
    for (int tap = 0; tap < RS; ++tap) {
      if (tap + 1 < RS) read_frags((tap + 1) & 1, tap + 1, wb, pb);
      mma(tap & 1);
      if (tap == 3) {
        // the other buffers were last read in the previous macro step: transpose the next macro
        // step into them under this one's matrix-core work, then start the loads of the one after
        if (m + 1 < m_end) {
          stage_weights(buf ^ 1);
          stage_patch(buf ^ 1);
          if (m + 2 < m_end) {
            load_weights(m + 2);
            load_patch(m + 2);
          }
        }
      }
    }
    // own LDS writes done, every wave through with this macro step's buffers
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
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
}

}  // namespace amos
