// Implicit-GEMM forward convolution (3x3 windows, conv2d / conv3d) that reads the activations as
// the caller holds them (NCDHW) in ONE launch:
//
//   Out(i = output channel, j = (image, od, op, oq)) = sum_k W(i, k) * Col(j, k),  k = (t, c, r, s)
//
// The matrix core wants, per lane, 16 contiguous bytes of K of one row / column.  Neither tensor
// offers that (in NCDHW the positions are contiguous, in KCTRS the window taps):
//   * activations are transposed in registers on their way to LDS: a loader thread fetches, for
//     one 16-byte chunk of channels, one 8- or 16-byte run of input positions per channel (16
//     lanes cover 128 / 256 contiguous bytes of a channel plane), turns them with byte permutes
//     into one 16-byte vector of channels per position and stores those into the zero-padded
//     patch [position][64 bytes of channels] of the tile;
//   * weights come packed as [K][T*9][C] (amos_conv_pack_weights: by the same call into the
//     workspace, or once by their owner) and are copied into LDS as they are, 16 bytes a lane,
//     without passing through registers; or, with no workspace, from the caller's KCTRS tensor:
//     a loader thread fetches the nine taps of a chunk of channels of one output channel (144
//     contiguous bytes in 2-d; per channel an unaligned 18 / 9 byte run in 3-d) and writes one
//     16-byte vector of channels per tap into that tap's weight tile [row][64 bytes].
// A macro step is (depth tap, 64 bytes of channels): its patch serves all nine taps (a tap only
// shifts the position a lane reads) and its nine weight tiles are resident together, both double
// buffered, so a workgroup meets at ONE barrier per macro step = per nine K steps.  Loader waves
// bring in macro step m+1 (their loads two macro steps ahead of the use) while the matrix-core
// waves compute macro step m.
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
#if AMOS_SPLIT_IN_KERNEL
  SplitFinish fin;       // split-K: the last workgroup of a tile adds the slices
#endif
};

#define AMOS_LDS_ADDR(off) ((__attribute__((address_space(3))) char*)(size_t)(off))
enum { NCHW_W_KCTRS = 0, NCHW_W_KCRS = 1, NCHW_W_PACKED = 2 };
// a pointer that is the same in every lane, as a scalar register pair (what an "s" operand of an
// assembly statement needs; the compiler does not always see the uniformity by itself)
__device__ __forceinline__ const char* nchw_uniform(const char* ptr) {
  const uint64_t a = (uint64_t)ptr;
  const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)a), hi = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32));
  return (const char*)(((uint64_t)hi << 32) | lo);
}
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

// The same for nine taps (conv2d, T = 1) and 16-byte aligned weights: a thread takes the 144
// contiguous bytes of one (output channel, 16-byte chunk of channels) -- nine 16-byte loads --,
// transposes them in registers and writes one 16-byte vector per tap; threads of neighbouring
// chunks write neighbouring 16 bytes of a row.  A tenth of the memory instructions of the
// element-wise kernel above (C3's weights: 2.6 instead of 4.4 us).
template <int ES>
__global__ __launch_bounds__(256) void amos_conv_pack_weights9_kernel(const char* __restrict__ w, char* __restrict__ out,
                                                                      int K, int C, NchwDiv div_chunks) {
  constexpr int CG = 16 / ES;
  const int chunks = C / CG;
  const int total = K * chunks;
  for (int u = (int)(blockIdx.x * 256 + threadIdx.x); u < total; u += (int)(gridDim.x * 256)) {
    const int k = nchw_div(u, div_chunks), cq = u - k * chunks;
    const char* const src = w + ((int64_t)k * C + (int64_t)cq * CG) * 9 * ES;
    unsigned raw[36];
#pragma unroll
    for (int i = 0; i < 9; ++i) {
      const v4i x = *(const v4i*)(src + i * 16);
      raw[4 * i] = x.x; raw[4 * i + 1] = x.y; raw[4 * i + 2] = x.z; raw[4 * i + 3] = x.w;
    }
    // byte bb of channel ci at tap `tap` is byte (ci * 9 + tap) * ES + bb of the run
#pragma unroll
    for (int tap = 0; tap < 9; ++tap) {
      v4i o;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (ES == 2)
          o[j] = (int)nchw_gather<ES>(raw, ((2 * j) * 9 + tap) * 2, ((2 * j) * 9 + tap) * 2 + 1, ((2 * j + 1) * 9 + tap) * 2,
                                      ((2 * j + 1) * 9 + tap) * 2 + 1);
        else
          o[j] = (int)nchw_gather<ES>(raw, (4 * j) * 9 + tap, (4 * j + 1) * 9 + tap, (4 * j + 2) * 9 + tap, (4 * j + 3) * 9 + tap);
      }
      *(v4i*)(out + (((int64_t)k * 9 + tap) * C + (int64_t)cq * CG) * ES) = o;
    }
  }
}

// bytes of one patch buffer: a constant of the tile, so that the second buffer is an immediate
// offset of every LDS access; the last 1 KB of a buffer is a dump line for stores that have no
// position to go to (one 16-byte slot per lane)
constexpr int nchw_patch_buffer_bytes(int bj) { return bj <= 128 ? 32 * 1024 : 40 * 1024; }
constexpr int nchw_max_positions(int bj) { return nchw_patch_buffer_bytes(bj) / kNchwPosBytes - 16; }


// BI x BJ: output channels x output positions of a workgroup; WI x WJ: the grid of its
// matrix-core waves; NWL: its loader waves; PTL: load groups of the patch per loader thread (the
// loaders take 16 * NWL * PTL groups); LB: bytes of a patch load, i.e. of a load group's run of
// positions in one channel -- 8, or 16 where a channel plane is a whole number of 16-byte runs and
// the tensor is 16-byte aligned (half the load instructions, which are what bounds the loaders);
// WMODE: where the weights come from -- NCHW_W_KCTRS: the caller's tensor, per channel
// an unaligned run of nine taps; NCHW_W_KCRS: the same where a chunk of channels is one
// contiguous, 16-byte aligned run (conv2d with aligned weights); NCHW_W_PACKED: [K][T*9][C],
// written by amos_conv_pack_weights (into the workspace by the same call, or once by the owner of
// the weights): copied into LDS as they are, 16 bytes a lane, without passing through registers.
//
// Two kinds of waves.  A memory instruction of 64 lanes occupies the CU's address unit for 10-25
// cycles, and a wave that cannot issue it stalls with everything behind it, matrix-core
// instructions included: with loads and matrix-core work in the same waves a macro step took twice
// its matrix-core time however the loads were spread.  So four loader waves fetch, transpose and
// store the operands of macro step m + 1 (their loads two macro steps ahead of their use) while
// the WI x WJ matrix-core waves do nothing but read fragments of macro step m and multiply; the
// two kinds meet at the one barrier per macro step.
//
// HV: halves of output channels.  With HV = 2 a workgroup computes 2 * BI output channels of its
// positions: every macro step's patch serves two weight halves one after the other (sequence step
// q = macro step * HV + half; the weight buffers alternate with q, the patch buffers with the
// macro step), at twice the accumulators.  Half as many workgroups, each with one set-up, one
// patch and one round of patch loads for twice the work: for shapes whose tiles would otherwise
// take two rounds of the compute units with the second one half empty.
template <int DT, int BI, int BJ, int WI, int WJ, int PTL, int WMODE, int NWL, int LB, int HV = 1>
__global__ __launch_bounds__(64 * (WI * WJ + NWL)) void amos_conv_nchw(const ConvNchwParams p) {
  typedef Mfma16<DT> MM;
  typedef typename MM::acc_t acc_t;
  typedef typename Mfma<DT>::out_t out_t;
  constexpr int ES = Mfma<DT>::ES;
  constexpr int NWM = WI * WJ, NTM = 64 * NWM, NTL = 64 * NWL, NTA = NTM + NTL;
  constexpr int TI = BI / (16 * WI), TJ = BJ / (16 * WJ);
  static_assert(TI >= 1 && TJ >= 1 && TI * WI * 16 == BI && TJ * WJ * 16 == BJ, "wave tile");
  static_assert(LB == 8 || LB == 16, "patch loads of 8 or 16 bytes");
  constexpr int PG = LB / ES;     // input positions per patch load
  constexpr int CG = 16 / ES;     // channels per 16-byte chunk
  constexpr int CK = 64 / ES;     // channels per macro step
  constexpr int RS = 9;
  constexpr int WTILE = BI * 64;  // one tap's weight tile
  constexpr int WBUF = RS * WTILE;
  constexpr int PBUF = nchw_patch_buffer_bytes(BJ);
  constexpr bool T1 = WMODE == NCHW_W_KCRS, PACKED = WMODE == NCHW_W_PACKED;
  constexpr int CHW = T1 ? 0 : (ES == 2 ? 5 : 3);       // dwords of one channel's taps (3-d path)
  constexpr int WRAW = T1 ? 36 : CG * CHW;              // dwords of a unit's raw weights
  constexpr int UNITS = BI * 4;   // (row, chunk of channels) pairs of a macro step's weights
  static_assert(UNITS <= NTL, "one weight unit per loader thread at most");
  // packed weights: copied in 1 KB blocks (16 rows x 64 bytes); a tap's tile is NB of them
  constexpr int NB = BI / 16;
  // LDS, by byte offset from 0 (the kernel has no static LDS; the host checks that):
  //   [2][9][BI * 64] weight tiles | [2][PBUF] patches, the last 1 KB of each a dump line
  constexpr unsigned PBASE = 2 * WBUF;
  constexpr unsigned DUMP = PBUF - 1024;

  const NchwShape& s = p.s;
  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);

  // Workgroups are dealt round-robin to the 8 XCDs: give each XCD a contiguous run of tiles, the
  // tiles of one patch (tile_i fastest) next to each other, so that an XCD's L2 sees a patch once
  int logical;
  {
    const int n_wg = (int)gridDim.x, wg = (int)blockIdx.x;
    const int x = wg & 7, per = n_wg >> 3, rem = n_wg & 7;
    logical = x * per + (x < rem ? x : rem) + (wg >> 3);
  }
  const int tile_j = logical / p.tiles_i, tile_i = logical - tile_j * p.tiles_i;
  const int bi0 = tile_i * BI * HV, bj0 = tile_j * BJ;
  static_assert(HV == 1 || HV == 2, "one or two halves of output channels");
  const int HW = s.H * s.W;
  const int64_t DHW = (int64_t)s.D * HW;
  const int TRS = s.T * RS;
  const int m_begin = blockIdx.y * p.macro_per_split;
  int m_end = m_begin + p.macro_per_split;
  if (m_end > p.macro_steps) m_end = p.macro_steps;
  const int nq = (m_end - m_begin) * HV;   // sequence steps: (macro step, half of the output channels)

  // both kinds of waves: clear the patch buffers (padding positions are never written), meet
  auto clear_patches = [&]() __attribute__((always_inline)) {
    for (int i = t; i < p.max_pos * 4; i += NTA) {
      *(v4i*)AMOS_LDS_ADDR(PBASE + i * 16) = v4i{0, 0, 0, 0};
      *(v4i*)AMOS_LDS_ADDR(PBASE + PBUF + i * 16) = v4i{0, 0, 0, 0};
    }
  };
  auto meet = [&]() __attribute__((always_inline)) { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

  if (wave >= NWM) {
    // ==================================== loader waves ==============================================
    // (The direct copies of packed weights are issued by the matrix-core waves: a direct copy into
    // LDS costs the issuing wave the time LDS takes to accept it.)
    const int tl = t - NTM;
    constexpr int NTP = NTL;
    const int tlp = tl;
    // ---- this thread's share of the weights ----------------------------------------------------
    unsigned w_src[HV] = {0};  // byte offset of (row, first channel of the chunk) per half: below 4 GiB
    unsigned w_dst = 0;        // LDS address inside a tap's tile of the first buffer
    bool w_on = !PACKED;
    if (!PACKED) {
      // (with fewer units than loader threads they go to the last waves)
      const int u = tl - (NTL - UNITS);
      // (lanes 4x .. 4x+3 of a wave take row nchw_row_of_slot(x) of their sixteen: no bank conflicts)
      const int cq = u & 3, row = ((u >> 6) * 16 + nchw_row_of_slot((u >> 2) & 15)) & (BI - 1);
      w_on = u >= 0;
#pragma unroll
      for (int h = 0; h < HV; ++h) {
        const int k = bi0 + h * BI + row < s.K ? bi0 + h * BI + row : s.K - 1;
        w_src[h] = (unsigned)((((int64_t)k * s.C + cq * CG) * TRS) * ES);
      }
      w_dst = (unsigned)nchw_position_offset(row, cq);
    }
    unsigned wraw[PACKED ? 1 : WRAW];
    // The patch loads of a macro step are on their way for a whole macro step, across the loop's
    // back edge.  The compiler takes the result of an assembly load for present as soon as the
    // statement is behind it and is free to copy such a register to another one at any join of
    // the control flow -- which copies what the register held before the data arrived.  So the
    // loads land in the 32 highest registers a wave of this workgroup size can have (v136 .. v167
    // with twelve waves on a compute unit, v224 .. v255 with eight), named in the assembly text
    // and far above what the compiler needs for either kind of wave -- tests/test_conv_nchw_isa.py
    // reads the compiled code of every instance and fails if anything outside these statements
    // touches them -- and landed() moves them into ordinary registers behind the wait; the next
    // loads go out right after that, before the transposes, so one set of registers keeps loads
    // in flight all the time.
    constexpr int LW = LB / 4;            // dwords of a load
    constexpr int NAG = PTL * CG * LW;    // staging registers the loads of a macro step fill
    static_assert(NAG <= 32, "staging registers");
    constexpr int SBASE = NWM + NWL == 12 ? 136 : NWM + NWL == 8 ? 224 : -1;
    static_assert(SBASE > 0, "workgroups of eight or twelve waves");
    typedef unsigned nchw_ul __attribute__((ext_vector_type(LW)));

    // weights that pass through registers: the raw taps of this thread's unit
    auto load_weights = [&](int m, auto half_c) __attribute__((always_inline)) {
      if (!w_on) return;
      const int tt = nchw_div(m, p.div_cc), cc = m - tt * p.c_chunks;
      const char* const src = p.w + ((int64_t)cc * CK * TRS + tt * RS) * ES + w_src[decltype(half_c)::value];
      if (T1) {
#pragma unroll
        for (int i = 0; i < 9; ++i) {
          const v4i x = *(const v4i*)(src + i * 16);
          wraw[4 * i] = x.x; wraw[4 * i + 1] = x.y; wraw[4 * i + 2] = x.z; wraw[4 * i + 3] = x.w;
        }
      } else {
#pragma unroll
        for (int ci = 0; ci < CG; ++ci) {
          const char* sc = src + (int64_t)ci * TRS * ES;
          if (ES == 2) {
            const v4i x = ((const NchwUnaligned16*)sc)->v;
            wraw[ci * CHW] = x.x; wraw[ci * CHW + 1] = x.y; wraw[ci * CHW + 2] = x.z; wraw[ci * CHW + 3] = x.w;
            wraw[ci * CHW + 4] = *(const unsigned short*)(sc + 16);
          } else {
            const uint2 x = ((const NchwUnaligned8*)sc)->v;
            wraw[ci * CHW] = x.x; wraw[ci * CHW + 1] = x.y;
            wraw[ci * CHW + 2] = *(const unsigned char*)(sc + 8);
          }
        }
      }
    };
    // raw byte index of byte bb of channel ci at tap tap
    auto wbyte = [](int ci, int tap, int bb) __attribute__((always_inline)) {
      return T1 ? (ci * 9 + tap) * ES + bb : ci * CHW * 4 + tap * ES + bb;
    };
    // ... transposed: per tap one 16-byte vector of channels into that tap's tile
    auto store_weights = [&](auto buf_c) __attribute__((always_inline)) {
      if (!w_on) return;
#pragma unroll
      for (int tap = 0; tap < RS; ++tap) {
        v4i o;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (ES == 2)
            o[j] = (int)nchw_gather<ES>(wraw, wbyte(2 * j, tap, 0), wbyte(2 * j, tap, 1), wbyte(2 * j + 1, tap, 0),
                                        wbyte(2 * j + 1, tap, 1));
          else
            o[j] = (int)nchw_gather<ES>(wraw, wbyte(4 * j, tap, 0), wbyte(4 * j + 1, tap, 0), wbyte(4 * j + 2, tap, 0),
                                        wbyte(4 * j + 3, tap, 0));
        }
        *(v4i*)AMOS_LDS_ADDR(w_dst + decltype(buf_c)::value * WBUF + tap * WTILE) = o;
      }
    };
    // the first weights go out before the tile's geometry is worked out
    if constexpr (!PACKED) load_weights(m_begin, NchwSet<0>{});

    const NchwTile tile = nchw_tile(s, bj0, BJ);
    // ---- this thread's load groups of the patch ------------------------------------------------
    // First what the loads need (a wave issues an instruction every five to seven cycles when it
    // is alone on its SIMD, every nine to seventeen next to two waves of matrix-core work: the
    // length of this stretch is the time to the first load), then the loads, then -- while they
    // are on their way -- where the positions go in LDS.
    unsigned p_src[PTL];      // byte offset of (image, first channel of the chunk, depth 0, group): below 4 GiB
    int p_d0[PTL];            // input depth at depth tap 0
    unsigned p_dst[PTL][PG];  // LDS addresses (first buffer) of the group's positions; the dump line
                              // for positions that are not part of the window
    const unsigned plane_bytes = (unsigned)(DHW * ES);
    // byte selectors that pick position i (lower half of the wave) or i ^ 1 (upper half) out of a
    // staging dword: 16-bit types hold two positions per dword, int8 four
    unsigned p_sel[ES == 2 ? 2 : 4];
#pragma unroll
    for (int v = 0; v < PTL; ++v) {
      const int q = tlp + NTP * v;
      const int cg = q & 3, grp = q >> 2;
      const bool on = grp < tile.ngroups;
      int f = 0;
      const NchwSeg seg = nchw_group(s, tile, on ? grp : 0, &f);
      p_src[v] = (unsigned)((((int64_t)seg.n * s.C + cg * CG) * DHW + f) * ES);
      p_d0[v] = seg.d0;
    }
#define AMOS_NCHW_S136 "v136", "v137", "v138", "v139", "v140", "v141", "v142", "v143", "v144", "v145", "v146", "v147", "v148", "v149", "v150", "v151", \
                       "v152", "v153", "v154", "v155", "v156", "v157", "v158", "v159", "v160", "v161", "v162", "v163", "v164", "v165", "v166", "v167"
#define AMOS_NCHW_S224 "v224", "v225", "v226", "v227", "v228", "v229", "v230", "v231", "v232", "v233", "v234", "v235", "v236", "v237", "v238", "v239", \
                       "v240", "v241", "v242", "v243", "v244", "v245", "v246", "v247", "v248", "v249", "v250", "v251", "v252", "v253", "v254", "v255"
    // the patch loads of macro step m.  Every lane loads, from a depth clamped into the tensor (a
    // depth in the padding stores zeros instead, lanes without a group store into the dump line).
    // One scalar base per macro step (the chunk of channels), per load the lane's offset plus the
    // channel's plane: two instructions a load.
    // Where a macro step's loads take half of the staging registers or less there are two sets: the
    // loads of macro step m + 2 go out (into the other set) BEFORE macro step m + 1 is transposed
    // out of its set, a transposition longer on their way; else one set, and the loads follow the
    // permutes that read it.
    constexpr bool TWO_SETS = NAG <= 16 && PACKED;   // (unpacked weights: their loads go first, measured)
    auto load_patch = [&](auto set_c, int m) __attribute__((always_inline)) {
      constexpr int SB = SBASE + (TWO_SETS ? decltype(set_c)::value * 16 : 0);
      const int tt = nchw_div(m, p.div_cc), cc = m - tt * p.c_chunks;
      const char* const base = nchw_uniform(p.x + (int64_t)cc * CK * DHW * ES);
      nchw_static_for<0, PTL>([&](auto v_c) {
        constexpr int v = decltype(v_c)::value;
        int d = p_d0[v] + tt * s.dd;
        d = d < 0 ? 0 : d >= s.D ? s.D - 1 : d;
        // (the depth is the lane's own: its offset stays below 4 GiB like the rest of the tensor)
        const unsigned off_v = p_src[v] + (unsigned)d * (unsigned)(HW * ES);
        nchw_static_for<0, CG>([&](auto ci_c) {
          constexpr int ci = decltype(ci_c)::value, r0 = SB + (v * CG + ci) * LW;
          const unsigned off = off_v + (unsigned)ci * plane_bytes;
          const char* const plane = base;
          // (five wait states between the v_readfirstlane that may have made the base and its first
          // use; the compiler cannot insert them inside a statement)
#define AMOS_NCHW_LOAD(width, last, clobbers)                                                                                   \
  if constexpr (v == 0 && ci == 0)                                                                                              \
    asm volatile("s_nop 4\n\tglobal_load_" width " v[%2:%3], %0, %1" ::"v"(off), "s"(plane), "n"(r0), "n"(r0 + last) : "memory", clobbers); \
  else                                                                                                                          \
    asm volatile("global_load_" width " v[%2:%3], %0, %1" ::"v"(off), "s"(plane), "n"(r0), "n"(r0 + last) : "memory", clobbers)
          if constexpr (LB == 16 && SBASE == 136) { AMOS_NCHW_LOAD("dwordx4", 3, AMOS_NCHW_S136); }
          else if constexpr (LB == 16) { AMOS_NCHW_LOAD("dwordx4", 3, AMOS_NCHW_S224); }
          else if constexpr (SBASE == 136) { AMOS_NCHW_LOAD("dwordx2", 1, AMOS_NCHW_S136); }
          else { AMOS_NCHW_LOAD("dwordx2", 1, AMOS_NCHW_S224); }
#undef AMOS_NCHW_LOAD
        });
      });
    };
    // every load of this wave has landed (the compiler's own loads of unpacked weights too)
    auto landed = [&]() __attribute__((always_inline)) { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };
    // dword `k` of channel `c` of load group `v`, out of the staging registers, as an operand of
    // an assembly statement: "v[n]"
    // The patch of macro step m out of the staging registers into patch buffer BUF: per position
    // one 16-byte vector of channels.  The byte permutes read the staging registers where the
    // loads left them (assembly: the compiler does not know these registers), so the next loads
    // go out behind them.  A group whose depth lies in the padding stores zeros.
    auto store_patch = [&](auto buf_c, auto set_c, int m) __attribute__((always_inline)) {
      constexpr int SB = SBASE + (TWO_SETS ? decltype(set_c)::value * 16 : 0);
      const int tt = nchw_div(m, p.div_cc);
      nchw_static_for<0, PTL>([&](auto v_c) {
        constexpr int v = decltype(v_c)::value;
        const bool ok = (unsigned)(p_d0[v] + tt * s.dd) < (unsigned)s.D;
        if (ok) {
          nchw_static_for<0, PG>([&](auto i_c) {
            constexpr int i = decltype(i_c)::value;
            unsigned o[4];
            nchw_static_for<0, 4>([&](auto j_c) {
              constexpr int j = decltype(j_c)::value;
              if constexpr (ES == 2) {
                const unsigned sel = p_sel[i & 1];
                unsigned x;   // (an assembly operand cannot name a variable of an enclosing lambda)
                asm volatile("v_perm_b32 %0, v[%1], v[%2], %3" : "=v"(x)
                             : "n"(SB + (v * CG + 2 * j + 1) * LW + (i >> 1)), "n"(SB + (v * CG + 2 * j) * LW + (i >> 1)), "v"(sel));
                o[j] = x;
              } else {
                const unsigned sel = p_sel[i & 3];
                unsigned lo, hi;
                asm volatile("v_perm_b32 %0, v[%1], v[%2], %3" : "=v"(lo)
                             : "n"(SB + (v * CG + 4 * j + 1) * LW + (i >> 2)), "n"(SB + (v * CG + 4 * j) * LW + (i >> 2)), "v"(sel));
                asm volatile("v_perm_b32 %0, v[%1], v[%2], %3" : "=v"(hi)
                             : "n"(SB + (v * CG + 4 * j + 3) * LW + (i >> 2)), "n"(SB + (v * CG + 4 * j + 2) * LW + (i >> 2)), "v"(sel));
                o[j] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
              }
            });
            *(v4i*)AMOS_LDS_ADDR(p_dst[v][i] + decltype(buf_c)::value * PBUF) = v4i{(int)o[0], (int)o[1], (int)o[2], (int)o[3]};
          });
        } else {
#pragma unroll
          for (int i = 0; i < PG; ++i) *(v4i*)AMOS_LDS_ADDR(p_dst[v][i] + decltype(buf_c)::value * PBUF) = v4i{0, 0, 0, 0};
        }
      });
    };

    // ---- prologue: the first loads, then the rest of the set-up while they are on their way -------
    // (every blockIdx.y has at least one macro step: the host checks that)
    load_patch(NchwSet<0>{}, m_begin);
    {
      // (the thread index passes through an empty assembly statement: what depends on it stays
      // behind the loads instead of being merged with the arithmetic in front of them)
      int tl2 = tlp;
      asm volatile("" : "+v"(tl2));
      const int hi_half = (tl2 >> 5) & 1;
#pragma unroll
      for (int i = 0; i < (ES == 2 ? 2 : 4); ++i) {
        const int pos = i ^ hi_half;
        p_sel[i] = ES == 2 ? (pos ? 0x07060302u : 0x05040100u) : ((unsigned)pos | ((unsigned)(4 + pos) << 8));
      }
#pragma unroll
      for (int v = 0; v < PTL; ++v) {
        const int q = tl2 + NTP * v;
        const int cg = q & 3, grp = q >> 2;
        const bool on = grp < tile.ngroups;
        int f = 0;
        const NchwSeg seg = nchw_group(s, tile, on ? grp : 0, &f);
#pragma unroll
        for (int i = 0; i < PG; ++i) {
          // (the upper half of a wave stores its positions in the order 1, 0, 3, 2, ...: see the bank
          // conflict notes of the geometry header)
          const int off = on ? nchw_writer_offset(s, seg, f + (i ^ hi_half), cg) : -1;
          p_dst[v][i] = PBASE + (off >= 0 ? (unsigned)off : DUMP + (unsigned)(tl2 & 63) * 16);
        }
      }
    }
    clear_patches();
    meet();
    landed();
    // (unpacked weights first: the compiler waits for its own loads in front of their first use, and
    // that wait would take the patch loads behind it along)
    if constexpr (!PACKED) store_weights(NchwSet<0>{});
    if (TWO_SETS && m_begin + 1 < m_end) load_patch(NchwSet<1>{}, m_begin + 1);
    store_patch(NchwSet<0>{}, NchwSet<0>{}, m_begin);
    if (!TWO_SETS && m_begin + 1 < m_end) load_patch(NchwSet<1>{}, m_begin + 1);
    meet();
    // ---- under sequence step q of the matrix-core waves: step q + 1 into the other weight buffer
    // and, where it starts a macro step, that macro step's patch into the other patch buffer (last
    // read a macro step ago); then the loads of the macro step after that go out.  Unpacked
    // weights: their loads are on their way while the patch is transposed.
    // U = (q + 1) % (2 * HV): weight buffer U & 1, patch buffer and staging set (U / HV) & 1, half U % HV
    auto under = [&](auto u_c, int q) __attribute__((always_inline)) {
      constexpr int U = decltype(u_c)::value, WB = U & 1, PB = (U / HV) & 1, HALF = U % HV;
      if (q + 1 < nq) {
        const int m1 = m_begin + (q + 1) / HV;   // the macro step of sequence step q + 1
        if constexpr (HALF == 0) {
          landed();
          if (TWO_SETS && m1 + 1 < m_end) load_patch(NchwSet<PB ^ 1>{}, m1 + 1);
          if constexpr (!PACKED) load_weights(m1, NchwSet<0>{});
          store_patch(NchwSet<PB>{}, NchwSet<PB>{}, m1);
          if constexpr (!PACKED) store_weights(NchwSet<WB>{});
          if (!TWO_SETS && m1 + 1 < m_end) load_patch(NchwSet<PB ^ 1>{}, m1 + 1);
        } else if constexpr (!PACKED) {
          load_weights(m1, NchwSet<HALF>{});
          store_weights(NchwSet<WB>{});
        }
      }
      meet();
    };
    for (int q = 0; q < nq; q += 2 * HV)
      nchw_static_for<0, 2 * HV>([&](auto u_c) {
        constexpr int u = decltype(u_c)::value;
        if (q + u < nq) under(NchwSet<(u + 1) % (2 * HV)>{}, q + u);
      });
#undef AMOS_NCHW_S136
#undef AMOS_NCHW_S224
    return;
  }

  // ==================================== matrix-core waves ===========================================
  // Packed weights are copied straight into LDS (global_load_lds, 16 bytes a lane, no registers)
  // in 1 KB blocks of 16 rows x 64 bytes: wave w takes block w % NB of the taps w / NB + 2 * i.
  // Lane l's bytes land at l * 16 of the block, so the lane fetches the (row, chunk) that lives
  // in that slot.  A copy costs the wave some 30 cycles of issue; the copies of macro step m + 1
  // go out at the start of macro step m and are waited for at its end.
  //   As assembly: after the builtin the compiler makes every later LDS instruction wait until
  //   the copy has landed (it cannot tell which LDS bytes the copy writes).  The wait states are
  //   the ones the compiler would insert, and cannot inside an assembly statement: five between
  //   a v_readfirstlane that may have produced the address registers and the memory instruction
  //   that reads them, one between the write of M0 and the copy that takes its LDS address from
  //   there; without them the copy can run with stale registers.
  static_assert(NWM % NB == 0, "a wave copies the same block of rows of every tap it takes");
  constexpr int TPR = NWM / NB;               // taps per round of the matrix-core waves' copies
  constexpr int NWC = (RS + TPR - 1) / TPR;
  const int wblock = wave % NB, wtap0 = wave / NB;
  unsigned w_lane[HV] = {0};
  if (PACKED) {
    int row16, cq;
    nchw_unit_of_slot(lane, &row16, &cq);
    const int row = wblock * 16 + row16;
#pragma unroll
    for (int h = 0; h < HV; ++h) {
      const int k = bi0 + h * BI + row < s.K ? bi0 + h * BI + row : s.K - 1;
      w_lane[h] = (unsigned)(((int64_t)k * TRS * s.C) * ES + cq * 16);
    }
  }
  auto copy_weights = [&](auto buf_c, int m, auto half_c) __attribute__((always_inline)) {
    const int tt = nchw_div(m, p.div_cc), cc = m - tt * p.c_chunks;
    const char* const wm = p.w + ((int64_t)tt * RS * s.C + (int64_t)cc * CK) * ES;
    const unsigned lane_off = w_lane[decltype(half_c)::value];
#pragma unroll
    for (int i = 0; i < NWC; ++i) {
      const int tap = wtap0 + TPR * i;
      if (tap < RS) {
        const char* const src = nchw_uniform(wm + (int64_t)tap * s.C * ES);
        const unsigned dst = decltype(buf_c)::value * WBUF + tap * WTILE + wblock * 1024;
        asm volatile("s_nop 4\n\ts_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(dst), "v"(lane_off), "s"(src)
                     : "memory");
      }
    }
  };
  // the first weights go out before anything else
  if (PACKED) copy_weights(NchwSet<0>{}, m_begin, NchwSet<0>{});
  const int wi = wave / WJ, wj = wave % WJ;
  const int frag_row = lane & 15, frag_q = lane >> 4;
  const NchwTile tile = nchw_tile(s, bj0, BJ);
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

  acc_t acc[HV][TI][TJ];
#pragma unroll
  for (int h = 0; h < HV; ++h)
#pragma unroll
    for (int a = 0; a < TI; ++a)
#pragma unroll
      for (int b = 0; b < TJ; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[h][a][b][r] = 0;

  // operand fragments are read NF - 1 taps ahead: a batch of LDS reads takes some 200 cycles to
  // come back, a tap's matrix-core work of a wave 64
  constexpr int NF = TI * TJ >= 8 ? 2 : 3;
  v4i af[NF][TI], bf[NF][TJ];
  auto read_frags = [&](auto wb_c, auto pb_c, auto tap_c) __attribute__((always_inline)) {
    constexpr int WB = decltype(wb_c)::value, PB = decltype(pb_c)::value, tap = decltype(tap_c)::value, slot = tap % NF;
#pragma unroll
    for (int a = 0; a < TI; ++a) af[slot][a] = *(const v4i*)AMOS_LDS_ADDR(a_addr[WB][a] + tap * WTILE);
#pragma unroll
    for (int b = 0; b < TJ; ++b) bf[slot][b] = *(const v4i*)AMOS_LDS_ADDR(b_addr[tap][b] + PB * PBUF);
  };
  auto mma = [&](auto half_c, int slot) __attribute__((always_inline)) {
    constexpr int h = decltype(half_c)::value;
#pragma unroll
    for (int b = 0; b < TJ; ++b)
#pragma unroll
      for (int a = 0; a < TI; ++a) acc[h][a][b] = MM::run(af[slot][a], bf[slot][b], acc[h][a][b]);
  };

  // Every address is worked out HERE, while the loaders' first loads are on their way: left to
  // itself the compiler sinks this arithmetic (some 150 instructions, a wave's instructions issue
  // 5-7 cycles apart) behind the barriers to its first use, into the one stretch of the
  // kernel where the loaders have delivered and every other wave waits for the first result.
#pragma unroll
  for (int a = 0; a < TI; ++a) asm volatile("" : "+v"(a_addr[0][a]), "+v"(a_addr[1][a]));
#pragma unroll
  for (int b = 0; b < TJ; ++b)
#pragma unroll
    for (int tap = 0; tap < RS; ++tap) asm volatile("" : "+v"(b_addr[tap][b]));
#pragma unroll
  for (int h = 0; h < HV; ++h)
#pragma unroll
    for (int a = 0; a < TI; ++a)
#pragma unroll
      for (int b = 0; b < TJ; ++b) asm volatile("" : "+v"(acc[h][a][b]));
  clear_patches();
  meet();
  if (PACKED) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the first macro step's weights
  meet();
  // One sequence step: nine taps out of weight buffer U & 1 and patch buffer (U / HV) & 1 into the
  // accumulators of half U % HV, then the barrier behind which the loaders have the next step's
  // buffers ready and may overwrite what this one has read
  auto seq_step = [&](auto u_c, int q) __attribute__((always_inline)) {
    constexpr int U = decltype(u_c)::value, WB = U & 1, PB = (U / HV) & 1, HALF = U % HV;
    constexpr int U1 = (U + 1) % (2 * HV);
    if (PACKED && q + 1 < nq) copy_weights(NchwSet<(U1 & 1)>{}, m_begin + (q + 1) / HV, NchwSet<U1 % HV>{});
    nchw_static_for<0, NF - 1>([&](auto tap_c) { read_frags(NchwSet<WB>{}, NchwSet<PB>{}, tap_c); });
    __builtin_amdgcn_sched_barrier(0);
    nchw_static_for<0, RS>([&](auto tap_c) {
      constexpr int tap = decltype(tap_c)::value;
      // (the order is pinned: left to itself the scheduler moves a tap's fragment reads next to
      // its matrix-core instructions, and every tap then waits for LDS)
      if constexpr (tap + NF - 1 < RS) read_frags(NchwSet<WB>{}, NchwSet<PB>{}, NchwSet<tap + NF - 1>{});
      __builtin_amdgcn_sched_barrier(0);
      mma(NchwSet<HALF>{}, tap % NF);
      __builtin_amdgcn_sched_barrier(0);
    });
    if (PACKED) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wave's copies have landed
    meet();
  };
  for (int q = 0; q < nq; q += 2 * HV)
    nchw_static_for<0, 2 * HV>([&](auto u_c) {
      constexpr int u = decltype(u_c)::value;
      if (q + u < nq) seq_step(u_c, q + u);
    });

  // ---- epilogue: Y[(n * K + i) * ODPQ + s], a lane holds column j of rows 4 * frag_q + r ----------
  out_t* const out = (out_t*)p.y + (int64_t)blockIdx.y * p.split_stride;
  const int ODPQ = s.OD * s.OP * s.OQ;
  const bool add_d = p.epi.dt != EPI_NONE && blockIdx.y == 0;
  // Where four consecutive output positions are one aligned 16-byte run of the result (an image's
  // positions a multiple of four, the tensor 16-byte aligned) and there is no fused tail, a 16-row
  // block of the wave tile goes through an LDS strip of the wave (the operand buffers are free
  // behind the last barrier; LDS operations of one wave complete in issue order, so the strip needs
  // no barrier of its own) and leaves as 16-byte stores that cover whole rows of the wave tile:
  // 64 / (4 TJ) rows x 64 TJ bytes per instruction instead of four rows x 64 bytes.
  constexpr int SP = TJ * 16 + 4;                 // strip row pitch in elements
  constexpr int CPR = TJ * 4, RPI = 64 / CPR;     // 16-byte chunks per row, rows per store instruction
  static_assert((TJ & (TJ - 1)) == 0 && TJ <= 16 && NWM * 16 * SP * 4 <= 2 * WBUF, "output strip");
  const bool strips = !add_d && (ODPQ & 3) == 0 && (((uintptr_t)out) & 15) == 0;
  if (strips) {
    out_t* const strip = (out_t*)AMOS_LDS_ADDR(wave * (16 * SP * 4));
    // this lane's four positions of the wave tile's row: one image, one 16-byte run
    const int j4 = bj0 + wj * TJ * 16 + (lane % CPR) * 4;
    const int jc = j4 < s.J ? j4 : 0;
    const int n = nchw_div(jc, p.div_odpq);
    const int64_t coff = (int64_t)n * s.K * ODPQ + (jc - n * ODPQ);
#pragma unroll
    for (int ha = 0; ha < HV * TI; ++ha) {
      const int h = ha / TI, a = ha % TI;
#pragma unroll
      for (int b = 0; b < TJ; ++b)
#pragma unroll
        for (int r = 0; r < 4; ++r) strip[(4 * frag_q + r) * SP + b * 16 + frag_row] = acc[h][a][b][r];
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      acc_t v[TJ];
#pragma unroll
      for (int x = 0; x < TJ; ++x) v[x] = *(const acc_t*)(strip + (x * RPI + lane / CPR) * SP + (lane % CPR) * 4);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int x = 0; x < TJ; ++x) {
        const int i = bi0 + h * BI + (wi * TI + a) * 16 + x * RPI + lane / CPR;
        // (J is a multiple of four here: the four positions are inside the tensor together)
        if (i < s.K && j4 < s.J) *(acc_t*)(out + coff + (int64_t)i * ODPQ) = v[x];
      }
    }
  } else {
#pragma unroll
  for (int b = 0; b < TJ; ++b) {
    const int j = bj0 + (wj * TJ + b) * 16 + frag_row;
    const int jc = j < s.J ? j : s.J - 1;
    const int n = nchw_div(jc, p.div_odpq);
    const int64_t coff = (int64_t)n * s.K * ODPQ + (jc - n * ODPQ);
#pragma unroll
    for (int ha = 0; ha < HV * TI; ++ha) {
      const int h = ha / TI, a = ha % TI;
      const int i0 = bi0 + h * BI + (wi * TI + a) * 16 + 4 * frag_q;
      if (add_d) {
        out_t dv[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) dv[r] = epi_value<out_t>(p.epi, coff + (int64_t)(i0 + r < s.K ? i0 + r : s.K - 1) * ODPQ);
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[h][a][b][r] += dv[r];
      }
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (i0 + r < s.K && j < s.J) out[coff + (int64_t)(i0 + r) * ODPQ] = acc[h][a][b][r];
    }
  }
  }
#if AMOS_SPLIT_IN_KERNEL
  if (p.fin.tickets) {
    // (the loader waves have left: the matrix-core waves' threads are the workgroup now)
    split_finish<out_t>(p.fin, blockIdx.x, (const out_t*)p.y, t, NTM, BI * HV, BJ, (lds_flag_t)(size_t)0,
                        [&](int r, int c) -> int64_t {
                          const int i = bi0 + r, j = bj0 + c;
                          if (i >= s.K || j >= s.J) return -1;
                          const int n = nchw_div(j, p.div_odpq);
                          return ((int64_t)n * s.K + i) * ODPQ + (j - n * ODPQ);
                        });
  }
#endif
}

}  // namespace amos
