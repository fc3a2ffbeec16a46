// Implicit-GEMM forward convolution (conv2d / conv3d, NCDHW x KCTRS -> NKDPQ) that never
// forms the im2col matrix, not even in LDS.
//
//   Out(i = output channel, j = (image, od, op, oq)) = sum_k W'(i, k) * Col(j, k),
//   k = (t, r, s, c) with the channel c innermost.
//
// Two launches per call:
//
// 1. amos_conv_prepare relays both operands so that channels are innermost:
//    weights KCTRS -> K,(TRS),C and activations NCDHW -> NDHWC, into the caller's
//    workspace (and clears the output for a split-K launch).  The reference spends
//    separate kernels on this too, but writes the whole im2col matrix -- R*S times the
//    activations -- where this writes them once (reference: README.md:344-361,
//    src/auto_tensorize/compute_transform.cc:181-293).
// 2. amos_conv_fprop.  With c innermost a K step is (tap, 128 bytes of channels):
//    * per output channel the weights of a K step are one contiguous 128-byte run, so
//      the weight tile is copied global -> LDS directly like a GEMM operand, through
//      a ring of NSW stages (the tiles are small, so several steps must be in flight
//      to cover the memory latency);
//    * for a block's BJ output positions and one channel chunk, the zero-padded input
//      patch they touch is staged ONCE in LDS as [position][128 bytes of channels]
//      and serves all R*S taps: a tap only shifts the position a lane reads.  The
//      patch is copied global -> LDS directly as well (8 positions per wave
//      instruction); positions outside the image read a block of zeros.  The patch of
//      the next (depth tap, channel chunk) is fetched during the tap loop of the
//      current one.
//    * operand fragments are double buffered in registers, one barrier per K step.
//
// A block's BJ positions may straddle image (or depth-slice) boundaries: the patch is a
// list of up to kConvMaxSeg segments, one per slice, each a zero-padded [rows][cols] window.
#pragma once
#define AMOS_CONV_FPROP_KERNEL_INCLUDED 1
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fast_div.h"
#include "gemm_tn_kernel.h"
#include "igemm_kernel.h"

namespace amos {

constexpr int kConvMaxSeg = 4;

#define AMOS_LDS_PTR_FROM(off) ((const __attribute__((address_space(3))) char*)(size_t)(off))
#define AMOS_LDS_PTR_RW(off) ((__attribute__((address_space(3))) char*)(size_t)(off))

struct ConvFpropParams {
  const char* x;     // original NCDHW activations (prepare kernel input)
  const char* w;     // original KCTRS weights (prepare kernel input)
  char* xt;          // NDHWC activations (workspace)
  char* wp;          // packed weights [K][T*R*S][C] (workspace)
  char* zeros;       // 128 zero bytes (workspace)
  char* y;           // NKDPQ, fp32 / int32
  int N, C, D, H, W, K, T, R, S;   // C: channels of the relaid operands (whole 128-byte K steps)
  int Csrc;          // channels of the caller's tensors (<= C; the rest is zero-filled by the relayout)
  int sd, sh, sw, pd, ph, pw, dd, dh, dw;
  int OD, OP, OQ;
  int J;             // N*OD*OP*OQ
  int Wp;            // patch columns: (OQ-1)*sw + (S-1)*dw + 1
  int max_pos;       // LDS positions reserved per patch buffer (multiple of 64)
  int nsw;           // weight ring stages (>= 2)
  int pls;           // patch copy instructions per wave per K step (the instance's PL)
  int xbufs;         // patch buffers: 2, or 1 when a block handles a single (depth tap, channel chunk)
  int sx_off, tab_off, dump_off;   // LDS byte offsets: patch buffers, position table, dump line
  int tab1_off;      // second position table (blocks that walk several tiles)
  int total_steps;   // macro_steps * R * S
  void* steps;       // [total_steps + 1] step table (workspace), written by the prepare kernel
  int c_chunks;      // C*ES / 128
  int macro_steps;   // T * c_chunks
  int macro_per_split;
  int tiles_i, tiles_j;
  int atomic_out;        // split-K without room for partial sums: accumulate into the zeroed output
  int64_t split_stride;  // split-K with it: blockIdx.y stores its partial sums at y + blockIdx.y * split_stride
  FastDiv fd_opq, fd_oq, fd_od, fd_wp, fd_odpq, fd_cc, fd_c, fd_slab;   // divisions by OP*OQ, OQ, OD, Wp, OD*OP*OQ, c_chunks, C, C*T*R*S
  // prepare kernel work split (in blocks)
  int prep_w_blocks, prep_x_blocks, prep_z_blocks;
  int64_t zero_words;
  EpiParams epi;     // fused tail: Y = acc + cast(D), D laid out like Y
#if AMOS_SPLIT_IN_KERNEL
  SplitFinish fin;   // split-K: the last workgroup of a tile adds the slices
#endif
  // tensor layouts (AMOS_LAYOUT_*): 0 = NCDHW / KCTRS / NKDPQ, 1 = NDHWC / TRSCK / NDPQK,
  // 2 = DHWNC / TRSCK / DPQNK.  Output element (i, j), j = n*ODPQ + s, at i*y_si + n*y_sn + s*y_ss.
  int layout;
  int64_t y_si, y_sn, y_ss;
  int y_vec4;        // y_si == 1, K % 4 == 0, Y (and D) 16-byte aligned: four output channels per store
};

// ---- launch 1: relayout ---------------------------------------------------------------------
// Step table: what differs between the K steps of amos_conv_fprop, 8 words per step
// g = macro step * R*S + tap (macro step = (depth tap, channel chunk)):
//   [0] byte offset, inside a packed weight row, of the tile FETCHED during step g (that of step
//       g + nsw)            [7] the same for step g's own tile
//   [1] LDS offset the fragments of step g+1 read their patch at (buffer + tap shift)
//   [2] source offset of macro step m+1 from the zero block, [3] its depth shift - 32768
//   [4] first patch copy of step g | first patch copy of step g+1 << 16
//   [5] macro step m of g    [6] LDS offset of the patch buffer of macro step m+1
__device__ __forceinline__ void conv_write_steps(const ConvFpropParams& p, int es, int t) {
  const int RS = p.R * p.S, total = p.total_steps;
  const unsigned pos_bytes = (unsigned)p.C * es;
  const unsigned xbuf_bytes = (unsigned)p.max_pos * 128u;
  int* const tb = (int*)p.steps;
  auto wk_of = [&](int g) {
    if (g > total - 1) g = total - 1;
    const int m = g / RS, tap = g - m * RS;
    const int tt = m / p.c_chunks, cc = m - tt * p.c_chunks;
    return (unsigned)(tt * RS + tap) * pos_bytes + (unsigned)cc * 128u;
  };
  for (int g = t; g <= total; g += 256) {
    const int gc = g < total - 1 ? g : total - 1;
    const int m = gc / RS, tap = gc - m * RS;
    const int g1 = g + 1 < total - 1 ? g + 1 : total - 1;
    const int m1 = g1 / RS, tap1 = g1 - m1 * RS;
    const int tr = tap1 / p.S, ts = tap1 - tr * p.S;
    unsigned po = 0;
    int pdb = -32768;
    if (m + 1 < p.macro_steps) {
      const int tt = (m + 1) / p.c_chunks, cc = (m + 1) - tt * p.c_chunks;
      po = 256u + (unsigned)(tt * p.dd * p.H * p.W) * pos_bytes + (unsigned)cc * 128u;
      pdb = tt * p.dd - 32768;
    }
    int v0 = tap * p.pls, v0n = (tap + 1 == RS ? 0 : tap + 1) * p.pls;
    if (v0 > 0x7ff0) v0 = 0x7ff0;
    if (v0n > 0x7ff0) v0n = 0x7ff0;
    int* const e = tb + (int64_t)g * 8;
    e[0] = (int)wk_of(g + p.nsw);
    e[1] = (int)((unsigned)p.sx_off + (unsigned)(m1 & (p.xbufs - 1)) * xbuf_bytes +
                 (unsigned)(tr * p.dh * p.Wp + ts * p.dw) * 128u);
    e[2] = (int)po;
    e[3] = pdb;
    e[4] = v0 | (v0n << 16);
    e[5] = m;
    e[6] = (int)((unsigned)p.sx_off + (unsigned)((m + 1) & (p.xbufs - 1)) * xbuf_bytes);
    e[7] = (int)wk_of(g);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void amos_conv_prepare(const ConvFpropParams p) {
  __shared__ __attribute__((aligned(16))) T tile[64][128 / sizeof(T) + 8 / sizeof(T)];
  const int t = threadIdx.x;
  int b = blockIdx.x;
  const int TRS = p.T * p.R * p.S;
  if (b < p.prep_w_blocks) {
    // wp[k][tap][c] = w[k][c][tap], walking the OUTPUT order (writes coalesce, the gathered
    // reads of a wave stay inside one channel's C*TRS slab); four independent elements per
    // thread so that the loads overlap
    const T* w = (const T*)p.w;
    T* wp = (T*)p.wp;
    const int slab = p.C * TRS, slab_src = p.Csrc * TRS;
    const int64_t total = (int64_t)p.K * slab;
    for (int64_t base = (int64_t)b * 1024; base < total; base += (int64_t)p.prep_w_blocks * 1024) {
      T v[4];
      int64_t of[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        of[u] = base + t + 256 * u;
        const int64_t oc = of[u] < total ? of[u] : total - 1;
        const int k = fast_div((int)oc, p.fd_slab);   // the host keeps the packed weights under 2^31 elements
        const int o = (int)(oc - (int64_t)k * slab);
        const int tap = fast_div(o, p.fd_c), c = o - tap * p.C;
        v[u] = c >= p.Csrc ? (T)0
                           : p.layout == 0 ? w[(int64_t)k * slab_src + c * TRS + tap]
                                           : w[((int64_t)tap * p.Csrc + c) * p.K + k];
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (of[u] < total) wp[of[u]] = v[u];
    }
    if (b == 0) {
      if (t < 64) ((int*)p.zeros)[t] = 0;
      conv_write_steps(p, (int)sizeof(T), t);
    }
    return;
  }
  b -= p.prep_w_blocks;
  if (b < p.prep_x_blocks && p.layout != 0) {
    // channels are innermost already: 16-byte chunks, four per thread; DHWNC moves image n's
    // positions from [s][n] to [n][s]
    const int cpp = p.C * (int)sizeof(T) / 16;           // chunks per position
    const int cpp_src = p.Csrc * (int)sizeof(T) / 16;    // (the host pads channels only in whole chunks here)
    const int64_t dhw = (int64_t)p.D * p.H * p.W;
    const int64_t total = (int64_t)p.N * dhw * cpp;
    const uint4* x = (const uint4*)p.x;
    uint4* xt = (uint4*)p.xt;
    uint4 v[4];
    int64_t of[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      of[u] = (int64_t)b * 1024 + t + 256 * u;
      const int64_t oc = of[u] < total ? of[u] : total - 1;
      const int64_t pos = oc / cpp;
      const int ch = (int)(oc - pos * cpp);
      int64_t spos = pos;
      if (p.layout == 2) {
        const int64_t n = pos / dhw, s = pos - n * dhw;
        spos = s * p.N + n;
      }
      v[u] = ch < cpp_src ? x[spos * cpp_src + ch] : uint4{0, 0, 0, 0};
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (of[u] < total) xt[of[u]] = v[u];
    return;
  }
  if (b < p.prep_x_blocks) {
    // xt[slice][s][c] = x[n][c][d][s] through an LDS tile of 128 bytes of channels x 64
    // positions, moved 8 bytes per lane on both sides where the rows of x are 8-byte aligned
    constexpr int ES = (int)sizeof(T);
    constexpr int CT = 128 / ES;          // channels per tile
    constexpr int VE = 8 / ES;            // elements per 8-byte access
    constexpr int PITCH = CT + VE;        // LDS row (one position) in elements: 136 bytes
    constexpr int LTR = 64 / VE;          // loading threads per channel row
    constexpr int LROWS = 256 / LTR;      // channel rows per pass
    T* const tl = &tile[0][0];
    static_assert(sizeof(tile) >= (size_t)64 * PITCH * ES, "transpose tile");
    const int HW = p.H * p.W;
    const int s_tiles = (HW + 63) / 64, c_tiles = p.C / CT;
    const int per_slice = s_tiles * c_tiles;
    const int slice = b / per_slice;
    const int rem = b - slice * per_slice;
    const int st = rem / c_tiles, ct = rem - st * c_tiles;
    const int n = slice / p.D, d = slice - n * p.D;
    const T* x = (const T*)p.x;
    T* xt = (T*)p.xt;
    const bool vec = ((((uintptr_t)x) | (uintptr_t)((int64_t)HW * ES)) & 7) == 0;
    const int ls = (t % LTR) * VE, lc = t / LTR;   // this thread's positions / channel row in a pass
#pragma unroll
    for (int r = 0; r < CT / LROWS; ++r) {
      const int cl = lc + LROWS * r;
      const int sg = st * 64 + ls;
      const int ch = ct * CT + cl;
      const T* src = x + ((((int64_t)n * p.Csrc + (ch < p.Csrc ? ch : 0)) * p.D + d) * HW + sg);
      T v[VE];
      if (ch >= p.Csrc) {
#pragma unroll
        for (int e = 0; e < VE; ++e) v[e] = (T)0;
      } else if (vec && sg + VE <= HW) {
        *(uint2*)v = *(const uint2*)src;
      } else {
#pragma unroll
        for (int e = 0; e < VE; ++e) v[e] = sg + e < HW ? src[e] : (T)0;
      }
#pragma unroll
      for (int e = 0; e < VE; ++e) tl[(ls + e) * PITCH + cl] = v[e];
    }
    __syncthreads();
    const int oc = (t % 16) * VE, os = t / 16;   // 16 lanes x 8 bytes = one position's 128 bytes
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int sl = os + 16 * r, so = st * 64 + sl;
      if (so < HW)
        *(uint2*)(xt + ((int64_t)slice * HW + so) * p.C + ct * CT + oc) = *(const uint2*)(tl + sl * PITCH + oc);
    }
    return;
  }
  b -= p.prep_x_blocks;
  int* z = (int*)p.y;
  for (int64_t idx = (int64_t)b * 256 + t; idx < p.zero_words; idx += (int64_t)p.prep_z_blocks * 256)
    z[idx] = 0;
}

// wait until at most n of this wave's vector-memory loads are outstanding (n is wave-uniform;
// values without a case of their own round down, which only waits longer)
__device__ __forceinline__ void wait_vmcnt_le(int n) {
  if (n <= 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  else if (n < 2) asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
  else if (n < 3) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
  else if (n < 4) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
  else if (n < 6) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
  else if (n < 8) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
  else if (n < 10) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  else if (n < 12) asm volatile("s_waitcnt vmcnt(10)" ::: "memory");
  else if (n < 16) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
  else if (n < 20) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
  else if (n < 24) asm volatile("s_waitcnt vmcnt(20)" ::: "memory");
  else if (n < 32) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(32)" ::: "memory");
}

// ---- launch 2: the convolution -----------------------------------------------------------------
// Every K step does exactly the same work, so that its body is one straight run of instructions the
// MFMAs can overlap: PL patch copies (of the next macro step's patch; copies a wave has no use for
// fetch zeros into a dump line), one weight tile (steps past the end re-fetch the last tile), the
// operand fragments of the next step, the MFMAs of this one.  What differs between steps is read
// from the step table with one scalar load a step ahead.  With all steps alike, the number of
// copies in flight behind the tile a step waits for is the same at every step.
//
// OCC = workgroups the compiler must leave room for on a CU (register budget 512 / OCC per lane)
//
// BI64 x BJ64 = block tile in units of 64; NW = 4 or 8 waves.  A SIMD issues one instruction of a
// wave every ~4 cycles, and a step of a small wave tile is ~100 instructions around a handful of
// MFMAs: with 8 waves a SIMD holds two instruction streams and interleaves them.
//
// W9 = 1: the window has nine taps per macro step (3x3, also 3x3x3 per depth tap) and the ring
// three stages.  The tap loop is unrolled, so ring stages, patch buffers, patch read addresses
// per tap, copy slots and wait counts are compile-time or precomputed registers, and a step is
// about half the instructions of the table-driven one.  The patch buffers are a fixed distance
// apart, a multiple of 8 KB so that a position has the same swizzle in both: 48 KB next to
// 128-row weight tiles (fits the 16-bit offset field of ds_read), 64 KB next to 64-row ones
// (512 positions; the second buffer's read addresses cost an addition each).
constexpr unsigned conv_w9_xbuf(int bi) { return bi <= 64 ? 64 * 1024 : 48 * 1024; }
template <int N> struct IntC { static constexpr int value = N; };

template <int DT, int BI64, int BJ64, int NW, int PL, int OCC, int W9 = 0>
__global__ __launch_bounds__(64 * NW, OCC) void amos_conv_fprop(const ConvFpropParams p) {
  typedef Mfma<DT> MM;
  typedef typename MM::acc_t acc_t;
  typedef typename MM::out_t out_t;
  constexpr int ES = MM::ES;
  constexpr int BI = 64 * BI64, BJ = 64 * BJ64;
  constexpr int WJ = NW == 4 ? 2 : (BJ >= 128 ? 4 : 2), WI = NW / WJ;   // wave grid
  constexpr int TI = BI / (32 * WI), TJ = BJ / (32 * WJ);               // 32x32 tiles per wave
  static_assert(TI >= 1 && TJ >= 1 && TI * WI * 32 == BI && TJ * WJ * 32 == BJ, "wave tile");
  constexpr int WCH = BI / 8 / NW;    // 1 KB weight copy instructions per wave per K step
  static_assert(WCH >= 1 && WCH * NW * 8 == BI, "weight copies");
  constexpr int WSTAGE = BI * 128;

  // dynamic LDS: [nsw][BI*128] weight ring | [xbufs][max_pos*128] patches (at sx_off, 8 KB
  // multiples) | [max_pos] position table (tab_off) | 1 KB dump line (dump_off)
  // All LDS addressing below is by byte offset from 0: the kernel has no static LDS, so its
  // dynamic LDS starts there (the host checks the kernel's static LDS size before the first launch).
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wi = wave / WJ, wj = wave % WJ;
  const int frag_row = lane & 31, frag_half = lane >> 5;

  // W9 = 2: the block walks the tiles blockIdx.x, blockIdx.x + gridDim.x, ...; else one tile
  constexpr bool PERSIST = W9 == 2;
  const int m_begin = blockIdx.y * p.macro_per_split;
  int m_end = m_begin + p.macro_per_split;
  if (m_end > p.macro_steps) m_end = p.macro_steps;
  const int RS = p.R * p.S;
  const int OPQ = p.OP * p.OQ;
  const int HW = p.H * p.W;
  const int n_steps = (m_end - m_begin) * RS;
  const int NSW = p.nsw;
  const unsigned xbuf_bytes = (unsigned)p.max_pos * 128u;
  const unsigned pos_bytes = (unsigned)p.C * ES;

  // ---- what depends on the tile: its origin and image slices (wave-uniform scalars) --------------
  typedef int seg4_t __attribute__((ext_vector_type(4)));
  struct TileGeo {
    int bi0, bj0, j_last, sl_a, nseg, npos;
    // per slice, as vector values (arrays inside the struct would live in scratch memory)
    seg4_t seg_pos0, seg_pa, seg_base, seg_d0;
  };
  static_assert(kConvMaxSeg == 4, "TileGeo holds four segments");
  const int halo_rows = (p.R - 1) * p.dh + 1;
  auto geo_of = [&](int tile_i, int tile_j) {
    TileGeo q;
    q.bi0 = tile_i * BI;
    q.bj0 = tile_j * BJ;
    q.j_last = (q.bj0 + BJ - 1 < p.J ? q.bj0 + BJ - 1 : p.J - 1);
    q.sl_a = fast_div(q.bj0, p.fd_opq);
    const int sl_b = fast_div(q.j_last, p.fd_opq);
    q.nseg = sl_b - q.sl_a + 1;
    int pos = 0;
#pragma unroll
    for (int g = 0; g < kConvMaxSeg; ++g) {
      const int sl = q.sl_a + (g < q.nseg ? g : q.nseg - 1);
      const int lo = q.bj0 > sl * OPQ ? q.bj0 : sl * OPQ;
      const int hi = q.j_last < (sl + 1) * OPQ - 1 ? q.j_last : (sl + 1) * OPQ - 1;
      const int pa = fast_div(lo - sl * OPQ, p.fd_oq), pb = fast_div(hi - sl * OPQ, p.fd_oq);
      const int rows = (pb - pa) * p.sh + halo_rows;
      const int n = fast_div(sl, p.fd_od);
      q.seg_pos0[g] = pos;
      q.seg_pa[g] = pa;
      q.seg_d0[g] = (sl - n * p.OD) * p.sd - p.pd;
      q.seg_base[g] = (n * p.D + q.seg_d0[g]) * HW;   // position index of (n, d0, 0, 0)
      pos += g < q.nseg ? rows * p.Wp : 0;
    }
    q.npos = pos;
    return q;
  };
  // ---- weight copy slots ---------------------------------------------------------------------
  const unsigned w_row_bytes = (unsigned)(p.T * RS) * pos_bytes;
  auto weight_rows = [&](int bi0, unsigned (&wo)[WCH]) {
#pragma unroll
    for (int u = 0; u < WCH; ++u) {
      const int q = wave + NW * u;   // 1 KB chunk = 8 rows
      const int row = q * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ ((row ^ (row >> 3)) & 7);
      const int r = bi0 + row < p.K ? bi0 + row : p.K - 1;
      wo[u] = (unsigned)r * w_row_bytes + chunk * 16;
    }
  };
  unsigned w_off[WCH];
  const int tile_j0 = (int)(blockIdx.x / (unsigned)p.tiles_i), tile_i0 = (int)blockIdx.x - tile_j0 * p.tiles_i;
  weight_rows(tile_i0 * BI, w_off);
  // weight tile whose K slice starts wk bytes into a packed weight row -> ring stage at stage_off
  // (32-bit offsets from the packed weights: the host keeps them under 4 GiB)
  auto issue_weights = [&](const unsigned (&wo)[WCH], unsigned wk, unsigned stage_off) {
#pragma unroll
    for (int u = 0; u < WCH; ++u)
      __builtin_amdgcn_global_load_lds(AMOS_GLOBAL_PTR(p.wp + (size_t)(wo[u] + wk)),
                                       AMOS_LDS_PTR_RW(stage_off + (unsigned)(wave + NW * u) * 1024), 16, 0, 0);
  };

  // step table, read with scalar loads
  typedef int v8i_t __attribute__((ext_vector_type(8)));
  const __attribute__((address_space(4))) v8i_t* const tbl =
      (const __attribute__((address_space(4))) v8i_t*)p.steps;
  int g = m_begin * RS;   // table index of the current step
  // the first NSW weight tiles go out before anything else: they need no set-up, and their
  // latency covers the position table and the first patch
  if (n_steps > 0) {
    const unsigned last = (unsigned)(p.total_steps - 1);
    for (int u = 0; u < NSW; ++u) {
      const unsigned gu = (unsigned)(g + u) < last ? (unsigned)(g + u) : last;
      issue_weights(w_off, (unsigned)tbl[gu][7], (unsigned)u * WSTAGE);
    }
  }

  TileGeo geo = geo_of(tile_i0, tile_j0);

  // position table of a tile: {byte offset of the position's channels in NDHWC at depth tap 0
  // (modulo 2^32; a depth shift is added before use), d0 + 32768, or 0 when (h, w) lies outside
  // the image}
  auto write_table = [&](const TileGeo& q, int tab_off) {
    const int npos8 = (q.npos + 7) & ~7;
    for (int pos = t; pos < npos8; pos += 64 * NW) {
      int g_pos0 = 0, g_pa = q.seg_pa[0], g_base = q.seg_base[0], g_d0 = q.seg_d0[0];
#pragma unroll
      for (int g = 1; g < kConvMaxSeg; ++g)
        if (g < q.nseg && pos >= q.seg_pos0[g]) { g_pos0 = q.seg_pos0[g]; g_pa = q.seg_pa[g]; g_base = q.seg_base[g]; g_d0 = q.seg_d0[g]; }
      const int rel = pos - g_pos0;
      const int hr = fast_div(rel, p.fd_wp);
      const int wc = rel - hr * p.Wp;
      const int h = g_pa * p.sh - p.ph + hr, w = wc - p.pw;
      const bool ok = pos < q.npos && (unsigned)h < (unsigned)p.H && (unsigned)w < (unsigned)p.W;
      const int2 e = int2{(int)((unsigned)(g_base + h * p.W + w) * pos_bytes), ok ? g_d0 + 32768 : 0};
      ((int2*)(smem + tab_off))[pos] = e;
    }
  };
  write_table(geo, p.tab_off);

  // ---- patch copies: copy v of this wave fills positions [8q, 8q+8), q = wave + NW*v -------------
  auto copies_of = [&](int npos) {   // copies this wave owns per patch
    const int n_chunks8 = (npos + 7) >> 3;
    return n_chunks8 > wave ? (n_chunks8 - wave + NW - 1) / NW : 0;
  };
  int n_pl = copies_of(geo.npos);
  // table and copy count the patch copies read from: those of the tile whose patch is fetched
  unsigned tab_lane = (unsigned)p.tab_off + (unsigned)(lane >> 3) * 8;
  int n_pl_rd = n_pl;
  // 16-byte chunk a lane fetches: the swizzle of the LDS position it fills (8 KB-aligned buffers)
  const unsigned lane_c16 = (unsigned)((lane & 7) ^ (lane >> 3)) << 4;
  // The table is read with an explicit ds_read the compiler does not see as a memory access: next
  // to outstanding global -> LDS copies it would otherwise wait for all of them before an LDS
  // load it cannot tell apart from their destinations.  The caller waits (lgkmcnt) before use.
  auto read_tab = [&](int v) {
    int vq = v < n_pl_rd - 1 ? v : n_pl_rd - 1;
    if (vq < 0) vq = 0;
    int2 e;
    asm volatile("ds_read_b64 %0, %1" : "=v"(e) : "v"(tab_lane + (unsigned)(wave + NW * vq) * 64));
    return e;
  };
  // one copy: table entry e of the lane's position; po = the macro step's uniform source offset
  // from the zero block, pdb = its depth shift - 32768, cq = the lane's chunk for the LDS line
  // being filled; depth_limit = D, or 0 for a copy that only moves zeros
  auto patch_copy = [&](int2 e, unsigned cq, unsigned po, int pdb, unsigned dst_off, unsigned depth_limit) {
    const int d = e.y + pdb;
    const unsigned src = (unsigned)e.x + po + cq;
    const unsigned voff = (unsigned)d < depth_limit ? src : cq;
    __builtin_amdgcn_global_load_lds(AMOS_GLOBAL_PTR(p.zeros + (size_t)voff), AMOS_LDS_PTR_RW(dst_off), 16, 0, 0);
  };
  // q & 7 = (wave + NW * (v & 1)) & 7: two chunk patterns per lane (one with 8 waves)
  const unsigned lane_cq[2] = {lane_c16 ^ ((unsigned)(wave & 7) << 4), lane_c16 ^ ((unsigned)((wave + NW) & 7) << 4)};

  // ---- this lane's output columns -> patch positions ---------------------------------------------
  unsigned col_byte[TJ];
  auto column_bytes = [&](const TileGeo& q) {
#pragma unroll
    for (int b = 0; b < TJ; ++b) {
      int j = q.bj0 + (wj * TJ + b) * 32 + frag_row;
      if (j > q.j_last) j = q.j_last;
      const int sl = fast_div(j, p.fd_opq), rem = j - sl * OPQ;
      const int op = fast_div(rem, p.fd_oq), oq = rem - op * p.OQ;
      int g_pos0 = q.seg_pos0[0], g_pa = q.seg_pa[0];
#pragma unroll
      for (int g = 1; g < kConvMaxSeg; ++g)
        if (sl - q.sl_a == g) { g_pos0 = q.seg_pos0[g]; g_pa = q.seg_pa[g]; }
      col_byte[b] = (unsigned)(g_pos0 + (op - g_pa) * p.sh * p.Wp + oq * p.sw) * 128u;
    }
  };
  column_bytes(geo);
  // LDS byte offsets: weights by (parity of the 32-row tile, sub-step), the lane's chunk per sub-step
  unsigned a_off[2][4], kh[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    kh[ks] = (unsigned)(ks * 2 + frag_half) << 4;
#pragma unroll
    for (int par = 0; par < 2; ++par)
      a_off[par][ks] = (unsigned)lds_chunk_offset(wi * TI * 32 + par * 32 + frag_row, ks * 2 + frag_half);
  }

  acc_t acc[TI][TJ];
#pragma unroll
  for (int a = 0; a < TI; ++a)
#pragma unroll
    for (int b = 0; b < TJ; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0;

  // Operand fragments of a whole K step (4 sub-steps) are read one step ahead: with wave tiles
  // this small, the MFMAs of one sub-step are too few to cover the LDS latency of the next.
  v4i af[2][4][TI], bf[2][4][TJ];
  // xo: LDS offset of the patch buffer plus the tap's shift, 128 bytes per position
  auto read_step = [&](unsigned wstage_off, unsigned xo, int slot) {
    unsigned xb[TJ], xsw[TJ];   // per column: LDS address of its position at this tap, swizzle term
#pragma unroll
    for (int b = 0; b < TJ; ++b) {
      xb[b] = col_byte[b] + xo;
      xsw[b] = ((xb[b] >> 3) ^ (xb[b] >> 6)) & 0x70;   // ((pos ^ pos >> 3) & 7) << 4, pos = byte / 128
    }
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
      for (int a = 0; a < TI; ++a)
        af[slot][ks][a] = *(const v4i*)AMOS_LDS_PTR_FROM(a_off[a & 1][ks] + wstage_off + (a >> 1) * (64 * 128));
#pragma unroll
      for (int b = 0; b < TJ; ++b) bf[slot][ks][b] = *(const v4i*)AMOS_LDS_PTR_FROM(xb[b] + (kh[ks] ^ xsw[b]));
    }
  };
  auto mma_step = [&](int slot) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int a = 0; a < TI; ++a)
#pragma unroll
        for (int b = 0; b < TJ; ++b) acc[a][b] = MM::run(af[slot][ks][a], bf[slot][ks][b], acc[a][b]);
  };

  // ---- epilogue: Y[(n*K + i)*ODPQ + (od*OPQ + opq)] ---------------------------------------------
  auto store_tile = [&](const TileGeo& q) {
  out_t* const out = (out_t*)p.y + (int64_t)blockIdx.y * p.split_stride;
  const int ODPQ = p.OD * OPQ;
  const bool full = q.bi0 + BI <= p.K && q.bj0 + BJ <= p.J && !p.atomic_out;
  const int64_t y_si = p.y_si;
#pragma unroll
  for (int b = 0; b < TJ; ++b) {
    const int j = q.bj0 + (wj * TJ + b) * 32 + frag_row;
    const int jc = j < p.J ? j : p.J - 1;
    const int n = fast_div(jc, p.fd_odpq);
    const int64_t coff = (int64_t)n * p.y_sn + (int64_t)(jc - n * ODPQ) * p.y_ss;
#pragma unroll
    for (int a = 0; a < TI; ++a) {
      const int i0 = q.bi0 + (wi * TI + a) * 32 + 4 * frag_half;
      out_t* const dst0 = out + (int64_t)i0 * y_si + coff;
      if (p.epi.dt != EPI_NONE && blockIdx.y == 0) {   // one K split adds D; all loads first
        out_t dv[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int i = i0 + 8 * (r >> 2) + (r & 3);
          dv[r] = epi_value<out_t>(p.epi, (int64_t)(i < p.K ? i : p.K - 1) * y_si + coff);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][b][r] += dv[r];
      }
      if (full && p.y_vec4) {
        // channels innermost: a lane's four consecutive channels in one store, a position's 32
        // channels of the tile 128 contiguous bytes
        typedef out_t out4_t __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const out4_t v = {acc[a][b][4 * g4], acc[a][b][4 * g4 + 1], acc[a][b][4 * g4 + 2], acc[a][b][4 * g4 + 3]};
          *(out4_t*)(dst0 + 8 * g4) = v;
        }
      } else if (full) {
#pragma unroll
        for (int r = 0; r < 16; ++r) dst0[(int64_t)(8 * (r >> 2) + (r & 3)) * y_si] = acc[a][b][r];
      } else if (j < p.J) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int di = 8 * (r >> 2) + (r & 3);
          if (i0 + di < p.K) {
            if (p.atomic_out)
              atomicAdd(dst0 + (int64_t)di * y_si, acc[a][b][r]);
            else
              dst0[(int64_t)di * y_si] = acc[a][b][r];
          }
        }
      }
    }
  }
  };

  int2 pt[PL > 0 ? PL : 1];   // table entries of the patch copies of the coming step

  // ---- prologue: the whole first patch, the first NSW weight tiles -------------------------------
  __syncthreads();   // position table visible
  v8i_t cur = tbl[g];
  if (n_steps > 0) {
    {
      const int tt = fast_div(m_begin, p.fd_cc), cc = m_begin - tt * p.c_chunks;
      const unsigned po = 256u + (unsigned)(tt * p.dd * HW) * pos_bytes + (unsigned)cc * 128u;
      const unsigned buf = (unsigned)p.sx_off + (W9 ? 0u : (unsigned)(m_begin & (p.xbufs - 1)) * xbuf_bytes);
      for (int v = 0; v < n_pl; v += 4) {   // four table entries per LDS round trip
        int2 e[4];
#pragma unroll
        for (int x = 0; x < 4; ++x) e[x] = read_tab(v + x);
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(e[0]), "+v"(e[1]), "+v"(e[2]), "+v"(e[3]));
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          const bool live = v + x < n_pl;
          patch_copy(e[x], lane_cq[x & 1], po, tt * p.dd - 32768,
                     live ? buf + (unsigned)(wave + NW * (v + x)) * 1024 : (unsigned)p.dump_off,
                     live ? (unsigned)p.D : 0u);
        }
      }
      // everything issued so far has landed before the first step: its wait then allows the
      // youngest nsw-2 steps' worth of copies in flight, and there are none yet
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      read_step(0, buf, 0);
    }
  }

  // cur = {wk of the tile fetched during this step, xo of the NEXT step's fragments, po and pdb of
  //        the next macro step, v0 | v0 of the next step << 16, macro step, LDS offset of the next
  //        macro step's patch buffer, wk of this step's own tile}
  unsigned istage = 0;   // ring stage (byte offset) this step's fetch goes to = the stage step-1 read
  v8i_t nxt = cur;
  auto one_step = [&](int slot, const v8i_t& e, v8i_t& e_next) {
    // This wave's reads of the current step's operands (issued a step ago) are complete, and so
    // are its copies of everything older than the youngest NSW-2 steps' worth: the next weight
    // tile and, at a macro step's last tap, the next patch.  After the barrier that holds for
    // every wave.
    // The table entries of this step's patch copies: read here, waited for and tied to the barrier
    // statement below.  (An explicit ds_read's result must not be live across a loop edge: the
    // compiler does not know it arrives late and may copy the register before it has.)
    if (PL > 0) {
      const int v0 = e[4] & 0xffff;
#pragma unroll
      for (int x = 0; x < PL; ++x) pt[x] = read_tab(v0 + x);
    }
    if (NSW >= 4) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (PL + WCH)) : "memory");
    else if (NSW == 3) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(PL + WCH) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    // (the table entries read a step ago are tied to the wait, so that nothing uses them before it)
    if (PL == 4)
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : "+v"(pt[0]), "+v"(pt[1]), "+v"(pt[PL > 2 ? 2 : 0]), "+v"(pt[PL > 2 ? 3 : 0])::"memory");
    else if (PL == 2)
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : "+v"(pt[0]), "+v"(pt[PL > 1 ? 1 : 0])::"memory");
    else
      asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    // (every word of the entry stays live up to here: a register of the tuple that is reused
    // earlier makes the compiler wait for the scalar load right after issuing it)
    asm volatile("" ::"s"(e[0]), "s"(e[1]), "s"(e[2]), "s"(e[3]), "s"(e[4]), "s"(e[5]), "s"(e[6]), "s"(e[7]));
    // operands of the next K step first: LDS is the busiest unit of a step, the MFMAs of this step
    // (whose operands are in registers already) run while it delivers
    const unsigned rstage = istage + WSTAGE == (unsigned)NSW * WSTAGE ? 0u : istage + WSTAGE;
    read_step(rstage, (unsigned)e[1], slot ^ 1);
    mma_step(slot);
    // patch of the next (depth tap, channel chunk): BEFORE this step's weight tile, so that the
    // copies are older than a tile that is waited for before the patch is first read
    if (PL > 0) {
      const int n_live = e[5] + 1 < m_end ? n_pl : 0;
      const int v0 = e[4] & 0xffff;   // even with 4 waves: their copies per step come in twos
      const unsigned dst0 = (unsigned)e[6] + (unsigned)wave * 1024 + (unsigned)v0 * (NW * 1024);
#pragma unroll
      for (int x = 0; x < PL; ++x) {
        const bool live = v0 + x < n_live;
        patch_copy(pt[x], lane_cq[x & 1], (unsigned)e[2], e[3], live ? dst0 + x * (NW * 1024) : (unsigned)p.dump_off,
                   live ? (unsigned)p.D : 0u);
      }
    }
    issue_weights(w_off, (unsigned)e[0], istage);   // tile step+NSW into the stage just freed
    istage = rstage;
    // the next step's table entry, last: it has until the top of the next step to arrive
    __builtin_amdgcn_sched_barrier(0);
    ++g;
    e_next = tbl[g];
  };
  if constexpr (!W9) {
    int step = 0;
    for (; step + 1 < n_steps; step += 2) {
      one_step(0, cur, nxt);
      one_step(1, nxt, cur);
    }
    if (step < n_steps) one_step(0, cur, nxt);
  } else {
    // ---- nine unrolled taps per macro step ------------------------------------------------------
    // patch read addresses per tap (buffer 0): position shift and swizzle term folded in
    unsigned baddr[9][TJ][4];
    auto tap_addresses = [&]() {
      int tr = 0, ts = 0;
#pragma unroll
      for (int tap = 0; tap < 9; ++tap) {
        const unsigned shift = (unsigned)p.sx_off + (unsigned)(tr * p.dh * p.Wp + ts * p.dw) * 128u;
#pragma unroll
        for (int b = 0; b < TJ; ++b) {
          const unsigned xb = col_byte[b] + shift;
          const unsigned key = ((xb >> 3) ^ (xb >> 6)) & 0x70;
#pragma unroll
          for (int ks = 0; ks < 4; ++ks) baddr[tap][b][ks] = xb + (kh[ks] ^ key);
        }
        if (++ts == p.S) { ts = 0; ++tr; }
      }
    };
    tap_addresses();
    const int n_macro = m_end - m_begin;
    // blocks that walk several tiles: the weight rows of the next macro step's tile, whether
    // this macro step is a tile's last with another tile to follow (its last tap then leaves
    // the next operands to the tile switch), whether it is the first after a switch (the
    // stores of the finished tile are then still in flight)
    unsigned w_off_nx[WCH];
#pragma unroll
    for (int u = 0; u < WCH; ++u) w_off_nx[u] = w_off[u];
    bool hand_over = false;
    int after_switch = 0;   // 1: sixteen stores per 32x32 tile in flight, 2: four (vector stores)
    auto wk_of_macro = [&](int m) {
      if (m > p.macro_steps - 1) m = p.macro_steps - 1;
      const int tt = fast_div(m, p.fd_cc), cc = m - tt * p.c_chunks;
      return (unsigned)(tt * 9) * pos_bytes + (unsigned)cc * 128u;
    };
    // one K step: TAP of the macro step in patch buffer BUF
    auto step9 = [&](auto tap_c, auto buf_c, unsigned wk_cur, unsigned wk_nxt, int n_live, unsigned po, int pdb) {
      constexpr int TAP = decltype(tap_c)::value, BUF = decltype(buf_c)::value;
      constexpr int SLOT = (TAP + BUF) & 1;            // nine steps per macro step: the parity flips with BUF
      if constexpr (PL > 0 && TAP <= 6) {
#pragma unroll
        for (int x = 0; x < PL; ++x) pt[x] = read_tab(TAP * PL + x);
      }
      // the copies of the previous step may still be in flight: WCH of the weight tile, PL of the
      // patch if that step was one of the taps 0..6 that fetch it
      constexpr int IN_FLIGHT = WCH + ((TAP >= 1 && TAP <= 7) ? PL : 0);
      if constexpr (PERSIST && TAP <= 1) {
        // memory instructions complete in issue order: the 16 stores per 32x32 tile of the
        // finished tile sit between the copies waited for here and the younger ones
        constexpr int WITH_STORES = IN_FLIGHT + 16 * TI * TJ > 63 ? 63 : IN_FLIGHT + 16 * TI * TJ;
        constexpr int WITH_VSTORES = IN_FLIGHT + 4 * TI * TJ;
        if (after_switch == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(WITH_STORES) : "memory");
        else if (after_switch == 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(WITH_VSTORES) : "memory");
        else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(IN_FLIGHT) : "memory");
      } else {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(IN_FLIGHT) : "memory");
      }
      if (PL == 2)
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : "+v"(pt[0]), "+v"(pt[PL > 1 ? 1 : 0])::"memory");
      else if (PL == 1)
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : "+v"(pt[0])::"memory");
      else
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
      // operands of the next K step
      // (PL = 0: a block runs one macro step and has one patch buffer; its last read is unused)
      constexpr int TN = TAP == 8 ? 0 : TAP + 1, BN = (TAP == 8 && PL > 0) ? BUF ^ 1 : BUF;
      if (!(PERSIST && TAP == 8) || !hand_over) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
          for (int a = 0; a < TI; ++a)
            af[SLOT ^ 1][ks][a] = *(const v4i*)AMOS_LDS_PTR_FROM(a_off[a & 1][ks] + (unsigned)((TN % 3) * WSTAGE + (a >> 1) * (64 * 128)));
#pragma unroll
          for (int b = 0; b < TJ; ++b)
            bf[SLOT ^ 1][ks][b] = *(const v4i*)AMOS_LDS_PTR_FROM(baddr[TN][b][ks] + (unsigned)BN * conv_w9_xbuf(BI));
        }
      }
      mma_step(SLOT);
      // patch of the next macro step, on taps 0..6, before this step's weight tile
      if constexpr (PL > 0 && TAP <= 6) {
#pragma unroll
        for (int x = 0; x < PL; ++x) {
          const int v = TAP * PL + x;
          const bool live = v < n_live;
          const unsigned dst = (unsigned)p.sx_off + (unsigned)(BUF ^ 1) * conv_w9_xbuf(BI) + (unsigned)(wave + NW * v) * 1024;
          patch_copy(pt[x], lane_cq[v & 1], po, pdb, live ? dst : (unsigned)p.dump_off, live ? (unsigned)p.D : 0u);
        }
      }
      // weight tile of the step three ahead, into the stage the previous step read
      constexpr int NT = TAP + 3;
      if constexpr (NT < 9) issue_weights(w_off, wk_cur + (unsigned)NT * pos_bytes, (unsigned)((TAP % 3) * WSTAGE));
      else issue_weights(w_off_nx, wk_nxt + (unsigned)(NT - 9) * pos_bytes, (unsigned)((TAP % 3) * WSTAGE));
    };
    auto nine_taps = [&](auto buf_c, unsigned wk_cur, unsigned wk_nxt, int n_live, unsigned po, int pdb) {
      step9(IntC<0>{}, buf_c, wk_cur, wk_nxt, n_live, po, pdb);
      step9(IntC<1>{}, buf_c, wk_cur, wk_nxt, n_live, po, pdb);
      step9(IntC<2>{}, buf_c, wk_cur, wk_nxt, n_live, po, pdb);
      step9(IntC<3>{}, buf_c, wk_cur, wk_nxt, n_live, po, pdb);
      step9(IntC<4>{}, buf_c, wk_cur, wk_nxt, n_live, po, pdb);
      step9(IntC<5>{}, buf_c, wk_cur, wk_nxt, n_live, po, pdb);
      step9(IntC<6>{}, buf_c, wk_cur, wk_nxt, n_live, po, pdb);
      step9(IntC<7>{}, buf_c, wk_cur, wk_nxt, n_live, po, pdb);
      step9(IntC<8>{}, buf_c, wk_cur, wk_nxt, n_live, po, pdb);
    };
    auto macro9 = [&](auto buf_c, int mi) {
      const int m = m_begin + mi;
      const unsigned wk_cur = wk_of_macro(m), wk_nxt = wk_of_macro(m + 1);
      const int n_live = m + 1 < m_end ? n_pl : 0;
      const int tt1 = fast_div(m + 1, p.fd_cc), cc1 = (m + 1) - tt1 * p.c_chunks;
      const unsigned po = 256u + (unsigned)(tt1 * p.dd * HW) * pos_bytes + (unsigned)cc1 * 128u;
      const int pdb = tt1 * p.dd - 32768;
      nine_taps(buf_c, wk_cur, wk_nxt, n_live, po, pdb);
    };
    if constexpr (!PERSIST) {
      for (int mi = 0; mi < n_macro; mi += 2) {
        macro9(IntC<0>{}, mi);
        if (mi + 1 < n_macro) macro9(IntC<1>{}, mi + 1);
      }
    } else {
      // ---- a block's tiles, one after the other ---------------------------------------------------
      // The macro steps of all its tiles form one sequence: the last macro step of a tile fetches
      // the first patch and the first weight tiles of the next tile, so that only the output
      // stores and the new tile's addresses stand between two tiles.  The position table of the
      // next tile is written (into the other of two tables) when a tile starts; the step barriers
      // of the macro steps before its first use publish it.  The host launches such blocks
      // without split-K and with at least two macro steps per tile.
      const int total_tiles = p.tiles_i * p.tiles_j;
      int tile = (int)blockIdx.x;
      int buf = 0;            // patch buffer of the current macro step
      int tab_cur = p.tab_off, tab_oth = p.tab1_off;
      for (;;) {
        const int next_tile = tile + (int)gridDim.x;
        const bool has_next = next_tile < total_tiles;
        TileGeo geo_n = geo;
        int n_pl_n = n_pl;
        if (has_next) {
          const int tj = (int)((unsigned)next_tile / (unsigned)p.tiles_i);
          geo_n = geo_of(next_tile - tj * p.tiles_i, tj);
          write_table(geo_n, tab_oth);
          n_pl_n = copies_of(geo_n.npos);
        }
        for (int m = 0; m < n_macro; ++m) {
          const bool last = m == n_macro - 1;
          hand_over = last && has_next;
          unsigned wk_nxt, po;
          int pdb, n_live;
          if (!last) {
            const int tt1 = fast_div(m + 1, p.fd_cc), cc1 = (m + 1) - tt1 * p.c_chunks;
            wk_nxt = wk_of_macro(m + 1);
            po = 256u + (unsigned)(tt1 * p.dd * HW) * pos_bytes + (unsigned)cc1 * 128u;
            pdb = tt1 * p.dd - 32768;
            n_live = n_pl;
            n_pl_rd = n_pl;
            tab_lane = (unsigned)tab_cur + (unsigned)(lane >> 3) * 8;
          } else {
            // macro step 0 of the next tile (of this one again, unused, when there is none)
            wk_nxt = 0;
            po = 256u;
            pdb = -32768;
            n_live = has_next ? n_pl_n : 0;
            n_pl_rd = n_pl_n;
            tab_lane = (unsigned)(has_next ? tab_oth : tab_cur) + (unsigned)(lane >> 3) * 8;
            if (has_next) weight_rows(geo_n.bi0, w_off_nx);
          }
          if (buf == 0) nine_taps(IntC<0>{}, wk_of_macro(m), wk_nxt, n_live, po, pdb);
          else nine_taps(IntC<1>{}, wk_of_macro(m), wk_nxt, n_live, po, pdb);
          buf ^= 1;
          after_switch = 0;
        }
        store_tile(geo);
        if (!has_next) break;
        // a ragged tile issues fewer stores than the waits after the switch allow for
        const bool counted = geo.bi0 + BI <= p.K && geo.bj0 + BJ <= p.J;
        if (!counted) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        after_switch = counted ? (p.y_vec4 ? 2 : 1) : 0;
        geo = geo_n;
        n_pl = n_pl_n;
        tile = next_tile;
        { const int x = tab_cur; tab_cur = tab_oth; tab_oth = x; }
#pragma unroll
        for (int u = 0; u < WCH; ++u) w_off[u] = w_off_nx[u];
        column_bytes(geo);
        tap_addresses();
#pragma unroll
        for (int a = 0; a < TI; ++a)
#pragma unroll
          for (int b = 0; b < TJ; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0;
        // operands of the new tile's first step: tap 0 in the buffer its patch was fetched to,
        // into the fragment slot that step computes from (the parity of tap + buffer)
        auto first_operands = [&](auto buf_c) {
          constexpr int B = decltype(buf_c)::value;
#pragma unroll
          for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
            for (int a = 0; a < TI; ++a)
              af[B][ks][a] = *(const v4i*)AMOS_LDS_PTR_FROM(a_off[a & 1][ks] + (unsigned)((a >> 1) * (64 * 128)));
#pragma unroll
            for (int b = 0; b < TJ; ++b)
              bf[B][ks][b] = *(const v4i*)AMOS_LDS_PTR_FROM(baddr[0][b][ks] + (unsigned)B * conv_w9_xbuf(BI));
          }
        };
        if (buf == 0) first_operands(IntC<0>{});
        else first_operands(IntC<1>{});
      }
    }
  }

  if constexpr (!PERSIST) store_tile(geo);
  // the re-fetched tiles of the last steps still target this block's LDS
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#if AMOS_SPLIT_IN_KERNEL
  if constexpr (!PERSIST) {
    if (p.fin.tickets) {
      const int ODPQ = p.OD * OPQ;
      split_finish<out_t>(p.fin, blockIdx.x, (const out_t*)p.y, (int)threadIdx.x, (int)blockDim.x, BI, BJ,
                          (lds_flag_t)(size_t)0, [&](int r, int c) -> int64_t {
                            const int i = geo.bi0 + r, j = geo.bj0 + c;
                            if (i >= p.K || j >= p.J) return -1;
                            const int n = fast_div(j, p.fd_odpq);
                            return (int64_t)n * p.y_sn + (int64_t)(j - n * ODPQ) * p.y_ss + (int64_t)i * p.y_si;
                          });
    }
  }
#endif
}

}  // namespace amos
