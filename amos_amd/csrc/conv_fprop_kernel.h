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

#include "gemm_tn_kernel.h"
#include "igemm_kernel.h"

namespace amos {

constexpr int kConvMaxSeg = 4;

// n / d for 0 <= n < 2^31 with a host-built multiplier: two scalar (or vector) instructions
// where a hardware-less integer division costs dozens
struct FastDiv {
  uint32_t magic, shift, one;
};
inline FastDiv make_fast_div(uint32_t d) {
  FastDiv f = {0, 0, 0};
  if (d <= 1) { f.one = 1; return f; }
  uint32_t l = 0;
  while ((1ull << l) < d) ++l;               // ceil(log2 d), >= 1
  const uint64_t s = 31 + l;
  f.magic = (uint32_t)(((1ull << s) + d - 1) / d);   // ceil(2^s / d) < 2^32
  f.shift = (uint32_t)(s - 32);
  return f;
}
__device__ __forceinline__ int fast_div(int n, const FastDiv& f) {
  return f.one ? n : (int)(__umulhi((unsigned)n, f.magic) >> f.shift);
}

#define AMOS_LDS_PTR_FROM(off) ((const __attribute__((address_space(3))) char*)(size_t)(off))

struct ConvFpropParams {
  const char* x;     // original NCDHW activations (prepare kernel input)
  const char* w;     // original KCTRS weights (prepare kernel input)
  char* xt;          // NDHWC activations (workspace)
  char* wp;          // packed weights [K][T*R*S][C] (workspace)
  char* zeros;       // 128 zero bytes (workspace)
  char* y;           // NKDPQ, fp32 / int32
  int N, C, D, H, W, K, T, R, S;
  int sd, sh, sw, pd, ph, pw, dd, dh, dw;
  int OD, OP, OQ;
  int J;             // N*OD*OP*OQ
  int Wp;            // patch columns: (OQ-1)*sw + (S-1)*dw + 1
  int max_pos;       // LDS positions reserved per patch buffer (multiple of 8)
  int nsw;           // weight ring stages (>= 2)
  int pls;           // patch copy instructions per wave per K step
  int xbufs;         // patch buffers: 2, or 1 when a block handles a single (depth tap, channel chunk)
  int c_chunks;      // C*ES / 128
  int macro_steps;   // T * c_chunks
  int macro_per_split;
  int tiles_i, tiles_j;
  int atomic_out;
  FastDiv fd_opq, fd_oq, fd_od, fd_wp, fd_odpq, fd_cc, fd_c;   // divisions by OP*OQ, OQ, OD, Wp, OD*OP*OQ, c_chunks, C
  // prepare kernel work split (in blocks)
  int prep_w_blocks, prep_x_blocks, prep_z_blocks;
  int64_t zero_words;
};

// ---- launch 1: relayout ---------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void amos_conv_prepare(const ConvFpropParams p) {
  __shared__ T tile[64][64 + 2];
  const int t = threadIdx.x;
  int b = blockIdx.x;
  const int TRS = p.T * p.R * p.S;
  if (b < p.prep_w_blocks) {
    // wp[k][tap][c] = w[k][c][tap]: one block per output channel k (grid-strided); the
    // k-th slab of C*TRS elements is read contiguously into LDS-free registers by walking the
    // OUTPUT order (writes coalesce, reads stay inside one 1-2 KB slab that L1 holds)
    const T* w = (const T*)p.w;
    T* wp = (T*)p.wp;
    const int slab = p.C * TRS;
    for (int k = b; k < p.K; k += p.prep_w_blocks) {
      const T* src = w + (int64_t)k * slab;
      T* dst = wp + (int64_t)k * slab;
      for (int o = t; o < slab; o += 256) {
        const int tap = fast_div(o, p.fd_c), c = o - tap * p.C;
        dst[o] = src[c * TRS + tap];
      }
    }
    if (b == 0 && t < 32) ((int*)p.zeros)[t] = 0;
    return;
  }
  b -= p.prep_w_blocks;
  if (b < p.prep_x_blocks) {
    // xt[slice][s][c] = x[n][c][d][s] through a 64(c) x 64(s) LDS tile
    const int HW = p.H * p.W;
    const int s_tiles = (HW + 63) / 64, c_tiles = p.C / 64;
    const int per_slice = s_tiles * c_tiles;
    const int slice = b / per_slice;
    const int rem = b - slice * per_slice;
    const int st = rem / c_tiles, ct = rem - st * c_tiles;
    const int n = slice / p.D, d = slice - n * p.D;
    const int tx = t & 63, ty = t >> 6;
    const T* x = (const T*)p.x;
    T* xt = (T*)p.xt;
    const int s = st * 64 + tx;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int c = ct * 64 + ty + 4 * r;
      if (s < HW) tile[ty + 4 * r][tx] = x[(((int64_t)n * p.C + c) * p.D + d) * HW + s];
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int so = st * 64 + ty + 4 * r;
      if (so < HW) xt[((int64_t)slice * HW + so) * p.C + ct * 64 + tx] = tile[tx][ty + 4 * r];
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
  else if (n < 4) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
  else if (n < 6) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
  else if (n < 8) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
  else if (n < 12) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  else if (n < 16) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
  else if (n < 24) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
  else if (n < 32) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(32)" ::: "memory");
}

// ---- launch 2: the convolution -----------------------------------------------------------------
// OCC = workgroups the compiler must leave room for on a CU (register budget 512 / OCC per lane)
template <int DT, int TI, int TJ, int OCC>
__global__ __launch_bounds__(256, OCC) void amos_conv_fprop(const ConvFpropParams p) {
  typedef Mfma<DT> MM;
  typedef typename MM::acc_t acc_t;
  typedef typename MM::out_t out_t;
  constexpr int ES = MM::ES;
  constexpr int BI = 64 * TI, BJ = 64 * TJ;
  constexpr int WCH = BI / 32;    // 1 KB weight copy instructions per wave per K step
  constexpr int WSTAGE = BI * 128;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* const sW = smem;                                            // [nsw][BI*128]
  char* const sX = smem + (size_t)p.nsw * WSTAGE;                   // [xbufs][max_pos*128]
  int2* const sTab = (int2*)(sX + (size_t)p.xbufs * p.max_pos * 128);   // [max_pos] position table

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int wi = wave >> 1, wj = wave & 1;
  const int frag_row = lane & 31, frag_half = lane >> 5;

  const int tile_j = blockIdx.x / p.tiles_i, tile_i = blockIdx.x - tile_j * p.tiles_i;
  const int bi0 = tile_i * BI, bj0 = tile_j * BJ;
  const int m_begin = blockIdx.y * p.macro_per_split;
  int m_end = m_begin + p.macro_per_split;
  if (m_end > p.macro_steps) m_end = p.macro_steps;
  const int n_macro = m_end - m_begin;
  const int RS = p.R * p.S;
  const int OPQ = p.OP * p.OQ;
  const int HW = p.H * p.W;
  const int n_steps = n_macro * RS;
  const int NSW = p.nsw;
  const size_t xbuf_bytes = (size_t)p.max_pos * 128;

  // ---- segments of this tile (wave-uniform scalars) -------------------------------------------
  const int j_last = (bj0 + BJ - 1 < p.J ? bj0 + BJ - 1 : p.J - 1);
  const int sl_a = fast_div(bj0, p.fd_opq), sl_b = fast_div(j_last, p.fd_opq);
  const int nseg = sl_b - sl_a + 1;
  int seg_pos0[kConvMaxSeg + 1], seg_pa[kConvMaxSeg], seg_base[kConvMaxSeg], seg_d0[kConvMaxSeg];
  {
    int pos = 0;
#pragma unroll
    for (int g = 0; g < kConvMaxSeg; ++g) {
      const int sl = sl_a + (g < nseg ? g : nseg - 1);
      const int lo = bj0 > sl * OPQ ? bj0 : sl * OPQ;
      const int hi = j_last < (sl + 1) * OPQ - 1 ? j_last : (sl + 1) * OPQ - 1;
      const int pa = fast_div(lo - sl * OPQ, p.fd_oq), pb = fast_div(hi - sl * OPQ, p.fd_oq);
      const int rows = (pb - pa) * p.sh + (p.R - 1) * p.dh + 1;
      const int n = fast_div(sl, p.fd_od);
      seg_pos0[g] = pos;
      seg_pa[g] = pa;
      seg_d0[g] = (sl - n * p.OD) * p.sd - p.pd;
      seg_base[g] = (n * p.D + seg_d0[g]) * HW;   // position index of (n, d0, 0, 0)
      if (g < nseg) pos += rows * p.Wp;
    }
    seg_pos0[kConvMaxSeg] = pos;
  }
  const int npos = seg_pos0[kConvMaxSeg];
  const int npos8 = (npos + 7) & ~7;

  // position table: {position index in NDHWC for depth tap 0, (h,w outside ? sign bit) | d0 + 32768}
  for (int pos = t; pos < npos8; pos += 256) {
    int g_pos0 = 0, g_pa = seg_pa[0], g_base = seg_base[0], g_d0 = seg_d0[0];
#pragma unroll
    for (int g = 1; g < kConvMaxSeg; ++g)
      if (g < nseg && pos >= seg_pos0[g]) { g_pos0 = seg_pos0[g]; g_pa = seg_pa[g]; g_base = seg_base[g]; g_d0 = seg_d0[g]; }
    const int rel = pos - g_pos0;
    const int hr = fast_div(rel, p.fd_wp);
    const int wc = rel - hr * p.Wp;
    const int h = g_pa * p.sh - p.ph + hr, w = wc - p.pw;
    const bool ok = pos < npos && (unsigned)h < (unsigned)p.H && (unsigned)w < (unsigned)p.W;
    sTab[pos] = int2{g_base + h * p.W + w, (ok ? 0 : (int)0x80000000) | (g_d0 + 32768)};
  }

  // ---- weight copy slots ---------------------------------------------------------------------
  const int64_t w_row_bytes = (int64_t)p.T * RS * p.C * ES;
  unsigned w_off[WCH];
#pragma unroll
  for (int u = 0; u < WCH; ++u) {
    const int q = wave + 4 * u;   // 1 KB chunk = 8 rows
    const int row = q * 8 + (lane >> 3);
    const int chunk = (lane & 7) ^ ((row ^ (row >> 3)) & 7);
    const int r = bi0 + row < p.K ? bi0 + row : p.K - 1;
    w_off[u] = (unsigned)r * (unsigned)w_row_bytes + chunk * 16;
  }
  // next weight tile to issue: (macro step, tap), its ring stage and its (uniform) source
  int iw_m = m_begin, iw_tap = 0, iw_stage = 0, iw_step = 0;
  const int64_t tap_bytes = (int64_t)p.C * ES;
  auto macro_weight_src = [&](int m) {
    const int tt = fast_div(m, p.fd_cc), cc = m - tt * p.c_chunks;
    return p.wp + ((int64_t)tt * RS * tap_bytes + (int64_t)cc * 128);
  };
  const char* iw_src = macro_weight_src(m_begin);
  auto issue_next_weights = [&]() {
    char* s = sW + iw_stage * WSTAGE;
#pragma unroll
    for (int u = 0; u < WCH; ++u)
      __builtin_amdgcn_global_load_lds(AMOS_GLOBAL_PTR(iw_src + w_off[u]), AMOS_LDS_PTR(s + (wave + 4 * u) * 1024),
                                       16, 0, 0);
    ++iw_step;
    iw_src += tap_bytes;
    if (++iw_tap == RS) { iw_tap = 0; ++iw_m; iw_src = macro_weight_src(iw_m); }
    if (++iw_stage == NSW) iw_stage = 0;
  };

  // ---- patch copies: instruction v of this wave fills positions [8q, 8q+8), q = wave + 4v -------
  const int n_chunks8 = npos8 >> 3;
  const int n_pl = n_chunks8 > wave ? (n_chunks8 - wave + 3) >> 2 : 0;   // copies this wave owns per patch
  const unsigned tab_lds = (unsigned)(size_t)AMOS_LDS_PTR(sTab) + (unsigned)(lane >> 3) * 8;
  const int64_t pos_bytes = (int64_t)p.C * ES;
  // patch of macro step m into buffer `buf`: uniform part of the source and the depth shift
  auto issue_patch = [&](int m, int buf, int v) {
    const int tt = fast_div(m, p.fd_cc), cc = m - tt * p.c_chunks;
    const int q = wave + 4 * v;
    // The table is read with an explicit ds_read: next to outstanding global -> LDS copies
    // the compiler would otherwise wait for all of them before any LDS load it cannot
    // tell apart from their destinations.
    int2 e;
    asm volatile("ds_read_b64 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(e) : "v"(tab_lds + (unsigned)q * 64) : "memory");
    const int pos = q * 8 + (lane >> 3);
    const int d = (e.y & 0xffff) - 32768 + tt * p.dd;
    const bool ok = e.y >= 0 && (unsigned)d < (unsigned)p.D;
    const int chunk = (lane & 7) ^ ((pos ^ (pos >> 3)) & 7);
    const char* base = p.xt + ((int64_t)tt * p.dd * HW * pos_bytes + (int64_t)cc * 128);
    const char* src = ok ? base + ((int64_t)e.x * pos_bytes + chunk * 16) : p.zeros + chunk * 16;
    char* dst = sX + (size_t)buf * xbuf_bytes + q * 1024;
    __builtin_amdgcn_global_load_lds(AMOS_GLOBAL_PTR(src), AMOS_LDS_PTR(dst), 16, 0, 0);
  };

  // ---- this lane's output columns -> patch positions ---------------------------------------------
  int col_pos[TJ];
#pragma unroll
  for (int b = 0; b < TJ; ++b) {
    int j = bj0 + (wj * TJ + b) * 32 + frag_row;
    if (j > j_last) j = j_last;
    const int sl = fast_div(j, p.fd_opq), rem = j - sl * OPQ;
    const int op = fast_div(rem, p.fd_oq), oq = rem - op * p.OQ;
    int g_pos0 = seg_pos0[0], g_pa = seg_pa[0];
#pragma unroll
    for (int g = 1; g < kConvMaxSeg; ++g)
      if (sl - sl_a == g) { g_pos0 = seg_pos0[g]; g_pa = seg_pa[g]; }
    col_pos[b] = g_pos0 + (op - g_pa) * p.sh * p.Wp + oq * p.sw;
  }
  // LDS byte offsets: weights by (parity of the 32-row tile, sub-step), the lane's chunk per sub-step
  unsigned a_off[2][4], kh[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    kh[ks] = (unsigned)(ks * 2 + frag_half) << 4;
#pragma unroll
    for (int par = 0; par < 2; ++par)
      a_off[par][ks] = (unsigned)(size_t)AMOS_LDS_PTR(sW) +
                       lds_chunk_offset(wi * TI * 32 + par * 32 + frag_row, ks * 2 + frag_half);
  }
  const unsigned x_lds = (unsigned)(size_t)AMOS_LDS_PTR(sX);

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
  auto read_step = [&](unsigned wstage_off, unsigned xbuf_lds, int dpos, int slot) {
    unsigned xb[TJ], xsw[TJ];   // per column: LDS address of its position at this tap, swizzle term
#pragma unroll
    for (int b = 0; b < TJ; ++b) {
      const int pos = col_pos[b] + dpos;
      xb[b] = xbuf_lds + (unsigned)pos * 128;
      xsw[b] = (unsigned)((pos ^ (pos >> 3)) & 7) << 4;
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
  // wait until at most `later` weight tiles (the youngest) are still in flight
  auto wait_weights = [&](int later) {
    if (later >= 2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * WCH) : "memory");
    else if (later == 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(WCH) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  };

  // ---- prologue: the whole first patch, the first NSW weight tiles -------------------------------
  __syncthreads();   // position table visible
  if (n_steps > 0) {
    for (int v = 0; v < n_pl; ++v) issue_patch(m_begin, 0, v);
    while (iw_step < NSW && iw_step < n_steps) issue_next_weights();
    wait_weights(iw_step - 1);   // patch and tile 0 landed (NSW <= 4: never more than 3 later tiles)
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    read_step(0, x_lds, 0, 0);
  }

  // current K step: macro step index mi (of this block), tap = (tr, ts), ring stage
  int mi = 0, tap = 0, tr = 0, ts = 0, stage = 0;
  auto one_step = [&](int step, int slot) {
    // This wave's reads of the current step's operands (issued a step ago) and its copies of the
    // next weight tile are complete; after the barrier that holds for every wave: the next tile
    // (and, past a patch's last tap, the next patch) may be read, the current stage overwritten.
    wait_weights(iw_step - (step + 2));   // weight tiles issued after tile step+1
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    // Patch of the next (depth tap, channel chunk): a few copies per step on the early taps,
    // issued BEFORE this step's weight tile so that they are older than a tile that is
    // waited for before the patch is first read.
    if (mi + 1 < n_macro && tap * p.pls < n_pl) {
      const int v_end = (tap + 1) * p.pls < n_pl ? (tap + 1) * p.pls : n_pl;
      for (int v = tap * p.pls; v < v_end; ++v) issue_patch(m_begin + mi + 1, (mi + 1) & (p.xbufs - 1), v);
    }
    if (iw_step < n_steps) issue_next_weights();   // tile step+NSW into the stage just freed
    // operands of the next K step, then the MFMAs of this one
    ++tap;
    if (++ts == p.S) { ts = 0; ++tr; }
    if (tap == RS) { tap = 0; tr = 0; ++mi; }
    if (++stage == NSW) stage = 0;
    if (step + 1 < n_steps)
      read_step((unsigned)stage * WSTAGE, x_lds + (unsigned)(mi & (p.xbufs - 1)) * (unsigned)xbuf_bytes,
                tr * p.dh * p.Wp + ts * p.dw, slot ^ 1);
    mma_step(slot);
  };
  int step = 0;
  for (; step + 1 < n_steps; step += 2) {
    one_step(step, 0);
    one_step(step + 1, 1);
  }
  if (step < n_steps) one_step(step, 0);

  // ---- epilogue: Y[(n*K + i)*ODPQ + (od*OPQ + opq)] ---------------------------------------------
  out_t* const out = (out_t*)p.y;
  const int ODPQ = p.OD * OPQ;
  const bool full = bi0 + BI <= p.K && bj0 + BJ <= p.J && !p.atomic_out;
#pragma unroll
  for (int b = 0; b < TJ; ++b) {
    const int j = bj0 + (wj * TJ + b) * 32 + frag_row;
    const int jc = j < p.J ? j : p.J - 1;
    const int n = fast_div(jc, p.fd_odpq);
    const int64_t coff = (int64_t)n * p.K * ODPQ + (jc - n * ODPQ);
#pragma unroll
    for (int a = 0; a < TI; ++a) {
      const int i0 = bi0 + (wi * TI + a) * 32 + 4 * frag_half;
      out_t* const dst0 = out + (int64_t)i0 * ODPQ + coff;
      if (full) {
#pragma unroll
        for (int r = 0; r < 16; ++r) dst0[(int64_t)(8 * (r >> 2) + (r & 3)) * ODPQ] = acc[a][b][r];
      } else if (j < p.J) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int di = 8 * (r >> 2) + (r & 3);
          if (i0 + di < p.K) {
            if (p.atomic_out)
              atomicAdd(dst0 + (int64_t)di * ODPQ, acc[a][b][r]);
            else
              dst0[(int64_t)di * ODPQ] = acc[a][b][r];
          }
        }
      }
    }
  }
}

}  // namespace amos
