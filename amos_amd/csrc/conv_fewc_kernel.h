// 2-D convolution on few input channels (an RGB stem: C * esize <= 16 bytes) for gfx950.
//
// The patch-staged kernel wants whole 128-byte chunks of channels and the register-staged one
// gathers im2col elements one by one.  Here a PIXEL is the 16-byte unit: the activations are
// relaid once to [N][H][W][16 bytes] (channels zero-padded), and the reduction runs over
// (tap, padded channel), so that the 16 bytes of K a lane feeds to v_mfma are exactly one pixel
// of one tap.  A workgroup (8 waves) computes 64 output channels x 256 output pixels of one image:
// it loads its 64 x taps weight pixels and the zero-padded input patch under its output pixels
// into LDS once -- nothing else comes from memory -- and every K sub-step (two taps) is two
// weight fragments, one gathered patch fragment and two MFMAs per wave.  Most of the MFMA work
// multiplies padding (3 of 8 channels are real); the kernel is bound by its loads and stores.
//
// In the reference's terms this is the mapping i<-{k}, j<-{n,p,q}, rk<-{rr,rs,rc} with rc padded
// to the intrinsic's K (python/tvm/auto_tensorize/hw_abstraction/cuda/wmma_base.py handles a
// short reduction by zero-padding the fragment the same way).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fast_div.h"
#include "gemm_tn_kernel.h"
#include "igemm_kernel.h"

namespace amos {

struct ConvFewcParams {
  const char* x;      // NCHW activations
  const char* w;      // KCRS weights
  char* xt;           // workspace: [N][H][W] pixels of 16 bytes, then one zero pixel
  char* wp;           // workspace: [k_tiles * 64][taps_p] pixels of 16 bytes, zero-filled
  char* y;            // NKPQ, fp32 / int32
  int N, C, H, W, K, R, S;
  int OP, OQ, sh, sw, ph, pw, dh, dw;
  int taps, taps_p;   // R * S, and rounded up to even
  int Wp;             // patch row in pixels: W + 2 * pw
  int rows_max;       // patch rows a workgroup may need
  int tiles_j;        // pixel tiles (256) per image
  int k_tiles;        // ceil(K / 64)
  int prep_x_blocks, prep_w_blocks;
  int patch_off, zero_off, tab_off;   // LDS bytes: patch buffers, the zero pixel, the tap table
  int patch_bytes, nbuf;              // bytes of one patch buffer (a multiple of 1 KB); 1 or 2 of them
  int grid_x;                         // workgroups per tile of output channels
  FastDiv fd_oq, fd_wp, fd_hw, fd_taps_p, fd_s, fd_tiles_j;
  EpiParams epi;
};

// launch 1: xt[n][h][w][c16] = x[n][c][h][w]; wp[k][tap][c16] = w[k][c][tap]; zeros elsewhere
template <typename T>
__global__ __launch_bounds__(256) void amos_conv_fewc_prepare(const ConvFewcParams p) {
  constexpr int CE = 16 / (int)sizeof(T);
  const int t = threadIdx.x;
  int b = blockIdx.x;
  const int HW = p.H * p.W;
  if (b < p.prep_x_blocks) {   // four pixels per thread, 256 apart: their loads overlap
    const int64_t total = (int64_t)p.N * HW;
    if (b == 0 && t == 0) *(uint4*)(p.xt + total * 16) = uint4{0, 0, 0, 0};   // the zero pixel behind the last image
    T v[4][CE];
    int64_t idx[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      idx[u] = (int64_t)b * 1024 + t + 256 * u;
      const int ic = (int)(idx[u] < total ? idx[u] : total - 1);
      const int n = fast_div(ic, p.fd_hw);
      const T* src = (const T*)p.x + (int64_t)n * p.C * HW + (ic - n * HW);
#pragma unroll
      for (int c = 0; c < CE; ++c) v[u][c] = c < p.C ? src[(int64_t)c * HW] : (T)0;   // (uniform)
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (idx[u] < total) *(uint4*)(p.xt + idx[u] * 16) = *(const uint4*)v[u];
    return;
  }
  b -= p.prep_x_blocks;
  const int total = p.k_tiles * 64 * p.taps_p;
  const int idx = b * 256 + t;
  if (idx >= total) return;
  const int k = fast_div(idx, p.fd_taps_p);
  const int tap = idx - k * p.taps_p;
  T v[CE];
#pragma unroll
  for (int c = 0; c < CE; ++c)
    v[c] = (k < p.K && tap < p.taps && c < p.C) ? ((const T*)p.w)[((int64_t)k * p.C + c) * p.taps + tap] : (T)0;
  *(uint4*)(p.wp + (int64_t)idx * 16) = *(const uint4*)v;
}

// launch 2: grid (workgroups per tile of output channels, k_tiles), 512 threads, dynamic LDS =
// tab_off + 4 * taps_p.  A workgroup keeps its weights and walks pixel tiles item = blockIdx.x,
// + gridDim.x, ... (item = image * tiles_j + tile); with two patch buffers (nbuf == 2) the next
// tile's patch is in flight while this one is computed.
template <int DT>
__global__ __launch_bounds__(512) void amos_conv_fewc(const ConvFewcParams p) {
  typedef Mfma<DT> MM;
  typedef typename MM::acc_t acc_t;
  typedef typename MM::out_t out_t;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int k0 = blockIdx.y * 64;
  const int OPQ = p.OP * p.OQ;
  const int items = p.tiles_j * p.N;

  // Both operands go global -> LDS directly (a wave instruction fills 1 KB of LDS linearly, each
  // lane fetching the 16 bytes that belong at its position): no staging registers, every copy
  // of the workgroup in flight at once.
  // ---- weights of this tile of output channels: a linear copy of 64 * taps_p pixels
  {
    const char* src = p.wp + (int64_t)k0 * p.taps_p * 16 + lane * 16;
    const int chunks = p.taps_p;                      // 64 * taps_p * 16 bytes / 1 KB
    for (int c = wave; c < chunks; c += 8)
      __builtin_amdgcn_global_load_lds(AMOS_GLOBAL_PTR(src + c * 1024), AMOS_LDS_PTR(smem + c * 1024), 16, 0, 0);
  }
  // ---- a tile's patch: every slot written; slots outside the image fetch the zero pixel that
  // the relayout launch left behind the last image (a buffer is a whole number of 1 KB chunks:
  // the lanes past the last slot fetch that pixel too)
  const char* const zero = p.xt + (int64_t)p.N * p.H * p.W * 16;
  auto issue_patch = [&](int item, int buf) {
    const int n = fast_div(item, p.fd_tiles_j);
    const int j0 = (item - n * p.tiles_j) * 256;
    const int j_last = (j0 + 255 < OPQ ? j0 + 255 : OPQ - 1);
    const int p_lo = fast_div(j0, p.fd_oq), p_hi = fast_div(j_last, p.fd_oq);
    const int ih_lo = p_lo * p.sh - p.ph;
    const int rows = (p_hi - p_lo) * p.sh + (p.R - 1) * p.dh + 1;   // <= rows_max (host)
    const char* img = p.xt + (int64_t)n * p.H * p.W * 16;
    const int total = rows * p.Wp;
    const int chunks = (total + 63) >> 6;
    char* dst = smem + p.patch_off + buf * p.patch_bytes;
    for (int c = wave; c < chunks; c += 8) {
      const int slot = c * 64 + lane;
      const int r = fast_div(slot, p.fd_wp);
      const int ih = ih_lo + r, iw = slot - r * p.Wp - p.pw;
      const bool ok = slot < total && (unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W;
      const char* src = ok ? img + (int64_t)(ih * p.W + iw) * 16 : zero;
      __builtin_amdgcn_global_load_lds(AMOS_GLOBAL_PTR(src), AMOS_LDS_PTR(dst + c * 1024), 16, 0, 0);
    }
  };
  int item = blockIdx.x;
  issue_patch(item, 0);
  if (t == 0) *(uint4*)(smem + p.zero_off) = uint4{0, 0, 0, 0};

  const int col = lane & 31, half = lane >> 5;
  const int steps = p.taps_p >> 1;
  const int a_row = col * p.taps_p, a_row1 = (32 + col) * p.taps_p;
  out_t* const out = (out_t*)p.y;
  int buf = 0;
  bool counted = false;   // the previous tile ended with exactly 32 store instructions per wave
  for (; item < items; item += gridDim.x) {
    // This wave's copies are done; then everybody's are, and everybody is past the previous
    // tile's reads of the other buffer.  Memory operations complete in order and the previous
    // tile's stores were issued after this tile's copies: where their number is known they may
    // stay in flight and drain under this tile's MFMAs.
    // (the barrier as an instruction: __syncthreads() is also a fence that drains every store)
    if (counted) asm volatile("s_waitcnt vmcnt(32) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    const int next = item + gridDim.x;
    if (p.nbuf == 2 && next < items) issue_patch(next, buf ^ 1);

    // ---- this lane's output pixel and its window's first slot
    const int n = fast_div(item, p.fd_tiles_j);
    const int j0 = (item - n * p.tiles_j) * 256;
    const int p_lo = fast_div(j0, p.fd_oq);
    const int j = j0 + wave * 32 + col;
    const int jc = j < OPQ ? j : OPQ - 1;
    const int pp = fast_div(jc, p.fd_oq), qq = jc - pp * p.OQ;
    const int slot0 = (pp - p_lo) * p.sh * p.Wp + qq * p.sw;
    const char* const patch = smem + p.patch_off + buf * p.patch_bytes;

    acc_t acc[2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][r] = 0;

    // Fragments of sub-step ks + 1 are read while the MFMAs of sub-step ks issue (two register
    // sets, the loop unrolled by two).  This lane's tap 2*ks + half advances by two per sub-step:
    // its window coordinates follow with a carry instead of a division or a table in LDS.
    int tr = 0, ts = half;                 // (row, column) of the lane's tap in the window
    if (ts >= p.S) { ts -= p.S; ++tr; }
    int tap = half;
    auto read_frags = [&](v4i& b, v4i& x0, v4i& x1) {
      const int off = tr * p.dh * p.Wp + ts * p.dw;
      b = *(const v4i*)(tap < p.taps ? patch + (slot0 + off) * 16 : smem + p.zero_off);
      x0 = *(const v4i*)(smem + (a_row + tap) * 16);
      x1 = *(const v4i*)(smem + (a_row1 + tap) * 16);
      tap += 2;
      ts += 2;               // (two steps of the carry cover every S >= 1)
      int over = ts >= p.S;
      ts -= over ? p.S : 0; tr += over;
      over = ts >= p.S;
      ts -= over ? p.S : 0; tr += over;
    };
    v4i b0, x00, x01, b1, x10, x11;
    read_frags(b0, x00, x01);
    int ks = 0;
    for (; ks + 2 < steps; ks += 2) {
      read_frags(b1, x10, x11);
      acc[0] = MM::run(x00, b0, acc[0]);
      acc[1] = MM::run(x01, b0, acc[1]);
      read_frags(b0, x00, x01);
      acc[0] = MM::run(x10, b1, acc[0]);
      acc[1] = MM::run(x11, b1, acc[1]);
    }
    if (steps - ks == 2) {
      read_frags(b1, x10, x11);
      acc[0] = MM::run(x00, b0, acc[0]);
      acc[1] = MM::run(x01, b0, acc[1]);
      acc[0] = MM::run(x10, b1, acc[0]);
      acc[1] = MM::run(x11, b1, acc[1]);
    } else {
      acc[0] = MM::run(x00, b0, acc[0]);
      acc[1] = MM::run(x01, b0, acc[1]);
    }

    // ---- store: register r of a 32x32 tile is row 8*(r/4) + 4*half + r%4, column col
    // (uniform) every pixel and output channel of the tile exists, nothing to add: 32 plain stores
    const bool full = j0 + 255 < OPQ && k0 + 64 <= p.K && p.epi.dt == EPI_NONE && p.nbuf == 2;
    if (full) {
      out_t* const o = out + (int64_t)n * p.K * OPQ + (int64_t)(k0 + 4 * half) * OPQ + j;
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[(int64_t)(a * 32 + 8 * (r >> 2) + (r & 3)) * OPQ] = acc[a][r];
    } else if (j < OPQ) {
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        const int i0 = k0 + a * 32 + 4 * half;
        const int64_t on = (int64_t)n * p.K * OPQ + j;      // (image, pixel); row i adds i * OPQ
        if (p.epi.dt != EPI_NONE) {   // all sixteen loads in flight before the first addition
          out_t dv[16];
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int di = 8 * (r >> 2) + (r & 3);
            const int ic = i0 + di < p.K ? i0 + di : p.K - 1;   // (rows past K are not stored)
            dv[r] = epi_value<out_t>(p.epi, on + (int64_t)ic * OPQ);
          }
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[a][r] += dv[r];
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int di = 8 * (r >> 2) + (r & 3);
          if (i0 + di < p.K) out[on + (int64_t)(i0 + di) * OPQ] = acc[a][r];
        }
      }
    }
    counted = full;
    if (p.nbuf == 2) {
      buf ^= 1;
    } else if (next < items) {   // one buffer: refill it once everybody has read it
      __syncthreads();
      issue_patch(next, 0);
    }
  }
  // (a copy issued for a tile beyond the last one does not exist: `next < items` guards them)
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

const char* conv_fewc_name(int dt);
// sets the kernel's LDS limit on first use; returns hipSuccess or the error
hipError_t launch_conv_fewc(int dt, const ConvFewcParams& p, size_t lds, hipStream_t stream);

}  // namespace amos
