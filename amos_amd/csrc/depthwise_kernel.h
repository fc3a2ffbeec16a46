// Depthwise convolution (groups == input channels: every output channel reads ONE input channel)
// for gfx950.  There is nothing to reduce over but the window's taps, so the matrix cores have
// no work here: an implicit GEMM would fill one row of a 64-row tile.  The op moves bytes --
// input read once, output written once -- and runs on the vector ALUs: a lane computes four
// adjacent outputs of one to four output rows from the input rows in its registers and stores
// 16 bytes per row.
// (reference: benchmark/amos/mapping_depthwiseconv2d_tensorcore.py:7-48 states the op; the
// reference maps it onto Tensor Core fragments like any other convolution.)
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fast_div.h"
#include "igemm_kernel.h"

namespace amos {

struct DepthwiseParams {
  const char* x;     // [N][C][D][H][W]
  const char* w;     // [K][T][R][S], K = C * mult
  char* y;           // [N][K][OD][OP][OQ], fp32 / int32
  int N, C, D, H, W;
  int K, mult;
  int T, R, S;
  int OD, OP, OQ;
  int sd, sh, sw, pd, ph, pw, dd, dh, dw;
  int qgroups;       // ceil(OQ / 4): lanes per output row
  int pgroups;       // ceil(OP / rows per lane)
  unsigned items;    // N * K * OD * pgroups * qgroups, below 2^31
  int vec_store;     // OQ % 4 == 0 and y 16-byte aligned
  FastDiv fd_qg, fd_pg, fd_od, fd_k, fd_mult;
  EpiParams epi;
};

enum { DW_GENERIC = 0, DW_3x3_S1 = 1, DW_3x3_S2 = 2, DW_3x3_S1_SMALL = 3 };
// output rows per lane: the 3x3 kinds keep the input rows that output rows share in registers;
// four rows where that still leaves every SIMD several waves, two for smaller problems
constexpr int dw_rows_per_lane(int kind) {
  return kind == DW_3x3_S1 ? 4 : (kind == DW_3x3_S2 || kind == DW_3x3_S1_SMALL) ? 2 : 1;
}

template <int DT> struct DwTypes { typedef unsigned short in_t; typedef float acc_t; };
template <> struct DwTypes<DT_I8> { typedef signed char in_t; typedef int acc_t; };

template <int DT>
__device__ __forceinline__ typename DwTypes<DT>::acc_t dw_widen(typename DwTypes<DT>::in_t v) {
  if constexpr (DT == DT_F16) return (float)__builtin_bit_cast(_Float16, v);
  else if constexpr (DT == DT_BF16) return __builtin_bit_cast(float, (unsigned)v << 16);
  else return (int)v;
}

__device__ __forceinline__ int dw_clamp(int v, int hi) { return v < 0 ? 0 : v > hi ? hi : v; }
// all ones where ok, zero elsewhere -- as a value the compiler knows nothing about: a load that
// is ANDed with it stays an unconditional load (a select of "loaded value or zero" is turned
// back into a branch around the load, and then every load waits for the one before)
__device__ __forceinline__ unsigned dw_mask(bool ok) {
  unsigned m = ok ? 0xffffffffu : 0u;
  asm("" : "+v"(m));
  return m;
}

// KIND: DW_3x3_S1 / DW_3x3_S2 = R = S = 3, unit dilation, row and column stride 1 / 2 (the
// windows of a lane's outputs overlap: each input row is loaded once); DW_GENERIC = any.
// Loads are unconditional at clamped addresses and zeroed afterwards where the window hangs
// over the edge, so that the compiler can issue a lane's loads together.
template <int DT, int KIND>
__global__ __launch_bounds__(256) void amos_depthwise_conv(const DepthwiseParams p) {
  typedef typename DwTypes<DT>::in_t in_t;
  typedef typename DwTypes<DT>::acc_t acc_t;
  constexpr int PR = dw_rows_per_lane(KIND);
  const in_t* __restrict__ x = (const in_t*)p.x;
  const in_t* __restrict__ wt = (const in_t*)p.w;
  acc_t* __restrict__ y = (acc_t*)p.y;
  const unsigned step = gridDim.x * 256u;
  for (unsigned item = blockIdx.x * 256u + threadIdx.x; item < p.items; item += step) {
    int rest = fast_div((int)item, p.fd_qg);
    const int q0 = ((int)item - rest * p.qgroups) * 4;
    int nx = fast_div(rest, p.fd_pg);
    const int op0 = (rest - nx * p.pgroups) * PR;
    int od = 0;
    if (p.OD > 1) {          // (uniform: 2-D convolutions skip the division)
      rest = nx;
      nx = fast_div(rest, p.fd_od);
      od = rest - nx * p.OD;
    }
    const int n = fast_div(nx, p.fd_k);
    const int k = nx - n * p.K;
    // input plane n * C + k / mult: the output plane's own index where each channel has one output
    const int plane = p.mult == 1 ? nx : n * p.C + fast_div(k, p.fd_mult);
    const in_t* xp = x + (int64_t)plane * ((int64_t)p.D * p.H * p.W);
    const in_t* wp = wt + (int64_t)k * (p.T * p.R * p.S);
    acc_t acc[PR][4];
#pragma unroll
    for (int r = 0; r < PR; ++r)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[r][j] = 0;
    const int w0 = q0 * p.sw - p.pw, h0 = op0 * p.sh - p.ph, d0 = od * p.sd - p.pd;
    for (int t = 0; t < p.T; ++t) {
      const int d = d0 + t * p.dd;
      if ((unsigned)d >= (unsigned)p.D) continue;
      if constexpr (KIND != DW_GENERIC) {
        constexpr int ST = KIND == DW_3x3_S2 ? 2 : 1;
        constexpr int NV = 3 * ST + 3;            // input columns under four outputs
        constexpr int NH = (PR - 1) * ST + 3;     // input rows under PR output rows
        acc_t wv[9];
#pragma unroll
        for (int i = 0; i < 9; ++i) wv[i] = dw_widen<DT>(wp[t * 9 + i]);
        int col[NV];
        unsigned col_ok[NV];
#pragma unroll
        for (int j = 0; j < NV; ++j) {
          col_ok[j] = dw_mask((unsigned)(w0 + j) < (unsigned)p.W);
          col[j] = dw_clamp(w0 + j, p.W - 1);
        }
#pragma unroll
        for (int hr = 0; hr < NH; ++hr) {
          const int h = h0 + hr;
          const unsigned row_ok = dw_mask((unsigned)h < (unsigned)p.H);
          const in_t* row = xp + ((int64_t)d * p.H + dw_clamp(h, p.H - 1)) * p.W;
          acc_t v[NV];
#pragma unroll
          for (int j = 0; j < NV; ++j) {
            const unsigned raw = (unsigned)row[col[j]] & (row_ok & col_ok[j]);
            v[j] = dw_widen<DT>((in_t)raw);
          }
#pragma unroll
          for (int pr = 0; pr < PR; ++pr) {
            const int r = hr - pr * ST;          // the window row of output row pr this input row is
            if (r < 0 || r > 2) continue;
#pragma unroll
            for (int s = 0; s < 3; ++s)
#pragma unroll
              for (int j = 0; j < 4; ++j) acc[pr][j] += v[j * ST + s] * wv[r * 3 + s];
          }
        }
      } else {
        for (int r = 0; r < p.R; ++r) {
          const int h = h0 + r * p.dh;
          const unsigned row_ok = dw_mask((unsigned)h < (unsigned)p.H);
          const in_t* row = xp + ((int64_t)d * p.H + dw_clamp(h, p.H - 1)) * p.W;
          for (int s = 0; s < p.S; ++s) {
            const acc_t wv = dw_widen<DT>(wp[(t * p.R + r) * p.S + s]);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const int wi = w0 + j * p.sw + s * p.dw;
              const unsigned raw = (unsigned)row[dw_clamp(wi, p.W - 1)] &
                                   (row_ok & dw_mask((unsigned)wi < (unsigned)p.W));
              acc[0][j] += dw_widen<DT>((in_t)raw) * wv;
            }
          }
        }
      }
    }
#pragma unroll
    for (int pr = 0; pr < PR; ++pr) {
      if (op0 + pr >= p.OP) continue;
      // flat output index of (n, k, od, op0 + pr, q0)
      const int64_t o = ((int64_t)nx * p.OD * p.OP + (int64_t)od * p.OP + op0 + pr) * p.OQ + q0;
      if (p.epi.ptr) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (q0 + j < p.OQ) acc[pr][j] += epi_value<acc_t>(p.epi, o + j);
      }
      if (p.vec_store) {
        typedef acc_t vec4 __attribute__((ext_vector_type(4)));
        vec4 out = {acc[pr][0], acc[pr][1], acc[pr][2], acc[pr][3]};
        __builtin_nontemporal_store(out, (vec4*)(y + o));   // written once, not read again here
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (q0 + j < p.OQ) y[o + j] = acc[pr][j];
      }
    }
  }
}

// kind: DW_*; returns the instance's name, launches when run != 0 (defined in inst_depthwise.hip)
const char* depthwise_name(int dt, int kind);
void launch_depthwise(int dt, int kind, const DepthwiseParams& p, hipStream_t stream);

}  // namespace amos
