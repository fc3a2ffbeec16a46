// GEMM with one skinny side (a few rows: a GEMV, a dense layer on a small batch) for gfx950.
//
// Out[r][m] = sum_k Big[r][k] * Small[m][k], both operands K-contiguous.  With so few rows on one
// side there is one pass over the big operand and almost no reuse: the op moves bytes, and an MFMA
// tile would be 1/4 .. 1/64 full.  It runs on the vector ALUs instead: the small operand sits in
// LDS (zero-padded to MSP rows), sixteen lanes share a row of the big operand and stride over K in
// 16-byte chunks (a wave covers four rows, a workgroup sixteen), every chunk is multiplied with
// the MSP chunks of the small operand (packed dot products, fp32 / int32 accumulation), and the
// sixteen partial sums of a row meet in a four-step butterfly.
//
// Role in the reference: the GEMV of benchmark/amos/mapping_gemv_tensorcore.py:7-16 and the dense
// layers of its networks at small batch, which it pads onto Tensor Core fragments.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "igemm_kernel.h"
#include "mapper.h"

namespace amos {

struct SkinnyParams {
  const char* big;       // [NB][ld_big] elements
  const char* small;     // [MS][ld_small]
  char* out;             // fp32 / int32: element (r, m) at r * out_s_big + m * out_s_small
  int NB, MS, K;         // K a multiple of 16 bytes of elements
  int64_t ld_big, ld_small;
  int64_t out_s_big, out_s_small;
  EpiParams epi;         // fused tail: D(r, m) at r * epi_s_big + m * epi_s_small
  int64_t epi_s_big, epi_s_small;
};

template <int DT>
__device__ __forceinline__ typename Mfma<DT>::out_t skinny_dot(v4i a, v4i b, typename Mfma<DT>::out_t c) {
  if constexpr (DT == DT_I8) {
#pragma unroll
    for (int i = 0; i < 4; ++i) c = __builtin_amdgcn_sdot4(a[i], b[i], c, false);
    return c;
  } else if constexpr (DT == DT_F16) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int ai = a[i], bi = b[i];   // (a bit cast straight from a vector element reads element 0)
      c = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, ai), __builtin_bit_cast(h2, bi), c, false);
    }
    return c;
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const unsigned ua = (unsigned)a[i], ub = (unsigned)b[i];
      c += __builtin_bit_cast(float, ua << 16) * __builtin_bit_cast(float, ub << 16);
      c += __builtin_bit_cast(float, ua & 0xffff0000u) * __builtin_bit_cast(float, ub & 0xffff0000u);
    }
    return c;
  }
}

// MSP = the small operand's rows rounded up to 1, 2, 4 or 8; dynamic LDS = MSP * K * esize
template <int DT, int MSP>
__global__ __launch_bounds__(256) void amos_skinny_gemm(const SkinnyParams p) {
  typedef Mfma<DT> MM;
  typedef typename MM::out_t out_t;
  constexpr int ES = MM::ES;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int t = threadIdx.x;
  const int chunks = p.K * ES / 16;          // 16-byte chunks per row
  // ---- the small operand, rows past MS as zeros
  for (int i = t; i < MSP * chunks; i += 256) {
    const int m = i / chunks, c = i - m * chunks;
    v4i v = {0, 0, 0, 0};
    if (m < p.MS) v = *(const v4i*)(p.small + ((int64_t)m * p.ld_small) * ES + (int64_t)c * 16);
    *(v4i*)(smem + (int64_t)i * 16) = v;
  }
  __syncthreads();
  const int lane = t & 63, wave = t >> 6;
  const int kl = lane & 15;
  const int r = (blockIdx.x * 4 + wave) * 4 + (lane >> 4);
  const int rc = r < p.NB ? r : p.NB - 1;    // (rows past the end repeat the last one and are not stored)
  const char* row = p.big + (int64_t)rc * p.ld_big * ES;
  out_t acc[MSP];
#pragma unroll
  for (int m = 0; m < MSP; ++m) acc[m] = 0;
  // two chunks of the big operand in flight per lane
  int c = kl;
  for (; c + 16 < chunks; c += 32) {
    const v4i x0 = *(const v4i*)(row + (int64_t)c * 16);
    const v4i x1 = *(const v4i*)(row + (int64_t)(c + 16) * 16);
#pragma unroll
    for (int m = 0; m < MSP; ++m) {
      acc[m] = skinny_dot<DT>(x0, *(const v4i*)(smem + ((int64_t)m * chunks + c) * 16), acc[m]);
      acc[m] = skinny_dot<DT>(x1, *(const v4i*)(smem + ((int64_t)m * chunks + c + 16) * 16), acc[m]);
    }
  }
  if (c < chunks) {
    const v4i x0 = *(const v4i*)(row + (int64_t)c * 16);
#pragma unroll
    for (int m = 0; m < MSP; ++m)
      acc[m] = skinny_dot<DT>(x0, *(const v4i*)(smem + ((int64_t)m * chunks + c) * 16), acc[m]);
  }
  // ---- the sixteen lanes of a row add up: afterwards every one of them holds every sum
#pragma unroll
  for (int step = 1; step < 16; step <<= 1)
#pragma unroll
    for (int m = 0; m < MSP; ++m) acc[m] += __shfl_xor(acc[m], step, 64);
  // lane kl stores output m = kl (MSP <= 16 lanes of a row)
  out_t mine = 0;
#pragma unroll
  for (int m = 0; m < MSP; ++m) mine = kl == m ? acc[m] : mine;
  if (r < p.NB && kl < p.MS) {
    if (p.epi.dt != EPI_NONE) mine += epi_value<out_t>(p.epi, (int64_t)r * p.epi_s_big + (int64_t)kl * p.epi_s_small);
    ((out_t*)p.out)[(int64_t)r * p.out_s_big + (int64_t)kl * p.out_s_small] = mine;
  }
}

const char* skinny_gemm_name(int dt);
hipError_t launch_skinny_gemm(int dt, const SkinnyParams& p, hipStream_t stream);
// LDS bytes the launch needs; the route exists where they fit
inline int64_t skinny_gemm_lds(int ms, int64_t K, int es) {
  int msp = 1;
  while (msp < ms) msp <<= 1;
  return (int64_t)msp * K * es;
}

}  // namespace amos
