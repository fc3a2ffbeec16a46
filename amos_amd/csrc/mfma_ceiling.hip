// What the matrix cores of this chip sustain when nothing else limits them: a measurement kernel
// with the instruction mix of the 8192^3 fp16 product (256 workgroups x 4 waves, each wave the
// matrix-core instructions of a 128x128 wave tile x 512 K steps of 64 = 1.0995e12 flop per launch)
// and, optionally, the data movement a 256x256x64 tiling needs next to them -- global -> LDS
// copies (64 KB per K step and workgroup) and LDS fragment reads (32 x 16 bytes per lane and K
// step) -- with no barrier and no wait for a copy anywhere; a read's data is consumed (XORed into
// a running value) behind the next two (32x32x16) / four (16x16x32) matrix-core instructions, so a
// wave has one read in flight and waits for it only if LDS takes longer than those take to issue.  The operands of the matrix-core instructions never
// change: either small constants or random fp16 values read once from the caller's buffers, which
// is what decides the clock the chip holds (the switching activity of the multipliers).
//
// The figure is the "sustained peak" next to the published one in the benchmark's report (the
// reference divides by nothing: it reports seconds, python/tvm/auto_tensorize/search/measure.py:175-207).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

#include "amos_mi355x.h"
#include "mapper.h"

namespace amos {

typedef int cv4i __attribute__((ext_vector_type(4)));
typedef float cv4f __attribute__((ext_vector_type(4)));
typedef float cv16f __attribute__((ext_vector_type(16)));
typedef _Float16 cv8h __attribute__((ext_vector_type(8)));

struct CeilingParams {
  const char* a;   // operands: at least 256 * 256 * 128 bytes each; with copies an [8192][8192] fp16 matrix
  const char* b;
  float* sink;     // 256 floats that are never written (the stores exist so that the work is kept)
  int k_steps;     // K steps of 64 per workgroup
  int ld;          // row length of a and b in elements (copies)
};

#define AMOS_CEIL_GLOBAL(p) ((const __attribute__((address_space(1))) void*)(p))
#define AMOS_CEIL_LDS(p) ((__attribute__((address_space(3))) void*)(p))

// SHAPE 16: v_mfma_f32_16x16x32_f16 (128 per wave and K step); 32: v_mfma_f32_32x32x16_f16 (64).
// The accumulators are a 4x4 (16: 64 registers) / 2x4 (32: 128 registers) grid of tiles, every
// tile written once per eight rounds -- few enough registers that the compiler keeps every
// accumulator in place (with the product's full 128x128 wave tile it shuffles them between
// register files inside the loop, which is not what is to be measured).
template <int SHAPE, int DATA, int COPIES, int READS>
__global__ __launch_bounds__(256) void amos_mfma_ceiling_kernel(const CeilingParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  constexpr int TA = SHAPE == 16 ? 4 : 2, TB = 4;
  constexpr int ROUNDS = (SHAPE == 16 ? 128 : 64) / (TA * TB);   // per K step
  constexpr int NF = 8;   // operand fragments per side held in registers
  cv4i fa[NF], fb[NF];
#pragma unroll
  for (int i = 0; i < NF; ++i) {
    if (DATA) {
      const size_t at = ((size_t)(blockIdx.x * 256 + threadIdx.x) * NF + i) * 16;
      fa[i] = *(const cv4i*)(p.a + at);
      fb[i] = *(const cv4i*)(p.b + at);
    } else {
      fa[i] = cv4i{lane, i, 2, 3};
      fb[i] = cv4i{4, 5, lane, i};
    }
  }
  // the copies a workgroup of the 256x256 tile issues per K step: 64 blocks of 8 rows x 128 bytes,
  // 16 per wave; the workgroup's tile of the caller's matrices
  const int tile_i = blockIdx.x & 15, tile_j = blockIdx.x >> 4;
  const char* const abase = p.a + (int64_t)tile_i * 256 * p.ld * 2;
  const char* const bbase = p.b + (int64_t)tile_j * 256 * p.ld * 2;
  unsigned g_off[16];
#pragma unroll
  for (int u = 0; u < 16; ++u) {
    const int q = wave + 4 * u, row = (q & 31) * 8 + (lane >> 3);
    g_off[u] = (unsigned)row * (unsigned)(p.ld * 2) + (unsigned)(lane & 7) * 16;
  }
  cv4i seen = {0, 0, 0, 0};
  typedef typename std::conditional<SHAPE == 16, cv4f, cv16f>::type acc_t;
  acc_t acc[TA * TB];
#pragma unroll
  for (int i = 0; i < TA * TB; ++i)
#pragma unroll
    for (int r = 0; r < (SHAPE == 16 ? 4 : 16); ++r) acc[i][r] = 0;
  for (int kt = 0; kt < p.k_steps; ++kt) {
#pragma unroll
    for (int rd = 0; rd < ROUNDS; ++rd)
#pragma unroll
      for (int a = 0; a < TA; ++a)
#pragma unroll
        for (int b = 0; b < TB; ++b) {
          constexpr int PER = TA * TB;
          const int m = rd * PER + a * TB + b;   // 0 .. 127 (16) / 0 .. 63 (32): a constant once unrolled
          const cv8h x = __builtin_bit_cast(cv8h, fa[(rd * TA + a) % NF]), y = __builtin_bit_cast(cv8h, fb[(rd + b) % NF]);
          // (as assembly with the accumulator tied to its own registers: the builtin leaves the
          // compiler free to rotate the accumulators through other registers at the loop's back
          // edge, hundreds of moves per K step.  A tile is written again 15 instructions later,
          // long after the matrix core has delivered it.)
          if constexpr (SHAPE == 16)
            asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[a * TB + b]) : "v"(x), "v"(y));
          else
            asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc[a * TB + b]) : "v"(x), "v"(y));
          constexpr int CE = SHAPE == 16 ? 8 : 4, RE = SHAPE == 16 ? 4 : 2;   // sixteen copies, 32 reads per K step
          if (COPIES && m % CE == CE - 1) {
            const int u = m / CE, q = wave + 4 * u;
            const char* src = (q < 32 ? abase : bbase) + (int64_t)(kt & 127) * 128 + g_off[u];
            __builtin_amdgcn_global_load_lds(AMOS_CEIL_GLOBAL(src), AMOS_CEIL_LDS(smem + (kt & 1) * 65536 + q * 1024), 16, 0, 0);
          }
          if (READS && m % RE == RE - 1) {
            const cv4i v = *(const cv4i*)(smem + ((kt & 1) * 65536 + (m / RE) * 2048 + wave * 512 + lane * 16));
            seen.x ^= v.x; seen.y ^= v.w;
          }
        }
  }
  // (the last results are on their way for up to 16 passes: the compiler does not know that of
  // an assembly statement)
  asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  float sum = 0;
#pragma unroll
  for (int i = 0; i < TA * TB; ++i)
#pragma unroll
    for (int r = 0; r < (SHAPE == 16 ? 4 : 16); ++r) sum += acc[i][r];
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  // (never true for finite operands of this size; keeps the accumulators and the reads alive)
  if (sum == 12345.678f || seen.x == 0x7fffffff) p.sink[threadIdx.x] = sum + (float)seen.y;
}

typedef void (*CeilingFn)(const CeilingParams);
template <int SHAPE, int DATA>
static CeilingFn ceiling_pick(int copies, int reads) {
  if (copies && reads) return amos_mfma_ceiling_kernel<SHAPE, DATA, 1, 1>;
  if (copies) return amos_mfma_ceiling_kernel<SHAPE, DATA, 1, 0>;
  if (reads) return amos_mfma_ceiling_kernel<SHAPE, DATA, 0, 1>;
  return amos_mfma_ceiling_kernel<SHAPE, DATA, 0, 0>;
}

}  // namespace amos

using namespace amos;

extern "C" int amos_mfma_ceiling(int shape, int random_operands, int copies, int reads, const void* a, const void* b,
                                 size_t operand_bytes, void* sink, int launches, void* stream_v, double* out_seconds,
                                 double* out_flop) {
  if ((shape != 16 && shape != 32) || !a || !b || !sink || launches < 1 || !out_seconds || !out_flop)
    return set_error(AMOS_ERR_BAD_ARG, "amos_mfma_ceiling: shape 16 or 32, non-null buffers, launches >= 1");
  const size_t need = copies ? (size_t)8192 * 8192 * 2 : (size_t)256 * 256 * 128;
  if (operand_bytes < need || ((uintptr_t)a & 15) || ((uintptr_t)b & 15))
    return set_error(AMOS_ERR_BAD_ARG, "amos_mfma_ceiling: operands of %zu bytes each, 16-byte aligned", need);
  CeilingFn fn = shape == 16 ? (random_operands ? ceiling_pick<16, 1>(copies, reads) : ceiling_pick<16, 0>(copies, reads))
                             : (random_operands ? ceiling_pick<32, 1>(copies, reads) : ceiling_pick<32, 0>(copies, reads));
  const size_t lds = (copies || reads) ? 131072 : 0;
  hipError_t e = hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  if (e != hipSuccess) return set_error(AMOS_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  hipStream_t stream = (hipStream_t)stream_v;
  CeilingParams p = {(const char*)a, (const char*)b, (float*)sink, 512, 8192};
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess)
    return set_error(AMOS_ERR_HIP, "hipEventCreate failed");
  hipLaunchKernelGGL(fn, dim3(256), dim3(256), lds, stream, p);   // warm-up
  (void)hipEventRecord(e0, stream);
  for (int i = 0; i < launches; ++i) hipLaunchKernelGGL(fn, dim3(256), dim3(256), lds, stream, p);
  (void)hipEventRecord(e1, stream);
  e = hipEventSynchronize(e1);
  float ms = 0;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (e == hipSuccess) e = hipGetLastError();
  if (e != hipSuccess) return set_error(AMOS_ERR_HIP, "amos_mfma_ceiling: %s", hipGetErrorString(e));
  *out_seconds = (double)ms * 1e-3 / launches;
  *out_flop = 256.0 * 4 * 512 * (2.0 * 128 * 128 * 64);
  return 0;
}
