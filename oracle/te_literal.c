/*
 * TEST INFRASTRUCTURE -- CPU restatement of what the reference executes when a
 * TE GEMM / batched GEMM / conv compute is built with
 *     tvm.build(te.create_schedule(op), args, "llvm")
 * (reference: tests/python/auto_tensorize/test_compute_transform_gemm.py:121-128).
 * The reference's TVM cannot be built here (empty 3rdparty submodules, no LLVM
 * development tree), so this file restates its semantics as plain loop nests.
 * Nothing shipped links against it; tests, the smoke check and the benchmark's
 * CPU-baseline leg use it as the checker / the timed CPU path.
 *
 * Semantics followed (mode AMOS_ORACLE_TE_LITERAL):
 *   - the multiply happens in the INPUT dtype: fp16*fp16 rounded to fp16
 *     (reference: src/tir/op/op.cc:101-102,314-319 -- same dtype, no promotion;
 *      src/target/llvm/codegen_llvm.cc:899-924 -- FMul on half), bf16*bf16 rounded
 *     to bf16, int8*int8 wrapping to int8;
 *   - then the cast to the output dtype (fpext / sext, codegen_llvm.cc:593-625);
 *   - then a sequential += from 0 in declared reduce-axis order, rc outermost
 *     (reference: src/te/operation/compute_op.cc:293-329);
 *   - conv: the zero-padded input is a separate, materialised tensor
 *     (reference: benchmark/amos/mapping_conv2d_tensorcore.py:16-24), single
 *     thread, every stage at root.
 * Mode AMOS_ORACLE_EXACT keeps the product exact before accumulating (fp32
 * product of two halves is exact; int8 operands are sign-extended first, the
 * spelling  a.astype("int32") * b.astype("int32")  of
 * tutorials/auto_tensorize/mapping_ops/explore_mapping_conv2d_u8s8s32_avx512.py:44-45);
 * this is what a matrix core computes and, for int8, the bit-exact target.
 *
 * Parity pins: tests/test_oracle.py checks every function here against numpy /
 * torch-CPU closed forms (exact integer arithmetic, fp64 matmul / conv with a
 * rounding bound, all-ones inputs counting in-bounds taps, one-hot operands) and
 * the wrap-around mode against  int32(int8(a*b))  by brute force.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

enum { ORACLE_F16 = 0, ORACLE_BF16 = 1, ORACLE_I8 = 2 };
enum { AMOS_ORACLE_TE_LITERAL = 0, AMOS_ORACLE_EXACT = 1 };

/* ---- scalar conversions ------------------------------------------------------- */
static inline float bits_to_float(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline uint32_t float_to_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}

static float half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0) {
    if (man == 0) return bits_to_float(sign);
    /* subnormal: man * 2^-24 */
    float f = (float)man * (1.0f / 16777216.0f);
    return bits_to_float(float_to_bits(f) | sign);
  }
  if (exp == 31) return bits_to_float(sign | 0x7f800000u | (man << 13));
  return bits_to_float(sign | ((exp + 112u) << 23) | (man << 13));
}

/* round-to-nearest-even float -> half, the rounding FMul on half performs */
static uint16_t float_to_half(float f) {
  uint32_t x = float_to_bits(f);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) { /* inf / nan */
    return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? 0x200u : 0u));
  }
  if (ax >= 0x477ff000u) { /* >= 65520 rounds to inf */
    return (uint16_t)(sign | 0x7c00u);
  }
  if (ax < 0x38800000u) { /* below the smallest normal half: subnormal or zero */
    if (ax < 0x33000000u) return (uint16_t)sign; /* < 2^-25 rounds to 0 */
    uint32_t e = ax >> 23;                        /* biased fp32 exponent */
    uint32_t man = (ax & 0x7fffffu) | 0x800000u;  /* 24-bit significand   */
    uint32_t shift = 126u - e;                    /* 14..24               */
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1u);
    if (rem > halfway || (rem == halfway && (q & 1u))) q++;
    return (uint16_t)(sign | q);
  }
  uint32_t man = ax & 0x7fffffu;
  uint32_t e = (ax >> 23) - 112u;
  uint32_t h = (e << 10) | (man >> 13);
  uint32_t rem = man & 0x1fffu;
  if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
  return (uint16_t)(sign | h);
}

static inline float bf16_to_float(uint16_t b) { return bits_to_float((uint32_t)b << 16); }
static uint16_t float_to_bf16(float f) {
  uint32_t x = float_to_bits(f);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
  uint32_t lsb = (x >> 16) & 1u;
  x += 0x7fffu + lsb;
  return (uint16_t)(x >> 16);
}

/* exported for the tests that pin the conversions against numpy */
float oracle_half_to_float(uint16_t h) { return half_to_float(h); }
uint16_t oracle_float_to_half(float f) { return float_to_half(f); }
float oracle_bf16_to_float(uint16_t h) { return bf16_to_float(h); }
uint16_t oracle_float_to_bf16(float f) { return float_to_bf16(f); }

/* one multiply, as the llvm build performs it, widened to the accumulator type */
static inline float mul_f(int dtype, int mode, uint16_t a, uint16_t b) {
  if (dtype == ORACLE_F16) {
    float p = half_to_float(a) * half_to_float(b); /* exact in fp32 */
    return mode == AMOS_ORACLE_EXACT ? p : half_to_float(float_to_half(p));
  }
  float p = bf16_to_float(a) * bf16_to_float(b); /* exact in fp32 */
  return mode == AMOS_ORACLE_EXACT ? p : bf16_to_float(float_to_bf16(p));
}
static inline int32_t mul_i(int mode, int8_t a, int8_t b) {
  int32_t p = (int32_t)a * (int32_t)b;
  return mode == AMOS_ORACLE_EXACT ? p : (int32_t)(int8_t)(uint8_t)(p & 0xff);
}

static int set_threads(int threads) {
#ifdef _OPENMP
  if (threads < 1) threads = 1;
  omp_set_num_threads(threads);
  return threads;
#else
  (void)threads;
  return 1;
#endif
}
int oracle_max_threads(void) {
#ifdef _OPENMP
  return omp_get_num_procs();
#else
  return 1;
#endif
}

/*
 * C[m,n] = sum_k A(m,k) * B(k,n) for rows m in [m_begin, m_end).
 * trans_a = 0: A[m*lda + k], 1: A[k*lda + m];  trans_b = 0: B[k*ldb + n], 1: B[n*ldb + k].
 * (reference compute: benchmark/amos/mapping_gemm_tensorcore.py:7-15; transposed
 *  spellings: python/tvm/tensor_graph/nn/functional.py:1662-1722)
 * Returns 0, or -1 on a bad argument.
 */
int oracle_gemm(int dtype, int mode, int64_t M, int64_t N, int64_t K, int trans_a, int trans_b,
                const void* A, int64_t lda, const void* B, int64_t ldb, void* C, int64_t ldc,
                int64_t m_begin, int64_t m_end, int threads) {
  if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0 || m_begin < 0 || m_end > M) return -1;
  set_threads(threads);
  const int64_t sa_m = trans_a ? 1 : lda, sa_k = trans_a ? lda : 1;
  const int64_t sb_k = trans_b ? 1 : ldb, sb_n = trans_b ? ldb : 1;
  if (dtype == ORACLE_I8) {
    const int8_t* a = (const int8_t*)A;
    const int8_t* b = (const int8_t*)B;
    int32_t* c = (int32_t*)C;
#pragma omp parallel for schedule(static)
    for (int64_t m = m_begin; m < m_end; ++m)
      for (int64_t n = 0; n < N; ++n) {
        int32_t acc = 0;
        for (int64_t k = 0; k < K; ++k) acc += mul_i(mode, a[m * sa_m + k * sa_k], b[k * sb_k + n * sb_n]);
        c[m * ldc + n] = acc;
      }
    return 0;
  }
  if (dtype != ORACLE_F16 && dtype != ORACLE_BF16) return -1;
  const uint16_t* a = (const uint16_t*)A;
  const uint16_t* b = (const uint16_t*)B;
  float* c = (float*)C;
#pragma omp parallel for schedule(static)
  for (int64_t m = m_begin; m < m_end; ++m)
    for (int64_t n = 0; n < N; ++n) {
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) acc += mul_f(dtype, mode, a[m * sa_m + k * sa_k], b[k * sb_k + n * sb_n]);
      c[m * ldc + n] = acc;
    }
  return 0;
}

/* batch of GEMMs, batches [b_begin, b_end); operand x of batch b starts at x + b*stride_x
 * (reference: python/tvm/tensor_graph/nn/functional.py:1725-1793) */
int oracle_bgemm(int dtype, int mode, int64_t batch, int64_t M, int64_t N, int64_t K, int trans_a,
                 int trans_b, const void* A, int64_t lda, int64_t stride_a, const void* B,
                 int64_t ldb, int64_t stride_b, void* C, int64_t ldc, int64_t stride_c,
                 int64_t b_begin, int64_t b_end, int threads) {
  if (batch <= 0 || b_begin < 0 || b_end > batch) return -1;
  const int es = dtype == ORACLE_I8 ? 1 : 2;
  for (int64_t b = b_begin; b < b_end; ++b) {
    int rc = oracle_gemm(dtype, mode, M, N, K, trans_a, trans_b, (const char*)A + b * stride_a * es,
                         lda, (const char*)B + b * stride_b * es, ldb, (char*)C + b * stride_c * 4,
                         ldc, 0, M, threads);
    if (rc) return rc;
  }
  return 0;
}

static int64_t out_extent(int64_t in, int64_t pad, int64_t dil, int64_t k, int64_t stride) {
  int64_t eff = (k - 1) * dil + 1;
  if (in + 2 * pad < eff) return 0;
  return (in + 2 * pad - eff) / stride + 1;
}

/*
 * NCDHW convolution for images n in [n_begin, n_end) (conv2d: D = T = 1, sd = dd = 1, pd = 0).
 *   Pad[n,c,d,h,w] = in-range ? X[n,c,d-pd,h-ph,w-pw] : 0            (materialised)
 *   Y[n,k,od,op,oq] = sum_{rc,rd,rr,rs} Pad[n,rc,od*sd+rd*dd,op*sh+rr*dh,oq*sw+rs*dw] * Wt[k,rc,rd,rr,rs]
 * (reference computes: benchmark/amos/mapping_conv2d_tensorcore.py:7-42,
 *  benchmark/amos/mapping_conv3d_tensorcore.py:7-55)
 */
int oracle_conv(int dtype, int mode, int64_t N, int64_t C, int64_t D, int64_t H, int64_t W,
                int64_t K, int64_t T, int64_t R, int64_t S, int64_t sd, int64_t sh, int64_t sw,
                int64_t pd, int64_t ph, int64_t pw, int64_t dd, int64_t dh, int64_t dw,
                const void* X, const void* Wt, void* Y, int64_t n_begin, int64_t n_end,
                int threads) {
  if (!X || !Wt || !Y || N <= 0 || C <= 0 || D <= 0 || H <= 0 || W <= 0 || K <= 0 || T <= 0 ||
      R <= 0 || S <= 0 || sd <= 0 || sh <= 0 || sw <= 0 || dd <= 0 || dh <= 0 || dw <= 0 ||
      pd < 0 || ph < 0 || pw < 0 || n_begin < 0 || n_end > N)
    return -1;
  const int64_t OD = out_extent(D, pd, dd, T, sd), OP = out_extent(H, ph, dh, R, sh),
                OQ = out_extent(W, pw, dw, S, sw);
  if (OD <= 0 || OP <= 0 || OQ <= 0) return -1;
  set_threads(threads);
  const int64_t PD = D + 2 * pd, PH = H + 2 * ph, PW = W + 2 * pw;
  const int es = dtype == ORACLE_I8 ? 1 : 2;
  const int64_t nimg = n_end - n_begin;
  if (nimg <= 0) return 0;
  /* the Pad stage, materialised for the images of this slab */
  char* pad = (char*)calloc((size_t)(nimg * C * PD * PH * PW), (size_t)es);
  if (!pad) return -2;
  for (int64_t n = 0; n < nimg; ++n)
    for (int64_t c = 0; c < C; ++c)
      for (int64_t d = 0; d < D; ++d)
        for (int64_t h = 0; h < H; ++h) {
          const char* src = (const char*)X + ((((n + n_begin) * C + c) * D + d) * H + h) * W * es;
          char* dst = pad + ((((n * C + c) * PD + d + pd) * PH + h + ph) * PW + pw) * es;
          memcpy(dst, src, (size_t)(W * es));
        }
#pragma omp parallel for schedule(static) collapse(2)
  for (int64_t n = 0; n < nimg; ++n)
    for (int64_t k = 0; k < K; ++k)
      for (int64_t od = 0; od < OD; ++od)
        for (int64_t op = 0; op < OP; ++op)
          for (int64_t oq = 0; oq < OQ; ++oq) {
            const int64_t yidx = ((((n + n_begin) * K + k) * OD + od) * OP + op) * OQ + oq;
            if (dtype == ORACLE_I8) {
              const int8_t* p8 = (const int8_t*)pad;
              const int8_t* w8 = (const int8_t*)Wt;
              int32_t acc = 0;
              for (int64_t rc = 0; rc < C; ++rc)
                for (int64_t rd = 0; rd < T; ++rd)
                  for (int64_t rr = 0; rr < R; ++rr)
                    for (int64_t rs = 0; rs < S; ++rs) {
                      int64_t pi = (((n * C + rc) * PD + od * sd + rd * dd) * PH + op * sh + rr * dh) * PW +
                                   oq * sw + rs * dw;
                      int64_t wi = (((k * C + rc) * T + rd) * R + rr) * S + rs;
                      acc += mul_i(mode, p8[pi], w8[wi]);
                    }
              ((int32_t*)Y)[yidx] = acc;
            } else {
              const uint16_t* p16 = (const uint16_t*)pad;
              const uint16_t* w16 = (const uint16_t*)Wt;
              float acc = 0.0f;
              for (int64_t rc = 0; rc < C; ++rc)
                for (int64_t rd = 0; rd < T; ++rd)
                  for (int64_t rr = 0; rr < R; ++rr)
                    for (int64_t rs = 0; rs < S; ++rs) {
                      int64_t pi = (((n * C + rc) * PD + od * sd + rd * dd) * PH + op * sh + rr * dh) * PW +
                                   oq * sw + rs * dw;
                      int64_t wi = (((k * C + rc) * T + rd) * R + rr) * S + rs;
                      acc += mul_f(dtype, mode, p16[pi], w16[wi]);
                    }
              ((float*)Y)[yidx] = acc;
            }
          }
  free(pad);
  return 0;
}
