/*
 * amos_mi355x.h -- C ABI of libamos_mi355x.so
 *
 * The library is the runnable end of the AMOS auto-tensorize path on an
 * AMD MI355X (gfx950): tiled GEMM, batched GEMM and implicit-GEMM
 * conv2d / conv3d kernels that run the v_mfma inner loop with fp32 / int32
 * accumulation, plus the mapper (matcher, mapping enumeration, feasibility
 * and resource checks, per-shape kernel configuration) that decides how a
 * compute is laid onto the intrinsic.
 *
 * In the reference the same seam is `tvm.build(sch, args, "cuda")` returning a
 * `tvm.runtime.Module` whose `func(*ndarrays)` ends in cuLaunchKernel
 * (reference: src/runtime/cuda/cuda_module.cc:105-172,
 * python/tvm/auto_tensorize/auto_tensorize.py:294-301).  Here every entry
 * point takes plain pointers and sizes:
 *
 *   - all data pointers are raw DEVICE pointers owned by the caller;
 *     the library never frees or retains them;
 *   - `stream` is a hipStream_t (NULL = the default stream); launches are
 *     asynchronous on that stream; only amos_time() synchronises;
 *   - return value 0 = ok, negative = error (see AMOS_ERR_*), a message is
 *     kept per thread and read with amos_last_error().
 */
#ifndef AMOS_MI355X_H_
#define AMOS_MI355X_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AMOS_ABI_VERSION 1

/* error codes */
#define AMOS_OK 0
#define AMOS_ERR_BAD_ARG (-1)      /* null pointer, non-positive extent, ...          */
#define AMOS_ERR_UNSUPPORTED (-2)  /* dtype / layout combination with no kernel       */
#define AMOS_ERR_INFEASIBLE (-3)   /* kernel config over the LDS / register budget,   */
                                   /* or a mapping whose fused extent is too small    */
#define AMOS_ERR_HIP (-4)          /* a HIP runtime call failed                       */
#define AMOS_ERR_WORKSPACE (-5)    /* split-K asked for but workspace too small       */

/* element types: inputs F16/BF16/I8, outputs F32/I32
 * (reference dtype pairs: python/tvm/auto_tensorize/hw_abs_dag/cuda/wmma_fp16.py:33-43,
 *  wmma_bf16.py, wmma_int8.py) */
typedef enum {
  AMOS_F16 = 0,
  AMOS_BF16 = 1,
  AMOS_I8 = 2,
  AMOS_F32 = 3,
  AMOS_I32 = 4
} amos_dtype_t;

typedef enum {
  AMOS_OP_GEMM = 0,
  AMOS_OP_BGEMM = 1,
  AMOS_OP_CONV2D = 2,
  AMOS_OP_CONV3D = 3
} amos_op_t;

/* device facts the mapper and the roofline report need
 * (replaces python/tvm/auto_tensorize/target.py:56-88 `CUDA(arch)`) */
typedef struct {
  int32_t compute_units;
  int32_t wave_size;
  int32_t max_clock_khz;
  int32_t lds_bytes_per_block;   /* largest LDS allocation one workgroup may ask for */
  int64_t hbm_bytes;
  char arch[64];
  double peak_tflops_f16;        /* CUs x clock x 4096 flop/clk/CU (dense)   */
  double peak_tops_i8;           /* CUs x clock x 8192 op/clk/CU (dense)     */
} amos_device_info_t;

/*
 * C[M,N] = sum_k A(m,k) * B(k,n), out dtype F32 (F16/BF16 in) or I32 (I8 in).
 * trans_a = 0: A stored [M,K] with row stride lda;  1: stored [K,M].
 * trans_b = 0: B stored [K,N] with row stride ldb;  1: stored [N,K]
 *              ("column-major B", the reference's compute key "ntn").
 * C is row-major [M,N] with row stride ldc.  Leading dimensions count elements.
 * (reference compute: benchmark/amos/mapping_gemm_tensorcore.py:7-15; the four
 *  transpose spellings: python/tvm/tensor_graph/nn/functional.py:1662-1722;
 *  intrinsic semantics: python/tvm/auto_tensorize/hw_abstraction/cuda/wmma_base.py:439-491)
 */
typedef struct {
  int64_t M, N, K;
  int32_t in_dtype, out_dtype;
  int32_t trans_a, trans_b;
  int64_t lda, ldb, ldc;
} amos_gemm_desc_t;

/* batch of independent GEMMs; operand b starts at base + b*stride_x (elements).
 * (reference: python/tvm/tensor_graph/nn/functional.py:1725-1793) */
typedef struct {
  int64_t batch;
  amos_gemm_desc_t g;
  int64_t stride_a, stride_b, stride_c;
} amos_bgemm_desc_t;

/*
 * Y[n,k,od,op,oq] = sum_{c,t,r,s} X[n,c, od*sd+t*dd-pd, op*sh+r*dh-ph, oq*sw+s*dw-pw] * Wt[k,c,t,r,s]
 * with out-of-range X reads = 0.  X is NCDHW, Wt is KCTRS, Y is NKDPQ, all dense.
 * conv2d is the D = T = 1, sd = dd = 1, pd = 0 case.
 * (reference computes: benchmark/amos/mapping_conv2d_tensorcore.py:7-42,
 *  benchmark/amos/mapping_conv3d_tensorcore.py:7-55)
 */
typedef struct {
  int64_t N, C, D, H, W;
  int64_t K, T, R, S;
  int32_t stride_d, stride_h, stride_w;
  int32_t pad_d, pad_h, pad_w;
  int32_t dil_d, dil_h, dil_w;
  int32_t in_dtype, out_dtype;
} amos_conv_desc_t;

/*
 * How the implicit GEMM is tiled on the chip -- the counterpart of the
 * reference's schedule parameters (spatial_factors / reduce_factors /
 * vectorize, python/tvm/auto_tensorize/tensorization_phases/schedulers/cuda_v2.py:42-52).
 * A zeroed struct (or a NULL pointer where one is accepted) = let the mapper choose.
 */
typedef struct {
  int32_t tile_i, tile_j;   /* block tile of the MFMA row / column operand: 64, 128 or 256 */
  int32_t split_k;          /* >= 1: blocks along the fused reduction                       */
  int32_t pipeline;         /* AMOS_PIPE_*; 0 = mapper's choice                             */
  int32_t reserved[4];
} amos_kernel_config_t;

/* how tiles travel from HBM to the MFMA operands */
#define AMOS_PIPE_AUTO 0
#define AMOS_PIPE_STAGED 1    /* global -> registers -> LDS, any layout, ragged K             */
#define AMOS_PIPE_DIRECT4 2   /* global -> LDS direct copies, 256x256 tile, 4 waves           */
#define AMOS_PIPE_DIRECT8 3   /* same with 8 waves (two per SIMD)                             */
#define AMOS_PIPE_PATCH 4     /* conv: input patch staged once per channel chunk, weights     */
                              /* repacked into the workspace; needs amos_workspace_bytes()    */

int amos_version(void);
const char* amos_last_error(void);

/* replaces target.py:27-49 get_cuda_compute_version + target.py:56-88 */
int amos_device_info(amos_device_info_t* out);

/* the mapper's per-shape choice; `desc` points at the op's descriptor struct */
int amos_default_config(int op, const void* desc, amos_kernel_config_t* out);
/* resource check of a config (reference: python/tvm/auto_tensorize/search/checker.py:43-82,
 * src/auto_tensorize/utils.cc:31-57): fills LDS bytes and accumulator registers per lane,
 * returns AMOS_ERR_INFEASIBLE when over budget */
int amos_check_config(int op, const void* desc, const amos_kernel_config_t* cfg,
                      int64_t* lds_bytes, int64_t* acc_regs);
/* bytes of device scratch the op's fastest pipeline wants (conv: repacked weights); calls
 * that get less fall back to the register-staged pipeline, which needs none */
size_t amos_workspace_bytes(int op, const void* desc, const amos_kernel_config_t* cfg);

/* the runnable kernels: replace `func(A, B, C)` of the module tvm.build returns
 * (reference: python/tvm/auto_tensorize/auto_tensorize.py:294-301,
 *  python/tvm/auto_tensorize/search/measure.py:192-206) */
int amos_gemm(const amos_gemm_desc_t* desc, const amos_kernel_config_t* cfg, const void* A,
              const void* B, void* C, void* workspace, size_t ws_bytes, void* stream);
int amos_bgemm(const amos_bgemm_desc_t* desc, const amos_kernel_config_t* cfg, const void* A,
               const void* B, void* C, void* workspace, size_t ws_bytes, void* stream);
int amos_conv2d(const amos_conv_desc_t* desc, const amos_kernel_config_t* cfg, const void* X,
                const void* Wt, void* Y, void* workspace, size_t ws_bytes, void* stream);
int amos_conv3d(const amos_conv_desc_t* desc, const amos_kernel_config_t* cfg, const void* X,
                const void* Wt, void* Y, void* workspace, size_t ws_bytes, void* stream);

/*
 * Mean seconds per launch, measured the way the reference's time_evaluator does
 * (reference: src/runtime/rpc/rpc_module.cc:355-388): one warm-up launch, then
 * `number` back-to-back launches bracketed by HIP events on `stream`; `number`
 * grows until one repeat lasts at least `min_repeat_ms`; `repeat` such
 * measurements are written to out_seconds[0..repeat).  Synchronises the stream.
 */
int amos_time(int op, const void* desc, const amos_kernel_config_t* cfg, const void* in0,
              const void* in1, void* out, void* workspace, size_t ws_bytes, void* stream,
              int number, int repeat, int min_repeat_ms, double* out_seconds);

/* name of the kernel instance a (desc, cfg) pair dispatches to, e.g.
 * "amos_igemm<f16,vec,vec,256x256>"; replaces func.imported_modules[0].get_source()
 * as the way to see what was chosen (reference: README.md:340). */
const char* amos_kernel_name(int op, const void* desc, const amos_kernel_config_t* cfg);

#ifdef __cplusplus
}
#endif
#endif /* AMOS_MI355X_H_ */
