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

#define AMOS_ABI_VERSION 2

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
 * groups > 1: channel group g of X (C/groups channels) meets output channels
 * [g*K/groups, (g+1)*K/groups) only; Wt is [K][C/groups][T][R][S].  groups = C is the
 * depthwise convolution with K/C outputs per channel.
 * layout: how the three tensors (and a fused tail's D, like Y) are stored:
 *   AMOS_LAYOUT_NCHW  X [N][C][D][H][W]   Wt [K][C][T][R][S]   Y [N][K][OD][OP][OQ]
 *   AMOS_LAYOUT_NHWC  X [N][D][H][W][C]   Wt [T][R][S][C][K]   Y [N][OD][OP][OQ][K]
 *   AMOS_LAYOUT_HWNC  X [D][H][W][N][C]   Wt [T][R][S][C][K]   Y [OD][OP][OQ][N][K]
 * (groups > 1 exists for AMOS_LAYOUT_NCHW only.)
 * (reference computes: benchmark/amos/mapping_conv2d_tensorcore.py:7-104 (the three layouts),
 *  benchmark/amos/mapping_conv3d_tensorcore.py:7-55, mapping_groupedconv2d_tensorcore.py:7-60,
 *  mapping_depthwiseconv2d_tensorcore.py:7-48)
 */
typedef struct {
  int64_t N, C, D, H, W;
  int64_t K, T, R, S;
  int32_t stride_d, stride_h, stride_w;
  int32_t pad_d, pad_h, pad_w;
  int32_t dil_d, dil_h, dil_w;
  int32_t in_dtype, out_dtype;
  int32_t groups;        /* 0 or 1 = ordinary convolution */
  int32_t layout;        /* AMOS_LAYOUT_* */
} amos_conv_desc_t;

#define AMOS_LAYOUT_NCHW 0
#define AMOS_LAYOUT_NHWC 1
#define AMOS_LAYOUT_HWNC 2

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
  int32_t reserved[4];      /* [0]: AMOS_FLAG_* bits; the rest 0                            */
} amos_kernel_config_t;

/* conv: do not use the instances whose 3x3 window taps are unrolled (they are preferred where
 * they apply; the flag lets a sweep time the table-driven ones) */
#define AMOS_FLAG_NO_UNROLLED_TAPS 1
/* conv: one tile per workgroup also where the unrolled instance would let a workgroup walk
 * several tiles (more tiles than compute units, no split-K) */
#define AMOS_FLAG_NO_TILE_WALK 2
/* conv, AMOS_PIPE_NCHW: `Wt` points at weights that amos_conv_pack_weights has written (their owner
 * packs them once instead of every call packing them into its workspace) */
#define AMOS_FLAG_WEIGHTS_PACKED 4

/* how tiles travel from HBM to the MFMA operands */
#define AMOS_PIPE_AUTO 0      /* the mapper's choice; a depthwise convolution (groups == C,  */
                              /* NCDHW) and a GEMM with at most 8 rows on one side (K-       */
                              /* contiguous operands, that side within 16 KB) run on the     */
                              /* vector-ALU kernels under this value only                    */
#define AMOS_PIPE_STAGED 1    /* global -> registers -> LDS, any layout, ragged K             */
#define AMOS_PIPE_DIRECT4 2   /* withdrawn (was: direct copies, 256x256 tile, 4 waves - it   */
                              /* spilled registers and was slower): AMOS_ERR_INFEASIBLE       */
#define AMOS_PIPE_DIRECT8 3   /* same with 8 waves (two per SIMD)                             */
#define AMOS_PIPE_PATCH 4     /* conv: input patch staged once per channel chunk, weights     */
                              /* repacked into the workspace; needs amos_workspace_bytes();   */
                              /* 4 waves per workgroup                                        */
#define AMOS_PIPE_PATCH8 5    /* same with 8 waves (two per SIMD)                             */

#define AMOS_PIPE_NCHW 6      /* conv, 3x3 windows, NCDHW: the activations are read as they are   */
                              /* and transposed in registers on their way to LDS; the weights   */
                              /* are packed to [K][T*9][C] -- into the workspace by the call     */
                              /* (amos_workspace_bytes), or once by their owner                  */
                              /* (amos_conv_pack_weights, AMOS_FLAG_WEIGHTS_PACKED) -- or        */
                              /* transposed in registers as well: without a workspace, and for   */
                              /* a conv2d with 16-byte aligned weights also with one where the   */
                              /* mapper's model says the packing launch would cost more; tiles   */
                              /* 32 or 64 output channels x 128 or 256 output positions          */

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
/* bytes of device scratch the op's fastest pipeline wants (conv: repacked weights and
 * activations; GEMM and 1x1 convolutions: K-contiguous copies of operands); calls that get less
 * fall back to the register-staged pipeline, which needs none.  With cfg->split_k > 1 the figure
 * includes, behind the pipeline's own share, one slice of the output per split: the splits store
 * their partial sums there and a second launch adds them in the order of the splits, so that a
 * split-K result has the same bits on every run and the fused tail's operand may be the output
 * (the reference reduces its split through shared memory,
 * python/tvm/auto_tensorize/tensorization_phases/schedulers/cuda_split_K.py:868-914).  A call
 * with split_k > 1 and less workspace accumulates with atomicAdd into the zeroed output where the
 * kernel can (AMOS_PIPE_STAGED, AMOS_PIPE_PATCH*: sums in any order, an epilogue operand that
 * aliases the output is refused) and returns AMOS_ERR_WORKSPACE where it cannot
 * (AMOS_PIPE_DIRECT8, AMOS_PIPE_NCHW). */
size_t amos_workspace_bytes(int op, const void* desc, const amos_kernel_config_t* cfg);
/* the mapper's analytical estimate (seconds per launch) for a config: wave quantisation of the
 * grid over the CUs against MFMA issue time, HBM time for the algorithmic bytes, a launch floor
 * (stands where the reference ranks candidates with its analytical model,
 *  python/tvm/auto_tensorize/backend/tenet_integrate.py:168-202) */
int amos_estimate_seconds(int op, const void* desc, const amos_kernel_config_t* cfg, double* seconds);

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
 * amos_conv2d without a workspace argument and without any allocation: the scratch memory the
 * patch-staged pipeline wants (relaid weights and activations, the step table, split-K partial
 * sums) is an array of AMOS_NOALLOC_SCRATCH_BYTES that the library keeps on every GPU it has run
 * on, from the first call there until the process ends.  This entry point has no counterpart in
 * the reference; it is for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It calls no hipMalloc / hipFree
 * and no allocating library routine.  A convolution whose amos_workspace_bytes() exceeds the
 * array is refused with AMOS_ERR_WORKSPACE.  All calls on one GPU share that GPU's array: calls
 * that overlap in time on one GPU (two streams, two threads) race; serialise them.
 */
#define AMOS_NOALLOC_SCRATCH_BYTES (8u << 20)
int amos_conv2d_noalloc(const amos_conv_desc_t* desc, const amos_kernel_config_t* cfg, const void* X,
                        const void* Wt, void* Y, void* stream);

/*
 * Weights KCTRS -> [K][T*R*S][C] for AMOS_PIPE_NCHW (3x3 windows, one group, channels in whole
 * 16-byte chunks): amos_conv_packed_weights_bytes() bytes at `packed` (16-byte aligned; 0 = no
 * packed form for this descriptor).  A convolution called with AMOS_FLAG_WEIGHTS_PACKED takes the
 * packed weights as its `Wt`.  In the reference the reordered weight operand is a stage of its own
 * in front of the main kernel, recomputed on every call
 * (src/auto_tensorize/compute_transform.cc:181-293); a caller whose weights do not change between
 * calls can do it once here.
 */
size_t amos_conv_packed_weights_bytes(int op, const amos_conv_desc_t* desc);
int amos_conv_pack_weights(int op, const amos_conv_desc_t* desc, const void* Wt, void* packed, void* stream);

/* A tail operation fused into the store of the accumulators.  AMOS_EPI_ADD: out = acc + cast(D),
 * D an operand with the output's shape: GEMM / batched GEMM [M][ld] (ld 0 = N) with `stride`
 * elements between batches (0 = M*ld); convolution NKDPQ, contiguous.  D is fp32, fp16 or bf16
 * for fp32 outputs and int32 for int32 outputs.  (reference: the element-wise stage behind the
 * main op, python/tvm/auto_tensorize/hw_abstraction/cuda/wmma_bias.py:12-80 and
 * tests/python/auto_tensorize/test_compute_transform_gemm.py:7-23, "E = C + D") */
#define AMOS_EPI_NONE 0
#define AMOS_EPI_ADD 1
typedef struct {
  int32_t kind;          /* AMOS_EPI_* */
  int32_t dtype;         /* amos_dtype_t of the operand */
  const void* operand;   /* device pointer */
  int64_t ld;
  int64_t stride;
} amos_epilogue_t;
/* any of the four ops with a fused tail (epilogue NULL = none); in0, in1, out as in the op's own
 * entry point */
int amos_run_fused(int op, const void* desc, const amos_kernel_config_t* cfg,
                   const amos_epilogue_t* epilogue, const void* in0, const void* in1, void* out,
                   void* workspace, size_t ws_bytes, void* stream);

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

int amos_time_fused(int op, const void* desc, const amos_kernel_config_t* cfg,
                    const amos_epilogue_t* epilogue, const void* in0, const void* in1, void* out,
                    void* workspace, size_t ws_bytes, void* stream, int number, int repeat,
                    int min_repeat_ms, double* out_seconds);

/*
 * Dimension-separable gather:  out[o0, ..., o(n-1)] = in[ sum_d table_d[o_d] ]  where every
 * table_d[o_d] >= 0, else 0 (out dense, row-major).  It materialises the stages the reference
 * computes in front of an operand and that are not folded into a kernel's loader -- the zero
 * expansion and one-sided padding of a transposed convolution's input, its flipped and
 * transposed weights (benchmark/amos/mapping_transposedconv2d_tensorcore.py:7-102) -- as TVM's
 * default schedule would, each stage at root.  `tables` is device memory: for dimension d,
 * out_shape[d] entries from tables[table_offset[d]], each the source element offset that index
 * contributes (index * stride of the source dimension it maps to) or -1 where the stage's
 * predicate is false.  Sums that fall outside [0, in_elems) read as 0.
 */
typedef struct {
  int32_t ndim;             /* 1..5 */
  int32_t elem_bytes;       /* 1, 2 or 4 */
  int64_t out_shape[5];
  int64_t table_offset[5];
  int64_t in_elems;
} amos_gather_desc_t;

int amos_gather(const amos_gather_desc_t* desc, const void* in, const int32_t* tables, void* out,
                void* stream);
/* amos_time's loop around amos_gather */
int amos_time_gather(const amos_gather_desc_t* desc, const void* in, const int32_t* tables, void* out,
                     void* stream, int number, int repeat, int min_repeat_ms, double* out_seconds);

/* An element-wise stage in front of an operand: out[e] = f(in_0[e], ..., in_{n-1}[e]) for tensors
 * of one shape and element type, f a short postfix program over +, -, * and constants.  The
 * reference's default schedule computes such stages at root like any other TE stage (the
 * squared differences of benchmark/amos/mapping_variance_tensorcore.py:12-16); every operation
 * rounds to the element type as the compute's own arithmetic does (int8 wraps).
 *   program[k] = opcode | (argument << 8):  AMOS_ELT_LOAD  pushes in_argument[e],
 *   AMOS_ELT_CONST pushes consts[argument], AMOS_ELT_ADD / _SUB / _MUL replace the two topmost
 *   values (below OP top); at most four values on the stack, one left at the end */
#define AMOS_ELT_LOAD 1
#define AMOS_ELT_CONST 2
#define AMOS_ELT_ADD 3
#define AMOS_ELT_SUB 4
#define AMOS_ELT_MUL 5
typedef struct {
  int32_t dtype;      /* AMOS_F16 / AMOS_BF16 / AMOS_I8: inputs and output */
  int32_t n_inputs;   /* 1..4 */
  int32_t n_ops;      /* 1..16 */
  int32_t reserved;
  int64_t elems;
  int32_t program[16];
  float consts[4];
} amos_eltwise_desc_t;

int amos_eltwise(const amos_eltwise_desc_t* desc, const void* const* inputs, void* out, void* stream);
/* amos_time's loop around amos_eltwise */
int amos_time_eltwise(const amos_eltwise_desc_t* desc, const void* const* inputs, void* out, void* stream,
                      int number, int repeat, int min_repeat_ms, double* out_seconds);

/*
 * What the matrix cores sustain on this device when nothing else limits them: `launches`
 * back-to-back launches of a measurement kernel with the matrix-core instruction stream of the
 * 8192^3 fp16 product (256 workgroups x 4 waves, 1.0995e12 flop per launch), no barrier and no
 * wait for a copy anywhere (a wave keeps one LDS read in flight and consumes it behind the next
 * two to four matrix-core instructions); mean seconds per launch by HIP events on `stream` and the
 * flop of a launch are written out.  Synchronises the stream.
 *   shape            16: v_mfma_f32_16x16x32_f16, 32: v_mfma_f32_32x32x16_f16
 *   random_operands  0: small constants built in registers; 1: the operands of the instructions are
 *                    read (once) from a and b -- the switching activity of the multipliers, and
 *                    with it the clock the chip holds, depends on the operand values
 *   copies / reads   add the global -> LDS copies (64 KB per K step and workgroup) / the LDS
 *                    fragment reads (32 x 16 bytes per lane and K step) of a 256x256x64 tiling
 * a, b: device buffers of operand_bytes each, 16-byte aligned: at least 8 MiB, with copies an
 * [8192][8192] fp16 matrix (128 MiB); sink: 1 KiB of device memory (never written for finite
 * operands).  The reference has no counterpart: it reports seconds per call
 * (python/tvm/auto_tensorize/search/measure.py:175-207) and leaves the peak to its reader; the
 * benchmark here reports this figure next to the published peak.
 */
int amos_mfma_ceiling(int shape, int random_operands, int copies, int reads, const void* a, const void* b,
                      size_t operand_bytes, void* sink, int launches, void* stream, double* out_seconds,
                      double* out_flop);

/* name of the kernel instance a (desc, cfg) pair dispatches to, e.g.
 * "amos_igemm<f16,vec,vec,256x256>"; replaces func.imported_modules[0].get_source()
 * as the way to see what was chosen (reference: README.md:340). */
const char* amos_kernel_name(int op, const void* desc, const amos_kernel_config_t* cfg);

/* ---- the mapper: which loops of a compute can sit on the intrinsic's axes ------------------ */

/*
 * A compute as the matcher sees it: the structure of its body and, for every tensor
 * load in it, the index expressions in affine form over the compute's iteration
 * variables (spatial ones first, then reduce).
 *   tokens      the body in prefix order, one per node: (kind << 8) | dtype code, with
 *               kind 1 reduce, 2 cast, 3 mul, 4 add, 5 sub, 6 load, 7 select, 8 constant,
 *               9 anything else; index expressions are not part of the token stream
 *   iter_kinds  0 = spatial, 2 = reduce (TVM's IterVarType numbering)
 *   load_ndim   dimensions of each load, in token order
 *   coeffs      for every load and every dimension a row of n_iters + 2 values:
 *               the n_iters coefficients, the constant term, and 1 if the index is affine
 *               (0 = opaque: no variable that occurs in it can be mapped)
 */
typedef struct {
  int32_t n_tokens;
  const int32_t* tokens;
  int32_t n_iters;
  const int32_t* iter_kinds;
  const int64_t* iter_extents;
  int32_t n_loads;
  const int32_t* load_ndim;
  const int64_t* coeffs;
} amos_compute_t;

/*
 * Match points of `target` against the intrinsic `intrin`: every injective assignment of
 * the intrinsic's iteration variables to target variables of the same kind such that, load
 * by load, each intrinsic index equals a distinct target index dimension up to a positive
 * factor and a constant once unmapped variables are set to 0, and every other dimension
 * is constant.  Writes n_iters(intrin) target variable ids per point into `points`, in
 * enumeration order; returns the number of points (which may exceed max_points: only
 * max_points are written), 0 if the bodies do not line up, negative on a bad argument.
 * (reference: src/auto_tensorize/matcher.cc:47-310, include/tvm/auto_tensorize/matcher.h:42-331)
 */
int amos_match(const amos_compute_t* target, const amos_compute_t* intrin, int32_t* points,
               int32_t max_points);

/*
 * Mappings = non-empty subsets of the match points.  Two subsets that put the same sets of
 * loops on every intrinsic axis are one mapping (the first in binary counting order, first
 * point = most significant bit, is kept); with more than 15 points only single points whose
 * extents equal the intrinsic's and the all-ones subset are considered.  For each mapping
 * `feasible` says whether every fused extent reaches the intrinsic's extent.  Returns the
 * number of mappings (rows of n_points bytes in `bits`).
 * (reference: python/tvm/auto_tensorize/tensorization_phases/compute_transform.py:115-207,427-499)
 */
int amos_enumerate_mappings(int32_t n_points, int32_t n_axes, const int32_t* points,
                            const int64_t* target_extents, const int64_t* intrin_extents,
                            uint8_t* bits, uint8_t* feasible, int32_t max_mappings);

#ifdef __cplusplus
}
#endif
#endif /* AMOS_MI355X_H_ */
