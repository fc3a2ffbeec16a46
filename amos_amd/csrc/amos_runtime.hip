// Host side of libamos_mi355x.so: descriptor validation, kernel-instance
// dispatch, launch, timing.  The C ABI is declared in include/amos_mi355x.h.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <mutex>
#include <string>

#include "amos_mi355x.h"
#include "conv_fprop_kernel.h"
#include "conv_fewc_kernel.h"
#include "conv_nchw_kernel.h"
#include "depthwise_kernel.h"
#include "gemm_tn_kernel.h"
#include "igemm_instances.h"
#include "mapper.h"
#include "skinny_gemm_kernel.h"

namespace amos {

static thread_local char g_err[512] = "";

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

#define HIP_TRY(expr)                                                                   \
  do {                                                                                  \
    hipError_t e_ = (expr);                                                             \
    if (e_ != hipSuccess)                                                               \
      return set_error(AMOS_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_));    \
  } while (0)

// out[o] = in[sum_d tab_d[o_d]] where all table entries are >= 0 (else 0); five dimensions,
// the innermost fastest, unused leading ones of extent 1
struct GatherParams {
  int shape[5];
  int use[5];
  int64_t tab[5];
  int64_t total, in_elems;
};
template <typename T>
__global__ __launch_bounds__(256) void amos_gather_kernel(const GatherParams g, const T* __restrict__ in,
                                                         const int* __restrict__ tables, T* __restrict__ out) {
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < g.total; idx += (int64_t)gridDim.x * 256) {
    int64_t rest = idx, off = 0;
    bool ok = true;
#pragma unroll
    for (int k = 4; k >= 0; --k) {
      const int64_t q = rest / g.shape[k];
      const int o = (int)(rest - q * g.shape[k]);
      rest = q;
      if (g.use[k]) {
        const int e = tables[g.tab[k] + o];
        ok = ok && e >= 0;
        off += e;
      }
    }
    ok = ok && off < g.in_elems;
    out[idx] = ok ? in[off] : (T)0;
  }
}

// out[e] = program(in_0[e], ...): a postfix program on a four-deep register stack; every value is
// rounded to the element type (fp16 / bf16 round-to-nearest-even, int8 wraps) as soon as it exists
struct EltwiseParams {
  const void* in[4];
  void* out;
  int64_t elems;
  int n_ops;
  int program[16];
  float consts[4];
};
template <int DT> struct EltType { typedef unsigned short raw_t; };
template <> struct EltType<DT_I8> { typedef signed char raw_t; };
template <int DT>
__device__ __forceinline__ float elt_round(float v) {
  if constexpr (DT == DT_F16) {
    return (float)(_Float16)v;
  } else if constexpr (DT == DT_BF16) {
    unsigned u = __builtin_bit_cast(unsigned, v);
    if ((u & 0x7f800000u) != 0x7f800000u) u += 0x7fffu + ((u >> 16) & 1u);   // (NaN / Inf keep their bits)
    return __builtin_bit_cast(float, u & 0xffff0000u);
  } else {
    return (float)(signed char)(int)v;      // |v| < 2^17 here: exact in float, wraps like int8
  }
}
template <int DT>
__device__ __forceinline__ float elt_load(const void* p, int64_t e) {
  typedef typename EltType<DT>::raw_t raw_t;
  const raw_t r = ((const raw_t*)p)[e];
  if constexpr (DT == DT_F16) return (float)__builtin_bit_cast(_Float16, r);
  else if constexpr (DT == DT_BF16) return __builtin_bit_cast(float, (unsigned)r << 16);
  else return (float)r;
}
template <int DT>
__global__ __launch_bounds__(256) void amos_eltwise_kernel(const EltwiseParams p) {
  typedef typename EltType<DT>::raw_t raw_t;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < p.elems; e += (int64_t)gridDim.x * 256) {
    float s0 = 0, s1 = 0, s2 = 0, s3 = 0;     // s0 = top of the stack
    for (int k = 0; k < p.n_ops; ++k) {       // (uniform control flow: the program is a kernel argument)
      const int op = p.program[k] & 255, arg = p.program[k] >> 8;
      if (op == AMOS_ELT_LOAD || op == AMOS_ELT_CONST) {
        const float v = op == AMOS_ELT_LOAD ? elt_load<DT>(p.in[arg], e) : elt_round<DT>(p.consts[arg]);
        s3 = s2; s2 = s1; s1 = s0; s0 = v;
      } else {
        const float r = op == AMOS_ELT_ADD ? s1 + s0 : op == AMOS_ELT_SUB ? s1 - s0 : s1 * s0;
        s0 = elt_round<DT>(r); s1 = s2; s2 = s3;
      }
    }
    raw_t o;
    if constexpr (DT == DT_F16) o = __builtin_bit_cast(unsigned short, (_Float16)s0);
    else if constexpr (DT == DT_BF16) o = (unsigned short)(__builtin_bit_cast(unsigned, s0) >> 16);
    else o = (signed char)(int)s0;
    ((raw_t*)p.out)[e] = o;
  }
}

// dst[b][c][r] = src[b][r][c] for r < rows, c < cols (src rows ld_src apart, dst dense): an
// operand whose rows are the contiguous direction becomes K-contiguous.  64 x 64 tiles through
// LDS, 8 bytes per lane on both sides where alignment allows.
struct TransposeJob {
  const char* src;
  char* dst;
  int rows, cols;          // of the source: rows = the reduction index K of a row-contiguous operand
  int64_t ld_src, batch_src, batch_dst;
  int batch;
  int ld_dst;              // >= rows; the result's rows are zero-filled from `rows` up to it
  int copy;                // 1: no transposition, dst[r][k] = src[r][k] (k < cols), zero up to ld_dst
  // col_w > 0: column c of the source is the element (c / col_w) * col_so + (c % col_w) * col_si
  // of its row (every stride-th pixel of an image plane); 0: the element c
  int col_w, col_si;
  int64_t col_so;
  FastDiv fd_col_w;
};
template <typename T>
__global__ __launch_bounds__(256) void amos_transpose_kernel(const TransposeJob j) {
  constexpr int VE = 8 / (int)sizeof(T);      // elements per 8-byte access
  constexpr int PITCH = 64 + VE;              // LDS row in elements (keeps 8-byte alignment)
  __shared__ __attribute__((aligned(16))) T tile[64 * PITCH];
  const int t = threadIdx.x;
  const int c0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
  const T* src = (const T*)j.src + (int64_t)blockIdx.z * j.batch_src;
  T* dst = (T*)j.dst + (int64_t)blockIdx.z * j.batch_dst;
  constexpr int LT = 64 / VE;                 // threads per 64-element row
  constexpr int RPP = 256 / LT;               // rows per pass
  const bool vec_in = (((uintptr_t)src | (uintptr_t)(j.ld_src * sizeof(T))) & 7) == 0 && j.col_w == 0;
  const int lc = (t % LT) * VE, lr = t / LT;
  auto col_at = [&](int c) -> int64_t {
    if (j.col_w == 0) return c;
    const int outer = fast_div(c, j.fd_col_w);
    return outer * j.col_so + (int64_t)(c - outer * j.col_w) * j.col_si;
  };
#pragma unroll
  for (int pass = 0; pass < 64 / RPP; ++pass) {
    const int r = lr + pass * RPP;
    const int gr = r0 + r, gc = c0 + lc;
    T v[VE];
    if (gr < j.rows && vec_in && gc + VE <= j.cols) {
      *(uint2*)v = *(const uint2*)(src + (int64_t)gr * j.ld_src + gc);
    } else {
#pragma unroll
      for (int e = 0; e < VE; ++e)
        v[e] = (gr < j.rows && gc + e < j.cols) ? src[(int64_t)gr * j.ld_src + col_at(gc + e)] : (T)0;
    }
#pragma unroll
    for (int e = 0; e < VE; ++e) tile[(lc + e) * PITCH + r] = v[e];     // transposed into LDS
  }
  __syncthreads();
  const bool vec_out = (((uintptr_t)dst | (uintptr_t)((int64_t)j.ld_dst * sizeof(T))) & 7) == 0;
#pragma unroll
  for (int pass = 0; pass < 64 / RPP; ++pass) {
    const int c = lr + pass * RPP;           // a column of the source = a row of the result
    const int gc = c0 + c, gr = r0 + lc;
    if (gc >= j.cols) continue;
    if (vec_out && gr + VE <= j.ld_dst) {    // (rows of the source past `rows` were read as zeros)
      *(uint2*)(dst + (int64_t)gc * j.ld_dst + gr) = *(const uint2*)(tile + c * PITCH + lc);
    } else {
#pragma unroll
      for (int e = 0; e < VE; ++e)
        if (gr + e < j.ld_dst) dst[(int64_t)gc * j.ld_dst + gr + e] = tile[c * PITCH + lc + e];
    }
  }
}

// dst[b][r][k] = src[b][r][k] for k < cols, 0 for cols <= k < ld_dst (rows of a K-contiguous
// operand copied to whole, aligned K steps)
template <typename T>
__global__ __launch_bounds__(256) void amos_padcopy_kernel(const TransposeJob j) {
  constexpr int VE = 8 / (int)sizeof(T);
  const T* src = (const T*)j.src + (int64_t)blockIdx.z * j.batch_src;
  T* dst = (T*)j.dst + (int64_t)blockIdx.z * j.batch_dst;
  const int per_row = j.ld_dst / VE;          // ld_dst is a multiple of a K step
  const bool vec_in = (((uintptr_t)src | (uintptr_t)(j.ld_src * sizeof(T))) & 7) == 0;
  const int64_t total = (int64_t)j.rows * per_row;
  for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
    const int r = (int)(idx / per_row), k = (int)(idx - (int64_t)r * per_row) * VE;
    T v[VE];
    if (vec_in && k + VE <= j.cols) {
      *(uint2*)v = *(const uint2*)(src + (int64_t)r * j.ld_src + k);
    } else {
#pragma unroll
      for (int e = 0; e < VE; ++e) v[e] = k + e < j.cols ? src[(int64_t)r * j.ld_src + k + e] : (T)0;
    }
    *(uint2*)(dst + (int64_t)r * j.ld_dst + k) = *(const uint2*)v;
  }
}

template <typename T>
__global__ void fill_zero_kernel(T* p, int64_t rows, int64_t cols, int64_t ld) {
  int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  int64_t n = rows * cols;
  for (; idx < n; idx += (int64_t)gridDim.x * blockDim.x) p[(idx / cols) * ld + idx % cols] = 0;
}

// out[b][r][c] = part[0][b][r][c] + part[1][b][r][c] + ... in that order (split-K partial sums);
// blockIdx.y walks the batches, `batch_stride` elements apart in the output and in every slice
template <typename T>
__global__ void reduce_splits_kernel(T* out, const T* part, int64_t rows, int64_t cols, int64_t ld, int nsplit,
                                     int64_t stride, int64_t batch_stride, int64_t nbatch) {
  const int64_t n = rows * cols;
  for (int64_t b = blockIdx.y; b < nbatch; b += gridDim.y)
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n; idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t off = b * batch_stride + (idx / cols) * ld + idx % cols;
    T acc = part[off];
    for (int s = 1; s < nsplit; ++s) acc += part[(int64_t)s * stride + off];
    out[off] = acc;
  }
}

// ---- kernel instance table (defined in inst_*.hip) -------------------------------------
static Instance* pick(int dt, int rl, int cl, int ti, int tj) {
  if (rl == LD_TVEC) {
    if (dt == DT_F16) return pick_f16_tvec(cl, ti, tj);
    if (dt == DT_BF16) return pick_bf16_tvec(cl, ti, tj);
    return nullptr;
  }
  switch (dt * 2 + (rl == LD_STRIDED)) {
    case DT_F16 * 2: return pick_f16_vec(cl, ti, tj);
    case DT_F16 * 2 + 1: return pick_f16_strided(cl, ti, tj);
    case DT_BF16 * 2: return pick_bf16_vec(cl, ti, tj);
    case DT_BF16 * 2 + 1: return pick_bf16_strided(cl, ti, tj);
    case DT_I8 * 2: return pick_i8_vec(cl, ti, tj);
    case DT_I8 * 2 + 1: return pick_i8_strided(cl, ti, tj);
  }
  return nullptr;
}

// ---- descriptor -> launch plan --------------------------------------------------------
// Col[n][od,op,oq][k] = X[n][c][od*sd - pd + t*dd][op*sh - ph + r*dh][oq*sw - pw + s*dw] for
// k = ((c*T + t)*R + r)*S + s < Kred, zero where the window hangs over the edge and for
// Kred <= k < Kp.  One thread per 16 bytes of the result; loads at clamped addresses, masked.
struct Im2colParams {
  const char* x;
  char* dst;
  int C, D, H, W, T, R, S, OD, OP, OQ;
  int sd, sh, sw, pd, ph, pw, dd, dh, dw;
  int Kred, chunks;        // chunks = Kp / elements per 16 bytes
  unsigned total;          // N * OD * OP * OQ * chunks, below 2^31
  int64_t x_image;         // elements per image
  FastDiv fd_chunks, fd_oq, fd_op, fd_od, fd_trs, fd_rs, fd_s;
};
template <typename T>
__global__ __launch_bounds__(256) void amos_im2col_kernel(const Im2colParams p) {
  constexpr int VE = 16 / (int)sizeof(T);
  const T* __restrict__ x = (const T*)p.x;
  const unsigned step = gridDim.x * 256u;
  for (unsigned idx = blockIdx.x * 256u + threadIdx.x; idx < p.total; idx += step) {
    const int row = fast_div((int)idx, p.fd_chunks);
    const int k0 = ((int)idx - row * p.chunks) * VE;
    int rest = fast_div(row, p.fd_oq);
    const int oq = row - rest * p.OQ;
    int nx = fast_div(rest, p.fd_op);
    const int op = rest - nx * p.OP;
    const int n = fast_div(nx, p.fd_od);
    const int od = nx - n * p.OD;
    int c = fast_div(k0, p.fd_trs);
    rest = k0 - c * (p.T * p.R * p.S);
    int t = fast_div(rest, p.fd_rs);
    rest -= t * (p.R * p.S);
    int r = fast_div(rest, p.fd_s);
    int s = rest - r * p.S;
    const T* img = x + (int64_t)n * p.x_image;
    const int d0 = od * p.sd - p.pd, h0 = op * p.sh - p.ph, w0 = oq * p.sw - p.pw;
    T v[VE];
#pragma unroll
    for (int e = 0; e < VE; ++e) {
      const int id = d0 + t * p.dd, ih = h0 + r * p.dh, iw = w0 + s * p.dw;
      const bool ok = k0 + e < p.Kred && (unsigned)id < (unsigned)p.D && (unsigned)ih < (unsigned)p.H &&
                      (unsigned)iw < (unsigned)p.W;
      unsigned m = ok ? 0xffffffffu : 0u;
      asm("" : "+v"(m));       // (a select of "loaded or zero" would become a branch around the load)
      const int cc = c < p.C ? c : p.C - 1;
      const int dc = id < 0 ? 0 : id >= p.D ? p.D - 1 : id;
      const int hc = ih < 0 ? 0 : ih >= p.H ? p.H - 1 : ih;
      const int wc = iw < 0 ? 0 : iw >= p.W ? p.W - 1 : iw;
      const unsigned raw = (unsigned)img[((cc * p.D + dc) * p.H + hc) * p.W + wc];
      v[e] = (T)(raw & m);
      if (++s == p.S) { s = 0; if (++r == p.R) { r = 0; if (++t == p.T) { t = 0; ++c; } } }
    }
    *(uint4*)(p.dst + (int64_t)idx * 16) = *(const uint4*)v;
  }
}

struct Plan {
  IgemmParams p;
  int dt, rl, cl;
  amos_kernel_config_t cfg;
  int64_t batch;
  int split;
  // zero fill of the output before a split-K launch that accumulates with atomics
  int64_t fill_rows, fill_cols, fill_ld;
  int fill_once;
  // split-K with partial sums in the workspace (behind what the pipeline itself keeps there): every
  // split stores its tile into its own slice, a second launch adds the slices in the order of the
  // splits -- the same bits on every run, and the output is written after every read of the call
  char* ws_base;
  size_t ws_bytes, ws_own;     // the caller's workspace; the pipeline's own share of it
  char* part;                  // the slices (nullptr: none)
  int64_t part_stride;         // elements between them
  char* part_out;              // the output that the reduction writes
  // direct-to-LDS GEMM pipeline (0 = not used, else waves per block)
  int tn_waves;
  GemmTnParams tn;
  // patch-staged convolution (0 = not used)
  int conv_ups;
  ConvFpropParams cv;
  size_t conv_lds;
  int conv_occ;
  int conv_waves;
  int conv_w9;
  // GEMM operands copied K-contiguous into the workspace in front of the kernel
  int n_transposes;
  TransposeJob tr[2];
  // depthwise convolution on the vector ALUs (0 = not used, else 1 + DW_* kind)
  int dw;
  DepthwiseParams dwp;
  // im2col copy of a convolution's activations in front of the GEMM (0 = not used)
  int im2col;
  Im2colParams icp;
  // GEMM with at most 16 rows on one side, on the vector ALUs (0 = not used)
  int skinny;
  int skinny_big_is_a;
  SkinnyParams sk;
  // convolution on few input channels (0 = not used)
  int fewc;
  ConvFewcParams fcp;
  size_t fewc_lds;
  // convolution read straight from NCDHW / KCTRS (0 = not used)
  int nchw;
  int nchw_wmode, nchw_pt, nchw_groups, nchw_nwl, nchw_lb;
  int nchw_pack;            // 1: the weights are packed into the workspace in front of the kernel
  const void* nchw_w_src;   // ... from here
  ConvNchwParams nc;
  size_t nchw_lds;
};

static int dtype_pair(int in_dtype, int out_dtype, int* dt) {
  if (in_dtype == AMOS_F16 && out_dtype == AMOS_F32) { *dt = DT_F16; return 0; }
  if (in_dtype == AMOS_BF16 && out_dtype == AMOS_F32) { *dt = DT_BF16; return 0; }
  if (in_dtype == AMOS_I8 && out_dtype == AMOS_I32) { *dt = DT_I8; return 0; }
  return set_error(AMOS_ERR_UNSUPPORTED,
                   "unsupported dtype pair in=%d out=%d (f16->f32, bf16->f32, i8->i32 exist)",
                   in_dtype, out_dtype);
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

static int fits_int(int64_t v) { return v > 0 && v < (int64_t)1 << 31; }

// elements from the first to the last element of the planned output, rounded up to 64
static int64_t plan_out_footprint(const Plan& pl) {
  const int64_t n = (pl.fill_once ? 0 : (pl.batch - 1) * pl.p.out_batch) + (pl.fill_rows - 1) * pl.fill_ld + pl.fill_cols;
  return (n + 63) & ~(int64_t)63;
}
// whether the caller's workspace has room for `split` slices of partial sums behind the pipeline's own share
// The plan takes `bytes` from the front of the caller's workspace (operand copies, packed weights,
// relaid activations): the slices of a split's partial sums start behind the largest such claim.
// amos_workspace_bytes() assumes 16-byte aligned operands; a misaligned one can add a copy, and
// the slices must not start inside it.
static void claim_workspace(Plan& pl, int64_t bytes) {
  const size_t b = ((size_t)(bytes > 0 ? bytes : 0) + 255) & ~(size_t)255;
  if (b > pl.ws_own) pl.ws_own = b;
}
static bool split_partials_fit(const Plan& pl, int split) {
  if (!pl.ws_base || ((uintptr_t)pl.ws_base & 255) || split < 2) return false;
  return pl.ws_bytes >= pl.ws_own + (size_t)split * (size_t)plan_out_footprint(pl) * 4;
}

static int plan_finish(Plan& pl, int op, const void* desc, const amos_kernel_config_t* cfg) {
  amos_kernel_config_t c;
  if (cfg && cfg->tile_i > 0 && cfg->tile_j > 0) {
    c = *cfg;
    if (c.split_k < 1) c.split_k = 1;
  } else {
    int rc = amos_default_config(op, desc, &c);
    if (rc) return rc;
    if (cfg && cfg->split_k > 0) c.split_k = cfg->split_k;
  }
  pl.cfg = c;
  const int es = pl.dt == DT_I8 ? 1 : 2;
  const int bke = 128 / es;
  IgemmParams& p = pl.p;
  p.k_tiles = (p.Kred + bke - 1) / bke;
  int split = c.split_k;
  if (split > p.k_tiles) split = p.k_tiles;
  p.k_tiles_per_split = (p.k_tiles + split - 1) / split;
  split = (p.k_tiles + p.k_tiles_per_split - 1) / p.k_tiles_per_split;
  pl.split = split;
  p.atomic_out = split > 1;
  p.tiles_i = (p.I + c.tile_i - 1) / c.tile_i;
  p.tiles_j = (p.J + c.tile_j - 1) / c.tile_j;
  if ((int64_t)p.tiles_i * p.tiles_j >= ((int64_t)1 << 31))
    return set_error(AMOS_ERR_BAD_ARG, "too many tiles");
  if (split > 65535 || pl.batch > 65535)
    return set_error(AMOS_ERR_UNSUPPORTED, "batch (%lld) or split_k (%d) above 65535",
                     (long long)pl.batch, split);
  return 0;
}

static int plan_gemm(Plan& pl, int op, const void* desc_any, const amos_gemm_desc_t* d,
                     int64_t batch, int64_t sa, int64_t sb, int64_t sc,
                     const amos_kernel_config_t* cfg, const void* A, const void* B, void* C,
                     void* workspace = nullptr, size_t ws_bytes = 0);

// plan a GEMM on copies of its operands (see gemm_repack)
static int plan_gemm_repacked(Plan& pl, int op, const amos_gemm_desc_t* d, const GemmRepack& rp, int64_t batch,
                              int64_t sa, int64_t sb, int64_t sc, const amos_kernel_config_t* cfg,
                              const void* A, const void* B, void* C, void* workspace,
                              const ConvSubsample* sub = nullptr) {
  amos_bgemm_desc_t e;
  memset(&e, 0, sizeof(e));
  e.g = *d;
  e.g.K = rp.Kp;
  e.batch = batch;
  e.stride_a = sa; e.stride_b = sb; e.stride_c = sc;
  TransposeJob jobs[2];
  int n = 0;
  char* ws = (char*)workspace;
  const void *A2 = A, *B2 = B;
  if (rp.copy_a) {
    if (d->trans_a)   // stored [K][M] -> [M][Kp]
      jobs[n++] = TransposeJob{(const char*)A, ws, (int)d->K, (int)d->M, d->lda, sa, d->M * rp.Kp, (int)batch, (int)rp.Kp, 0};
    else              // stored [M][K] -> [M][Kp]
      jobs[n++] = TransposeJob{(const char*)A, ws, (int)d->M, (int)d->K, d->lda, sa, d->M * rp.Kp, (int)batch, (int)rp.Kp, 1};
    A2 = ws;
    ws += rp.bytes_a;
    e.g.trans_a = 0; e.g.lda = rp.Kp; e.stride_a = d->M * rp.Kp;
  }
  if (rp.copy_b) {
    if (!d->trans_b) {  // stored [K][N] -> [N][Kp]
      jobs[n++] = TransposeJob{(const char*)B, ws, (int)d->K, (int)d->N, d->ldb, sb, d->N * rp.Kp, (int)batch, (int)rp.Kp, 0};
      if (sub) {        // the logical row is gathered from an image plane
        TransposeJob& j = jobs[n - 1];
        j.ld_src = sub->chan_step;
        j.col_w = sub->out_w; j.col_si = sub->col_step; j.col_so = sub->row_step;
        j.fd_col_w = make_fast_div((uint32_t)sub->out_w);
      }
    } else
      jobs[n++] = TransposeJob{(const char*)B, ws, (int)d->N, (int)d->K, d->ldb, sb, d->N * rp.Kp, (int)batch, (int)rp.Kp, 1};
    B2 = ws;
    e.g.trans_b = 1; e.g.ldb = rp.Kp; e.stride_b = d->N * rp.Kp;
  }
  const bool batched = batch > 1 || op == AMOS_OP_BGEMM;
  // without a tile from the caller: the mapper's choice for the product on the copies (the same
  // one amos_default_config makes for the original problem, whose estimate differs by the copies'
  // constant time)
  int rc = plan_gemm(pl, batched ? AMOS_OP_BGEMM : AMOS_OP_GEMM, batched ? (const void*)&e : (const void*)&e.g,
                     &e.g, batch, e.stride_a, e.stride_b, e.stride_c, cfg, A2, B2, C);
  if (rc) return rc;
  pl.n_transposes = n;
  for (int k = 0; k < n; ++k) pl.tr[k] = jobs[k];
  return 0;
}

static int plan_gemm(Plan& pl, int op, const void* desc_any, const amos_gemm_desc_t* d,
                     int64_t batch, int64_t sa, int64_t sb, int64_t sc,
                     const amos_kernel_config_t* cfg, const void* A, const void* B, void* C,
                     void* workspace, size_t ws_bytes) {
  if (!d || !A || !B || !C) return set_error(AMOS_ERR_BAD_ARG, "null pointer argument");
  // (a one-column row-major B or a one-row transposed A is K-contiguous memory: say so)
  const amos_gemm_desc_t norm = batch == 1 ? gemm_normalized(*d) : *d;
  d = &norm;
  pl.n_transposes = 0;
  if (workspace && (!cfg || cfg->pipeline != AMOS_PIPE_STAGED) && ((uintptr_t)workspace & 255) == 0 &&
      fits_int(d->M) && fits_int(d->N) && fits_int(d->K) && d->K < (1 << 30) &&
      d->lda >= (d->trans_a ? d->M : d->K) && d->ldb >= (d->trans_b ? d->K : d->N) &&
      (d->in_dtype == AMOS_F16 || d->in_dtype == AMOS_BF16 || d->in_dtype == AMOS_I8)) {
    const GemmRepack rp = gemm_repack(*d, batch, !aligned16(A), !aligned16(B));
    if (rp.total() > 0 && ws_bytes >= (size_t)rp.total()) {
      claim_workspace(pl, rp.total());
      return plan_gemm_repacked(pl, op, d, rp, batch, sa, sb, sc, cfg, A, B, C, workspace);
    }
  }
  if (!fits_int(d->M) || !fits_int(d->N) || !fits_int(d->K) || batch <= 0)
    return set_error(AMOS_ERR_BAD_ARG, "extents must be in [1, 2^31): M=%lld N=%lld K=%lld batch=%lld",
                     (long long)d->M, (long long)d->N, (long long)d->K, (long long)batch);
  int rc = dtype_pair(d->in_dtype, d->out_dtype, &pl.dt);
  if (rc) return rc;
  const int64_t min_lda = d->trans_a ? d->M : d->K;
  const int64_t min_ldb = d->trans_b ? d->K : d->N;
  if (d->lda < min_lda || d->ldb < min_ldb || d->ldc < d->N)
    return set_error(AMOS_ERR_BAD_ARG, "leading dimension too small (lda=%lld ldb=%lld ldc=%lld)",
                     (long long)d->lda, (long long)d->ldb, (long long)d->ldc);
  const int es = pl.dt == DT_I8 ? 1 : 2;
  const int ce = 16 / es;
  IgemmParams& p = pl.p;
  memset(&p, 0, sizeof(p));
  p.I = (int)d->M;
  p.J = (int)d->N;
  p.Kred = (int)d->K;
  p.row_base = (const char*)A;
  p.col_base = (const char*)B;
  p.row_batch = sa;
  p.col_batch = sb;
  if (d->trans_a) { p.row_s_row = 1; p.row_s_k = d->lda; } else { p.row_s_row = d->lda; p.row_s_k = 1; }
  if (d->trans_b) { p.col_s_row = d->ldb; p.col_s_k = 1; } else { p.col_s_row = 1; p.col_s_k = d->ldb; }
  auto vec_ok = [&](const void* base, int64_t s_row, int64_t s_k, int64_t bstride) {
    return s_k == 1 && aligned16(base) && (s_row % ce) == 0 && (d->K % ce) == 0 &&
           (batch == 1 || (bstride % ce) == 0);
  };
  // rows contiguous instead of K (a transposed A, a row-major B), 16-bit elements: vector loads
  // along the rows, transposed in registers
  auto tvec_ok = [&](const void* base, int64_t s_row, int64_t s_k, int64_t bstride, int64_t rows) {
    return es == 2 && s_row == 1 && (s_k % 8) == 0 && aligned16(base) && (rows % 8) == 0 &&
           (batch == 1 || (bstride % 8) == 0);
  };
  pl.rl = vec_ok(A, p.row_s_row, p.row_s_k, sa) ? LD_VEC
          : tvec_ok(A, p.row_s_row, p.row_s_k, sa, d->M) ? LD_TVEC : LD_STRIDED;
  pl.cl = vec_ok(B, p.col_s_row, p.col_s_k, sb) ? LD_VEC
          : tvec_ok(B, p.col_s_row, p.col_s_k, sb, d->N) ? LD_TVEC : LD_STRIDED;
  // a tvec loader runs next to vec or tvec only: with a strided partner both take element loads
  if ((pl.rl == LD_TVEC && pl.cl == LD_STRIDED) || (pl.cl == LD_TVEC && pl.rl == LD_STRIDED))
    pl.rl = pl.rl == LD_VEC ? LD_VEC : LD_STRIDED, pl.cl = pl.cl == LD_VEC ? LD_VEC : LD_STRIDED;
  p.out = (char*)C;
  p.out_si = d->ldc;
  p.out_sjo = 0;
  p.out_sj = 1;
  p.out_jmod = 0x7fffffff;
  p.out_batch = sc;
  pl.batch = batch;
  pl.fill_rows = d->M;
  pl.fill_cols = d->N;
  pl.fill_ld = d->ldc;
  rc = plan_finish(pl, op, desc_any, cfg);
  if (rc) return rc;
  // direct-to-LDS pipeline: both operands K-contiguous and 16-byte aligned, whole K steps,
  // 32-bit byte offsets inside a 256-row tile
  const int bke = 128 / es;
  const bool tn_ok = pl.rl == LD_VEC && pl.cl == LD_VEC && d->K % bke == 0 &&
                     (pl.split == 1 || split_partials_fit(pl, pl.split)) &&
                     256 * d->lda * es + 128 < ((int64_t)1 << 32) &&
                     256 * d->ldb * es + 128 < ((int64_t)1 << 32);
  const int pipe = pl.cfg.pipeline;
  // The four-wave instance of the direct-to-LDS kernel is withdrawn: its 128x128 wave tile made the
  // compiler spill over a kilobyte of registers per lane, it measured behind the eight-wave one at
  // every size, and a launch of it at 8192^3 ended in a memory fault whose cause is not found.
  if (pipe == AMOS_PIPE_DIRECT4)
    return set_error(AMOS_ERR_INFEASIBLE, "AMOS_PIPE_DIRECT4 is withdrawn (the four-wave direct-to-LDS instance "
                     "spilled registers and was slower than AMOS_PIPE_DIRECT8 everywhere): use AMOS_PIPE_DIRECT8 "
                     "or AMOS_PIPE_AUTO");
  if (pipe == AMOS_PIPE_DIRECT8) {
    const int waves = 8;
    if (!tn_ok || !pick_gemm_tn(pl.dt, pl.cfg.tile_i, pl.cfg.tile_j, waves))
      return set_error(AMOS_ERR_INFEASIBLE,
                       "direct-to-LDS pipeline needs K-contiguous 16-byte aligned operands, "
                       "K %% %d == 0, a tile of 256x256, 128x128, 128x256 or 256x128 and, for split-K, "
                       "the workspace that amos_workspace_bytes() names", bke);
    pl.tn_waves = waves;
  } else if (pipe == AMOS_PIPE_AUTO && tn_ok && pick_gemm_tn(pl.dt, pl.cfg.tile_i, pl.cfg.tile_j, 8)) {
    pl.tn_waves = 8;  // measured a few percent ahead of 4 waves on the 8192^3 fp16 GEMM
  }
  // One side of a few rows: a byte mover on the vector ALUs, under the mapper's own pipeline
  if (pipe == AMOS_PIPE_AUTO && gemm_is_skinny(*d, batch) && pl.rl == LD_VEC && pl.cl == LD_VEC) {
    pl.tn_waves = 0;
    pl.skinny = 1;
    pl.skinny_big_is_a = d->N <= kSkinnyMaxRows && (d->M > kSkinnyMaxRows || d->N <= d->M);
    SkinnyParams& q = pl.sk;
    memset(&q, 0, sizeof(q));
    q.out = (char*)C;
    q.K = (int)d->K;
    if (pl.skinny_big_is_a) {
      q.big = (const char*)A; q.small = (const char*)B;
      q.NB = (int)d->M; q.MS = (int)d->N; q.ld_big = d->lda; q.ld_small = d->ldb;
      q.out_s_big = d->ldc; q.out_s_small = 1;
    } else {
      q.big = (const char*)B; q.small = (const char*)A;
      q.NB = (int)d->N; q.MS = (int)d->M; q.ld_big = d->ldb; q.ld_small = d->lda;
      q.out_s_big = 1; q.out_s_small = d->ldc;
    }
    pl.split = 1;
    return 0;
  }
  if (pl.tn_waves) {
    GemmTnParams& q = pl.tn;
    q.a = (const char*)A; q.b = (const char*)B; q.c = (char*)C;
    q.I = p.I; q.J = p.J; q.K = p.Kred;
    q.lda = d->lda; q.ldb = d->ldb; q.ldc = d->ldc;
    q.batch_a = sa; q.batch_b = sb; q.batch_c = sc;
    q.tiles_i = p.tiles_i; q.tiles_j = p.tiles_j;
    q.kt_per_split = pl.split > 1 ? p.k_tiles_per_split : 0;
    q.split_stride = 0;
  }
  return 0;
}

static int conv_out_extent(int64_t in, int pad, int dil, int64_t k, int stride) {
  int64_t eff = (k - 1) * dil + 1;
  int64_t o = (in + 2 * (int64_t)pad - eff) / stride + 1;
  if (in + 2 * (int64_t)pad < eff) return 0;
  return (int)o;
}

static int plan_conv(Plan& pl, int op, const amos_conv_desc_t* d, const amos_kernel_config_t* cfg,
                     const void* X, const void* Wt, void* Y, void* workspace, size_t ws_bytes) {
  if (!d || !X || !Wt || !Y) return set_error(AMOS_ERR_BAD_ARG, "null pointer argument");
  amos_conv_desc_t c = *d;
  if (op == AMOS_OP_CONV2D) {
    if (c.D > 1 || c.T > 1) return set_error(AMOS_ERR_BAD_ARG, "conv2d needs D = T = 1");
    c.D = 1; c.T = 1; c.stride_d = 1; c.pad_d = 0; c.dil_d = 1;
  }
  if (c.N <= 0 || c.C <= 0 || c.D <= 0 || c.H <= 0 || c.W <= 0 || c.K <= 0 || c.T <= 0 ||
      c.R <= 0 || c.S <= 0 || c.stride_d <= 0 || c.stride_h <= 0 || c.stride_w <= 0 ||
      c.dil_d <= 0 || c.dil_h <= 0 || c.dil_w <= 0 || c.pad_d < 0 || c.pad_h < 0 || c.pad_w < 0)
    return set_error(AMOS_ERR_BAD_ARG, "conv extents, strides and dilations must be positive, pads >= 0");
  int rc = dtype_pair(c.in_dtype, c.out_dtype, &pl.dt);
  if (rc) return rc;
  const int64_t G = c.groups > 1 ? c.groups : 1;
  if (c.C % G || c.K % G)
    return set_error(AMOS_ERR_BAD_ARG, "groups (%lld) must divide C (%lld) and K (%lld)", (long long)G,
                     (long long)c.C, (long long)c.K);
  const int layout = c.layout;
  if (layout < AMOS_LAYOUT_NCHW || layout > AMOS_LAYOUT_HWNC)
    return set_error(AMOS_ERR_BAD_ARG, "unknown tensor layout %d", layout);
  if (layout != AMOS_LAYOUT_NCHW && G > 1)
    return set_error(AMOS_ERR_UNSUPPORTED, "grouped convolution exists for the NCHW layout only");
  const int64_t Cg = c.C / G, Kg = c.K / G;
  int OD = conv_out_extent(c.D, c.pad_d, c.dil_d, c.T, c.stride_d);
  int OP = conv_out_extent(c.H, c.pad_h, c.dil_h, c.R, c.stride_h);
  int OQ = conv_out_extent(c.W, c.pad_w, c.dil_w, c.S, c.stride_w);
  if (OD <= 0 || OP <= 0 || OQ <= 0)
    return set_error(AMOS_ERR_BAD_ARG, "kernel window larger than the padded input");
  int64_t J = c.N * OD * (int64_t)OP * OQ;
  int64_t Kred = Cg * c.T * c.R * c.S;
  int64_t per_image = c.C * c.D * c.H * c.W;
  if (!fits_int(J) || !fits_int(Kred) || !fits_int(per_image) || !fits_int(c.K) ||
      (layout == AMOS_LAYOUT_HWNC && !fits_int(per_image * c.N)))
    return set_error(AMOS_ERR_UNSUPPORTED, "conv extents above 2^31");
  if ((c.T - 1) * c.dil_d >= 1024 || (c.R - 1) * c.dil_h >= 1024 || (c.S - 1) * c.dil_w >= 1024)
    return set_error(AMOS_ERR_UNSUPPORTED, "dilated kernel extent above 1023");
  // A pointwise convolution runs on the GEMM kernels, vector loaders and operand copies
  // included, unless the patch-staged pipeline is asked for.
  amos_bgemm_desc_t b;
  // (... or the NCDHW-direct one, whose planner then says why it does not apply)
  if ((!cfg || (cfg->pipeline != AMOS_PIPE_PATCH && cfg->pipeline != AMOS_PIPE_PATCH8 && cfg->pipeline != AMOS_PIPE_NCHW)) &&
      conv_as_gemm(c, op, &b)) {
    b.g.out_dtype = c.out_dtype;
    const bool w_first = layout == AMOS_LAYOUT_NCHW;
    return plan_gemm(pl, AMOS_OP_BGEMM, &b, &b.g, b.batch, b.stride_a, b.stride_b, b.stride_c, cfg,
                     w_first ? Wt : X, w_first ? X : Wt, Y, workspace, ws_bytes);
  }
  // ... and with a stride where the copy that makes the activations K-contiguous pays: it picks
  // every stride-th pixel on its way
  ConvSubsample sub;
  if ((!cfg || conv_subsample_pipeline(cfg->pipeline)) && workspace && ((uintptr_t)workspace & 255) == 0 &&
      conv_as_subsampled_gemm(c, op, &b, &sub)) {
    const GemmRepack rp = gemm_repack(b.g, b.batch, !aligned16(Wt), false, true);
    if (ws_bytes >= (size_t)rp.total()) {
      b.g.out_dtype = c.out_dtype;
      claim_workspace(pl, rp.total());
      return plan_gemm_repacked(pl, AMOS_OP_BGEMM, &b.g, rp, b.batch, b.stride_a, b.stride_b, b.stride_c, cfg,
                                Wt, X, Y, workspace, &sub);
    }
  }
  // Input channels that fit one 16-byte pixel: the kernel whose reduction unit is the pixel
  ConvFewcPlan fw;
  if ((!cfg || cfg->pipeline == AMOS_PIPE_AUTO) && workspace && ((uintptr_t)workspace & 255) == 0 &&
      conv_fewc_plan(c, op, &fw) && ws_bytes >= (size_t)(fw.bytes_x + fw.bytes_w)) {
    ConvFewcParams& q = pl.fcp;
    memset(&q, 0, sizeof(q));
    q.x = (const char*)X; q.w = (const char*)Wt; q.y = (char*)Y;
    q.xt = (char*)workspace; q.wp = (char*)workspace + fw.bytes_x;
    q.N = (int)c.N; q.C = (int)c.C; q.H = (int)c.H; q.W = (int)c.W; q.K = (int)c.K; q.R = (int)c.R; q.S = (int)c.S;
    q.OP = fw.OP; q.OQ = fw.OQ;
    q.sh = c.stride_h; q.sw = c.stride_w; q.ph = c.pad_h; q.pw = c.pad_w; q.dh = c.dil_h; q.dw = c.dil_w;
    q.taps = fw.taps; q.taps_p = fw.taps_p; q.Wp = fw.Wp; q.rows_max = fw.rows_max;
    q.tiles_j = fw.tiles_j; q.k_tiles = fw.k_tiles;
    q.prep_x_blocks = (int)((c.N * c.H * c.W + 1023) / 1024);
    q.prep_w_blocks = (int)(((int64_t)fw.k_tiles * 64 * fw.taps_p + 255) / 256);
    q.patch_off = fw.patch_off; q.zero_off = fw.zero_off; q.tab_off = fw.tab_off;
    q.patch_bytes = fw.patch_bytes; q.nbuf = fw.nbuf; q.grid_x = fw.grid_x;
    q.fd_tiles_j = make_fast_div((uint32_t)fw.tiles_j);
    q.fd_oq = make_fast_div((uint32_t)fw.OQ);
    q.fd_wp = make_fast_div((uint32_t)fw.Wp);
    q.fd_hw = make_fast_div((uint32_t)(c.H * c.W));
    q.fd_taps_p = make_fast_div((uint32_t)fw.taps_p);
    q.fd_s = make_fast_div((uint32_t)c.S);
    pl.fewc = 1;
    pl.fewc_lds = fw.lds;
    memset(&pl.cfg, 0, sizeof(pl.cfg));
    if (cfg) pl.cfg = *cfg;
    memset(&pl.p, 0, sizeof(pl.p));
    pl.batch = 1;
    pl.split = 1;
    return 0;
  }
  // Few channels (no whole 128-byte chunk of them for the patch-staged pipeline): an im2col copy
  // of the activations and zero-padded weights in the workspace, then the direct-to-LDS GEMM
  ConvIm2col ic;
  if ((!cfg || conv_subsample_pipeline(cfg->pipeline)) && workspace && ((uintptr_t)workspace & 255) == 0 &&
      conv_as_im2col_gemm(c, op, &b, &ic) && ws_bytes >= (size_t)(ic.bytes_w + ic.bytes_x)) {
    char* wpad = (char*)workspace;
    char* col = wpad + ic.bytes_w;
    b.g.out_dtype = c.out_dtype;
    claim_workspace(pl, ic.bytes_w + ic.bytes_x);
    // without a tile from the caller: the convolution's own default (the best direct tile)
    amos_kernel_config_t own;
    if (!cfg || cfg->tile_i <= 0 || cfg->tile_j <= 0) {
      rc = amos_default_config(op, &c, &own);
      if (rc) return rc;
      if (cfg && cfg->split_k > 0) own.split_k = cfg->split_k;
      cfg = &own;
    }
    rc = plan_gemm(pl, AMOS_OP_BGEMM, &b, &b.g, b.batch, b.stride_a, b.stride_b, b.stride_c, cfg, wpad, col, Y);
    if (rc) return rc;
    // weights [K][Kred] -> [K][Kp], zero-filled
    pl.n_transposes = 1;
    pl.tr[0] = TransposeJob{(const char*)Wt, wpad, (int)c.K, (int)ic.Kred, ic.Kred, 0, 0, 1, (int)ic.Kp, 1};
    const int es2 = pl.dt == DT_I8 ? 1 : 2;
    Im2colParams& q = pl.icp;
    memset(&q, 0, sizeof(q));
    q.x = (const char*)X; q.dst = col;
    q.C = (int)c.C; q.D = (int)c.D; q.H = (int)c.H; q.W = (int)c.W;
    q.T = (int)c.T; q.R = (int)c.R; q.S = (int)c.S;
    q.OD = ic.OD; q.OP = ic.OP; q.OQ = ic.OQ;
    q.sd = c.stride_d; q.sh = c.stride_h; q.sw = c.stride_w;
    q.pd = c.pad_d; q.ph = c.pad_h; q.pw = c.pad_w;
    q.dd = c.dil_d; q.dh = c.dil_h; q.dw = c.dil_w;
    q.Kred = (int)ic.Kred;
    q.chunks = (int)(ic.Kp / (16 / es2));
    q.total = (unsigned)(c.N * ic.OD * (int64_t)ic.OP * ic.OQ * q.chunks);
    q.x_image = c.C * c.D * c.H * c.W;
    q.fd_chunks = make_fast_div((uint32_t)q.chunks);
    q.fd_oq = make_fast_div((uint32_t)ic.OQ);
    q.fd_op = make_fast_div((uint32_t)ic.OP);
    q.fd_od = make_fast_div((uint32_t)ic.OD);
    q.fd_trs = make_fast_div((uint32_t)(c.T * c.R * c.S));
    q.fd_rs = make_fast_div((uint32_t)(c.R * c.S));
    q.fd_s = make_fast_div((uint32_t)c.S);
    pl.im2col = 1;
    return 0;
  }
  // Depthwise (one input channel per group): no reduction but over the window, so it runs on the
  // vector ALUs as the byte mover it is, unless a matrix-core pipeline is asked for by name.
  if (conv_is_depthwise(c) && (!cfg || cfg->pipeline == AMOS_PIPE_AUTO)) {
    // (the 3x3 kinds assume one stride for rows and columns)
    const bool win3 = c.R == 3 && c.S == 3 && c.dil_h == 1 && c.dil_w == 1 && c.stride_h == c.stride_w;
    int kind = win3 && c.stride_w == 1 ? DW_3x3_S1 : win3 && c.stride_w == 2 ? DW_3x3_S2 : DW_GENERIC;
    const int64_t qgroups = (OQ + 3) / 4;
    // four output rows per lane only where that leaves 4096 waves or more (four per SIMD): below,
    // one generation of waves is all there is and its latency the whole kernel (measured: N16
    // C512 14x14 9.2 -> 8.6 us, C1024 7x7 6.7 -> 5.8 us with two rows)
    if (kind == DW_3x3_S1 && c.N * c.K * OD * ((OP + 3) / 4) * qgroups < 4096 * 64) kind = DW_3x3_S1_SMALL;
    const int64_t pgroups = (OP + dw_rows_per_lane(kind) - 1) / dw_rows_per_lane(kind);
    const int64_t items = c.N * c.K * OD * pgroups * qgroups;
    if (fits_int(items) && fits_int(c.D * c.H * c.W) && fits_int(c.T * c.R * c.S) && fits_int(c.N) && fits_int(c.K)) {
      DepthwiseParams& q = pl.dwp;
      memset(&q, 0, sizeof(q));
      q.x = (const char*)X; q.w = (const char*)Wt; q.y = (char*)Y;
      q.N = (int)c.N; q.C = (int)c.C; q.D = (int)c.D; q.H = (int)c.H; q.W = (int)c.W;
      q.K = (int)c.K; q.mult = (int)Kg;
      q.T = (int)c.T; q.R = (int)c.R; q.S = (int)c.S;
      q.OD = OD; q.OP = OP; q.OQ = OQ;
      q.sd = c.stride_d; q.sh = c.stride_h; q.sw = c.stride_w;
      q.pd = c.pad_d; q.ph = c.pad_h; q.pw = c.pad_w;
      q.dd = c.dil_d; q.dh = c.dil_h; q.dw = c.dil_w;
      q.qgroups = (int)qgroups;
      q.pgroups = (int)pgroups;
      q.items = (unsigned)items;
      q.vec_store = OQ % 4 == 0 && aligned16(Y);
      q.fd_qg = make_fast_div((uint32_t)qgroups);
      q.fd_pg = make_fast_div((uint32_t)pgroups);
      q.fd_od = make_fast_div((uint32_t)OD);
      q.fd_k = make_fast_div((uint32_t)c.K);
      q.fd_mult = make_fast_div((uint32_t)Kg);
      pl.dw = 1 + kind;
      memset(&pl.cfg, 0, sizeof(pl.cfg));
      if (cfg) pl.cfg = *cfg;
      memset(&pl.p, 0, sizeof(pl.p));
      pl.batch = 1;
      pl.split = 1;
      return 0;
    }
  }
  // The kernel that reads the activations as they are: named by the caller, or the default's
  // choice where the caller names no tile and brings the workspace for the packed weights (the
  // default's estimate is for packed weights)
  amos_kernel_config_t nchw_default;
  if ((!cfg || (cfg->pipeline == AMOS_PIPE_AUTO && (cfg->tile_i <= 0 || cfg->tile_j <= 0) && cfg->split_k <= 1)) &&
      workspace && ((uintptr_t)workspace & 255) == 0 && ws_bytes >= amos_conv_packed_weights_bytes(op, &c) &&
      ((uintptr_t)X & 7) == 0 &&   // (its 8-byte loads of the activations; other kernels take any address)
      amos_default_config(op, &c, &nchw_default) == 0 && nchw_default.pipeline == AMOS_PIPE_NCHW) {
    if (cfg) nchw_default.reserved[0] = cfg->reserved[0];
    cfg = &nchw_default;
  }
  if (cfg && cfg->pipeline == AMOS_PIPE_NCHW) {
    const int BI = cfg->tile_i > 0 ? cfg->tile_i : 64;
    const int BJ = cfg->tile_j > 0 ? cfg->tile_j : 128;
    // Weights: already packed by the caller (AMOS_FLAG_WEIGHTS_PACKED), packed into the workspace by
    // this call, or -- without a workspace -- transposed by every workgroup on its way to LDS
    const size_t packed_bytes = (size_t)(c.K * c.C * (op == AMOS_OP_CONV2D ? 1 : c.T) * 9) * (pl.dt == DT_I8 ? 1 : 2);
    // (a conv2d whose weights are 16-byte aligned can read them as they are: where the mapper's
    // model says that this costs less than the packing launch, the workspace stays unused)
    const bool t1_direct = op == AMOS_OP_CONV2D && aligned16(Wt);
    bool prefer_unpacked = false;
    if (t1_direct && !(cfg->reserved[0] & AMOS_FLAG_WEIGHTS_PACKED)) {
      Problem pb;
      if (problem_of(op, &c, &pb) == 0) conv_nchw_estimate(c, op, pb, BI, BJ, &prefer_unpacked);
    }
    const bool will_pack = (cfg->reserved[0] & AMOS_FLAG_WEIGHTS_PACKED) ||
                           (!prefer_unpacked && workspace && ws_bytes >= packed_bytes && ((uintptr_t)workspace & 255) == 0);
    // patch loads of 16 bytes where the shape and the tensor's address allow them, the weights are
    // packed and one round of the loaders covers the largest tile; else of 8
    int lb = 8;
    ConvNchwPlan np;
    if ((will_pack || t1_direct) && conv_nchw_load_bytes(c) == 16 && aligned16(X)) {
      np = conv_nchw_plan(c, op, BI, BJ, 16);
      if (!np.why && np.max_groups <= 16 * nchw_loader_waves(true, np.max_groups)) lb = 16;
    }
    if (lb == 8) np = conv_nchw_plan(c, op, BI, BJ, 8);
    const char* why = np.why;
    if (!why && ((uintptr_t)X & 7)) why = "activations not 8-byte aligned";
    if (why) return set_error(AMOS_ERR_INFEASIBLE, "NCDHW-direct convolution not applicable: %s", why);
    ConvNchwParams& q = pl.nc;
    memset(&q, 0, sizeof(q));
    q.x = (const char*)X; q.w = (const char*)Wt; q.y = (char*)Y;
    conv_nchw_shape(c, op, np.Wp, &q.s, lb);
    pl.nchw_lb = lb;
    pl.nchw_pack = 0;
    pl.nchw_w_src = Wt;
    if (cfg->reserved[0] & AMOS_FLAG_WEIGHTS_PACKED) {
      if (!aligned16(Wt)) return set_error(AMOS_ERR_BAD_ARG, "packed weights must be 16-byte aligned");
      pl.nchw_wmode = NCHW_W_PACKED;
    } else if (will_pack) {
      pl.nchw_wmode = NCHW_W_PACKED;
      pl.nchw_pack = 1;
      q.w = (const char*)workspace;
      claim_workspace(pl, (int64_t)packed_bytes);
    } else {
      pl.nchw_wmode = (np.t1 && aligned16(Wt)) ? NCHW_W_KCRS : NCHW_W_KCTRS;
    }
    const int es1 = pl.dt == DT_I8 ? 1 : 2;
    q.c_chunks = (int)(c.C * es1 / 64);
    q.macro_steps = q.s.T * q.c_chunks;
    int nsplit = cfg->split_k < 1 ? 1 : cfg->split_k;
    if (nsplit > q.macro_steps) nsplit = q.macro_steps;
    q.macro_per_split = (q.macro_steps + nsplit - 1) / nsplit;
    nsplit = (q.macro_steps + q.macro_per_split - 1) / q.macro_per_split;
    q.tiles_i = (int)((c.K + BI - 1) / BI);
    q.tiles_j = (int)((J + BJ - 1) / BJ);
    q.max_pos = np.max_pos;
    q.split_stride = 0;
    q.div_cc = nchw_make_div((uint32_t)q.c_chunks);
    q.div_odpq = nchw_make_div((uint32_t)(OD * OP * OQ));
    pl.nchw = 1;
    // rounds of the loader waves over the patch's load groups: two at most; one for int8 (sixteen
    // channels per chunk) and for 16-byte loads, which take twice the staging registers per group
    const bool packed = pl.nchw_wmode == NCHW_W_PACKED;
    pl.nchw_nwl = nchw_loader_waves(packed, np.max_groups);
    const int per_round = 16 * pl.nchw_nwl;
    pl.nchw_pt = std::max(1, (np.max_groups + per_round - 1) / per_round);
    pl.nchw_groups = np.max_groups;
    if (pl.nchw_pt > (lb == 16 || pl.dt == DT_I8 ? 1 : 2))
      return set_error(AMOS_ERR_INFEASIBLE, "NCDHW-direct convolution not applicable: input patch of a tile above the threads' load budget");
    pl.nchw_lds = np.lds;
    memset(&pl.cfg, 0, sizeof(pl.cfg));
    pl.cfg = *cfg;
    pl.cfg.tile_i = BI; pl.cfg.tile_j = BJ; pl.cfg.split_k = nsplit;
    memset(&pl.p, 0, sizeof(pl.p));
    pl.p.out_si = (int64_t)OD * OP * OQ;     // (the fused tail's operand is laid out like the output)
    pl.p.out_batch = 0;
    pl.batch = 1;
    pl.split = nsplit;                       // (partial sums in the workspace: make_plan)
    pl.fill_rows = 1;
    pl.fill_cols = c.N * c.K * (int64_t)OD * OP * OQ;
    pl.fill_ld = pl.fill_cols;
    pl.fill_once = 1;
    return 0;
  }
  const int es = pl.dt == DT_I8 ? 1 : 2;
  const int ce = 16 / es;
  IgemmParams& p = pl.p;
  memset(&p, 0, sizeof(p));
  p.I = (int)Kg;
  p.J = (int)J;
  p.Kred = (int)Kred;
  p.row_base = (const char*)Wt;
  p.row_s_row = Kred;
  p.row_s_k = 1;
  p.row_batch = Kg * Kred;                        // group g: its Kg output channels' weights ...
  p.col_batch = Cg * c.D * c.H * c.W;             // ... its Cg input channels of every image ...
  pl.rl = (aligned16(Wt) && Kred % ce == 0) ? LD_VEC : LD_STRIDED;
  p.col_base = (const char*)X;
  pl.cl = LD_CONV;
  ConvGeom& g = p.g;
  g.C = (int)Cg; g.D = (int)c.D; g.H = (int)c.H; g.W = (int)c.W;
  const int64_t dhw = c.D * c.H * c.W;
  if (layout == AMOS_LAYOUT_NCHW) {
    g.x_sn = c.C * dhw; g.x_sc = (int)dhw; g.x_sd = (int)(c.H * c.W); g.x_sh = (int)c.W; g.x_sw = 1;
    g.k_order = 0;
  } else {
    // channels innermost; weights [T][R][S][C][K]: the reduction runs tap-major, and a weight
    // row (one output channel) has its K index strided by the number of output channels
    g.x_sc = 1; g.k_order = 1;
    if (layout == AMOS_LAYOUT_NHWC) {
      g.x_sn = dhw * c.C; g.x_sd = (int)(c.H * c.W * c.C); g.x_sh = (int)(c.W * c.C); g.x_sw = (int)c.C;
    } else {
      g.x_sn = c.C; g.x_sw = (int)(c.N * c.C); g.x_sh = (int)(c.W * c.N * c.C); g.x_sd = (int)(c.H * c.W * c.N * c.C);
    }
    p.row_s_row = 1;
    p.row_s_k = c.K;
    pl.rl = LD_STRIDED;
  }
  g.T = (int)c.T; g.R = (int)c.R; g.S = (int)c.S;
  g.sd = c.stride_d; g.sh = c.stride_h; g.sw = c.stride_w;
  g.pd = c.pad_d; g.ph = c.pad_h; g.pw = c.pad_w;
  g.dd = c.dil_d; g.dh = c.dil_h; g.dw = c.dil_w;
  g.OD = OD; g.OP = OP; g.OQ = OQ;
  g.use_mask = (c.T * c.R * c.S <= 64) ? 1 : 0;
  int64_t odpq = (int64_t)OD * OP * OQ;
  p.out = (char*)Y;
  p.out_si = odpq;
  p.out_sjo = c.K * odpq;
  p.out_sj = 1;
  p.out_jmod = (int)odpq;
  if (layout == AMOS_LAYOUT_NHWC) { p.out_si = 1; p.out_sjo = odpq * c.K; p.out_sj = c.K; }
  if (layout == AMOS_LAYOUT_HWNC) { p.out_si = 1; p.out_sjo = c.K; p.out_sj = c.N * c.K; }
  p.out_batch = Kg * odpq;                        // ... its Kg channels of every output image
  pl.batch = G;
  pl.fill_rows = 1;
  pl.fill_cols = c.N * c.K * odpq;
  pl.fill_ld = pl.fill_cols;
  pl.fill_once = 1;                               // the whole output in one fill, not per group
  rc = plan_finish(pl, op, d, cfg);
  if (rc) return rc;
  p.out_vec4 = layout != AMOS_LAYOUT_NCHW && c.K % 4 == 0 && aligned16(Y) && !p.atomic_out;

  // ---- patch-staged pipeline: channels fill whole 128-byte K steps, the relaid operands fit
  // the workspace, the patch of a tile fits LDS next to a ring of weight tiles
  const int pipe = pl.cfg.pipeline;
  if (pipe == AMOS_PIPE_STAGED) return 0;
  const int BI = pl.cfg.tile_i, BJ = pl.cfg.tile_j;
  const int64_t packed = conv_packed_bytes(c, op);
  const int64_t need_ws = conv_workspace_bytes(c, op);
  const int RS = (int)(c.R * c.S);
  const int Wp = (OQ - 1) * c.stride_w + ((int)c.S - 1) * c.dil_w + 1;
  ConvPatchPlan pp = conv_patch_plan(c, op, BI, BJ, pl.cfg.split_k,
                                     pipe == AMOS_PIPE_PATCH ? 4 : pipe == AMOS_PIPE_PATCH8 ? 8 : 0,
                                     conv_unroll_level(pl.cfg.reserved[0]));
  const char* why = pp.why;
  if (!why && (!workspace || ws_bytes < (size_t)need_ws || ((uintptr_t)workspace & 255)))
    why = "workspace smaller than amos_workspace_bytes() or not 256-byte aligned";
  if (!why && layout != AMOS_LAYOUT_NCHW && !aligned16(X))
    why = "channel-innermost activations not 16-byte aligned";
  const int max_pos = pp.max_pos, nsw = pp.nsw, pls = pp.pls;
  pl.conv_occ = pp.occ;
  pl.conv_waves = pp.waves;
  pl.conv_w9 = pp.w9;
  const size_t lds = pp.lds;
  if (why) {
    if (pipe == AMOS_PIPE_PATCH || pipe == AMOS_PIPE_PATCH8)
      return set_error(AMOS_ERR_INFEASIBLE, "patch-staged convolution not applicable: %s", why);
    return 0;   // register-staged implicit GEMM handles it
  }
  pl.conv_ups = 1;
  pl.conv_lds = lds;
  claim_workspace(pl, need_ws);
  ConvFpropParams& q = pl.cv;
  memset(&q, 0, sizeof(q));
  q.x = (const char*)X; q.w = (const char*)Wt; q.y = (char*)Y;
  q.wp = (char*)workspace;
  q.zeros = (char*)workspace + packed;
  q.xt = (char*)workspace + packed + 256;
  q.steps = (char*)workspace + packed + 256 + conv_relaid_bytes(c, op);
  const int64_t Cp = conv_padded_channels(c);   // whole K steps; the relayout zero-fills [C, Cp)
  q.N = (int)c.N; q.C = (int)Cp; q.Csrc = (int)c.C; q.D = (int)c.D; q.H = (int)c.H; q.W = (int)c.W; q.K = (int)c.K;
  q.T = (int)c.T; q.R = (int)c.R; q.S = (int)c.S;
  q.sd = c.stride_d; q.sh = c.stride_h; q.sw = c.stride_w;
  q.pd = c.pad_d; q.ph = c.pad_h; q.pw = c.pad_w;
  q.dd = c.dil_d; q.dh = c.dil_h; q.dw = c.dil_w;
  q.OD = OD; q.OP = OP; q.OQ = OQ;
  q.J = (int)J;
  q.Wp = Wp;
  q.max_pos = max_pos;
  q.nsw = nsw;
  q.pls = pls;
  q.xbufs = pp.xbufs;
  q.sx_off = nsw * BI * 128;
  q.tab_off = q.sx_off + pp.xbufs * max_pos * 128;
  q.dump_off = q.tab_off + max_pos * 8;
  q.tab1_off = q.tab_off;
  if (pp.w9) {
    q.tab_off = q.sx_off + pp.tab_rel;
    q.tab1_off = q.sx_off + pp.tab1_rel;
    q.dump_off = q.sx_off + pp.dump_rel;
  }
  q.c_chunks = (int)(Cp * es / 128);
  q.macro_steps = (int)c.T * q.c_chunks;
  q.total_steps = q.macro_steps * RS;
  int split = pl.cfg.split_k < 1 ? 1 : pl.cfg.split_k;
  if (split > q.macro_steps) split = q.macro_steps;
  q.macro_per_split = (q.macro_steps + split - 1) / split;
  split = (q.macro_steps + q.macro_per_split - 1) / q.macro_per_split;
  pl.split = split;
  q.atomic_out = split > 1;
  q.tiles_i = (int)((c.K + BI - 1) / BI);
  q.tiles_j = (int)((J + BJ - 1) / BJ);
  q.zero_words = split > 1 ? c.N * c.K * odpq : 0;
  q.fd_opq = make_fast_div((uint32_t)(OP * OQ));
  q.fd_oq = make_fast_div((uint32_t)OQ);
  q.fd_od = make_fast_div((uint32_t)OD);
  q.fd_wp = make_fast_div((uint32_t)Wp);
  q.fd_odpq = make_fast_div((uint32_t)odpq);
  q.fd_cc = make_fast_div((uint32_t)q.c_chunks);
  q.fd_c = make_fast_div((uint32_t)Cp);
  const int64_t welems = c.K * c.T * c.R * c.S * Cp;
  q.fd_slab = make_fast_div((uint32_t)(Cp * c.T * c.R * c.S));
  q.prep_w_blocks = (int)((welems + 1023) / 1024 < 2048 ? (welems + 1023) / 1024 : 2048);
  q.prep_x_blocks = (int)(c.N * c.D * (((int64_t)c.H * c.W + 63) / 64) * (Cp * es / 128));
  if (layout != AMOS_LAYOUT_NCHW) q.prep_x_blocks = (int)((c.N * dhw * (Cp * es / 16) + 1023) / 1024);
  q.layout = layout;
  q.y_si = p.out_si; q.y_sn = p.out_sjo; q.y_ss = p.out_sj;
  q.y_vec4 = layout != AMOS_LAYOUT_NCHW && c.K % 4 == 0 && aligned16(Y);
  q.prep_z_blocks = q.zero_words ? (int)((q.zero_words + 4095) / 4096 < 2048 ? (q.zero_words + 4095) / 4096 : 2048) : 0;
  return 0;
}

static int make_plan_inner(Plan& pl, int op, const void* desc, const amos_kernel_config_t* cfg,
                           const void* in0, const void* in1, void* out, void* workspace, size_t ws_bytes);

static int make_plan(Plan& pl, int op, const void* desc, const amos_kernel_config_t* cfg,
                     const void* in0, const void* in1, void* out, void* workspace = nullptr,
                     size_t ws_bytes = 0) {
  pl.ws_base = (char*)workspace;
  pl.ws_bytes = ws_bytes;
  pl.part = nullptr;
  pl.part_stride = 0;
  pl.part_out = nullptr;
  pl.split = 1;
  // the pipeline's own share of the workspace: what the same configuration asks for without a split
  {
    amos_kernel_config_t c1;
    if (cfg) { c1 = *cfg; c1.split_k = 1; }
    pl.ws_own = (amos_workspace_bytes(op, desc, cfg ? &c1 : nullptr) + 255) & ~(size_t)255;
  }
  int rc = make_plan_inner(pl, op, desc, cfg, in0, in1, out, workspace, ws_bytes);
  if (rc) return rc;
  if (pl.split > 1 && split_partials_fit(pl, pl.split)) {
    pl.part = pl.ws_base + pl.ws_own;
    pl.part_stride = plan_out_footprint(pl);
    if (pl.nchw) {
      pl.part_out = pl.nc.y;
      pl.nc.y = pl.part;
      pl.nc.split_stride = pl.part_stride;
    } else if (pl.conv_ups) {
      pl.part_out = pl.cv.y;
      pl.cv.y = pl.part;
      pl.cv.split_stride = pl.part_stride;
      pl.cv.atomic_out = 0;
      pl.cv.zero_words = 0;
      pl.cv.prep_z_blocks = 0;
    } else if (pl.tn_waves) {
      pl.part_out = pl.tn.c;
      pl.tn.c = pl.part;
      pl.tn.split_stride = pl.part_stride;
    } else {
      pl.part_out = pl.p.out;
      pl.p.out = pl.part;
      pl.p.split_stride = pl.part_stride;
      pl.p.atomic_out = 0;
    }
  } else if (pl.split > 1 && (pl.tn_waves || pl.nchw)) {
    return set_error(AMOS_ERR_WORKSPACE, "split-K of this pipeline keeps partial sums in the workspace: "
                     "amos_workspace_bytes() of the same configuration says how much");
  }
  return 0;
}

static int make_plan_inner(Plan& pl, int op, const void* desc, const amos_kernel_config_t* cfg,
                           const void* in0, const void* in1, void* out, void* workspace, size_t ws_bytes) {
  pl.tn_waves = 0;
  pl.conv_ups = 0;
  pl.fill_once = 0;
  pl.n_transposes = 0;
  pl.dw = 0;
  pl.im2col = 0;
  pl.fewc = 0;
  pl.skinny = 0;
  pl.nchw = 0;
  switch (op) {
    case AMOS_OP_GEMM:
      return plan_gemm(pl, op, desc, (const amos_gemm_desc_t*)desc, 1, 0, 0, 0, cfg, in0, in1, out, workspace,
                       ws_bytes);
    case AMOS_OP_BGEMM: {
      const amos_bgemm_desc_t* b = (const amos_bgemm_desc_t*)desc;
      if (!b) return set_error(AMOS_ERR_BAD_ARG, "null descriptor");
      return plan_gemm(pl, op, desc, &b->g, b->batch, b->stride_a, b->stride_b, b->stride_c, cfg,
                       in0, in1, out, workspace, ws_bytes);
    }
    case AMOS_OP_CONV2D:
    case AMOS_OP_CONV3D:
      return plan_conv(pl, op, (const amos_conv_desc_t*)desc, cfg, in0, in1, out, workspace, ws_bytes);
  }
  return set_error(AMOS_ERR_BAD_ARG, "unknown op %d", op);
}

static int resolve(const Plan& pl, Instance** out) {
  Instance* inst = pick(pl.dt, pl.rl, pl.cl, pl.cfg.tile_i, pl.cfg.tile_j);
  if (!inst)
    return set_error(AMOS_ERR_INFEASIBLE, "no kernel instance with block tile %dx%d",
                     pl.cfg.tile_i, pl.cfg.tile_j);
  *out = inst;
  return 0;
}

static int launch_tn(const Plan& pl, hipStream_t stream) {
  TnInstance* inst = pick_gemm_tn(pl.dt, pl.cfg.tile_i, pl.cfg.tile_j, pl.tn_waves);
  if (!inst) return set_error(AMOS_ERR_INFEASIBLE, "no direct-to-LDS instance");
  hipError_t attr_err = hipSuccess;
  std::call_once(inst->once, [&] {
    attr_err = hipFuncSetAttribute((const void*)inst->fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)inst->lds);
    // The kernel decides that a direct-to-LDS tile has landed by counting its own outstanding
    // vector-memory operations (s_waitcnt vmcnt(n)); register spills are vector-memory operations
    // too, so an instance the compiler gave scratch memory would wait on the wrong ones.
    hipFuncAttributes fa;
    if (attr_err == hipSuccess) attr_err = hipFuncGetAttributes(&fa, (const void*)inst->fn);
    if (attr_err == hipSuccess) inst->scratch_bytes = (int)fa.localSizeBytes;
  });
  if (attr_err != hipSuccess)
    return set_error(AMOS_ERR_HIP, "hipFuncSetAttribute(%s): %s", inst->name,
                     hipGetErrorString(attr_err));
  if (inst->scratch_bytes)
    return set_error(AMOS_ERR_INFEASIBLE, "%s was built with %d bytes of scratch memory per lane (register "
                     "spills), which its wait counts do not allow for", inst->name, inst->scratch_bytes);
  dim3 grid((unsigned)(pl.tn.tiles_i * pl.tn.tiles_j), (unsigned)pl.split, (unsigned)pl.batch);
  hipLaunchKernelGGL(inst->fn, grid, dim3(inst->threads), inst->lds, stream, pl.tn);
  HIP_TRY(hipGetLastError());
  return 0;
}

static ConvInstance* pick_conv(int dt, int ti, int tj, int waves, int pls, int occ, int w9) {
  if (dt == DT_F16) return pick_conv_f16(ti, tj, waves, pls, occ, w9);
  if (dt == DT_BF16) return pick_conv_bf16(ti, tj, waves, pls, occ, w9);
  return pick_conv_i8(ti, tj, waves, pls, occ, w9);
}

static int launch_conv(const Plan& pl, hipStream_t stream) {
  ConvInstance* inst = pick_conv(pl.dt, pl.cfg.tile_i, pl.cfg.tile_j, pl.conv_waves, pl.cv.pls, pl.conv_occ, pl.conv_w9);
  if (!inst) return set_error(AMOS_ERR_INFEASIBLE, "no patch-staged convolution instance");
  hipError_t attr_err = hipSuccess;
  std::call_once(inst->once, [&] {
    attr_err = hipFuncSetAttribute((const void*)inst->fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   160 * 1024 - 512);
    // the kernel addresses its dynamic LDS from byte 0
    hipFuncAttributes fa;
    if (attr_err == hipSuccess) attr_err = hipFuncGetAttributes(&fa, (const void*)inst->fn);
    if (attr_err == hipSuccess && fa.sharedSizeBytes != 0) inst->static_lds = (int)fa.sharedSizeBytes;
  });
  if (attr_err != hipSuccess)
    return set_error(AMOS_ERR_HIP, "hipFuncSetAttribute(%s): %s", inst->name,
                     hipGetErrorString(attr_err));
  if (inst->static_lds)
    return set_error(AMOS_ERR_HIP, "%s was built with %d bytes of static LDS", inst->name, inst->static_lds);
  const ConvFpropParams& q = pl.cv;
  launch_conv_prepare(pl.dt == DT_I8 ? 1 : 2, q, stream);
  dim3 grid((unsigned)(q.tiles_i * q.tiles_j), (unsigned)pl.split, 1);
  // blocks that walk their tiles: one per compute unit, tiles blockIdx.x, + gridDim.x, ...
  if (pl.conv_w9 == 2 && grid.x > (unsigned)device_compute_units()) grid.x = (unsigned)device_compute_units();
  hipLaunchKernelGGL(inst->fn, grid, dim3(inst->threads), pl.conv_lds, stream, q);
  HIP_TRY(hipGetLastError());
  return 0;
}

static ConvNchwInstance* pick_conv_nchw(int dt, int ti, int tj, int wmode, int pt, int nwl, int lb) {
  if (dt == DT_F16) return pick_conv_nchw_f16(ti, tj, wmode, pt, nwl, lb);
  if (dt == DT_BF16) return pick_conv_nchw_bf16(ti, tj, wmode, pt, nwl, lb);
  return pick_conv_nchw_i8(ti, tj, wmode, pt, nwl, lb);
}

static int launch_conv_nchw(const Plan& pl, hipStream_t stream) {
  ConvNchwInstance* inst = pick_conv_nchw(pl.dt, pl.cfg.tile_i, pl.cfg.tile_j, pl.nchw_wmode, pl.nchw_pt, pl.nchw_nwl, pl.nchw_lb);
  if (!inst) return set_error(AMOS_ERR_INFEASIBLE, "no NCDHW-direct convolution instance");
  hipError_t attr_err = hipSuccess;
  std::call_once(inst->once, [&] {
    attr_err = hipFuncSetAttribute((const void*)inst->fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   160 * 1024 - 1024);
    hipFuncAttributes fa;
    if (attr_err == hipSuccess) attr_err = hipFuncGetAttributes(&fa, (const void*)inst->fn);
    if (attr_err == hipSuccess) { inst->scratch_bytes = (int)fa.localSizeBytes; inst->static_lds = (int)fa.sharedSizeBytes; }
    int blocks = 0;
    if (attr_err == hipSuccess)
      attr_err = hipOccupancyMaxActiveBlocksPerMultiprocessor(
          &blocks, (const void*)inst->fn, inst->threads,
          (size_t)2 * 9 * inst->bi * 64 + (size_t)2 * nchw_patch_buffer_bytes(inst->bj));
    inst->fits = blocks >= 1;
  });
  if (attr_err != hipSuccess)
    return set_error(AMOS_ERR_HIP, "hipFuncSetAttribute(%s): %s", inst->name, hipGetErrorString(attr_err));
  if (inst->static_lds)   // the kernel addresses its dynamic LDS from byte 0
    return set_error(AMOS_ERR_HIP, "%s was built with %d bytes of static LDS", inst->name, inst->static_lds);
  // (the loaders' staging registers are accumulation registers named in assembly: a build whose
  // registers no longer leave room for a workgroup on a compute unit cannot be launched)
  if (!inst->fits)
    return set_error(AMOS_ERR_INFEASIBLE, "%s needs more registers than a workgroup of %d threads can have",
                     inst->name, inst->threads);
  const ConvNchwParams& q = pl.nc;
  // what the kernel assumes of its launch: the tile of the instance, whole 64-byte chunks of
  // channels, a patch that fits the LDS asked for
  // ... and at least one macro step for every block along the reduction
  if (inst->bi * inst->halves != pl.cfg.tile_i || inst->bj != pl.cfg.tile_j || q.c_chunks < 1 || q.max_pos < 4 ||
      q.macro_per_split < 1 || pl.split < 1 || (int64_t)(pl.split - 1) * q.macro_per_split >= q.macro_steps ||
      q.max_pos > nchw_max_positions(inst->bj) ||
      pl.nchw_lds != (size_t)2 * 9 * inst->bi * 64 + (size_t)2 * nchw_patch_buffer_bytes(inst->bj) ||
      inst->threads != 64 * (inst->mma_waves + pl.nchw_nwl) || inst->loader_waves != pl.nchw_nwl ||
      inst->groups_per_thread != pl.nchw_pt || pl.nchw_pt * 16 * pl.nchw_nwl < pl.nchw_groups ||
      inst->load_bytes != pl.nchw_lb || (inst->load_bytes >> (pl.dt == DT_I8 ? 0 : 1)) != (1 << q.s.pg_shift) ||
      ((uintptr_t)q.x & (uintptr_t)(inst->load_bytes - 1)) ||
      ((int64_t)q.s.H * q.s.W * (pl.dt == DT_I8 ? 1 : 2)) % inst->load_bytes)
    return set_error(AMOS_ERR_BAD_ARG, "inconsistent plan for %s", inst->name);
  if (pl.nchw_pack)
    launch_conv_pack_weights(pl.dt == DT_I8 ? 1 : 2, pl.nchw_w_src, (void*)q.w, q.s.K, q.s.C, q.s.T * 9, stream);
  dim3 grid((unsigned)(q.tiles_i * q.tiles_j), (unsigned)pl.split, 1);
  hipLaunchKernelGGL(inst->fn, grid, dim3(inst->threads), pl.nchw_lds, stream, q);
  HIP_TRY(hipGetLastError());
  return 0;
}

static int launch_kernels(const Plan& pl, hipStream_t stream);

#if AMOS_SPLIT_IN_KERNEL
// Ticket counters of the in-kernel split-K reduction (SplitFinish): the library's own, one array per
// GPU, zero when the module is loaded and put back to zero by the workgroup that draws a tile's
// last ticket.  A launch takes a run of counters of its own from a rotating position, so launches
// that overlap on one GPU (other streams, other threads) do not share counters as long as fewer
// than kTicketSlots tiles are in flight at once.
constexpr int kTicketSlots = 1 << 16;
static __device__ unsigned g_split_tickets[kTicketSlots];
constexpr int kTicketMaxDevices = 64;
static unsigned* g_ticket_ptr[kTicketMaxDevices];
static std::mutex g_ticket_mutex;
static std::atomic<unsigned> g_ticket_next{0};
static unsigned* tickets_for(int64_t n) {
  if (n <= 0 || n > kTicketSlots / 8) return nullptr;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kTicketMaxDevices) return nullptr;
  unsigned* base;
  {
    std::lock_guard<std::mutex> lock(g_ticket_mutex);
    if (!g_ticket_ptr[dev] && hipGetSymbolAddress((void**)&g_ticket_ptr[dev], HIP_SYMBOL(g_split_tickets)) != hipSuccess) {
      g_ticket_ptr[dev] = nullptr;
      (void)hipGetLastError();
    }
    base = g_ticket_ptr[dev];
  }
  if (!base) return nullptr;
  for (;;) {
    const unsigned start = g_ticket_next.fetch_add((unsigned)n) % kTicketSlots;
    if (start + n <= kTicketSlots) return base + start;   // (a run that would wrap is skipped)
  }
}

// In a library built with the tails (-DAMOS_SPLIT_IN_KERNEL=1) the in-kernel reduction is still
// opt-in (environment AMOS_SPLIT_IN_KERNEL=1, read once): without it every split adds its slices
// with the launch of its own below, the path every test has run on.
static bool split_in_kernel() {
  static const bool on = [] {
    const char* v = getenv("AMOS_SPLIT_IN_KERNEL");
    return v && v[0] == '1';
  }();
  return on;
}
#endif

// the kernels of the plan; split-K with partial sums: a launch of its own adds the slices, or --
// opted in, no more tiles than there are counters, a kernel with that tail -- the last workgroup
// of every tile does
static int launch(const Plan& pl, hipStream_t stream) {
#if AMOS_SPLIT_IN_KERNEL
  if (pl.part && split_in_kernel()) {
    const bool own_tail = pl.nchw || pl.tn_waves || (pl.conv_ups && !(pl.conv_w9 == 2)) ||
                          (!pl.conv_ups && !pl.skinny && !pl.dw && !pl.fewc);
    const int64_t tiles = pl.nchw ? (int64_t)pl.nc.tiles_i * pl.nc.tiles_j
                          : pl.conv_ups ? (int64_t)pl.cv.tiles_i * pl.cv.tiles_j
                          : pl.tn_waves ? (int64_t)pl.tn.tiles_i * pl.tn.tiles_j * pl.batch
                                        : (int64_t)pl.p.tiles_i * pl.p.tiles_j * pl.batch;
    unsigned* const tk = own_tail ? tickets_for(tiles) : nullptr;
    if (tk) {
      Plan armed = pl;
      const SplitFinish fin = {tk, pl.part_out, pl.split, pl.part_stride};
      armed.p.fin = armed.tn.fin = armed.cv.fin = armed.nc.fin = fin;
      return launch_kernels(armed, stream);
    }
  }
#endif
  int rc = launch_kernels(pl, stream);
  if (rc || !pl.part) return rc;
  const int64_t n = pl.fill_rows * pl.fill_cols;
  // one launch for all batches: blockIdx.y walks them
  const int64_t nb = pl.fill_once ? 1 : pl.batch;
  const int by = (int)std::min<int64_t>(nb, 65535);
  const int blocks = (int)std::min<int64_t>((n + 255) / 256, std::max<int64_t>(8192 / by, 1));
  if (pl.dt == DT_I8)
    hipLaunchKernelGGL(reduce_splits_kernel<int>, dim3(blocks, by), dim3(256), 0, stream, (int*)pl.part_out,
                       (const int*)pl.part, pl.fill_rows, pl.fill_cols, pl.fill_ld, pl.split, pl.part_stride,
                       pl.p.out_batch, nb);
  else
    hipLaunchKernelGGL(reduce_splits_kernel<float>, dim3(blocks, by), dim3(256), 0, stream, (float*)pl.part_out,
                       (const float*)pl.part, pl.fill_rows, pl.fill_cols, pl.fill_ld, pl.split, pl.part_stride,
                       pl.p.out_batch, nb);
  HIP_TRY(hipGetLastError());
  return 0;
}

static int launch_kernels(const Plan& pl, hipStream_t stream) {
  if (pl.nchw) return launch_conv_nchw(pl, stream);
  if (pl.im2col) {
    const unsigned want = (pl.icp.total + 255u) / 256u;
    dim3 grid(want < (1u << 20) ? want : (1u << 20));
    if (pl.dt == DT_I8)
      hipLaunchKernelGGL(amos_im2col_kernel<unsigned char>, grid, dim3(256), 0, stream, pl.icp);
    else
      hipLaunchKernelGGL(amos_im2col_kernel<unsigned short>, grid, dim3(256), 0, stream, pl.icp);
  }
  for (int k = 0; k < pl.n_transposes; ++k) {
    const TransposeJob& j = pl.tr[k];
    if (j.copy) {
      const int ve = pl.dt == DT_I8 ? 8 : 4;
      const int64_t want = ((int64_t)j.rows * (j.ld_dst / ve) + 255) / 256;
      dim3 grid((unsigned)(want < 16384 ? want : 16384), 1, (unsigned)j.batch);
      if (pl.dt == DT_I8)
        hipLaunchKernelGGL(amos_padcopy_kernel<unsigned char>, grid, dim3(256), 0, stream, j);
      else
        hipLaunchKernelGGL(amos_padcopy_kernel<unsigned short>, grid, dim3(256), 0, stream, j);
      continue;
    }
    // (the tiles over the result's zero-filled K steps read past the source's rows as zeros)
    dim3 grid((unsigned)((j.cols + 63) / 64), (unsigned)((j.ld_dst + 63) / 64), (unsigned)j.batch);
    if (pl.dt == DT_I8)
      hipLaunchKernelGGL(amos_transpose_kernel<unsigned char>, grid, dim3(256), 0, stream, j);
    else
      hipLaunchKernelGGL(amos_transpose_kernel<unsigned short>, grid, dim3(256), 0, stream, j);
  }
  if (pl.fewc) {
    HIP_TRY(launch_conv_fewc(pl.dt, pl.fcp, pl.fewc_lds, stream));
    return 0;
  }
  if (pl.skinny) {
    HIP_TRY(launch_skinny_gemm(pl.dt, pl.sk, stream));
    return 0;
  }
  if (pl.dw) {
    launch_depthwise(pl.dt, pl.dw - 1, pl.dwp, stream);
    HIP_TRY(hipGetLastError());
    return 0;
  }
  if (pl.tn_waves) return launch_tn(pl, stream);
  if (pl.conv_ups) return launch_conv(pl, stream);
  Instance* inst;
  int rc = resolve(pl, &inst);
  if (rc) return rc;
  hipError_t attr_err = hipSuccess;
  std::call_once(inst->once, [&] {
    attr_err = hipFuncSetAttribute((const void*)inst->fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)inst->lds);
  });
  if (attr_err != hipSuccess)
    return set_error(AMOS_ERR_HIP, "hipFuncSetAttribute(%s, %zu B LDS): %s", inst->name, inst->lds,
                     hipGetErrorString(attr_err));
  if (pl.split > 1 && !pl.part) {
    int64_t n = pl.fill_rows * pl.fill_cols * pl.batch;
    int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
    // batched outputs are contiguous per batch only when stride_c == M*ldc; fill per batch
    for (int64_t b = 0; b < (pl.fill_once ? 1 : pl.batch); ++b) {
      char* base = pl.p.out + b * pl.p.out_batch * 4;
      if (pl.dt == DT_I8)
        hipLaunchKernelGGL(fill_zero_kernel<int>, dim3(blocks), dim3(256), 0, stream, (int*)base,
                           pl.fill_rows, pl.fill_cols, pl.fill_ld);
      else
        hipLaunchKernelGGL(fill_zero_kernel<float>, dim3(blocks), dim3(256), 0, stream,
                           (float*)base, pl.fill_rows, pl.fill_cols, pl.fill_ld);
    }
  }
  dim3 grid((unsigned)(pl.p.tiles_i * pl.p.tiles_j), (unsigned)pl.split, (unsigned)pl.batch);
  hipLaunchKernelGGL(inst->fn, grid, dim3(256), inst->lds, stream, pl.p);
  HIP_TRY(hipGetLastError());
  return 0;
}

// fused tail operation: validate it against the planned op and hand it to whichever kernel runs
static int plan_epilogue(Plan& pl, int op, const void* desc, const amos_epilogue_t* e, const void* out) {
  EpiParams ep = {nullptr, 0, 0, EPI_NONE};
  if (e && e->kind != AMOS_EPI_NONE) {
    if (e->kind != AMOS_EPI_ADD) return set_error(AMOS_ERR_UNSUPPORTED, "unknown epilogue kind %d", e->kind);
    if (!e->operand) return set_error(AMOS_ERR_BAD_ARG, "epilogue operand is null");
    const bool int_out = pl.dt == DT_I8;
    if (int_out ? e->dtype != AMOS_I32
                : (e->dtype != AMOS_F32 && e->dtype != AMOS_F16 && e->dtype != AMOS_BF16))
      return set_error(AMOS_ERR_UNSUPPORTED, "epilogue operand dtype %d does not go with the output type "
                       "(int32 output: int32; fp32 output: fp32, fp16 or bf16)", e->dtype);
    ep.ptr = (const char*)e->operand;
    ep.dt = e->dtype == AMOS_F16 ? EPI_F16 : e->dtype == AMOS_BF16 ? EPI_BF16 : EPI_OUT_TYPE;
    // split-K that accumulates into the output with atomics (no workspace for partial sums): the
    // output is zeroed and added to while the first split still reads D
    if (pl.split > 1 && !pl.part && out && ep.ptr >= (const char*)out &&
        ep.ptr < (const char*)out + plan_out_footprint(pl) * 4)
      return set_error(AMOS_ERR_BAD_ARG, "the epilogue operand aliases the output of a split-K launch without a "
                       "workspace for its partial sums (amos_workspace_bytes() of the configuration)");
    if (op == AMOS_OP_GEMM || op == AMOS_OP_BGEMM) {
      const amos_gemm_desc_t& g = op == AMOS_OP_GEMM ? *(const amos_gemm_desc_t*)desc
                                                     : ((const amos_bgemm_desc_t*)desc)->g;
      ep.si = e->ld > 0 ? e->ld : g.N;
      if (ep.si < g.N) return set_error(AMOS_ERR_BAD_ARG, "epilogue ld %lld below N", (long long)e->ld);
      ep.batch = e->stride > 0 ? e->stride : g.M * ep.si;
    } else {
      ep.si = pl.p.out_si;   // D is laid out like the output, NKDPQ
      ep.batch = pl.p.out_batch;
    }
  }
#if AMOS_SPLIT_IN_KERNEL
  // (no in-kernel reduction of a split unless the launch arms it)
  const SplitFinish no_fin = {nullptr, nullptr, 0, 0};
  pl.p.fin = no_fin; pl.tn.fin = no_fin; pl.cv.fin = no_fin; pl.nc.fin = no_fin;
#endif
  pl.p.epi = ep;
  pl.tn.epi = ep;
  pl.cv.epi = ep;
  pl.dwp.epi = ep;
  pl.fcp.epi = ep;
  pl.nc.epi = ep;
  pl.sk.epi = ep;
  pl.sk.epi_s_big = pl.skinny_big_is_a ? ep.si : 1;
  pl.sk.epi_s_small = pl.skinny_big_is_a ? 1 : ep.si;
  return 0;
}

static int run_op(int op, const void* desc, const amos_kernel_config_t* cfg, const amos_epilogue_t* epi,
                  const void* in0, const void* in1, void* out, void* workspace, size_t ws_bytes,
                  void* stream) {
  Plan pl;
  int rc = make_plan(pl, op, desc, cfg, in0, in1, out, workspace, ws_bytes);
  if (rc) return rc;
  rc = plan_epilogue(pl, op, desc, epi, out);
  if (rc) return rc;
  return launch(pl, (hipStream_t)stream);
}

}  // namespace amos

using namespace amos;

static int launch_eltwise(const amos_eltwise_desc_t* d, const void* const* inputs, void* out, hipStream_t stream) {
  if (!d || !inputs || !out) return set_error(AMOS_ERR_BAD_ARG, "null pointer argument");
  if (d->n_inputs < 1 || d->n_inputs > 4 || d->n_ops < 1 || d->n_ops > 16 || d->elems < 0)
    return set_error(AMOS_ERR_BAD_ARG, "element-wise stage with %d inputs, %d operations", d->n_inputs, d->n_ops);
  if (d->dtype != AMOS_F16 && d->dtype != AMOS_BF16 && d->dtype != AMOS_I8)
    return set_error(AMOS_ERR_UNSUPPORTED, "element-wise stage on dtype %d", d->dtype);
  EltwiseParams p;
  memset(&p, 0, sizeof(p));
  int depth = 0;
  for (int k = 0; k < d->n_ops; ++k) {     // the program must keep its stack within 1..4 and read what exists
    const int op = d->program[k] & 255, arg = d->program[k] >> 8;
    if (op == AMOS_ELT_LOAD || op == AMOS_ELT_CONST) {
      if (arg < 0 || arg >= (op == AMOS_ELT_LOAD ? d->n_inputs : 4) || ++depth > 4)
        return set_error(AMOS_ERR_BAD_ARG, "element-wise program: bad operand or stack deeper than 4 at %d", k);
    } else if (op == AMOS_ELT_ADD || op == AMOS_ELT_SUB || op == AMOS_ELT_MUL) {
      if (--depth < 1) return set_error(AMOS_ERR_BAD_ARG, "element-wise program: stack underflow at %d", k);
    } else {
      return set_error(AMOS_ERR_BAD_ARG, "element-wise program: unknown opcode %d at %d", op, k);
    }
    p.program[k] = d->program[k];
  }
  if (depth != 1) return set_error(AMOS_ERR_BAD_ARG, "element-wise program leaves %d values", depth);
  for (int k = 0; k < d->n_inputs; ++k) {
    if (!inputs[k]) return set_error(AMOS_ERR_BAD_ARG, "element-wise stage: input %d is null", k);
    p.in[k] = inputs[k];
  }
  for (int k = 0; k < 4; ++k) p.consts[k] = d->consts[k];
  p.out = out;
  p.elems = d->elems;
  p.n_ops = d->n_ops;
  if (d->elems == 0) return 0;
  const int64_t want = (d->elems + 255) / 256;
  dim3 grid((unsigned)(want < 65536 ? want : 65536));
  if (d->dtype == AMOS_F16) hipLaunchKernelGGL(amos_eltwise_kernel<DT_F16>, grid, dim3(256), 0, stream, p);
  else if (d->dtype == AMOS_BF16) hipLaunchKernelGGL(amos_eltwise_kernel<DT_BF16>, grid, dim3(256), 0, stream, p);
  else hipLaunchKernelGGL(amos_eltwise_kernel<DT_I8>, grid, dim3(256), 0, stream, p);
  HIP_TRY(hipGetLastError());
  return 0;
}

static int launch_gather(const amos_gather_desc_t* d, const void* in, const int32_t* tables, void* out,
                         hipStream_t stream) {
  if (!d || !in || !tables || !out) return set_error(AMOS_ERR_BAD_ARG, "null pointer argument");
  if (d->ndim < 1 || d->ndim > 5) return set_error(AMOS_ERR_BAD_ARG, "gather of %d dimensions", d->ndim);
  if (d->elem_bytes != 1 && d->elem_bytes != 2 && d->elem_bytes != 4)
    return set_error(AMOS_ERR_UNSUPPORTED, "gather of %d-byte elements", d->elem_bytes);
  GatherParams g;
  memset(&g, 0, sizeof(g));
  int64_t total = 1;
  for (int k = 0; k < 5; ++k) {   // right-aligned: unused leading dimensions have extent 1
    const int src = k - (5 - d->ndim);
    g.shape[k] = 1;
    g.tab[k] = 0;
    g.use[k] = 0;
    if (src >= 0) {
      if (d->out_shape[src] <= 0 || d->out_shape[src] >= (1ll << 31) || d->table_offset[src] < 0)
        return set_error(AMOS_ERR_BAD_ARG, "gather extent or table offset out of range");
      g.shape[k] = (int)d->out_shape[src];
      g.tab[k] = d->table_offset[src];
      g.use[k] = 1;
      total *= d->out_shape[src];
    }
  }
  if (total >= (1ll << 40) || d->in_elems <= 0 || d->in_elems >= (1ll << 31))
    return set_error(AMOS_ERR_UNSUPPORTED, "gather size out of range");
  g.total = total;
  g.in_elems = d->in_elems;
  const int64_t want = (total + 255) / 256;
  const int blocks = (int)(want < 65536 ? want : 65536);
  if (d->elem_bytes == 1)
    hipLaunchKernelGGL(amos_gather_kernel<unsigned char>, dim3(blocks), dim3(256), 0, stream, g,
                       (const unsigned char*)in, tables, (unsigned char*)out);
  else if (d->elem_bytes == 2)
    hipLaunchKernelGGL(amos_gather_kernel<unsigned short>, dim3(blocks), dim3(256), 0, stream, g,
                       (const unsigned short*)in, tables, (unsigned short*)out);
  else
    hipLaunchKernelGGL(amos_gather_kernel<unsigned>, dim3(blocks), dim3(256), 0, stream, g, (const unsigned*)in,
                       tables, (unsigned*)out);
  HIP_TRY(hipGetLastError());
  return 0;
}

// ---- scratch memory for the entry point that allocates nothing ---------------------------------
// One array per GPU, held from the moment the code object is loaded there until the process ends.
// In host code the array's name is only a stand-in: the address a kernel may use is the one
// hipGetSymbolAddress returns with that device current, looked up once per device and kept.
static __device__ __align__(256) unsigned char scratch[AMOS_NOALLOC_SCRATCH_BYTES];
constexpr int kScratchMaxDevices = 64;
static void* g_scratch_ptr[kScratchMaxDevices];
static std::mutex g_scratch_mutex;

static int scratch_of_current_device(void** out) {
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kScratchMaxDevices)
    return set_error(AMOS_ERR_UNSUPPORTED, "device ordinal %d above %d", dev, kScratchMaxDevices - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) return set_error(AMOS_ERR_HIP, "hipGetSymbolAddress returned a null address for the scratch array");
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

// time_evaluator's loop (src/runtime/rpc/rpc_module.cc:355-388) around a launch
template <typename Launch>
static int time_launches(Launch launch_once, hipStream_t stream, int number, int repeat, int min_repeat_ms,
                         double* out_seconds) {
  int rc = launch_once();  // warm-up
  if (rc) return rc;
  HIP_TRY(hipStreamSynchronize(stream));
  hipEvent_t e0, e1;
  HIP_TRY(hipEventCreate(&e0));
  HIP_TRY(hipEventCreate(&e1));
  long long n = number;  // like the reference, a grown `number` carries over to later repeats
  for (int r = 0; r < repeat; ++r) {
    double ms = 0.0;
    for (;;) {
      if (ms > 0.0) {
        double want = (double)min_repeat_ms / (ms / (double)n) + 1.0;
        double grown = (double)n * 1.618;
        double nn = want > grown ? want : grown;
        if (nn > 1e8) nn = 1e8;
        n = (long long)nn;
      }
      HIP_TRY(hipEventRecord(e0, stream));
      for (long long i = 0; i < n; ++i) {
        rc = launch_once();
        if (rc) return rc;
      }
      HIP_TRY(hipEventRecord(e1, stream));
      HIP_TRY(hipEventSynchronize(e1));
      float f = 0.f;
      HIP_TRY(hipEventElapsedTime(&f, e0, e1));
      ms = f;
      if (ms >= (double)min_repeat_ms || n >= 100000000LL) break;
    }
    out_seconds[r] = ms * 1e-3 / (double)n;
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return 0;
}

extern "C" {

int amos_version(void) { return AMOS_ABI_VERSION; }
const char* amos_last_error(void) { return g_err; }

int amos_device_info(amos_device_info_t* out) {
  if (!out) return set_error(AMOS_ERR_BAD_ARG, "null pointer argument");
  int dev = 0;
  HIP_TRY(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  HIP_TRY(hipGetDeviceProperties(&prop, dev));
  memset(out, 0, sizeof(*out));
  out->compute_units = prop.multiProcessorCount;
  out->wave_size = prop.warpSize;
  out->max_clock_khz = prop.clockRate;
  out->lds_bytes_per_block = (int32_t)prop.sharedMemPerBlockOptin ? (int32_t)prop.sharedMemPerBlockOptin
                                                                  : (int32_t)prop.sharedMemPerBlock;
  out->hbm_bytes = (int64_t)prop.totalGlobalMem;
  snprintf(out->arch, sizeof(out->arch), "%s", prop.gcnArchName);
  double clk = prop.clockRate * 1e3;
  out->peak_tflops_f16 = prop.multiProcessorCount * clk * 4096.0 / 1e12;
  out->peak_tops_i8 = prop.multiProcessorCount * clk * 8192.0 / 1e12;
  return 0;
}

int amos_gemm(const amos_gemm_desc_t* desc, const amos_kernel_config_t* cfg, const void* A,
              const void* B, void* C, void* workspace, size_t ws_bytes, void* stream) {
  return run_op(AMOS_OP_GEMM, desc, cfg, nullptr, A, B, C, workspace, ws_bytes, stream);
}
int amos_bgemm(const amos_bgemm_desc_t* desc, const amos_kernel_config_t* cfg, const void* A,
               const void* B, void* C, void* workspace, size_t ws_bytes, void* stream) {
  return run_op(AMOS_OP_BGEMM, desc, cfg, nullptr, A, B, C, workspace, ws_bytes, stream);
}
int amos_conv2d(const amos_conv_desc_t* desc, const amos_kernel_config_t* cfg, const void* X,
                const void* Wt, void* Y, void* workspace, size_t ws_bytes, void* stream) {
  return run_op(AMOS_OP_CONV2D, desc, cfg, nullptr, X, Wt, Y, workspace, ws_bytes, stream);
}
int amos_conv3d(const amos_conv_desc_t* desc, const amos_kernel_config_t* cfg, const void* X,
                const void* Wt, void* Y, void* workspace, size_t ws_bytes, void* stream) {
  return run_op(AMOS_OP_CONV3D, desc, cfg, nullptr, X, Wt, Y, workspace, ws_bytes, stream);
}

int amos_conv2d_noalloc(const amos_conv_desc_t* desc, const amos_kernel_config_t* cfg, const void* X,
                        const void* Wt, void* Y, void* stream) {
  if (!desc) return set_error(AMOS_ERR_BAD_ARG, "null descriptor");
  const size_t need = amos_workspace_bytes(AMOS_OP_CONV2D, desc, cfg);
  if (need > (size_t)AMOS_NOALLOC_SCRATCH_BYTES)
    return set_error(AMOS_ERR_WORKSPACE, "this convolution wants %zu bytes of scratch memory, the library's own "
                     "array holds %zu (amos_conv2d with a caller-owned workspace has no such limit)",
                     need, (size_t)AMOS_NOALLOC_SCRATCH_BYTES);
  void* ptr = nullptr;
  int rc = scratch_of_current_device(&ptr);
  if (rc) return rc;
  // every launch below is handed `ptr`; what a kernel needs cleared in it (the zero block, the step
  // table) is rewritten by the relayout launch of this very call
  return run_op(AMOS_OP_CONV2D, desc, cfg, nullptr, X, Wt, Y, ptr, (size_t)AMOS_NOALLOC_SCRATCH_BYTES, stream);
}

size_t amos_conv_packed_weights_bytes(int op, const amos_conv_desc_t* desc) {
  if (!desc || (op != AMOS_OP_CONV2D && op != AMOS_OP_CONV3D) || desc->K <= 0 || desc->C <= 0 || desc->R != 3 ||
      desc->S != 3 || desc->groups > 1 || desc->layout != AMOS_LAYOUT_NCHW)
    return 0;
  const int64_t T = op == AMOS_OP_CONV2D ? 1 : desc->T;
  const int es = desc->in_dtype == AMOS_I8 ? 1 : 2;
  if (T <= 0 || (desc->C * es) % 16) return 0;
  return (size_t)(desc->K * desc->C * T * 9 * es);
}

int amos_conv_pack_weights(int op, const amos_conv_desc_t* desc, const void* Wt, void* packed, void* stream) {
  if (!desc || !Wt || !packed) return set_error(AMOS_ERR_BAD_ARG, "null pointer argument");
  const size_t bytes = amos_conv_packed_weights_bytes(op, desc);
  if (!bytes) return set_error(AMOS_ERR_UNSUPPORTED, "packed weights exist for 3x3 windows, one group, KCTRS weights "
                                                     "with channels in whole 16-byte chunks");
  if (bytes >= ((size_t)1 << 32)) return set_error(AMOS_ERR_UNSUPPORTED, "weights of 4 GiB or more");
  if ((uintptr_t)packed & 15) return set_error(AMOS_ERR_BAD_ARG, "packed weights must be 16-byte aligned");
  const int es = desc->in_dtype == AMOS_I8 ? 1 : 2;
  launch_conv_pack_weights(es, Wt, packed, (int)desc->K, (int)desc->C, (int)((op == AMOS_OP_CONV2D ? 1 : desc->T) * 9),
                           (hipStream_t)stream);
  HIP_TRY(hipGetLastError());
  return 0;
}

int amos_run_fused(int op, const void* desc, const amos_kernel_config_t* cfg,
                   const amos_epilogue_t* epilogue, const void* in0, const void* in1, void* out,
                   void* workspace, size_t ws_bytes, void* stream) {
  if (op != AMOS_OP_GEMM && op != AMOS_OP_BGEMM && op != AMOS_OP_CONV2D && op != AMOS_OP_CONV3D)
    return set_error(AMOS_ERR_BAD_ARG, "unknown op %d", op);
  return run_op(op, desc, cfg, epilogue, in0, in1, out, workspace, ws_bytes, stream);
}

// elements from the first to the last element of the output a descriptor names, rounded up to 64
static int64_t desc_out_footprint(int op, const void* desc) {
  int64_t n = 0;
  if (op == AMOS_OP_GEMM || op == AMOS_OP_BGEMM) {
    const amos_gemm_desc_t& g = op == AMOS_OP_GEMM ? *(const amos_gemm_desc_t*)desc : ((const amos_bgemm_desc_t*)desc)->g;
    const int64_t ldc = g.ldc > 0 ? g.ldc : g.N;
    n = (g.M - 1) * ldc + g.N;
    if (op == AMOS_OP_BGEMM) {
      const amos_bgemm_desc_t* b = (const amos_bgemm_desc_t*)desc;
      n += (b->batch - 1) * (b->stride_c > 0 ? b->stride_c : g.M * ldc);
    }
  } else if (op == AMOS_OP_CONV2D || op == AMOS_OP_CONV3D) {
    const amos_conv_desc_t& c = *(const amos_conv_desc_t*)desc;
    auto ext = [](int64_t in, int64_t pad, int64_t dil, int64_t k, int64_t st) {
      const int64_t eff = (k - 1) * dil + 1;
      return in + 2 * pad < eff || st <= 0 ? (int64_t)0 : (in + 2 * pad - eff) / st + 1;
    };
    const int64_t od = op == AMOS_OP_CONV2D ? 1 : ext(c.D, c.pad_d, c.dil_d, c.T, c.stride_d);
    n = c.N * c.K * od * ext(c.H, c.pad_h, c.dil_h, c.R, c.stride_h) * ext(c.W, c.pad_w, c.dil_w, c.S, c.stride_w);
  }
  return n <= 0 ? 0 : (n + 63) & ~(int64_t)63;
}

static size_t workspace_bytes_unsplit(int op, const void* desc, const amos_kernel_config_t* cfg);

size_t amos_workspace_bytes(int op, const void* desc, const amos_kernel_config_t* cfg) {
  if (!desc) return 0;
  if (!cfg || cfg->split_k <= 1) return workspace_bytes_unsplit(op, desc, cfg);
  // split-K: behind the pipeline's own share, one slice of the output per split for the partial
  // sums (a workspace without that room: the kernels that can accumulate with atomics do so)
  amos_kernel_config_t c1 = *cfg;
  c1.split_k = 1;
  const size_t own = (workspace_bytes_unsplit(op, desc, &c1) + 255) & ~(size_t)255;
  return own + (size_t)cfg->split_k * (size_t)desc_out_footprint(op, desc) * 4;
}

static size_t workspace_bytes_unsplit(int op, const void* desc, const amos_kernel_config_t* cfg) {
  // GEMM: room for K-contiguous copies of row-contiguous operands (a transposed A, a row-major B)
  // where the problem is large enough for the copies to pay; none otherwise (split-K accumulates
  // straight into the zero-filled output).
  // conv: room for the weights repacked to K,(TRS),C when the patch-staged pipeline applies.
  if (!desc) return 0;
  if (cfg && cfg->pipeline == AMOS_PIPE_STAGED && (op == AMOS_OP_GEMM || op == AMOS_OP_BGEMM)) return 0;
  if (op == AMOS_OP_GEMM) return (size_t)gemm_repack(*(const amos_gemm_desc_t*)desc, 1, false, false).total();
  if (op == AMOS_OP_BGEMM) {
    const amos_bgemm_desc_t* b = (const amos_bgemm_desc_t*)desc;
    return (size_t)gemm_repack(b->g, b->batch, false, false).total();
  }
  if (op != AMOS_OP_CONV2D && op != AMOS_OP_CONV3D) return 0;
  if (cfg && cfg->pipeline == AMOS_PIPE_NCHW) {
    // the activations are read as they are; the weights are packed into the workspace by every
    // call unless the caller has packed them already (without a workspace every workgroup
    // transposes its own share)
    if (cfg->reserved[0] & AMOS_FLAG_WEIGHTS_PACKED) return 0;
    return amos_conv_packed_weights_bytes(op, (const amos_conv_desc_t*)desc);
  }
  const amos_conv_desc_t& c = *(const amos_conv_desc_t*)desc;
  int64_t need = conv_workspace_bytes(c, op);
  // (no pipeline named: the default may be the kernel above)
  if (!cfg || cfg->pipeline == AMOS_PIPE_AUTO) need = std::max<int64_t>(need, (int64_t)amos_conv_packed_weights_bytes(op, &c));
  // a pointwise convolution runs as a matrix product; its row-contiguous operand (NCDHW
  // activations, [C][K] weights) may want a K-contiguous copy
  amos_bgemm_desc_t b;
  if (conv_as_gemm(c, op, &b) && b.batch < 65536) {
    const int64_t t = gemm_repack(b.g, b.batch, false, false).total();
    if (t > need) need = t;
  } else if ((!cfg || conv_subsample_pipeline(cfg->pipeline)) && conv_as_subsampled_gemm(c, op, &b, nullptr)) {
    const int64_t t = gemm_repack(b.g, b.batch, false, false, true).total();
    if (t > need) need = t;
  } else {
    ConvIm2col ic;
    ConvFewcPlan fw;
    if ((!cfg || cfg->pipeline == AMOS_PIPE_AUTO) && conv_fewc_plan(c, op, &fw)) {
      if (fw.bytes_x + fw.bytes_w > need) need = fw.bytes_x + fw.bytes_w;
    } else if ((!cfg || conv_subsample_pipeline(cfg->pipeline)) && conv_as_im2col_gemm(c, op, &b, &ic) &&
               ic.bytes_w + ic.bytes_x > need) {
      need = ic.bytes_w + ic.bytes_x;
    }
  }
  return (size_t)need;
}

const char* amos_kernel_name(int op, const void* desc, const amos_kernel_config_t* cfg) {
  // pointers only matter for their alignment here; use aligned dummies
  static char dummy[16] __attribute__((aligned(16)));
  Plan pl;
  // a workspace "large enough" so that the name is the one a caller who provides
  // amos_workspace_bytes() gets
  static char dummy_ws[256] __attribute__((aligned(256)));
  if (make_plan(pl, op, desc, cfg, dummy, dummy, dummy, dummy_ws, (size_t)-1)) return nullptr;
  if (pl.nchw) {
    ConvNchwInstance* ni = pick_conv_nchw(pl.dt, pl.cfg.tile_i, pl.cfg.tile_j, pl.nchw_wmode, pl.nchw_pt, pl.nchw_nwl, pl.nchw_lb);
    return ni ? ni->name : nullptr;
  }
  if (pl.dw) return depthwise_name(pl.dt, pl.dw - 1);
  if (pl.fewc) return conv_fewc_name(pl.dt);
  if (pl.skinny) return skinny_gemm_name(pl.dt);
  if (pl.conv_ups) {
    ConvInstance* ci = pick_conv(pl.dt, pl.cfg.tile_i, pl.cfg.tile_j, pl.conv_waves, pl.cv.pls, pl.conv_occ, pl.conv_w9);
    return ci ? ci->name : nullptr;
  }
  if (pl.tn_waves) {
    TnInstance* tn = pick_gemm_tn(pl.dt, pl.cfg.tile_i, pl.cfg.tile_j, pl.tn_waves);
    return tn ? tn->name : nullptr;
  }
  Instance* inst;
  if (resolve(pl, &inst)) return nullptr;
  return inst->name;
}

int amos_gather(const amos_gather_desc_t* desc, const void* in, const int32_t* tables, void* out,
                void* stream) {
  return launch_gather(desc, in, tables, out, (hipStream_t)stream);
}

int amos_time_gather(const amos_gather_desc_t* desc, const void* in, const int32_t* tables, void* out,
                     void* stream_v, int number, int repeat, int min_repeat_ms, double* out_seconds) {
  if (!out_seconds || number < 1 || repeat < 1)
    return set_error(AMOS_ERR_BAD_ARG, "amos_time_gather needs number >= 1, repeat >= 1 and an output array");
  hipStream_t stream = (hipStream_t)stream_v;
  return time_launches([&] { return launch_gather(desc, in, tables, out, stream); }, stream, number, repeat,
                       min_repeat_ms, out_seconds);
}

int amos_eltwise(const amos_eltwise_desc_t* desc, const void* const* inputs, void* out, void* stream) {
  return launch_eltwise(desc, inputs, out, (hipStream_t)stream);
}

int amos_time_eltwise(const amos_eltwise_desc_t* desc, const void* const* inputs, void* out, void* stream_v,
                      int number, int repeat, int min_repeat_ms, double* out_seconds) {
  if (!out_seconds || number < 1 || repeat < 1)
    return set_error(AMOS_ERR_BAD_ARG, "amos_time_eltwise needs number >= 1, repeat >= 1 and an output array");
  hipStream_t stream = (hipStream_t)stream_v;
  return time_launches([&] { return launch_eltwise(desc, inputs, out, stream); }, stream, number, repeat,
                       min_repeat_ms, out_seconds);
}

int amos_time(int op, const void* desc, const amos_kernel_config_t* cfg, const void* in0,
              const void* in1, void* out, void* workspace, size_t ws_bytes, void* stream_v,
              int number, int repeat, int min_repeat_ms, double* out_seconds) {
  return amos_time_fused(op, desc, cfg, nullptr, in0, in1, out, workspace, ws_bytes, stream_v, number,
                         repeat, min_repeat_ms, out_seconds);
}

int amos_time_fused(int op, const void* desc, const amos_kernel_config_t* cfg,
                    const amos_epilogue_t* epilogue, const void* in0, const void* in1, void* out,
                    void* workspace, size_t ws_bytes, void* stream_v, int number, int repeat,
                    int min_repeat_ms, double* out_seconds) {
  if (!out_seconds || number < 1 || repeat < 1)
    return set_error(AMOS_ERR_BAD_ARG, "amos_time needs number >= 1, repeat >= 1 and an output array");
  hipStream_t stream = (hipStream_t)stream_v;
  Plan pl;
  int rc = make_plan(pl, op, desc, cfg, in0, in1, out, workspace, ws_bytes);
  if (rc) return rc;
  rc = plan_epilogue(pl, op, desc, epilogue, out);
  if (rc) return rc;
  return time_launches([&] { return launch(pl, stream); }, stream, number, repeat, min_repeat_ms, out_seconds);
}

}  // extern "C"
