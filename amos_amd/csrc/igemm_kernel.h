// Implicit-GEMM kernel family for gfx950 (MI355X), 64-lane wavefronts.
//
// One kernel template covers GEMM, batched GEMM and conv2d/conv3d.  The problem
// is always   Out(i, j) = sum_k Row(i, k) * Col(j, k)
// with i on the MFMA row side, j on the MFMA column side (the lane-fast,
// hence coalesced, direction of the accumulator) and k the fused reduction:
//
//   GEMM   : i = m, j = n, Row = A, Col = B                 (C row-major)
//   conv   : i = output channel, j = (image, od, op, oq) fused, k = (c, t, r, s)
//            Row = weights KCTRS (k is contiguous there), Col = im2col view of
//            NCDHW activations computed on the fly, Out = NKDPQ
//
// It is what the reference's generated "kernel2" does (global->shared copy,
// load_matrix_sync, mma_sync chain, store_matrix_sync; reference: README.md:344-424,
// python/tvm/auto_tensorize/tensorization_phases/schedulers/cuda_v2.py:582-825)
// with the separate im2col, relayout and scatter kernels
// (reference: src/auto_tensorize/compute_transform.cc:181-293,439-497) folded
// into the loader and the epilogue.
//
// Block = 256 threads = 4 waves in a 2x2 arrangement; every wave owns TI x TJ
// MFMA 32x32 accumulator tiles, so the block tile is (64*TI) x (64*TJ).
// K advances 128 bytes per row per step (64 halves / 128 int8).  Tiles are staged
// in LDS as rows of eight 16-byte chunks with an XOR swizzle of the chunk index,
// double buffered with register prefetch of the next K step.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace amos {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

enum { DT_F16 = 0, DT_BF16 = 1, DT_I8 = 2 };
// LD_VEC: K contiguous, 16-byte loads.  LD_STRIDED: any strides, element loads.  LD_CONV: im2col
// gather.  LD_TVEC (16-bit types): ROWS contiguous (a transposed A, a row-major B): vector loads
// along the rows, transposed in registers on the way to LDS.
enum { LD_VEC = 0, LD_STRIDED = 1, LD_CONV = 2, LD_TVEC = 3 };

// v_mfma 32x32 with 32 bytes of K per row per issue.  Operand fragment layout:
// lane l holds the 16 bytes  k-bytes [16*(l/32), 16*(l/32)+16)  of row (l%32) for
// the first operand and of column (l%32) for the second; accumulator register r
// of lane l is element (i = 8*(r/4) + 4*(l/32) + r%4, j = l%32).
template <int DT>
struct Mfma;
template <>
struct Mfma<DT_F16> {
  typedef v16f acc_t;
  typedef float out_t;
  static constexpr int ES = 2;
  static __device__ __forceinline__ acc_t run(v4i a, v4i b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a),
                                                  __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
};
template <>
struct Mfma<DT_BF16> {
  typedef v16f acc_t;
  typedef float out_t;
  static constexpr int ES = 2;
  static __device__ __forceinline__ acc_t run(v4i a, v4i b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a),
                                                   __builtin_bit_cast(v8bf, b), c, 0, 0, 0);
  }
};
template <>
struct Mfma<DT_I8> {
  typedef v16i acc_t;
  typedef int out_t;
  static constexpr int ES = 1;
  static __device__ __forceinline__ acc_t run(v4i a, v4i b, acc_t c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
  }
};

// Tail operation fused into the store: out = acc + cast(D), D an operand of the output's shape
// (reference: the element-wise stage after the main op, hw_abstraction/cuda/wmma_bias.py:12-80,
// tests/python/auto_tensorize/test_compute_transform_gemm.py:7-23 "E = C + D").
enum { EPI_NONE = 0, EPI_OUT_TYPE = 1, EPI_F16 = 2, EPI_BF16 = 3 };
struct EpiParams {
  const char* ptr;     // D
  int64_t si;          // elements between output rows i in D
  int64_t batch;       // elements between batches in D
  int dt;              // EPI_*: element type of D (EPI_OUT_TYPE = fp32 / int32 like the output)
};
template <typename out_t>
__device__ __forceinline__ out_t epi_value(const EpiParams& e, int64_t idx);
template <>
__device__ __forceinline__ float epi_value<float>(const EpiParams& e, int64_t idx) {
  if (e.dt == EPI_F16) return (float)((const _Float16*)e.ptr)[idx];
  if (e.dt == EPI_BF16) return __builtin_bit_cast(float, (unsigned)((const unsigned short*)e.ptr)[idx] << 16);
  return ((const float*)e.ptr)[idx];
}
template <>
__device__ __forceinline__ int epi_value<int>(const EpiParams& e, int64_t idx) {
  return ((const int*)e.ptr)[idx];
}

// (Compiled in only with -DAMOS_SPLIT_IN_KERNEL=1: the default build's kernels are, instruction for
// instruction, the ones without this tail.)
#ifndef AMOS_SPLIT_IN_KERNEL
#define AMOS_SPLIT_IN_KERNEL 0
#endif
#if AMOS_SPLIT_IN_KERNEL
// Split-K without a second launch: every split stores its partial tile into its own slice (as
// for the reduction launch), then takes a ticket of the tile; the workgroup that draws the last
// one adds the slices IN THE ORDER OF THE SPLITS -- the same bits whichever workgroup that is --
// and writes the output.  The counters are the library's own, zero between launches (the last
// arrival puts its counter back).  (The reference reduces a split inside one kernel as well,
// through shared memory: python/tvm/auto_tensorize/tensorization_phases/schedulers/cuda_split_K.py:868-914.)
struct SplitFinish {
  unsigned* tickets;     // nullptr: a launch of its own adds the slices
  char* out;             // the output proper (the kernel's own output pointer names the slices)
  int nsplit;
  int64_t slice_stride;  // elements between the slices
};
// Called by every thread of the workgroup behind its last store, `flag` a pointer to an LDS word
// nobody else uses any more -- IN THE LDS ADDRESS SPACE where it is made from a byte offset: the
// compiler folds a cast of LDS offset 0 to a generic pointer into the null pointer, and the
// access into one of global address 0.  elem(r, c) gives the element offset of row r, column c of
// the workgroup's rows x cols tile in the output (the same in every slice), or a negative value
// outside the tensor.
typedef volatile __attribute__((address_space(3))) unsigned* lds_flag_t;
template <typename T, typename Flag, typename Elem>
__device__ __forceinline__ void split_finish(const SplitFinish& f, unsigned tile_id, const T* slices, int tid, int nthreads,
                                             int rows, int cols, Flag flag, Elem elem) {
  __threadfence();   // this workgroup's slice, visible to every other one before the ticket is
  __syncthreads();
  if (tid == 0) *flag = atomicAdd(f.tickets + tile_id, 1u) == (unsigned)(f.nsplit - 1) ? 1u : 0u;
  __syncthreads();
  if (!*flag) return;
  __threadfence();   // ... and theirs to this one behind it
  T* const out = (T*)f.out;
  for (int idx = tid; idx < rows * cols; idx += nthreads) {
    const int r = idx / cols, c = idx - r * cols;
    const int64_t at = elem(r, c);
    if (at < 0) continue;
    T acc = slices[at];
    for (int sp = 1; sp < f.nsplit; ++sp) acc += slices[(int64_t)sp * f.slice_stride + at];
    out[at] = acc;
  }
  if (tid == 0) atomicExch(f.tickets + tile_id, 0u);
}
#endif

template <int N> struct NSlots { static constexpr int value = N; };

struct ConvGeom {
  int C, D, H, W;   // C = channels that are reduced over (of one group)
  int64_t x_sn;     // element strides of the activations: image, channel, depth, row, column
  int x_sc, x_sd, x_sh, x_sw;
  int k_order;      // reduction index k = c*TRS + tap (0, weights KCTRS) or tap*C + c (1, weights TRSCK)
  int T, R, S;
  int sd, sh, sw;
  int pd, ph, pw;
  int dd, dh, dw;
  int OD, OP, OQ;
  int use_mask;  // T*R*S <= 64: per-row tap validity bitmask instead of compares
};

struct IgemmParams {
  int I, J, Kred;         // extents in elements
  int k_tiles;            // ceil(Kred / elements per K step)
  int k_tiles_per_split;  // K steps one blockIdx.y handles
  int tiles_i, tiles_j;
  // row operand
  const char* row_base;
  int64_t row_s_row, row_s_k;   // element strides (LD_VEC: row_s_k == 1)
  int64_t row_batch;            // elements between batches
  // column operand
  const char* col_base;
  int64_t col_s_row, col_s_k;
  int64_t col_batch;
  ConvGeom g;                   // LD_CONV only
  // output: element (i, j) at  i*out_si + (j / out_jmod)*out_sjo + (j % out_jmod)*out_sj
  char* out;
  int64_t out_si, out_sjo, out_sj;
  int out_jmod;
  int64_t out_batch;
  int out_vec4;                 // out_si == 1, rows % 4 == 0, 16-byte aligned, no atomics: 4 rows per store
  int atomic_out;               // split-K without a workspace: accumulate into a zeroed output
  int64_t split_stride;         // split-K with one: blockIdx.y stores its partial sums at out + blockIdx.y * split_stride
  EpiParams epi;                // D is indexed like the output, with its own row stride
#if AMOS_SPLIT_IN_KERNEL
  SplitFinish fin;              // split-K with slices: the last workgroup of a tile adds them
#endif
};

__device__ __forceinline__ int lds_chunk_offset(int row, int chunk) {
  return row * 128 + ((chunk ^ ((row ^ (row >> 3)) & 7)) << 4);
}

// Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Give
// every XCD a contiguous range of logical tile ids, then walk tiles in column
// groups so that concurrently running blocks share row / column panels.
__device__ __forceinline__ void block_to_tile(int wg, int n_wg, int tiles_i, int tiles_j, int& ti,
                                              int& tj) {
  int logical = wg;
  if ((n_wg & 7) == 0) logical = (wg & 7) * (n_wg >> 3) + (wg >> 3);
  const int GROUP = 8;  // tile rows per group
  int per_group = GROUP * tiles_j;
  int gidx = logical / per_group;
  int first_i = gidx * GROUP;
  int rows_here = tiles_i - first_i < GROUP ? tiles_i - first_i : GROUP;
  int in_group = logical - gidx * per_group;
  ti = first_i + in_group % rows_here;
  tj = in_group / rows_here;
}

template <int DT, int RL, int CL, int TI, int TJ>
__global__ __launch_bounds__(256) void amos_igemm(const IgemmParams p) {
  typedef Mfma<DT> MM;
  typedef typename MM::acc_t acc_t;
  typedef typename MM::out_t out_t;
  constexpr int ES = MM::ES;
  constexpr int CE = 16 / ES;     // elements per 16-byte chunk
  constexpr int BKE = 128 / ES;   // elements of K per step
  constexpr int BI = 64 * TI, BJ = 64 * TJ;
  constexpr int NR = BI / 32, NC = BJ / 32;  // 16-byte chunks per thread per step
  static_assert(RL != LD_CONV, "the row operand is never an im2col view");

  extern __shared__ __attribute__((aligned(16))) char smem[];
  char* const sR = smem;                       // [2][BI*128]
  char* const sC = smem + 2 * BI * 128;        // [2][BJ*128]
  int2* const sT = (int2*)(smem + 2 * (BI + BJ) * 128);  // [2][BKE] (LD_CONV)

  const int t = threadIdx.x;
  const int lane = t & 63;
  const int wave = t >> 6;
  const int wi = wave >> 1, wj = wave & 1;

  int tile_i, tile_j;
  block_to_tile(blockIdx.x, gridDim.x, p.tiles_i, p.tiles_j, tile_i, tile_j);
  const int bi0 = tile_i * BI, bj0 = tile_j * BJ;
  const int kt_begin = blockIdx.y * p.k_tiles_per_split;
  int kt_end = kt_begin + p.k_tiles_per_split;
  if (kt_end > p.k_tiles) kt_end = p.k_tiles;
  const int64_t batch = blockIdx.z;

  const char* const rbase = p.row_base + batch * p.row_batch * ES;
  const char* const cbase = p.col_base + batch * p.col_batch * ES;

  // ---- per-thread load slots -------------------------------------------------
  // LD_VEC: chunk fastest across lanes (8 lanes cover one 128-byte row segment).
  // LD_STRIDED / LD_CONV: row fastest across lanes (rows are the contiguous
  // direction in memory), one fixed row per thread.
  int r_row[NR], r_chunk[NR];
#pragma unroll
  for (int u = 0; u < NR; ++u) {
    int item = t + 256 * u;
    if (RL == LD_VEC) {
      r_chunk[u] = item & 7;
      r_row[u] = item >> 3;
    } else if (RL == LD_TVEC) {     // thread = (group of NR adjacent rows, K chunk): one row per slot
      r_row[u] = (t & 31) * NR + u;
      r_chunk[u] = t >> 5;
    } else {
      r_row[u] = item % BI;
      r_chunk[u] = item / BI;
    }
  }
  int c_row[NC], c_chunk[NC];
#pragma unroll
  for (int u = 0; u < NC; ++u) {
    int item = t + 256 * u;
    if (CL == LD_VEC) {
      c_chunk[u] = item & 7;
      c_row[u] = item >> 3;
    } else if (CL == LD_TVEC) {
      c_row[u] = (t & 31) * NC + u;
      c_chunk[u] = t >> 5;
    } else {
      c_row[u] = item % BJ;
      c_chunk[u] = item / BJ;
    }
  }

  // im2col state of this thread's (single) column-operand row
  int64_t cv_base = 0;
  int cv_d0 = 0, cv_h0 = 0, cv_w0 = 0;
  unsigned long long cv_mask = 0;
  bool cv_valid = false;
  if (CL == LD_CONV) {
    int j = bj0 + c_row[0];
    cv_valid = j < p.J;
    int jj = cv_valid ? j : 0;
    int opq = p.g.OP * p.g.OQ;
    int img = jj / (p.g.OD * opq);
    int rem = jj - img * (p.g.OD * opq);
    int od = rem / opq;
    rem -= od * opq;
    int op = rem / p.g.OQ;
    int oq = rem - op * p.g.OQ;
    cv_d0 = od * p.g.sd - p.g.pd;
    cv_h0 = op * p.g.sh - p.g.ph;
    cv_w0 = oq * p.g.sw - p.g.pw;
    cv_base = (int64_t)img * p.g.x_sn + (int64_t)cv_d0 * p.g.x_sd + (int64_t)cv_h0 * p.g.x_sh +
              (int64_t)cv_w0 * p.g.x_sw;
    if (p.g.use_mask && cv_valid) {
      int tap = 0;
      for (int tt = 0; tt < p.g.T; ++tt)
        for (int rr = 0; rr < p.g.R; ++rr)
          for (int ss = 0; ss < p.g.S; ++ss, ++tap) {
            bool ok = (unsigned)(cv_d0 + tt * p.g.dd) < (unsigned)p.g.D &&
                      (unsigned)(cv_h0 + rr * p.g.dh) < (unsigned)p.g.H &&
                      (unsigned)(cv_w0 + ss * p.g.dw) < (unsigned)p.g.W;
            if (ok) cv_mask |= 1ull << tap;
          }
    }
  }

  auto build_table = [&](int kt) {
    if (CL == LD_CONV && t < BKE) {
      int k = kt * BKE + t;
      int2 e;
      if (k < p.Kred) {
        int rs = p.g.R * p.g.S;
        int trs = p.g.T * rs;
        int c, tap;
        if (p.g.k_order == 0) { c = k / trs; tap = k - c * trs; }
        else { tap = k / p.g.C; c = k - tap * p.g.C; }
        int tt = tap / rs;
        int rem = tap - tt * rs;
        int rr = rem / p.g.S;
        int ss = rem - rr * p.g.S;
        e.x = c * p.g.x_sc + tt * p.g.dd * p.g.x_sd + rr * p.g.dh * p.g.x_sh + ss * p.g.dw * p.g.x_sw;
        e.y = p.g.use_mask ? tap : ((tt * p.g.dd) << 20 | (rr * p.g.dh) << 10 | (ss * p.g.dw));
      } else {
        e.x = 0;
        e.y = p.g.use_mask ? 255 : -1;
      }
      sT[(kt & 1) * BKE + t] = e;
    }
  };

  v4i rreg[NR], creg[NC];

  auto load_elem = [&](const char* ptr, bool ok) -> unsigned {
    if (ES == 2) return ok ? (unsigned)*(const unsigned short*)ptr : 0u;
    return ok ? (unsigned)*(const unsigned char*)ptr : 0u;
  };
  auto pack = [&](const unsigned* e) -> v4i {
    v4i v;
    if (ES == 2) {
      v.x = e[0] | (e[1] << 16);
      v.y = e[2] | (e[3] << 16);
      v.z = e[4] | (e[5] << 16);
      v.w = e[6] | (e[7] << 16);
    } else {
      v.x = e[0] | (e[1] << 8) | (e[2] << 16) | (e[3] << 24);
      v.y = e[4] | (e[5] << 8) | (e[6] << 16) | (e[7] << 24);
      v.z = e[8] | (e[9] << 8) | (e[10] << 16) | (e[11] << 24);
      v.w = e[12] | (e[13] << 8) | (e[14] << 16) | (e[15] << 24);
    }
    return v;
  };

  // LD_TVEC: the thread's N adjacent rows (2*N contiguous bytes) at 8 consecutive k -> N chunks
  // of 8 k each.  Rows come in groups that are entirely inside or outside the operand (the host
  // takes this loader only for row extents that are multiples of 8), k is checked per load.
  auto tvec_load = [&](const char* base, int64_t s_k, int row0, int rows, int k0c, v4i* dst, auto n_c) {
    constexpr int N = decltype(n_c)::value;     // 2, 4 or 8 rows per thread
    unsigned in[8][N / 2];
#pragma unroll
    for (int x = 0; x < 8; ++x) {
      const bool ok = row0 < rows && k0c + x < p.Kred;
      const char* src = base + ((int64_t)(k0c + x) * s_k + row0) * 2;
      if (N == 8) {
        v4i v = {0, 0, 0, 0};
        if (ok) v = *(const v4i*)src;
        in[x][0] = v.x; in[x][1 % (N / 2)] = v.y; in[x][2 % (N / 2)] = v.z; in[x][3 % (N / 2)] = v.w;
      } else if (N == 4) {
        int2 v = {0, 0};
        if (ok) v = *(const int2*)src;
        in[x][0] = v.x; in[x][1 % (N / 2)] = v.y;
      } else {
        in[x][0] = ok ? *(const unsigned*)src : 0u;
      }
    }
#pragma unroll
    for (int r = 0; r < N; ++r) {
      const unsigned sel = (r & 1) ? 0x07060302u : 0x05040100u;   // high / low halves of (b, a)
      v4i o;
      o.x = (int)__builtin_amdgcn_perm(in[1][r / 2], in[0][r / 2], sel);
      o.y = (int)__builtin_amdgcn_perm(in[3][r / 2], in[2][r / 2], sel);
      o.z = (int)__builtin_amdgcn_perm(in[5][r / 2], in[4][r / 2], sel);
      o.w = (int)__builtin_amdgcn_perm(in[7][r / 2], in[6][r / 2], sel);
      dst[r] = o;
    }
  };

  auto gload = [&](int kt) {
    const int k0 = kt * BKE;
    if (RL == LD_TVEC)
      tvec_load(rbase, p.row_s_k, bi0 + r_row[0], p.I, k0 + r_chunk[0] * CE, rreg, NSlots<NR>{});
    if (CL == LD_TVEC)
      tvec_load(cbase, p.col_s_k, bj0 + c_row[0], p.J, k0 + c_chunk[0] * CE, creg, NSlots<NC>{});
#pragma unroll
    for (int u = 0; u < (RL == LD_TVEC ? 0 : NR); ++u) {
      int row = bi0 + r_row[u];
      int k = k0 + r_chunk[u] * CE;
      if (RL == LD_VEC) {
        v4i v = {0, 0, 0, 0};
        if (row < p.I && k < p.Kred)
          v = *(const v4i*)(rbase + ((int64_t)row * p.row_s_row + k) * ES);
        rreg[u] = v;
      } else {
        unsigned e[CE];
        const char* base = rbase + ((int64_t)row * p.row_s_row + (int64_t)k * p.row_s_k) * ES;
#pragma unroll
        for (int x = 0; x < CE; ++x)
          e[x] = load_elem(base + (int64_t)x * p.row_s_k * ES, row < p.I && k + x < p.Kred);
        rreg[u] = pack(e);
      }
    }
#pragma unroll
    for (int u = 0; u < (CL == LD_TVEC ? 0 : NC); ++u) {
      int row = bj0 + c_row[u];
      int k = k0 + c_chunk[u] * CE;
      if (CL == LD_VEC) {
        v4i v = {0, 0, 0, 0};
        if (row < p.J && k < p.Kred)
          v = *(const v4i*)(cbase + ((int64_t)row * p.col_s_row + k) * ES);
        creg[u] = v;
      } else if (CL == LD_STRIDED) {
        unsigned e[CE];
        const char* base = cbase + ((int64_t)row * p.col_s_row + (int64_t)k * p.col_s_k) * ES;
#pragma unroll
        for (int x = 0; x < CE; ++x)
          e[x] = load_elem(base + (int64_t)x * p.col_s_k * ES, row < p.J && k + x < p.Kred);
        creg[u] = pack(e);
      } else {
        unsigned e[CE];
        const int2* tbl = sT + (kt & 1) * BKE + c_chunk[u] * CE;
        const char* base = cbase + cv_base * ES;
#pragma unroll
        for (int x = 0; x < CE; ++x) {
          int2 ent = tbl[x];
          bool ok;
          if (p.g.use_mask) {
            ok = cv_valid && ent.y < 64 && ((cv_mask >> ent.y) & 1ull);
          } else {
            ok = cv_valid && ent.y >= 0 &&
                 (unsigned)(cv_d0 + (ent.y >> 20)) < (unsigned)p.g.D &&
                 (unsigned)(cv_h0 + ((ent.y >> 10) & 1023)) < (unsigned)p.g.H &&
                 (unsigned)(cv_w0 + (ent.y & 1023)) < (unsigned)p.g.W;
          }
          e[x] = load_elem(base + (int64_t)ent.x * ES, ok);
        }
        creg[u] = pack(e);
      }
    }
  };

  auto lstore = [&](int buf) {
    char* r = sR + buf * (BI * 128);
    char* c = sC + buf * (BJ * 128);
#pragma unroll
    for (int u = 0; u < NR; ++u) *(v4i*)(r + lds_chunk_offset(r_row[u], r_chunk[u])) = rreg[u];
#pragma unroll
    for (int u = 0; u < NC; ++u) *(v4i*)(c + lds_chunk_offset(c_row[u], c_chunk[u])) = creg[u];
  };

  acc_t acc[TI][TJ];
#pragma unroll
  for (int a = 0; a < TI; ++a)
#pragma unroll
    for (int b = 0; b < TJ; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0;

  const int frag_row = lane & 31;
  const int frag_half = lane >> 5;

  auto compute = [&](int buf) {
    const char* r = sR + buf * (BI * 128);
    const char* c = sC + buf * (BJ * 128);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      v4i af[TI], bf[TJ];
#pragma unroll
      for (int a = 0; a < TI; ++a)
        af[a] = *(const v4i*)(r + lds_chunk_offset((wi * TI + a) * 32 + frag_row, ks * 2 + frag_half));
#pragma unroll
      for (int b = 0; b < TJ; ++b)
        bf[b] = *(const v4i*)(c + lds_chunk_offset((wj * TJ + b) * 32 + frag_row, ks * 2 + frag_half));
#pragma unroll
      for (int a = 0; a < TI; ++a)
#pragma unroll
        for (int b = 0; b < TJ; ++b) acc[a][b] = MM::run(af[a], bf[b], acc[a][b]);
    }
  };

  // ---- main loop ---------------------------------------------------------------
  if (kt_begin < kt_end) {
    if (CL == LD_CONV) {
      build_table(kt_begin);
      __syncthreads();
    }
    gload(kt_begin);
    if (CL == LD_CONV && kt_begin + 1 < kt_end) build_table(kt_begin + 1);
    lstore(0);
    __syncthreads();
    for (int kt = kt_begin; kt < kt_end; ++kt) {
      const int buf = (kt - kt_begin) & 1;
      const bool more = kt + 1 < kt_end;
      if (more) gload(kt + 1);
      if (CL == LD_CONV && kt + 2 < kt_end) build_table(kt + 2);
      compute(buf);
      if (more) lstore(buf ^ 1);
      __syncthreads();
    }
  }

  // ---- epilogue: accumulators straight to the final layout -----------------------
  out_t* const out = (out_t*)p.out + batch * p.out_batch + (int64_t)blockIdx.y * p.split_stride;
  const bool add_d = p.epi.dt != EPI_NONE && blockIdx.y == 0;   // one K split adds D
#pragma unroll
  for (int b = 0; b < TJ; ++b) {
    const int j = bj0 + (wj * TJ + b) * 32 + frag_row;
    if (j >= p.J) continue;
    const int jo = j / p.out_jmod;
    const int64_t coff = (int64_t)jo * p.out_sjo + (int64_t)(j - jo * p.out_jmod) * p.out_sj;
#pragma unroll
    for (int a = 0; a < TI; ++a) {
      if (add_d) {   // all sixteen loads of the tile in flight before the first addition
        out_t dv[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int i = bi0 + (wi * TI + a) * 32 + 8 * (r >> 2) + 4 * frag_half + (r & 3);
          dv[r] = epi_value<out_t>(p.epi, batch * p.epi.batch + (int64_t)(i < p.I ? i : p.I - 1) * p.epi.si + coff);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][b][r] += dv[r];
      }
      if (p.out_vec4) {   // rows (output channels) innermost
        typedef out_t out4_t __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          const int i = bi0 + (wi * TI + a) * 32 + 8 * g4 + 4 * frag_half;
          const out4_t v = {acc[a][b][4 * g4], acc[a][b][4 * g4 + 1], acc[a][b][4 * g4 + 2], acc[a][b][4 * g4 + 3]};
          if (i < p.I) *(out4_t*)(out + i + coff) = v;
        }
        continue;
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int i = bi0 + (wi * TI + a) * 32 + 8 * (r >> 2) + 4 * frag_half + (r & 3);
        if (i < p.I) {
          out_t* dst = out + (int64_t)i * p.out_si + coff;
          if (p.atomic_out)
            atomicAdd(dst, acc[a][b][r]);
          else
            *dst = acc[a][b][r];
        }
      }
    }
  }
#if AMOS_SPLIT_IN_KERNEL
  if (p.fin.tickets) {
    split_finish<out_t>(p.fin, (unsigned)(batch * gridDim.x + blockIdx.x), (const out_t*)p.out, t, 256, BI, BJ, (lds_flag_t)smem,
                        [&](int r, int c) -> int64_t {
                          const int i = bi0 + r, j = bj0 + c;
                          if (i >= p.I || j >= p.J) return -1;
                          const int jo = j / p.out_jmod;
                          return batch * p.out_batch + (int64_t)i * p.out_si + (int64_t)jo * p.out_sjo +
                                 (int64_t)(j - jo * p.out_jmod) * p.out_sj;
                        });
  }
#endif
}

template <int TI, int TJ>
constexpr size_t igemm_lds_bytes() {
  return (size_t)2 * (64 * TI + 64 * TJ) * 128 + 2 * 128 * sizeof(int2);
}

}  // namespace amos
