// Host-side mapper shared by the runtime and the C ABI: problem extents of an
// op descriptor, resource check and per-shape kernel configuration.
#pragma once
#include <stdint.h>

#include "amos_mi355x.h"

namespace amos {

int set_error(int code, const char* fmt, ...);

// Compute units of the current device (hipGetDeviceProperties, read once per device and kept); with
// no device visible -- the mapper also runs on hosts without a GPU -- the full MI355X's 256.
int device_compute_units();

// gfx950 limits the mapper plans against (one workgroup of 4 waves per CU slot)
struct Gfx950 {
  static constexpr int kXcds = 8;
  static constexpr int kLdsBytes = 160 * 1024;      // per CU and per workgroup
  static constexpr int kVgprsPerLane = 512;         // unified VGPR+AGPR file, one wave per SIMD
  static constexpr int kWaveSize = 64;
  static constexpr double kClockGhz = 2.4;
  static constexpr double kFlopsPerClkCuF16 = 4096.0;
  static constexpr double kOpsPerClkCuI8 = 8192.0;
  static constexpr double kHbmBytesPerSec = 8e12;
};

// the implicit GEMM an op descriptor denotes: Out(i,j) = sum_k Row(i,k) Col(j,k), `batch` times
struct Problem {
  int64_t I, J, K, batch;
  int in_dtype;
  int64_t in_bytes, out_bytes;  // algorithmic bytes: every input read once, output written once
  // how the register-staged kernel would load the two operands (leading dimensions assumed
  // aligned): 0 = 16-byte vectors along K, 1 = element loads, 2 = im2col gather, 3 = vectors
  // along the rows transposed in registers
  int row_loader, col_loader;
  int direct_ok;                // the direct-to-LDS GEMM kernel applies (256x256 tile)
  // the runtime copies operands into the caller's workspace first (see gemm_repack) unless the
  // register-staged pipeline is asked for: K as the kernel then sees it, what the copies cost
  int repack;
  int64_t Kp;
  double repack_seconds;
};

// Which operands of a GEMM are copied into the workspace so that the direct-to-LDS kernel can run:
// row-contiguous ones (a transposed A, a row-major B) are transposed, K-contiguous ones whose rows
// are not whole, 16-byte aligned K steps are copied with the K steps zero-filled (a ragged K
// concerns both operands: garbage times the other side's zeros could be a NaN).
struct GemmRepack {
  bool copy_a, copy_b;
  int64_t Kp;              // K rounded up to whole K steps
  int64_t bytes_a, bytes_b;
  int64_t total() const { return bytes_a + bytes_b; }
};
// b_gathered: B is not stored as the descriptor says but gathered by the copy (see
// conv_as_subsampled_gemm): it is always copied
GemmRepack gemm_repack(const amos_gemm_desc_t& g, int64_t batch, bool a_unaligned, bool b_unaligned,
                       bool b_gathered = false);
// A 1x1(x1) window with unit stride, no padding and one group is a matrix product as it stands:
// per image Y[K][DHW] = Wt[K][C] X[C][DHW] (NCDHW, batch = N, the weights shared), or
// Y[NDHW][K] = X[NDHW][C] Wt[C][K] (channels innermost).  Fills *out and returns true for such a
// convolution (out->g is the product with A = the weights resp. the activations).
bool conv_as_gemm(const amos_conv_desc_t& c, int op, amos_bgemm_desc_t* out);
// A 2-D 1x1 window with a stride (no padding, one group, NCHW) is the same product over every
// stride-th pixel: X'[C][OP*OQ] with X'[c][p*OQ + q] = X[c][p*sh][q*sw].  The copy that makes the
// activations K-contiguous for the direct-to-LDS kernel picks those pixels on its way, so the
// route exists where that copy pays (gemm_repack's bar for element-wise loaded operands) and the
// caller provides the workspace.  Fills *out like conv_as_gemm (ldb = OP*OQ, the logical row).
struct ConvSubsample {
  int out_w;           // OQ: logical column j = p * OQ + q
  int64_t row_step;    // elements between source rows p: sh * W
  int col_step;        // elements between source columns q: sw
  int64_t chan_step;   // elements between channels (the source's leading dimension): H * W
};
bool conv_subsample_pipeline(int pipeline);   // the pipelines of a config that take this route
bool conv_as_subsampled_gemm(const amos_conv_desc_t& c, int op, amos_bgemm_desc_t* out, ConvSubsample* sub);
// A convolution on few channels (the patch-staged pipeline wants whole 128-byte chunks of
// channels; a 7x7 stem on RGB has 6 bytes) as a batched matrix product over an im2col copy of
// the activations: per image Y[K][ODPQ] = Wt'[K][Kp] Col[ODPQ][Kp]^T with Kp = C*T*R*S rounded up
// to whole K steps, both operands K-contiguous and zero-filled, so the direct-to-LDS kernel runs.
// NCDHW, one group, where the copy pays (0.2 GFLOP, 256 output channels or more) and stays under
// 1 GiB; needs the workspace.
struct ConvIm2col {
  int64_t Kred, Kp;
  int64_t bytes_w, bytes_x;     // workspace: padded weights, then the im2col matrix
  int OD, OP, OQ;
};
bool conv_as_im2col_gemm(const amos_conv_desc_t& c, int op, amos_bgemm_desc_t* out, ConvIm2col* info);
// A 2-D convolution whose input channels fit 16 bytes (an RGB stem) on the kernel that treats a
// pixel as the 16-byte unit of the reduction (conv_fewc_kernel.h): NCHW, one group, from 0.1 GFLOP
// on, where a workgroup's weights and input patch fit LDS; needs the workspace.
struct ConvFewcPlan {
  int taps, taps_p, Wp, rows_max, tiles_j, k_tiles, OP, OQ;
  int patch_off, zero_off, tab_off, patch_bytes, nbuf, grid_x;
  size_t lds;
  int64_t bytes_x, bytes_w;    // workspace: pixel-major activations, then the packed weights
};
bool conv_fewc_plan(const amos_conv_desc_t& c, int op, ConvFewcPlan* out);
// A single GEMM with at most 8 rows on one side, both operands K-contiguous in whole 16-byte
// chunks, the skinny side (rows rounded up to a power of two) within 16 KB of LDS: runs on the
// vector ALUs (skinny_gemm_kernel.h) unless a matrix-core pipeline is named.  The limits are where
// it stopped winning against the split-K matrix-core kernel when timed: every row of the skinny
// side costs a pass of LDS reads and packed dot products over the big operand's chunk (at 16
// rows that rate is below the matrix cores'), and past 16 KB too few workgroups fit on a CU to
// hide the loads' latency.
constexpr int kSkinnyMaxRows = 8;
constexpr int64_t kSkinnyMaxLds = 16 * 1024;
bool gemm_is_skinny(const amos_gemm_desc_t& g, int64_t batch);
// a one-column row-major B ([K][1], ldb 1) is the same memory as a one-row column-major one
// ([1][K]); likewise a one-row transposed A: the descriptor with those spelled K-contiguous
amos_gemm_desc_t gemm_normalized(const amos_gemm_desc_t& g);
// groups == input channels (NCDHW): runs on the vector ALUs unless a matrix-core pipeline is named
bool conv_is_depthwise(const amos_conv_desc_t& c);

int problem_of(int op, const void* desc, Problem* out);

// ---- patch-staged convolution: what one block needs, and whether it can run -------------------
constexpr int kConvMaxSegHost = 4;
struct ConvPatchPlan {
  const char* why;   // nullptr = applicable, else the reason it is not
  int max_pos;       // LDS positions per patch buffer (multiple of 64)
  int max_seg;       // image slices a tile may touch
  int nsw;           // weight ring stages
  int pls;           // patch copies per wave per K step: 0 (single macro step), 2 or 4
  int xbufs;         // patch buffers (1 when a block runs a single macro step)
  int occ;           // workgroups per CU the instance is built for (2 when LDS and registers allow)
  int waves;         // waves per workgroup: 4 or 8
  int w9;            // 1: the instance with the nine taps of a 3x3 window unrolled; 2: that
                     // instance with blocks that walk several tiles
  size_t lds;        // dynamic LDS bytes of the block
  int tab_rel, tab1_rel, dump_rel;   // w9: position tables and dump line, bytes from the first patch buffer
};
int64_t conv_padded_channels(const amos_conv_desc_t& c);
int64_t conv_packed_bytes(const amos_conv_desc_t& c, int op);
int64_t conv_relaid_bytes(const amos_conv_desc_t& c, int op);
int64_t conv_workspace_bytes(const amos_conv_desc_t& c, int op);
// allow_w9: 0 = table-driven instances only, 1 = unrolled taps, 2 = unrolled taps and tile walk
ConvPatchPlan conv_patch_plan(const amos_conv_desc_t& c, int op, int BI, int BJ, int split_k, int waves,
                              int allow_w9 = 2);
int conv_unroll_level(int config_flags);

// ---- convolution read straight from NCDHW / KCTRS (conv_nchw_kernel.h): one launch, no workspace ----
// 3x3 windows, one group, NCDHW, channels in whole 64-byte chunks, channel planes (H*W elements) in
// whole 8-byte loads; block tile 64 output channels x 128 or 256 output positions.
struct ConvNchwPlan {
  const char* why;      // nullptr = applicable, else the reason it is not
  int max_pos;          // LDS positions of a patch buffer (the largest tile's, multiple of 4)
  int Wp;               // row pitch of the patch in positions
  int max_groups;       // load groups of the largest tile
  int groups_per_thread;   // (set by the launch plan: it depends on where the weights come from)
  int t1;               // conv2d: a chunk's weights are one contiguous run (needs 16-byte aligned weights)
  size_t lds;           // dynamic LDS bytes of a workgroup
};
// load_bytes: bytes of a patch load, i.e. of a load group's run of positions in one channel (8 or 16)
ConvNchwPlan conv_nchw_plan(const amos_conv_desc_t& c, int op, int BI, int BJ, int load_bytes = 8);
// the widest patch load the shape allows (16 for 16-bit types whose channel planes are whole
// 16-byte runs; the tensor itself must then be 16-byte aligned, which only the launch knows)
int conv_nchw_load_bytes(const amos_conv_desc_t& c);
// estimated seconds of a call that brings a workspace for packed weights; <= 0 where the kernel
// does not apply.  *unpacked: the call is better off reading the weights as they are (conv2d with
// 16-byte aligned weights) than packing them first
double conv_nchw_estimate(const amos_conv_desc_t& c, int op, const Problem& pb, int ti, int tj, bool* unpacked = nullptr);
// the kernel's geometry descriptor of a convolution (extents, patch pitch, dividers)
struct NchwShape;
void conv_nchw_shape(const amos_conv_desc_t& c, int op, int patch_pitch, NchwShape* out, int load_bytes = 8);

}  // namespace amos
