// Per-shape mapping decisions.  The reference spreads these over
// python/tvm/auto_tensorize/tensorization_phases/schedulers/cuda_v2.py (tile
// factors), python/tvm/auto_tensorize/search/checker.py:43-82 with
// src/auto_tensorize/utils.cc:31-57 (resource check) and a measured search
// (python/tvm/auto_tensorize/search/parameter.py:386-459).  Here the choice is
// analytical: a wave-quantisation + roofline estimate over the compiled tile
// shapes.
#include "mapper.h"

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "conv_nchw_geom.h"

namespace amos {

int device_compute_units() {
  constexpr int kMaxDevices = 64;
  static std::atomic<int> cached[kMaxDevices];   // 0 = not read yet
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();                     // no device: the host-only uses of the mapper
    return 256;
  }
  int cu = cached[dev].load(std::memory_order_relaxed);
  if (cu == 0) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) {
      (void)hipGetLastError();
      v = 256;
    }
    cached[dev].store(v, std::memory_order_relaxed);
    cu = v;
  }
  return cu;
}

static int64_t conv_out(int64_t in, int pad, int dil, int64_t k, int stride) {
  int64_t eff = (k - 1) * dil + 1;
  if (in + 2 * (int64_t)pad < eff) return 0;
  return (in + 2 * (int64_t)pad - eff) / stride + 1;
}

GemmRepack gemm_repack(const amos_gemm_desc_t& g, int64_t batch, bool a_unaligned, bool b_unaligned,
                       bool b_gathered) {
  GemmRepack r = {false, false, 0, 0, 0};
  const int es = g.in_dtype == AMOS_I8 ? 1 : 2;
  const int bke = 128 / es;
  if (g.M <= 0 || g.N <= 0 || g.K <= 0 || batch <= 0 || batch >= 65536) return r;
  const bool ragged = g.K % bke != 0;
  const bool a_bad = !g.trans_a && ((g.lda * es) % 16 != 0 || a_unaligned);
  const bool b_bad = g.trans_b && ((g.ldb * es) % 16 != 0 || b_unaligned);
  const bool copy_a = g.trans_a || ragged || a_bad, copy_b = !g.trans_b || ragged || b_bad || b_gathered;
  if (!copy_a && !copy_b) return r;
  // below ~8 GFLOP the copies cost what the faster kernel gains; ~1 GFLOP where the register-staged
  // kernel would have to load an operand element by element
  const bool vectors = es == 2 && !a_bad && !b_bad && !b_gathered && g.K % 8 == 0 &&
                       (!g.trans_a || g.M % 8 == 0) && (g.trans_b || g.N % 8 == 0);
  // (0.2 GFLOP where the copy also spares an im2col gather; ~40 GFLOP where both operands are
  // K-contiguous vectors already and only K is not whole steps: the register-staged kernel is at
  // its best there - 3000 x 1000 x 2000 fp16 measured 29.2 us on it, 37.7 us through the copies)
  const bool ragged_only = vectors && !g.trans_a && g.trans_b;
  if (2.0 * (double)g.M * (double)g.N * (double)g.K * (double)batch <
      (ragged_only ? 4e10 : vectors ? 8e9 : b_gathered ? 2e8 : 1e9))
    return r;
  r.Kp = (g.K + bke - 1) / bke * bke;
  r.copy_a = copy_a;
  r.copy_b = copy_b;
  if (copy_a) r.bytes_a = (batch * g.M * r.Kp * es + 255) / 256 * 256;
  if (copy_b) r.bytes_b = (batch * g.N * r.Kp * es + 255) / 256 * 256;
  return r;
}


amos_gemm_desc_t gemm_normalized(const amos_gemm_desc_t& gin) {
  amos_gemm_desc_t g = gin;
  if (g.N == 1 && !g.trans_b && g.ldb == 1) { g.trans_b = 1; g.ldb = g.K; }
  if (g.M == 1 && g.trans_a && g.lda == 1) { g.trans_a = 0; g.lda = g.K; }
  return g;
}

bool gemm_is_skinny(const amos_gemm_desc_t& gin, int64_t batch) {
  const amos_gemm_desc_t g = gemm_normalized(gin);
  const int es = g.in_dtype == AMOS_I8 ? 1 : 2;
  const int ce = 16 / es;
  if (batch != 1 || g.trans_a || !g.trans_b || g.M <= 0 || g.N <= 0 || g.K <= 0) return false;
  if (g.K % ce || g.lda % ce || g.ldb % ce || g.K >= (1 << 30) || g.M >= (1ll << 31) || g.N >= (1ll << 31)) return false;
  const int64_t small = std::min(g.M, g.N);
  if (small > kSkinnyMaxRows) return false;
  int msp = 1;
  while (msp < small) msp <<= 1;
  return (int64_t)msp * g.K * es <= kSkinnyMaxLds;
}

bool conv_subsample_pipeline(int pipeline) {
  return pipeline == AMOS_PIPE_AUTO || pipeline == AMOS_PIPE_DIRECT4 || pipeline == AMOS_PIPE_DIRECT8;
}

bool conv_is_depthwise(const amos_conv_desc_t& c) {
  return c.groups > 1 && c.groups == c.C && c.layout == AMOS_LAYOUT_NCHW;
}

bool conv_as_gemm(const amos_conv_desc_t& c, int op, amos_bgemm_desc_t* out) {
  const bool is2d = op == AMOS_OP_CONV2D;
  const int64_t G = c.groups > 1 ? c.groups : 1;
  if (!(is2d || (c.T == 1 && c.stride_d == 1 && c.pad_d == 0)) || c.R != 1 || c.S != 1 || c.stride_h != 1 ||
      c.stride_w != 1 || c.pad_h != 0 || c.pad_w != 0 || G != 1 || c.N <= 0)
    return false;
  const int64_t dhw = (is2d ? 1 : c.D) * c.H * c.W;
  amos_bgemm_desc_t& b = *out;
  memset(&b, 0, sizeof(b));
  b.g.in_dtype = c.in_dtype;
  b.g.out_dtype = c.out_dtype;
  b.g.K = c.C;
  if (c.layout == AMOS_LAYOUT_NCHW) {
    b.batch = c.N;
    b.g.M = c.K; b.g.N = dhw;
    b.g.lda = c.C; b.g.ldb = dhw; b.g.ldc = dhw;
    b.stride_a = 0; b.stride_b = c.C * dhw; b.stride_c = c.K * dhw;
    return true;
  }
  b.batch = 1;
  b.g.M = c.N * dhw; b.g.N = c.K;
  b.g.lda = c.C; b.g.ldb = c.K; b.g.ldc = c.K;
  b.stride_a = b.g.M * c.C; b.stride_b = c.C * c.K; b.stride_c = b.g.M * c.K;
  return true;
}

bool conv_as_subsampled_gemm(const amos_conv_desc_t& c, int op, amos_bgemm_desc_t* out, ConvSubsample* sub) {
  const bool flat = op == AMOS_OP_CONV2D || (c.D == 1 && c.T == 1 && c.pad_d == 0);
  const int64_t G = c.groups > 1 ? c.groups : 1;
  if (!flat || c.R != 1 || c.S != 1 || c.pad_h != 0 || c.pad_w != 0 || G != 1 || c.N <= 0 ||
      c.layout != AMOS_LAYOUT_NCHW || c.stride_h < 1 || c.stride_w < 1 || (c.stride_h == 1 && c.stride_w == 1) ||
      c.H <= 0 || c.W <= 0)
    return false;
  const int64_t OP = (c.H - 1) / c.stride_h + 1, OQ = (c.W - 1) / c.stride_w + 1;
  if (OP * OQ >= (1ll << 31) || c.H * c.W >= (1ll << 31)) return false;
  amos_bgemm_desc_t& b = *out;
  memset(&b, 0, sizeof(b));
  b.g.in_dtype = c.in_dtype;
  b.g.out_dtype = c.out_dtype;
  b.batch = c.N;
  b.g.M = c.K; b.g.N = OP * OQ; b.g.K = c.C;
  b.g.lda = c.C; b.g.ldb = OP * OQ; b.g.ldc = OP * OQ;
  b.stride_a = 0; b.stride_b = c.C * c.H * c.W; b.stride_c = c.K * OP * OQ;
  if (gemm_repack(b.g, b.batch, false, false, true).total() <= 0) return false;
  if (sub) {
    sub->out_w = (int)OQ;
    sub->row_step = (int64_t)c.stride_h * c.W;
    sub->col_step = c.stride_w;
    sub->chan_step = c.H * c.W;
  }
  return true;
}

bool conv_fewc_plan(const amos_conv_desc_t& c, int op, ConvFewcPlan* out) {
  const bool flat = op == AMOS_OP_CONV2D || (c.D == 1 && c.T == 1 && c.pad_d == 0);
  const int64_t G = c.groups > 1 ? c.groups : 1;
  const int es = c.in_dtype == AMOS_I8 ? 1 : 2;
  if (!flat || G != 1 || c.layout != AMOS_LAYOUT_NCHW || c.C <= 0 || c.C * es > 16 || c.K <= 0 || c.N <= 0 ||
      c.N > 65535 || c.H <= 0 || c.W <= 0 || c.R <= 0 || c.S <= 0 || c.N * c.H * c.W >= (1ll << 31))
    return false;
  const int64_t OP = conv_out(c.H, c.pad_h, c.dil_h, c.R, c.stride_h);
  const int64_t OQ = conv_out(c.W, c.pad_w, c.dil_w, c.S, c.stride_w);
  if (OP <= 0 || OQ <= 0 || OP * OQ >= (1ll << 30) || c.K * OP * OQ >= (1ll << 40)) return false;
  const int64_t taps = c.R * c.S, taps_p = (taps + 1) / 2 * 2;
  if (taps < 2 || taps_p > 512) return false;   // (a 1x1 window is a matrix product as it stands)
  if (2.0 * (double)c.N * (double)(OP * OQ) * (double)c.K * (double)(c.C * taps) < 1e8) return false;
  const int64_t k_tiles = (c.K + 63) / 64, tiles_j = (OP * OQ + 255) / 256;
  if (k_tiles > 65535 || tiles_j >= (1ll << 31)) return false;
  const int64_t Wp = c.W + 2 * (int64_t)c.pad_w;
  // the most patch rows a tile of 256 consecutive output pixels touches
  int64_t rows_max = 0;
  for (int64_t tile = 0; tile < tiles_j; ++tile) {
    const int64_t j0 = tile * 256, j1 = std::min<int64_t>(j0 + 255, OP * OQ - 1);
    const int64_t rows = (j1 / OQ - j0 / OQ) * c.stride_h + (c.R - 1) * c.dil_h + 1;
    rows_max = std::max(rows_max, rows);
    if (tile > 4096) { rows_max = std::max<int64_t>(rows_max, (255 / OQ + 1) * c.stride_h + (c.R - 1) * c.dil_h + 1); break; }
  }
  // (the patch is filled in 1 KB chunks)
  const int64_t w_bytes = 64 * taps_p * 16, patch_bytes = (rows_max * Wp * 16 + 1023) / 1024 * 1024;
  // two patch buffers where they fit: the next tile's patch travels while this one is computed
  int64_t lds = w_bytes + 2 * patch_bytes + 16 + taps_p * 4;
  int nbuf = 2;
  if (lds > 160 * 1024) { lds -= patch_bytes; nbuf = 1; }
  if (lds > 160 * 1024) return false;
  if (tiles_j * c.N >= (1ll << 31)) return false;
  // one workgroup per CU, shared between the tiles of output channels
  const int64_t per_ktile = std::max<int64_t>(1, device_compute_units() / k_tiles);
  const int64_t grid_x = std::min<int64_t>(tiles_j * c.N, per_ktile);
  if (out) {
    out->taps = (int)taps; out->taps_p = (int)taps_p; out->Wp = (int)Wp; out->rows_max = (int)rows_max;
    out->tiles_j = (int)tiles_j; out->k_tiles = (int)k_tiles; out->OP = (int)OP; out->OQ = (int)OQ;
    out->patch_off = (int)w_bytes; out->zero_off = (int)(w_bytes + nbuf * patch_bytes);
    out->tab_off = (int)(w_bytes + nbuf * patch_bytes + 16);
    out->patch_bytes = (int)patch_bytes; out->nbuf = nbuf; out->grid_x = (int)grid_x;
    out->lds = (size_t)lds;
    out->bytes_x = (c.N * c.H * c.W * 16 + 16 + 255) / 256 * 256;   // + the zero pixel
    out->bytes_w = (k_tiles * 64 * taps_p * 16 + 255) / 256 * 256;
  }
  return true;
}

bool conv_as_im2col_gemm(const amos_conv_desc_t& cin, int op, amos_bgemm_desc_t* out, ConvIm2col* info) {
  amos_conv_desc_t c = cin;
  if (op == AMOS_OP_CONV2D) { c.D = 1; c.T = 1; c.stride_d = 1; c.pad_d = 0; c.dil_d = 1; }
  const int64_t G = c.groups > 1 ? c.groups : 1;
  if (G != 1 || c.layout != AMOS_LAYOUT_NCHW || c.N <= 0 || c.N >= 65536 || c.C <= 0 || c.K <= 0) return false;
  if (conv_padded_channels(c) != 0) return false;            // the patch-staged pipeline applies
  // the copy is made once, the on-the-fly gather once per 64 output channels: measured ahead from
  // 256 output channels on (N16 3->256 7x7/2 @224: 111 us against 231 us), behind at 64-128
  if (c.K < 256) return false;
  if (c.T * c.R * c.S == 1) return false;                    // pointwise: a product as it stands
  if (conv_fewc_plan(c, op, nullptr)) return false;          // the few-channel kernel applies
  const int es = c.in_dtype == AMOS_I8 ? 1 : 2;
  const int64_t bke = 128 / es;
  const int64_t Kred = c.C * c.T * c.R * c.S;
  if (Kred > 4096) return false;
  const int64_t OD = conv_out(c.D, c.pad_d, c.dil_d, c.T, c.stride_d);
  const int64_t OP = conv_out(c.H, c.pad_h, c.dil_h, c.R, c.stride_h);
  const int64_t OQ = conv_out(c.W, c.pad_w, c.dil_w, c.S, c.stride_w);
  if (OD <= 0 || OP <= 0 || OQ <= 0) return false;
  const int64_t J = OD * OP * OQ, Kp = (Kred + bke - 1) / bke * bke;
  if (2.0 * (double)c.N * (double)J * (double)c.K * (double)Kred < 2e8) return false;
  const int64_t bytes_x = (c.N * J * Kp * es + 255) / 256 * 256;
  if (bytes_x > (1ll << 30) || c.N * J * (Kp / (16 / es)) >= (1ll << 31) || c.C * c.D * c.H * c.W >= (1ll << 31))
    return false;
  amos_bgemm_desc_t& b = *out;
  memset(&b, 0, sizeof(b));
  b.g.in_dtype = c.in_dtype;
  b.g.out_dtype = c.out_dtype;
  b.batch = c.N;
  b.g.M = c.K; b.g.N = J; b.g.K = Kp;
  b.g.trans_a = 0; b.g.trans_b = 1;
  b.g.lda = Kp; b.g.ldb = Kp; b.g.ldc = J;
  b.stride_a = 0; b.stride_b = J * Kp; b.stride_c = c.K * J;
  if (info) {
    info->Kred = Kred; info->Kp = Kp;
    info->bytes_w = (c.K * Kp * es + 255) / 256 * 256;
    info->bytes_x = bytes_x;
    info->OD = (int)OD; info->OP = (int)OP; info->OQ = (int)OQ;
  }
  return true;
}

// what the copies of gemm_repack cost: each reads and writes its operand once at about a third of
// the HBM rate (64x64 blocks through LDS), plus a launch
static void note_repack(Problem* pb, const amos_gemm_desc_t& g, int64_t batch, bool b_gathered = false) {
  const GemmRepack rp = gemm_repack(g, batch, false, false, b_gathered);
  if (rp.total() <= 0) return;
  pb->repack = 1;
  pb->Kp = rp.Kp;
  pb->repack_seconds = 2.0 * (double)rp.total() / 2.5e12 + 2.5e-6 * ((rp.copy_a ? 1 : 0) + (rp.copy_b ? 1 : 0));
}

int problem_of(int op, const void* desc, Problem* out) {
  if (!desc || !out) return set_error(AMOS_ERR_BAD_ARG, "null descriptor");
  memset(out, 0, sizeof(*out));
  auto esize = [](int dt) { return dt == AMOS_I8 ? 1 : 2; };
  switch (op) {
    case AMOS_OP_GEMM:
    case AMOS_OP_BGEMM: {
      const amos_gemm_desc_t* g;
      int64_t batch = 1;
      if (op == AMOS_OP_BGEMM) {
        const amos_bgemm_desc_t* b = (const amos_bgemm_desc_t*)desc;
        g = &b->g;
        batch = b->batch;
      } else {
        g = (const amos_gemm_desc_t*)desc;
      }
      if (g->M <= 0 || g->N <= 0 || g->K <= 0 || batch <= 0)
        return set_error(AMOS_ERR_BAD_ARG, "non-positive GEMM extent");
      const amos_gemm_desc_t norm = gemm_normalized(*g);
      if (batch == 1) g = &norm;
      out->I = g->M; out->J = g->N; out->K = g->K; out->batch = batch;
      out->in_dtype = g->in_dtype;
      {
        const int es = esize(g->in_dtype), ce = 16 / es;
        auto loader = [&](bool k_contiguous, int64_t ld, int64_t rows) {
          if (k_contiguous) return (ld % ce == 0 && g->K % ce == 0) ? 0 : 1;
          return (es == 2 && ld % 8 == 0 && rows % 8 == 0) ? 3 : 1;
        };
        out->row_loader = loader(!g->trans_a, g->lda, g->M);
        out->col_loader = loader(g->trans_b != 0, g->ldb, g->N);
        if ((out->row_loader == 3 && out->col_loader == 1) || (out->col_loader == 3 && out->row_loader == 1))
          out->row_loader = out->row_loader == 0 ? 0 : 1, out->col_loader = out->col_loader == 0 ? 0 : 1;
        out->direct_ok = out->row_loader == 0 && out->col_loader == 0 && g->K % (128 / es) == 0;
      }
      out->in_bytes = batch * (g->M * g->K + g->K * g->N) * esize(g->in_dtype);
      out->out_bytes = batch * g->M * g->N * 4;
      note_repack(out, *g, batch);
      return 0;
    }
    case AMOS_OP_CONV2D:
    case AMOS_OP_CONV3D: {
      const amos_conv_desc_t* c = (const amos_conv_desc_t*)desc;
      int64_t D = op == AMOS_OP_CONV2D ? 1 : c->D, T = op == AMOS_OP_CONV2D ? 1 : c->T;
      if (c->N <= 0 || c->C <= 0 || D <= 0 || c->H <= 0 || c->W <= 0 || c->K <= 0 || T <= 0 ||
          c->R <= 0 || c->S <= 0 || c->stride_h <= 0 || c->stride_w <= 0 || c->dil_h <= 0 ||
          c->dil_w <= 0)
        return set_error(AMOS_ERR_BAD_ARG, "non-positive conv extent");
      int64_t OD = op == AMOS_OP_CONV2D ? 1 : conv_out(D, c->pad_d, c->dil_d, T, c->stride_d);
      int64_t OP = conv_out(c->H, c->pad_h, c->dil_h, c->R, c->stride_h);
      int64_t OQ = conv_out(c->W, c->pad_w, c->dil_w, c->S, c->stride_w);
      if (OD <= 0 || OP <= 0 || OQ <= 0)
        return set_error(AMOS_ERR_BAD_ARG, "kernel window larger than the padded input");
      const int64_t G = c->groups > 1 ? c->groups : 1;
      if (c->C % G || c->K % G)
        return set_error(AMOS_ERR_BAD_ARG, "groups (%lld) must divide C and K", (long long)G);
      out->I = c->K / G;
      out->J = c->N * OD * OP * OQ;
      out->K = c->C / G * T * c->R * c->S;
      out->batch = G;
      out->in_dtype = c->in_dtype;
      out->in_bytes = (c->N * c->C * D * c->H * c->W + c->K * out->K) * esize(c->in_dtype);
      out->out_bytes = c->K * out->J * 4;
      out->row_loader = (c->layout == AMOS_LAYOUT_NCHW && out->K % (16 / esize(c->in_dtype)) == 0) ? 0 : 1;
      out->col_loader = 2;
      // a pointwise convolution runs as a (batched) matrix product: the activations' rows are the
      // contiguous direction (NCDHW), or both operands go through vector loaders
      if (T == 1 && c->R == 1 && c->S == 1 && c->stride_h == 1 && c->stride_w == 1 && c->pad_h == 0 &&
          c->pad_w == 0 && (op == AMOS_OP_CONV2D || (c->stride_d == 1 && c->pad_d == 0)) && G == 1) {
        const bool wide = esize(c->in_dtype) == 2;
        if (c->layout == AMOS_LAYOUT_NCHW) {
          out->col_loader = (wide && (D * c->H * c->W) % 8 == 0 && out->row_loader == 0) ? 3 : 1;
          if (out->col_loader == 1) out->row_loader = 1;
        } else {
          const bool vec = c->C % (16 / esize(c->in_dtype)) == 0;
          out->row_loader = (wide && c->K % 8 == 0 && vec) ? 3 : 1;
          out->col_loader = (vec && out->row_loader == 3) ? 0 : 1;
        }
        amos_bgemm_desc_t b;
        if (conv_as_gemm(*c, op, &b)) note_repack(out, b.g, b.batch);
      }
      return 0;
    }
  }
  return set_error(AMOS_ERR_BAD_ARG, "unknown op %d", op);
}

// worst case over the J tiles of the patch a block stages: LDS positions and slices touched
static void conv_patch_extent(int64_t J, int OPQ, int OQ, int BJ, int sh, int R, int dh, int Wp,
                              int* max_pos, int* max_seg) {
  *max_pos = 0;
  *max_seg = 0;
  const int64_t tiles = (J + BJ - 1) / BJ;
  // the pattern of (tile start mod OPQ) repeats after OPQ / gcd(BJ, OPQ) tiles
  int64_t a = BJ, b = OPQ;
  while (b) { int64_t r = a % b; a = b; b = r; }
  int64_t period = OPQ / a + 1;
  const int64_t scan = tiles < period ? tiles : period;
  for (int64_t tj = 0; tj <= scan; ++tj) {
    int64_t t2 = tj == scan ? tiles - 1 : tj;   // the ragged last tile too
    int64_t j0 = t2 * BJ, j1 = j0 + BJ - 1 < J - 1 ? j0 + BJ - 1 : J - 1;
    int64_t sa = j0 / OPQ, sb = j1 / OPQ;
    int pos = 0;
    for (int64_t sl = sa; sl <= sb; ++sl) {
      int64_t lo = j0 > sl * OPQ ? j0 : sl * OPQ;
      int64_t hi = j1 < (sl + 1) * OPQ - 1 ? j1 : (sl + 1) * OPQ - 1;
      int pa = (int)((lo - sl * OPQ) / OQ), pb = (int)((hi - sl * OPQ) / OQ);
      pos += ((pb - pa) * sh + (R - 1) * dh + 1) * Wp;
    }
    if (pos > *max_pos) *max_pos = pos;
    if ((int)(sb - sa + 1) > *max_seg) *max_seg = (int)(sb - sa + 1);
  }
}

// workspace of the patch-staged pipeline:
// [packed weights | 256 zero bytes | NDHWC activations | step table, 32 bytes per K step + 1]
// channels of the relaid operands: C rounded up to whole 128-byte K steps, zero-filled by the
// relayout launch, where that at most doubles the work (0: the patch-staged pipeline does not apply);
// channel-innermost layouts want whole 16-byte chunks of real channels
int64_t conv_padded_channels(const amos_conv_desc_t& c) {
  const int es = c.in_dtype == AMOS_I8 ? 1 : 2;
  const int64_t step = 128 / es;
  if (c.C <= 0) return 0;
  const int64_t cp = (c.C + step - 1) / step * step;
  if (cp == c.C) return cp;
  if (cp > 2 * c.C) return 0;
  if (c.layout != AMOS_LAYOUT_NCHW && (c.C * es) % 16 != 0) return 0;
  return cp;
}
int64_t conv_packed_bytes(const amos_conv_desc_t& c, int op) {
  int64_t T = op == AMOS_OP_CONV2D ? 1 : c.T;
  int es = c.in_dtype == AMOS_I8 ? 1 : 2;
  const int64_t cp = conv_padded_channels(c);
  if (cp == 0) return 0;
  return (c.K * T * c.R * c.S * cp * es + 255) / 256 * 256;
}
int64_t conv_relaid_bytes(const amos_conv_desc_t& c, int op) {
  int64_t D = op == AMOS_OP_CONV2D ? 1 : c.D;
  int es = c.in_dtype == AMOS_I8 ? 1 : 2;
  return (c.N * conv_padded_channels(c) * D * c.H * c.W * es + 255) / 256 * 256;
}
int64_t conv_workspace_bytes(const amos_conv_desc_t& c, int op) {
  int64_t packed = conv_packed_bytes(c, op);
  if (packed == 0 || c.groups > 1) return 0;
  int64_t T = op == AMOS_OP_CONV2D ? 1 : c.T;
  int es = c.in_dtype == AMOS_I8 ? 1 : 2;
  int64_t steps = T * c.R * c.S * (conv_padded_channels(c) * es / 128);
  return packed + 256 + conv_relaid_bytes(c, op) + (steps + 1) * 32;
}


static ConvPatchPlan conv_patch_plan_waves(const amos_conv_desc_t& cin, int op, int BI, int BJ, int split_k,
                                           int waves, int allow_w9);

// waves: 4, 8, or 0 = 8 where that applies and four waves would leave a CU with a single workgroup
// (or where the unrolled 3x3 instance applies, which exists with 8 waves)
ConvPatchPlan conv_patch_plan(const amos_conv_desc_t& c, int op, int BI, int BJ, int split_k, int waves,
                              int allow_w9) {
  if (waves == 4 || waves == 8) return conv_patch_plan_waves(c, op, BI, BJ, split_k, waves, allow_w9);
  ConvPatchPlan p8 = conv_patch_plan_waves(c, op, BI, BJ, split_k, 8, allow_w9);
  if (!p8.why && p8.w9) return p8;
  ConvPatchPlan p4 = conv_patch_plan_waves(c, op, BI, BJ, split_k, 4, allow_w9);
  if (!p4.why && p4.occ == 2) return p4;
  return p8.why ? p4 : p8;
}

static ConvPatchPlan conv_patch_plan_waves(const amos_conv_desc_t& cin, int op, int BI, int BJ, int split_k,
                                           int waves, int allow_w9) {
  ConvPatchPlan pp = {nullptr, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  pp.waves = waves;
  amos_conv_desc_t c = cin;
  if (op == AMOS_OP_CONV2D) { c.D = 1; c.T = 1; c.stride_d = 1; c.pad_d = 0; c.dil_d = 1; }
  const int es = c.in_dtype == AMOS_I8 ? 1 : 2;
  const int64_t OD = conv_out(c.D, c.pad_d, c.dil_d, c.T, c.stride_d);
  const int64_t OP = conv_out(c.H, c.pad_h, c.dil_h, c.R, c.stride_h);
  const int64_t OQ = conv_out(c.W, c.pad_w, c.dil_w, c.S, c.stride_w);
  const int64_t J = c.N * OD * OP * OQ;
  const int64_t packed = conv_packed_bytes(c, op);
  const int RS = (int)(c.R * c.S);
  const int Wp = (int)((OQ - 1) * c.stride_w + (c.S - 1) * c.dil_w + 1);
  const bool tile_ok = waves == 8 ? ((BI == 128 && (BJ == 64 || BJ == 128 || BJ == 256)) ||
                                     (BI == 64 && BJ == 128) || (BI == 256 && BJ == 128))
                                  : ((BI == 64 && (BJ == 64 || BJ == 128 || BJ == 256)) ||
                                     (BI == 128 && (BJ == 64 || BJ == 128 || BJ == 256)) ||
                                     (BI == 256 && (BJ == 64 || BJ == 128)));
  if (OD <= 0 || OP <= 0 || OQ <= 0) { pp.why = "empty output"; return pp; }
  if (c.groups > 1) { pp.why = "grouped convolution runs on the register-staged kernel"; return pp; }
  if (packed == 0) { pp.why = "channels fill less than half of the 128-byte K steps they would be padded to"; return pp; }
  if (packed >= ((int64_t)1 << 31)) { pp.why = "packed weights above 2 GiB"; return pp; }
  if (conv_relaid_bytes(c, op) + 256 >= ((int64_t)1 << 32)) { pp.why = "activations above 4 GiB"; return pp; }
  if (c.N * c.D * c.H * c.W >= ((int64_t)1 << 31) || J >= ((int64_t)1 << 31) - 512) {
    pp.why = "more than 2^31 input or output positions";
    return pp;
  }
  if (c.D + 2 * (int64_t)c.pad_d + c.T * c.dil_d >= 30000) { pp.why = "depth extent above 30000"; return pp; }
  if (!tile_ok) { pp.why = "no patch-staged instance with this block tile"; return pp; }
  int real_pos = 0, max_seg = 0;
  conv_patch_extent(J, (int)(OP * OQ), (int)OQ, BJ, c.stride_h, (int)c.R, c.dil_h, Wp, &real_pos, &max_seg);
  real_pos = (real_pos + 7) & ~7;
  // patch buffers start at multiples of 8 KB, so that the LDS swizzle of a position can be
  // taken from its address
  const int max_pos = (real_pos + 63) & ~63;
  const size_t budget = (size_t)160 * 1024 - 512;
  const int64_t macro_steps = c.T * (conv_padded_channels(c) * es / 128);
  const int split = split_k < 1 ? 1 : split_k;
  const bool one_macro = (macro_steps + split - 1) / split <= 1;   // no next patch at all
  pp.xbufs = one_macro ? 1 : 2;
  // patch buffers, position table, dump line
  const size_t patch = (size_t)pp.xbufs * max_pos * 128 + (size_t)max_pos * 8 + 1024;
  const size_t wstage = (size_t)BI * 128;
  pp.max_pos = max_pos;
  pp.max_seg = max_seg;
  if (max_seg > kConvMaxSegHost) { pp.why = "a tile spans more than 4 image slices"; return pp; }
  if (max_pos >= 4096) { pp.why = "input patch of a tile has 4096 or more positions"; return pp; }
  if (patch + 2 * wstage > budget) { pp.why = "input patch of a tile does not fit LDS"; return pp; }
  const int per_wave = ((real_pos / 8) + waves - 1) / waves;   // patch copies of the busiest wave
  // Ring depth and patch copies per step for an LDS budget.  The next patch is copied during the
  // taps of the current one; a copy issued on tap u has landed for everybody at the barrier of
  // the patch's last tap only if it is older than the nsw-2 steps' worth of copies still allowed
  // in flight there: u <= RS - nsw.  Kernel instances exist for 0, 2 and 4 copies per step
  // (4 waves), 0, 1 and 2 (8 waves).
  auto fit = [&](size_t lds_budget, int* nsw_out, int* pls_out) -> const char* {
    if (patch + 2 * wstage > lds_budget) return "input patch of a tile does not fit LDS";
    int nsw = (int)((lds_budget - patch) / wstage);
    if (nsw > 4) nsw = 4;
    if (nsw > RS + 1) nsw = RS + 1;
    if (nsw < 2) nsw = 2;
    if (one_macro) { *nsw_out = nsw; *pls_out = 0; return nullptr; }
    for (; nsw >= 2; --nsw) {
      const int taps = RS + 1 - nsw;
      if (taps < 1) continue;
      const int pls = (per_wave + taps - 1) / taps;
      if (pls > (waves == 8 ? 2 : 4)) continue;
      *nsw_out = nsw;
      *pls_out = waves == 8 ? pls : (pls <= 2 ? 2 : 4);
      return nullptr;
    }
    return RS == 1 ? "1x1 window with several channel chunks per block"
                   : "input patch too large to prefetch behind the window's taps";
  };
  // the instance with the nine taps unrolled: 8 waves, three ring stages, patch buffers a fixed
  // 48 KB (64 KB next to 64-row weight tiles) apart, the next patch fetched on taps 0..6 with at
  // most two copies per wave and step
  if (allow_w9 && waves == 8 && RS == 9 && BI <= 128 && BJ <= 128 && !(BI == 64 && BJ == 64)) {
    const int max_pos9 = one_macro ? max_pos : (BI <= 64 ? 512 : 384);
    const size_t patch9 = (size_t)pp.xbufs * max_pos9 * 128 + (size_t)max_pos9 * 8 + 1024;
    const int pls9 = one_macro ? 0 : (per_wave + 6) / 7;
    if (real_pos <= max_pos9 && 3 * wstage + patch9 <= budget && pls9 <= 2) {
      pp.w9 = 1;
      pp.nsw = 3;
      pp.pls = pls9;
      pp.max_pos = max_pos9;
      pp.occ = 1;
      pp.lds = 3 * wstage + patch9;
      pp.tab_rel = pp.xbufs * max_pos9 * 128;
      pp.dump_rel = pp.tab_rel + max_pos9 * 8;
      pp.tab1_rel = pp.tab_rel;
      // Blocks that walk several tiles (more tiles than CUs, no split-K, at least two macro steps
      // per tile) need a second position table: tables and dump line go behind the used part of
      // each patch buffer where they fit there, behind the second buffer otherwise
      const int64_t tiles = ((c.K + BI - 1) / BI) * ((J + BJ - 1) / BJ);
      if (allow_w9 >= 2 && !one_macro && split == 1 && tiles > device_compute_units() && !(BI == 128 && BJ == 128)) {
        const int xbuf = BI <= 64 ? 64 * 1024 : 48 * 1024;
        const int P = real_pos * 128, TB = real_pos * 8;
        int tab, tab1, dump;
        size_t total;
        if (P + TB + 1024 <= xbuf) {
          tab = P; dump = P + TB; tab1 = xbuf + P;
          total = 3 * wstage + (size_t)xbuf + P + TB;
        } else {
          tab = 2 * xbuf; tab1 = tab + TB; dump = tab1 + TB;
          total = 3 * wstage + (size_t)dump + 1024;
        }
        if (total <= budget) {
          pp.w9 = 2;
          pp.tab_rel = tab; pp.tab1_rel = tab1; pp.dump_rel = dump;
          pp.lds = total;
        }
      }
      return pp;
    }
  }
  pp.why = fit(budget, &pp.nsw, &pp.pls);
  if (pp.why) return pp;
  pp.lds = (size_t)pp.nsw * wstage + patch;
  pp.occ = 1;
  // two workgroups per CU when both fit: 80 KB of LDS each, accumulators + two steps of operand
  // fragments within 256 registers (tiles up to 128x128); pointless when every block already has
  // a CU to itself
  const int64_t blocks = ((c.K + BI - 1) / BI) * ((J + BJ - 1) / BJ) * split;
  if (waves == 4 && BI <= 128 && BJ <= 128 && blocks > device_compute_units()) {
    int nsw2 = 0, pls2 = 0;
    if (!fit((size_t)79 * 1024, &nsw2, &pls2)) {
      pp.occ = 2;
      pp.nsw = nsw2;
      pp.pls = pls2;
      pp.lds = (size_t)nsw2 * wstage + patch;
    }
  }
  return pp;
}

static const int kTiles[][2] = {{256, 256}, {256, 128}, {128, 256}, {128, 128},
                                {256, 64},  {128, 64},  {64, 128},  {64, 64},   {64, 256}};

static int64_t lds_bytes_of(int ti, int tj) { return 2ll * (ti + tj) * 128 + 2 * 128 * 8; }
// accumulator registers per lane: (ti/2 x tj/2 wave tile) / 64 lanes
static int64_t acc_regs_of(int ti, int tj) { return (int64_t)(ti / 2) * (tj / 2) / 64; }

// Estimated seconds of one launch of the register-staged kernel (or, for a 256x256 tile on
// eligible operands, the direct-to-LDS GEMM kernel) for a tile shape and split.  A model of the
// kernel's own structure with measured constants (profiles/mapper_model_calibration.md):
//   * a workgroup advances one 128-byte K step in L1(tile) microseconds when it has a CU to itself;
//   * a CU saturated with co-resident workgroups completes one workgroup-step every tau(tile)
//     microseconds (tau < L1: the loads of one workgroup hide behind the MFMAs of another);
//   * a CU that holds c workgroups therefore needs max(L1, c * tau) per step of all of them, and
//     the busiest CU has ceil(workgroups / CUs) of them, at most occ(tile) at a time;
//   * operands that are not loaded as 16-byte vectors along K slow both constants down;
//   * split-K adds the zero fill and the atomic read-modify-writes of the output.
//   * a round of workgroups has a fixed cost (prologue, the stores of the accumulators), large for
//     the 256x256 tile of the register-staged kernel (256 scattered stores per lane from four
//     waves per CU: 83 us for a 256 x 50176 x 64 product against 16 us with 128x64 tiles);
struct TileCost { int ti, tj, occ; double tau_us, alone_us, fixed_us; };
static const TileCost kTileCost[] = {
    {256, 256, 1, 2.45, 2.75, 70.0}, {256, 128, 1, 1.38, 1.55, 8.0}, {128, 256, 1, 1.46, 1.65, 8.0},
    {128, 128, 2, 0.654, 1.03, 2.0}, {256, 64, 1, 1.09, 1.17, 4.0}, {128, 64, 3, 0.394, 0.69, 1.0},
    {64, 128, 3, 0.403, 0.69, 1.0},  {64, 64, 4, 0.24, 0.50, 0.5},  {64, 256, 1, 1.26, 1.22, 4.0}};
// amos_gemm_tn (direct-to-LDS copies, 8 waves)
static const TileCost kDirectCost[] = {
    {256, 256, 1, 1.72, 1.65, 4.0}, {128, 256, 1, 0.98, 0.95, 2.0}, {256, 128, 1, 0.99, 0.92, 2.0},
    {128, 128, 2, 0.51, 0.70, 1.0}};

// A convolution that runs as a batched matrix product on a copy of its activations (every
// stride-th pixel of a 1x1 window, or an im2col matrix for few channels): that product, with
// the copy's time, as the mapper's problem.
static bool conv_copied_gemm_problem(const amos_conv_desc_t& c, int op, Problem* pg) {
  amos_bgemm_desc_t g;
  if (conv_as_subsampled_gemm(c, op, &g, nullptr)) {
    if (problem_of(AMOS_OP_BGEMM, &g, pg)) return false;
    note_repack(pg, g.g, g.batch, true);
    return true;
  }
  ConvIm2col ic;
  if (conv_as_im2col_gemm(c, op, &g, &ic)) {
    if (problem_of(AMOS_OP_BGEMM, &g, pg)) return false;
    pg->repack = 1;
    pg->Kp = ic.Kp;
    // the copy writes the im2col matrix at about a quarter of the HBM rate (8 element loads and
    // their index arithmetic per 16 bytes) and pads the weights in a second launch
    pg->repack_seconds = (double)ic.bytes_x / 2.0e12 + 6e-6;
    pg->direct_ok = 1;
    return true;
  }
  return false;
}

static double loader_factor(int loader) {
  switch (loader) {
    case 1: return 3.0;    // element loads: 8 (fp16) or 16 (int8) per 16-byte chunk
    case 2: return 4.5;    // im2col gather: element loads plus the tap arithmetic
    case 3: return 1.12;   // vectors along the rows, transposed in registers
  }
  return 1.0;
}

static double estimate_seconds(const Problem& pb, int ti, int tj, int split, bool allow_direct = true) {
  const double es = pb.in_dtype == AMOS_I8 ? 1.0 : 2.0;
  const TileCost* tc = nullptr;
  for (auto& t : kTileCost)
    if (t.ti == ti && t.tj == tj) tc = &t;
  if (!tc) return 1e9;
  bool direct = false;
  const bool repacked = allow_direct && pb.repack;    // the kernel runs on K-contiguous copies
  if (allow_direct && (pb.direct_ok || repacked) && split == 1)
    for (auto& t : kDirectCost)
      if (t.ti == ti && t.tj == tj) { tc = &t; direct = true; }
  const double k_tiles = std::ceil((double)(repacked ? pb.Kp : pb.K) / (128.0 / es));
  const int eff_split = (int)std::min<double>(split, k_tiles);
  const double ksteps = std::ceil(k_tiles / eff_split);
  const double lf = (direct || repacked) ? 1.0 : loader_factor(pb.row_loader) * loader_factor(pb.col_loader);
  const double tau = tc->tau_us * lf, alone = tc->alone_us * lf;
  const int64_t blocks = ((pb.I + ti - 1) / ti) * ((pb.J + tj - 1) / tj) * pb.batch * eff_split;
  const int64_t per_cu = (blocks + device_compute_units() - 1) / device_compute_units();
  const int64_t groups = per_cu / tc->occ, rest = per_cu % tc->occ;
  double step_us = (double)groups * std::max(alone, tc->occ * tau);
  if (rest) step_us += std::max(alone, (double)rest * tau);
  const double rounds = (double)groups + (rest ? 1.0 : 0.0);
  double t = 3e-6 + (ksteps * step_us + rounds * tc->fixed_us) * 1e-6;
  // output: written once; a split-K launch zero-fills it and accumulates with atomics (measured:
  // (1 + 2*split) passes over the output at ~3.5 TB/s)
  if (eff_split > 1) t += (double)pb.out_bytes * (1.0 + 2.0 * eff_split) / 3.5e12;
  // memory floor; the shorter of the two legs is not hidden completely, which also orders
  // memory-bound candidates by their compute time
  // (on copies the kernel reads the padded operands; the copies' own time is the same for every
  // configuration and stays outside the comparison of the two legs)
  const double in_bytes = repacked ? (double)pb.batch * (double)(pb.I + pb.J) * (double)pb.Kp * es : (double)pb.in_bytes;
  const double t_hbm = (in_bytes + (double)pb.out_bytes) / (0.7 * Gfx950::kHbmBytesPerSec) + 3e-6;
  return std::max(t, t_hbm) + 0.1 * std::min(t, t_hbm) + (repacked ? pb.repack_seconds : 0.0);
}

// patch_pitch 0: the smallest row pitch
int conv_nchw_load_bytes(const amos_conv_desc_t& c) {
  return c.in_dtype != AMOS_I8 && (c.H * c.W * 2) % 16 == 0 ? 16 : 8;
}

void conv_nchw_shape(const amos_conv_desc_t& c, int op, int patch_pitch, NchwShape* out, int load_bytes) {
  NchwShape& s = *out;
  const bool two_d = op == AMOS_OP_CONV2D;
  s.N = (int)c.N; s.C = (int)c.C; s.D = two_d ? 1 : (int)c.D; s.H = (int)c.H; s.W = (int)c.W; s.K = (int)c.K;
  s.T = two_d ? 1 : (int)c.T; s.R = (int)c.R; s.S = (int)c.S;
  s.sd = two_d ? 1 : c.stride_d; s.sh = c.stride_h; s.sw = c.stride_w;
  s.pd = two_d ? 0 : c.pad_d; s.ph = c.pad_h; s.pw = c.pad_w;
  s.dd = two_d ? 1 : c.dil_d; s.dh = c.dil_h; s.dw = c.dil_w;
  auto ext = [](int64_t in, int pad, int dil, int64_t k, int stride) {
    const int64_t eff = (k - 1) * dil + 1;
    return in + 2 * (int64_t)pad < eff ? 0 : (int)((in + 2 * (int64_t)pad - eff) / stride + 1);
  };
  s.OD = ext(s.D, s.pd, s.dd, s.T, s.sd);
  s.OP = ext(s.H, s.ph, s.dh, s.R, s.sh);
  s.OQ = ext(s.W, s.pw, s.dw, s.S, s.sw);
  s.J = s.N * s.OD * s.OP * s.OQ;
  s.Wp = patch_pitch > 0 ? patch_pitch : nchw_patch_pitch(s.OQ, s.S, s.sw, s.dw, s.sh, 1);
  s.pg_shift = (c.in_dtype == AMOS_I8 ? 3 : 2) + (load_bytes == 16 ? 1 : 0);
  s.div_opq = nchw_make_div((uint32_t)(s.OP * s.OQ));
  s.div_oq = nchw_make_div((uint32_t)s.OQ);
  s.div_w = nchw_make_div((uint32_t)s.W);
  s.div_od = nchw_make_div((uint32_t)s.OD);
}

ConvNchwPlan conv_nchw_plan(const amos_conv_desc_t& c, int op, int BI, int BJ, int load_bytes) {
  ConvNchwPlan r;
  memset(&r, 0, sizeof(r));
  const int es = c.in_dtype == AMOS_I8 ? 1 : 2;
  const int64_t T = op == AMOS_OP_CONV2D ? 1 : c.T, D = op == AMOS_OP_CONV2D ? 1 : c.D;
  if (c.layout != AMOS_LAYOUT_NCHW) { r.why = "tensors not in the NCDHW / KCTRS layout"; return r; }
  if (c.groups > 1) { r.why = "grouped convolution"; return r; }
  if (c.R != 3 || c.S != 3) { r.why = "window not 3x3"; return r; }
  if ((c.C * es) % 64) { r.why = "channels do not fill whole 64-byte chunks"; return r; }
  if (load_bytes != 8 && (load_bytes != 16 || es != 2)) { r.why = "patch loads of 16 bytes are for 16-bit types"; return r; }
  if ((c.H * c.W * es) % load_bytes) { r.why = "a channel plane is not a whole number of patch loads"; return r; }
  // (128 rows: two halves of 64 that share every macro step's patch)
  if ((BI != 128 && BI != 64 && BI != 32) || (BJ != 128 && BJ != 256)) { r.why = "block tile not 32, 64 or 128 by 128 or 256"; return r; }
  // (lanes address both tensors by 32-bit byte offsets)
  if (c.N * c.C * D * c.H * c.W * es >= ((int64_t)1 << 32) || c.K * c.C * T * 9 * es >= ((int64_t)1 << 32)) { r.why = "a tensor of 4 GiB or more"; return r; }
  NchwShape s;
  conv_nchw_shape(c, op, 0, &s, load_bytes);
  if (s.OD <= 0 || s.OP <= 0 || s.OQ <= 0) { r.why = "window larger than the padded input"; return r; }
  // nine weight tiles and a patch buffer of the tile's fixed size (its last 1 KB a dump line), both twice
  const int pbuf = BJ <= 128 ? 32 * 1024 : 40 * 1024;
  const int pos_limit = pbuf / kNchwPosBytes - 16;
  // The largest tile: every tile's geometry, kept per shape (a launch plans again on every call).
  // The row pitch of the patch: pitch - outputs per row a multiple of 8 (fragment reads free of bank
  // conflicts also where they wrap into the next row) where the largest patch then fits the
  // buffer, else the smallest.
  struct Key { int v[24]; };
  struct Entry { Key k; int max_pos, max_groups, max_seg; };
  static std::mutex mu;
  static std::vector<Entry> cache;
  int max_pos = -1, max_groups = 0, max_seg = 0;
  for (int align : {8, 1}) {
    s.Wp = nchw_patch_pitch(s.OQ, s.S, s.sw, s.dw, s.sh, align);
    Key key = {{s.N, s.D, s.H, s.W, s.T, s.sd, s.sh, s.sw, s.pd, s.ph, s.pw, s.dd, s.dh, s.dw, s.OD, s.OP, s.OQ, s.pg_shift, BJ, s.Wp, 0, 0, 0, 0}};
    max_pos = -1; max_groups = 0; max_seg = 0;
    {
      std::lock_guard<std::mutex> lock(mu);
      for (const Entry& e : cache)
        if (!memcmp(&e.k, &key, sizeof(key))) { max_pos = e.max_pos; max_groups = e.max_groups; max_seg = e.max_seg; }
    }
    if (max_pos < 0) {
      max_pos = 0;
      for (int64_t bj0 = 0; bj0 < s.J; bj0 += BJ) {
        const NchwTile t = nchw_tile(s, (int)bj0, BJ);
        max_seg = std::max(max_seg, t.nseg);
        if (t.nseg > kNchwMaxSeg) break;
        max_pos = std::max(max_pos, t.npos);
        max_groups = std::max(max_groups, t.ngroups);
      }
      std::lock_guard<std::mutex> lock(mu);
      if (cache.size() >= 64) cache.erase(cache.begin());
      cache.push_back(Entry{key, max_pos, max_groups, max_seg});
    }
    if (max_seg > kNchwMaxSeg || max_pos <= pos_limit) break;
  }
  if (max_seg > kNchwMaxSeg) { r.why = "a tile of output positions touches more than four images"; return r; }
  r.max_pos = max_pos;   // (whole 8-position blocks)
  r.Wp = s.Wp;
  r.max_groups = max_groups;
  // (how many rounds of the loader waves that is depends on where the weights come from: the
  // launch plan decides and refuses what is above the loaders' budget)
  r.groups_per_thread = 0;
  if (r.max_pos > pos_limit) { r.why = "input patch of a tile does not fit its LDS buffer"; return r; }
  r.lds = (size_t)2 * 9 * (BI == 128 ? 64 : BI) * 64 + (size_t)2 * pbuf;
  r.t1 = T == 1;
  return r;
}

int conv_unroll_level(int flags) {
  return (flags & AMOS_FLAG_NO_UNROLLED_TAPS) ? 0 : (flags & AMOS_FLAG_NO_TILE_WALK) ? 1 : 2;
}

// Patch-staged convolution: blocks of one per CU; a K step costs its MFMA issue time plus a
// per-step instruction overhead that does not shrink with the tile; split-K pays for atomic
// accumulation into the output.  Returns <= 0 where the pipeline does not apply.
static double conv_patch_estimate(const amos_conv_desc_t& c, int op, const Problem& pb, int ti, int tj,
                                  int split, int waves = 0, int allow_w9 = 2) {
  ConvPatchPlan pp = conv_patch_plan(c, op, ti, tj, split, waves, allow_w9);
  if (pp.why) return -1.0;
  const bool two_streams = pp.occ == 2 || pp.waves == 8;   // two waves per SIMD
  const double es = pb.in_dtype == AMOS_I8 ? 1.0 : 2.0;
  const int64_t T = op == AMOS_OP_CONV2D ? 1 : c.T;
  const double steps_all = (double)T * c.R * c.S * std::ceil(c.C * es / 128.0);
  const double macro_steps = (double)T * std::ceil(c.C * es / 128.0);
  if (split > macro_steps) split = (int)macro_steps;     // what the launch clamps it to
  const double blocks = std::ceil((double)pb.I / ti) * std::ceil((double)pb.J / tj) * split;
  // two resident workgroups take turns on the matrix cores while their per-step instruction
  // overheads overlap
  const double rounds = std::ceil(blocks / (device_compute_units() * (double)pp.occ));
  const double steps = std::ceil(steps_all / split);
  const double mfma_per_step = (ti / 64.0) * (tj / 64.0) * 4.0 * 32.0;
  // measured (profiles/conv_fprop_kernel_trace.md): a 128x64 step takes ~700 cycles with the taps
  // unrolled, ~760 with two instruction streams per SIMD, ~850 with one; set-up 6000-8000 cycles
  const double overhead = pp.w9 ? 440.0 : two_streams ? 500.0 : 600.0;
  double cycles = rounds * (steps * (pp.occ * mfma_per_step + overhead) + (pp.w9 ? 8000.0 : 6000.0));
  // blocks that walk their tiles set up once; a tile switch costs the stores and the new addresses
  if (pp.w9 == 2) cycles = rounds * (steps * (mfma_per_step + overhead) + 1500.0) + 8000.0;
  const double relayout = ((double)pb.in_bytes * 2.0) / 2.5e12 + 3e-6;
  return cycles / 2.1e9 + relayout + (split > 1 ? (double)pb.out_bytes * split / 1.2e12 : 0.0);
}

// NCDHW-direct convolution (conv_nchw_kernel.h), weights packed by the call: one workgroup per CU
// at a time; a tile pays its set-up, the latency of its first loads and its stores (~9000 cycles
// at the 2.4 GHz of the cycle counter, measured), then per macro step (nine taps x 64 bytes of
// channels) the longer of the matrix-core waves' time (the tile's flops at 72-85 % of the CU's
// rate, measured with the loaders switched off) and the loader waves' time (a fixed ~1800 cycles
// of latency that their two-step lookahead does not cover, plus ~45 per load instruction of a
// wave, measured on 14x14 and 56x56 planes; int8 loads twice the channels per group).
// Returns <= 0 where the kernel does not apply.
double conv_nchw_estimate(const amos_conv_desc_t& c, int op, const Problem& pb, int ti, int tj, bool* unpacked) {
  if (unpacked) *unpacked = false;
  if ((ti != 128 && ti != 64 && ti != 32) || (tj != 128 && tj != 256)) return -1.0;
  const int halves = ti == 128 ? 2 : 1;   // a 128-row workgroup: two sequence steps of 64 rows per macro step
  const int tr = ti / halves;
  // (as the launch plans it: patch loads of 16 bytes where the shape allows them and one round of
  // the loaders covers the largest tile)
  int s_lb = conv_nchw_load_bytes(c);
  ConvNchwPlan np = conv_nchw_plan(c, op, ti, tj, s_lb);
  if (s_lb == 16 && (np.why || np.max_groups > 16 * nchw_loader_waves(true, np.max_groups))) {
    s_lb = 8;
    np = conv_nchw_plan(c, op, ti, tj, 8);
  }
  if (np.why) return -1.0;
  const bool i8 = pb.in_dtype == AMOS_I8;
  const double es = i8 ? 1.0 : 2.0;
  const int nwl = nchw_loader_waves(true, np.max_groups);
  if (np.max_groups > 16 * nwl * (i8 || s_lb == 16 ? 1 : 2)) return -1.0;
  const int64_t T = op == AMOS_OP_CONV2D ? 1 : c.T;
  const double macro_steps = (double)T * (c.C * es / 64.0);
  const double tiles = std::ceil((double)pb.I / ti) * std::ceil((double)pb.J / tj);
  const double rounds = std::ceil(tiles / device_compute_units());
  const double flop_per_cycle = (i8 ? 2.0 : 1.0) * 3850.0 * (tr * tj >= 64 * 256 ? 0.85 : tr * tj >= 64 * 128 ? 0.72 : 0.6);
  const double mma = 2.0 * tr * tj * 9.0 * (64.0 / es) / flop_per_cycle;
  // the loaders of a macro step: a fixed part, the bytes they move and their load instructions
  // (fitted: 64x128 tile, 24 instructions of 8 bytes a lane 2400 cycles, of 16 bytes 3500; 64x256,
  // 32 of 16 bytes 4600)
  const double load_instr = std::ceil(np.max_groups * 4.0 / 64.0) * (16.0 / es);
  const double loaders = 1300.0 + 5.0 * load_instr * s_lb + 20.0 * load_instr;
  const double prologue = 9000.0 + 40.0 * load_instr;
  // (the second half of a macro step has no patch to bring in: its weights only; twice the stores)
  const double cycles = rounds * (prologue + (halves - 1) * 2500.0 + macro_steps * (std::max(mma, loaders) + (halves - 1) * std::max(mma, 900.0)));
  const double kernel = cycles / 2.4e9 + 2.5e-6;
  // the weights: packed by a launch in front of the kernel (its cost is the dependent launch more
  // than the copy), or -- conv2d, where a chunk's taps are one aligned run -- transposed by the
  // loaders of every tile, some 600 cycles more per macro step and 64 rows
  const double pack = (double)(c.K * c.C * T * 9) * es * 2.0 / 2.5e12 + 3.5e-6;
  const double in_kernel = rounds * macro_steps * 600.0 * halves / 2.4e9;
  if (op == AMOS_OP_CONV2D && in_kernel < pack) {
    if (unpacked) *unpacked = true;
    return kernel + in_kernel;
  }
  return kernel + pack;
}

}  // namespace amos

using namespace amos;

extern "C" {

int amos_check_config(int op, const void* desc, const amos_kernel_config_t* cfg,
                      int64_t* lds_bytes, int64_t* acc_regs) {
  Problem pb;
  int rc = problem_of(op, desc, &pb);
  if (rc) return rc;
  if (!cfg) return set_error(AMOS_ERR_BAD_ARG, "null config");
  // the NCDHW-direct convolution has tiles of its own (32 / 64 / 128 rows by 128 / 256 positions):
  // its planner says whether the shape and the tile go together and how much LDS a workgroup takes
  if ((op == AMOS_OP_CONV2D || op == AMOS_OP_CONV3D) && cfg->pipeline == AMOS_PIPE_NCHW) {
    const amos_conv_desc_t& c = *(const amos_conv_desc_t*)desc;
    int lb = conv_nchw_load_bytes(c);
    ConvNchwPlan np = conv_nchw_plan(c, op, cfg->tile_i, cfg->tile_j, lb);
    if (np.why && lb == 16) np = conv_nchw_plan(c, op, cfg->tile_i, cfg->tile_j, 8);
    if (np.why) return set_error(AMOS_ERR_INFEASIBLE, "NCDHW-direct convolution not applicable: %s", np.why);
    if (lds_bytes) *lds_bytes = (int64_t)np.lds;
    // (accumulators of a matrix-core wave: its share of the tile, four bytes an element, 64 lanes)
    const int waves = cfg->tile_i >= 64 ? 8 : 4;
    if (acc_regs) *acc_regs = (int64_t)cfg->tile_i * cfg->tile_j / (64 * waves);
    if ((int64_t)np.lds > Gfx950::kLdsBytes)
      return set_error(AMOS_ERR_INFEASIBLE, "LDS over budget: %lld (required) vs. %d (given)", (long long)np.lds, Gfx950::kLdsBytes);
    if (cfg->split_k < 0) return set_error(AMOS_ERR_BAD_ARG, "negative split_k");
    return 0;
  }
  bool known = false;
  for (auto& t : kTiles) known |= (t[0] == cfg->tile_i && t[1] == cfg->tile_j);
  if (!known)
    return set_error(AMOS_ERR_INFEASIBLE, "no kernel instance with block tile %dx%d", cfg->tile_i,
                     cfg->tile_j);
  int64_t lds = lds_bytes_of(cfg->tile_i, cfg->tile_j);
  int64_t regs = acc_regs_of(cfg->tile_i, cfg->tile_j);
  if (lds_bytes) *lds_bytes = lds;
  if (acc_regs) *acc_regs = regs;
  if (lds > Gfx950::kLdsBytes)
    return set_error(AMOS_ERR_INFEASIBLE, "LDS over budget: %lld (required) vs. %d (given)",
                     (long long)lds, Gfx950::kLdsBytes);
  // accumulators + two operand fragments sets + prefetch registers must fit the file
  int64_t prefetch = (cfg->tile_i + cfg->tile_j) / 32 * 4;
  if (regs + prefetch + 64 > Gfx950::kVgprsPerLane)
    return set_error(AMOS_ERR_INFEASIBLE, "registers over budget: %lld (required) vs. %d (given)",
                     (long long)(regs + prefetch + 64), Gfx950::kVgprsPerLane);
  if (cfg->split_k < 0) return set_error(AMOS_ERR_BAD_ARG, "negative split_k");
  return 0;
}

int amos_estimate_seconds(int op, const void* desc, const amos_kernel_config_t* cfg, double* seconds) {
  Problem pb;
  int rc = problem_of(op, desc, &pb);
  if (rc) return rc;
  if (!cfg || !seconds) return set_error(AMOS_ERR_BAD_ARG, "null pointer argument");
  rc = amos_check_config(op, desc, cfg, nullptr, nullptr);
  if (rc) return rc;
  const int split = cfg->split_k < 1 ? 1 : cfg->split_k;
  if ((op == AMOS_OP_CONV2D || op == AMOS_OP_CONV3D) && cfg->pipeline == AMOS_PIPE_AUTO &&
      conv_is_depthwise(*(const amos_conv_desc_t*)desc)) {
    // bytes in and out at about a third of the HBM rate (element loads), plus a launch
    *seconds = ((double)pb.in_bytes + (double)pb.out_bytes) / (0.35 * Gfx950::kHbmBytesPerSec) + 3e-6;
    return 0;
  }
  if ((op == AMOS_OP_GEMM || op == AMOS_OP_BGEMM) && cfg->pipeline == AMOS_PIPE_AUTO &&
      gemm_is_skinny(op == AMOS_OP_GEMM ? *(const amos_gemm_desc_t*)desc : ((const amos_bgemm_desc_t*)desc)->g,
                     op == AMOS_OP_GEMM ? 1 : ((const amos_bgemm_desc_t*)desc)->batch)) {
    // one pass over the operands at about half the HBM rate, plus a launch
    *seconds = ((double)pb.in_bytes + (double)pb.out_bytes) / (0.5 * Gfx950::kHbmBytesPerSec) + 3.5e-6;
    return 0;
  }
  ConvFewcPlan fp;
  if ((op == AMOS_OP_CONV2D || op == AMOS_OP_CONV3D) && cfg->pipeline == AMOS_PIPE_AUTO &&
      conv_fewc_plan(*(const amos_conv_desc_t*)desc, op, &fp)) {
    // the relayout launch, then rounds of workgroups that each load ~100 KB, compute for ~1 us and
    // store 64 KB; floored by the bytes
    const amos_conv_desc_t& c = *(const amos_conv_desc_t*)desc;
    const double rounds = std::ceil((double)fp.tiles_j * c.N / fp.grid_x);
    const double t_conv = 6e-6 + rounds * 4.5e-6;
    const double t_mem = ((double)pb.in_bytes * 2 + (double)fp.bytes_x * 2 + (double)pb.out_bytes) / (0.5 * Gfx950::kHbmBytesPerSec);
    *seconds = 4e-6 + (double)fp.bytes_x / 2.5e12 + std::max(t_conv, t_mem);
    return 0;
  }
  if ((op == AMOS_OP_CONV2D || op == AMOS_OP_CONV3D) && cfg->pipeline == AMOS_PIPE_NCHW) {
    const double s = conv_nchw_estimate(*(const amos_conv_desc_t*)desc, op, pb, cfg->tile_i, cfg->tile_j);
    if (s <= 0) return set_error(AMOS_ERR_INFEASIBLE, "NCDHW-direct convolution not applicable to this config");
    *seconds = s;
    return 0;
  }
  amos_bgemm_desc_t as_gemm;
  if ((op == AMOS_OP_CONV2D || op == AMOS_OP_CONV3D) && cfg->pipeline != AMOS_PIPE_PATCH &&
      cfg->pipeline != AMOS_PIPE_PATCH8 && conv_as_gemm(*(const amos_conv_desc_t*)desc, op, &as_gemm))
    return amos_estimate_seconds(AMOS_OP_BGEMM, &as_gemm, cfg, seconds);   // what the launch runs
  if ((op == AMOS_OP_CONV2D || op == AMOS_OP_CONV3D) && conv_subsample_pipeline(cfg->pipeline)) {
    Problem pg;
    if (conv_copied_gemm_problem(*(const amos_conv_desc_t*)desc, op, &pg)) {
      *seconds = estimate_seconds(pg, cfg->tile_i, cfg->tile_j, cfg->split_k < 1 ? 1 : cfg->split_k);
      return 0;
    }
  }
  if ((op == AMOS_OP_CONV2D || op == AMOS_OP_CONV3D) && cfg->pipeline != AMOS_PIPE_STAGED) {
    const int waves = cfg->pipeline == AMOS_PIPE_PATCH ? 4 : cfg->pipeline == AMOS_PIPE_PATCH8 ? 8 : 0;
    double s = conv_patch_estimate(*(const amos_conv_desc_t*)desc, op, pb, cfg->tile_i, cfg->tile_j, split,
                                   waves, conv_unroll_level(cfg->reserved[0]));
    if (s > 0) { *seconds = s; return 0; }
    if (waves) return set_error(AMOS_ERR_INFEASIBLE, "patch-staged convolution not applicable to this config");
  }
  *seconds = estimate_seconds(pb, cfg->tile_i, cfg->tile_j, split, cfg->pipeline != AMOS_PIPE_STAGED);
  return 0;
}

// The choice is a function of the operator, its descriptor and the device's compute units, and
// costs some 150 evaluations of the model: a call that names no configuration would pay that on
// the host every time (tens of microseconds, more than many of the kernels take).  The last few
// hundred choices are therefore kept, keyed by the descriptor's bytes.
static int default_config_of(int op, const void* desc, amos_kernel_config_t* result);

int amos_default_config(int op, const void* desc, amos_kernel_config_t* result) {
  const size_t n = op == AMOS_OP_GEMM ? sizeof(amos_gemm_desc_t) : op == AMOS_OP_BGEMM ? sizeof(amos_bgemm_desc_t)
                   : (op == AMOS_OP_CONV2D || op == AMOS_OP_CONV3D) ? sizeof(amos_conv_desc_t) : 0;
  if (!desc || !result || n == 0) return default_config_of(op, desc, result);
  static std::mutex mu;
  static std::unordered_map<std::string, amos_kernel_config_t> kept;
  std::string key((const char*)desc, n);
  const int tag[2] = {op, device_compute_units()};
  key.append((const char*)tag, sizeof(tag));
  {
    std::lock_guard<std::mutex> lock(mu);
    auto it = kept.find(key);
    if (it != kept.end()) { *result = it->second; return 0; }
  }
  const int rc = default_config_of(op, desc, result);
  if (rc == 0) {
    std::lock_guard<std::mutex> lock(mu);
    if (kept.size() >= 512) kept.clear();
    kept[key] = *result;
  }
  return rc;
}

static int default_config_of(int op, const void* desc, amos_kernel_config_t* result) {
  Problem pb;
  int rc = problem_of(op, desc, &pb);
  if (rc) return rc;
  if (!result) return set_error(AMOS_ERR_BAD_ARG, "null config");
  // so does a GEMM with one skinny side
  if ((op == AMOS_OP_GEMM || op == AMOS_OP_BGEMM) &&
      gemm_is_skinny(op == AMOS_OP_GEMM ? *(const amos_gemm_desc_t*)desc : ((const amos_bgemm_desc_t*)desc)->g,
                     op == AMOS_OP_GEMM ? 1 : ((const amos_bgemm_desc_t*)desc)->batch)) {
    memset(result, 0, sizeof(*result));
    result->tile_i = 64; result->tile_j = 64; result->split_k = 1; result->pipeline = AMOS_PIPE_AUTO;
    return 0;
  }
  // a depthwise convolution runs on the vector ALUs, whatever the tile
  if ((op == AMOS_OP_CONV2D || op == AMOS_OP_CONV3D) && conv_is_depthwise(*(const amos_conv_desc_t*)desc)) {
    memset(result, 0, sizeof(*result));
    result->tile_i = 64; result->tile_j = 64; result->split_k = 1; result->pipeline = AMOS_PIPE_AUTO;
    return 0;
  }
  // few input channels: one kernel, one tile
  if ((op == AMOS_OP_CONV2D || op == AMOS_OP_CONV3D) && conv_fewc_plan(*(const amos_conv_desc_t*)desc, op, nullptr)) {
    memset(result, 0, sizeof(*result));
    result->tile_i = 64; result->tile_j = 256; result->split_k = 1; result->pipeline = AMOS_PIPE_AUTO;
    return 0;
  }
  // a pointwise convolution runs as a batched matrix product: that product's configuration
  amos_bgemm_desc_t as_gemm;
  if ((op == AMOS_OP_CONV2D || op == AMOS_OP_CONV3D) && conv_as_gemm(*(const amos_conv_desc_t*)desc, op, &as_gemm))
    return amos_default_config(AMOS_OP_BGEMM, &as_gemm, result);
  // ... a strided one, or one on few channels, after a copy of its activations: the product on
  // the copies
  Problem pg;
  const bool copied = (op == AMOS_OP_CONV2D || op == AMOS_OP_CONV3D) &&
                      conv_copied_gemm_problem(*(const amos_conv_desc_t*)desc, op, &pg);
  if (copied) { pb = pg; op = AMOS_OP_BGEMM; }
  memset(result, 0, sizeof(*result));
  amos_kernel_config_t* out = result;
  const double es = pb.in_dtype == AMOS_I8 ? 1.0 : 2.0;
  const int k_tiles = (int)std::ceil((double)pb.K / (128.0 / es));
  double best = 1e30;
  if (op == AMOS_OP_CONV2D || op == AMOS_OP_CONV3D) {
    // patch-staged pipeline where it applies: blocks of one per CU, a K step costs its MFMA
    // issue time plus a per-step instruction overhead that does not shrink with the tile;
    // split-K pays for atomic accumulation into the output
    const amos_conv_desc_t& c = *(const amos_conv_desc_t*)desc;
    for (auto& t : kTiles) {
      for (int split = 1; split <= 4; split *= 2) {
        const double s = conv_patch_estimate(c, op, pb, t[0], t[1], split);
        if (s > 0 && s < best * 0.995) {
          best = s;
          out->tile_i = t[0];
          out->tile_j = t[1];
          out->split_k = split;
        }
      }
    }
  }
  // a convolution leaves the patch-staged pipeline only for a clearly better estimate of the
  // register-staged kernel (whose im2col constants are the less certain ones)
  const double patch_best = best;
  amos_kernel_config_t staged = *out;
  if (patch_best < 1e30) best = patch_best / 1.25;
  const double staged_bar = best;
  out = &staged;
  for (auto& t : kTiles) {
    for (int split = 1; split <= 16; split *= 2) {
      if (split > 1 && (split > k_tiles / 2 || pb.batch > 1)) break;
      double s = estimate_seconds(pb, t[0], t[1], split);
      if (s < best * 0.995) {
        best = s;
        out->tile_i = t[0];
        out->tile_j = t[1];
        out->split_k = split;
        out->pipeline = patch_best < 1e30 ? AMOS_PIPE_STAGED : AMOS_PIPE_AUTO;
      }
    }
  }
  *result = staged;
  // the kernel that reads the activations as they are, where it applies and its estimate is lower
  if (op == AMOS_OP_CONV2D || op == AMOS_OP_CONV3D) {
    const amos_conv_desc_t& c = *(const amos_conv_desc_t*)desc;
    if (patch_best < 1e30 && best >= staged_bar) best = patch_best;   // (the estimate of what was chosen)
    for (int ti : {64, 32, 128})
      for (int tj : {128, 256}) {
        const double s = conv_nchw_estimate(c, op, pb, ti, tj);
        if (s > 0 && s < best * 0.97) {
          best = s;
          memset(result, 0, sizeof(*result));
          result->tile_i = ti; result->tile_j = tj; result->split_k = 1; result->pipeline = AMOS_PIPE_NCHW;
        }
      }
  }
  return 0;
}

}  // extern "C"
