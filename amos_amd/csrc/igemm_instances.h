// Kernel-instance table: one translation unit per (dtype, row loader) pair keeps
// the build parallel.  Each unit defines pick_<dtype>_<loader>(col loader, tile).
#pragma once
#include <mutex>
#include <string>

#include "igemm_kernel.h"

namespace amos {

typedef void (*igemm_fn)(const IgemmParams);

struct Instance {
  igemm_fn fn;
  size_t lds;
  const char* name;
  std::once_flag once;  // guards the one-time LDS-size attribute call
};

template <int DT, int RL, int CL, int TI, int TJ>
Instance* instance() {
  static Instance inst;
  static const char* dtn[] = {"f16", "bf16", "i8"};
  static const char* ldn[] = {"vec", "strided", "im2col", "tvec"};
  static std::string name = std::string("amos_igemm<") + dtn[DT] + "," + ldn[RL] + "," + ldn[CL] +
                            "," + std::to_string(64 * TI) + "x" + std::to_string(64 * TJ) + ">";
  inst.fn = amos_igemm<DT, RL, CL, TI, TJ>;
  inst.lds = igemm_lds_bytes<TI, TJ>();
  inst.name = name.c_str();
  return &inst;
}

template <int DT, int RL, int CL>
Instance* pick_tile(int ti, int tj) {
  if (ti == 64 && tj == 64) return instance<DT, RL, CL, 1, 1>();
  if (ti == 128 && tj == 128) return instance<DT, RL, CL, 2, 2>();
  if (ti == 256 && tj == 256) return instance<DT, RL, CL, 4, 4>();
  if (ti == 128 && tj == 64) return instance<DT, RL, CL, 2, 1>();
  if (ti == 64 && tj == 128) return instance<DT, RL, CL, 1, 2>();
  if (ti == 256 && tj == 128) return instance<DT, RL, CL, 4, 2>();
  if (ti == 128 && tj == 256) return instance<DT, RL, CL, 2, 4>();
  if (ti == 256 && tj == 64) return instance<DT, RL, CL, 4, 1>();
  if (ti == 64 && tj == 256) return instance<DT, RL, CL, 1, 4>();
  return nullptr;
}

template <int DT, int RL>
Instance* pick_col(int cl, int ti, int tj) {
  switch (cl) {
    case LD_VEC: return pick_tile<DT, RL, LD_VEC>(ti, tj);
    case LD_STRIDED: return pick_tile<DT, RL, LD_STRIDED>(ti, tj);
    case LD_CONV: return pick_tile<DT, RL, LD_CONV>(ti, tj);
    case LD_TVEC:
      // 16-bit types, next to a vec or tvec row loader
      if constexpr (DT != DT_I8 && RL != LD_STRIDED) return pick_tile<DT, RL, LD_TVEC>(ti, tj);
      return nullptr;
  }
  return nullptr;
}
// row loader tvec: column loaders vec and tvec
template <int DT>
Instance* pick_col_tvec(int cl, int ti, int tj) {
  if (cl == LD_VEC) return pick_tile<DT, LD_TVEC, LD_VEC>(ti, tj);
  if (cl == LD_TVEC) return pick_tile<DT, LD_TVEC, LD_TVEC>(ti, tj);
  return nullptr;
}

struct GemmTnParams;
typedef void (*gemm_tn_fn)(const GemmTnParams);
struct TnInstance {
  gemm_tn_fn fn;
  size_t lds;
  int threads;
  const char* name;
  std::once_flag once;
  int scratch_bytes = 0;   // per-lane scratch memory of the built kernel, read before its first launch
};
// direct-to-LDS GEMM (defined in inst_gemm_tn.hip); 256x256 with 4 or 8 waves, 128x128 / 128x256 /
// 256x128 with 8
TnInstance* pick_gemm_tn(int dt, int ti, int tj, int waves);

// patch-staged convolution (defined in inst_conv_*.hip)
struct ConvFpropParams;
typedef void (*conv_fprop_fn)(const ConvFpropParams);
struct ConvInstance {
  conv_fprop_fn fn;
  const char* name;
  int threads;
  std::once_flag once;
  int static_lds = 0;   // must stay 0: the kernel addresses dynamic LDS from byte 0
};
ConvInstance* pick_conv_f16(int ti, int tj, int waves, int pls, int occ, int w9);
ConvInstance* pick_conv_bf16(int ti, int tj, int waves, int pls, int occ, int w9);
ConvInstance* pick_conv_i8(int ti, int tj, int waves, int pls, int occ, int w9);
void launch_conv_prepare(int es, const ConvFpropParams& p, hipStream_t stream);

#ifdef AMOS_CONV_FPROP_KERNEL_INCLUDED
template <int DT, int TI, int TJ, int NW, int PL, int OCC, int W9 = 0>
ConvInstance* conv_instance() {
  static ConvInstance inst;
  static const char* dtn[] = {"f16", "bf16", "i8"};
  static std::string name = std::string("amos_conv_fprop<") + dtn[DT] + "," + std::to_string(64 * TI) +
                            "x" + std::to_string(64 * TJ) + "," + std::to_string(NW) + "w,pl" +
                            std::to_string(PL) + (OCC == 2 ? ",occ2" : "") + (W9 == 2 ? ",9taps,walk>" : W9 ? ",9taps>" : ">");
  inst.fn = amos_conv_fprop<DT, TI, TJ, NW, PL, OCC, W9>;
  inst.name = name.c_str();
  inst.threads = 64 * NW;
  return &inst;
}
template <int DT, int PL>
ConvInstance* pick_conv_tile4(int ti, int tj, int occ) {
  if (occ == 2) {
    if (ti == 64 && tj == 64) return conv_instance<DT, 1, 1, 4, PL, 2>();
    if (ti == 128 && tj == 64) return conv_instance<DT, 2, 1, 4, PL, 2>();
    if (ti == 64 && tj == 128) return conv_instance<DT, 1, 2, 4, PL, 2>();
    if (ti == 128 && tj == 128) return conv_instance<DT, 2, 2, 4, PL, 2>();
    return nullptr;
  }
  if (ti == 64 && tj == 64) return conv_instance<DT, 1, 1, 4, PL, 1>();
  if (ti == 128 && tj == 64) return conv_instance<DT, 2, 1, 4, PL, 1>();
  if (ti == 64 && tj == 128) return conv_instance<DT, 1, 2, 4, PL, 1>();
  if (ti == 128 && tj == 128) return conv_instance<DT, 2, 2, 4, PL, 1>();
  if (ti == 256 && tj == 64) return conv_instance<DT, 4, 1, 4, PL, 1>();
  if (ti == 256 && tj == 128) return conv_instance<DT, 4, 2, 4, PL, 1>();
  if (ti == 128 && tj == 256) return conv_instance<DT, 2, 4, 4, PL, 1>();
  if (ti == 64 && tj == 256) return conv_instance<DT, 1, 4, 4, PL, 1>();
  return nullptr;
}
template <int DT, int PL>
ConvInstance* pick_conv_tile8(int ti, int tj) {
  if (ti == 128 && tj == 64) return conv_instance<DT, 2, 1, 8, PL, 1>();
  if (ti == 64 && tj == 128) return conv_instance<DT, 1, 2, 8, PL, 1>();
  if (ti == 128 && tj == 128) return conv_instance<DT, 2, 2, 8, PL, 1>();
  if (ti == 256 && tj == 128) return conv_instance<DT, 4, 2, 8, PL, 1>();
  if (ti == 128 && tj == 256) return conv_instance<DT, 2, 4, 8, PL, 1>();
  return nullptr;
}
template <int DT, int PL, int W9>
ConvInstance* pick_conv_tile9(int ti, int tj) {
  if (ti == 128 && tj == 64) return conv_instance<DT, 2, 1, 8, PL, 1, W9>();
  if (ti == 64 && tj == 128) return conv_instance<DT, 1, 2, 8, PL, 1, W9>();
  if constexpr (W9 != 2) {   // (walking tiles, a 128x128 block would not fit the register file)
    if (ti == 128 && tj == 128) return conv_instance<DT, 2, 2, 8, PL, 1, W9>();
  }
  return nullptr;
}
// waves = 4 or 8; pls = patch copies per wave per K step the plan asks for: 0, 2 or 4 with 4
// waves, 0, 1 or 2 with 8; w9 = 1: the instance with nine unrolled taps, 2: the one whose
// blocks walk several tiles
template <int DT>
ConvInstance* pick_conv_tile(int ti, int tj, int waves, int pls, int occ, int w9) {
  if (w9 == 2) {
    if (waves != 8 || occ != 1) return nullptr;
    if (pls == 1) return pick_conv_tile9<DT, 1, 2>(ti, tj);
    if (pls == 2) return pick_conv_tile9<DT, 2, 2>(ti, tj);
    return nullptr;
  }
  if (w9) {
    if (waves != 8 || occ != 1) return nullptr;
    if (pls == 0) return pick_conv_tile9<DT, 0, 1>(ti, tj);
    if (pls == 1) return pick_conv_tile9<DT, 1, 1>(ti, tj);
    if (pls == 2) return pick_conv_tile9<DT, 2, 1>(ti, tj);
    return nullptr;
  }
  if (waves == 8) {
    if (occ != 1) return nullptr;
    if (pls == 0) return pick_conv_tile8<DT, 0>(ti, tj);
    if (pls == 1) return pick_conv_tile8<DT, 1>(ti, tj);
    if (pls == 2) return pick_conv_tile8<DT, 2>(ti, tj);
    return nullptr;
  }
  if (pls == 0) return pick_conv_tile4<DT, 0>(ti, tj, occ);
  if (pls == 2) return pick_conv_tile4<DT, 2>(ti, tj, occ);
  if (pls == 4) return pick_conv_tile4<DT, 4>(ti, tj, occ);
  return nullptr;
}
#endif

// convolution straight from NCDHW / KCTRS (defined in inst_conv_nchw_*.hip): 3x3 windows, block
// tiles 64 x 128 and 64 x 256, eight waves; t1 = the weights of a chunk of channels are one
// contiguous aligned run (conv2d)
struct ConvNchwParams;
typedef void (*conv_nchw_fn)(const ConvNchwParams);
struct ConvNchwInstance {
  conv_nchw_fn fn;
  const char* name;
  int threads;
  int bi, bj;
  int groups_per_thread;   // load groups of the patch a loader thread may own (x 4 chunks of channels)
  int loader_waves;
  int mma_waves;
  int load_bytes;          // bytes of a patch load (8, or 16: needs 16-byte aligned channel planes)
  int halves;              // halves of output channels a workgroup computes (bi rows each)
  std::once_flag once;
  int scratch_bytes = 0;   // per-lane scratch memory of the built kernel (register spills)
  bool fits = true;        // a workgroup of `threads` fits a compute unit's registers
  int static_lds = 0;      // must stay 0: the kernel addresses dynamic LDS from byte 0
};
// wmode: NCHW_W_KCTRS (0), NCHW_W_KCRS (1), NCHW_W_PACKED (2)
ConvNchwInstance* pick_conv_nchw_f16(int ti, int tj, int wmode, int pt, int nwl, int lb);
ConvNchwInstance* pick_conv_nchw_bf16(int ti, int tj, int wmode, int pt, int nwl, int lb);
ConvNchwInstance* pick_conv_nchw_i8(int ti, int tj, int wmode, int pt, int nwl, int lb);
void launch_conv_pack_weights(int es, const void* w, void* out, int K, int C, int TRS, hipStream_t stream);

#ifdef AMOS_CONV_NCHW_KERNEL_INCLUDED
template <int DT, int BI, int BJ, int WI, int WJ, int PTL, int WMODE, int NWL, int LB, int HV = 1>
ConvNchwInstance* conv_nchw_instance() {
  static ConvNchwInstance inst;
  static const char* dtn[] = {"f16", "bf16", "i8"};
  static const char* wmn[] = {",kctrs", ",kcrs", ",packed"};
  static std::string name = std::string("amos_conv_nchw<") + dtn[DT] + "," + (HV > 1 ? std::to_string(HV) + "x" : std::string()) + std::to_string(BI) + "x" +
                            std::to_string(BJ) + "," + std::to_string(WI * WJ) + "+" + std::to_string(NWL) + "w" +
                            wmn[WMODE] + (LB == 16 ? ",ld16" : "") + (PTL > 1 ? ",pt" + std::to_string(PTL) + ">" : std::string(">"));
  inst.fn = amos_conv_nchw<DT, BI, BJ, WI, WJ, PTL, WMODE, NWL, LB, HV>;
  inst.halves = HV;
  inst.name = name.c_str();
  inst.threads = 64 * (WI * WJ + NWL);
  inst.bi = BI;
  inst.bj = BJ;
  inst.groups_per_thread = PTL;
  inst.loader_waves = NWL;
  inst.mma_waves = WI * WJ;
  inst.load_bytes = LB;
  return &inst;
}
// 64-row tiles: eight matrix-core waves, 32-row tiles: four; beside them nwl loader waves, which
// take 16 * nwl load groups of the patch per round (pt = rounds)
template <int DT, int WMODE, int PTL, int NWL, int LB = 8>
ConvNchwInstance* pick_conv_nchw_p(int ti, int tj) {
  if (ti == 64 && tj == 128) return conv_nchw_instance<DT, 64, 128, 2, 4, PTL, WMODE, NWL, LB>();
  if (ti == 64 && tj == 256) return conv_nchw_instance<DT, 64, 256, 1, 8, PTL, WMODE, NWL, LB>();
  if (ti == 32 && tj == 128) return conv_nchw_instance<DT, 32, 128, 1, 4, PTL, WMODE, NWL, LB>();
  if (ti == 32 && tj == 256) return conv_nchw_instance<DT, 32, 256, 1, 4, PTL, WMODE, NWL, LB>();
  // 128 rows: two halves of 64 that share every macro step's patch
  if (ti == 128 && tj == 256) return conv_nchw_instance<DT, 64, 256, 1, 8, PTL, WMODE, NWL, LB, 2>();
  if (ti == 128 && tj == 128) return conv_nchw_instance<DT, 64, 128, 2, 4, PTL, WMODE, NWL, LB, 2>();
  return nullptr;
}
// lb: bytes of a patch load; 16 only for 16-bit types, one round, and not with weights whose taps
// are unaligned runs (3-d without packing).  The staging
// registers of a loader thread are pt * (16 channels' worth of loads): int8 (sixteen channels per
// chunk) and 16-byte loads take one round only.
template <int DT, int WMODE>
ConvNchwInstance* pick_conv_nchw_t(int ti, int tj, int pt, int nwl, int lb) {
  if (nwl != 4) return nullptr;
  if (lb == 16) {
    if constexpr (WMODE != NCHW_W_KCTRS && DT != DT_I8) {
      if (pt == 1) return pick_conv_nchw_p<DT, WMODE, 1, 4, 16>(ti, tj);
    }
    return nullptr;
  }
  if (pt == 1) return pick_conv_nchw_p<DT, WMODE, 1, 4>(ti, tj);
  if constexpr (DT != DT_I8) {
    if (pt == 2) return pick_conv_nchw_p<DT, WMODE, 2, 4>(ti, tj);
  }
  return nullptr;
}
template <int DT>
ConvNchwInstance* pick_conv_nchw_tile(int ti, int tj, int wmode, int pt, int nwl, int lb) {
  return wmode == NCHW_W_PACKED ? pick_conv_nchw_t<DT, NCHW_W_PACKED>(ti, tj, pt, nwl, lb)
         : wmode == NCHW_W_KCRS ? pick_conv_nchw_t<DT, NCHW_W_KCRS>(ti, tj, pt, nwl, lb)
                                : pick_conv_nchw_t<DT, NCHW_W_KCTRS>(ti, tj, pt, nwl, lb);
}
#endif

Instance* pick_f16_tvec(int cl, int ti, int tj);
Instance* pick_bf16_tvec(int cl, int ti, int tj);
Instance* pick_f16_vec(int cl, int ti, int tj);
Instance* pick_f16_strided(int cl, int ti, int tj);
Instance* pick_bf16_vec(int cl, int ti, int tj);
Instance* pick_bf16_strided(int cl, int ti, int tj);
Instance* pick_i8_vec(int cl, int ti, int tj);
Instance* pick_i8_strided(int cl, int ti, int tj);

}  // namespace amos
