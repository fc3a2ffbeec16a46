#include "gemm_tn_kernel.h"
#include "igemm_instances.h"
namespace amos {
template <int DT, int WI, int WJ, int BI, int BJ, int NS>
static TnInstance* tn_instance() {
  static TnInstance inst;
  static const char* dtn[] = {"f16", "bf16", "i8"};
  static std::string name = std::string("amos_gemm_tn<") + dtn[DT] + "," + std::to_string(BI) + "x" +
                            std::to_string(BJ) + "," + std::to_string(WI * WJ) + "w>";
  inst.fn = amos_gemm_tn<DT, WI, WJ, BI, BJ, NS>;
  inst.lds = NS * (BI + BJ) * 128;
  inst.threads = 64 * WI * WJ;
  inst.name = name.c_str();
  return &inst;
}
template <int DT>
static TnInstance* pick_tn(int ti, int tj, int waves) {
  if (waves != 8) return nullptr;   // (a four-wave 256x256 instance existed: spills, slower, withdrawn)
  // (wave grid 4 x 2, wave tile 64x128: 901 us on fp16 8192^3 where 2 x 4 took 905)
  if (ti == 256 && tj == 256) return tn_instance<DT, 4, 2, 256, 256, 2>();
  if (ti == 128 && tj == 128) return tn_instance<DT, 2, 4, 128, 128, 2>();
  if (ti == 128 && tj == 256) return tn_instance<DT, 2, 4, 128, 256, 3>();
  if (ti == 256 && tj == 128) return tn_instance<DT, 4, 2, 256, 128, 3>();
  return nullptr;
}
TnInstance* pick_gemm_tn(int dt, int ti, int tj, int waves) {
  if (dt == DT_F16) return pick_tn<DT_F16>(ti, tj, waves);
  if (dt == DT_BF16) return pick_tn<DT_BF16>(ti, tj, waves);
  if (dt == DT_I8) return pick_tn<DT_I8>(ti, tj, waves);
  return nullptr;
}
}  // namespace amos
