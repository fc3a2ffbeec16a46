#include "gemm_tn_kernel.h"
#include "igemm_instances.h"
namespace amos {
template <int DT, int WI, int WJ>
static TnInstance* tn_instance(const char* name) {
  static TnInstance inst;
  inst.fn = amos_gemm_tn<DT, WI, WJ>;
  inst.lds = 4 * 256 * 128;
  inst.threads = 64 * WI * WJ;
  inst.name = name;
  return &inst;
}
TnInstance* pick_gemm_tn(int dt, int waves) {
  if (waves == 4) {
    if (dt == DT_F16) return tn_instance<DT_F16, 2, 2>("amos_gemm_tn<f16,256x256,4w>");
    if (dt == DT_BF16) return tn_instance<DT_BF16, 2, 2>("amos_gemm_tn<bf16,256x256,4w>");
    if (dt == DT_I8) return tn_instance<DT_I8, 2, 2>("amos_gemm_tn<i8,256x256,4w>");
  } else if (waves == 8) {
    if (dt == DT_F16) return tn_instance<DT_F16, 2, 4>("amos_gemm_tn<f16,256x256,8w>");
    if (dt == DT_BF16) return tn_instance<DT_BF16, 2, 4>("amos_gemm_tn<bf16,256x256,8w>");
    if (dt == DT_I8) return tn_instance<DT_I8, 2, 4>("amos_gemm_tn<i8,256x256,8w>");
  }
  return nullptr;
}
}  // namespace amos
