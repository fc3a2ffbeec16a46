#include <mutex>

#include "skinny_gemm_kernel.h"
namespace amos {
const char* skinny_gemm_name(int dt) {
  return dt == DT_F16 ? "amos_skinny_gemm<f16>" : dt == DT_BF16 ? "amos_skinny_gemm<bf16>" : "amos_skinny_gemm<i8>";
}
template <int DT, int MSP>
static hipError_t skinny_launch(const SkinnyParams& p, size_t lds, hipStream_t stream) {
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute((const void*)amos_skinny_gemm<DT, MSP>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)kSkinnyMaxLds);
  });
  if (attr_err != hipSuccess) return attr_err;
  hipLaunchKernelGGL((amos_skinny_gemm<DT, MSP>), dim3((p.NB + 15) / 16), dim3(256), lds, stream, p);
  return hipGetLastError();
}
template <int DT>
static hipError_t skinny_pick(const SkinnyParams& p, hipStream_t stream) {
  const size_t lds = (size_t)skinny_gemm_lds(p.MS, p.K, Mfma<DT>::ES);
  if (p.MS < 1 || p.MS > kSkinnyMaxRows || (int64_t)lds > kSkinnyMaxLds || p.NB < 1) return hipErrorInvalidValue;
  if (p.MS <= 1) return skinny_launch<DT, 1>(p, lds, stream);
  if (p.MS <= 2) return skinny_launch<DT, 2>(p, lds, stream);
  if (p.MS <= 4) return skinny_launch<DT, 4>(p, lds, stream);
  return skinny_launch<DT, 8>(p, lds, stream);
}
hipError_t launch_skinny_gemm(int dt, const SkinnyParams& p, hipStream_t stream) {
  if (dt == DT_F16) return skinny_pick<DT_F16>(p, stream);
  if (dt == DT_BF16) return skinny_pick<DT_BF16>(p, stream);
  return skinny_pick<DT_I8>(p, stream);
}
}  // namespace amos
