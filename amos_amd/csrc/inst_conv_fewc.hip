#include <mutex>

#include "conv_fewc_kernel.h"
namespace amos {
const char* conv_fewc_name(int dt) {
  return dt == DT_F16 ? "amos_conv_few_channels<f16>" : dt == DT_BF16 ? "amos_conv_few_channels<bf16>"
                                                                       : "amos_conv_few_channels<i8>";
}
template <int DT>
static hipError_t fewc_launch(const ConvFewcParams& p, size_t lds, hipStream_t stream) {
  static std::once_flag once;
  static hipError_t attr_err = hipSuccess;
  std::call_once(once, [&] {
    attr_err = hipFuncSetAttribute((const void*)amos_conv_fewc<DT>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                   160 * 1024);
  });
  if (attr_err != hipSuccess) return attr_err;
  const int prep = p.prep_x_blocks + p.prep_w_blocks;
  if (DT == DT_I8)
    hipLaunchKernelGGL(amos_conv_fewc_prepare<unsigned char>, dim3(prep), dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL(amos_conv_fewc_prepare<unsigned short>, dim3(prep), dim3(256), 0, stream, p);
  hipLaunchKernelGGL(amos_conv_fewc<DT>, dim3(p.grid_x, p.k_tiles), dim3(512), lds, stream, p);
  return hipGetLastError();
}
hipError_t launch_conv_fewc(int dt, const ConvFewcParams& p, size_t lds, hipStream_t stream) {
  if (dt == DT_F16) return fewc_launch<DT_F16>(p, lds, stream);
  if (dt == DT_BF16) return fewc_launch<DT_BF16>(p, lds, stream);
  return fewc_launch<DT_I8>(p, lds, stream);
}
}  // namespace amos
