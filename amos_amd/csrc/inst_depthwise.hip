#include <string>

#include "depthwise_kernel.h"
namespace amos {
template <int DT, int KIND>
static const char* dw_name() {
  static const char* dtn[] = {"f16", "bf16", "i8"};
  static const char* kn[] = {"", ",3x3", ",3x3/2", ",3x3"};
  static std::string name = std::string("amos_depthwise_conv<") + dtn[DT] + kn[KIND] + ">";
  return name.c_str();
}
template <int DT>
static const char* dw_name_of(int kind) {
  return (kind == DW_3x3_S1 || kind == DW_3x3_S1_SMALL) ? dw_name<DT, DW_3x3_S1>()
         : kind == DW_3x3_S2 ? dw_name<DT, DW_3x3_S2>() : dw_name<DT, DW_GENERIC>();
}
const char* depthwise_name(int dt, int kind) {
  return dt == DT_F16 ? dw_name_of<DT_F16>(kind) : dt == DT_BF16 ? dw_name_of<DT_BF16>(kind) : dw_name_of<DT_I8>(kind);
}
template <int DT>
static void dw_launch(int kind, const DepthwiseParams& p, dim3 grid, hipStream_t stream) {
  if (kind == DW_3x3_S1)
    hipLaunchKernelGGL((amos_depthwise_conv<DT, DW_3x3_S1>), grid, dim3(256), 0, stream, p);
  else if (kind == DW_3x3_S1_SMALL)
    hipLaunchKernelGGL((amos_depthwise_conv<DT, DW_3x3_S1_SMALL>), grid, dim3(256), 0, stream, p);
  else if (kind == DW_3x3_S2)
    hipLaunchKernelGGL((amos_depthwise_conv<DT, DW_3x3_S2>), grid, dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL((amos_depthwise_conv<DT, DW_GENERIC>), grid, dim3(256), 0, stream, p);
}
void launch_depthwise(int dt, int kind, const DepthwiseParams& p, hipStream_t stream) {
  const unsigned want = (p.items + 255u) / 256u;
  dim3 grid(want < (1u << 20) ? want : (1u << 20));
  if (dt == DT_F16) dw_launch<DT_F16>(kind, p, grid, stream);
  else if (dt == DT_BF16) dw_launch<DT_BF16>(kind, p, grid, stream);
  else dw_launch<DT_I8>(kind, p, grid, stream);
}
}  // namespace amos
