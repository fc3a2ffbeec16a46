#include "conv_fprop_kernel.h"
#include "igemm_instances.h"
namespace amos {
void launch_conv_prepare(int es, const ConvFpropParams& p, hipStream_t stream) {
  const int blocks = p.prep_w_blocks + p.prep_x_blocks + p.prep_z_blocks;
  if (es == 2)
    hipLaunchKernelGGL(amos_conv_prepare<unsigned short>, dim3(blocks), dim3(256), 0, stream, p);
  else
    hipLaunchKernelGGL(amos_conv_prepare<unsigned char>, dim3(blocks), dim3(256), 0, stream, p);
}
}  // namespace amos
