#include "conv_nchw_kernel.h"
#include "igemm_instances.h"
namespace amos {
void launch_conv_pack_weights(int es, const void* w, void* out, int K, int C, int TRS, hipStream_t stream) {
  const int chunks = C / (16 / es);
  if (TRS == 9 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)out & 15) == 0) {
    const int units = K * chunks;
    const int nb = (units + 255) / 256 < 4096 ? (units + 255) / 256 : 4096;
    const NchwDiv du = nchw_make_div((uint32_t)chunks);
    if (es == 2)
      hipLaunchKernelGGL(amos_conv_pack_weights9_kernel<2>, dim3(nb), dim3(256), 0, stream, (const char*)w, (char*)out, K, C, du);
    else
      hipLaunchKernelGGL(amos_conv_pack_weights9_kernel<1>, dim3(nb), dim3(256), 0, stream, (const char*)w, (char*)out, K, C, du);
    return;
  }
  const int64_t total = (int64_t)K * TRS * chunks;
  const int blocks = (int)((total + 255) / 256 < 8192 ? (total + 255) / 256 : 8192);
  const NchwDiv dc = nchw_make_div((uint32_t)chunks), dt = nchw_make_div((uint32_t)TRS);
  if (es == 2)
    hipLaunchKernelGGL(amos_conv_pack_weights_kernel<unsigned short>, dim3(blocks), dim3(256), 0, stream,
                       (const unsigned short*)w, (unsigned short*)out, K, C, TRS, dc, dt);
  else
    hipLaunchKernelGGL(amos_conv_pack_weights_kernel<unsigned char>, dim3(blocks), dim3(256), 0, stream,
                       (const unsigned char*)w, (unsigned char*)out, K, C, TRS, dc, dt);
}
}  // namespace amos
