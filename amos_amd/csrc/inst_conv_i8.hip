#include "conv_fprop_kernel.h"
#include "igemm_instances.h"
namespace amos {
ConvInstance* pick_conv_i8(int ti, int tj, int waves, int pls, int occ, int w9) {
  return pick_conv_tile<DT_I8>(ti, tj, waves, pls, occ, w9);
}
}  // namespace amos
