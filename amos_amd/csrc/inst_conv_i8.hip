#include "conv_fprop_kernel.h"
#include "igemm_instances.h"
namespace amos {
ConvInstance* pick_conv_i8(int ti, int tj, int pls, int occ) { return pick_conv_tile<DT_I8>(ti, tj, pls, occ); }
}  // namespace amos
