#include "conv_nchw_kernel.h"
#include "igemm_instances.h"
namespace amos {
ConvNchwInstance* pick_conv_nchw_i8(int ti, int tj, int wmode, int pt) { return pick_conv_nchw_tile<DT_I8>(ti, tj, wmode, pt); }
}  // namespace amos
