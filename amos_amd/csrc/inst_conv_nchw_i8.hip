#include "conv_nchw_kernel.h"
#include "igemm_instances.h"
namespace amos {
ConvNchwInstance* pick_conv_nchw_i8(int ti, int tj, int wmode, int pt, int nwl, int lb) { return pick_conv_nchw_tile<DT_I8>(ti, tj, wmode, pt, nwl, lb); }
}  // namespace amos
