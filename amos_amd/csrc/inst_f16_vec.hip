#include "igemm_instances.h"
namespace amos {
Instance* pick_f16_vec(int cl, int ti, int tj) { return pick_col<DT_F16, LD_VEC>(cl, ti, tj); }
}  // namespace amos
