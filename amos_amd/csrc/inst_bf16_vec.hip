#include "igemm_instances.h"
namespace amos {
Instance* pick_bf16_vec(int cl, int ti, int tj) { return pick_col<DT_BF16, LD_VEC>(cl, ti, tj); }
}  // namespace amos
