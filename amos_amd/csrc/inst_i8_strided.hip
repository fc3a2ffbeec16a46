#include "igemm_instances.h"
namespace amos {
Instance* pick_i8_strided(int cl, int ti, int tj) { return pick_col<DT_I8, LD_STRIDED>(cl, ti, tj); }
}  // namespace amos
