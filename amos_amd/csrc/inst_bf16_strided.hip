#include "igemm_instances.h"
namespace amos {
Instance* pick_bf16_strided(int cl, int ti, int tj) { return pick_col<DT_BF16, LD_STRIDED>(cl, ti, tj); }
}  // namespace amos
