#include "igemm_instances.h"
namespace amos {
Instance* pick_f16_tvec(int cl, int ti, int tj) { return pick_col_tvec<DT_F16>(cl, ti, tj); }
}  // namespace amos
