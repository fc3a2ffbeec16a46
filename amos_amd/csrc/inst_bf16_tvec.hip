#include "igemm_instances.h"
namespace amos {
Instance* pick_bf16_tvec(int cl, int ti, int tj) { return pick_col_tvec<DT_BF16>(cl, ti, tj); }
}  // namespace amos
