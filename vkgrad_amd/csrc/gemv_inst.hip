// Instantiations of the skinny-M kernel: rows of A held 1, 2, 4, 8; K up to 512, 768, 1024, 2048.
#include "gemv_kernel.h"

namespace mg {
#define KS(dt, mp) {launch_gemv<dt, mp, 1, false>, launch_gemv<dt, mp, 1, true>, launch_gemv<dt, mp, 2, false>, launch_gemv<dt, mp, 4, false>}
#define ROW(dt) {KS(dt, 1), KS(dt, 2), KS(dt, 4), KS(dt, 8)}
gemv_launch_fn gemv_table[2][4][4] = {ROW(D_F16), ROW(D_BF16)};
#undef ROW
#undef KS
}  // namespace mg
