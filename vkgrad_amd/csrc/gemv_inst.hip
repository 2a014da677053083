// Instantiations of the skinny-M kernels.  v_dot2 stream: rows of A held 1, 2, 4, 8; K up to 512, 768, 1024, 2048.
#include "gemv_kernel.h"
#include "skinny_kernel.h"

namespace mg {
#define KS(dt, mp) {launch_gemv<dt, mp, 1, false>, launch_gemv<dt, mp, 1, true>, launch_gemv<dt, mp, 2, false>, launch_gemv<dt, mp, 4, false>}
#define ROW(dt) {KS(dt, 1), KS(dt, 2), KS(dt, 4), KS(dt, 8)}
gemv_launch_fn gemv_table[2][4][4] = {ROW(D_F16), ROW(D_BF16)};
#undef ROW
#undef KS

// the skinny-M stream on the matrix cores: one and two blocks of 32 rows of A
#define SK(dt) {launch_skinny<dt, 1, 4, SKINNY_KP, 4>, launch_skinny<dt, 2, 8, SKINNY_KP, 4>}
skinny_launch_fn skinny_table[2][SKINNY_MAX_TMB] = {SK(D_F16), SK(D_BF16)};
#undef SK
}  // namespace mg
