// Instantiations of the skinny-M kernel: rows of A held 1, 2, 4; K chunks held 1, 2, 4.
#include "gemv_kernel.h"

namespace mg {
#define ROW(dt)                                                                           \
    {{launch_gemv<dt, 1, 1>, launch_gemv<dt, 1, 2>, launch_gemv<dt, 1, 4>},                \
     {launch_gemv<dt, 2, 1>, launch_gemv<dt, 2, 2>, launch_gemv<dt, 2, 4>},                \
     {launch_gemv<dt, 4, 1>, launch_gemv<dt, 4, 2>, launch_gemv<dt, 4, 4>}}
gemv_launch_fn gemv_table[2][3][3] = {ROW(D_F16), ROW(D_BF16)};
#undef ROW
}  // namespace mg
