// Instantiations of the GEMM template: layout NT, dtype F16, every tile, aligned and general.
#include "gemm_kernel.h"
#include "tiles.h"

namespace mg {
#define X(id, bm, bn, bk, wgm, wgn)                                                   \
    {launch_gemm<L_NT, D_F16, bm, bn, bk, wgm, wgn, false>, launch_gemm<L_NT, D_F16, bm, bn, bk, wgm, wgn, true>},
launch_fn launch_table_nt_f16[MG_NUM_TILES][2] = {MG_TILE_LIST(X)};
#undef X
}  // namespace mg
