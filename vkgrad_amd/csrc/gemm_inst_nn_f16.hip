// Instantiations of the GEMM templates: layout NN, dtype F16, every tile.
// Entry [tile][0] serves aligned operands, [tile][1] arbitrary alignment (absent
// for direct-to-LDS tiles, which fall back to a register-staged tile instead).
// Persistent and stream-K tiles use [0] for the plain epilogue and [1] for the one with bias.
#include "gemm_dma_kernel.h"
#include "gemm_kernel.h"
#include "tiles.h"

namespace mg {
#define V(id, bm, bn, bk, wgm, wgn) \
    {launch_gemm<L_NN, D_F16, bm, bn, bk, wgm, wgn, false>, launch_gemm<L_NN, D_F16, bm, bn, bk, wgm, wgn, true>},
#define D(id, bm, bn, bk, wgm, wgn, ns, fb) {launch_gemm_dma<L_NN, D_F16, bm, bn, bk, wgm, wgn, ns>, nullptr},
#define P(id, bm, bn, bk, wgm, wgn, ns, fb)                          \
    {launch_gemm_dmap<L_NN, D_F16, bm, bn, bk, wgm, wgn, ns, false, false>, \
     launch_gemm_dmap<L_NN, D_F16, bm, bn, bk, wgm, wgn, ns, true, false>},
#define G(id, bm, bn, bk, fb) {nullptr, nullptr},   // launched through gemv_table
#define S(id, bm, bn, bk, wgm, wgn, ns, fb)                                \
    {launch_gemm_dmap<L_NN, D_F16, bm, bn, bk, wgm, wgn, ns, false, true>, \
     launch_gemm_dmap<L_NN, D_F16, bm, bn, bk, wgm, wgn, ns, true, true>},
launch_fn launch_table_nn_f16[MG_NUM_TILES][2] = {MG_TILE_LIST(V, D, P, S, G)};
#undef V
#undef D
#undef P
#undef S
#undef G
}  // namespace mg
