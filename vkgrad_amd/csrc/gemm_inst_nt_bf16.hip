// Instantiations of the GEMM templates: layout NT, dtype BF16, every tile.
// Entry [tile][0] serves aligned operands, [tile][1] arbitrary alignment (absent
// for direct-to-LDS tiles, which fall back to a register-staged tile instead).
// Persistent and stream-K tiles use [0] for the plain epilogue and [1] for the one with bias.
// Entry [tile][2] is the variant whose epilogue also writes the activated 16-bit output
// (forward layouts NN and NT, tiles 3, 4, 10, 11 and 21; null elsewhere).
#include "gemm_dma_kernel.h"
#include "gemm_pp_kernel.h"
#include "gemm_kernel.h"
#include "tiles.h"

namespace mg {
template <int ID, int BM, int BN, int BK, int WGM, int WGN>
constexpr launch_fn act_variant_v() {
    if constexpr ((ID == 3 || ID == 4) && L_NT != L_TN) return launch_gemm<L_NT, D_BF16, BM, BN, BK, WGM, WGN, true, true>;
    else return nullptr;
}
template <int ID, int BM, int BN, int BK, int WGM, int WGN, int NS>
constexpr launch_fn act_variant_d() {
    if constexpr ((ID == 10 || ID == 11) && L_NT != L_TN) return launch_gemm_dma<L_NT, D_BF16, BM, BN, BK, WGM, WGN, NS, true>;
    else return nullptr;
}
template <int BM, int BN, int BK, int WGM, int WGN>
constexpr launch_fn act_variant_q() {
    if constexpr (L_NT != L_TN) return launch_gemm_pp<L_NT, D_BF16, BM, BN, BK, WGM, WGN, true>;
    else return nullptr;
}
// The bias epilogue of the persistent kernels keeps its bias values in registers across the
// tile; for the 256 x 256 x 64 tiles in the NN layout that no longer fits the register file
// (the compiler spills 7 to 9 registers), so those have no such variant and hand calls with a
// bias to their fallback tile.
template <int BM, int BN, int BK, int WGM, int WGN, int NS, bool SK>
constexpr launch_fn bias_variant_p() {
    if constexpr (BM * BN <= 128 * 128 || BK < 64 || L_NT != L_NN) return launch_gemm_dmap<L_NT, D_BF16, BM, BN, BK, WGM, WGN, NS, true, SK>;
    else return nullptr;
}
#define V(id, bm, bn, bk, wgm, wgn) \
    {launch_gemm<L_NT, D_BF16, bm, bn, bk, wgm, wgn, false>, launch_gemm<L_NT, D_BF16, bm, bn, bk, wgm, wgn, true>, \
     act_variant_v<id, bm, bn, bk, wgm, wgn>()},
#define D(id, bm, bn, bk, wgm, wgn, ns, fb) \
    {launch_gemm_dma<L_NT, D_BF16, bm, bn, bk, wgm, wgn, ns>, nullptr, act_variant_d<id, bm, bn, bk, wgm, wgn, ns>()},
#define P(id, bm, bn, bk, wgm, wgn, ns, fb)                          \
    {launch_gemm_dmap<L_NT, D_BF16, bm, bn, bk, wgm, wgn, ns, false, false>, \
     bias_variant_p<bm, bn, bk, wgm, wgn, ns, false>(), nullptr},
#define G(id, bm, bn, bk, fb) {nullptr, nullptr, nullptr},   // launched through gemv_table
#define W(id, bm, bn, bk, fb) {nullptr, nullptr, nullptr},   // launched through skinny_table
#define Q(id, bm, bn, bk, wgm, wgn, ns, fb) \
    {launch_gemm_pp<L_NT, D_BF16, bm, bn, bk, wgm, wgn>, nullptr, act_variant_q<bm, bn, bk, wgm, wgn>()},
#define S(id, bm, bn, bk, wgm, wgn, ns, fb)                                \
    {launch_gemm_dmap<L_NT, D_BF16, bm, bn, bk, wgm, wgn, ns, false, true>, \
     bias_variant_p<bm, bn, bk, wgm, wgn, ns, true>(), nullptr},
launch_fn launch_table_nt_bf16[MG_NUM_TILES][3] = {MG_TILE_LIST(V, D, P, S, G, Q, W)};
#undef V
#undef D
#undef P
#undef S
#undef G
#undef Q
#undef W
}  // namespace mg
