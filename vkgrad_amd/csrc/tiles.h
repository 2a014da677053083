// The tile table: every block-tile configuration the library is built with.
// The analogue of the reference's CONFIGS comprehension (kernels.py:326-331).
//
// Two kernel families share one id space:
//   register-staged (gemm_kernel.h): any shape and alignment
//     V(id, BM, BN, BK, WGM, WGN)
//   direct-to-LDS   (gemm_dma_kernel.h): aligned operands and pitches
//     D(id, BM, BN, BK, WGM, WGN, NSTAGE, fallback_id) — fallback_id names the
//     register-staged tile of the same BM x BN used when the preconditions fail.
//   persistent direct-to-LDS: additionally K slices that are multiples of BK
//     P(id, BM, BN, BK, WGM, WGN, NSTAGE, fallback_id) — falls back to the
//     one-tile-per-workgroup direct-to-LDS tile of the same shape.
//   stream-K: the persistent kernel again, but the tiles that do not fill a whole
//     round of the resident grid are cut along K into equal pieces, one per workgroup
//     (pieces meet in the context's workspace), so the last round fills the chip too.
//     S(id, BM, BN, BK, WGM, WGN, NSTAGE, fallback_id) — falls back to the
//     persistent tile of the same shape (no workspace, or ragged K).
//   skinny-M stream (gemv_kernel.h): NT layout with at most 8 rows of A and K <= 2048;
//     no matrix cores, B is read once as it lies in memory.
//     G(id, BM, BN, BK, fallback_id) — BM rows of A at most, BN output columns per
//     workgroup, BK elements of K per register chunk; falls back to a skinny
//     register-staged tile.
//   ping-pong direct-to-LDS (gemm_pp_kernel.h): the preconditions of the direct-to-LDS tiles;
//     the two wavefronts of a SIMD alternate between reading operands and multiplying.
//     Q(id, BM, BN, BK, WGM, WGN, NSTAGE, fallback_id)
//   skinny-M stream on the matrix cores (skinny_kernel.h): NT layout, at most BM rows of A, which
//     sits in LDS whole; every wavefront streams 32 rows of B by itself, BK elements of K at a time.
//     W(id, bm, bn, bk, fallback_id) - BN output columns per workgroup of four wavefronts
// WGM x WGN wavefronts of 64 lanes per workgroup.
#pragma once

#define MG_TILE_LIST(V, D, P, S, G, Q, W) \
    V(0, 256, 256, 32, 2, 4)       \
    V(1, 256, 128, 64, 2, 2)       \
    V(2, 128, 256, 64, 2, 2)       \
    V(3, 128, 128, 64, 2, 2)       \
    V(4, 64, 64, 64, 2, 2)         \
    V(5, 64, 256, 64, 1, 4)        \
    V(6, 32, 256, 64, 1, 4)        \
    V(7, 256, 64, 64, 4, 1)        \
    V(8, 256, 32, 64, 4, 1)        \
    D(9, 256, 256, 32, 2, 4, 4, 0) \
    D(10, 256, 256, 64, 2, 4, 2, 0) \
    D(11, 128, 128, 64, 2, 2, 2, 3) \
    D(12, 128, 256, 32, 2, 2, 3, 2) \
    D(13, 256, 128, 32, 2, 2, 3, 1) \
    D(14, 128, 128, 32, 2, 2, 3, 3) \
    P(15, 256, 256, 64, 2, 4, 2, 10) \
    P(16, 256, 256, 32, 2, 4, 4, 9) \
    P(17, 128, 128, 64, 2, 2, 2, 11) \
    S(18, 256, 256, 64, 2, 4, 2, 15) \
    S(19, 128, 128, 64, 2, 2, 2, 17) \
    G(20, 8, 64, 512, 4) \
    Q(21, 256, 256, 64, 2, 4, 2, 10) \
    W(22, 64, 128, 64, 4)

#define MG_NUM_TILES 23
