// The tile table: every block-tile configuration the library is built with.
// X(id, BM, BN, BK, WGM, WGN) — WGM x WGN wavefronts of 64 lanes per workgroup.
// The analogue of the reference's CONFIGS comprehension (kernels.py:326-331).
#pragma once

#define MG_TILE_LIST(X)      \
    X(0, 256, 256, 64, 2, 2) \
    X(1, 256, 128, 64, 2, 2) \
    X(2, 128, 256, 64, 2, 2) \
    X(3, 128, 128, 64, 2, 2) \
    X(4, 64, 64, 64, 2, 2)   \
    X(5, 64, 256, 64, 1, 4)  \
    X(6, 32, 256, 64, 1, 4)  \
    X(7, 256, 64, 64, 4, 1)  \
    X(8, 256, 32, 64, 4, 1)

#define MG_NUM_TILES 9
