// Workgroup id -> tile of the Gram matrix (the launch geometry of gram.hip), as plain C++ so that the
// host can walk the same map (the launch does, and so does a CPU test of the map).
#pragma once
#include <math.h>
#ifndef __HIPCC__
#define QMLL_HD inline
#else
#define QMLL_HD __host__ __device__ __forceinline__
#endif

constexpr int TILE = 128;     // C tile edge per workgroup
constexpr int SUPER = 8;      // tiles per edge of a super-tile (L2 locality unit)
constexpr int NXCD = 8;       // workgroup ids go round-robin over the 8 XCDs

// Workgroup id -> C tile.  Hardware deals consecutive workgroup ids to the 8 XCDs in turn
// and every XCD has its own L2.  The tiles are grouped in super-tiles of 8x8, dealt to the
// XCDs round-robin; the k-th workgroup of an XCD works on tile k%64 of that XCD's (k/64)-th
// super-tile, so the ~64 tiles an XCD runs at a time share 16 panels of Z.
// Symmetric mode: every XCD must get the same number of REAL tiles per id range, because
// ids are handed out in order and a full XCD holds back the ids of the others.  So the
// super-tiles strictly above the diagonal (64 tiles each) are dealt first, then the diagonal
// super-tiles, whose 36 tiles on or above the diagonal are numbered without gaps.  Whole
// super-tiles are dealt as long as every XCD gets one; the off_rem super-tiles left over are
// shared by all XCDs, XCD x taking tile row x of each (at F = 8192 that is 4 of 28: dealt whole
// they would leave four XCDs with 292 tiles and four with 228), and the tiles of the diag_rem
// diagonal super-tiles left over go round the XCDs one by one.
constexpr int DIAG_TILES = SUPER * (SUPER + 1) / 2;

struct TileMap {
    int off_per;    // whole super-tiles per XCD: the strictly-upper ones (symmetric) / all (full mode)
    int off_rem;    // those left over (fewer than one per XCD), shared by the XCDs row by row
    int diag_per;   // symmetric: whole diagonal super-tiles per XCD
    int diag_rem;   // symmetric: diagonal super-tiles left over, dealt tile by tile
    // split launch of the last tiles (symmetric mode with a workspace, see gram_launch): workgroup w
    // takes rows [piece * piece_rows, ...) of tile id tail_first + w / pieces, piece = w % pieces, and
    // writes its partial tile to the workspace; pieces = 0: the ordinary launch
    int pieces;
    int piece_rows;
    unsigned tail_first;
};

template <bool SYM>
QMLL_HD void tile_of_block(unsigned b, int nti, int ntj, TileMap tm, int& ti, int& tj) {
    const unsigned xcd = b % NXCD, k = b / NXCD;
    const int sr_n = (nti + SUPER - 1) / SUPER, sc_n = (ntj + SUPER - 1) / SUPER;
    ti = tj = -1;
    if (!SYM) {
        unsigned g, in_super;
        if (k < (unsigned)tm.off_per * (SUPER * SUPER)) {
            g = (k / (SUPER * SUPER)) * NXCD + xcd;
            in_super = k % (SUPER * SUPER);
        } else {                                                // tile row xcd of a shared super-tile
            const unsigned k1 = k - (unsigned)tm.off_per * (SUPER * SUPER);
            if (k1 >= (unsigned)tm.off_rem * SUPER) return;
            g = (unsigned)tm.off_per * NXCD + k1 / SUPER;
            in_super = xcd * SUPER + k1 % SUPER;
        }
        const int sr = (int)(g / sc_n), sc = (int)(g % sc_n);
        if (sr >= sr_n) return;
        ti = sr * SUPER + (int)(in_super / SUPER);
        tj = sc * SUPER + (int)(in_super % SUPER);
    } else if (k < (unsigned)tm.off_per * (SUPER * SUPER) + (unsigned)tm.off_rem * SUPER) {
        unsigned g, in_super;
        if (k < (unsigned)tm.off_per * (SUPER * SUPER)) {
            g = (k / (SUPER * SUPER)) * NXCD + xcd;
            in_super = k % (SUPER * SUPER);
        } else {                                                // tile row xcd of a shared super-tile
            const unsigned k1 = k - (unsigned)tm.off_per * (SUPER * SUPER);
            g = (unsigned)tm.off_per * NXCD + k1 / SUPER;
            in_super = xcd * SUPER + k1 % SUPER;
        }
        const int n1 = sc_n - 1;                                // row r holds n1 - r super-tiles
        if (g >= (unsigned)(sc_n * n1 / 2)) return;
        const float bb = (float)(2 * n1 + 1);
        int r = (int)((bb - sqrtf(fmaxf(bb * bb - 8.0f * (float)g, 0.0f))) * 0.5f);
        r = r < 0 ? 0 : (r > n1 - 1 ? n1 - 1 : r);
        while (r > 0 && (unsigned)(r * n1 - (r * (r - 1)) / 2) > g) --r;
        while (r + 1 < n1 && (unsigned)((r + 1) * n1 - ((r + 1) * r) / 2) <= g) ++r;
        const int sc = r + 1 + (int)(g - (unsigned)(r * n1 - (r * (r - 1)) / 2));
        ti = r * SUPER + (int)(in_super / SUPER);
        tj = sc * SUPER + (int)(in_super % SUPER);
    } else {
        const unsigned k2 = k - (unsigned)tm.off_per * (SUPER * SUPER) - (unsigned)tm.off_rem * SUPER;
        unsigned dg;
        int t;
        if (k2 < (unsigned)tm.diag_per * DIAG_TILES) {
            dg = (k2 / DIAG_TILES) * NXCD + xcd;
            t = (int)(k2 % DIAG_TILES);
        } else {
            const unsigned u = (k2 - (unsigned)tm.diag_per * DIAG_TILES) * NXCD + xcd;
            if (u >= (unsigned)tm.diag_rem * DIAG_TILES) return;
            dg = (unsigned)tm.diag_per * NXCD + u / DIAG_TILES;
            t = (int)(u % DIAG_TILES);
        }
        if (dg >= (unsigned)sc_n) return;
        int a = 0;
        while (t >= SUPER - a) { t -= SUPER - a; ++a; }         // row a of the triangle holds 8 - a tiles
        ti = (int)dg * SUPER + a;
        tj = (int)dg * SUPER + a + t;
    }
    if (ti >= nti || tj >= ntj) ti = tj = -1;
}


// the map of a launch over nti x ntj tiles (symmetric: ntj x ntj, tiles on or above the diagonal) and
// the number of workgroup ids every XCD gets
inline TileMap gram_tile_map(int nti, int ntj, bool sym, long long& per_xcd) {
    const long long sr = (nti + SUPER - 1) / SUPER, sc = (ntj + SUPER - 1) / SUPER;
    TileMap tm;
    if (sym) {
        const long long noff = sc * (sc - 1) / 2;
        tm.off_per = (int)(noff / NXCD);
        tm.off_rem = (int)(noff % NXCD);
        tm.diag_per = (int)(sc / NXCD);
        tm.diag_rem = (int)(sc % NXCD);
        per_xcd = (long long)tm.off_per * SUPER * SUPER + (long long)tm.off_rem * SUPER +
                  (long long)tm.diag_per * DIAG_TILES + ((long long)tm.diag_rem * DIAG_TILES + NXCD - 1) / NXCD;
    } else {
        tm.off_per = (int)(sr * sc / NXCD);
        tm.off_rem = (int)(sr * sc % NXCD);
        tm.diag_per = 0;
        tm.diag_rem = 0;
        per_xcd = (long long)tm.off_per * SUPER * SUPER + (long long)tm.off_rem * SUPER;
    }
    tm.pieces = 0;
    tm.piece_rows = 0;
    tm.tail_first = 0;
    return tm;
}
