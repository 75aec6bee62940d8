// Walks the workgroup-id -> tile map of the Gram kernel on the CPU: in the symmetric mode every tile on or
// above the diagonal must be met exactly once, no id may yield a tile below it, and the XCDs (id modulo 8)
// must get nearly equal shares; in the full mode every tile exactly once.
#include <cstdio>
#include <vector>
#include "gram_tiles.h"

int main() {
    int worst = 0;
    for (int nt = 1; nt <= 140; ++nt) {
        long long per;
        TileMap tm = gram_tile_map(nt, nt, true, per);
        std::vector<int> seen((size_t)nt * nt, 0);
        long long share[NXCD] = {0};
        for (long long b = 0; b < per * NXCD; ++b) {
            int ti, tj;
            tile_of_block<true>((unsigned)b, nt, nt, tm, ti, tj);
            if (ti < 0) continue;
            if (ti > tj || tj >= nt) { std::printf("nt=%d id=%lld: tile (%d,%d) outside the upper triangle\n", nt, b, ti, tj); return 1; }
            ++seen[(size_t)ti * nt + tj];
            ++share[b % NXCD];
        }
        for (int i = 0; i < nt; ++i)
            for (int j = i; j < nt; ++j)
                if (seen[(size_t)i * nt + j] != 1) { std::printf("nt=%d: tile (%d,%d) met %d times\n", nt, i, j, seen[(size_t)i * nt + j]); return 1; }
        long long lo = share[0], hi = share[0];
        for (int x = 1; x < NXCD; ++x) { lo = share[x] < lo ? share[x] : lo; hi = share[x] > hi ? share[x] : hi; }
        // whole super-tiles (nt a multiple of 8): the shares differ by the leftover diagonal tiles only
        if (nt % SUPER == 0) {
            if (hi - lo > 1) { std::printf("nt=%d: XCD shares %lld..%lld\n", nt, lo, hi); return 1; }
            if ((int)(hi - lo) > worst) worst = (int)(hi - lo);
        }
    }
    for (int nti = 1; nti <= 40; nti += 3)
        for (int ntj = 1; ntj <= 40; ntj += 5) {
            long long per;
            TileMap tm = gram_tile_map(nti, ntj, false, per);
            std::vector<int> seen((size_t)nti * ntj, 0);
            for (long long b = 0; b < per * NXCD; ++b) {
                int ti, tj;
                tile_of_block<false>((unsigned)b, nti, ntj, tm, ti, tj);
                if (ti < 0) continue;
                if (ti >= nti || tj >= ntj) { std::printf("full %dx%d id=%lld: tile (%d,%d)\n", nti, ntj, b, ti, tj); return 1; }
                ++seen[(size_t)ti * ntj + tj];
            }
            for (size_t e = 0; e < seen.size(); ++e)
                if (seen[e] != 1) { std::printf("full %dx%d: tile %zu met %d times\n", nti, ntj, e, seen[e]); return 1; }
        }
    std::printf("ok, largest difference between XCD shares with whole super-tiles: %d tiles\n", worst);
    return 0;
}
