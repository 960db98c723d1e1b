// Host-side check of the workgroup -> output tile map of the GEMM kernels (kernels.h: make_tile_map, xcd_tile).
// For every grid shape given on stdin ("row_tiles tok_tiles concurrent" per line) it verifies that
//   * every tile is visited exactly once and workgroups past the last tile get the out-of-range coordinate,
//   * the eight XCDs (workgroup id modulo 8) get tile counts that differ by at most one stretch remainder,
//   * the tiles one XCD works on at a time (consecutive stretch positions) stay within a few blocks of the map.
// Prints "ok <shapes>" or the first violation; no device code runs.
#include <cstdio>
#include <cstdlib>
#include <vector>
#include "kernels.h"

using namespace chip;

int main() {
    long rt, tt, conc, shapes = 0;
    while (scanf("%ld %ld %ld", &rt, &tt, &conc) == 3) {
        const TileMap m = make_tile_map(rt, tt, (int)conc);
        if ((long)m.tiles != rt * tt || m.grid < m.tiles || m.grid % XCDS != 0 || m.grid - m.tiles >= (unsigned)XCDS) {
            printf("bad sizes for %ld x %ld: tiles %u grid %u\n", rt, tt, m.tiles, m.grid);
            return 1;
        }
        std::vector<int> seen((size_t)(rt * tt), 0);
        long per_xcd[XCDS] = {0};
        for (unsigned wg = 0; wg < m.grid; wg++) {
            const TileCoord t = xcd_tile(wg, m);
            if (t.row_tile == rt && t.tok_tile == tt) continue;                      // idle workgroup
            if (t.row_tile < 0 || t.row_tile >= rt || t.tok_tile < 0 || t.tok_tile >= tt) {
                printf("out of range for %ld x %ld: wg %u -> (%d, %d)\n", rt, tt, wg, t.row_tile, t.tok_tile);
                return 1;
            }
            seen[(size_t)t.row_tile * tt + t.tok_tile]++;
            per_xcd[wg % XCDS]++;
        }
        for (size_t i = 0; i < seen.size(); i++)
            if (seen[i] != 1) {
                printf("tile (%zu, %zu) of %ld x %ld visited %d times\n", i / tt, i % tt, rt, tt, seen[i]);
                return 1;
            }
        long lo = per_xcd[0], hi = per_xcd[0];
        for (int x = 1; x < XCDS; x++) { lo = per_xcd[x] < lo ? per_xcd[x] : lo; hi = per_xcd[x] > hi ? per_xcd[x] : hi; }
        if (hi - lo > (long)XCDS) {
            printf("unbalanced XCDs for %ld x %ld: %ld .. %ld tiles\n", rt, tt, lo, hi);
            return 1;
        }
        // locality: a window of `sr * sc` consecutive stretch positions of one XCD stays within a few blocks (remainder
        // blocks at the edges are at least half a block in each direction, so a window covers at most four of them along
        // the rows and two along the tokens); a row-major numbering of a wide grid fails this
        const unsigned window = (unsigned)(m.sr * m.sc);
        for (int x = 0; x < XCDS; x++) {
            for (unsigned s0 = 0; s0 + window <= m.per_xcd; s0 += window) {
                std::vector<char> rows((size_t)rt, 0), toks((size_t)tt, 0);
                long nr = 0, nt = 0;
                for (unsigned s = s0; s < s0 + window; s++) {
                    const TileCoord t = xcd_tile(s * XCDS + x, m);
                    if (t.row_tile == rt) continue;
                    if (!rows[t.row_tile]) { rows[t.row_tile] = 1; nr++; }
                    if (!toks[t.tok_tile]) { toks[t.tok_tile] = 1; nt++; }
                }
                if (nr > 4L * m.sr + 1 || nt > 2L * m.sc) {
                    printf("window of XCD %d at %u of %ld x %ld touches %ld row tiles and %ld token tiles (block %d x %d)\n", x,
                           s0, rt, tt, nr, nt, m.sr, m.sc);
                    return 1;
                }
            }
        }
        shapes++;
    }
    printf("ok %ld\n", shapes);
    return 0;
}
