// CPU check of the arithmetic that cuts the last round of an attention launch into pieces (SplitGeo, csrc/internal.h).
// The device code and the host planner share these formulas; here they are checked by brute force against their
// definition: the pieces of a group tile its tail steps exactly once, piece_of() inverts piece_begin(), the parts of
// a tile are numbered 0 .. n-1 without gaps and never exceed max_parts as the planner computes it.
// Compiled for the host by hipcc (the header pulls in the HIP runtime declarations); runs without a GPU.
#include <cstdio>
#include <vector>

#include "internal.h"

static int g_failures = 0;
#define CHECK(cond)                                                              \
    do {                                                                         \
        if (!(cond)) { std::printf("CHECK failed %s:%d: %s\n", __FILE__, __LINE__, #cond); ++g_failures; } \
    } while (0)

int main() {
    int cases = 0;
    for (int n_blocks : {256, 257, 300, 312, 384, 432, 511, 520, 1000, 4097})
        for (int T : {16, 17, 52, 64, 72, 1000})
            for (int cu_g : {8, 32, 38}) {
                mi::SplitGeo g{};
                g.T = T; g.n_blocks = n_blocks; g.chunk = (n_blocks + 7) / 8; g.cu_g = cu_g;
                int covered_tiles = 0;
                for (int xg = 0; xg < 8; ++xg) {
                    const int tiles = g.tiles_of(xg), full = g.full_of(xg), tail = g.tail_of(xg);
                    CHECK(tiles >= 0 && full % cu_g == 0 && full + tail == tiles && tail < cu_g);
                    covered_tiles += tiles;
                    const int S = tail * T, np = g.pieces_for(S);
                    if (S == 0) { CHECK(np == 0); continue; }
                    CHECK(np >= 1 && np <= cu_g);
                    // pieces tile [0, S) exactly, in order, none empty
                    std::vector<int> owner(S, -1);
                    CHECK(mi::SplitGeo::piece_begin(0, S, np) == 0 && mi::SplitGeo::piece_begin(np, S, np) == S);
                    for (int c = 0; c < np; ++c) {
                        const int b0 = mi::SplitGeo::piece_begin(c, S, np), b1 = mi::SplitGeo::piece_begin(c + 1, S, np);
                        CHECK(b1 > b0);
                        for (int x = b0; x < b1; ++x) { CHECK(owner[x] == -1); owner[x] = c; }
                    }
                    for (int x = 0; x < S; ++x) CHECK(owner[x] == mi::SplitGeo::piece_of(x, S, np));
                    // parts of a tile: consecutive pieces first .. last; the kernel's part index is piece - first
                    int max_parts = 0;
                    for (int tt = 0; tt < tail; ++tt) {
                        const int first = mi::SplitGeo::piece_of(tt * T, S, np), last = mi::SplitGeo::piece_of((tt + 1) * T - 1, S, np);
                        CHECK(first == owner[tt * T] && last == owner[(tt + 1) * T - 1] && last >= first);
                        max_parts = last - first + 1 > max_parts ? last - first + 1 : max_parts;
                        // walking a piece the way the kernel does visits exactly its steps of this tile
                        for (int c = first; c <= last; ++c) {
                            int s = mi::SplitGeo::piece_begin(c, S, np);
                            const int end = mi::SplitGeo::piece_begin(c + 1, S, np);
                            int seen = 0;
                            while (s < end) {
                                const int t2 = s / T, s0 = s - t2 * T, s1 = (end - t2 * T < T) ? end - t2 * T : T;
                                if (t2 == tt) seen += s1 - s0;
                                CHECK(s1 > s0);
                                s = t2 * T + s1;
                            }
                            int expect = 0;
                            for (int x = tt * T; x < (tt + 1) * T; ++x) expect += owner[x] == c;
                            CHECK(seen == expect && expect > 0);
                        }
                    }
                    CHECK(max_parts >= 1 && max_parts <= (T + (S / np) - 1) / (S / np) + 1);
                }
                CHECK(covered_tiles == n_blocks);
                ++cases;
            }
    CHECK(mi::SplitGeo::slot_bytes(128) == 256L * 128 * 2 + 2048 && mi::SplitGeo::slot_bytes(72) % 16 == 0);
    if (g_failures == 0) std::printf("test_split_geo: OK (%d configurations)\n", cases);
    return g_failures == 0 ? 0 : 1;
}
