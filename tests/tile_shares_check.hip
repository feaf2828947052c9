// Host-side brute force of the share-out arithmetic that the decode workers and the merge kernel have in common
// (g4b::TileShares): begin() is monotone from 0 to the total, no worker below nw is left without a tile, and owner()
// inverts begin() for every tile asked.  Built host-only by tests/test_tile_shares.py; prints "<checks> checks, <bad> bad".
#include "attn_decode.hpp"

#include <cstdio>
#include <cstdlib>

int main() {
    srand(1);
    long checks = 0, bad = 0;
    for (int it = 0; it < 200000; ++it) {
        const int num_workers = 1 + rand() % 2100;
        const int total = 1 + (rand() % 3 == 0 ? rand() % 200 : (rand() % 4 == 0 ? rand() % 40000000 : rand() % 200000));
        const int shifts[3] = {-1, 0, 2};
        const g4b::TileShares s = g4b::make_tile_shares(num_workers, shifts[rand() % 3], total);
        if (s.begin(0) != 0 || s.begin(s.nw) != total) {
            ++bad;
            printf("ends: workers %d tiles %d shift %d\n", num_workers, total, s.shift);
            continue;
        }
        for (int k = 0; k < 40; ++k) {
            const int w = rand() % s.nw;
            const int64_t b0 = s.begin(w), b1 = s.begin(w + 1);
            if (b1 <= b0) {
                ++bad;
                printf("empty share: workers %d tiles %d shift %d worker %d\n", num_workers, total, s.shift, w);
                break;
            }
            const int64_t x = b0 + rand() % (b1 - b0);
            if (s.owner(x) != w || s.owner(b0) != w || s.owner(b1 - 1) != w) {
                ++bad;
                printf("owner: workers %d tiles %d shift %d worker %d tile %lld -> %d\n", num_workers, total, s.shift, w, (long long)x, s.owner(x));
                break;
            }
            ++checks;
        }
    }
    // at the benchmark's size a worker on an even XCD gets more tiles than its neighbour on an odd one
    const g4b::TileShares s = g4b::make_tile_shares(1024, 0, 36300);
    printf("shares at 36300 tiles: even %lld odd %lld\n", (long long)(s.begin(1) - s.begin(0)), (long long)(s.begin(2) - s.begin(1)));
    printf("%ld checks, %ld bad\n", checks, bad);
    return bad ? 1 : 0;
}
