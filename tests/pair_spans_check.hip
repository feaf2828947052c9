// Host-side brute force of the walk that cuts the key tiles of a pair of query tiles into spans (g4b::pf_pair_spans,
// prefill_map.hpp): every workgroup of a pair runs the same walk and keeps its own span, so the spans must tile the
// list -- in order, without gaps or overlaps, from 0 to the total -- whatever the tile counts and the split count are,
// and no span may cost much more than a fair share.  Built host-only by tests/test_pair_spans.py; prints
// "<checks> checks, <bad> bad".
#include "prefill_map.hpp"

#include <cstdio>
#include <cstdlib>

int main() {
    long checks = 0, bad = 0;
    for (int n_first = 0; n_first <= 300; n_first += (n_first < 40 ? 1 : 13))
        for (int n_second = 0; n_second <= n_first + 2; n_second += (n_second < 40 ? 1 : 17))
            for (int nsplit = 2; nsplit <= 16; ++nsplit) {
                int expect = 0, count = 0, worst = 0;
                bool ok = true;
                g4b::pf_pair_spans(n_first, n_second, nsplit, [&](int k, int begin, int end) {
                    ok = ok && k == count && begin == expect && end >= begin;
                    // cost of the span in key tiles: its tiles plus a start for every query tile it touches
                    const int starts = (begin < n_first && end > begin ? 1 : 0) + (end > n_first && end > begin && n_second > 0 ? 1 : 0);
                    const int cost = end - begin + g4b::PF_ITEM_COST * starts;
                    worst = cost > worst ? cost : worst;
                    expect = end;
                    ++count;
                });
                ok = ok && count == nsplit && expect == n_first + n_second;
                // a fair share of tiles and starts, plus the rounding of the walk and the short span at the change-over
                const int fair = (n_first + n_second + g4b::PF_ITEM_COST * (nsplit + 1) + nsplit - 1) / nsplit;
                if (n_first + n_second >= 4 * nsplit) ok = ok && worst <= fair + 2 * g4b::PF_ITEM_COST + nsplit;
                ++checks;
                if (!ok) {
                    ++bad;
                    printf("first %d second %d splits %d: %d spans, end %d, worst cost %d of fair %d\n", n_first, n_second, nsplit, count, expect, worst, fair);
                }
            }
    printf("%ld checks, %ld bad\n", checks, bad);
    return bad ? 1 : 0;
}
