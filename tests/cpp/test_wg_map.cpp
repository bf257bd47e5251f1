// CPU test of the prefill launch's workgroup -> (head, query tile) mapping: for every launch shape tried, every
// pair must be visited exactly once and nothing outside the grid.  Built with g++ (no GPU needed).
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../tscale_amd/csrc/wg_map.h"

using namespace tsattn;

static long n_checked = 0;

static bool check(int n_qtiles, int n_heads, int head_dim, int period_tiles)
{
    const WgMap m = wg_plan(n_qtiles, n_heads, head_dim, 128, period_tiles);
    const uint32_t n_wg = (uint32_t)n_qtiles * (uint32_t)n_heads;
    std::vector<unsigned char> seen((size_t)n_wg, 0);
    for (uint32_t b = 0; b < n_wg; ++b) {
        int head = -1, tile = -1;
        wg_locate(m, b, n_wg, n_qtiles, head, tile);
        if (head < 0 || head >= n_heads || tile < 0 || tile >= n_qtiles) {
            printf("FAIL qtiles %d heads %d d %d period %d: block %u -> head %d tile %d (group %d)\n", n_qtiles, n_heads, head_dim,
                   period_tiles, b, head, tile, m.period_group);
            return false;
        }
        unsigned char &s = seen[(size_t)head * n_qtiles + tile];
        if (s) {
            printf("FAIL qtiles %d heads %d d %d period %d: (head %d, tile %d) visited twice\n", n_qtiles, n_heads, head_dim, period_tiles, head, tile);
            return false;
        }
        s = 1;
    }
    ++n_checked;
    return true;
}

int main()
{
    // the reciprocal division itself, divisor 1 included
    const uint32_t ds[] = {1, 2, 3, 5, 7, 8, 12, 96, 127, 128, 1000, 4096, 65535, 65536, 1000003, 0x40000000u};
    const uint32_t xs[] = {0, 1, 2, 3, 7, 8, 95, 96, 97, 1023, 1024, 65535, 65536, 1000002, 1000003, 1000004, 0x3fffffffu, 0x40000000u, 0x7ffffffeu, 0x7fffffffu};
    for (uint32_t d : ds)
        for (uint32_t x : xs) {
            uint32_t r;
            const uint32_t q = wg_divmod(x, wg_make_div(d), r);
            if (q != x / d || r != x % d) {
                printf("FAIL divmod %u / %u -> %u rem %u\n", x, d, q, r);
                return 1;
            }
        }
    bool ok = true;
    const int heads[] = {1, 2, 3, 5, 8, 12, 16, 24, 32};
    const int qtiles[] = {1, 2, 3, 4, 7, 8, 16, 24, 32, 64, 128, 256};
    for (int d : {64, 128})
        for (int h : heads)
            for (int nq : qtiles) {
                ok = check(nq, h, d, 0) && ok;
                for (int T = 1; T <= nq; ++T)
                    if (nq % T == 0) ok = check(nq, h, d, T) && ok;
                ok = check(nq, h, d, 3 * nq) && ok; // a period the grid is not a multiple of
            }
    if (!ok) return 1;
    printf("OK %ld launch shapes\n", n_checked);
    return 0;
}
