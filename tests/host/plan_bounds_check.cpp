// Host-side check of the sizes the compacted backward's launch is given against what its device-made work plan can
// ask for (built and run by tests/test_plan_bounds.py with g++: the functions under test are the library's own, from
// flash-dmattn_amd/csrc/fdma_params.h).
//
// The plan (plan_block in fdma_compact.hip) deals the 128-key units of every (batch, kv head) pair to k lists in a
// snake, the lists to the 8 XCDs (list number & 7), and enters Gs * n_seg parts per unit into its XCD's list, with
// n_seg <= Sm segments; the dK/dV kernel is launched with grid / 8 workgroups per XCD and the partial sums have `slots`
// places.  Checked here, for swept pair counts, group sizes and (ragged) unit counts: no XCD list can hold more
// parts than the launch has workgroups for, and U * Gs * Sm partial slots always fit.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "fdma_params.h"

using namespace fdma;

static long long checked = 0;

static bool check(int pairs, int G, int n_max, const std::vector<int> &units) {
    int grid = 0, slots = 0;
    dkdv_split_bounds(pairs, n_max, G, grid, slots);
    const int cap = grid / 8, k = dkdv_lists_per_pair(pairs);
    int U = 0;
    for (int n : units) U += n;
    int Gs, Sm;
    dkdv_split(U, G, Gs, Sm);
    checked++;
    if (U == 0) return true;
    if (Gs * Sm <= 1 || pairs >= DKDV_ENOUGH_UNITS || pairs * k > 1024) {
        // no split: the kernel walks unit lists of plan[3] = list_len(largest pair) entries per list
        int largest = 0;
        for (int n : units) largest = n > largest ? n : largest;
        const long long need = (long long)dkdv_list_len(largest, k) * (pairs * k / 8);
        if (need > cap) {
            std::printf("unit lists do not fit: pairs %d G %d n_max %d largest %d: need %lld per XCD, launch has %d\n", pairs, G, n_max, largest, need, cap);
            return false;
        }
        return true;
    }
    long long per_xcd[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int i = 0; i < pairs; i++)
        for (int un = 0; un < units[i]; un++) per_xcd[(i * k + dkdv_list_of(un, k)) & 7] += (long long)Gs * Sm;  // n_seg at its maximum
    for (int x = 0; x < 8; x++)
        if (per_xcd[x] > cap) {
            std::printf("parts do not fit: pairs %d G %d n_max %d U %d Gs %d Sm %d: XCD %d holds %lld parts, launch has %d\n", pairs, G, n_max, U, Gs,
                        Sm, x, per_xcd[x], cap);
            return false;
        }
    if ((long long)U * Gs * Sm > slots) {
        std::printf("partial slots do not fit: pairs %d G %d n_max %d U %d Gs %d Sm %d: %lld > %d\n", pairs, G, n_max, U, Gs, Sm, (long long)U * Gs * Sm, slots);
        return false;
    }
    return true;
}

int main() {
    const int Gs_list[] = {1, 2, 3, 4, 6, 8, 12, 16, 32};
    const int nmax_list[] = {1, 2, 3, 4, 5, 7, 8, 16, 33, 64, 130, 400};
    unsigned rng = 12345u;
    auto next = [&]() { rng = rng * 1664525u + 1013904223u; return rng >> 8; };
    bool ok = true;
    for (int pairs = 1; pairs <= 72 && ok; pairs++)
        for (int G : Gs_list)
            for (int n_max : nmax_list) {
                std::vector<int> u(pairs, n_max);
                ok = ok && check(pairs, G, n_max, u);  // every pair full
                std::fill(u.begin(), u.end(), 0);
                u[pairs - 1] = n_max;
                ok = ok && check(pairs, G, n_max, u);  // one pair alone
                u[0] = n_max;
                ok = ok && check(pairs, G, n_max, u);
                for (int rep = 0; rep < 6 && ok; rep++) {  // ragged
                    for (int i = 0; i < pairs; i++) u[i] = (int)(next() % (unsigned)(n_max + 1));
                    u[next() % pairs] = n_max;
                    ok = ok && check(pairs, G, n_max, u);
                    for (int i = 0; i < pairs; i++) u[i] = (next() & 3) ? 0 : (int)(next() % (unsigned)(n_max + 1));
                    ok = ok && check(pairs, G, n_max, u);
                }
                if (!ok) break;
            }
    // monotone split: more units never means more parts per unit (what the bounds above rest on)
    for (int G : Gs_list)
        for (int U = 1; U < DKDV_ENOUGH_UNITS + 2 && ok; U++) {
            int a, b, c, d;
            dkdv_split(U, G, a, b);
            dkdv_split(U + 1, G, c, d);
            if (c * d > a * b) { std::printf("split grows: G %d U %d: %d x %d -> %d x %d\n", G, U, a, b, c, d); ok = false; }
        }
    std::printf("%s (%lld cases)\n", ok ? "OK" : "FAILED", checked);
    return ok ? 0 : 1;
}
