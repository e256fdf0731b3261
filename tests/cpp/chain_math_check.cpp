// Exhaustive host-side check of the persistent chain's work decomposition (llama.cl_amd/csrc/chain_math.h):
// replays, for many shapes and grid sizes, exactly the index arithmetic the kernel performs and verifies
// that every step of an FC is streamed once, that the fixed-size LDS tables are never overrun and that
// every partial-sum slot of every strip is written exactly once (by its owner or as a zero).
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "chain_math.h"

using namespace llmops;

static int check(int Ng, int T, int P) {
    ChainGeom g;
    int active = 0, contrib = 0;
    if (!chain_plan_geom(Ng, T, P, g, active, contrib)) return 1;  // rejected shapes are fine
    std::vector<int> seen((size_t)g.Ttot, 0);
    std::vector<int> slots((size_t)Ng * contrib, 0);
    for (int wg = 0; wg < P; wg++) {
        const int ga = chain_wg_begin(g, wg), gb = chain_wg_end(g, wg);
        if (ga > gb || gb > g.Ttot) return -1;
        if (ga == gb) {
            if (wg < active) return -2;
            continue;
        }
        if (wg >= active) return -3;
        const int s_lo = ga / T, s_hi = (gb - 1) / T;
        if (s_hi - s_lo + 1 > kChainMaxStripsPerWg) return -4;
        int prev_b = ga;
        std::vector<int> strip_hit((size_t)(s_hi - s_lo + 1), 0);
        for (int w = 0; w < kChainWaves; w++) {
            int a, b;
            chain_wave_range(ga, gb, w, a, b);
            if (a != prev_b || b < a) return -5;
            prev_b = b;
            // the kernel's streaming loop
            int ts = a % T, nseg = 0;
            const int fs = a / T;
            for (int c = 0; c < b - a; c++) {
                seen[(size_t)(a + c)]++;
                if (ts >= T) return -6;
                if (++ts == T || c + 1 == b - a) {
                    if (nseg >= 2) return -7;  // red[wave][2][32]
                    const int s = fs + nseg;
                    if (s != (a + c) / T) return -8;
                    if (s < s_lo || s > s_hi) return -9;
                    strip_hit[(size_t)(s - s_lo)]++;
                    nseg++;
                    ts = 0;
                }
            }
        }
        if (prev_b != gb) return -10;
        // the kernel's partial-sum store
        for (int s = s_lo; s <= s_hi; s++) {
            if (strip_hit[(size_t)(s - s_lo)] == 0) return -11;
            const int first = chain_first_wg(g, s), last = chain_last_wg(g, s);
            const int c = wg - first;
            if (c < 0 || c >= contrib || wg > last) return -12;
            slots[(size_t)s * contrib + c]++;
            if (c == 0)
                for (int z = last - first + 1; z < contrib; z++) slots[(size_t)s * contrib + z]++;
        }
    }
    for (int v : seen)
        if (v != 1) return -13;
    for (int v : slots)
        if (v != 1) return -14;
    return 0;
}

int main() {
    long ok = 0, rejected = 0;
    const int grids[] = {1, 2, 7, 64, 104, 128, 255, 256, 304};
    for (int P : grids)
        for (int T = 1; T <= 130; T += (T < 40 ? 1 : 7))
            for (int Ng = 1; Ng <= 1800; Ng += (Ng < 70 ? 1 : 37)) {
                const int rc = check(Ng, T, P);
                if (rc < 0) {
                    std::printf("FAIL rc=%d Ng=%d T=%d P=%d\n", rc, Ng, T, P);
                    return 1;
                }
                (rc == 0 ? ok : rejected)++;
            }
    // the shapes of the benchmark, at the real grid
    const int shapes[][2] = {{384, 32}, {128, 32}, {688, 32}, {128, 86}, {1728, 32}, {1000, 32}, {384, 64}, {688, 64}, {128, 172}};
    for (auto& sh : shapes)
        if (check(sh[0], sh[1], 256) != 0) {
            std::printf("FAIL benchmark shape Ng=%d T=%d\n", sh[0], sh[1]);
            return 1;
        }
    std::printf("ok %ld rejected %ld\n", ok, rejected);
    return 0;
}
