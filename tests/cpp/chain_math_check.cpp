// Exhaustive host-side check of the persistent chain's work decomposition (llama.cl_amd/csrc/chain_math.h):
// replays, for many shapes and grid sizes, exactly the index arithmetic the kernel performs and verifies
// that every step of an FC is streamed once, that the fixed-size LDS tables are never overrun and that
// every output column is finished by exactly one (unit slot, column) thread of one workgroup.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "chain_math.h"

using namespace llmops;

static int check(int Ng, int T, int us, int P, int rot) {
    ChainGeom g;
    if (!chain_plan_geom(Ng, T, us, P, rot, g)) return 1;  // rejected shapes are fine
    const int total = Ng * T;
    std::vector<int> seen((size_t)total, 0);
    std::vector<int> unit_done((size_t)g.units, 0);
    int active_seen = 0;
    for (int wg = 0; wg < P; wg++) {
        int u0, u1;
        chain_wg_units(g, wg, P, u0, u1);
        if (u0 > u1 || u1 > g.units) return -1;
        if (u0 == u1) continue;
        active_seen++;
        if (u1 - u0 > kChainServiceWaves * 64 / 32) return -2;  // one (unit slot, column) thread per output
        const int s_lo = u0 * us, s_hi = u1 * us - 1;
        std::vector<int> strip_segments((size_t)(s_hi - s_lo + 1), 0);
        int prev_b = u0 * us * T;
        for (int w = 0; w < kChainStreamWaves; w++) {
            int a, b;
            chain_wave_range(g, u0, u1, w, a, b);
            if (a != prev_b || b < a) return -3;
            prev_b = b;
            int ts = a % T, nseg = 0;
            const int fs = a / T;
            for (int c = 0; c < b - a; c++) {
                if (a + c >= total) return -4;
                seen[(size_t)(a + c)]++;
                if (++ts == T || c + 1 == b - a) {
                    if (nseg >= 2) return -5;  // red[wave][2][32]
                    const int s = fs + nseg;
                    if (s != (a + c) / T) return -6;
                    if (s < s_lo || s > s_hi) return -7;
                    strip_segments[(size_t)(s - s_lo)]++;
                    nseg++;
                    ts = 0;
                }
            }
        }
        if (prev_b != u1 * us * T) return -8;
        for (int v : strip_segments)
            if (v == 0) return -9;
        for (int u = u0; u < u1; u++) unit_done[(size_t)u]++;
    }
    if (active_seen != g.active) return -10;
    for (int v : seen)
        if (v != 1) return -11;
    for (int v : unit_done)
        if (v != 1) return -12;
    return 0;
}

int main() {
    long ok = 0, rejected = 0;
    const int grids[] = {1, 2, 7, 64, 104, 128, 255, 256, 304};
    for (int P : grids)
        for (int us = 1; us <= 2; us++)
            for (int T = 1; T <= 130; T += (T < 40 ? 1 : 7))
                for (int Ng = us; Ng <= 2100; Ng += us * (Ng < 70 ? 1 : 37)) {
                    const int rc = check(Ng, T, us, P, (Ng * 7 + T) % P);
                    if (rc < 0) {
                        std::printf("FAIL rc=%d Ng=%d T=%d us=%d P=%d\n", rc, Ng, T, us, P);
                        return 1;
                    }
                    (rc == 0 ? ok : rejected)++;
                }
    // the shapes of the benchmark, at the real grid: {Ng, T, us}
    const int shapes[][3] = {{384, 32, 1}, {128, 32, 1}, {688, 32, 2}, {128, 86, 1}, {1728, 32, 1}, {1000, 32, 1},
                             {384, 64, 1}, {688, 64, 2}, {128, 172, 1}};
    for (auto& sh : shapes)
        if (check(sh[0], sh[1], sh[2], 256, 17) != 0) {
            std::printf("FAIL benchmark shape Ng=%d T=%d\n", sh[0], sh[1]);
            return 1;
        }
    std::printf("ok %ld rejected %ld\n", ok, rejected);
    return 0;
}
