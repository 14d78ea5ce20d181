// Walks every workgroup of a gemm_stream launch through the unit numbering the kernel itself uses
// (operators-rs_amd/csrc/kernels/params.h, compiled here for the host) and checks what the kernel relies on:
// every (strip, K range) exactly once, every range non-empty, inside K and in whole steps of 32, the ranges of a
// strip covering K without gaps, and no unit for blocks past the last strip.
// usage: stream_units N K split_k k_per_split slow_mask split_slow   (all alignments of Q's first granule are tried)
#include <cstdio>
#include <cstdlib>
#include <map>
#include <utility>
#include <vector>

#include "params.h"

static int fail(const char *what, unsigned long a, unsigned long b, unsigned long c) {
    std::printf("FAIL %s (%lu %lu %lu)\n", what, a, b, c);
    return 1;
}

int main(int argc, char **argv) {
    if (argc != 7) return fail("usage", 0, 0, 0);
    GemmParams p{};
    p.N = (uint32_t)std::strtoul(argv[1], nullptr, 0);
    p.K = (uint32_t)std::strtoul(argv[2], nullptr, 0);
    p.split_k = (uint32_t)std::strtoul(argv[3], nullptr, 0);
    p.k_per_split = (uint32_t)std::strtoul(argv[4], nullptr, 0);
    p.slow_mask = (uint32_t)std::strtoul(argv[5], nullptr, 0);
    p.split_slow = (uint32_t)std::strtoul(argv[6], nullptr, 0);
    const uint32_t nstrips = (p.N + 127) / 128;
    unsigned long total_units = 0;
    for (uint64_t g0 = 0; g0 < 8; ++g0) {
        const uint64_t q_addr = 0x7f0000000000ull + g0 * 256;
        const uint32_t grid = gemm_stream_units(&p, q_addr);
        std::map<std::pair<uint32_t, uint32_t>, std::pair<uint32_t, uint32_t>> seen;  // (strip, range) -> [kbeg, kend)
        std::vector<uint32_t> ranges_of(nstrips, 0);
        for (uint32_t b = 0; b < grid; ++b) {
            const GemmStreamUnit u = gemm_stream_unit(&p, q_addr, b);
            if (!u.valid) continue;
            if (u.strip >= nstrips) return fail("strip out of range", b, u.strip, nstrips);
            const uint32_t want = gemm_stream_ranges(&p, (uint32_t)(q_addr >> 8) + u.strip);
            if (u.ranges != want || u.range >= u.ranges) return fail("ranges of the strip", b, u.ranges, want);
            if (!(u.kbeg < u.kend && u.kend <= p.K)) return fail("empty or overlong K range", b, u.kbeg, u.kend);
            if (u.kbeg % 32 || (u.kend - u.kbeg) % 32) return fail("K range not in whole steps", b, u.kbeg, u.kend);
            if (!seen.emplace(std::make_pair(u.strip, u.range), std::make_pair(u.kbeg, u.kend)).second)
                return fail("unit taken twice", b, u.strip, u.range);
            ranges_of[u.strip] = u.ranges;
        }
        for (uint32_t s = 0; s < nstrips; ++s) {
            if (ranges_of[s] == 0) return fail("strip without a unit", s, g0, 0);
            uint32_t at = 0;
            for (uint32_t r = 0; r < ranges_of[s]; ++r) {
                auto it = seen.find(std::make_pair(s, r));
                if (it == seen.end()) return fail("range missing", s, r, g0);
                if (it->second.first != at) return fail("gap between ranges", s, r, it->second.first);
                at = it->second.second;
            }
            if (at != p.K) return fail("ranges do not reach K", s, at, p.K);
        }
        // a block past the grid must not turn into a unit either
        for (uint32_t b = grid; b < grid + 16; ++b)
            if (gemm_stream_unit(&p, q_addr, b).valid && gemm_stream_unit(&p, q_addr, b).strip < nstrips && p.slow_mask == 0)
                return fail("unit past the grid", b, grid, 0);
        total_units += seen.size();
    }
    std::printf("OK %lu units over 8 alignments\n", total_units);
    return 0;
}
