// The weight-streaming mat_mul kernels (operators-rs_amd/csrc/kernels/gemm.hip) compiled for the host and run
// work-item by work-item on small products (tests/cpu_sim/hip/hip_runtime.h), under AddressSanitizer: every operand is
// a heap block of exactly its size, so a load or store outside an operand stops the program; results are compared
// with a double-precision product; buffer loads that ran past a resource's records are counted (none may).
// The grid comes from the same function the library's host side uses (gemm_stream_units).
//
// usage: gemm_cpu kernel M N K batch split_k slow_mask split_slow [q_granule_offset [overstate_k]]
//   kernel = stream | skinny   (skinny: gemm_skinny_m1_q0, grid (strips, split_k, batch), no mask)
//   overstate_k: the kernel is told K + overstate_k while the operands hold K rows: the run must then be stopped by
//   the sanitizer (the check that this build does catch an access outside an operand)
#define OPHIP_CPU_SIM 1
#include "../../operators-rs_amd/csrc/kernels/gemm.hip"

#include <string>
#include <vector>

static uint16_t to_half_bits(float f) {
    const _Float16 h = (_Float16)f;
    uint16_t u;
    std::memcpy(&u, &h, 2);
    return u;
}
static float from_half_bits(uint16_t u) {
    _Float16 h;
    std::memcpy(&h, &u, 2);
    return (float)h;
}
static uint32_t hash32(uint32_t x) {
    x ^= x >> 16;
    x *= 0x7feb352dU;
    x ^= x >> 15;
    x *= 0x846ca68bU;
    x ^= x >> 16;
    return x;
}
static float noise(uint32_t i, uint32_t seed) { return ((hash32(i * 2654435761u + seed) >> 8) * (1.0f / 16777216.0f) - 0.5f) * 2.0f; }

int main(int argc, char **argv) {
    if (argc < 9) {
        std::printf("usage: gemm_cpu kernel M N K batch split_k slow_mask split_slow [granule]\n");
        return 2;
    }
    const std::string kernel = argv[1];
    const uint32_t M = std::strtoul(argv[2], nullptr, 0), N = std::strtoul(argv[3], nullptr, 0), K = std::strtoul(argv[4], nullptr, 0);
    const uint32_t batch = std::strtoul(argv[5], nullptr, 0), split_k = std::strtoul(argv[6], nullptr, 0);
    const uint32_t mask = std::strtoul(argv[7], nullptr, 0), split_slow = std::strtoul(argv[8], nullptr, 0);
    const uint32_t granule = argc > 9 ? std::strtoul(argv[9], nullptr, 0) : 0;
    const uint32_t overstate = argc > 10 ? std::strtoul(argv[10], nullptr, 0) : 0;

    // operands: exact-size heap blocks (Q starts `granule` 256-byte granules into a 2 KiB-aligned block, so that its
    // strips fall on chosen granule classes; what lies before it is part of the same block and must never be read: poisoned)
    // (rows of P start on 16-byte boundaries, which the library's planner requires of the streaming kernels)
    const size_t p_pitch = (K + 7) / 8 * 8;
    const size_t q_elems = (size_t)batch * K * N, p_elems = (size_t)batch * M * p_pitch, d_elems = (size_t)batch * M * N;
    const size_t q_pad = (size_t)granule * 256;
    char *q_block = static_cast<char *>(std::aligned_alloc(2048, (q_pad + q_elems * 2 + 2047) / 2048 * 2048));
    uint16_t *q = reinterpret_cast<uint16_t *>(q_block + q_pad);
    std::vector<uint16_t> pm(p_elems), dm(d_elems, 0x7e00);  // D starts as NaNs: beta = 0 must never read it
    for (size_t i = 0; i < q_elems; ++i) q[i] = to_half_bits(0.05f * noise((uint32_t)i, 1));
    for (size_t i = 0; i < p_elems; ++i) pm[i] = to_half_bits(noise((uint32_t)i, 2));
    const uint32_t ranges = std::max(split_k, mask ? split_slow : 0u);
    std::vector<float> partial(ranges > 1 ? (size_t)ranges * d_elems : 4, std::nanf(""));  // what a workspace held before: NaNs
    const uint32_t nstrips = (N + 127) / 128;
    std::vector<uint32_t> counters((size_t)nstrips * batch, 0);

    GemmParams p{};
    p.d = dm.data();
    p.p = pm.data();
    p.q = q;
    p.partial = partial.data();
    p.counters = counters.data();
    p.d_si = N, p.d_sj = 1, p.d_sb = (int64_t)M * N;
    p.p_si = (int64_t)p_pitch, p.p_sl = 1, p.p_sb = (int64_t)M * p_pitch;
    p.q_sl = N, p.q_sj = 1, p.q_sb = (int64_t)K * N;
    p.M = M, p.N = N, p.K = K + overstate, p.batch = batch;
    p.alpha = 0.5f, p.beta = 0.f, p.read_dst = 0;
    const uint32_t steps = (p.K + 31) / 32, sps = (steps + split_k - 1) / split_k;
    p.split_k = split_k;
    p.k_per_split = sps * 32;
    p.slow_mask = mask;
    p.split_slow = mask ? split_slow : 0;

    if (kernel == "stream") {
        const uint32_t grid = gemm_stream_units(&p, reinterpret_cast<uint64_t>(p.q));
        cpusim::launch({grid, 1, batch}, {256, 1, 1}, 0, [&] { gemm_stream_m1(p); });
    } else if (kernel == "skinny") {
        cpusim::launch({nstrips, split_k, batch}, {256, 1, 1}, 0, [&] { gemm_skinny_m1_q0(p); });
    } else {
        std::printf("unknown kernel\n");
        return 2;
    }

    double worst = 0;
    size_t bad = 0;
    for (uint32_t b = 0; b < batch; ++b)
        for (uint32_t i = 0; i < M; ++i)
            for (uint32_t j = 0; j < N; ++j) {
                double s = 0;
                for (uint32_t k = 0; k < K; ++k)
                    s += (double)from_half_bits(pm[((size_t)b * M + i) * p_pitch + k]) * (double)from_half_bits(q[((size_t)b * K + k) * N + j]);
                s *= 0.5;
                const double got = from_half_bits(dm[((size_t)b * M + i) * N + j]), err = std::fabs(got - s);
                if (!(err <= 2e-3 + 1e-2 * std::fabs(s))) ++bad;  // (a NaN left in D fails here)
                worst = std::max(worst, err);
            }
    size_t dirty = 0;
    for (uint32_t c : counters) dirty += c != 0;
    const uint64_t oor = cpusim::worker().out_of_range_loads + cpusim::worker().out_of_range_stores;
    std::printf("%s M=%u N=%u K=%u batch=%u split=%u mask=%#x slow=%u granule=%u: max err %.3g, %zu bad, %zu counters not back at zero, %llu accesses past a resource's records\n",
                kernel.c_str(), M, N, K, batch, split_k, mask, split_slow, granule, worst, bad, dirty, (unsigned long long)oor);
    std::free(q_block);
    return bad || dirty || oor ? 1 : 0;
}
