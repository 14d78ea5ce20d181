// The C ABI used from several threads at once, against the stand-in build of the library under ThreadSanitizer
// (tests/cpu_sim/build_sim.py with `thread`; the stand-in runs one kernel at a time, so what the sanitizer watches is the
// library's host side: the per-device kernel and module tables, the operators' plan caches and counter buffers, the
// registry of hooks that streams and operators share, the per-thread error text).
//
// Threads share one device, one rms_norm operator and one mat_mul operator; each has its own stream, queue allocator and
// buffers, and repeats: rms_norm [16, 1024], mat_mul [16, 1024] x [1024, 512] on a split K (workspace from the queue
// allocator, arrival counters from the operator), copy back, compare with what thread 0 computed on the host.  Every
// few rounds a thread also creates and destroys an operator and a stream of its own, which adds and removes hooks while
// the others launch.  Exit status 0 when every result agreed; a data race ends the run through the sanitizer.
//
//   threads_driver [threads = 4] [rounds = 12]
#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

#include "ophip.h"

namespace {

typedef _Float16 f16;
constexpr int N = 16, D = 1024, NN = 512;

std::atomic<int> g_failures{0};

#define CHECK(call)                                                                              \
    do {                                                                                         \
        const int rc_ = (call);                                                                  \
        if (rc_ != OPHIP_OK) {                                                                   \
            std::fprintf(stderr, "%s -> %d (%s)\n", #call, rc_, ophip_last_error());             \
            g_failures++;                                                                        \
            return;                                                                              \
        }                                                                                        \
    } while (0)

struct Shared {
    ophip_device *dev;
    ophip_rms_norm *rms;
    ophip_mat_mul *mm;
    std::vector<f16> x, w, b, y_ref, c_ref;
};

void worker(const Shared &sh, int id, int rounds) {
    ophip_stream stream = nullptr;
    CHECK(ophip_stream_create(sh.dev, &stream));
    ophip_queue_alloc qa;
    CHECK(ophip_queue_alloc_from_stream(sh.dev, stream, &qa));
    void *xd, *wd, *yd, *bd, *cd;
    CHECK(ophip_malloc(sh.dev, N * D * 2, &xd));
    CHECK(ophip_malloc(sh.dev, D * 2, &wd));
    CHECK(ophip_malloc(sh.dev, N * D * 2, &yd));
    CHECK(ophip_malloc(sh.dev, D * NN * 2, &bd));
    CHECK(ophip_malloc(sh.dev, N * NN * 2, &cd));
    CHECK(ophip_memcpy_h2d(sh.dev, xd, sh.x.data(), N * D * 2, stream));
    CHECK(ophip_memcpy_h2d(sh.dev, wd, sh.w.data(), D * 2, stream));
    CHECK(ophip_memcpy_h2d(sh.dev, bd, sh.b.data(), D * NN * 2, stream));

    const size_t shape2[2] = {N, D}, shape1[1] = {D};
    const ptrdiff_t strides2[2] = {D * 2, 2}, strides1[1] = {2};
    ophip_rms_norm_args ra;
    std::memset(&ra, 0, sizeof ra);
    ra.y_layout = ophip_tensor_layout{OPHIP_DT_F16, 2, shape2, strides2};
    ra.x_layout = ra.y_layout;
    ra.w_layout = ophip_tensor_layout{OPHIP_DT_F16, 1, shape1, strides1};
    ra.y_base = yd, ra.x_base = xd, ra.w_base = wd, ra.epsilon = 1e-5f;

    const size_t sa[3] = {1, N, D}, sb[3] = {1, D, NN}, sc[3] = {1, N, NN};
    const ptrdiff_t ta[3] = {N * D * 2, D * 2, 2}, tb[3] = {D * NN * 2, NN * 2, 2}, tc[3] = {N * NN * 2, NN * 2, 2};
    ophip_mat_mul_args ma;
    std::memset(&ma, 0, sizeof ma);
    ma.c_layout = ophip_tensor_layout{OPHIP_DT_F16, 3, sc, tc};
    ma.a_layout = ophip_tensor_layout{OPHIP_DT_F16, 3, sa, ta};
    ma.b_layout = ophip_tensor_layout{OPHIP_DT_F16, 3, sb, tb};
    ma.c_base = cd, ma.a_base = yd, ma.b_base = bd, ma.alpha = 1.0f, ma.beta = 0.0f;

    std::vector<f16> y(N * D), c(N * NN);
    for (int r = 0; r < rounds; ++r) {
        size_t ws = 0;
        CHECK(ophip_rms_norm_scheme(sh.rms, &ra, 0, &ws));
        CHECK(ophip_rms_norm_launch(sh.rms, &ra, nullptr, 0, &qa));
        CHECK(ophip_mat_mul_scheme(sh.mm, &ma, (size_t)1 << 30, &ws));
        CHECK(ophip_mat_mul_launch(sh.mm, &ma, nullptr, 0, &qa));  // no workspace of the caller's: the queue allocator's
        CHECK(ophip_memcpy_d2h(sh.dev, y.data(), yd, N * D * 2, stream));
        CHECK(ophip_memcpy_d2h(sh.dev, c.data(), cd, N * NN * 2, stream));
        CHECK(ophip_stream_synchronize(sh.dev, stream));
        if (std::memcmp(y.data(), sh.y_ref.data(), N * D * 2) != 0 || std::memcmp(c.data(), sh.c_ref.data(), N * NN * 2) != 0) {
            std::fprintf(stderr, "thread %d round %d: results differ from the first run's\n", id, r);
            g_failures++;
        }
        if (r % 3 == id % 3) {  // hooks come and go while the others launch
            ophip_mat_mul *own = nullptr;
            CHECK(ophip_mat_mul_create(sh.dev, &own));
            CHECK(ophip_mat_mul_launch(own, &ma, nullptr, 0, &qa));
            ophip_stream s2 = nullptr;
            CHECK(ophip_stream_create(sh.dev, &s2));
            CHECK(ophip_stream_synchronize(sh.dev, stream));
            ophip_mat_mul_destroy(own);
            CHECK(ophip_stream_destroy(sh.dev, s2));
        }
        // an error on this thread leaves the others' error text alone
        ophip_rms_norm_args bad = ra;
        bad.w_layout.dt = OPHIP_DT_U32;
        if (ophip_rms_norm_launch(sh.rms, &bad, nullptr, 0, &qa) != OPHIP_TYPE_NOT_SUPPORT || !ophip_last_error()[0]) g_failures++;
    }
    void *all[] = {xd, wd, yd, bd, cd};
    for (void *p : all) CHECK(ophip_free(sh.dev, p));
    CHECK(ophip_stream_destroy(sh.dev, stream));
}

}  // namespace

int main(int argc, char **argv) {
    const int threads = argc > 1 ? std::atoi(argv[1]) : 4, rounds = argc > 2 ? std::atoi(argv[2]) : 12;
    if (ophip_device_count() < 1) {
        std::printf("no device\n");
        return 2;
    }
    Shared sh;
    if (ophip_device_create(0, nullptr, &sh.dev) != OPHIP_OK || ophip_rms_norm_create(sh.dev, &sh.rms) != OPHIP_OK ||
        ophip_mat_mul_create(sh.dev, &sh.mm) != OPHIP_OK) {
        std::fprintf(stderr, "set-up failed: %s\n", ophip_last_error());
        return 1;
    }
    uint32_t seed = 1;
    auto uniform = [&] {
        seed = seed * 1664525u + 1013904223u;
        return (float)(seed >> 8) / 16777216.0f * 2.0f - 1.0f;
    };
    sh.x.resize(N * D), sh.w.resize(D), sh.b.resize(D * NN), sh.y_ref.resize(N * D), sh.c_ref.resize(N * NN);
    for (auto &v : sh.x) v = (f16)(2.0f * uniform());
    for (auto &v : sh.w) v = (f16)(1.0f + 0.5f * uniform());
    for (auto &v : sh.b) v = (f16)(0.125f * uniform());
    // the reference: one run on one thread (its agreement with the oracle is the parity tests' business), checked
    // loosely against plain arithmetic here so that a stand-in that computes nothing is noticed
    {
        // run once, single-threaded, and keep what came back
        struct Grab {
            static void run(Shared &s, std::vector<f16> &y, std::vector<f16> &c) {
                ophip_stream stream = nullptr;
                ophip_stream_create(s.dev, &stream);
                ophip_queue_alloc qa;
                ophip_queue_alloc_from_stream(s.dev, stream, &qa);
                void *xd, *wd, *yd, *bd, *cd;
                ophip_malloc(s.dev, N * D * 2, &xd), ophip_malloc(s.dev, D * 2, &wd), ophip_malloc(s.dev, N * D * 2, &yd);
                ophip_malloc(s.dev, D * NN * 2, &bd), ophip_malloc(s.dev, N * NN * 2, &cd);
                ophip_memcpy_h2d(s.dev, xd, s.x.data(), N * D * 2, stream);
                ophip_memcpy_h2d(s.dev, wd, s.w.data(), D * 2, stream);
                ophip_memcpy_h2d(s.dev, bd, s.b.data(), D * NN * 2, stream);
                const size_t shape2[2] = {N, D}, shape1[1] = {D};
                const ptrdiff_t strides2[2] = {D * 2, 2}, strides1[1] = {2};
                ophip_rms_norm_args ra;
                std::memset(&ra, 0, sizeof ra);
                ra.y_layout = ophip_tensor_layout{OPHIP_DT_F16, 2, shape2, strides2};
                ra.x_layout = ra.y_layout;
                ra.w_layout = ophip_tensor_layout{OPHIP_DT_F16, 1, shape1, strides1};
                ra.y_base = yd, ra.x_base = xd, ra.w_base = wd, ra.epsilon = 1e-5f;
                const size_t sa[3] = {1, N, D}, sb[3] = {1, D, NN}, sc[3] = {1, N, NN};
                const ptrdiff_t ta[3] = {N * D * 2, D * 2, 2}, tb[3] = {D * NN * 2, NN * 2, 2}, tc[3] = {N * NN * 2, NN * 2, 2};
                ophip_mat_mul_args ma;
                std::memset(&ma, 0, sizeof ma);
                ma.c_layout = ophip_tensor_layout{OPHIP_DT_F16, 3, sc, tc};
                ma.a_layout = ophip_tensor_layout{OPHIP_DT_F16, 3, sa, ta};
                ma.b_layout = ophip_tensor_layout{OPHIP_DT_F16, 3, sb, tb};
                ma.c_base = cd, ma.a_base = yd, ma.b_base = bd, ma.alpha = 1.0f, ma.beta = 0.0f;
                if (ophip_rms_norm_launch(s.rms, &ra, nullptr, 0, &qa) != OPHIP_OK || ophip_mat_mul_launch(s.mm, &ma, nullptr, 0, &qa) != OPHIP_OK) {
                    std::fprintf(stderr, "first run: %s\n", ophip_last_error());
                    g_failures++;
                }
                ophip_memcpy_d2h(s.dev, y.data(), yd, N * D * 2, stream);
                ophip_memcpy_d2h(s.dev, c.data(), cd, N * NN * 2, stream);
                ophip_stream_synchronize(s.dev, stream);
                void *all[] = {xd, wd, yd, bd, cd};
                for (void *p : all) ophip_free(s.dev, p);
                ophip_stream_destroy(s.dev, stream);
            }
        };
        Grab::run(sh, sh.y_ref, sh.c_ref);
        int off = 0;
        for (int i = 0; i < N; ++i) {
            float ss = 0.f;
            for (int j = 0; j < D; ++j) ss += (float)sh.x[i * D + j] * (float)sh.x[i * D + j];
            const float k = 1.0f / std::sqrt(ss / D + 1e-5f);
            for (int j = 0; j < D; ++j) {
                const float ref = k * (float)sh.w[j] * (float)sh.x[i * D + j], got = (float)sh.y_ref[i * D + j];
                if (std::fabs(got - ref) > 2e-3f && std::fabs(got - ref) > 1e-2f * std::fabs(ref)) off++;
            }
            for (int j = 0; j < NN; ++j) {
                float ref = 0.f;
                for (int l = 0; l < D; ++l) ref += (float)sh.y_ref[i * D + l] * (float)sh.b[l * NN + j];
                const float got = (float)sh.c_ref[i * NN + j];
                if (std::fabs(got - ref) > 4e-3f && std::fabs(got - ref) > 1e-2f * std::fabs(ref)) off++;
            }
        }
        if (off) {
            std::fprintf(stderr, "first run: %d elements off\n", off);
            return 3;
        }
    }
    std::vector<std::thread> pool;
    for (int t = 0; t < threads; ++t) pool.emplace_back(worker, std::cref(sh), t, rounds);
    for (auto &t : pool) t.join();
    ophip_mat_mul_destroy(sh.mm);
    ophip_rms_norm_destroy(sh.rms);
    ophip_device_release(sh.dev);
    std::printf("%d threads x %d rounds: %d failures\n", threads, rounds, g_failures.load());
    if (!g_failures) std::printf("ok\n");
    return g_failures ? 1 : 0;
}
