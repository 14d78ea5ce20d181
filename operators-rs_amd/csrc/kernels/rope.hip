// rope for gfx950: in-place rotary embedding on adjacent pairs (2k, 2k+1).
//
// One workgroup serves one token (optionally one slice of its heads).  The dh/2
// (sin, cos) pairs of the token depend only on its position, so they are
// evaluated once per workgroup into LDS with the accurate powf / sinf / cosf
// (angles reach hundreds of radians, so the range reduction matters) and then
// shared by every head: nh times fewer transcendentals than one evaluation per
// element.  Each thread then rotates 16 bytes (4 pairs) per step in registers;
// every byte of t is read once and written once.
//   ang = f32(pos) / powf(theta, f32(k) / f32(dh/2));  [a, b] <- [a c - b s, a s + b c]
#include "device_util.h"

extern __shared__ float2 rope_sc[];  // dh/2 entries of (sin, cos)

__device__ __forceinline__ float rope_pos(const RopeParams &p, uint32_t token) {
    const char *pp = reinterpret_cast<const char *>(p.pos) + (int64_t)token * p.sp;
    if (p.pos_is_u64) return (float)*reinterpret_cast<const uint64_t *>(pp);
    return (float)*reinterpret_cast<const uint32_t *>(pp);
}

__device__ __forceinline__ void rope_fill_table(const RopeParams &p, uint32_t token) {
    const uint32_t H = p.dh / 2;
    const float pos = rope_pos(p, token);
    // one entry of the table per thread, the sines by the first H threads and the cosines by the next H: the
    // table is the kernel's critical path (everything else waits for it at the barrier)
    float *flat = reinterpret_cast<float *>(rope_sc);
    for (uint32_t e = threadIdx.x; e < 2 * H; e += WG_THREADS) {
        const uint32_t k = e < H ? e : e - H;
        const float ang = pos / (p.has_den ? p.den[k] : powf(p.theta, (float)k / (float)H));
        // the same evaluation as in rope_vec_multi (one sincosf, of which this thread keeps one half), so that a token
        // gets the same bits whichever kernel its call is given
        float sn, cs;
        sincosf(ang, &sn, &cs);
        flat[2 * k + (e < H ? 0 : 1)] = e < H ? sn : cs;
    }
    __syncthreads();
}

template <typename T>
__device__ __forceinline__ void rope_vec(const RopeParams &p) {  // T: f16 or bf16
    const uint32_t token = blockIdx.x;
    const uint32_t cpv = p.dh / 8;  // 16-byte chunks per head
    const uint32_t h0 = blockIdx.y * p.heads_per_block;
    const uint32_t h1 = min(h0 + p.heads_per_block, p.nh);
    const uint32_t total = (h1 - h0) * cpv;
    char *base = reinterpret_cast<char *>(p.t) + (int64_t)token * p.st;
    auto chunk = [&](uint32_t v) { return base + (int64_t)(h0 + v / cpv) * p.sh + (size_t)(v % cpv) * 16; };
    // The thread's first chunk is requested before the table is filled (a load of pos, the transcendentals, a
    // barrier): on a few tokens the kernel is nothing but latency, and this takes one memory latency out of it.
    PackOf<T> first;
    first.u = u32x4{0, 0, 0, 0};
    if (threadIdx.x < total) first.u = ld128(chunk(threadIdx.x));
    rope_fill_table(p, token);
    for (uint32_t v = threadIdx.x; v < total; v += WG_THREADS) {
        const uint32_t c = v % cpv;
        char *ptr = chunk(v);
        PackOf<T> x, o;
        if (v == threadIdx.x) x.u = first.u;
        else x.u = ld128(ptr);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float2 sc = rope_sc[4 * c + i];
            const float a = (float)x.e[2 * i], b = (float)x.e[2 * i + 1];
            o.e[2 * i] = (T)(a * sc.y - b * sc.x);
            o.e[2 * i + 1] = (T)(a * sc.x + b * sc.y);
        }
        st128(ptr, o.u);
    }
}
// Many tokens: a workgroup takes tokens_per_block consecutive ones (about 1024 vectors), one table per token, every
// entry's sine and cosine from one evaluation (sincosf: one range reduction for both) spread over all 256 threads; with a
// token per workgroup half the threads idle through the table and a token of 8 heads gives the other half one vector
// each.
template <typename T>
__device__ __forceinline__ void rope_vec_multi(const RopeParams &p) {  // T: f16 or bf16
    const uint32_t H = p.dh / 2, cpv = p.dh / 8, per_token = p.nh * cpv;
    const uint32_t t0 = blockIdx.x * p.tokens_per_block, tokens = min(p.tokens_per_block, p.nt - t0);
    const uint32_t total = tokens * per_token;
    auto chunk = [&](uint32_t v) {
        const uint32_t tt = v / per_token, r = v - tt * per_token;
        return reinterpret_cast<char *>(p.t) + (int64_t)(t0 + tt) * p.st + (int64_t)(r / cpv) * p.sh + (size_t)(r % cpv) * 16;
    };
    PackOf<T> first;
    first.u = u32x4{0, 0, 0, 0};
    if (threadIdx.x < total) first.u = ld128(chunk(threadIdx.x));
    for (uint32_t e = threadIdx.x; e < tokens * H; e += WG_THREADS) {
        const uint32_t tt = e / H, k = e - tt * H;
        const float ang = rope_pos(p, t0 + tt) / (p.has_den ? p.den[k] : powf(p.theta, (float)k / (float)H));
        float sn, cs;
        sincosf(ang, &sn, &cs);
        rope_sc[e] = float2{sn, cs};
    }
    __syncthreads();
    for (uint32_t v = threadIdx.x; v < total; v += WG_THREADS) {
        const uint32_t tt = v / per_token, c = (v - tt * per_token) % cpv;
        char *ptr = chunk(v);
        PackOf<T> x, o;
        if (v == threadIdx.x) x.u = first.u;
        else x.u = ld128(ptr);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float2 sc = rope_sc[tt * H + 4 * c + i];
            const float a = (float)x.e[2 * i], b = (float)x.e[2 * i + 1];
            o.e[2 * i] = (T)(a * sc.y - b * sc.x);
            o.e[2 * i + 1] = (T)(a * sc.x + b * sc.y);
        }
        st128(ptr, o.u);
    }
}
extern "C" __global__ void __launch_bounds__(256) rope_f16_vec_multi(RopeParams p) { rope_vec_multi<f16>(p); }
extern "C" __global__ void __launch_bounds__(256) rope_bf16_vec_multi(RopeParams p) { rope_vec_multi<bf16>(p); }
extern "C" __global__ void __launch_bounds__(256) rope_f16_vec(RopeParams p) { rope_vec<f16>(p); }
// bf16: neither backend of the reference has it for this operator; the f16 kernels on bf16 elements (f32 inside, one rounding)
extern "C" __global__ void __launch_bounds__(256) rope_bf16_vec(RopeParams p) { rope_vec<bf16>(p); }

template <typename T>
__device__ __forceinline__ void rope_pairs(const RopeParams &p) {
    const uint32_t token = blockIdx.x;
    rope_fill_table(p, token);
    const uint32_t H = p.dh / 2;
    const uint32_t h0 = blockIdx.y * p.heads_per_block;
    const uint32_t h1 = min(h0 + p.heads_per_block, p.nh);
    const uint32_t total = (h1 - h0) * H;
    char *base = reinterpret_cast<char *>(p.t) + (int64_t)token * p.st;
    for (uint32_t v = threadIdx.x; v < total; v += WG_THREADS) {
        const uint32_t h = h0 + v / H, k = v % H;
        T *ptr = reinterpret_cast<T *>(base + (int64_t)h * p.sh) + 2 * k;
        const float2 sc = rope_sc[k];
        const float a = (float)ptr[0], b = (float)ptr[1];
        ptr[0] = (T)(a * sc.y - b * sc.x);
        ptr[1] = (T)(a * sc.x + b * sc.y);
    }
}

extern "C" __global__ void __launch_bounds__(256) rope_f16_pairs(RopeParams p) { rope_pairs<f16>(p); }
extern "C" __global__ void __launch_bounds__(256) rope_bf16_pairs(RopeParams p) { rope_pairs<bf16>(p); }
extern "C" __global__ void __launch_bounds__(256) rope_f32_pairs(RopeParams p) { rope_pairs<float>(p); }

// f64 tokens (rope/common_cpu/mod.rs:125-126): position, angle, sine and cosine in f64, as the reference computes them;
// the table holds dh/2 (sin, cos) pairs of 16 bytes.
extern "C" __global__ void __launch_bounds__(256) rope_f64_pairs(RopeParams p) {
    double2 *table = reinterpret_cast<double2 *>(rope_sc);
    const uint32_t token = blockIdx.x;
    const uint32_t H = p.dh / 2;
    const char *pp = reinterpret_cast<const char *>(p.pos) + (int64_t)token * p.sp;
    const double pos = p.pos_is_u64 ? (double)*reinterpret_cast<const uint64_t *>(pp) : (double)*reinterpret_cast<const uint32_t *>(pp);
    for (uint32_t k = threadIdx.x; k < H; k += WG_THREADS) {
        const double ang = pos / pow((double)p.theta, (double)k / (double)H);
        table[k] = double2{sin(ang), cos(ang)};
    }
    __syncthreads();
    const uint32_t h0 = blockIdx.y * p.heads_per_block;
    const uint32_t h1 = min(h0 + p.heads_per_block, p.nh);
    const uint32_t total = (h1 - h0) * H;
    char *base = reinterpret_cast<char *>(p.t) + (int64_t)token * p.st;
    for (uint32_t v = threadIdx.x; v < total; v += WG_THREADS) {
        const uint32_t h = h0 + v / H, k = v % H;
        double *ptr = reinterpret_cast<double *>(base + (int64_t)h * p.sh) + 2 * k;
        const double2 sc = table[k];
        const double a = ptr[0], b = ptr[1];
        ptr[0] = a * sc.y - b * sc.x;
        ptr[1] = a * sc.x + b * sc.y;
    }
}
