/* A consumer of the C ABI written in C11, as a binding of another language would see it: no Python, no ctypes.
 * Creates a device, runs rms_norm ([16, 4096] f16 with f32 weights) and mat_mul ([16, 256] x [256, 512] f16) through
 * create / scheme / launch, and checks both against the same arithmetic in C (f32, rounded to f16 by the conversion
 * routines below).  Exit status: 0 = results agree, 2 = no device (nothing to run on: reported, not an error of the
 * library), anything else = failure.  Built and run by tests/test_c_consumer.py. */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "ophip.h"

static float half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1fu, man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: value = man * 2^-24 */
            const float v = (float)man * 5.9604644775390625e-8f;
            memcpy(&bits, &v, 4);
            bits |= sign;
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static uint16_t float_to_half(float f) { /* round to nearest even; the test's values stay in the normal range */
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const int32_t e = (int32_t)((x >> 23) & 0xffu) - 127 + 15;
    uint32_t man = x & 0x7fffffu;
    if (e >= 31) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        const uint32_t shift = (uint32_t)(14 - e), half = 1u << (shift - 1), rem = man & ((1u << shift) - 1);
        uint32_t hm = man >> shift;
        if (rem > half || (rem == half && (hm & 1u))) hm++;
        return (uint16_t)(sign | hm);
    }
    uint32_t h = ((uint32_t)e << 10) | (man >> 13);
    const uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h++;
    return (uint16_t)(sign | h);
}

static uint32_t lcg(uint32_t *s) { return *s = *s * 1664525u + 1013904223u; }
static float uniform(uint32_t *s) { return (float)(lcg(s) >> 8) / 16777216.0f * 2.0f - 1.0f; } /* [-1, 1) */

#define CHECK(call)                                                                                    \
    do {                                                                                               \
        const int rc_ = (call);                                                                        \
        if (rc_ != OPHIP_OK) {                                                                         \
            fprintf(stderr, "%s -> %d (%s)\n", #call, rc_, ophip_last_error());                        \
            return 1;                                                                                  \
        }                                                                                              \
    } while (0)

int main(void) {
    if (ophip_device_count() < 1) {
        printf("no device\n");
        return 2;
    }
    ophip_device *dev = NULL;
    CHECK(ophip_device_create(0, NULL, &dev));
    ophip_device_info info;
    CHECK(ophip_device_get_info(dev, &info));
    printf("device %s (%s), %d CUs\n", info.name, info.arch, info.compute_units);
    ophip_stream stream = NULL;
    CHECK(ophip_stream_create(dev, &stream));
    ophip_queue_alloc qa;
    CHECK(ophip_queue_alloc_from_stream(dev, stream, &qa));
    uint32_t seed = 1;

    /* ---- rms_norm ---- */
    enum { N = 16, D = 4096 };
    uint16_t *x = malloc(N * D * 2), *y = malloc(N * D * 2);
    float *w = malloc(D * 4);
    for (int i = 0; i < N * D; ++i) x[i] = float_to_half(uniform(&seed) * 2.0f);
    for (int i = 0; i < D; ++i) w[i] = 1.0f + 0.5f * uniform(&seed);
    void *xd, *yd, *wd;
    CHECK(ophip_malloc(dev, N * D * 2, &xd));
    CHECK(ophip_malloc(dev, N * D * 2, &yd));
    CHECK(ophip_malloc(dev, D * 4, &wd));
    CHECK(ophip_memcpy_h2d(dev, xd, x, N * D * 2, stream));
    CHECK(ophip_memcpy_h2d(dev, wd, w, D * 4, stream));
    const size_t shape2[2] = {N, D}, shape1[1] = {D};
    const ptrdiff_t strides2[2] = {D * 2, 2}, strides1[1] = {4};
    ophip_rms_norm_args ra;
    memset(&ra, 0, sizeof ra);
    ra.y_layout = (ophip_tensor_layout){OPHIP_DT_F16, 2, shape2, strides2};
    ra.x_layout = ra.y_layout;
    ra.w_layout = (ophip_tensor_layout){OPHIP_DT_F32, 1, shape1, strides1};
    ra.y_base = yd;
    ra.x_base = xd;
    ra.w_base = wd;
    ra.epsilon = 1e-5f;
    ophip_rms_norm *rms = NULL;
    CHECK(ophip_rms_norm_create(dev, &rms));
    size_t ws = 0;
    CHECK(ophip_rms_norm_scheme(rms, &ra, 0, &ws));
    CHECK(ophip_rms_norm_launch(rms, &ra, NULL, 0, &qa));
    CHECK(ophip_memcpy_d2h(dev, y, yd, N * D * 2, stream));
    CHECK(ophip_stream_synchronize(dev, stream));
    int bad = 0;
    for (int i = 0; i < N; ++i) {
        float ss = 0.f;
        for (int j = 0; j < D; ++j) {
            const float v = half_to_float(x[i * D + j]);
            ss += v * v;
        }
        const float k = 1.0f / sqrtf(ss / (float)D + 1e-5f);
        for (int j = 0; j < D; ++j) {
            const float ref = k * w[j] * half_to_float(x[i * D + j]), got = half_to_float(y[i * D + j]);
            if (fabsf(got - ref) > 2e-3f && fabsf(got - ref) > 1e-2f * fabsf(ref)) bad++;
        }
    }
    printf("rms_norm [%d, %d]: %d elements off\n", N, D, bad);
    if (bad) return 3;
    /* a refusal comes back as a status and a message, not as an abort */
    ra.w_layout.dt = OPHIP_DT_U32;
    if (ophip_rms_norm_launch(rms, &ra, NULL, 0, &qa) != OPHIP_TYPE_NOT_SUPPORT || !ophip_last_error()[0]) {
        fprintf(stderr, "a u32 weight was not refused as TypeNotSupport\n");
        return 4;
    }
    ophip_rms_norm_destroy(rms);

    /* ---- mat_mul: c[16, 512] = a[16, 256] . b[256, 512] ---- */
    enum { M = 16, K = 256, NN = 512 };
    uint16_t *a = malloc(M * K * 2), *b = malloc(K * NN * 2), *c = malloc(M * NN * 2);
    for (int i = 0; i < M * K; ++i) a[i] = float_to_half(uniform(&seed));
    for (int i = 0; i < K * NN; ++i) b[i] = float_to_half(uniform(&seed) * 0.125f);
    void *ad, *bd, *cd;
    CHECK(ophip_malloc(dev, M * K * 2, &ad));
    CHECK(ophip_malloc(dev, K * NN * 2, &bd));
    CHECK(ophip_malloc(dev, M * NN * 2, &cd));
    CHECK(ophip_memcpy_h2d(dev, ad, a, M * K * 2, stream));
    CHECK(ophip_memcpy_h2d(dev, bd, b, K * NN * 2, stream));
    const size_t sa[3] = {1, M, K}, sb[3] = {1, K, NN}, sc[3] = {1, M, NN};
    const ptrdiff_t ta[3] = {M * K * 2, K * 2, 2}, tb[3] = {K * NN * 2, NN * 2, 2}, tc[3] = {M * NN * 2, NN * 2, 2};
    ophip_mat_mul_args ma;
    memset(&ma, 0, sizeof ma);
    ma.c_layout = (ophip_tensor_layout){OPHIP_DT_F16, 3, sc, tc};
    ma.a_layout = (ophip_tensor_layout){OPHIP_DT_F16, 3, sa, ta};
    ma.b_layout = (ophip_tensor_layout){OPHIP_DT_F16, 3, sb, tb};
    ma.c_base = cd;
    ma.a_base = ad;
    ma.b_base = bd;
    ma.alpha = 1.0f;
    ma.beta = 0.0f;
    ophip_mat_mul *mm = NULL;
    CHECK(ophip_mat_mul_create(dev, &mm));
    CHECK(ophip_mat_mul_scheme(mm, &ma, (size_t)1 << 30, &ws));
    void *wsd = NULL;
    if (ws) CHECK(ophip_malloc(dev, ws, &wsd));
    CHECK(ophip_mat_mul_launch(mm, &ma, wsd, ws, &qa));
    CHECK(ophip_memcpy_d2h(dev, c, cd, M * NN * 2, stream));
    CHECK(ophip_stream_synchronize(dev, stream));
    bad = 0;
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < NN; ++j) {
            float ref = 0.f;
            for (int l = 0; l < K; ++l) ref += half_to_float(a[i * K + l]) * half_to_float(b[l * NN + j]);
            const float got = half_to_float(c[i * NN + j]);
            if (fabsf(got - ref) > 2e-3f && fabsf(got - ref) > 1e-2f * fabsf(ref)) bad++;
        }
    printf("mat_mul %d x %d x %d: %d elements off\n", M, NN, K, bad);
    if (bad) return 5;
    ophip_mat_mul_destroy(mm);

    if (wsd) CHECK(ophip_free(dev, wsd));
    void *all[] = {xd, yd, wd, ad, bd, cd};
    for (size_t i = 0; i < sizeof all / sizeof all[0]; ++i) CHECK(ophip_free(dev, all[i]));
    CHECK(ophip_stream_destroy(dev, stream));
    ophip_device_release(dev);
    free(x); free(y); free(w); free(a); free(b); free(c);
    printf("ok\n");
    return 0;
}
