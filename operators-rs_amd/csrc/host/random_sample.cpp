// random_sample on the HIP backend.  Validation: random_sample/args.rs:93-120 and
// random_sample/cuda/mod.rs:84-150; mode selection: SampleArgs::is_argmax
// (args.rs:80-84).
#include <cstring>

#include "../kernels/params.h"
#include "handle.hpp"

using namespace ophip;

namespace {

constexpr size_t TOPK_FAST_MAX = 8192;  // candidates the single-workgroup top-k kernels sort in LDS (KCAP in random_sample.hip)

struct SampleMeta {
    uint64_t dt;
    size_t n;
};

SampleMeta sample_meta(const ophip_random_sample_args &a) {
    if (a.kv_pair.dt != OPHIP_DT_KVPAIR) throw type_not_support("output must be KVpair");
    const uint64_t dt = a.logits.dt;
    const size_t nb = ophip_dtype_nbytes(dt);
    if (nb == 0 || nb > sizeof(uint32_t)) throw type_not_support("element too large");
    if (a.indices.dt != OPHIP_DT_U32) throw type_not_support("indices must be u32");
    expect_rank(a.logits, "logits", 1);
    expect_rank(a.indices, "indices", 1);
    return {dt, a.logits.shape[0]};
}

size_t next_pow2(size_t n) {
    size_t p = 1;
    while (p < n) p <<= 1;
    return p;
}

// bytes of workspace the full-sort kernel needs for one row
size_t full_sort_workspace(size_t n) { return next_pow2(n) * 8 + ((n * 4 + 15) & ~(size_t)15); }

}  // namespace

struct ophip_random_sample {
    ophip_device *dev;
    hipFunction_t argmax[2], topk_k64[2], topk[2], topk_list[2], full[2];  // [0] f16, [1] f32
    explicit ophip_random_sample(ophip_device *d) : dev(d) {
        ophip_device_retain(d);
        argmax[0] = d->kernel("random_sample", "argmax_f16");
        argmax[1] = d->kernel("random_sample", "argmax_f32");
        topk[0] = d->kernel("random_sample", "sample_topk_f16");
        topk[1] = d->kernel("random_sample", "sample_topk_f32");
        topk_k64[0] = d->kernel("random_sample", "sample_topk_k64_f16");
        topk_k64[1] = d->kernel("random_sample", "sample_topk_k64_f32");
        topk_list[0] = d->kernel("random_sample", "sample_topk_list_f16");
        topk_list[1] = d->kernel("random_sample", "sample_topk_list_f32");
        full[0] = d->kernel("random_sample", "sample_full_f16");
        full[1] = d->kernel("random_sample", "sample_full_f32");
    }
    ~ophip_random_sample() { ophip_device_release(dev); }
};

extern "C" {

int ophip_sample_args_new(float temperature, float top_p, size_t top_k, ophip_sample_args *out) {
    if (!out) return OPHIP_ARGS_NOT_SUPPORT;
    if (temperature < 0.f) return 1;           // NegativeTemperature
    if (top_k == 0 || top_p <= 0.f) return 2;  // NonPositiveTop
    out->temperature = temperature;
    out->top_p = top_p < 1.f ? top_p : 1.f;
    out->top_k = top_k;
    return 0;
}

ophip_sample_args ophip_sample_args_argmax(void) { return ophip_sample_args{0.f, 1.f, SIZE_MAX}; }

int ophip_random_sample_create(ophip_device *dev, ophip_random_sample **out) {
    return guard([&] {
        if (!dev || !out) throw args_not_support("null argument");
        *out = new ophip_random_sample(dev);
    });
}
void ophip_random_sample_destroy(ophip_random_sample *op) { delete op; }

// The workspace answer follows random_sample/cuda/mod.rs:55-82: the larger of the
// two modes' needs if it fits, else the smaller, else 0; 0 for a dynamic n.
int ophip_random_sample_scheme(ophip_random_sample *, const ophip_random_sample_args *args, size_t max_ws,
                               size_t *ws) {
    return guard([&] {
        if (!args) throw args_not_support("null argument");
        if (ws) *ws = 0;
        const SampleMeta m = sample_meta(*args);
        if (m.dt != OPHIP_DT_F16 && m.dt != OPHIP_DT_F32) throw type_not_support("logits must be f16 or f32");
        if (is_dyn(m.n)) return;
        const size_t argmax_size = 0, sample_size = full_sort_workspace(m.n);
        if (ws) *ws = sample_size <= max_ws ? sample_size : argmax_size;
    });
}

static void sample_launch(const ophip_random_sample *op, const ophip_random_sample_args *args, size_t rows,
                          ptrdiff_t row_stride, const float *seeds, void *workspace, size_t workspace_len,
                          const ophip_queue_alloc *qa) {
    if (!op || !args) throw args_not_support("null argument");
    const SampleMeta m = sample_meta(*args);
    if (args->kv_pair.ndim != 0) throw rank_error("kv_pair", 0, args->kv_pair.ndim);
    const size_t n = static_of(m.n);
    const ptrdiff_t sp = static_of(args->logits.strides[0]);
    const ptrdiff_t si = static_of(args->indices.strides[0]);
    if (m.dt != OPHIP_DT_F16 && m.dt != OPHIP_DT_F32) throw type_not_support("logits must be f16 or f32");
    if (sp != (ptrdiff_t)ophip_dtype_nbytes(m.dt)) throw strides_not_support("logits must be contiguous");
    if (si != (ptrdiff_t)sizeof(uint32_t)) throw strides_not_support("indices must be contiguous");
    if (n == 0) throw shape_not_support("empty logits");  // the reference unwraps an empty maximum
    if (n > 0x7fffffffu) throw shape_not_support("too many logits");
    if (rows == 0) return;
    if (rows > 0x7fffffffu) throw shape_not_support("too many rows");
    if (row_stride % sp != 0) throw strides_not_support("row stride must be a multiple of the element size");
    // (Args::layout, random_sample/args.rs:34-49, makes arguments with null bases for scheme(): they must not reach a kernel)
    if (!args->kv_pair_base || !args->logits_base) throw args_not_support("null base address");

    const int ti = m.dt == OPHIP_DT_F16 ? 0 : 1;
    const ophip_sample_args &cfg = args->config;
    SampleParams p{};
    p.kv = args->kv_pair_base;
    p.logits = args->logits_base;
    p.row_stride = row_stride;
    p.n = (uint32_t)n;
    p.seeds = seeds;
    const Dim3 grid{(unsigned)rows};
    op->dev->make_current();
    if (cfg.temperature == 0.f || cfg.top_k == 1) {
        launch(op->argmax[ti], grid, Dim3{1024}, 0, stream_of(qa), p);
        return;
    }
    if (is_dyn(cfg.temperature) || is_dyn(cfg.top_p) || is_dyn(args->seed)) throw dyn_not_support("");
    if (!(cfg.temperature > 0.f) || cfg.top_k == 0 || !(cfg.top_p > 0.f))
        throw args_not_support("sampling needs temperature > 0, top_k >= 1, top_p > 0");
    const size_t k_eff = cfg.top_k < n ? cfg.top_k : n;
    p.k_eff = (uint32_t)k_eff;
    p.temperature = cfg.temperature;
    p.top_p = cfg.top_p;
    p.seed = args->seed;
    if (k_eff <= TOPK_FAST_MAX) {
        // rows of up to 32768 logits on 16-byte boundaries stay in the workgroup's registers; longer ones are
        // cut down to a short list in LDS after the first radix digit
        const bool in_registers = n <= 32768 && aligned16(p.logits) && (rows == 1 || row_stride % 16 == 0);
        // (top_k <= 64, the common case, has a kernel of its own among the register-row ones)
        launch(!in_registers ? op->topk_list[ti] : k_eff <= 64 ? op->topk_k64[ti] : op->topk[ti], grid, Dim3{1024}, 0, stream_of(qa), p);
        return;
    }
    // top_k beyond the LDS kernels (or none): they try first, with 64, 1024 and then 8192 candidates, and leave a
    // word per row saying whether those candidates already hold top_p of the probability; each kernel in line
    // only does the rows still open, the full sort last (on the peaked distributions of a language model the
    // first try settles every row)
    p.npow2 = (uint32_t)next_pow2(n);
    Workspace ws(qa, workspace, workspace_len, rows * full_sort_workspace(n));
    p.workspace = ws.ptr();
    const bool in_registers = n <= 32768 && aligned16(p.logits) && (rows == 1 || row_stride % 16 == 0);
    const hipFunction_t attempt = in_registers ? op->topk[ti] : op->topk_list[ti];
    SampleParams first = p;
    first.k_eff = 64;
    first.verify_cover = 1;
    launch(attempt, grid, Dim3{1024}, 0, stream_of(qa), first);
    first.verify_cover = 3;
    for (size_t k : {(size_t)1024, TOPK_FAST_MAX}) {
        first.k_eff = (uint32_t)k;
        launch(attempt, grid, Dim3{1024}, 0, stream_of(qa), first);
    }
    p.verify_cover = 2;
    launch(op->full[ti], grid, Dim3{1024}, 0, stream_of(qa), p);
}

int ophip_random_sample_launch(const ophip_random_sample *op, const ophip_random_sample_args *args, void *workspace,
                               size_t workspace_len, const ophip_queue_alloc *qa) {
    return guard([&] { sample_launch(op, args, 1, 0, nullptr, workspace, workspace_len, qa); });
}

int ophip_random_sample_launch_batch(const ophip_random_sample *op, const ophip_random_sample_args *args, size_t rows,
                                     ptrdiff_t row_stride, const float *seeds, void *workspace,
                                     size_t workspace_len, const ophip_queue_alloc *qa) {
    return guard([&] { sample_launch(op, args, rows, row_stride, seeds, workspace, workspace_len, qa); });
}

int ophip_random_sample_build_indices(size_t n, const ophip_queue_alloc *qa, void **out) {
    return guard([&] {
        if (!qa || !qa->alloc || !out) throw args_not_support("null argument");
        std::vector<uint32_t> host(n);
        for (size_t i = 0; i < n; ++i) host[i] = (uint32_t)i;
        void *mem = qa->alloc(qa->ctx, n * sizeof(uint32_t));
        if (!mem && n) throw execution_failed("queue allocator returned null");
        if (n) {
            check_hip(hipMemcpyAsync(mem, host.data(), n * sizeof(uint32_t), hipMemcpyHostToDevice, stream_of(qa)),
                      "hipMemcpyAsync");
            check_hip(hipStreamSynchronize(stream_of(qa)), "hipStreamSynchronize");
        }
        *out = mem;
    });
}

}  // extern "C"
