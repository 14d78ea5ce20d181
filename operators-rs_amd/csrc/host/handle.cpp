#include "handle.hpp"
#include "static_scratch.hpp"
#include "../kernels/params.h"

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <set>

namespace ophip {

static thread_local std::string g_last_error;
void set_last_error(const std::string &s) { g_last_error = s; }

void check_hip(hipError_t e, const char *what) {
    if (e != hipSuccess)
        throw execution_failed(std::string(what) + ": " + hipGetErrorName(e) + " (" + std::to_string((int)e) +
                               ") " + hipGetErrorString(e));
}

float round_to_bf16(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    if (((x >> 23) & 0xffu) == 0xffu) return f;
    x = (x + 0x7fffu + ((x >> 16) & 1u)) & 0xffff0000u;
    float r;
    std::memcpy(&r, &x, 4);
    return r;
}

float round_to_f16(float f) {
    // software round-to-nearest-even f32 -> f16 -> f32
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = x & 0x80000000u;
    const uint32_t exp = (x >> 23) & 0xffu;
    uint32_t man = x & 0x7fffffu;
    if (exp == 0xff) return f;
    const int e = (int)exp - 127 + 15;
    uint32_t hbits;
    if (e >= 31) {
        hbits = 0x7c00u;
    } else if (e <= 0) {
        if (e < -10) {
            hbits = 0;
        } else {
            man |= 0x800000u;
            const uint32_t shift = (uint32_t)(14 - e);
            uint32_t hm = man >> shift;
            const uint32_t rem = man & ((1u << shift) - 1), half = 1u << (shift - 1);
            if (rem > half || (rem == half && (hm & 1u))) hm++;
            hbits = hm;
        }
    } else {
        hbits = ((uint32_t)e << 10) | (man >> 13);
        const uint32_t rem = man & 0x1fffu;
        if (rem > 0x1000u || (rem == 0x1000u && (hbits & 1u))) hbits++;
    }
    // widen back
    const uint32_t he = (hbits >> 10) & 0x1fu;
    uint32_t hm = hbits & 0x3ffu, out;
    if (he == 0) {
        if (hm == 0) {
            out = sign;
        } else {
            int sh = -1;
            do {
                hm <<= 1;
                sh++;
            } while (!(hm & 0x400u));
            out = sign | ((uint32_t)(127 - 15 - sh) << 23) | ((hm & 0x3ffu) << 13);
        }
    } else if (he == 31) {
        out = sign | 0x7f800000u | (hm << 13);
    } else {
        out = sign | ((he + 127 - 15) << 23) | (hm << 13);
    }
    float r;
    std::memcpy(&r, &out, 4);
    return r;
}

// hip/hip_ext.h (its templates need the HIP compiler; the host side is built with g++, so only the one prototype)
extern "C" hipError_t hipExtModuleLaunchKernel(hipFunction_t f, uint32_t globalWorkSizeX, uint32_t globalWorkSizeY,
                                               uint32_t globalWorkSizeZ, uint32_t localWorkSizeX, uint32_t localWorkSizeY,
                                               uint32_t localWorkSizeZ, size_t sharedMemBytes, hipStream_t hStream,
                                               void **kernelParams, void **extra, hipEvent_t startEvent,
                                               hipEvent_t stopEvent, uint32_t flags);

// A pending ophip_time_next_launch of this thread: the next kernel launched on that stream carries the two
// events, which then hold the kernel's own begin and end on the device.
static thread_local struct {
    bool armed = false;
    hipStream_t stream = nullptr;
    hipEvent_t start = nullptr, stop = nullptr;
} g_timed;

void launch_raw(hipFunction_t fn, Dim3 grid, Dim3 block, size_t smem, hipStream_t stream, void *params,
                size_t params_size) {
    void *extra[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, params, HIP_LAUNCH_PARAM_BUFFER_SIZE, &params_size,
                     HIP_LAUNCH_PARAM_END};
    if (g_timed.armed && g_timed.stream == stream) {
        g_timed.armed = false;
        check_hip(hipExtModuleLaunchKernel(fn, grid.x * block.x, grid.y * block.y, grid.z * block.z, block.x, block.y,
                                           block.z, smem, stream, nullptr, extra, g_timed.start, g_timed.stop, 0),
                  "hipExtModuleLaunchKernel");
        return;
    }
    check_hip(hipModuleLaunchKernel(fn, grid.x, grid.y, grid.z, block.x, block.y, block.z, (unsigned)smem, stream,
                                    nullptr, extra),
              "hipModuleLaunchKernel");
}

Workspace::Workspace(const ophip_queue_alloc *qa, void *ext, size_t ext_len, size_t need) {
    if (need == 0) {
        ptr_ = ext;
        return;
    }
    // The kernels move 16 bytes at a time and use 64-bit atomics inside a workspace: a caller's slice that does not
    // start on a 16-byte boundary is used from the next boundary on, if enough of it is left.
    if (ext) {
        const uintptr_t a = reinterpret_cast<uintptr_t>(ext), up = (a + 15) & ~(uintptr_t)15;
        if (ext_len >= (up - a) && ext_len - (up - a) >= need) {
            ptr_ = reinterpret_cast<void *>(up);
            return;
        }
    }
    if (!qa || !qa->alloc) throw execution_failed("workspace too small and no queue allocator given");
    ptr_ = qa->alloc(qa->ctx, need);
    if (!ptr_) throw execution_failed("queue allocator returned null for " + std::to_string(need) + " bytes");
    qa_ = qa;
    owned_ = true;
}
Workspace::~Workspace() {
    if (owned_ && qa_->free) qa_->free(qa_->ctx, ptr_);
}

}  // namespace ophip

using namespace ophip;

// ---- embedded code objects (see embed.S, generated by the Makefile) --------
struct EmbeddedModule {
    const char *name;
    const unsigned char *begin;
    const unsigned char *end;
};
extern "C" const EmbeddedModule ophip_embedded_modules[];
extern "C" const unsigned ophip_embedded_module_count;

void ophip_device::make_current() const { check_hip(hipSetDevice(ordinal), "hipSetDevice"); }

hipFunction_t ophip_device::kernel(const char *module, const char *kernel) {
    const std::string key = std::string(module) + "::" + kernel;
    {
        std::shared_lock<std::shared_mutex> rd(mu);
        auto it = functions.find(key);
        if (it != functions.end()) return it->second;
    }
    std::unique_lock<std::shared_mutex> wr(mu);
    auto it = functions.find(key);
    if (it != functions.end()) return it->second;
    make_current();
    hipModule_t mod = nullptr;
    auto mit = modules.find(module);
    if (mit != modules.end()) {
        mod = mit->second;
    } else {
        const EmbeddedModule *em = nullptr;
        for (unsigned i = 0; i < ophip_embedded_module_count; ++i)
            if (std::strcmp(ophip_embedded_modules[i].name, module) == 0) em = &ophip_embedded_modules[i];
        if (!em) throw execution_failed(std::string("no embedded code object named ") + module);
        check_hip(hipModuleLoadData(&mod, em->begin), "hipModuleLoadData");
        modules[module] = mod;
    }
    hipFunction_t fn = nullptr;
    check_hip(hipModuleGetFunction(&fn, mod, kernel), (std::string("hipModuleGetFunction ") + kernel).c_str());
    functions[key] = fn;
    return fn;
}

ophip_device::~ophip_device() {
    for (auto &m : modules) (void)hipModuleUnload(m.second);
}

// A null device (or a null place for the result) from a binding comes back as a status, like every other bad argument.
static ophip_device *need(ophip_device *dev) {
    if (!dev) throw args_not_support("null device");
    return dev;
}
template <typename T>
static T *need_out(T *out) {
    if (!out) throw args_not_support("null argument");
    return out;
}

extern "C" {

const char *ophip_last_error(void) { return g_last_error.c_str(); }

const char *ophip_status_name(int s) {
    switch (s) {
        case OPHIP_OK: return "Ok";
        case OPHIP_TYPE_NOT_SUPPORT: return "TypeNotSupport";
        case OPHIP_TYPE_MISMATCH: return "TypeMismatch";
        case OPHIP_RANK_NOT_SUPPORT: return "RankNotSupport";
        case OPHIP_RANK_MISMATCH: return "RankMismatch";
        case OPHIP_SHAPE_NOT_SUPPORT: return "ShapeNotSupport";
        case OPHIP_SHAPE_MISMATCH: return "ShapeMismatch";
        case OPHIP_STRIDES_NOT_SUPPORT: return "StridesNotSupport";
        case OPHIP_ARGS_NOT_SUPPORT: return "ArgsNotSupport";
        case OPHIP_DYNAMIC_NOT_SUPPORT: return "DynamicNotSupport";
        case OPHIP_EXECUTION_FAILED: return "ExecutionFailed";
        default: return "Unknown";
    }
}

size_t ophip_dtype_nbytes(uint64_t dt) {
    switch (dt) {
        case OPHIP_DT_F16: case OPHIP_DT_BF16: case OPHIP_DT_U16: case OPHIP_DT_I16: return 2;
        case OPHIP_DT_F32: case OPHIP_DT_U32: case OPHIP_DT_I32: return 4;
        case OPHIP_DT_F64: case OPHIP_DT_U64: case OPHIP_DT_I64: case OPHIP_DT_KVPAIR: return 8;
        case OPHIP_DT_U8: case OPHIP_DT_I8: case OPHIP_DT_BOOL: return 1;
        default: return 0;
    }
}

int ophip_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

int ophip_device_create(int ordinal, const ophip_config *cfg, ophip_device **out) {
    return guard([&] {
        if (!out) throw args_not_support("out is null");
        int n = 0;
        check_hip(hipGetDeviceCount(&n), "hipGetDeviceCount");
        if (ordinal < 0 || ordinal >= n) throw execution_failed("no HIP device with ordinal " + std::to_string(ordinal));
        auto *d = new ophip_device();
        d->ordinal = ordinal;
        if (cfg) d->config = *cfg;
        try {
            d->make_current();
            check_hip(hipGetDeviceProperties(&d->props, ordinal), "hipGetDeviceProperties");
            if (std::strncmp(d->props.gcnArchName, "gfx950", 6) != 0)
                throw execution_failed(std::string("this library carries gfx950 code only, device is ") +
                                       d->props.gcnArchName);
            static_scratch_resolve(ordinal);  // the device is current: its copy of the library's scratch array
        } catch (...) {
            delete d;
            throw;
        }
        *out = d;
    });
}

void ophip_device_retain(ophip_device *dev) {
    if (dev) dev->refs.fetch_add(1);
}
void ophip_device_release(ophip_device *dev) {
    if (dev && dev->refs.fetch_sub(1) == 1) delete dev;
}

int ophip_device_get_info(const ophip_device *dev, ophip_device_info *out) {
    return guard([&] {
        if (!dev || !out) throw args_not_support("null argument");
        std::memset(out, 0, sizeof(*out));
        std::snprintf(out->name, sizeof(out->name), "%.*s", (int)sizeof(out->name) - 1, dev->props.name);
        std::snprintf(out->arch, sizeof(out->arch), "%.*s", (int)sizeof(out->arch) - 1, dev->props.gcnArchName);
        out->compute_units = dev->props.multiProcessorCount;
        out->wavefront_size = dev->props.warpSize;
        out->max_threads_per_block = dev->props.maxThreadsPerBlock;
        out->lds_per_block = dev->props.sharedMemPerBlock;
        out->total_memory = dev->props.totalGlobalMem;
        out->clock_khz = dev->props.clockRate;
    });
}

int ophip_malloc(ophip_device *dev, size_t size, void **out) {
    return guard([&] {
        need(dev)->make_current();
        *need_out(out) = nullptr;
        if (size) check_hip(hipMalloc(out, size), "hipMalloc");
    });
}
int ophip_free(ophip_device *dev, void *ptr) {
    return guard([&] {
        need(dev)->make_current();
        if (ptr) check_hip(hipFree(ptr), "hipFree");
    });
}
static int copy(ophip_device *dev, void *dst, const void *src, size_t size, ophip_stream stream, hipMemcpyKind kind) {
    return guard([&] {
        need(dev)->make_current();
        if (!size) return;
        if (!dst || !src) throw args_not_support("null pointer");
        // hipMemcpyAsync on the caller's stream; a null stream makes the call synchronous: the data is in
        // place when it returns.  HIP does not promise that a copy between device buffers or a fill has
        // finished when hipMemcpy / hipMemset return, and work on the caller's own (non-blocking) streams
        // does not wait for the null stream; hence the explicit wait.
        if (stream) {
            check_hip(hipMemcpyAsync(dst, src, size, kind, (hipStream_t)stream), "hipMemcpyAsync");
        } else {
            check_hip(hipMemcpy(dst, src, size, kind), "hipMemcpy");
            check_hip(hipStreamSynchronize(nullptr), "hipStreamSynchronize");
        }
    });
}
int ophip_memcpy_h2d(ophip_device *dev, void *dst, const void *src, size_t size, ophip_stream stream) {
    return copy(dev, dst, src, size, stream, hipMemcpyHostToDevice);
}
int ophip_memcpy_d2h(ophip_device *dev, void *dst, const void *src, size_t size, ophip_stream stream) {
    return copy(dev, dst, src, size, stream, hipMemcpyDeviceToHost);
}
int ophip_memcpy_d2d(ophip_device *dev, void *dst, const void *src, size_t size, ophip_stream stream) {
    return copy(dev, dst, src, size, stream, hipMemcpyDeviceToDevice);
}
int ophip_memset(ophip_device *dev, void *dst, int value, size_t size, ophip_stream stream) {
    return guard([&] {
        need(dev)->make_current();
        if (!size) return;
        if (!dst) throw args_not_support("null pointer");
        if (stream) {
            // a kernel, not hipMemsetAsync: callers record their streams into graphs, and a fill that is an
            // ordinary kernel node replays like every other launch
            const uintptr_t a = reinterpret_cast<uintptr_t>(dst);
            FillBytesParams f{};
            f.dst = dst;
            f.head = (uint32_t)std::min<size_t>(size, (16 - a % 16) % 16);
            f.body = (size - f.head) / 16;
            f.tail = (uint32_t)(size - f.head - f.body * 16);
            f.value = (uint32_t)(value & 0xff) * 0x01010101u;
            const uint64_t blocks = std::max<uint64_t>(1, std::min<uint64_t>((f.body + 255) / 256, 8192));
            launch(dev->kernel("rearrange", "fill_bytes"), Dim3{(unsigned)blocks}, Dim3{256}, 0, (hipStream_t)stream, f);
        } else {
            check_hip(hipMemset(dst, value, size), "hipMemset");
            check_hip(hipStreamSynchronize(nullptr), "hipStreamSynchronize");
        }
    });
}
int ophip_stream_create(ophip_device *dev, ophip_stream *out) {
    return guard([&] {
        need(dev)->make_current();
        hipStream_t s;
        need_out(out);
        check_hip(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "hipStreamCreate");
        *out = s;
    });
}
int ophip_stream_destroy(ophip_device *dev, ophip_stream stream) {
    return guard([&] {
        need(dev)->make_current();
        // What the hooks hand on to other streams (mat_mul's arrival counters) must be at rest first.  The wait happens
        // before the lock is taken, so that creating or destroying an operator on this device never waits for this
        // stream's work.  A stream that is still recording cannot be waited for; its buffers are then not handed on
        // (the graph being recorded may hold their addresses): the operators that own them free them when they go.
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        const bool recording = hipStreamIsCapturing((hipStream_t)stream, &capturing) == hipSuccess &&
                               capturing != hipStreamCaptureStatusNone;
        if (!recording) {
            check_hip(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
            std::lock_guard<std::mutex> lock(dev->hooks_mu);
            for (auto &h : dev->stream_gone) h.second((hipStream_t)stream);
        } else {
            (void)hipGetLastError();
        }
        check_hip(hipStreamDestroy((hipStream_t)stream), "hipStreamDestroy");
    });
}
int ophip_stream_synchronize(ophip_device *dev, ophip_stream stream) {
    return guard([&] {
        need(dev)->make_current();
        check_hip(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
    });
}
int ophip_event_create(ophip_device *dev, ophip_event *out) {
    return guard([&] {
        need(dev)->make_current();
        hipEvent_t e;
        need_out(out);
        check_hip(hipEventCreate(&e), "hipEventCreate");
        *out = e;
    });
}
int ophip_event_destroy(ophip_device *dev, ophip_event ev) {
    return guard([&] {
        need(dev)->make_current();
        if (ev) check_hip(hipEventDestroy((hipEvent_t)ev), "hipEventDestroy");
    });
}
int ophip_event_record(ophip_device *dev, ophip_event ev, ophip_stream stream) {
    return guard([&] {
        need(dev)->make_current();
        if (!ev) throw args_not_support("null event");
        check_hip(hipEventRecord((hipEvent_t)ev, (hipStream_t)stream), "hipEventRecord");
    });
}
int ophip_event_synchronize(ophip_device *dev, ophip_event ev) {
    return guard([&] {
        need(dev)->make_current();
        if (!ev) throw args_not_support("null event");
        check_hip(hipEventSynchronize((hipEvent_t)ev), "hipEventSynchronize");
    });
}
int ophip_event_elapsed_ms(ophip_device *dev, ophip_event start, ophip_event stop, float *ms) {
    return guard([&] {
        need(dev)->make_current();
        if (!start || !stop) throw args_not_support("null event");
        check_hip(hipEventElapsedTime(need_out(ms), (hipEvent_t)start, (hipEvent_t)stop), "hipEventElapsedTime");
    });
}

int ophip_time_next_launch(ophip_device *dev, ophip_stream stream, ophip_event start, ophip_event stop) {
    return guard([&] {
        if (!dev || !start || !stop) throw args_not_support("null argument");
        g_timed.armed = true;
        g_timed.stream = (hipStream_t)stream;
        g_timed.start = (hipEvent_t)start;
        g_timed.stop = (hipEvent_t)stop;
    });
}

// ---- launch graphs ------------------------------------------------------------
// Every launch() of this library only enqueues kernels (and stream-ordered allocations) on
// the caller's stream, so a fixed sequence of them can be recorded once and replayed.
int ophip_stream_begin_capture(ophip_device *dev, ophip_stream stream) {
    return guard([&] {
        need(dev)->make_current();
        check_hip(hipStreamBeginCapture((hipStream_t)stream, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
    });
}
int ophip_stream_end_capture(ophip_device *dev, ophip_stream stream, ophip_graph *out) {
    return guard([&] {
        need(dev)->make_current();
        hipGraph_t graph = nullptr;
        need_out(out);
        check_hip(hipStreamEndCapture((hipStream_t)stream, &graph), "hipStreamEndCapture");
        hipGraphExec_t exec = nullptr;
        const hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
        (void)hipGraphDestroy(graph);
        check_hip(e, "hipGraphInstantiate");
        *out = exec;
    });
}
int ophip_graph_launch(ophip_device *dev, ophip_graph graph, ophip_stream stream) {
    return guard([&] {
        need(dev)->make_current();
        if (!graph) throw args_not_support("null graph");
        check_hip(hipGraphLaunch((hipGraphExec_t)graph, (hipStream_t)stream), "hipGraphLaunch");
    });
}
int ophip_graph_destroy(ophip_device *dev, ophip_graph graph) {
    return guard([&] {
        need(dev)->make_current();
        if (graph) check_hip(hipGraphExecDestroy((hipGraphExec_t)graph), "hipGraphExecDestroy");
    });
}

// ---- impl QueueAlloc for Stream (handle/cuda/alloc.rs:103-123) --------------
static void *stream_alloc(void *ctx, size_t size) {
    void *p = nullptr;
    // zero-size requests still yield a valid (unique) allocation, as DevMem of length 0 would
    if (hipMallocAsync(&p, size ? size : 1, (hipStream_t)ctx) != hipSuccess) return nullptr;
    return p;
}
static void stream_free(void *ctx, void *ptr) {
    if (ptr) (void)hipFreeAsync(ptr, (hipStream_t)ctx);
}
int ophip_queue_alloc_from_stream(ophip_device *dev, ophip_stream stream, ophip_queue_alloc *out) {
    return guard([&] {
        if (!dev || !out) throw args_not_support("null argument");
        out->ctx = stream;
        out->stream = stream;
        out->alloc = stream_alloc;
        out->free = stream_free;
    });
}

}  // extern "C"

// ---- OffsetCalculator (common/calculator.rs:8-86) ---------------------------
struct ophip_offset_calculator {
    size_t alignment;
    std::set<std::pair<size_t, size_t>> free_list;  // (len, off): best fit = lower_bound
    std::unordered_map<size_t, size_t> heads, tails;

    void insert_area(size_t off, size_t len) {
        free_list.insert({len, off});
        heads[off] = len;
        tails[off + len] = len;
    }
    void put(size_t start, size_t end) {
        size_t len = (end - start + alignment - 1) / alignment * alignment;
        if (len == 0) return;
        size_t head = start, tail = head + len;
        auto t = tails.find(head);
        if (t != tails.end()) {
            const size_t l = t->second;
            tails.erase(t);
            head -= l;
            free_list.erase({l, head});
            heads.erase(head);
        }
        auto h = heads.find(tail);
        if (h != heads.end()) {
            const size_t l = h->second;
            heads.erase(h);
            free_list.erase({l, tail});
            tail += l;
            tails.erase(tail);
        }
        insert_area(head, tail - head);
    }
    bool take(size_t expect, size_t *start, size_t *end) {
        const size_t len = (expect + alignment - 1) / alignment * alignment;
        if (len == 0) {
            *start = *end = SIZE_MAX;
            return true;
        }
        auto it = free_list.lower_bound({len, 0});
        if (it == free_list.end()) return false;
        const size_t flen = it->first, foff = it->second;
        free_list.erase(it);
        heads.erase(foff);
        tails.erase(foff + flen);
        if (flen > len) insert_area(foff + len, flen - len);
        *start = foff;
        *end = foff + expect;
        return true;
    }
};

// ---- StreamMemPool (handle/cuda/alloc.rs:10-90) ----------------------------
struct ophip_mem_pool {
    ophip_device *dev;
    hipStream_t stream;
    std::mutex mu;
    std::vector<void *> slabs;
    ophip_offset_calculator calc;
    std::unordered_map<void *, size_t> live;  // ptr -> requested size
};

static void *pool_alloc(void *ctx, size_t size) {
    auto *pool = static_cast<ophip_mem_pool *>(ctx);
    std::lock_guard<std::mutex> lock(pool->mu);
    size_t s, e;
    if (!pool->calc.take(size, &s, &e)) return nullptr;  // the reference panics with "out of memory"
    void *p = reinterpret_cast<void *>(s);
    if (size) pool->live[p] = size;
    return p;
}
static void pool_free(void *ctx, void *ptr) {
    auto *pool = static_cast<ophip_mem_pool *>(ctx);
    std::lock_guard<std::mutex> lock(pool->mu);
    auto it = pool->live.find(ptr);
    if (it == pool->live.end()) return;
    const size_t s = reinterpret_cast<size_t>(ptr);
    pool->calc.put(s, s + it->second);
    pool->live.erase(it);
}

extern "C" {

ophip_offset_calculator *ophip_offset_calculator_create(size_t alignment) {
    auto *c = new ophip_offset_calculator();
    c->alignment = alignment ? alignment : 1;
    return c;
}
void ophip_offset_calculator_destroy(ophip_offset_calculator *c) { delete c; }
void ophip_offset_calculator_put(ophip_offset_calculator *c, size_t start, size_t end) {
    if (c) c->put(start, end);
}
int ophip_offset_calculator_take(ophip_offset_calculator *c, size_t size, size_t *start, size_t *end) {
    return c && start && end && c->take(size, start, end) ? 1 : 0;
}

int ophip_mem_pool_create(ophip_device *dev, ophip_stream stream, ophip_mem_pool **out) {
    return guard([&] {
        if (!dev || !out) throw args_not_support("null argument");
        auto *p = new ophip_mem_pool();
        p->dev = dev;
        ophip_device_retain(dev);
        p->stream = (hipStream_t)stream;
        p->calc.alignment = 256;  // the reference falls back to 256 when the device reports 0
        *out = p;
    });
}
int ophip_mem_pool_put(ophip_mem_pool *pool, size_t size) {
    return guard([&] {
        if (!pool) throw args_not_support("null argument");
        pool->dev->make_current();
        void *p = nullptr;
        check_hip(hipMalloc(&p, size), "hipMalloc");
        std::lock_guard<std::mutex> lock(pool->mu);
        pool->slabs.push_back(p);
        const size_t s = reinterpret_cast<size_t>(p);
        pool->calc.put(s, s + size);
    });
}
int ophip_mem_pool_queue_alloc(ophip_mem_pool *pool, ophip_queue_alloc *out) {
    return guard([&] {
        if (!pool || !out) throw args_not_support("null argument");
        out->ctx = pool;
        out->stream = pool->stream;
        out->alloc = pool_alloc;
        out->free = pool_free;
    });
}
void ophip_mem_pool_destroy(ophip_mem_pool *pool) {
    if (!pool) return;
    (void)hipSetDevice(pool->dev->ordinal);
    for (void *p : pool->slabs) (void)hipFree(p);
    ophip_device_release(pool->dev);
    delete pool;
}

}  // extern "C"
