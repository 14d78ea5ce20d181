// The host half of the CPU stand-in for the GPU (tests only): the functions of the HIP runtime that libophip's host
// code calls, with the declarations of the real <hip/hip_runtime_api.h>, so that the library's own host objects link
// against this file instead of libamdhip64 and run unchanged.
//
//   * device memory is host memory, every allocation between two inaccessible pages with its end against the upper one
//     (rounded up to 256 bytes, or to what CPUSIM_ALIGN says), filled with 0xFE (a NaN in every floating-point type the kernels use): an access past
//     an allocation, before it or after hipFree stops the process with the address and the nearest allocation;
//   * streams run in order at once: a launch returns when the kernel has run (cpusim_core.h runs it);
//   * a stream that records keeps the launches and copies; a graph replays them;
//   * code objects are the modules registered by the kernel sources compiled for the host (hip/hip_runtime.h here);
//     a launch checks the size of the argument block against the kernel's parameter type.
#include <hip/hip_runtime_api.h>
#include <signal.h>
#include <sys/mman.h>
#include <unistd.h>

#include <chrono>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "cpusim_core.h"

namespace {

// (everything here may be needed while the library is still being loaded -- the registration calls of hipcc's host
// objects run as static initializers -- so the state is built on first use, not in this file's own initializers)
std::recursive_mutex &mu() {
    static std::recursive_mutex *m = new std::recursive_mutex;
    return *m;
}
#define g_mu mu()

// ---- memory
struct Block {
    char *map;
    size_t map_len;
    size_t size;
};
std::map<uintptr_t, Block> &blocks() {  // by user address
    static auto *m = new std::map<uintptr_t, Block>;
    return *m;
}
std::map<uintptr_t, size_t> &freed() {  // user address -> size, of blocks given back (for the fault message)
    static auto *m = new std::map<uintptr_t, size_t>;
    return *m;
}
#define g_blocks blocks()
#define g_freed freed()
size_t g_live_bytes = 0;
uint64_t g_allocations = 0, g_frees = 0;  // calls that reached the allocator, over the life of the process

void on_fault(int sig, siginfo_t *info, void *) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(info->si_addr);
    char msg[512];
    int n = std::snprintf(msg, sizeof(msg), "\ncpusim: invalid access at %p", info->si_addr);
    const Block *best = nullptr;
    uintptr_t best_user = 0, best_d = ~(uintptr_t)0;
    for (auto &kv : g_blocks) {
        const uintptr_t lo = kv.first, hi = lo + kv.second.size;
        const uintptr_t d = a < lo ? lo - a : a >= hi ? a - hi + 1 : 0;
        if (d < best_d) best_d = d, best = &kv.second, best_user = lo;
    }
    if (best && best_d < (1u << 20))
        n += std::snprintf(msg + n, sizeof(msg) - n, ": %s the device allocation [%#zx, +%zu) by %zd bytes",
                           a < best_user ? "before" : "past the end of", (size_t)best_user, best->size,
                           a < best_user ? (ssize_t)(best_user - a) : (ssize_t)(a - best_user - best->size + 1));
    for (auto &kv : g_freed)
        if (a >= kv.first && a < kv.first + kv.second) n += std::snprintf(msg + n, sizeof(msg) - n, ": inside a device allocation that was freed");
    cpusim::Worker &w = cpusim::worker();
    if (w.cur)
        n += std::snprintf(msg + n, sizeof(msg) - n, "; workgroup (%u, %u, %u), work-item %u", w.block_idx.x, w.block_idx.y, w.block_idx.z, w.cur->flat);
    n += std::snprintf(msg + n, sizeof(msg) - n, "\n");
    (void)!write(2, msg, n);
    signal(sig, SIG_DFL);
    raise(sig);
}

void install_fault_handler() {
    static bool done = false;
    if (done) return;
    done = true;
    static char alt[64 << 10];
    stack_t ss{};
    ss.ss_sp = alt, ss.ss_size = sizeof(alt);
    sigaltstack(&ss, nullptr);
    struct sigaction sa{};
    sa.sa_sigaction = on_fault;
    sa.sa_flags = SA_SIGINFO | SA_ONSTACK;
    sigaction(SIGSEGV, &sa, nullptr);
    sigaction(SIGBUS, &sa, nullptr);
}

hipError_t sim_malloc(void **ptr, size_t size) {
    if (!ptr) return hipErrorInvalidValue;
    std::lock_guard<std::recursive_mutex> lock(g_mu);
    install_fault_handler();
    // hipMalloc hands out addresses on 256-byte boundaries; CPUSIM_ALIGN=16 (or another power of two) gives up that
    // much of it and moves the end of an allocation to within 15 bytes of the guard page: what reads past an
    // operand by a vector or two then shows
    static const size_t align = [] {
        const char *e = std::getenv("CPUSIM_ALIGN");
        const size_t a = e ? (size_t)std::atoi(e) : 256;
        return a >= 16 && a <= 4096 && (a & (a - 1)) == 0 ? a : 256;
    }();
    const size_t user_len = (std::max<size_t>(size, 1) + align - 1) / align * align;
    const size_t body = (user_len + 4095) / 4096 * 4096, map_len = body + 2 * 4096;
    // keep a runaway test from taking the machine's memory: 24 GiB of live allocations, or CPUSIM_MEMORY_GIB
    static const size_t cap = [] {
        const char *e = std::getenv("CPUSIM_MEMORY_GIB");
        return (size_t)(e && std::atoi(e) > 0 ? std::atoi(e) : 24) << 30;
    }();
    if (g_live_bytes + body > cap) return hipErrorOutOfMemory;
    char *m = static_cast<char *>(mmap(nullptr, map_len, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS, -1, 0));
    if (m == MAP_FAILED) return hipErrorOutOfMemory;
    mprotect(m, 4096, PROT_NONE);
    mprotect(m + 4096 + body, 4096, PROT_NONE);
    std::memset(m + 4096, 0xFE, body);
    char *user = m + 4096 + body - user_len;
    g_blocks[reinterpret_cast<uintptr_t>(user)] = Block{m, map_len, size};
    g_freed.erase(reinterpret_cast<uintptr_t>(user));
    g_live_bytes += body;
    ++g_allocations;
    *ptr = user;
    return hipSuccess;
}

hipError_t sim_free(void *ptr) {
    if (!ptr) return hipSuccess;
    std::lock_guard<std::recursive_mutex> lock(g_mu);
    auto it = g_blocks.find(reinterpret_cast<uintptr_t>(ptr));
    if (it == g_blocks.end()) {
        // the library gives back exactly what it took, once: anything else is a bug worth stopping for
        std::fprintf(stderr, "cpusim: hipFree(%p): %s\n", ptr, g_freed.count(reinterpret_cast<uintptr_t>(ptr)) ? "freed before" : "no device allocation starts there");
        std::abort();
    }
    g_live_bytes -= it->second.map_len - 2 * 4096;
    ++g_frees;
    // the pages stay reserved and inaccessible: a later access faults instead of landing in a newer allocation
    mmap(it->second.map, it->second.map_len, PROT_NONE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_FIXED | MAP_NORESERVE, -1, 0);
    g_freed[it->first] = it->second.size;
    g_blocks.erase(it);
    return hipSuccess;
}

// ---- streams, events, graphs
struct Node {
    enum Kind { Launch, Copy, Fill } kind;
    const cpusim::KernelInfo *fn = nullptr;
    cpusim::Dim3u grid, block;
    size_t smem = 0;
    std::vector<unsigned char> params;
    void *dst = nullptr;
    const void *src = nullptr;
    size_t bytes = 0;
    int value = 0;
};
struct SimGraph {
    std::vector<Node> nodes;
};
struct SimStream {
    std::unique_ptr<SimGraph> recording;
};
struct SimEvent {
    double ms = 0;
    bool recorded = false;
};
SimStream g_null_stream;
SimStream *stream_of(hipStream_t s) { return s ? reinterpret_cast<SimStream *>(s) : &g_null_stream; }
double now_ms() {
    return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

void run_node(const Node &n) {
    switch (n.kind) {
        case Node::Launch: {
            const void *params = n.params.data();
            const cpusim::KernelEntry entry = n.fn->entry;
            cpusim::launch(n.grid, n.block, n.smem, [=] { entry(params); });
            break;
        }
        case Node::Copy: std::memmove(n.dst, n.src, n.bytes); break;
        case Node::Fill: std::memset(n.dst, n.value, n.bytes); break;
    }
}
void submit(hipStream_t s, Node &&n) {
    std::lock_guard<std::recursive_mutex> lock(g_mu);
    SimStream *st = stream_of(s);
    if (st->recording) st->recording->nodes.push_back(std::move(n));
    else run_node(n);
}

struct SimModule {
    std::string name;
};

hipError_t launch(hipFunction_t f, cpusim::Dim3u grid, cpusim::Dim3u block, size_t smem, hipStream_t stream, void **kernel_params, void **extra) {
    if (!f || kernel_params || !extra) return hipErrorInvalidValue;  // the library passes one argument block through `extra`
    const void *buf = nullptr;
    size_t size = 0;
    for (void **e = extra; *e != HIP_LAUNCH_PARAM_END; e += 2) {
        if (*e == HIP_LAUNCH_PARAM_BUFFER_POINTER) buf = e[1];
        else if (*e == HIP_LAUNCH_PARAM_BUFFER_SIZE) size = *static_cast<size_t *>(e[1]);
        else return hipErrorInvalidValue;
    }
    const cpusim::KernelInfo *info = reinterpret_cast<const cpusim::KernelInfo *>(f);
    if (!buf || size != info->params_size) {
        std::fprintf(stderr, "cpusim: a launch with %zu bytes of arguments for a kernel whose parameter has %zu\n", size, info->params_size);
        return hipErrorInvalidValue;
    }
    const uint64_t threads = (uint64_t)block.x * block.y * block.z;
    if (!grid.x || !grid.y || !grid.z || !threads || threads > 1024 || grid.y > 65535 || grid.z > 65535 || smem > (160u << 10)) return hipErrorInvalidConfiguration;
    Node n;
    n.kind = Node::Launch;
    n.fn = info;
    n.grid = grid, n.block = block, n.smem = smem;
    n.params.assign(static_cast<const unsigned char *>(buf), static_cast<const unsigned char *>(buf) + size);
    submit(stream, std::move(n));
    return hipSuccess;
}

// device symbols of host + device objects (hipcc's registration calls): host-side name -> size, storage on first use
struct Symbol {
    size_t size;
    void *storage;
};
std::map<const void *, Symbol> &symbols() {
    static auto *m = new std::map<const void *, Symbol>;
    return *m;
}
#define g_symbols symbols()

}  // namespace

extern "C" {

// ---- what hipcc's host objects call when they are loaded
void **__hipRegisterFatBinary(const void *) {
    static void *handle[1];
    return handle;
}
void __hipUnregisterFatBinary(void **) {}
void __hipRegisterVar(void **, void *host_var, char *, char *, int, size_t size, int, int) {
    std::lock_guard<std::recursive_mutex> lock(g_mu);
    g_symbols[host_var] = Symbol{size, nullptr};
}
void __hipRegisterFunction(void **, const void *, char *, const char *, unsigned, void *, void *, void *, void *, int *) {}

hipError_t hipGetSymbolAddress(void **ptr, const void *symbol) {
    std::lock_guard<std::recursive_mutex> lock(g_mu);
    auto it = g_symbols.find(symbol);
    if (!ptr || !symbol) return hipErrorInvalidSymbol;
    if (it == g_symbols.end()) {
        // nobody registered it: the file that owns the array was compiled as plain C++ (the sanitizer build), the array is a host array
        *ptr = const_cast<void *>(symbol);
        return hipSuccess;
    }
    if (!it->second.storage) {
        // (module memory, not an allocation of the program: it stays out of the allocator's books)
        const size_t live = g_live_bytes;
        if (sim_malloc(&it->second.storage, it->second.size) != hipSuccess) return hipErrorOutOfMemory;
        g_live_bytes = live, --g_allocations;
        std::memset(it->second.storage, 0, it->second.size);  // a device array without an initializer is zero when its module is loaded
    }
    *ptr = it->second.storage;
    return hipSuccess;
}

// ---- devices
hipError_t hipGetDeviceCount(int *n) {
    *n = 1;
    return hipSuccess;
}
hipError_t hipSetDevice(int d) { return d == 0 ? hipSuccess : hipErrorInvalidDevice; }
hipError_t hipGetDeviceProperties(hipDeviceProp_t *p, int d) {
    if (d != 0 || !p) return hipErrorInvalidDevice;
    std::memset(p, 0, sizeof(*p));
    std::snprintf(p->name, sizeof(p->name), "MI355X stand-in on the CPU");
    std::snprintf(p->gcnArchName, sizeof(p->gcnArchName), "gfx950:cpusim");
    p->multiProcessorCount = 256;
    p->warpSize = 64;
    p->maxThreadsPerBlock = 1024;
    p->sharedMemPerBlock = 64 << 10;
    p->totalGlobalMem = (size_t)288 << 30;
    p->clockRate = 2400000;
    return hipSuccess;
}
const char *hipGetErrorName(hipError_t e) {
    switch (e) {
        case hipSuccess: return "hipSuccess";
        case hipErrorInvalidValue: return "hipErrorInvalidValue";
        case hipErrorOutOfMemory: return "hipErrorOutOfMemory";
        case hipErrorInvalidConfiguration: return "hipErrorInvalidConfiguration";
        case hipErrorNotFound: return "hipErrorNotFound";
        case hipErrorInvalidSymbol: return "hipErrorInvalidSymbol";
        case hipErrorInvalidDevice: return "hipErrorInvalidDevice";
        default: return "hipError (stand-in)";
    }
}
const char *hipGetErrorString(hipError_t e) { return hipGetErrorName(e); }
hipError_t hipGetLastError(void) { return hipSuccess; }

// ---- memory
hipError_t hipMalloc(void **ptr, size_t size) { return sim_malloc(ptr, size); }
hipError_t hipFree(void *ptr) { return sim_free(ptr); }
hipError_t hipMallocAsync(void **ptr, size_t size, hipStream_t) { return sim_malloc(ptr, size); }
hipError_t hipFreeAsync(void *ptr, hipStream_t) { return sim_free(ptr); }
hipError_t hipMemcpy(void *dst, const void *src, size_t n, hipMemcpyKind) {
    std::memmove(dst, src, n);
    return hipSuccess;
}
hipError_t hipMemcpyAsync(void *dst, const void *src, size_t n, hipMemcpyKind kind, hipStream_t s) {
    // a copy from host memory takes the bytes now, as a recording stream's copy node of pageable memory would not; the
    // library only records device-to-device copies
    if (stream_of(s)->recording && kind != hipMemcpyDeviceToDevice) return hipErrorStreamCaptureUnsupported;
    Node node;
    node.kind = Node::Copy;
    node.dst = dst, node.src = src, node.bytes = n;
    submit(s, std::move(node));
    return hipSuccess;
}
hipError_t hipMemset(void *dst, int value, size_t n) {
    std::memset(dst, value, n);
    return hipSuccess;
}

// ---- streams and events
hipError_t hipStreamCreateWithFlags(hipStream_t *s, unsigned) {
    *s = reinterpret_cast<hipStream_t>(new SimStream);
    return hipSuccess;
}
hipError_t hipStreamDestroy(hipStream_t s) {
    delete reinterpret_cast<SimStream *>(s);
    return hipSuccess;
}
hipError_t hipStreamSynchronize(hipStream_t s) { return stream_of(s)->recording ? hipErrorStreamCaptureUnsupported : hipSuccess; }
hipError_t hipEventCreate(hipEvent_t *e) {
    *e = reinterpret_cast<hipEvent_t>(new SimEvent);
    return hipSuccess;
}
hipError_t hipEventDestroy(hipEvent_t e) {
    delete reinterpret_cast<SimEvent *>(e);
    return hipSuccess;
}
hipError_t hipEventRecord(hipEvent_t e, hipStream_t) {
    SimEvent *ev = reinterpret_cast<SimEvent *>(e);
    ev->ms = now_ms(), ev->recorded = true;
    return hipSuccess;
}
hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
hipError_t hipEventElapsedTime(float *ms, hipEvent_t a, hipEvent_t b) {
    SimEvent *x = reinterpret_cast<SimEvent *>(a), *y = reinterpret_cast<SimEvent *>(b);
    if (!x->recorded || !y->recorded) return hipErrorInvalidHandle;
    *ms = (float)(y->ms - x->ms);
    return hipSuccess;
}

// ---- recording and replay
hipError_t hipStreamBeginCapture(hipStream_t s, hipStreamCaptureMode) {
    SimStream *st = stream_of(s);
    if (st->recording) return hipErrorIllegalState;
    st->recording = std::make_unique<SimGraph>();
    return hipSuccess;
}
hipError_t hipStreamEndCapture(hipStream_t s, hipGraph_t *g) {
    SimStream *st = stream_of(s);
    if (!st->recording) return hipErrorIllegalState;
    *g = reinterpret_cast<hipGraph_t>(st->recording.release());
    return hipSuccess;
}
hipError_t hipStreamIsCapturing(hipStream_t s, hipStreamCaptureStatus *status) {
    *status = stream_of(s)->recording ? hipStreamCaptureStatusActive : hipStreamCaptureStatusNone;
    return hipSuccess;
}
hipError_t hipGraphInstantiate(hipGraphExec_t *exec, hipGraph_t g, hipGraphNode_t *, char *, size_t) {
    *exec = reinterpret_cast<hipGraphExec_t>(new SimGraph(*reinterpret_cast<SimGraph *>(g)));
    return hipSuccess;
}
hipError_t hipGraphDestroy(hipGraph_t g) {
    delete reinterpret_cast<SimGraph *>(g);
    return hipSuccess;
}
hipError_t hipGraphExecDestroy(hipGraphExec_t g) {
    delete reinterpret_cast<SimGraph *>(g);
    return hipSuccess;
}
hipError_t hipGraphLaunch(hipGraphExec_t g, hipStream_t s) {
    if (stream_of(s)->recording) return hipErrorStreamCaptureUnsupported;
    std::lock_guard<std::recursive_mutex> lock(g_mu);
    for (const Node &n : reinterpret_cast<SimGraph *>(g)->nodes) run_node(n);
    return hipSuccess;
}

// ---- code objects: the "image" of a module is its name (sim_modules.cpp, generated)
hipError_t hipModuleLoadData(hipModule_t *m, const void *image) {
    *m = reinterpret_cast<hipModule_t>(new SimModule{static_cast<const char *>(image)});
    return hipSuccess;
}
hipError_t hipModuleUnload(hipModule_t m) {
    delete reinterpret_cast<SimModule *>(m);
    return hipSuccess;
}
hipError_t hipModuleGetFunction(hipFunction_t *f, hipModule_t m, const char *name) {
    auto &reg = cpusim::registry();
    auto it = reg.find(name);
    if (it == reg.end() || it->second.module != reinterpret_cast<SimModule *>(m)->name) return hipErrorNotFound;
    *f = reinterpret_cast<hipFunction_t>(&it->second);
    return hipSuccess;
}
hipError_t hipModuleLaunchKernel(hipFunction_t f, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned by, unsigned bz, unsigned smem,
                                 hipStream_t stream, void **kernel_params, void **extra) {
    return launch(f, {gx, gy, gz}, {bx, by, bz}, smem, stream, kernel_params, extra);
}
// (sizes in work-items, as OpenCL counts them)
hipError_t hipExtModuleLaunchKernel(hipFunction_t f, uint32_t wx, uint32_t wy, uint32_t wz, uint32_t bx, uint32_t by, uint32_t bz, size_t smem,
                                    hipStream_t stream, void **kernel_params, void **extra, hipEvent_t start, hipEvent_t stop, uint32_t) {
    if (!bx || !by || !bz || wx % bx || wy % by || wz % bz) return hipErrorInvalidConfiguration;
    if (start) hipEventRecord(start, stream);
    const hipError_t e = launch(f, {wx / bx, wy / by, wz / bz}, {bx, by, bz}, smem, stream, kernel_params, extra);
    if (stop) hipEventRecord(stop, stream);
    return e;
}

// ---- for the tests: counters of the stand-in itself
//   [0] launches run, [1] workgroups run, [2] buffer loads past a resource's records, [3] buffer stores past them, [4] bytes of live device allocations,
//   [5..7] bytes loaded through buffer resources with the plain, non-temporal and sc1 cache policy, [8..10] bytes stored likewise
//   (of the calling thread's launches: a launch runs on the thread that makes it), [11] device and pinned allocations made, [12] freed (by any thread)
void cpusim_counters(uint64_t out[13]) {
    cpusim::Worker &w = cpusim::worker();
    out[0] = w.launches, out[1] = w.workgroups, out[2] = w.out_of_range_loads, out[3] = w.out_of_range_stores, out[4] = g_live_bytes;
    for (int i = 0; i < 3; ++i) out[5 + i] = w.buffer_load_bytes[i], out[8 + i] = w.buffer_store_bytes[i];
    std::lock_guard<std::recursive_mutex> lock(g_mu);
    out[11] = g_allocations, out[12] = g_frees;
}

}  // extern "C"
