// The hardware handle of the HIP backend: what `Gpu(Arc<Handle>)`, `ModuleBox`
// and the `cuda` driver crate are to the reference's CUDA backend
// (operators/src/handle/cuda/{mod,module,alloc}.rs), on the HIP module API.
//
// Kernels are built offline into gfx950 code objects (one per operator) that
// are embedded in this library; a module is loaded with hipModuleLoadData the
// first time one of its kernels is asked for and functions are cached by name.
#pragma once
#include <hip/hip_runtime_api.h>

#include <atomic>
#include <functional>
#include <map>
#include <shared_mutex>
#include <string>

#include "common.hpp"

struct ophip_device {
    int ordinal = 0;
    std::atomic<long> refs{1};
    ophip_config config{4, 16, 64};
    hipDeviceProp_t props{};

    // module registry: RwLock<HashMap<name, module>> (handle/cuda/mod.rs:90,124-149)
    std::shared_mutex mu;
    std::map<std::string, hipModule_t> modules;
    std::map<std::string, hipFunction_t> functions;

    // Operators that keep per-stream state (mat_mul's arrival counters) ask to be told when a stream goes away.
    std::mutex hooks_mu;
    std::map<const void *, std::function<void(hipStream_t)>> stream_gone;

    // Function `kernel` of the embedded code object `module`; throws ExecutionFailed.
    hipFunction_t kernel(const char *module, const char *kernel);
    void make_current() const;
    ~ophip_device();
};

namespace ophip {

struct Dim3 {
    unsigned x = 1, y = 1, z = 1;
};

// ModuleBox::launch (handle/cuda/module.rs:39-55): one parameter block, passed by value.
void launch_raw(hipFunction_t fn, Dim3 grid, Dim3 block, size_t smem, hipStream_t stream,
                void *params, size_t params_size);

template <class P>
inline void launch(hipFunction_t fn, Dim3 grid, Dim3 block, size_t smem, hipStream_t stream, const P &params) {
    P copy = params;
    launch_raw(fn, grid, block, smem, stream, &copy, sizeof(P));
}

void check_hip(hipError_t e, const char *what);

// every operator object keeps its device alive
struct OpBase {
    ophip_device *dev;
    explicit OpBase(ophip_device *d) : dev(d) { ophip_device_retain(d); }
    ~OpBase() { ophip_device_release(dev); }
    OpBase(const OpBase &) = delete;
    OpBase &operator=(const OpBase &) = delete;
};

inline unsigned ceil_div(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }

inline hipStream_t stream_of(const ophip_queue_alloc *qa) {
    return qa ? reinterpret_cast<hipStream_t>(qa->stream) : nullptr;
}

// Workspace::new / Drop (common/workspace.rs:7-52): use the caller's slice when it
// is large enough, otherwise borrow from the queue allocator until `release`.
class Workspace {
   public:
    Workspace(const ophip_queue_alloc *qa, void *ext, size_t ext_len, size_t need);
    ~Workspace();
    void *ptr() const { return ptr_; }

   private:
    const ophip_queue_alloc *qa_ = nullptr;
    void *ptr_ = nullptr;
    bool owned_ = false;
};

}  // namespace ophip
