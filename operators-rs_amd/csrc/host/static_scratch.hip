// ophip_mat_mul_launch_static: mat_mul for callers that cannot allocate (a stream being recorded into a
// graph, a serving loop, a harness that forbids hipMalloc).  The split-K scratch of the launch -- f32
// partials and arrival counters, what ophip_mat_mul_launch takes from the caller's workspace, the queue
// allocator and the operator's own counter buffers -- lives in one file-scope device array of this
// library.  Each GPU the library runs on holds its own copy of the array, at its own address, until the
// process ends.
//
// This file is compiled by hipcc for host and device: the array is a device symbol, its host-side name is
// only a handle for hipGetSymbolAddress.  The address is resolved once per device (ophip_device_create,
// with that device current) and kept; everything that touches the array afterwards uses the resolved pointer.
#include <hip/hip_runtime.h>

#include <mutex>
#include <string>

#include "handle.hpp"
#include "static_scratch.hpp"

namespace {

constexpr size_t COUNTER_BYTES = ophip::STATIC_COUNTERS * sizeof(uint32_t);
constexpr size_t SCRATCH_BYTES = ophip::STATIC_PARTIAL_BYTES + COUNTER_BYTES;

// [0, STATIC_PARTIAL_BYTES): f32 partials; then STATIC_COUNTERS u32 arrival counters.  The array is zero when the
// module is loaded, and a kernel that counts arrivals sets the counters it used back to zero before it ends: the
// counters are zero between launches without anyone clearing them (calls that overlap on one GPU, which the entry
// point's contract rules out, would break that).
static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];

constexpr int MAX_DEVICES = 64;
std::mutex g_mu;
void *g_scratch_ptr[MAX_DEVICES];    // per device ordinal: the array's address on that device, null = not resolved
std::string g_why_not[MAX_DEVICES];  // per device ordinal: what hipGetSymbolAddress answered when it failed

}  // namespace

namespace ophip {

void static_scratch_resolve(int ordinal) {
    if (ordinal < 0 || ordinal >= MAX_DEVICES) return;  // such a device works, only the static entry point refuses it
    std::lock_guard<std::mutex> lock(g_mu);
    if (g_scratch_ptr[ordinal]) return;
    void *ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
        // the other entry points do not need the array: the device is created, ophip_mat_mul_launch_static reports this
        g_why_not[ordinal] = std::string("hipGetSymbolAddress(scratch): ") + (e != hipSuccess ? hipGetErrorString(e) : "null address");
        (void)hipGetLastError();
        return;
    }
    g_scratch_ptr[ordinal] = ptr;
}

}  // namespace ophip

using namespace ophip;

extern "C" OPHIP_API int ophip_mat_mul_launch_static(const ophip_mat_mul *op, const ophip_mat_mul_args *args,
                                                     ophip_stream stream) {
    return guard([&] {
        if (!op || !args) throw args_not_support("null argument");
        const ophip_device *dev = mat_mul_device(op);
        void *ptr = nullptr;
        {
            std::lock_guard<std::mutex> lock(g_mu);
            if (dev->ordinal < 0 || dev->ordinal >= MAX_DEVICES)
                throw execution_failed("the static scratch array serves device ordinals below " + std::to_string(MAX_DEVICES));
            ptr = g_scratch_ptr[dev->ordinal];
            if (!ptr)
                throw execution_failed("the static scratch array was not resolved on device " + std::to_string(dev->ordinal) +
                                       ": " + g_why_not[dev->ordinal]);
        }
        unsigned char *base = static_cast<unsigned char *>(ptr);
        mat_mul_launch_fixed_scratch(op, args, base, STATIC_PARTIAL_BYTES, base + STATIC_PARTIAL_BYTES, STATIC_COUNTERS,
                                     (hipStream_t)stream);
    });
}
