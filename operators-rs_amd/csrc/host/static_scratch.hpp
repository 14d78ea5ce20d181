// Scratch memory that belongs to the library itself: one file-scope device array per GPU, for the
// entry point that must not allocate (see static_scratch.hip).
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstddef>

#include "ophip.h"

namespace ophip {

// Bytes of f32 split-K partials and number of u32 arrival counters the static array holds.
constexpr size_t STATIC_PARTIAL_BYTES = (size_t)32 << 20;
constexpr size_t STATIC_COUNTERS = (size_t)1 << 16;

// Resolves the array's address on device `ordinal`, which must be the current device; called once per
// device from ophip_device_create.  Never throws: when the address cannot be had the reason is kept, the device is
// created all the same (nothing else needs the array), and ophip_mat_mul_launch_static reports the reason.
void static_scratch_resolve(int ordinal);

// mat_mul.cpp: one launch whose scratch (partials, counters) is all brought by the caller of this function.
void mat_mul_launch_fixed_scratch(const ophip_mat_mul *op, const ophip_mat_mul_args *args, void *partials,
                                  size_t partial_bytes, void *counters, size_t counter_count, hipStream_t stream);

const ophip_device *mat_mul_device(const ophip_mat_mul *op);

}  // namespace ophip
