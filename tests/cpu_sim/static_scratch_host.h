// Force-included when host/static_scratch.hip is compiled as plain C++ for a sanitizer build of the stand-in library:
// what the file needs from <hip/hip_runtime.h> beyond the runtime API (its device array becomes a host array, whose
// address hipGetSymbolAddress hands back).
#pragma once
#include <hip/hip_runtime_api.h>
#ifndef __device__
#define __device__
#endif
#define __align__(n) __attribute__((aligned(n)))
#ifndef HIP_SYMBOL
#define HIP_SYMBOL(x) (&(x))
#endif
