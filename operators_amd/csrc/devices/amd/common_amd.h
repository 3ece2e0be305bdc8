// Host-side helpers shared by the amd-gpu operators: HIP error mapping, element
// type comparison and the shape predicates the create functions use.  Plays the
// part of src/devices/cuda/common_cuda.h:10-21 and of the predicates in
// src/ops/utils.h:62-72,85-143,174-188 of the reference.
#ifndef INFINIOP_AMD_COMMON_H
#define INFINIOP_AMD_COMMON_H

#include "operators.h"
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <hip/hip_runtime_api.h>

// Report a failed HIP runtime call on stderr and leave the calling function
// with `code`.  The library never throws and never aborts.
#define AMD_CHECK_HIP(call, code)                                                  \
    do {                                                                           \
        hipError_t err__ = (call);                                                 \
        if (err__ != hipSuccess) {                                                 \
            std::fprintf(stderr, "infiniop[amd-gpu]: %s -> %s (%s:%d)\n", #call,   \
                         hipGetErrorString(err__), __FILE__, __LINE__);            \
            return (code);                                                         \
        }                                                                          \
    } while (0)

namespace amd {

// Element types this back end distinguishes.
enum class Elem : int { F16 = 0, BF16 = 1, F32 = 2, Other = 3 };

inline uint32_t dt_bits(DataLayout d) {
    uint32_t u;
    static_assert(sizeof(DataLayout) == 4, "DataLayout is a 32-bit image");
    std::memcpy(&u, &d, 4);
    return u;
}
inline bool same_dt(DataLayout a, DataLayout b) { return dt_bits(a) == dt_bits(b); }
inline Elem elem_of(DataLayout d) {
    if (same_dt(d, F16)) return Elem::F16;
    if (same_dt(d, BF16)) return Elem::BF16;
    if (same_dt(d, F32)) return Elem::F32;
    return Elem::Other;
}

// The reference's notion of contiguity: strides[i-1] == shape[i] * strides[i]
// for every i >= 1; the innermost stride is not examined and rank 0 passes.
inline bool ref_contiguous(infiniopTensorDescriptor_t t) {
    for (uint64_t i = 1; i < t->ndim; ++i) {
        if (t->strides[i - 1] != static_cast<int64_t>(t->shape[i]) * t->strides[i]) return false;
    }
    return true;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline uint64_t ceil_div(uint64_t a, uint64_t b) { return (a + b - 1) / b; }

// The largest 1-D grid of `lanes`-wide workgroups HIP accepts: a launch may
// not span 2^32 work-items or more along one axis.  Kernels launched with a
// capped grid stride over the rest of their range.
inline uint64_t max_grid_1d(unsigned lanes) { return 0xFFFFFFFFull / lanes; }

// Outputs of at least this many bytes are written through L2 (cache policy
// "sc1 nt") by the kernels that write one byte per byte read; smaller ones
// are left for L2 to absorb.  Measured on MI355X (32 MiB of L2 in all): a
// 16 MiB output is 7 % faster absorbed, a 32 MiB one is even, 128 MiB and
// more are 1-3 % faster written through.
constexpr uint64_t kWriteThroughBytes = 64ull << 20;

}// namespace amd

#endif
