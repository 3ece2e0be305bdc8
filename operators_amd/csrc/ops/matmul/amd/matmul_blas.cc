// Stage 4 of Matmul: one strided-batched GEMM in rocBLAS, fp32 accumulation.
//
// The BLAS library is a plain dependency of this one operator, so it is bound
// at first use (dlopen by its SONAME) rather than at link time: the memory-
// bound operators never pay for loading it, and inside a process that has
// already loaded a copy (PyTorch ships one with the same SONAME) that copy is
// the one that answers.  Handles are pooled per device, one per concurrent
// caller, as the reference pools its cuBLAS handles
// (src/devices/cuda/cuda_handle.h, use_cublas).
#include "matmul_amd.h"
#include <dlfcn.h>
#include <mutex>
#include <rocblas/rocblas.h>
#include <vector>

namespace {

struct Blas {
    decltype(&rocblas_create_handle) create_handle = nullptr;
    decltype(&rocblas_destroy_handle) destroy_handle = nullptr;
    decltype(&rocblas_set_stream) set_stream = nullptr;
    decltype(&rocblas_set_pointer_mode) set_pointer_mode = nullptr;
    decltype(&rocblas_gemm_strided_batched_ex) gemm_strided_batched_ex = nullptr;
    bool ok = false;
};

const Blas &blas() {
    static const Blas b = [] {
        Blas r;
        void *lib = dlopen("librocblas.so.5", RTLD_NOW | RTLD_LOCAL);
        if (lib == nullptr) lib = dlopen("librocblas.so", RTLD_NOW | RTLD_LOCAL);
        if (lib == nullptr) {
            std::fprintf(stderr, "infiniop[amd-gpu]: cannot load rocBLAS for Matmul: %s\n", dlerror());
            return r;
        }
        r.create_handle = reinterpret_cast<decltype(r.create_handle)>(dlsym(lib, "rocblas_create_handle"));
        r.destroy_handle = reinterpret_cast<decltype(r.destroy_handle)>(dlsym(lib, "rocblas_destroy_handle"));
        r.set_stream = reinterpret_cast<decltype(r.set_stream)>(dlsym(lib, "rocblas_set_stream"));
        r.set_pointer_mode = reinterpret_cast<decltype(r.set_pointer_mode)>(dlsym(lib, "rocblas_set_pointer_mode"));
        r.gemm_strided_batched_ex =
            reinterpret_cast<decltype(r.gemm_strided_batched_ex)>(dlsym(lib, "rocblas_gemm_strided_batched_ex"));
        r.ok = r.create_handle && r.destroy_handle && r.set_stream && r.set_pointer_mode && r.gemm_strided_batched_ex;
        if (!r.ok) std::fprintf(stderr, "infiniop[amd-gpu]: rocBLAS lacks an entry point Matmul needs\n");
        return r;
    }();
    return b;
}

// Idle handles per device.  A caller takes one (or makes one), uses it on its
// own stream and gives it back; handles live until the process ends.
struct HandlePool {
    std::mutex lock;
    std::vector<std::vector<rocblas_handle>> idle;

    rocblas_handle take(int device) {
        {
            std::lock_guard<std::mutex> g(lock);
            if (static_cast<size_t>(device) < idle.size() && !idle[device].empty()) {
                rocblas_handle h = idle[device].back();
                idle[device].pop_back();
                return h;
            }
        }
        rocblas_handle h = nullptr;
        if (blas().create_handle(&h) != rocblas_status_success) return nullptr;
        blas().set_pointer_mode(h, rocblas_pointer_mode_host);
        return h;
    }
    void give(int device, rocblas_handle h) {
        std::lock_guard<std::mutex> g(lock);
        if (static_cast<size_t>(device) >= idle.size()) idle.resize(device + 1);
        idle[device].push_back(h);
    }
};

HandlePool &pool() {
    static HandlePool p;
    return p;
}

}// namespace

infiniopStatus_t amdMatmul(MatmulAmdDescriptor_t desc, void *workspace, uint64_t workspace_size, void *c, void const *a, void const *b, void *stream) {
    if (c == nullptr || a == nullptr || b == nullptr) {
        return STATUS_BAD_PARAM;
    }
    if (desc->m == 0 || desc->n == 0 || desc->batch == 0) {
        return STATUS_SUCCESS;
    }
    AMD_CHECK_HIP(hipSetDevice(desc->device_id), STATUS_BAD_DEVICE);
    if (desc->operands_swapped) {
        void const *t = a;
        a = b;
        b = t;
    }
    // the two products of an attention while decoding are not shapes for a library GEMM
    if (amd_matmul_skinny(*desc, c, a, b, static_cast<hipStream_t>(stream)) ||
        amd_matmul_long_k(*desc, workspace, workspace_size, c, a, b, static_cast<hipStream_t>(stream))) {
        AMD_CHECK_HIP(hipGetLastError(), STATUS_EXECUTION_FAILED);
        return STATUS_SUCCESS;
    }
    if (!blas().ok) {
        return STATUS_EXECUTION_FAILED;
    }
    rocblas_datatype type;
    switch (desc->elem) {
        case amd::Elem::F16: type = rocblas_datatype_f16_r; break;
        case amd::Elem::BF16: type = rocblas_datatype_bf16_r; break;
        case amd::Elem::F32: type = rocblas_datatype_f32_r; break;
        default: return STATUS_BAD_TENSOR_DTYPE;
    }
    const rocblas_operation op_a = desc->a.column_major() ? rocblas_operation_none : rocblas_operation_transpose;
    const rocblas_operation op_b = desc->b.column_major() ? rocblas_operation_none : rocblas_operation_transpose;
    // a matrix with a single row or column may carry any leading dimension; BLAS wants at least the extent
    auto ld_of = [](const amd::GemmMatrix &mx, rocblas_operation op) {
        const int64_t need = op == rocblas_operation_none ? mx.rows : mx.cols;
        const int64_t ld = mx.ld();
        return static_cast<rocblas_int>(ld < need ? need : (ld < 1 ? 1 : ld));
    };
    const float alpha = desc->alpha, beta = desc->beta;

    rocblas_handle h = pool().take(desc->device_id);
    if (h == nullptr) {
        return STATUS_EXECUTION_FAILED;
    }
    infiniopStatus_t result = STATUS_SUCCESS;
    if (blas().set_stream(h, static_cast<hipStream_t>(stream)) != rocblas_status_success) {
        result = STATUS_EXECUTION_FAILED;
    } else {
        const rocblas_status st = blas().gemm_strided_batched_ex(
            h, op_a, op_b, static_cast<rocblas_int>(desc->m), static_cast<rocblas_int>(desc->n), static_cast<rocblas_int>(desc->k),
            &alpha, a, type, ld_of(desc->a, op_a), desc->a.stride, b, type, ld_of(desc->b, op_b), desc->b.stride, &beta,
            c, type, ld_of(desc->c, rocblas_operation_none), desc->c.stride,
            c, type, ld_of(desc->c, rocblas_operation_none), desc->c.stride,
            static_cast<rocblas_int>(desc->batch), rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
        if (st != rocblas_status_success) {
            std::fprintf(stderr, "infiniop[amd-gpu]: rocblas_gemm_strided_batched_ex -> status %d\n", static_cast<int>(st));
            result = STATUS_EXECUTION_FAILED;
        }
    }
    pool().give(desc->device_id, h);
    return result;
}
