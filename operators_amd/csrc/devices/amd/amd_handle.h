// Handle of the amd-gpu device: what infiniopCreateHandle(…, DevAmdGpu, id)
// returns.  Plays the part that src/devices/cuda/cuda_handle.h:12-21 plays for
// the NVIDIA device in the reference, without BLAS/DNN pools: the four
// operators of this back end launch their own kernels only.
#ifndef INFINIOP_AMD_HANDLE_H
#define INFINIOP_AMD_HANDLE_H

#include "operators.h"

// Plain C layout; `device` must stay first (the dispatchers read only it).
struct AmdContext {
    Device device;       // always DevAmdGpu
    int device_id;       // HIP ordinal the handle is bound to
    int cu_count;        // compute units (256 on MI355X)
    int lds_per_block;   // bytes of LDS one workgroup may use
    int max_grid_x;      // largest gridDim.x
    int wave_size;       // 64 on CDNA
};
typedef struct AmdContext *AmdHandle_t;

infiniopStatus_t createAmdHandle(AmdHandle_t *handle_ptr, int device_id);
infiniopStatus_t deleteAmdHandle(AmdHandle_t handle);

#endif
