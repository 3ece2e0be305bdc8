// gfx950 kernels for CausalSoftmax and their launch.
//
// Arithmetic contract (reference
// src/ops/causal_softmax/cpu/causal_softmax_cpu.cc:52-82): row i of each
// [seq, total] matrix keeps columns j <= total - seq + i; over those
//     m = max x[j],   s = sum expf(x[j] - m),   y[j] = narrow( expf(x[j] - m) / s )
// in fp32, and every other column becomes an exact zero.  The reference adds
// left to right; here the sum is a tree over lanes and waves, which (with the
// device expf's last bit) moves a small fraction of outputs by one unit in
// the last place.  fp16 narrows by the reference's truncation, bf16
// (extension) rounds to nearest even.
//
// A row is read once (only its kept part), held in registers as fp32 across
// the two reductions, and written once; masked vectors are written as zeros
// without being read.
#include "../../../devices/amd/kernel_amd.h"
#include "causal_softmax_amd.h"

namespace {

using namespace amd;

// One workgroup of BS lanes per row at a time; lane l owns vectors l, l+BS, ...
// (NV of them, 8 elements each), so total <= 8*BS*NV.  Workgroups stride over
// the batch*seq rows; neighbouring rows have nearly the same kept length, so
// the stride balances the causal triangle.
template<typename T, int BS, int NV>
__global__ __launch_bounds__(BS) void causal_softmax_rows(uint16_t *y, uint64_t rows, uint64_t seq, uint32_t total,
                                                          int64_t stride_b, int64_t stride_i) {
    constexpr int WAVES = BS / kWave;
    __shared__ float red[4 * WAVES];// two slot sets for the maxima, two for the sums
    const uint32_t nvec = total / 8;
    const float neg_inf = -__builtin_inff();
    int phase = 0;
    for (uint64_t r = blockIdx.x; r < rows; r += gridDim.x, phase ^= 1) {
        const uint64_t b = r / seq, i = r - b * seq;
        uint16_t *row = y + static_cast<int64_t>(b) * stride_b + static_cast<int64_t>(i) * stride_i;
        const uint32_t keep = static_cast<uint32_t>(total - seq + i) + 1;// columns kept, 1..total
        const uint32_t keep_vecs = (keep + 7) / 8;

        float f[NV][8];
        float mx = neg_inf;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = k * BS + threadIdx.x;
            if (v < keep_vecs) {
                widen8<T>(ld16_stream(row + static_cast<uint64_t>(v) * 8), f[k]);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    if (v * 8 + e >= keep) f[k][e] = neg_inf;
                    mx = fmaxf(mx, f[k][e]);
                }
            }
        }
        mx = block_max<WAVES>(mx, red, phase);

        float part = 0.0f;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = k * BS + threadIdx.x;
            if (v < keep_vecs) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    f[k][e] = v * 8 + e < keep ? expf(f[k][e] - mx) : 0.0f;
                    part += f[k][e];
                }
            }
        }
        const float sum = block_sum<WAVES>(part, red + 2 * WAVES, phase);

#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = k * BS + threadIdx.x;
            if (v < keep_vecs) {
                float o[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = f[k][e] / sum;
                st16_stream(row + static_cast<uint64_t>(v) * 8, narrow8<T>(o));
            } else if (v < nvec) {
                st16_stream(row + static_cast<uint64_t>(v) * 8, u32x4{0, 0, 0, 0});
            }
        }
    }
}

// Any row length, any alignment: three passes over the row with element
// accesses; the later passes find the row in cache.
template<typename T>
__global__ __launch_bounds__(256) void causal_softmax_generic(uint16_t *y, uint64_t rows, uint64_t seq, uint64_t total,
                                                              int64_t stride_b, int64_t stride_i) {
    constexpr int BS = 256, WAVES = BS / kWave;
    __shared__ float red[4 * WAVES];
    int phase = 0;
    for (uint64_t r = blockIdx.x; r < rows; r += gridDim.x, phase ^= 1) {
        const uint64_t b = r / seq, i = r - b * seq;
        uint16_t *row = y + static_cast<int64_t>(b) * stride_b + static_cast<int64_t>(i) * stride_i;
        const uint64_t keep = total - seq + i + 1;
        float mx = -__builtin_inff();
        for (uint64_t j = threadIdx.x; j < keep; j += BS) mx = fmaxf(mx, T::one(row[j]));
        mx = block_max<WAVES>(mx, red, phase);
        float part = 0.0f;
        for (uint64_t j = threadIdx.x; j < keep; j += BS) part += expf(T::one(row[j]) - mx);
        const float sum = block_sum<WAVES>(part, red + 2 * WAVES, phase);
        for (uint64_t j = threadIdx.x; j < total; j += BS) {
            row[j] = j < keep ? T::narrow1(expf(T::one(row[j]) - mx) / sum) : static_cast<uint16_t>(0);
        }
    }
}

template<typename T>
void launch_causal_softmax(const CausalSoftmaxAmdDescriptor &d, void *data, hipStream_t stream) {
    auto *py = static_cast<uint16_t *>(data);
    const uint64_t rows = d.batch * d.seq;
    const uint64_t nvec = d.total / 8;
    const uint64_t cap = static_cast<uint64_t>(d.cu_count) * 8;
    const unsigned grid = static_cast<unsigned>(rows < cap ? rows : cap);

    const bool vec_ok = d.total % 8 == 0 && nvec <= 4096 && d.stride_i % 8 == 0 && d.stride_b % 8 == 0 && aligned16(data);
    if (!vec_ok) {
        causal_softmax_generic<T><<<grid, 256, 0, stream>>>(py, rows, d.seq, d.total, d.stride_b, d.stride_i);
        return;
    }
#define CS_LAUNCH(BS, NV) \
    causal_softmax_rows<T, BS, NV><<<grid, BS, 0, stream>>>(py, rows, d.seq, static_cast<uint32_t>(d.total), d.stride_b, d.stride_i)
    if (nvec <= 64) CS_LAUNCH(64, 1);
    else if (nvec <= 128) CS_LAUNCH(128, 1);
    else if (nvec <= 256) CS_LAUNCH(256, 1);
    else if (nvec <= 512) CS_LAUNCH(256, 2);
    else if (nvec <= 1024) CS_LAUNCH(256, 4);
    else if (nvec <= 2048) CS_LAUNCH(512, 4);
    else CS_LAUNCH(1024, 4);
#undef CS_LAUNCH
}

}// namespace

// Stage 4 of CausalSoftmax.  The workspace is unused (its size is 0).
infiniopStatus_t amdCausalSoftmax(CausalSoftmaxAmdDescriptor_t desc, void *, uint64_t, void *data, void *stream) {
    if (desc->batch == 0 || desc->seq == 0 || desc->total == 0) {
        return STATUS_SUCCESS;
    }
    if (data == nullptr) {
        return STATUS_BAD_PARAM;
    }
    AMD_CHECK_HIP(hipSetDevice(desc->device_id), STATUS_BAD_DEVICE);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (desc->elem) {
        case amd::Elem::F16:
            launch_causal_softmax<amd::F16Ref>(*desc, data, s);
            break;
        case amd::Elem::BF16:
            launch_causal_softmax<amd::BF16Rne>(*desc, data, s);
            break;
        default:
            return STATUS_BAD_TENSOR_DTYPE;
    }
    AMD_CHECK_HIP(hipGetLastError(), STATUS_EXECUTION_FAILED);
    return STATUS_SUCCESS;
}
