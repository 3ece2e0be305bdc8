// gfx950 kernels for SwiGLU and their launch.
//
// Arithmetic contract (reference src/ops/swiglu/cpu/swiglu_cpu.cc:49-72):
//     c = narrow( a * ( b / (1 + expf(-b)) ) )       all in fp32,
// b gated, a linear; fp16 narrows with the reference's truncating conversion,
// bf16 (extension) rounds to nearest even.  The fp32 value is computed to
// within about one unit in its last place of the CPU's (see swiglu1_lean).
//
// Three streams (two in, one out) and about 20 VALU slots per element:
// bandwidth bound, but only just - the arithmetic is kept lean on purpose.  Rows are addressed through one row stride per tensor, so the same
// kernel serves separate a/b tensors and the gate/up halves of one fused
// buffer (reference caller: src/ops/mlp/operator.cc:50-57,111-115).
#include "../../../devices/amd/kernel_amd.h"
#include "swiglu_amd.h"

namespace {

using namespace amd;

constexpr int kBlock = 256;// lanes per workgroup of the element-wise fallback kernel

// The reference's formula with the library routines: expf and an IEEE
// division.  About 35 VALU slots per element - more than the memory system
// leaves time for at 6 bytes of traffic per element (a kernel built on this
// alone ran at 64 % of peak, compute bound) - so it serves only the rare
// elements the lean form below does not cover, and the element-wise fallback.
__device__ __forceinline__ float swiglu1_any(float up, float gate) {
    return up * (gate / (1.0f + expf(-gate)));
}

// The same value for |gate| <= 87 with two hardware transcendentals (exp2,
// rcp) and three correction steps, about 20 VALU slots per element.
//  - gate has at most 11 significant bits (it was an fp16 or bf16 value) and
//    kL2eHi has 11, so t = gate * -kL2eHi is exact; the rest of log2(e) enters
//    as the first-order factor (1 + gate * c) on the result of exp2.  The
//    neglected second-order term is (gate * 1.22e-4)^2 / 2 relative to e:
//    below one fp32 ulp for |gate| < 3, 5e-7 at |gate| = 8, and where it grows
//    further (gate < -10) the result is already in fp16's subnormal range or
//    below, where one unit in the last place is far coarser than that.
//  - |gate| <= 87 keeps e = exp(-gate) finite and normal, so the quotient's
//    correction step never meets inf * 0.
//  - q = gate * rcp(d) is refined once with the exact residual gate - d*q.
// Against the CPU's expf-and-divide the narrowed fp16 result differs by one
// unit in the last place on 2 to 9 elements in 10^5 (N(0,1) and N(0,16)
// inputs), never by more; the library-routine form differs on 4 to 6 in 10^6.
constexpr float kLeanGateLimit = 87.0f;
__device__ __forceinline__ float swiglu1_lean(float up, float gate) {
    constexpr float kL2eHi = 1.44287109375f;   // log2(e) rounded to 11 bits
    constexpr float kL2eLoLn2 = -1.2203054e-4f;// (log2(e) - kL2eHi) * ln 2
    float e = __builtin_amdgcn_exp2f(gate * -kL2eHi);
    e = __builtin_fmaf(e, gate * -kL2eLoLn2, e);
    const float d = 1.0f + e;
    const float r = __builtin_amdgcn_rcpf(d);
    float q = gate * r;
    q = __builtin_fmaf(__builtin_fmaf(-d, q, gate), r, q);
    return up * q;
}

// Eight elements.  Gates beyond the lean form's range (|gate| > 87, infinities,
// NaNs - none of which occur in activations of ordinary scale) send the whole
// wavefront through the library form; the test is wave-uniform, so the lean
// path carries no divergent branches.
template<typename T>
__device__ __forceinline__ u32x4 swiglu8(u32x4 va, u32x4 vb) {
    float up[8], gate[8];
    widen8<T>(va, up);
    widen8<T>(vb, gate);
    bool out_of_range = false;
#pragma unroll
    for (int i = 0; i < 8; ++i) out_of_range |= !(fabsf(gate[i]) <= kLeanGateLimit);
    if (__builtin_amdgcn_ballot_w64(out_of_range) == 0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) up[i] = swiglu1_lean(up[i], gate[i]);
    } else {
        // An empty volatile statement: it cannot be executed speculatively, so
        // the compiler keeps this side a real (wave-uniform) branch instead of
        // computing both forms for every element and selecting afterwards.
        asm volatile("" ::: "memory");
#pragma unroll
        for (int i = 0; i < 8; ++i) up[i] = swiglu1_any(up[i], gate[i]);
    }
    return narrow8<T>(up);
}

// Position of vector `v` of the [rows, di/8] index space in a tensor whose row
// stride is `stride` elements.  ROWWISE = false means all three tensors are
// dense and the flat index is the address.
template<typename Idx, bool ROWWISE>
struct Where {
    Idx vecs_per_row;
    FastDiv by_row;// division by vecs_per_row for 32-bit positions below kFastDivLimit
    __device__ __forceinline__ void split(uint64_t v, Idx &row, Idx &col) const {
        if constexpr (ROWWISE) {
            if constexpr (sizeof(Idx) == 4) row = fast_quotient(static_cast<uint32_t>(v), by_row);
            else row = static_cast<Idx>(v) / vecs_per_row;
            col = static_cast<Idx>(v) - row * vecs_per_row;
        } else {
            row = 0;
            col = static_cast<Idx>(v);
        }
    }
};

// One wavefront per workgroup, one vector per lane: the dispatcher hands out
// consecutive KiBs of the output in order and every wavefront gives its slot
// back the moment it is done.  Measured on MI355X: [8192, 28672] bf16 from a
// fused buffer 204.5 us with 64 lanes per workgroup, 207.9 with 128, 209.0 with
// 256; [4096, 11008] fp16 from a fused buffer (rows of 5.4 x 256 vectors) 42.7
// against 46.6 us.  (The loop only runs more than once beyond 2^31 workgroups.)
template<typename T, typename Idx, bool ROWWISE>
__global__ __launch_bounds__(kWave) void swiglu_vec(uint16_t *c, const uint16_t *a, const uint16_t *b,
                                                     uint64_t nvec, Idx vecs_per_row,
                                                     int64_t stride_c, int64_t stride_a, int64_t stride_b, FastDiv by_row) {
    AMD_ARGS_NOW(c, a, b, nvec, vecs_per_row, stride_c, stride_a, stride_b, arg_pair(by_row), gridDim.x);
    const Where<Idx, ROWWISE> where{vecs_per_row, by_row};
    const uint64_t step = static_cast<uint64_t>(gridDim.x) * kWave;
    for (uint64_t v = static_cast<uint64_t>(blockIdx.x) * kWave + threadIdx.x; v < nvec; v += step) {
        Idx row, col;
        where.split(v, row, col);
        const int64_t e = static_cast<int64_t>(col) * 8;
        const u32x4 va = ld16_stream(a + static_cast<int64_t>(row) * stride_a + e);
        const u32x4 vb = ld16_stream(b + static_cast<int64_t>(row) * stride_b + e);
        st16_stream(c + static_cast<int64_t>(row) * stride_c + e, swiglu8<T>(va, vb));
    }
}

// Row-strided tensors whose rows hold at least 16 wavefronts of vectors:
// blockIdx.y walks the rows and blockIdx.x the row's vectors, so no lane
// divides anything and no workgroup straddles two rows.
template<typename T, int LANES>
__global__ __launch_bounds__(LANES) void swiglu_rows(uint16_t *c, const uint16_t *a, const uint16_t *b,
                                                      uint64_t rows, uint32_t vecs_per_row,
                                                      int64_t stride_c, int64_t stride_a, int64_t stride_b) {
    AMD_ARGS_NOW(c, a, b, rows, vecs_per_row, stride_c, stride_a, stride_b);
    const uint32_t col = blockIdx.x * LANES + threadIdx.x;
    if (col >= vecs_per_row) return;
    const int64_t e = static_cast<int64_t>(col) * 8;
    for (uint64_t row = blockIdx.y; row < rows; row += gridDim.y) {
        const u32x4 va = ld16_stream(a + static_cast<int64_t>(row) * stride_a + e);
        const u32x4 vb = ld16_stream(b + static_cast<int64_t>(row) * stride_b + e);
        st16_stream(c + static_cast<int64_t>(row) * stride_c + e, swiglu8<T>(va, vb));
    }
}

// Any width, any alignment.  A lane takes 8 consecutive elements of one row: a
// whole group moves as 16 bytes at whatever 2-byte boundary it lies on (which
// gfx950 serves at a fraction of the aligned rate), a row's last, partial
// group element by element.  [4096, 11007] fp16 halves of a fused buffer:
// 113 us with element accesses only.
template<typename T>
__global__ __launch_bounds__(kBlock) void swiglu_scalar(uint16_t *c, const uint16_t *a, const uint16_t *b,
                                                        uint64_t rows, uint64_t di,
                                                        int64_t stride_c, int64_t stride_a, int64_t stride_b) {
    const uint64_t per_row = (di + 7) / 8, groups = rows * per_row;
    const uint64_t step = static_cast<uint64_t>(gridDim.x) * kBlock;
    for (uint64_t g = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x; g < groups; g += step) {
        const uint64_t row = g / per_row, col = (g - row * per_row) * 8;
        const uint16_t *pa = a + static_cast<int64_t>(row) * stride_a + col;
        const uint16_t *pb = b + static_cast<int64_t>(row) * stride_b + col;
        uint16_t *pc = c + static_cast<int64_t>(row) * stride_c + col;
        // the ballot inside swiglu8 is over the lanes that are here: a wavefront's lanes with partial groups take the other side
        if (col + 8 <= di) {
            st16_any(pc, swiglu8<T>(ld16_any(pa), ld16_any(pb)));
        } else {
            for (uint64_t e = 0; col + e < di; ++e) pc[e] = T::narrow1(swiglu1_any(T::one(pa[e]), T::one(pb[e])));
        }
    }
}

template<typename T>
void launch_swiglu(const SwiGLUAmdDescriptor &d, void *c, const void *a, const void *b, hipStream_t stream) {
    auto *pc = static_cast<uint16_t *>(c);
    auto *pa = static_cast<const uint16_t *>(a);
    auto *pb = static_cast<const uint16_t *>(b);
    const uint64_t n = d.rows * d.di;
    const int64_t di = static_cast<int64_t>(d.di);

    const bool vec_ok = d.di % 8 == 0 && d.stride_a % 8 == 0 && d.stride_b % 8 == 0 && d.stride_c % 8 == 0 &&
                        aligned16(c) && aligned16(a) && aligned16(b);
    // Dense tensors are one run of rows * di elements whatever the width: vectors as far as they go, the up to 7
    // elements behind them one by one ([4096, 11007] fp16: 42 us; 112 us element by element).
    const bool one_run = d.rows == 1 || (d.stride_a == di && d.stride_b == di && d.stride_c == di);
    if (!vec_ok && one_run && n >= 8 && aligned16(c) && aligned16(a) && aligned16(b)) {
        const uint64_t whole = n / 8, want = ceil_div(whole, kWave), max_grid = max_grid_1d(kWave);
        swiglu_vec<T, uint64_t, false><<<static_cast<unsigned>(want < max_grid ? want : max_grid), kWave, 0, stream>>>(
            pc, pa, pb, whole, whole, 0, 0, 0, FastDiv{});
        const uint64_t done = whole * 8;
        if (done < n) swiglu_scalar<T><<<1, kBlock, 0, stream>>>(pc + done, pa + done, pb + done, 1, n - done, 0, 0, 0);
        return;
    }
    if (!vec_ok) {
        const uint64_t want = ceil_div(d.rows * ceil_div(d.di, 8), kBlock), cap = max_grid_1d(kBlock);
        swiglu_scalar<T><<<static_cast<unsigned>(want < cap ? want : cap), kBlock, 0, stream>>>(
            pc, pa, pb, d.rows, d.di, d.stride_c, d.stride_a, d.stride_b);
        return;
    }

    const uint64_t nvec = n / 8;
    const uint64_t vpr = d.di / 8;
    const uint64_t want = ceil_div(nvec, kWave);
    const uint64_t max_grid = max_grid_1d(kWave);
    const unsigned grid = static_cast<unsigned>(want < max_grid ? want : max_grid);
    const bool dense = one_run;// one row, or every row stride equal to the width
    const bool small = nvec < (1ull << 31);
    // Row-strided tensors (the halves of a fused gate/up buffer).  Rows of at least 1024 vectors: a 2-D grid of
    // single-wavefront workgroups, no lane divides anything.  Shorter rows: the same tiles over the flat (row,
    // vector) space, split by a multiplication (see FastDiv) - a 2-D grid of single wavefronts needs at least 16
    // of them per row, and the 128- or 256-lane row workgroups it would take instead measure the same or worse
    // (bf16 from a fused buffer, us: [131072, 512] 60.3 against 69.4, [16384, 4096] 60.9 against 62.5,
    // [65536, 1024] 60.2 against 61.6, [23831, 2816] 60.7 against 60.2; at [8192, 28672] the two forms are
    // level, 204.8 and 204.4, where the split by a run-time division cost the flat form 4 %).
    if (!dense && vpr >= 16 * kWave && vpr < (1ull << 31)) {
        const unsigned gy = static_cast<unsigned>(d.rows < 65535 ? d.rows : 65535);
        swiglu_rows<T, kWave><<<dim3(static_cast<unsigned>(ceil_div(vpr, kWave)), gy), kWave, 0, stream>>>(
            pc, pa, pb, d.rows, static_cast<uint32_t>(vpr), d.stride_c, d.stride_a, d.stride_b);
        return;
    }
    if (dense) {
        swiglu_vec<T, uint64_t, false><<<grid, kWave, 0, stream>>>(pc, pa, pb, nvec, vpr, d.stride_c, d.stride_a, d.stride_b, FastDiv{});
    } else if (small) {
        swiglu_vec<T, uint32_t, true><<<grid, kWave, 0, stream>>>(pc, pa, pb, nvec, static_cast<uint32_t>(vpr),
                                                                   d.stride_c, d.stride_a, d.stride_b, fast_div(static_cast<uint32_t>(vpr)));
    } else {
        swiglu_vec<T, uint64_t, true><<<grid, kWave, 0, stream>>>(pc, pa, pb, nvec, vpr, d.stride_c, d.stride_a, d.stride_b, FastDiv{});
    }
}

}// namespace

// Stage 4 of SwiGLU: enqueue on the caller's stream and return.
infiniopStatus_t amdSwiGLU(SwiGLUAmdDescriptor_t desc, void *c, void const *a, void const *b, void *stream) {
    if (desc->rows == 0 || desc->di == 0) {
        return STATUS_SUCCESS;
    }
    if (c == nullptr || a == nullptr || b == nullptr) {
        return STATUS_BAD_PARAM;
    }
    AMD_CHECK_HIP(hipSetDevice(desc->device_id), STATUS_BAD_DEVICE);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (desc->elem) {
        case amd::Elem::F16:
            launch_swiglu<amd::F16Ref>(*desc, c, a, b, s);
            break;
        case amd::Elem::BF16:
            launch_swiglu<amd::BF16Rne>(*desc, c, a, b, s);
            break;
        default:
            return STATUS_BAD_TENSOR_DTYPE;
    }
    AMD_CHECK_HIP(hipGetLastError(), STATUS_EXECUTION_FAILED);
    return STATUS_SUCCESS;
}
