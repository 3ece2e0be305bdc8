// Device code of RMSNorm on gfx950, shared by the plain operator and the fused
// residual form (Add + RMSNorm in one pass).  Include from .hip files only.
//
// Arithmetic contract (reference src/ops/rms_norm/cpu/rms_norm_cpu.cc:46-86):
//     ss   = sum_j x[j]^2                      fp32
//     k    = (ss / d + eps) ^ -1/2             fp32 mean, double power
//     y[j] = narrow( (k * x[j]) * w[j] )
// The reference adds the squares left to right and carries the two products
// in double before narrowing; here the sum is a tree over lanes and waves and
// the products are fp32.  Both differences are below one fp32 ulp of y and
// show up, after narrowing to 16 bits, as a last-bit difference on roughly one
// element in 10^4.  fp16 narrows by the reference's truncation, bf16
// (extension) rounds to nearest even.
//
// Data movement is the whole cost: x is read once and kept in registers
// between the reduction and the scaling pass, y is written once, and the
// weight row - re-used by every row - is staged once per workgroup in LDS as
// fp32 when a workgroup serves more than one row.
#ifndef INFINIOP_AMD_RMS_NORM_KERNELS_H
#define INFINIOP_AMD_RMS_NORM_KERNELS_H

#include "../../../devices/amd/common_amd.h"
#include "../../../devices/amd/kernel_amd.h"
#include <algorithm>

// Internal linkage: each including translation unit owns its copies, and none
// of them appears in the library's dynamic symbol table.
namespace rms_norm_kernels {
namespace {

using namespace amd;

// ---- weight row access ----------------------------------------------------------
struct WF32 {
    typedef float scalar;
    struct raw {
        f32x4 a, b;
    };
    // eight weights through a buffer descriptor of the weight row: a per-lane byte offset plus a wavefront-uniform one
    __device__ static __forceinline__ raw fetch(__amdgpu_buffer_rsrc_t row, uint32_t lane, uint32_t ahead) {
        const u32x4 a = __builtin_amdgcn_raw_buffer_load_b128(row, static_cast<int>(lane), static_cast<int>(ahead), 0);
        const u32x4 b = __builtin_amdgcn_raw_buffer_load_b128(row, static_cast<int>(lane + 16), static_cast<int>(ahead), 0);
        return raw{__builtin_bit_cast(f32x4, a), __builtin_bit_cast(f32x4, b)};
    }
    __device__ static __forceinline__ void spread(const raw &r, float (&g)[8]) {
        g[0] = r.a.x, g[1] = r.a.y, g[2] = r.a.z, g[3] = r.a.w;
        g[4] = r.b.x, g[5] = r.b.y, g[6] = r.b.z, g[7] = r.b.w;
    }
    __device__ static __forceinline__ void load8(const void *w, uint32_t vec, float (&g)[8]) {
        const float *p = static_cast<const float *>(w) + static_cast<uint64_t>(vec) * 8;
        const f32x4 a = ld16f(p), b = ld16f(p + 4);
        g[0] = a.x, g[1] = a.y, g[2] = a.z, g[3] = a.w;
        g[4] = b.x, g[5] = b.y, g[6] = b.z, g[7] = b.w;
    }
    __device__ static __forceinline__ float one(const void *w, uint64_t j) { return static_cast<const float *>(w)[j]; }
};
template<typename T>
struct W16 {
    typedef uint16_t scalar;
    typedef u32x4 raw;
    __device__ static __forceinline__ raw fetch(__amdgpu_buffer_rsrc_t row, uint32_t lane, uint32_t ahead) {
        return __builtin_amdgcn_raw_buffer_load_b128(row, static_cast<int>(lane), static_cast<int>(ahead), 0);
    }
    __device__ static __forceinline__ void spread(const raw &r, float (&g)[8]) { widen8<T>(r, g); }
    __device__ static __forceinline__ void load8(const void *w, uint32_t vec, float (&g)[8]) {
        widen8<T>(ld16(static_cast<const uint16_t *>(w) + static_cast<uint64_t>(vec) * 8), g);
    }
    __device__ static __forceinline__ float one(const void *w, uint64_t j) {
        return T::one(static_cast<const uint16_t *>(w)[j]);
    }
};

// The weight row's element type is a run-time property of the call (kind), not
// a template parameter: it only matters where the weights are fetched, which
// is once per workgroup when they are staged in LDS.
enum WeightKind { kWKindF32 = 0, kWKindF16 = 1, kWKindBF16 = 2 };

__device__ __forceinline__ void load_w8(const void *w, int kind, uint32_t vec, float (&g)[8]) {
    if (kind == kWKindF32) WF32::load8(w, vec, g);
    else if (kind == kWKindF16) W16<F16Ref>::load8(w, vec, g);
    else W16<BF16Rne>::load8(w, vec, g);
}
__device__ __forceinline__ float load_w1(const void *w, int kind, uint64_t j) {
    if (kind == kWKindF32) return WF32::one(w, j);
    if (kind == kWKindF16) return W16<F16Ref>::one(w, j);
    return W16<BF16Rne>::one(w, j);
}

// ---- the sum of squares of a row, in one order whatever the launch shape ------
// Every vector of 8 elements gives one partial (pairwise inside the vector);
// 64 consecutive vectors are added by the wavefront's cross-lane tree
// (amd::wave_sum); those chunk sums are added in ascending order.  A row's
// sum therefore does not depend on how many lanes serve it or how many vectors
// a lane holds, and RMSNorm gives the same bits through every kernel below -
// which is what lets the fused Add + RMSNorm reproduce the two separate calls
// bit for bit while choosing its own launch shape.  Lane l of wavefront w
// holds vector k * 64 * WAVES + 64 * w + l in s[k]; absent vectors give 0.
// `slots` is LDS with room for NV * WAVES floats that nobody else uses until
// the next barrier.
template<int WAVES, int NV>
__device__ __forceinline__ float row_sum(const float (&s)[NV], float *slots) {
    float c[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) c[k] = wave_sum(s[k]);
    float total = 0.0f;
    if constexpr (WAVES == 1) {
#pragma unroll
        for (int k = 0; k < NV; ++k) total += c[k];
    } else {
        const int wave = threadIdx.x / kWave;
        if ((threadIdx.x & (kWave - 1)) == 0) {
#pragma unroll
            for (int k = 0; k < NV; ++k) slots[k * WAVES + wave] = c[k];
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < NV * WAVES; ++j) total += slots[j];
    }
    return total;
}

// The same sum for a lane count known only at launch (waves >= 2).  (Fetching
// the chunk sums with one LDS read, one per lane, and adding them out of that
// register lane by lane measured 1-8 % slower than this loop of LDS reads.)
template<int NV>
__device__ __forceinline__ float row_sum_any(const float (&s)[NV], float *slots, uint32_t waves) {
    const uint32_t wave = threadIdx.x / kWave;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const float c = wave_sum(s[k]);
        if ((threadIdx.x & (kWave - 1)) == 0) slots[k * waves + wave] = c;
    }
    __syncthreads();
    float total = 0.0f;
    for (uint32_t j = 0; j < NV * waves; ++j) total += slots[j];
    return total;
}

// One vector's sum of squares: pairwise, each pair as one product and one
// fused multiply-add (the library is compiled with contraction off for RoPE's
// sake; here fusing costs nothing - the sum's order already differs from the
// reference's left-to-right one - and saves four of fifteen instructions).
__device__ __forceinline__ float squares8(const float (&f)[8]) {
    const float s01 = __builtin_fmaf(f[1], f[1], f[0] * f[0]), s23 = __builtin_fmaf(f[3], f[3], f[2] * f[2]);
    const float s45 = __builtin_fmaf(f[5], f[5], f[4] * f[4]), s67 = __builtin_fmaf(f[7], f[7], f[6] * f[6]);
    return (s01 + s23) + (s45 + s67);
}

__device__ __forceinline__ float inv_rms(float sum_sq, uint64_t d, float eps) {
    const float mean_eps = sum_sq / static_cast<float>(d) + eps;
    return static_cast<float>(1.0 / sqrt(static_cast<double>(mean_eps)));
}

// ---- rows that fit in registers -----------------------------------------------
// One workgroup of BS lanes per row at a time; lane l owns vectors l, l+BS, ...
// (NV of them, 8 elements each), so d <= 8*BS*NV.  Workgroups stride over rows
// and fetch the next row's x before reducing the current one, so a load is
// always in flight while the reduction, the barrier and the stores happen.
//
// Where the weight row lives while a workgroup works through its rows:
//   kWGlobal: re-read from memory for every row (one row per workgroup, or a
//             row too long for LDS)
//   kWLds   : staged once in LDS as fp32
// Measured at [8192, 8192] bf16 with fp32 weights: 45.7 us with the weights in
// LDS, 47.0-50.6 us when every row re-reads them through L2 (one workgroup per
// row, or 8-16 looping workgroups per compute unit); keeping each lane's 8*NV
// weights in registers instead of LDS is no faster than LDS.  Giving every
// wavefront a row of its own (16 vectors per lane, DPP-only reduction, no
// barrier, weights shared in LDS by the 4 wavefronts of a workgroup) takes
// 50.3-53.4 us against 44.6 us for one row per 256 lanes.
//
// LDS layout of the staged weight row: the 8 floats of vector v are split into
// two 16-byte halves stored at lo[v] and hi[v] (hi = lo + nvec).  A wavefront
// reading lo[v..v+63] or hi[v..v+63] then touches 64 consecutive 16-byte words
// - no two lanes on the same bank in the same phase - where the natural
// 32-byte-per-lane layout would be a two-way conflict.
enum WeightHome { kWGlobal = 0, kWLds = 1 };

// EXACT means d == 8*BS*NV: every lane owns NV whole vectors and no access is
// predicated.  Otherwise loads of absent vectors are redirected to vector 0
// (and their value replaced by zero) rather than branched around: with
// straight-line loads the compiler can count how many are still in flight and
// wait for the current row only, not for the prefetched one.
//
// ADD is the fused residual form: x is one of two addends, res carries the
// other (b) and where their sum goes (c).  The sum is rounded to the element
// type exactly as the Add operator rounds it, stored, and that rounded row is
// what gets normalised - the results are those of Add followed by RMSNorm,
// with the sum read from registers instead of from memory.
}// namespace
// (plain data, with external linkage: it crosses translation units)
template<bool ADD>
struct Residual {};
template<>
struct Residual<true> {
    uint16_t *c;
    const uint16_t *b;
    int64_t stride_c, stride_b;
};
namespace {

// Every argument of a kernel below fetched at its top (see AMD_ARGS_NOW); `more` are the kernel's own beside the common ones.
#define RMS_ARGS_NOW(...)                                                                                                                 \
    do {                                                                                                                                  \
        if constexpr (ADD) AMD_ARGS_NOW(y, x, w, w_kind, n, d, stride_y, stride_x, eps, res.c, res.b, res.stride_c, res.stride_b, ##__VA_ARGS__); \
        else AMD_ARGS_NOW(y, x, w, w_kind, n, d, stride_y, stride_x, eps, ##__VA_ARGS__);                                                  \
    } while (0)

template<typename T, int BS, int NV, int WHOME, bool EXACT, bool THROUGH, bool ADD, bool AHEAD = true>
__global__ __launch_bounds__(BS != 0 ? BS : 1024) void rms_norm_rows(uint16_t *y, const uint16_t *x, const void *w, int w_kind,
                                                     uint64_t n, uint32_t d, int64_t stride_y, int64_t stride_x, float eps,
                                                     uint64_t first_mul, uint64_t hop, uint64_t span, Residual<ADD> res) {
    RMS_ARGS_NOW(first_mul, hop, span, blockDim.x);
    // BS = 0: the lane count is the launch's (any multiple of 64 up to 1024)
    constexpr int MAX_WAVES = (BS != 0 ? BS : 1024) / kWave;
    const uint32_t bs = BS != 0 ? BS : blockDim.x;
    [[maybe_unused]] const uint32_t waves = bs / kWave;
    __shared__ float red[2 * NV * MAX_WAVES];// two sets of chunk sums, used in turn: one barrier per row is enough
    extern __shared__ __attribute__((aligned(16))) unsigned char dyn_lds[];
    f32x4 *w_lo = reinterpret_cast<f32x4 *>(dyn_lds);
    const uint32_t nvec = d / 8;
    f32x4 *w_hi = w_lo + nvec;

    constexpr int NB = ADD ? NV : 1;// registers for the second addend only in the fused form
    auto load_row = [&](uint64_t row, u32x4(&dst)[NV], u32x4(&dst_b)[NB]) {
        const uint16_t *xr = x + static_cast<int64_t>(row) * stride_x;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = k * bs + threadIdx.x;
            dst[k] = ld16_stream(xr + static_cast<uint64_t>(EXACT || v < nvec ? v : 0) * 8);
        }
        if constexpr (ADD) {
            const uint16_t *br = res.b + static_cast<int64_t>(row) * res.stride_b;
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const uint32_t v = k * bs + threadIdx.x;
                dst_b[k] = ld16_stream(br + static_cast<uint64_t>(EXACT || v < nvec ? v : 0) * 8);
            }
        }
    };

    // This workgroup's rows: first, first + hop, ... below `last`.
    uint64_t row = blockIdx.x * first_mul;
    if (row >= n) return;
    const uint64_t last = row + span < n ? row + span : n;
    u32x4 xv[NV], xn[NV], bv[NB], bn[NB];
    load_row(row, xv, bv);// in flight while the weights are fetched below
    bool more = AHEAD && row + hop < last;// this workgroup owns a row after the current one, and fetches it ahead

    if constexpr (WHOME == kWLds) {
        // All of this lane's weight loads are issued before the first is
        // consumed, and the second row's loads go out behind them before
        // anything waits: the workgroup pays one memory latency before it
        // streams, not one for the weights and another for the prefetch.
        auto stage = [&](auto tag) {
            typedef decltype(tag) W;
            float g[NV][8];
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const uint32_t v = k * bs + threadIdx.x;
                W::load8(w, EXACT || v < nvec ? v : 0, g[k]);
            }
            if (more) load_row(row + hop, xn, bn);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const uint32_t v = k * bs + threadIdx.x;
                if (EXACT || v < nvec) {
                    w_lo[v] = f32x4{g[k][0], g[k][1], g[k][2], g[k][3]};
                    w_hi[v] = f32x4{g[k][4], g[k][5], g[k][6], g[k][7]};
                }
            }
        };
        if (w_kind == kWKindF32) stage(WF32{});
        else if (w_kind == kWKindF16) stage(W16<F16Ref>{});
        else stage(W16<BF16Rne>{});
        __syncthreads();
    } else {
        if (more) load_row(row + hop, xn, bn);
    }

    // One row: reduce, scale by the weights, store.
    auto finish_row = [&](uint64_t r, u32x4(&cur)[NV], const u32x4(&cur_b)[NB], int phase) {
        if constexpr (ADD) {// cur += cur_b, rounded as Add rounds, and out to c
            const StreamOut<THROUGH> cr(res.c + static_cast<int64_t>(r) * res.stride_c);
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const uint32_t v = k * bs + threadIdx.x;
                float p[8], q[8];
                widen8<T>(cur[k], p);
                widen8<T>(cur_b[k], q);
#pragma unroll
                for (int i = 0; i < 8; ++i) p[i] += q[i];
                cur[k] = narrow8<T>(p);
                if (EXACT || v < nvec) cr.st16(v * 16, cur[k]);
            }
        }
        float part[NV];
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            float f[8];
            widen8<T>(cur[k], f);
            part[k] = EXACT || k * bs + threadIdx.x < nvec ? squares8(f) : 0.0f;
        }
        const float k_row = inv_rms((BS != 0 ? row_sum<MAX_WAVES, NV>(part, red + phase * NV * MAX_WAVES) : row_sum_any<NV>(part, red + phase * NV * MAX_WAVES, waves)), d, eps);

        const StreamOut<THROUGH> yr(y + static_cast<int64_t>(r) * stride_y);// a row is far shorter than 4 GiB
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = k * bs + threadIdx.x;
            if (EXACT || v < nvec) {
                float f[8], g[8];
                widen8<T>(cur[k], f);
                if constexpr (WHOME == kWLds) {
                    const f32x4 a = w_lo[v], b = w_hi[v];
                    g[0] = a.x, g[1] = a.y, g[2] = a.z, g[3] = a.w;
                    g[4] = b.x, g[5] = b.y, g[6] = b.z, g[7] = b.w;
                } else {
                    load_w8(w, w_kind, v, g);
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) f[i] = (k_row * f[i]) * g[i];
                yr.st16(v * 16, narrow8<T>(f));
            }
        }
    };

    // Steady state: the next row's loads are issued, unconditionally, before
    // the current row is reduced.  Two register sets take turns (no copies, so
    // the wait for a prefetched row comes only when that row is reduced) and a
    // row's loads are never issued unless this workgroup owns that row.  The
    // first row is finished ahead of the loop - the second is already on its
    // way - so that the loop is entered with the memory operations in the
    // order every later pass leaves them in, and the waits inside it count
    // the younger operations instead of draining the queue.
    if constexpr (!AHEAD) {// one register set: a row is fetched only after the one before it has been stored
        int phase = 0;
        while (true) {
            finish_row(row, xv, bv, phase);
            phase ^= 1;
            row += hop;
            if (row >= last) return;
            load_row(row, xv, bv);
        }
    }
    if (!more) {
        finish_row(row, xv, bv, 0);
        return;
    }
    finish_row(row, xv, bv, 0);
    row += hop;
    while (true) {
        if (row + hop >= last) {
            finish_row(row, xn, bn, 1);
            break;
        }
        load_row(row + hop, xv, bv);
        finish_row(row, xn, bn, 1);
        row += hop;
        if (row + hop >= last) {
            finish_row(row, xv, bv, 0);
            break;
        }
        load_row(row + hop, xn, bn);
        finish_row(row, xv, bv, 0);
        row += hop;
    }
}

// ---- wide rows ----------------------------------------------------------------
// Rows of more than 32 768 elements and the fused form from 10 240 (one
// workgroup per compute unit, as many lanes as the row has vectors for, up to
// 1024); the fused form between 4097 and 8191 and plain rows for which
// rms_norm_rows has no exact launch shape (two workgroups per unit of up to
// 512 lanes).  NV raw vectors per lane, one row at a time.  What differs from
// rms_norm_rows:
// - the lane count is the launch's, so that no lane is idle whatever the width;
// - loads go through a buffer descriptor of one row (or of the weight row): a
//   lane's address is one per-lane byte offset plus a wavefront-uniform one, no
//   vector register carries an address across the loop over rows, and vectors
//   behind the row's end read as zeros without a test.  (rms_norm_rows at eight
//   vectors per lane kept 48 registers of addresses alive and spilled them.)
//   Stores take the same descriptor but the whole offset per lane: a 16-byte
//   buffer store whose uniform offset comes from a scalar register was seen,
//   on MI355X, to pick up the value that the next instructions write into its
//   first data register (about one row in four of [512, 32768] had a few
//   elements wrong) - the compiler separates such a store from a write to its
//   data only when that offset is a constant;
// - the widened values are formed anew for the scaling (kept from the squares
//   they would take 8 registers per vector);
// - weights from memory (rows whose fp32 weights do not fit LDS) are requested
//   WBATCH vectors at a time as raw words, the first batch in front of the
//   reduction, and the weight type is resolved once, outside the loop over rows.
// The sum of squares is row_sum_any's, in its order: the same bits as every
// other form.
// Measured on MI355X, bf16 with fp32 weights, against rms_norm_rows (us):
//   fused [8192, 16384]  181.6 / 187.5     fused [8192, 12288]  134.4 / 138.7
//   fused [8192, 10240]  117.8 / 119.5     fused [4096, 32768]  183.0 / 192.1
//   plain [4096, 32768]   94.3 /  93.7 (so the plain form stays with rms_norm_rows up to there)
// (Two halves of a workgroup on rows of their own, each with a counting
// barrier in LDS and both sharing the staged weights, measured slower: plain
// [4096, 32768] 100.2 us, fused 191.6 us.  Each lane's weights held in its
// registers for all of a workgroup's rows, no LDS, so that two or three
// 512-lane workgroups fit a compute unit: plain [4096, 32768] 92.2-93.4 us
// against 93.3, [8192, 16384] 90.6 against 89.9 - no different.)
template<typename T, int NV, int WHOME, bool THROUGH, bool ADD, int WBATCH = 4>
__global__ __launch_bounds__(1024) void rms_norm_wide(uint16_t *y, const uint16_t *x, const void *w, int w_kind,
                                                      uint64_t n, uint32_t d, int64_t stride_y, int64_t stride_x, float eps,
                                                      Residual<ADD> res) {
    RMS_ARGS_NOW(gridDim.x, blockDim.x);
    constexpr int MAX_WAVES = 1024 / kWave;
    __shared__ float red[2 * NV * MAX_WAVES];
    extern __shared__ __attribute__((aligned(16))) unsigned char dyn_lds[];
    f32x4 *w_lo = reinterpret_cast<f32x4 *>(dyn_lds);
    const uint32_t nvec = d / 8;
    f32x4 *w_hi = w_lo + nvec;
    const uint32_t bs = blockDim.x, waves = bs / kWave;
    const uint32_t lane16 = threadIdx.x * 16;
    constexpr uint32_t kNt = 2, kOut = THROUGH ? (16 | 2) : 2;// cache policies: nt; sc1 nt
    const auto row_of = [&](const uint16_t *base, uint64_t row, int64_t stride) {
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(base + static_cast<int64_t>(row) * stride), 0, static_cast<int>(d * 2), 0x00020000);
    };

    if constexpr (WHOME == kWLds) {// the weight row, staged once as fp32
        auto stage = [&](auto tag) {
            typedef decltype(tag) W;
            constexpr uint32_t kWVec = 8 * sizeof(typename W::scalar);
            const __amdgpu_buffer_rsrc_t w_row = __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(w), 0, static_cast<int>(d * sizeof(typename W::scalar)), 0x00020000);
            typename W::raw wr[NV];
#pragma unroll
            for (int k = 0; k < NV; ++k) wr[k] = W::fetch(w_row, threadIdx.x * kWVec, k * bs * kWVec);
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const uint32_t v = k * bs + threadIdx.x;
                float g[8];
                W::spread(wr[k], g);
                if (v < nvec) {
                    w_lo[v] = f32x4{g[0], g[1], g[2], g[3]};
                    w_hi[v] = f32x4{g[4], g[5], g[6], g[7]};
                }
            }
        };
        if (w_kind == kWKindF32) stage(WF32{});
        else if (w_kind == kWKindF16) stage(W16<F16Ref>{});
        else stage(W16<BF16Rne>{});
        __syncthreads();
    }

    auto serve = [&](auto wtag) {
        typedef decltype(wtag) W;
        constexpr int WB = WHOME == kWLds ? 1 : (NV < WBATCH ? NV : WBATCH);
        constexpr uint32_t kWVec = 8 * sizeof(typename W::scalar);
        [[maybe_unused]] const __amdgpu_buffer_rsrc_t w_row =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(w), 0, static_cast<int>(d * sizeof(typename W::scalar)), 0x00020000);
        int phase = 0;
        for (uint64_t row = blockIdx.x; row < n; row += gridDim.x, phase ^= 1) {
            const __amdgpu_buffer_rsrc_t xr = row_of(x, row, stride_x);
            u32x4 cur[NV];
#pragma unroll
            for (int k = 0; k < NV; ++k) cur[k] = __builtin_amdgcn_raw_buffer_load_b128(xr, static_cast<int>(lane16), static_cast<int>(k * bs * 16), kNt);
            if constexpr (ADD) {// cur += b, rounded as Add rounds, and out to c
                const __amdgpu_buffer_rsrc_t br = row_of(res.b, row, res.stride_b), cr = row_of(res.c, row, res.stride_c);
                u32x4 other[NV];
#pragma unroll
                for (int k = 0; k < NV; ++k) other[k] = __builtin_amdgcn_raw_buffer_load_b128(br, static_cast<int>(lane16), static_cast<int>(k * bs * 16), kNt);
#pragma unroll
                for (int k = 0; k < NV; ++k) {
                    float p[8], q[8];
                    widen8<T>(cur[k], p);
                    widen8<T>(other[k], q);
#pragma unroll
                    for (int i = 0; i < 8; ++i) p[i] += q[i];
                    cur[k] = narrow8<T>(p);
                    __builtin_amdgcn_raw_buffer_store_b128(cur[k], cr, static_cast<int>(lane16 + k * bs * 16), 0, kOut);// behind the row's end: dropped
                }
            }
            [[maybe_unused]] typename W::raw wr[WB];
            [[maybe_unused]] auto fetch_weights = [&](int k0) {
#pragma unroll
                for (int j = 0; j < WB; ++j) {
                    if (k0 + j < NV) wr[j] = W::fetch(w_row, threadIdx.x * kWVec, (k0 + j) * bs * kWVec);
                }
            };
            if constexpr (WHOME == kWGlobal) fetch_weights(0);
            float part[NV];
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                float f[8];
                widen8<T>(cur[k], f);
                part[k] = squares8(f);// vectors behind the row's end were read as zeros
            }
            const float k_row = inv_rms(row_sum_any<NV>(part, red + phase * NV * MAX_WAVES, waves), d, eps);
#pragma unroll
            for (int k = 0; k < NV; ++k) asm volatile("" : "+v"(cur[k]));// what follows widens the raw words anew

            const __amdgpu_buffer_rsrc_t yr = row_of(y, row, stride_y);
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const uint32_t v = k * bs + threadIdx.x;
                if constexpr (WHOME == kWGlobal) {
                    if (k != 0 && k % WB == 0) {
                        __builtin_amdgcn_sched_barrier(0);// the batch before is used up: its registers take the next one
                        fetch_weights(k);
                    }
                }
                float f[8], g[8];
                widen8<T>(cur[k], f);
                if constexpr (WHOME == kWLds) {
                    const uint32_t lv = v < nvec ? v : 0;
                    const f32x4 a = w_lo[lv], b = w_hi[lv];
                    g[0] = a.x, g[1] = a.y, g[2] = a.z, g[3] = a.w;
                    g[4] = b.x, g[5] = b.y, g[6] = b.z, g[7] = b.w;
                } else {
                    W::spread(wr[k % WB], g);
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) f[i] = (k_row * f[i]) * g[i];
                __builtin_amdgcn_raw_buffer_store_b128(narrow8<T>(f), yr, static_cast<int>(lane16 + k * bs * 16), 0, kOut);
                if constexpr (NV >= 8) __builtin_amdgcn_sched_barrier(0);// one vector's arithmetic at a time: 128 registers per lane in all
            }
        }
    };
    if constexpr (WHOME == kWLds) {
        serve(WF32{});
    } else {
        if (w_kind == kWKindF32) serve(WF32{});
        else if (w_kind == kWKindF16) serve(W16<F16Ref>{});
        else serve(W16<BF16Rne>{});
    }
}

// ---- one pass in dispatch order ----------------------------------------------
// A workgroup serves R consecutive rows and retires; the grid is n / R
// workgroups, handed out in address order.  Everything a workgroup will ever
// load - its rows and the weight row, which it keeps in registers - is
// requested before the first wait, so it pays one memory latency.  The weight
// row comes through L2 once per R rows.  The R sums of squares share one
// barrier.
template<typename T, int BS, int NV, int R, bool EXACT, bool THROUGH, bool ADD>
__global__ __launch_bounds__(BS) void rms_norm_once(uint16_t *y, const uint16_t *x, const void *w, int w_kind,
                                                     uint64_t n, uint32_t d, int64_t stride_y, int64_t stride_x, float eps,
                                                     Residual<ADD> res) {
    RMS_ARGS_NOW();
    constexpr int WAVES = BS / kWave;
    __shared__ float red[R * NV * WAVES];
    const uint32_t nvec = d / 8;
    const uint64_t row0 = static_cast<uint64_t>(blockIdx.x) * R;
    const int rows_here = n - row0 < static_cast<uint64_t>(R) ? static_cast<int>(n - row0) : R;

    u32x4 xv[R][NV];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const uint64_t row = row0 + (r < rows_here ? r : 0);
        const uint16_t *xr = x + static_cast<int64_t>(row) * stride_x;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = k * BS + threadIdx.x;
            xv[r][k] = ld16_stream(xr + static_cast<uint64_t>(EXACT || v < nvec ? v : 0) * 8);
        }
    }
    constexpr int RB = ADD ? R : 1;
    u32x4 bv[RB][NV];
    if constexpr (ADD) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const uint64_t row = row0 + (r < rows_here ? r : 0);
            const uint16_t *br = res.b + static_cast<int64_t>(row) * res.stride_b;
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const uint32_t v = k * BS + threadIdx.x;
                bv[r][k] = ld16_stream(br + static_cast<uint64_t>(EXACT || v < nvec ? v : 0) * 8);
            }
        }
    }
    // The rows' loads stay in front of the branches on the weight type: left alone, the compiler sinks them into
    // the branches, behind the wait for 16-bit weights that are widened there - two memory latencies in a row
    // ([131072, 512] bf16 with bf16 weights 45.9 us, with fp32 weights 41.4).
    asm volatile("" ::: "memory");
    float g[NV][8];
    if (w_kind == kWKindF32) {
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = k * BS + threadIdx.x;
            WF32::load8(w, EXACT || v < nvec ? v : 0, g[k]);
        }
    } else {
        u32x4 raw[NV];
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = k * BS + threadIdx.x;
            raw[k] = ld16(static_cast<const uint16_t *>(w) + static_cast<uint64_t>(EXACT || v < nvec ? v : 0) * 8);
        }
        if (w_kind == kWKindF16) {
#pragma unroll
            for (int k = 0; k < NV; ++k) widen8<F16Ref>(raw[k], g[k]);
        } else {
#pragma unroll
            for (int k = 0; k < NV; ++k) widen8<BF16Rne>(raw[k], g[k]);
        }
    }

    float part[R][NV];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if constexpr (ADD) {// the row becomes a + b, rounded as Add rounds, and goes out to c
            const StreamOut<THROUGH> cr(res.c + static_cast<int64_t>(row0 + r) * res.stride_c);
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const uint32_t v = k * BS + threadIdx.x;
                float p[8], q[8];
                widen8<T>(xv[r][k], p);
                widen8<T>(bv[r][k], q);
#pragma unroll
                for (int i = 0; i < 8; ++i) p[i] += q[i];
                xv[r][k] = narrow8<T>(p);
                if (r < rows_here && (EXACT || v < nvec)) cr.st16(v * 16, xv[r][k]);
            }
        }
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            float f[8];
            widen8<T>(xv[r][k], f);
            part[r][k] = EXACT || k * BS + threadIdx.x < nvec ? squares8(f) : 0.0f;
        }
    }
    // the R rows' chunk sums go through LDS side by side and share one barrier
    float total[R];
    if constexpr (WAVES == 1) {
#pragma unroll
        for (int r = 0; r < R; ++r) total[r] = row_sum<1, NV>(part[r], red);
    } else {
        const int wave = threadIdx.x / kWave;
#pragma unroll
        for (int r = 0; r < R; ++r) {
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                const float c = wave_sum(part[r][k]);
                if ((threadIdx.x & (kWave - 1)) == 0) red[(r * NV + k) * WAVES + wave] = c;
            }
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < R; ++r) {
            total[r] = 0.0f;
#pragma unroll
            for (int j = 0; j < NV * WAVES; ++j) total[r] += red[r * NV * WAVES + j];
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const float k_row = inv_rms(total[r], d, eps);
        const StreamOut<THROUGH> yr(y + static_cast<int64_t>(row0 + r) * stride_y);
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = k * BS + threadIdx.x;
            float f[8];
            widen8<T>(xv[r][k], f);
#pragma unroll
            for (int i = 0; i < 8; ++i) f[i] = (k_row * f[i]) * g[k][i];
            if (r < rows_here && (EXACT || v < nvec)) yr.st16(v * 16, narrow8<T>(f));
        }
    }
}

// ---- short rows: several rows per wavefront ---------------------------------------
// Rows of up to 256 elements (the per-head norms of attention: head_dim 64-256)
// would leave most of a wavefront idle at one row each.  Here P = 8, 16 or 32
// lanes serve a row, one vector per lane, and a wavefront takes 64 / P
// consecutive rows; the sum of squares is the first steps of the wavefront
// tree (amd::segment_sum), which adds the same values in the same order as
// the full tree would with zeros in the absent lanes - so these rows, too,
// give the bits every other form gives.  A turn of the wavefront takes U such
// groups of rows, with the loads of all of them in flight together.
template<typename T, int P, int U, bool THROUGH, bool ADD>
__global__ __launch_bounds__(kWave) void rms_norm_short(uint16_t *y, const uint16_t *x, const void *w, int w_kind,
                                                        uint64_t n, uint32_t d, int64_t stride_y, int64_t stride_x, float eps,
                                                        Residual<ADD> res) {
    RMS_ARGS_NOW(gridDim.x);
    constexpr uint32_t RPW = kWave / P;// rows per wavefront and group; U groups per turn
    const uint32_t nvec = d / 8;
    const uint32_t sub = threadIdx.x % P, rr = threadIdx.x / P;
    const uint32_t lv = sub < nvec ? sub : 0;
    const uint64_t hop = static_cast<uint64_t>(gridDim.x) * RPW * U;
    uint64_t row0 = static_cast<uint64_t>(blockIdx.x) * RPW * U;
    if (row0 >= n) return;
    // absent rows re-read the turn's first one; nothing of them is stored
    const auto row_of = [&](uint64_t first, int u) { return first + u * RPW + rr < n ? first + u * RPW + rr : first; };
    // The first rows are asked for in front of the weights: 16-bit weights are widened as soon as they arrive,
    // and with the weights asked for first that wait stood in front of the rows' request - two memory latencies
    // in a row for a wavefront that serves one group of rows ([524288, 128] bf16 with bf16 weights 47.2 us, with
    // fp32 weights, which need no widening, 42.0).
    u32x4 xv[U];
    [[maybe_unused]] u32x4 bv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        xv[u] = ld16_stream(x + static_cast<int64_t>(row_of(row0, u)) * stride_x + static_cast<uint64_t>(lv) * 8);
        if constexpr (ADD) bv[u] = ld16_stream(res.b + static_cast<int64_t>(row_of(row0, u)) * res.stride_b + static_cast<uint64_t>(lv) * 8);
    }
    float g[8];
    load_w8(w, w_kind, lv, g);
    while (true) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint64_t first = row0 + u * RPW;
            const bool have = first + rr < n && sub < nvec;
            if constexpr (ADD) {// the row becomes a + b, rounded as Add rounds, and goes out to c
                float p[8], q[8];
                widen8<T>(xv[u], p);
                widen8<T>(bv[u], q);
#pragma unroll
                for (int i = 0; i < 8; ++i) p[i] += q[i];
                xv[u] = narrow8<T>(p);
                const StreamOut<THROUGH> cr(res.c + static_cast<int64_t>(first) * res.stride_c);
                if (have) cr.st16(rr * static_cast<uint32_t>(res.stride_c) * 2 + sub * 16, xv[u]);
            }
            float f[8];
            widen8<T>(xv[u], f);
            const float k_row = inv_rms(segment_sum<P>(sub < nvec ? squares8(f) : 0.0f), d, eps);
#pragma unroll
            for (int i = 0; i < 8; ++i) f[i] = (k_row * f[i]) * g[i];
            const StreamOut<THROUGH> yr(y + static_cast<int64_t>(first) * stride_y);
            if (have) yr.st16(rr * static_cast<uint32_t>(stride_y) * 2 + sub * 16, narrow8<T>(f));
        }
        row0 += hop;
        if (row0 >= n) break;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            xv[u] = ld16_stream(x + static_cast<int64_t>(row_of(row0, u)) * stride_x + static_cast<uint64_t>(lv) * 8);
            if constexpr (ADD) bv[u] = ld16_stream(res.b + static_cast<int64_t>(row_of(row0, u)) * res.stride_b + static_cast<uint64_t>(lv) * 8);
        }
    }
}

// ---- any row length, any alignment ----------------------------------------------
// Two passes over the row; the second pass re-reads x, which the first pass
// left in cache for rows of ordinary length.  Whole groups of 8 elements move
// as 16 bytes at whatever 2-byte boundary they lie on, the last, partial group
// element by element ([8192, 8191] bf16: 295 us with element accesses only).  A lane owns
// whole groups of 8 elements - the vectors of the kernels above - and rows of
// up to 65 536 elements are summed in the same order as there (a group's
// pairwise partial, 64 groups by the wavefront tree, those chunk sums in
// ascending order), so a row gives the same bits whether its alignment and
// strides allow the vector kernels or not.  Longer rows, which only this
// kernel serves, add the chunk sums per wavefront first.
template<typename T, bool ADD>
__global__ __launch_bounds__(256) void rms_norm_generic(uint16_t *y, const uint16_t *x, const void *w, int w_kind,
                                                         uint64_t n, uint64_t d, int64_t stride_y, int64_t stride_x, float eps,
                                                         Residual<ADD> res) {
    RMS_ARGS_NOW(gridDim.x);
    constexpr int BS = 256, WAVES = BS / kWave;
    constexpr uint64_t kChunk = 8 * kWave, kMaxChunks = 128;
    __shared__ float red[2 * WAVES];
    __shared__ float chunk_sum[kMaxChunks];
    const uint32_t lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const uint64_t chunks = (d + kChunk - 1) / kChunk;
    const bool in_order = chunks <= kMaxChunks;
    int phase = 0;
    for (uint64_t row = blockIdx.x; row < n; row += gridDim.x, phase ^= 1) {
        const uint16_t *xr = x + static_cast<int64_t>(row) * stride_x;
        uint16_t *yr = y + static_cast<int64_t>(row) * stride_y;
        const uint16_t *br = nullptr;
        uint16_t *cr = nullptr;
        if constexpr (ADD) {// first pass forms and stores the sum; the second pass reads it back from c
            br = res.b + static_cast<int64_t>(row) * res.stride_b;
            cr = res.c + static_cast<int64_t>(row) * res.stride_c;
        }
        float part = 0.0f;
        for (uint64_t c = wave; c < chunks; c += WAVES) {
            const uint64_t j0 = (c * kWave + lane) * 8;
            float f[8];
            if (j0 + 8 <= d) {// a whole group: 16 bytes at whatever boundary the row puts them
                u32x4 raw = ld16_any(xr + j0);
                if constexpr (ADD) {
                    float q[8];
                    widen8<T>(raw, f);
                    widen8<T>(ld16_any(br + j0), q);
#pragma unroll
                    for (int e = 0; e < 8; ++e) f[e] += q[e];
                    raw = narrow8<T>(f);
                    st16_any(cr + j0, raw);
                }
                widen8<T>(raw, f);
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const uint64_t j = j0 + e;
                    f[e] = 0.0f;
                    if (j < d) {
                        if constexpr (ADD) {
                            const uint16_t sum = T::narrow1(T::one(xr[j]) + T::one(br[j]));
                            cr[j] = sum;
                            f[e] = T::one(sum);
                        } else {
                            f[e] = T::one(xr[j]);
                        }
                    }
                }
            }
            const float s = wave_sum(squares8(f));
            if (in_order) {
                if (lane == 0) chunk_sum[c] = s;
            } else {
                part += s;
            }
        }
        if constexpr (ADD) xr = cr;
        float total;
        if (in_order) {
            __syncthreads();
            total = 0.0f;
            for (uint64_t c = 0; c < chunks; ++c) total += chunk_sum[c];
            __syncthreads();// the next row's chunk sums wait for everyone to have read these
        } else {
            // every lane of a wavefront holds the wavefront's sum: one lane of each enters the workgroup's
            total = block_sum<WAVES>(lane == 0 ? part : 0.0f, red, phase);
        }
        const float k_row = inv_rms(total, d, eps);
        for (uint64_t c = wave; c < chunks; c += WAVES) {
            const uint64_t j0 = (c * kWave + lane) * 8;
            if (j0 + 8 <= d) {
                float f[8], g[8];
                widen8<T>(ld16_any(xr + j0), f);
                if (w_kind == kWKindF32) {
                    const float *wp = static_cast<const float *>(w) + j0;
                    const f32x4 a = *reinterpret_cast<const f32x4_any *>(wp), b = *reinterpret_cast<const f32x4_any *>(wp + 4);
                    g[0] = a.x, g[1] = a.y, g[2] = a.z, g[3] = a.w;
                    g[4] = b.x, g[5] = b.y, g[6] = b.z, g[7] = b.w;
                } else {
                    const u32x4 raw = ld16_any(static_cast<const uint16_t *>(w) + j0);
                    if (w_kind == kWKindF16) widen8<F16Ref>(raw, g);
                    else widen8<BF16Rne>(raw, g);
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) f[e] = (k_row * f[e]) * g[e];
                st16_any(yr + j0, narrow8<T>(f));
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const uint64_t j = j0 + e;
                    if (j < d) yr[j] = T::narrow1((k_row * T::one(xr[j])) * load_w1(w, w_kind, j));
                }
            }
        }
        // y may alias x (and c may alias a or b): every lane re-reads only elements it wrote itself.
    }
}

// ---- launch -----------------------------------------------------------------------
// What a launch needs to know about the operator instance.
}// namespace
struct RowsShape {// plain data, with external linkage: it crosses translation units
    int cu_count;
    int lds_per_block;
    uint64_t n, d;
    int64_t stride_y, stride_x;
    float epsilon;
};
namespace {

// Weight element type -> kind; negative when the type is not supported.
inline int weight_kind(amd::Elem w_elem) {
    switch (w_elem) {
        case amd::Elem::F32: return kWKindF32;
        case amd::Elem::F16: return kWKindF16;
        case amd::Elem::BF16: return kWKindBF16;
        default: return -1;
    }
}

template<typename T, bool ADD>
void launch_rms_norm(const RowsShape &desc, void *y, const void *x, const void *w, int w_kind, const Residual<ADD> &res, hipStream_t stream) {
    auto *py = static_cast<uint16_t *>(y);
    auto *px = static_cast<const uint16_t *>(x);
    const uint64_t n = desc.n, d = desc.d;
    const uint64_t nvec = d / 8;

    bool vec_ok = d % 8 == 0 && nvec <= 8192 && desc.stride_x % 8 == 0 && desc.stride_y % 8 == 0 &&
                  aligned16(x) && aligned16(y) && aligned16(w);
    if constexpr (ADD) {
        vec_ok = vec_ok && res.stride_b % 8 == 0 && res.stride_c % 8 == 0 && aligned16(res.b) && aligned16(res.c);
    }
    if (!vec_ok) {
        const uint64_t cap = static_cast<uint64_t>(desc.cu_count) * 8;
        rms_norm_generic<T, ADD><<<static_cast<unsigned>(n < cap ? n : cap), 256, 0, stream>>>(
            py, px, w, w_kind, n, d, desc.stride_y, desc.stride_x, desc.epsilon, res);
        return;
    }
    // Large outputs are written through L2 (see StreamOut).
    const bool through = n * d * sizeof(uint16_t) >= kWriteThroughBytes;

    // Which form.  Measured on MI355X, 128 MiB of bf16 rows with fp32 weights
    // (and [8192, 8192] for the fused form), one pass (R rows per workgroup,
    // weights in registers) against looping workgroups (weights in LDS):
    //   d =  512:  41.2 us one pass, R = 1          46.9 us looping
    //   d =  768:  43.9 us one pass with 128 lanes, R = 2 (45.6 with R = 4; 54.8 with 256 lanes)
    //   d = 1024:  43.8 us one pass with 128 lanes, R = 2 (45.1 with R = 4); 45.5-46.7 with 256 lanes, R = 2 (59.0 with R = 1)   51.2 us looping
    //   d = 2048:  44.4 us one pass, R = 2 (47.0 with R = 1)   47.9 us looping
    //   d = 4096:  45.5 us one pass, R = 1 (46.4 with R = 2)   46.6 us looping
    //   d = 8192:  45.6-50.3 us one pass            44.6 us looping
    //   d = 8192, fused Add: 86.5 us one pass with 1024 lanes, 88.1-89.7 with 256 or 512   89.0 us looping
    //   d >= 16384: looping (a row's weights are 64 KiB and more: too many registers); the fused form from 10240
    //   and plain rows beyond 32768: rms_norm_wide, below
    // One pass re-reads the weight row through L2 once per R rows - at d = 8192
    // that is twice the bytes of the row itself - which is what it loses to
    // the looping form there; the fused form moves twice the data per weight.
    // (Every one-pass shape of 64-512 lanes x 1-4 vectors x 1, 2 or 4 rows that covers the row, timed at eleven
    // widths from 768 to 4096, plain with fp32 and with 16-bit weights and fused: the best of them is 0-3 % ahead
    // of the shapes below, 384 x 1 x 2 at d = 2560 with fp32 weights 45.2 against 47.1 us being the largest gap.)
#define RMS_ONCE_GO(BS, NV, R, E, TH)                                                                              \
    rms_norm_once<T, BS, NV, R, E, TH, ADD><<<static_cast<unsigned>(ceil_div(n, R)), BS, 0, stream>>>(              \
        py, px, w, w_kind, n, static_cast<uint32_t>(d), desc.stride_y, desc.stride_x, desc.epsilon, res)
#define RMS_ONCE(BS, NV, R)                                                                                        \
    do {                                                                                                           \
        const bool exact = nvec == static_cast<uint64_t>(BS) * NV;                                                 \
        if (exact && through) RMS_ONCE_GO(BS, NV, R, true, true);                                                  \
        else if (exact) RMS_ONCE_GO(BS, NV, R, true, false);                                                       \
        else if (through) RMS_ONCE_GO(BS, NV, R, false, true);                                                     \
        else RMS_ONCE_GO(BS, NV, R, false, false);                                                                 \
    } while (0)
    // Rows of up to 256 elements, 8 consecutive ones within reach of a 32-bit
    // byte offset from the first: 2-8 rows per wavefront.
    bool near = desc.stride_y >= 0 && desc.stride_y < (1 << 26);
    if constexpr (ADD) near = near && res.stride_c >= 0 && res.stride_c < (1 << 26);
    if (nvec <= 32 && near) {
        const unsigned lanes = nvec <= 8 ? 8 : (nvec <= 16 ? 16 : 32);
        // A wavefront has one 16-byte load per lane in flight, and the compute unit's wavefronts together must cover
        // the memory latency: rows that leave a quarter or more of their lanes idle (72, 80, 96, 160, 192 elements)
        // take two groups of rows per turn.  Measured, [64 Mi / d, d] bf16 with fp32 weights, us, one / two / four
        // groups: d = 72: 58.9 / 49.3 / 48.4, 80: 53.9 / 46.7 / 47.3, 96: 46.2 / 45.3 / 46.9, 160: 53.7 / 47.2 / 47.1,
        // 192: 46.9 / 45.1 / 47.4; rows that fill their lanes lose by it (112: 42.7 / 45.2, 128: 41.9 / 43.6,
        // 256: 41.4 / 43.4), and so does the fused form, which has two loads per lane in flight as it is
        // (80: 66.2 / 68.8, 160: 65.7 / 68.1).
        const unsigned turns = !ADD && nvec * 4 <= lanes * 3 ? 2 : 1;
        const uint64_t want = ceil_div(n, kWave / lanes * turns), cap = amd::max_grid_1d(kWave);
        const unsigned grid = static_cast<unsigned>(want < cap ? want : cap);
#define RMS_SHORT_GO(P, U, TH)                                                                                      \
    rms_norm_short<T, P, U, TH, ADD><<<grid, kWave, 0, stream>>>(py, px, w, w_kind, n, static_cast<uint32_t>(d),    \
                                                                 desc.stride_y, desc.stride_x, desc.epsilon, res)
#define RMS_SHORT(P)                                                                                                   \
    do {                                                                                                               \
        if constexpr (!ADD) {                                                                                          \
            if (turns == 2) {                                                                                          \
                if (through) RMS_SHORT_GO(P, 2, true);                                                                 \
                else RMS_SHORT_GO(P, 2, false);                                                                        \
                break;                                                                                                 \
            }                                                                                                          \
        }                                                                                                              \
        if (through) RMS_SHORT_GO(P, 1, true);                                                                         \
        else RMS_SHORT_GO(P, 1, false);                                                                                \
    } while (0)
        if (lanes == 8) RMS_SHORT(8);
        else if (lanes == 16) RMS_SHORT(16);
        else RMS_SHORT(32);
#undef RMS_SHORT_GO
#undef RMS_SHORT
        return;
    }
    // A one-pass grid has a workgroup per R rows; beyond what one launch can
    // hold the looping kernels below take over.
    const auto once_fits = [&](unsigned lanes, unsigned rows) { return ceil_div(n, rows) <= amd::max_grid_1d(lanes); };
    if (nvec <= 64 && once_fits(64, 1)) {
        // (rows of 264-384 elements leave a quarter and more of the wavefront idle: two rows per wavefront, as above;
        // [64 Mi / d, d] bf16, us, one / two rows: d = 320: 51.7 / 43.4, 384: 45.1 / 43.4, 448: 41.7 / 44.0, 512: 41.1 / 44.3)
        bool two = false;
        if constexpr (!ADD) two = nvec <= 48 && once_fits(64, 2);
        if constexpr (!ADD) {
            if (two) {
                RMS_ONCE(64, 1, 2);
                return;
            }
        }
        RMS_ONCE(64, 1, 1);
        return;
    }
    if (nvec > 64 && nvec <= 128 && once_fits(128, 2)) {
        RMS_ONCE(128, 1, 2);
        return;
    }
    if (nvec > 128 && nvec <= 256 && once_fits(256, 2)) {
        RMS_ONCE(256, 1, 2);
        return;
    }
    if (nvec > 256 && nvec <= 512 && once_fits(256, 1)) {
        // fp32 weights are twice the row's own bytes through L2: two rows per workgroup share them where the
        // lanes are not all busy anyway (64 MiB of bf16 rows, us, one row per workgroup / two: d = 2304  52.1 / 47.6,
        // 2560  49.9 / 46.9, 3072  49.2 / 46.5, 3584  48.4 / 46.6, 3840  48.8 / 47.0; 4096  45.7 / 46.3; with 16-bit
        // weights one row per workgroup runs all of these in 44.3-45.1; the fused form loses by two: 3072  90.0 / 93.5)
        bool pair = false;
        if constexpr (!ADD) pair = w_kind == kWKindF32 && nvec < 512 && once_fits(256, 2);
        if constexpr (!ADD) {
            if (pair) RMS_ONCE(256, 2, 2);
        }
        if (!pair) RMS_ONCE(256, 2, 1);
        return;
    }
    if constexpr (ADD) {
        if (nvec == 1024 && once_fits(1024, 1)) {
            if (through) RMS_ONCE_GO(1024, 1, 1, true, true);
            else RMS_ONCE_GO(1024, 1, 1, true, false);
            return;
        }
        // (Wider rows in one pass with two vectors per lane: d = 16384 92.2 us against 93.9 us looping, and
        // 105-111 us against 92-95 us at 9216-14336, where a third of the lanes has nothing to load.)
    }
#undef RMS_ONCE
#undef RMS_ONCE_GO

    // rms_norm_wide.  Rows of more than 32 768 elements, and the fused form from 10 240: one workgroup per compute
    // unit with as many lanes as the row has vectors for.  Plain rows from 6144 elements whose vector count is no
    // multiple of 64, so that no launch shape below fits them exactly: two workgroups per unit of up to 512 lanes
    // (128 MiB of bf16 rows, us, against the predicated ladder of rms_norm_rows:
    //   d = 6720  45.9 / 57.5    7232  45.1 / 54.5    9280  45.2 / 49.9    10304  45.5 / 50.4    15424  45.4 / 47.4    18496  48.3 / 51.7
    //   and rows that do not even start on 128-byte boundaries: d = 7000  56.7 / 74.4    9000  55.0 / 64.1    10000  54.6 / 62.2;
    //   below 6144 elements the ladder is the faster one: d = 4544  48.7 against 52.8, 5184  47.2 against 51.7).
    // The fused form between 4097 and 8191 elements: two workgroups per unit of 2 or 3 vectors per lane (128 MiB per
    // operand, us, against rms_norm_rows: d = 4608  87.3 / 96.6    5120  88.2 / 98.7    6144  87.4 / 97.2    7168  89.1 / 91.1
    // 7680  89.7 / 91.1; from 8704 to 10 239 rms_norm_rows is level or ahead: 9216  92.4 against 94.4).
    const bool no_exact_shape = !ADD && nvec % kWave != 0 && nvec >= 768;
    const bool fused_mid = ADD && nvec > 512 && nvec < 1024;
    if (nvec > 4096 || (ADD && nvec >= 1280) || no_exact_shape || fused_mid) {
        const bool one_per_unit = nvec > 4096 || (ADD && nvec >= 1280);
        const unsigned per_lane = static_cast<unsigned>(one_per_unit ? ceil_div(nvec, 1024) : fused_mid ? (nvec <= 768 ? 2 : 3) : std::min<uint64_t>(4, ceil_div(nvec, 512)));// 2 .. 8
        const unsigned lanes = static_cast<unsigned>(ceil_div(ceil_div(nvec, per_lane), kWave)) * kWave;
        const uint64_t lds_need = d * sizeof(float) + 2048;
        const unsigned per_cu = !one_per_unit && 2 * lds_need <= static_cast<uint64_t>(desc.lds_per_block) ? 2 : 1;
        const uint64_t cap = static_cast<uint64_t>(desc.cu_count) * per_cu;
        const bool in_lds = lds_need <= static_cast<uint64_t>(desc.lds_per_block) && n > cap;
        const unsigned g = static_cast<unsigned>(n < cap ? n : cap);
#define RMS_WIDE_GO(NV, HOME, TH)                                                                                              \
    rms_norm_wide<T, NV, HOME, TH, ADD><<<g, lanes, HOME == kWLds ? d * sizeof(float) : 0, stream>>>(                             \
        py, px, w, w_kind, n, static_cast<uint32_t>(d), desc.stride_y, desc.stride_x, desc.epsilon, res)
#define RMS_WIDE(NV)                                        \
    do {                                                    \
        if (in_lds && through) RMS_WIDE_GO(NV, kWLds, true); \
        else if (in_lds) RMS_WIDE_GO(NV, kWLds, false);      \
        else if (through) RMS_WIDE_GO(NV, kWGlobal, true);   \
        else RMS_WIDE_GO(NV, kWGlobal, false);               \
    } while (0)
        switch (per_lane) {
            case 2: RMS_WIDE(2); break;
            case 3: RMS_WIDE(3); break;
            case 4: RMS_WIDE(4); break;
            case 5: RMS_WIDE(5); break;
            case 6: RMS_WIDE(6); break;
            case 7: RMS_WIDE(7); break;
            default: RMS_WIDE(8); break;
        }
#undef RMS_WIDE
#undef RMS_WIDE_GO
        return;
    }
    // What is left: plain rows of 4097 to 32 768 elements and fused ones below 10 240.  A workgroup that serves
    // several rows fetches the weights once, into LDS as fp32 (128 KiB at most here: it always fits the 160 KiB a
    // gfx950 workgroup may use; above 80 KiB only one workgroup fits a compute unit).
    const uint64_t lds_bytes = d * sizeof(float);
    // How many workgroups per compute unit.  With the next row always in flight
    // a workgroup keeps two rows' worth of loads outstanding, and what measures
    // best is 20-32 KiB of them per compute unit, not more: bf16 rows with fp32
    // weights, 128 MiB in all, 1 / 2 / 3 / 4 workgroups per unit -
    //   d =  5120:  49.4 / 44.9 / 46.6 / 47.4 us      d = 10240:  45.6 / 47.0 / 48.3 / 48.3 us
    //   d =  6144:  45.8 / 45.4 / 47.1 / 47.9 us      d = 12288:  45.3 / 46.9 / 47.2 / 47.1 us
    //   d =  7168:  45.6 / 47.0 / 46.3 / 47.4 us      d = 16384:  46.7 / 46.7 us
    //   d =  8192:  44.6 / 44.8 / 45.2 / 45.5 us
    // so rows of up to 12 KiB get two workgroups per unit and longer ones one.
    // The two widths that split into 512-lane workgroups of whole vectors are the exception: two of those per
    // unit measure the same or better than one (d = 8192: 43.7-44.6 against 44.3-44.7 us on two machines;
    // d = 16384: 45.0-45.9 against 46.0-46.6 us).
    uint64_t per_cu = d * sizeof(uint16_t) > 12 * 1024 ? 1 : 2;
    if (!ADD && (d == 8192 || d == 16384)) per_cu = 2;
    // (128 MiB of bf16 rows, weights in LDS against re-read through L2 per row:
    //   d = 18432  48.0 / 58.8 us     d = 24576  48.0 / 55.1 us     d = 32768  49.5 / 54.3 us)
    int home = kWLds;
    uint64_t grid = static_cast<uint64_t>(desc.cu_count) * per_cu;
    if (n <= grid) {
        grid = n;
        home = kWGlobal;// one row per workgroup: staging would only add a pass
    }
    // rows of a workgroup: blockIdx.x, + grid, + 2 * grid, ...  (Consecutive
    // rows per workgroup measure 2-13 % slower at [8192, 8192].)
    const uint64_t first_mul = 1, hop = grid, span = n;

    // The kernels that re-read the weights from memory per row exist in one
    // form only (inexact row length, plain non-temporal stores): they serve
    // one-row workgroups and rows too long for LDS, where neither refinement
    // is measurable.
    // Two register sets (the next row fetched ahead) fit the 128 registers a
    // lane of a 1024-lane workgroup may have up to 4 vectors per lane, 2 in
    // the fused form.
#define RMS_GO(BS, NV, HOME, LDS, EXACT, THROUGH)                                                                      \
    rms_norm_rows<T, BS, NV, HOME, EXACT, THROUGH, ADD, (BS * NV * (ADD ? 2 : 1) <= 4096)>                             \
        <<<static_cast<unsigned>(grid), BS, LDS, stream>>>(                                                            \
        py, px, w, w_kind, n, static_cast<uint32_t>(d), desc.stride_y, desc.stride_x, desc.epsilon, first_mul, hop, span, res)
#define RMS_LAUNCH(BS, NV)                                                                                             \
    do {                                                                                                               \
        if (home != kWLds) RMS_GO(BS, NV, kWGlobal, 0, false, false);                                                  \
        else if (through) RMS_GO(BS, NV, kWLds, lds_bytes, false, true);                                               \
        else RMS_GO(BS, NV, kWLds, lds_bytes, false, false);                                                           \
    } while (0)

    // Row lengths of common models get a launch shape that fits them exactly
    // (lanes x vectors per lane = the row), two or three vectors per lane
    // where that measures best (us per 128 MiB of bf16 rows; the last figure
    // of each line is the general ladder below, which predicates the vectors
    // a row does not have):
    //   d =  5120: 320 x 2  47.5   640 x 1  51.5                  256 x 4  48.4
    //   d =  6144: 256 x 3  46.8   384 x 2  47.6                  256 x 4  48.5
    //   d =  7168: 896 x 1  46.1   448 x 2  47.5                  256 x 4  48.0
    //   d =  8192: 512 x 2  43.4-44.7   1024 x 1  44.2-45.0       256 x 4  44.3-44.8
    //   d = 10240: 640 x 2  47.1                                  512 x 4  49.7
    //   d = 12288: 512 x 3  46.4   768 x 2  47.2                  512 x 4  48.9
    //   d = 14336: 896 x 2  48.0                                  512 x 4  48.3
    //   d = 16384: 512 x 4  46.4   1024 x 2  47.5
    // Any other multiple of 512 elements gets its exact shape from the same
    // kernel with the lane count taken from the launch (d = 4608: 46.6 against
    // 48.2 on the ladder; d = 9216: 45.6 against 50.3), which at the widths
    // above is 0.5-2.5 % slower than the kernels compiled for them.  The fused
    // form keeps the ladder: an exact shape gained it nothing (d = 5120: 96.6
    // against 97.6).
    if constexpr (!ADD) {
        if (home == kWLds && nvec % kWave == 0) {
#define RMS_EXACT(BS, NV, LANES)                                                                                       \
    do {                                                                                                               \
        if (through)                                                                                                   \
            rms_norm_rows<T, BS, NV, kWLds, true, true, ADD><<<static_cast<unsigned>(grid), LANES, lds_bytes, stream>>>( \
                py, px, w, w_kind, n, static_cast<uint32_t>(d), desc.stride_y, desc.stride_x, desc.epsilon, first_mul, hop, span, res); \
        else                                                                                                           \
            rms_norm_rows<T, BS, NV, kWLds, true, false, ADD><<<static_cast<unsigned>(grid), LANES, lds_bytes, stream>>>( \
                py, px, w, w_kind, n, static_cast<uint32_t>(d), desc.stride_y, desc.stride_x, desc.epsilon, first_mul, hop, span, res); \
        return;                                                                                                        \
    } while (0)
            switch (nvec) {
                case 640: RMS_EXACT(320, 2, 320);
                case 768: RMS_EXACT(256, 3, 256);
                case 896: RMS_EXACT(896, 1, 896);
                case 1024: RMS_EXACT(512, 2, 512);
                case 1280: RMS_EXACT(640, 2, 640);
                case 1536: RMS_EXACT(512, 3, 512);
                case 1792: RMS_EXACT(896, 2, 896);
                case 2048: RMS_EXACT(512, 4, 512);
                default: break;
            }
            const uint64_t m = nvec / kWave;
            for (int cand : {2, 3, 4, 1}) {
                const unsigned lanes = static_cast<unsigned>(kWave * m / cand);
                if (m % cand != 0 || lanes < 256 || lanes > 1024) continue;
                switch (cand) {
                    case 1: RMS_EXACT(0, 1, lanes);
                    case 2: RMS_EXACT(0, 2, lanes);
                    case 3: RMS_EXACT(0, 3, lanes);
                    default: RMS_EXACT(0, 4, lanes);
                }
            }
#undef RMS_EXACT
        }
    }
    if (nvec <= 1024) RMS_LAUNCH(256, 4);
    else if (nvec <= 2048) RMS_LAUNCH(512, 4);
    else RMS_LAUNCH(1024, 4);
#undef RMS_LAUNCH
#undef RMS_GO
}

}// namespace
}// namespace rms_norm_kernels

#endif
