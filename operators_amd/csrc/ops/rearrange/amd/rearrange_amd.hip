// gfx950 kernels for Rearrange and their launch: a strided copy that moves
// each innermost row as a block of bytes (reference
// src/ops/rearrange/cpu/rearrange_cpu.cc:70-92).  No arithmetic at all: the
// only questions are how wide an access the layout allows and how to find a
// row's two addresses cheaply.
#include "../../../devices/amd/kernel_amd.h"
#include "rearrange_amd.h"

namespace {

using namespace amd;

// Lanes per workgroup.  16-byte units go out in workgroups of one wavefront,
// one KiB each, handed out in address order by the dispatcher (measured on
// MI355X with a 128 MiB copy: 40.3 us against 41.5 us with 256 lanes);
// narrower units keep 256 lanes so that the launch rate of workgroups (about
// 4.5 per ns) does not become the limit.
template<int BYTES>
struct Lanes {
    static constexpr int value = BYTES == 16 ? kWave : 256;
};

struct OuterDims {
    int ndim;
    uint32_t shape[kRearrangeMaxDims];
    int64_t dst_stride[kRearrangeMaxDims];
    int64_t src_stride[kRearrangeMaxDims];
    FastDiv by_shape[kRearrangeMaxDims];// division by shape[k], for the FAST kernels
};

// All of an OuterDims argument as operands of AMD_ARGS_NOW: 22 of them, neighbours of 4 bytes taken two at a time.
#define ARGS_OF_DIMS(d)                                                                                                                          \
    d.ndim, arg_pair(d.shape[0], d.shape[1]), arg_pair(d.shape[2], d.shape[3]), arg_pair(d.shape[4], d.shape[5]), d.dst_stride[0], d.dst_stride[1],             \
        d.dst_stride[2], d.dst_stride[3], d.dst_stride[4], d.dst_stride[5], d.src_stride[0], d.src_stride[1], d.src_stride[2], d.src_stride[3], \
        d.src_stride[4], d.src_stride[5], arg_pair(d.by_shape[0]), arg_pair(d.by_shape[1]), arg_pair(d.by_shape[2]), arg_pair(d.by_shape[3]), arg_pair(d.by_shape[4]),   \
        arg_pair(d.by_shape[5])
static_assert(kRearrangeMaxDims == 6, "ARGS_OF_DIMS lists six dimensions");

// The access unit: the widest of 16, 8, 4, 2, 1 bytes that divides the row
// length, every stride and both base addresses.
template<int BYTES> struct Unit;
template<> struct Unit<16> { typedef u32x4 type; };
template<> struct Unit<8> { typedef uint64_t type; };
template<> struct Unit<4> { typedef uint32_t type; };
template<> struct Unit<2> { typedef uint16_t type; };
template<> struct Unit<1> { typedef uint8_t type; };

// ANY: rows of at least 16 bytes whose length, strides or bases are no multiples of 16.  The row still moves in
// 16-byte units, at whatever byte boundary they lie on (gfx950 serves such accesses, at a fraction of the
// aligned rate), and the last unit of a row is the row's last 16 bytes, overlapping the one before it: a
// copy may write a byte twice.  bf16 [8192, 64, 127] out of [8192, 80, 127]: 141 us in 2-byte units.
typedef u32x4 __attribute__((aligned(1))) u32x4_bytes;
__device__ __forceinline__ uint32_t unit_offset_any(uint32_t col, uint32_t last_offset) {
    const uint32_t at = col * 16;
    return at < last_offset ? at : last_offset;
}

// blockIdx.y walks the rows, blockIdx.x the units of a row: rows of at least a
// wavefront of units.  The row's offsets are found by splitting the row number
// by the merged outer extents - once per workgroup row, on the scalar unit,
// since the row number is uniform, and by multiplication (see FastDiv).
// BUFST (16-byte units, large outputs): stores are written through L2 as
// buffer stores relative to the start of the destination row (see StreamOut).
template<int BYTES, bool BUFST, int LANES, bool ANY = false>
__global__ __launch_bounds__(LANES) void rearrange_rows(uint8_t *dst, const uint8_t *src, OuterDims d, uint64_t rows, uint32_t units_per_row,
                                                        uint32_t last_offset) {
    typedef typename Unit<BYTES>::type U;
    static_assert(!ANY || (BYTES == 16 && !BUFST), "ANY: 16-byte units at any boundary, plain stores");
    // every argument up front (see AMD_ARGS_NOW; the number of rows to step by is not needed before the first load is out)
    AMD_ARGS_NOW(dst, src, rows, units_per_row, last_offset, ARGS_OF_DIMS(d));
    const uint32_t col = blockIdx.x * LANES + threadIdx.x;
    if (col >= units_per_row) return;
    for (uint64_t r = blockIdx.y; r < rows; r += gridDim.y) {
        int64_t od = 0, os = 0;
        uint32_t rest = static_cast<uint32_t>(r);// fewer than 2^31 rows (the host sends more to rearrange_flat): see FastDiv
#pragma unroll
        for (int k = 0; k < kRearrangeMaxDims; ++k) {
            if (k < d.ndim) {
                const uint32_t q = fast_quotient(rest, d.by_shape[k]);
                const uint32_t i = rest - q * d.shape[k];
                rest = q;
                od += static_cast<int64_t>(i) * d.dst_stride[k];
                os += static_cast<int64_t>(i) * d.src_stride[k];
            }
        }
        if constexpr (ANY) {
            const uint32_t at = unit_offset_any(col, last_offset);
            *reinterpret_cast<u32x4_bytes *>(dst + od + at) = *reinterpret_cast<const u32x4_bytes *>(src + os + at);
        } else {
            const U v = __builtin_nontemporal_load(reinterpret_cast<const U *>(src + os) + col);
            if constexpr (BUFST) {
                StreamOut<true>(dst + od).st16(col * 16, v);
            } else {
                __builtin_nontemporal_store(v, reinterpret_cast<U *>(dst + od) + col);
            }
        }
    }
}

// Short rows: one lane per unit over the flat (row, unit) space, one unit per
// lane.  Idx is 32-bit when the unit count
// allows, which makes the divisions cheap.  BUFST (16-byte units only): the
// whole destination lies within 4 GiB of its base and no stride is negative,
// so stores go out as buffer stores relative to the base (see StreamOut).
template<int BYTES, typename Idx, bool BUFST, bool FAST, bool ANY = false>
__global__ __launch_bounds__(Lanes<BYTES>::value) void rearrange_flat(uint8_t *dst, const uint8_t *src, OuterDims d, uint64_t total_units, Idx units_per_row,
                                                                    FastDiv by_row, uint32_t last_offset) {
    typedef typename Unit<BYTES>::type U;
    static_assert(!ANY || (BYTES == 16 && !BUFST), "ANY: 16-byte units at any boundary, plain stores");
    AMD_ARGS_NOW(dst, src, total_units, units_per_row, arg_pair(by_row), last_offset, gridDim.x, ARGS_OF_DIMS(d));
    // one pass for anything a single launch can span (2^32 work-items); the loop covers the rest
    const uint64_t step = static_cast<uint64_t>(gridDim.x) * Lanes<BYTES>::value;
    for (uint64_t idx64 = static_cast<uint64_t>(blockIdx.x) * Lanes<BYTES>::value + threadIdx.x; idx64 < total_units; idx64 += step) {
        const Idx idx = static_cast<Idx>(idx64);
        Idx rest, col;
        int64_t od = 0, os = 0;
        if constexpr (FAST) {// fewer than 2^31 units in all: multiplications instead of divisions
            static_assert(sizeof(Idx) == 4, "FAST numbers units with 32 bits");
            rest = fast_quotient(idx, by_row);
            col = idx - rest * units_per_row;
#pragma unroll
            for (int k = 0; k < kRearrangeMaxDims; ++k) {
                if (k < d.ndim) {
                    const uint32_t q = fast_quotient(rest, d.by_shape[k]);
                    const uint32_t i = rest - q * d.shape[k];
                    rest = q;
                    od += static_cast<int64_t>(i) * d.dst_stride[k];
                    os += static_cast<int64_t>(i) * d.src_stride[k];
                }
            }
        } else {
            rest = idx / units_per_row;
            col = idx - rest * units_per_row;
#pragma unroll
            for (int k = 0; k < kRearrangeMaxDims; ++k) {
                if (k < d.ndim) {
                    const Idx ext = static_cast<Idx>(d.shape[k]);
                    const Idx q = rest / ext;
                    const Idx i = rest - q * ext;
                    rest = q;
                    od += static_cast<int64_t>(i) * d.dst_stride[k];
                    os += static_cast<int64_t>(i) * d.src_stride[k];
                }
            }
        }
        if constexpr (ANY) {
            const uint32_t at = unit_offset_any(static_cast<uint32_t>(col), last_offset);
            *reinterpret_cast<u32x4_bytes *>(dst + od + at) = *reinterpret_cast<const u32x4_bytes *>(src + os + at);
        } else {
            const U v = __builtin_nontemporal_load(reinterpret_cast<const U *>(src + os) + col);
            if constexpr (BUFST) {
                StreamOut<true>(dst).st16(static_cast<uint32_t>(od) + static_cast<uint32_t>(col) * 16, v);
            } else {
                __builtin_nontemporal_store(v, reinterpret_cast<U *>(dst + od) + col);
            }
        }
    }
}

template<int BYTES, bool ANY = false>
void launch(const RearrangeAmdDescriptor &desc, const OuterDims &d, void *dst, const void *src, hipStream_t stream) {
    auto *pd = static_cast<uint8_t *>(dst);
    auto *ps = static_cast<const uint8_t *>(src);
    const uint64_t upr = ANY ? ceil_div(desc.row_bytes, BYTES) : desc.row_bytes / BYTES;
    const uint32_t last_offset = ANY ? static_cast<uint32_t>(desc.row_bytes - 16) : 0;// ANY: rows of 16 bytes to 4 GiB
    constexpr int kBlock = Lanes<BYTES>::value;
    const bool large = desc.rows * desc.row_bytes >= kWriteThroughBytes;// worth writing through L2
    // where the destination ends, in bytes from its base, when no stride is negative
    bool forward = true;
    uint64_t dst_span = desc.row_bytes;
    for (int k = 0; k < d.ndim; ++k) {
        forward = forward && d.dst_stride[k] >= 0;
        dst_span += (d.shape[k] - 1) * static_cast<uint64_t>(d.dst_stride[k] >= 0 ? d.dst_stride[k] : 0);
    }
    // Rows of fewer than 1024 units: single-wavefront tiles over the flat (row, unit) space, split by
    // multiplication, measure the same or better than a 2-D grid of 128- or 256-lane row workgroups once the
    // copy is large (bf16 rows out of a wider buffer, us: 64 units per row 21.4 against 29.6, 96 units 31.1
    // against 34.0, 192 units 31.2 against 32.1, 384 units 31.6 against 32.6, 512 units 22.2 against 22.7,
    // 352 units 16.2 both); a small copy of few rows is the exception (8192 rows of 128 units, 16 MiB: 9.5
    // against 8.8), so rows of at least two wavefronts keep the row workgroups below 32 MiB.
    const uint64_t units = desc.rows * upr;
    const bool tiles = BYTES == 16 && units < kFastDivLimit && (upr < 2 * kWave || (upr < 16 * kWave && units * BYTES >= (32ull << 20)));
    if (upr >= kWave && upr < (1ull << 31) && !tiles && desc.rows < kFastDivLimit) {
        // A 2-D grid of single-wavefront workgroups needs at least 16 of them per
        // row.  Measured on MI355X with 128 MiB of fp16 rows: 16 KiB rows 41.3 us
        // with 64 lanes and 42.1 us with 256; 8 KiB rows (8 wavefronts each) 57.5
        // against 42.1 us, 2 KiB rows 61.0 against 46.3 us.
        const bool wave_rows = kBlock == kWave && upr >= 16 * kWave;
        // Rows that fill 128-lane workgroups better than 256-lane ones get those: 128 MiB of bf16 rows out
        // of a buffer twice as wide, 2816 elements per row (352 units) 43.3 us against 51.5 us, 3072 per row
        // 42.8 against 50.0, 6912 per row 42.7 against 45.1; nothing between them where both fit equally.
        const bool half = !wave_rows && ceil_div(upr, 128) * 128 < ceil_div(upr, 256) * 256;
        const int lanes = wave_rows ? kWave : (half ? 128 : 256);
        const dim3 grid(static_cast<unsigned>(ceil_div(upr, lanes)), static_cast<unsigned>(desc.rows < 65535 ? desc.rows : 65535));
        const bool bufst = BYTES == 16 && !ANY && large && desc.row_bytes < (1ull << 32);
        const uint32_t upr32 = static_cast<uint32_t>(upr);
#define REARRANGE_ROWS_OF(LANES)                                                                                           \
    do {                                                                                                                   \
        if (bufst) rearrange_rows<BYTES, BYTES == 16 && !ANY, LANES, ANY><<<grid, LANES, 0, stream>>>(pd, ps, d, desc.rows, upr32, last_offset); \
        else rearrange_rows<BYTES, false, LANES, ANY><<<grid, LANES, 0, stream>>>(pd, ps, d, desc.rows, upr32, last_offset); \
    } while (0)
        if constexpr (BYTES == 16) {
            if (wave_rows) {
                REARRANGE_ROWS_OF(kWave);
                return;
            }
        }
        if (half) REARRANGE_ROWS_OF(128);
        else REARRANGE_ROWS_OF(256);
#undef REARRANGE_ROWS_OF
    } else {// short rows; or more rows, or a longer row, than 32 bits number (divisions, 64-bit)
        const uint64_t total = desc.rows * upr;
        const uint64_t want = ceil_div(total, kBlock);
        const uint64_t blocks = want < max_grid_1d(kBlock) ? want : max_grid_1d(kBlock);
        const unsigned grid = static_cast<unsigned>(blocks);
        const bool bufst = BYTES == 16 && !ANY && large && forward && dst_span < (1ull << 32);
        if (total < kFastDivLimit) {
            const FastDiv by_row = fast_div(static_cast<uint32_t>(upr));
            if (bufst) rearrange_flat<BYTES, uint32_t, BYTES == 16 && !ANY, true, ANY><<<grid, kBlock, 0, stream>>>(pd, ps, d, total, static_cast<uint32_t>(upr), by_row, last_offset);
            else rearrange_flat<BYTES, uint32_t, false, true, ANY><<<grid, kBlock, 0, stream>>>(pd, ps, d, total, static_cast<uint32_t>(upr), by_row, last_offset);
        } else {
            rearrange_flat<BYTES, uint64_t, false, false, ANY><<<grid, kBlock, 0, stream>>>(pd, ps, d, total, upr, FastDiv{}, last_offset);
        }
    }
}

}// namespace

// Stage 4 of Rearrange.
infiniopStatus_t amdRearrange(RearrangeAmdDescriptor_t desc, void *dst, void const *src, void *stream) {
    if (desc->rows == 0 || desc->row_bytes == 0) {
        return STATUS_SUCCESS;
    }
    if (dst == nullptr || src == nullptr) {
        return STATUS_BAD_PARAM;
    }
    OuterDims d;
    d.ndim = desc->ndim;
    uint64_t align = desc->row_bytes | reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src);
    for (int k = 0; k < kRearrangeMaxDims; ++k) {
        const bool used = k < desc->ndim;
        if (used && desc->shape[k] >= (1ull << 32)) {
            return STATUS_BAD_TENSOR_SHAPE;
        }
        d.shape[k] = used ? static_cast<uint32_t>(desc->shape[k]) : 1;
        d.dst_stride[k] = used ? desc->dst_stride[k] : 0;
        d.src_stride[k] = used ? desc->src_stride[k] : 0;
        d.by_shape[k] = fast_div(d.shape[k] < kFastDivLimit ? d.shape[k] : 1);// an extent beyond the limit means more rows than the FAST kernels take
        if (used) align |= static_cast<uint64_t>(desc->dst_stride[k]) | static_cast<uint64_t>(desc->src_stride[k]);
    }
    AMD_CHECK_HIP(hipSetDevice(desc->device_id), STATUS_BAD_DEVICE);
    hipStream_t s = static_cast<hipStream_t>(stream);
    // Rows that all start and end on 128-byte boundaries stream past the caches; rows that share lines with their
    // neighbours go through them, in 16-byte units at whatever boundary (bf16 [8192, 64, hd] out of [8192, 80, hd],
    // us, streaming hints against none: hd 104  78.7 / 37.7, hd 120  77.8 / 56.5, hd 200  123 / 102, hd 504  245 / 241;
    // [16384, 4104] out of a pitch of 4120  47.5 / 46.7).
    const bool any_ok = desc->row_bytes >= 16 && desc->row_bytes < (1ull << 32);
    if (align % 16 == 0 && (align % 128 == 0 || !any_ok)) launch<16>(*desc, d, dst, src, s);
    else if (any_ok) launch<16, true>(*desc, d, dst, src, s);
    else if (align % 8 == 0) launch<8>(*desc, d, dst, src, s);
    else if (align % 4 == 0) launch<4>(*desc, d, dst, src, s);
    else if (align % 2 == 0) launch<2>(*desc, d, dst, src, s);
    else launch<1>(*desc, d, dst, src, s);
    AMD_CHECK_HIP(hipGetLastError(), STATUS_EXECUTION_FAILED);
    return STATUS_SUCCESS;
}
