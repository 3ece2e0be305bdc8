// gfx950 kernels for Add and their launch.
//
// Arithmetic contract (reference src/ops/add/cpu/add_cpu.cc:72-89): fp16
// operands are widened to fp32, added in fp32 and narrowed with the reference's
// truncating conversion, bit for bit; fp32 is one IEEE add; bf16 (extension)
// is widened, added in fp32 and rounded to nearest even.
//
// The operation moves 3 bytes per byte of output and computes almost nothing,
// so everything here is about keeping HBM busy: 16 bytes per lane per access,
// memory walked in address order, non-temporal hints on data that is touched
// once.
#include "../../../devices/amd/kernel_amd.h"
#include "add_amd.h"

namespace {

using namespace amd;

// Launch shape of the flat kernel, chosen by measurement on MI355X with a
// stand-alone c = a + b over 3 x 128 MiB: workgroups of one wavefront with one
// 16-byte access per lane per operand, one workgroup per KiB of output, take
// 61.4 us; 128 lanes 61.6; 256 lanes 63.1-63.7; 2 or 4 accesses per lane
// 62.7-65.8; workgroups that loop over tiles (16-64 per compute unit)
// 65.4-69.6.  The general broadcast kernels keep 256 lanes: with an operand
// that is re-read through the caches, [8192, 4096] fp16 plus a [4096] row takes
// 24.4 us that way and 31-32 us as a 2-D grid of single-wavefront workgroups
// (only 8 of them per row); the same workgroups numbered along one grid axis
// are the form add_rowvec_tiles below takes for that shape.
constexpr int kBlock = 256;// lanes per workgroup of the broadcast and element-wise kernels

// ---- per-type arithmetic on one 128-bit word ---------------------------------
template<typename T>
struct Add16 {
    typedef uint16_t scalar;
    static constexpr int kPerVec = 8;
    __device__ static __forceinline__ u32x4 vec(u32x4 a, u32x4 b) {
        float x[8], y[8];
        widen8<T>(a, x);
        widen8<T>(b, y);
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] += y[i];
        return narrow8<T>(x);
    }
    __device__ static __forceinline__ scalar one(scalar a, scalar b) {
        return T::narrow1(T::one(a) + T::one(b));
    }
    __device__ static __forceinline__ u32x4 splat(scalar s) {
        const uint32_t w = static_cast<uint32_t>(s) * 0x00010001u;
        return u32x4{w, w, w, w};
    }
};

struct Add32 {
    typedef float scalar;
    static constexpr int kPerVec = 4;
    __device__ static __forceinline__ u32x4 vec(u32x4 a, u32x4 b) {
        const f32x4 r = __builtin_bit_cast(f32x4, a) + __builtin_bit_cast(f32x4, b);
        return __builtin_bit_cast(u32x4, r);
    }
    __device__ static __forceinline__ scalar one(scalar a, scalar b) { return a + b; }
    __device__ static __forceinline__ u32x4 splat(scalar s) {
        const uint32_t w = __float_as_uint(s);
        return u32x4{w, w, w, w};
    }
};

// ---- no broadcasting: c[i] = a[i] + b[i] over a flat range -------------------
// One wavefront per workgroup, one vector per lane, one workgroup per KiB: the
// dispatcher hands out consecutive KiBs in order and every wavefront gives its
// slot back the moment it is done.  (The loop only runs more than once for
// ranges beyond what one launch may span: 2^32 work-items.)
// ANY: the operands do not all start on 16-byte boundaries; the same vectors as 16-byte accesses at whatever
// boundary they lie on ([8192, 4096] fp16 on views one element into their buffers: 44 us; 113 us element by element).
template<typename Op, bool ANY = false>
__global__ __launch_bounds__(kWave) void add_flat_vec(u32x4 *c, const u32x4 *a, const u32x4 *b, uint64_t nvec) {
    AMD_ARGS_NOW(c, a, b, nvec, gridDim.x);
    const uint64_t step = static_cast<uint64_t>(gridDim.x) * kWave;
    for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * kWave + threadIdx.x; i < nvec; i += step) {
        if constexpr (ANY) {
            st16_any(c + i, Op::vec(ld16_any(a + i), ld16_any(b + i)));
        } else {
            const u32x4 va = ld16_stream(a + i);
            const u32x4 vb = ld16_stream(b + i);
            st16_stream(c + i, Op::vec(va, vb));
        }
    }
}

// Element-at-a-time form for ranges that are not 16-byte aligned and for the
// few elements left after the last whole vector.
template<typename Op>
__global__ __launch_bounds__(kBlock) void add_flat_scalar(typename Op::scalar *c, const typename Op::scalar *a,
                                                          const typename Op::scalar *b, uint64_t first, uint64_t n) {
    AMD_ARGS_NOW(c, a, b, first, n, gridDim.x);
    const uint64_t step = static_cast<uint64_t>(gridDim.x) * kBlock;
    for (uint64_t i = first + static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += step) {
        c[i] = Op::one(a[i], b[i]);
    }
}

// ---- broadcasting -------------------------------------------------------------
// Merged dimensions, innermost first.  c is flat; an operand's offset is the
// sum of index*stride over the dimensions.
struct BcastDims {
    int ndim;
    uint64_t shape[kAddMaxDims];
    int64_t a_stride[kAddMaxDims];
    int64_t b_stride[kAddMaxDims];
    FastDiv by_shape[kAddMaxDims];// division by shape[k], k >= 1, for the kernels that number positions with 32 bits
};

// The innermost four dimensions of a BcastDims argument as operands of AMD_ARGS_NOW (what nearly every
// broadcast has after merging; the rest are fetched when a fifth dimension is met).
#define ARGS_OF_BCAST(d)                                                                                                               \
    d.ndim, d.shape[0], d.shape[1], d.shape[2], d.shape[3], d.a_stride[0], d.a_stride[1], d.a_stride[2], d.a_stride[3], d.b_stride[0], \
        d.b_stride[1], d.b_stride[2], d.b_stride[3], arg_pair(d.by_shape[1]), arg_pair(d.by_shape[2]), arg_pair(d.by_shape[3])

// Split a flat position (in units of `first_extent` along the innermost
// dimension) into operand offsets.  Idx is 32-bit when every quantity is
// below 2^31, and the divisions are then multiplications (see FastDiv).
template<typename Idx>
__device__ __forceinline__ void bcast_offsets(const BcastDims &d, Idx pos, Idx inner_extent, FastDiv by_inner, int64_t inner_scale,
                                              int64_t &off_a, int64_t &off_b) {
    constexpr bool FAST = sizeof(Idx) == 4;
    Idx rest;
    if constexpr (FAST) rest = fast_quotient(static_cast<uint32_t>(pos), by_inner);
    else rest = pos / inner_extent;
    const Idx in = pos - rest * inner_extent;
    off_a = static_cast<int64_t>(in) * inner_scale * d.a_stride[0];
    off_b = static_cast<int64_t>(in) * inner_scale * d.b_stride[0];
#pragma unroll
    for (int k = 1; k < kAddMaxDims; ++k) {
        if (k < d.ndim) {
            const Idx ext = static_cast<Idx>(d.shape[k]);
            Idx q;
            if constexpr (FAST) q = fast_quotient(static_cast<uint32_t>(rest), d.by_shape[k]);
            else q = rest / ext;
            const Idx i = rest - q * ext;
            rest = q;
            off_a += static_cast<int64_t>(i) * d.a_stride[k];
            off_b += static_cast<int64_t>(i) * d.b_stride[k];
        }
    }
}

// How an operand is addressed by the vector form.
//   kFull : it has c's full shape, so its offset is c's flat offset; it is
//           touched once and streams past the caches like c.
//   kRuns : stride 1 along the innermost dimension but broadcast along some
//           outer one; 128-bit loads through the caches, because every
//           element is wanted again by other lanes.
//   kStill: broadcast along the innermost dimension; one element, replicated.
enum OperandMode { kFull = 0, kRuns = 1, kStill = 2 };

template<typename Op, int MODE>
__device__ __forceinline__ u32x4 fetch_operand(const typename Op::scalar *p, uint64_t flat_vec, int64_t offset) {
    if constexpr (MODE == kFull) return ld16_stream(p + flat_vec * Op::kPerVec);
    else if constexpr (MODE == kRuns) return ld16(p + offset);
    else return Op::splat(p[offset]);
}

// Vector form: the innermost merged dimension is a multiple of the vector
// width and each operand either runs along it with stride 1 (128-bit load) or
// stands still (one element, replicated).
template<typename Op, typename Idx, int A_MODE, int B_MODE>
__global__ __launch_bounds__(kBlock) void add_bcast_vec(u32x4 *c, const typename Op::scalar *a,
                                                        const typename Op::scalar *b, BcastDims d, uint64_t nvec, FastDiv by_inner) {
    AMD_ARGS_NOW(c, a, b, nvec, gridDim.x, arg_pair(by_inner), ARGS_OF_BCAST(d));
    const Idx inner_vecs = static_cast<Idx>(d.shape[0] / Op::kPerVec);
    const uint64_t step = static_cast<uint64_t>(gridDim.x) * kBlock;
    for (uint64_t v = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x; v < nvec; v += step) {
        int64_t oa = 0, ob = 0;
        bcast_offsets<Idx>(d, static_cast<Idx>(v), inner_vecs, by_inner, Op::kPerVec, oa, ob);
        const u32x4 va = fetch_operand<Op, A_MODE>(a, v, oa);
        const u32x4 vb = fetch_operand<Op, B_MODE>(b, v, ob);
        st16_stream(c + v, Op::vec(va, vb));
    }
}

// Two merged dimensions (an outer one of `rows` steps and the vectorised inner
// one): blockIdx.y walks the outer dimension, so no lane divides anything.
// This is the residual-add shape - a [rows, width] tensor plus a [width] row,
// or any pair of operands that broadcast along one of two merged dimensions.
// With one operand re-read from the caches this is a one-read-one-write
// stream: THROUGH writes large outputs through L2 (see StreamOut; 24.4 us
// against 24.9 us at [8192, 4096] fp16 plus a [4096] row).
template<typename Op, int A_MODE, int B_MODE, bool THROUGH>
__global__ __launch_bounds__(kBlock) void add_bcast_rows(u32x4 *c, const typename Op::scalar *a, const typename Op::scalar *b,
                                                         uint64_t rows, uint32_t inner_vecs,
                                                         int64_t a_outer, int64_t a_inner, int64_t b_outer, int64_t b_inner) {
    AMD_ARGS_NOW(c, a, b, rows, inner_vecs, a_outer, a_inner, b_outer, b_inner, gridDim.y);
    const uint32_t iv = blockIdx.x * kBlock + threadIdx.x;
    if (iv >= inner_vecs) return;
    for (uint64_t r = blockIdx.y; r < rows; r += gridDim.y) {
        const uint64_t flat = r * inner_vecs + iv;
        const int64_t oa = static_cast<int64_t>(r) * a_outer + static_cast<int64_t>(iv) * Op::kPerVec * a_inner;
        const int64_t ob = static_cast<int64_t>(r) * b_outer + static_cast<int64_t>(iv) * Op::kPerVec * b_inner;
        const u32x4 va = fetch_operand<Op, A_MODE>(a, flat, oa);
        const u32x4 vb = fetch_operand<Op, B_MODE>(b, flat, ob);
        if constexpr (THROUGH) {
            StreamOut<true>(c + r * inner_vecs).st16(iv * 16, Op::vec(va, vb));
        } else {
            st16_stream(c + flat, Op::vec(va, vb));
        }
    }
}

// ---- a whole tensor plus one row:  c[r, :] = full[r, :] + vec[:] ---------------
// The residual-plus-bias shape.  It is the flat kernel's launch shape -
// workgroups of one wavefront, one vector per lane, tiles in address order -
// with the row's tile found from the workgroup number; the row itself (a few
// KiB) comes through the caches.  One read and one write per output byte, so
// large outputs are written through L2 (THROUGH, see StreamOut).  Measured on
// MI355X, [8192, 4096] fp16 plus a [4096] row: 23.2 us, against 24.5 us for a
// 2-D grid of 256-lane workgroups (add_bcast_rows), 23.6-25.5 us for workgroups
// that keep their piece of the row in registers and walk down the rows, and
// 23.6-24.0 us for single-wavefront workgroups that own 2 or 4 rows of a tile;
// [8192, 8192] bf16: 40.9 against 42.7 us.
// SWAP says the row is operand a (the sum is formed as a + b either way).
template<typename Op, bool SWAP, bool THROUGH>
__global__ __launch_bounds__(kWave) void add_rowvec_tiles(u32x4 *c, const u32x4 *full, const u32x4 *vec, uint32_t tiles_per_row, FastDiv by_row) {
    AMD_ARGS_NOW(c, full, vec, tiles_per_row, by_row.mul, by_row.shift);
    const uint32_t tile = blockIdx.x;// one tile per workgroup: the host takes this form only for what one launch spans
    const uint32_t ct = tile - fast_quotient(tile, by_row) * tiles_per_row;// tile % tiles_per_row
    const u32x4 vv = ld16(vec + ct * kWave + threadIdx.x);
    const u32x4 vf = ld16_stream(full + static_cast<uint64_t>(tile) * kWave + threadIdx.x);
    const u32x4 r = SWAP ? Op::vec(vv, vf) : Op::vec(vf, vv);
    if constexpr (THROUGH) StreamOut<true>(c + static_cast<uint64_t>(tile) * kWave).st16(threadIdx.x * 16, r);
    else st16_stream(c + static_cast<uint64_t>(tile) * kWave + threadIdx.x, r);
}

// The same tiles for a whole tensor plus an operand that runs along the
// innermost dimension and is broadcast along some of the outer ones (a bias
// per batch entry [B, 1, H] onto [B, S, H], an attention mask [B, 1, S, S] onto
// [B, H, S, S]).  A tile of 64 vectors lies inside one innermost row, so where
// the broadcast operand's piece starts is wavefront-uniform: the outer indices
// come from scalar multiply-and-shift divisions (see FastDiv) and the lanes
// only add their own 16 bytes.  Measured on MI355X, fp16: [32, 1024, 4096] plus
// [32, 1, 4096] 79.7 us (84 %) against 91.5 us with 256-lane workgroups that
// split every vector's index by division (add_bcast_vec); [8, 32, 1024, 1024]
// plus a mask [8, 1, 1024, 1024] 172 against 187 us.
struct TileDims {
    int ndim;                         // merged dimensions, innermost first; [0] is covered by the tiles themselves
    uint32_t shape[kAddMaxDims];
    int64_t stride[kAddMaxDims];      // of the broadcast operand, in elements
    FastDiv by_shape[kAddMaxDims];
};
#define ARGS_OF_TILES(d)                                                                                                                      \
    d.ndim, arg_pair(d.shape[1], d.shape[2]), arg_pair(d.shape[3], d.shape[4]), arg_pair(d.shape[5], d.shape[6]), d.shape[7], d.stride[1],    \
        d.stride[2], d.stride[3], d.stride[4], d.stride[5], d.stride[6], d.stride[7], arg_pair(d.by_shape[1]), arg_pair(d.by_shape[2]),       \
        arg_pair(d.by_shape[3]), arg_pair(d.by_shape[4]), arg_pair(d.by_shape[5]), arg_pair(d.by_shape[6]), arg_pair(d.by_shape[7])
template<typename Op, bool SWAP, bool THROUGH>
__global__ __launch_bounds__(kWave) void add_bcast_tiles(u32x4 *c, const u32x4 *full, const typename Op::scalar *runs, uint32_t tiles_per_row,
                                                         FastDiv by_row, TileDims d) {
    AMD_ARGS_NOW(c, full, runs, tiles_per_row, arg_pair(by_row), ARGS_OF_TILES(d));
    const uint32_t tile = blockIdx.x;// one tile per workgroup: the host takes this form only for what one launch spans
    uint32_t rest = fast_quotient(tile, by_row);
    int64_t off = static_cast<int64_t>(tile - rest * tiles_per_row) * (kWave * Op::kPerVec);
#pragma unroll
    for (int k = 1; k < kAddMaxDims; ++k) {
        if (k < d.ndim) {
            const uint32_t q = fast_quotient(rest, d.by_shape[k]);
            off += static_cast<int64_t>(rest - q * d.shape[k]) * d.stride[k];
            rest = q;
        }
    }
    const u32x4 vv = ld16(runs + off + threadIdx.x * Op::kPerVec);
    const u32x4 vf = ld16_stream(full + static_cast<uint64_t>(tile) * kWave + threadIdx.x);
    const u32x4 r = SWAP ? Op::vec(vv, vf) : Op::vec(vf, vv);
    if constexpr (THROUGH) StreamOut<true>(c + static_cast<uint64_t>(tile) * kWave).st16(threadIdx.x * 16, r);
    else st16_stream(c + static_cast<uint64_t>(tile) * kWave + threadIdx.x, r);
}

// Any strides, any alignment.  A lane takes kPerVec consecutive elements of c:
// when they lie in one run of the innermost dimension and both operands either
// run along it or stand still, they move as 16 bytes at whatever boundary they
// lie on (which gfx950 serves at a fraction of the aligned rate); otherwise
// element by element.  [8192, 4095] fp16 plus a row of 4095: 77 us with element accesses only.
template<typename Op, typename Idx>
__global__ __launch_bounds__(kBlock) void add_bcast_scalar(typename Op::scalar *c, const typename Op::scalar *a,
                                                           const typename Op::scalar *b, BcastDims d, uint64_t n, FastDiv by_inner) {
    AMD_ARGS_NOW(c, a, b, n, gridDim.x, arg_pair(by_inner), ARGS_OF_BCAST(d));
    constexpr uint64_t W = Op::kPerVec;
    const Idx inner = static_cast<Idx>(d.shape[0]);
    const bool unit = (d.a_stride[0] == 0 || d.a_stride[0] == 1) && (d.b_stride[0] == 0 || d.b_stride[0] == 1);
    const uint64_t groups = (n + W - 1) / W;
    const uint64_t step = static_cast<uint64_t>(gridDim.x) * kBlock;
    for (uint64_t g = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x; g < groups; g += step) {
        const uint64_t i0 = g * W;
        Idx outer;
        if constexpr (sizeof(Idx) == 4) outer = fast_quotient(static_cast<uint32_t>(i0), by_inner);
        else outer = static_cast<Idx>(i0) / inner;
        const uint64_t in = i0 - static_cast<uint64_t>(outer) * inner;
        if (unit && in + W <= inner && i0 + W <= n) {
            int64_t oa, ob;
            bcast_offsets<Idx>(d, static_cast<Idx>(i0), inner, by_inner, 1, oa, ob);
            const u32x4 va = d.a_stride[0] == 1 ? ld16_any(a + oa) : Op::splat(a[oa]);
            const u32x4 vb = d.b_stride[0] == 1 ? ld16_any(b + ob) : Op::splat(b[ob]);
            st16_any(c + i0, Op::vec(va, vb));
        } else {
            for (uint64_t i = i0; i < i0 + W && i < n; ++i) {
                int64_t oa, ob;
                bcast_offsets<Idx>(d, static_cast<Idx>(i), inner, by_inner, 1, oa, ob);
                c[i] = Op::one(a[oa], b[ob]);
            }
        }
    }
}

// ---- launch -------------------------------------------------------------------
inline unsigned grid_for(uint64_t work_items, uint64_t per_block, int cu_count, int blocks_per_cu) {
    const uint64_t want = ceil_div(work_items, per_block);
    const uint64_t cap = blocks_per_cu > 0 ? static_cast<uint64_t>(cu_count) * blocks_per_cu : want;
    uint64_t g = want < cap ? want : cap;
    g = g < max_grid_1d(static_cast<unsigned>(per_block)) ? g : max_grid_1d(static_cast<unsigned>(per_block));// the kernels stride over the rest
    return static_cast<unsigned>(g == 0 ? 1 : g);
}

template<typename Op>
infiniopStatus_t launch_add(const AddAmdDescriptor &desc, void *c, const void *a, const void *b, hipStream_t stream) {
    typedef typename Op::scalar S;
    const uint64_t n = desc.total;
    const int cus = desc.cu_count;

    if (desc.flat) {
        const uint64_t nvec = n / Op::kPerVec;
        if (nvec > 0) {
            const unsigned grid = grid_for(nvec, kWave, cus, 0);
            if (aligned16(c) && aligned16(a) && aligned16(b)) {
                add_flat_vec<Op><<<grid, kWave, 0, stream>>>(static_cast<u32x4 *>(c), static_cast<const u32x4 *>(a),
                                                              static_cast<const u32x4 *>(b), nvec);
            } else {
                add_flat_vec<Op, true><<<grid, kWave, 0, stream>>>(static_cast<u32x4 *>(c), static_cast<const u32x4 *>(a),
                                                                    static_cast<const u32x4 *>(b), nvec);
            }
        }
        const uint64_t done = nvec * Op::kPerVec;
        if (done < n) {
            const unsigned grid = grid_for(n - done, kBlock, cus, 32);
            add_flat_scalar<Op><<<grid, kBlock, 0, stream>>>(static_cast<S *>(c), static_cast<const S *>(a),
                                                             static_cast<const S *>(b), done, n);
        }
        return STATUS_SUCCESS;
    }

    BcastDims d;
    d.ndim = desc.ndim;
    bool small = n < (1ull << 31);
    for (int k = 0; k < kAddMaxDims; ++k) {
        d.shape[k] = k < desc.ndim ? desc.shape[k] : 1;
        d.a_stride[k] = k < desc.ndim ? desc.a_stride[k] : 0;
        d.b_stride[k] = k < desc.ndim ? desc.b_stride[k] : 0;
        d.by_shape[k] = fast_div(small ? static_cast<uint32_t>(d.shape[k]) : 1);
    }

    // 128-bit access needs: inner extent a multiple of the vector width, inner
    // strides 0 or 1, and every address a running operand can reach 16-byte
    // aligned (base pointer and all outer strides multiples of the width).
    const int64_t w = Op::kPerVec;
    bool vec_ok = desc.shape[0] % w == 0 && aligned16(c) &&
                  (desc.a_stride[0] == 0 || desc.a_stride[0] == 1) && (desc.b_stride[0] == 0 || desc.b_stride[0] == 1);
    const bool a_runs = desc.a_stride[0] == 1, b_runs = desc.b_stride[0] == 1;
    for (int k = 1; k < desc.ndim && vec_ok; ++k) {
        if (a_runs && desc.a_stride[k] % w != 0) vec_ok = false;
        if (b_runs && desc.b_stride[k] % w != 0) vec_ok = false;
    }
    if (a_runs && !aligned16(a)) vec_ok = false;
    if (b_runs && !aligned16(b)) vec_ok = false;

    if (vec_ok) {
        const uint64_t nvec = n / w;
        const unsigned grid = grid_for(nvec, kBlock, cus, 64);
        auto mode_of = [&](const int64_t *stride) {
            if (stride[0] == 0) return static_cast<int>(kStill);
            for (int k = 1; k < desc.ndim; ++k)
                if (stride[k] == 0) return static_cast<int>(kRuns);
            return static_cast<int>(kFull);
        };
        const int ma = mode_of(desc.a_stride), mb = mode_of(desc.b_stride);
        auto go = [&](auto kernel) {// (single-wavefront tiles measure 1-3 % slower here: the operand that stands still is a 2-byte load per lane)
            kernel<<<grid, kBlock, 0, stream>>>(static_cast<u32x4 *>(c), static_cast<const S *>(a), static_cast<const S *>(b), d, nvec,
                                                fast_div(small ? static_cast<uint32_t>(desc.shape[0] / w) : 1));
        };
        // rows form: two merged dimensions with at least a wavefront of vectors in the inner one
        const uint64_t inner_vecs = desc.shape[0] / w;
        const bool rows_form = desc.ndim == 2 && inner_vecs >= kWave && inner_vecs < (1ull << 31);
        auto go_rows = [&](auto kernel) {
            const uint64_t rows = desc.shape[1];
            const dim3 g(static_cast<unsigned>(ceil_div(inner_vecs, kBlock)), static_cast<unsigned>(rows < 65535 ? rows : 65535));
            kernel<<<g, kBlock, 0, stream>>>(static_cast<u32x4 *>(c), static_cast<const S *>(a), static_cast<const S *>(b), rows,
                                             static_cast<uint32_t>(inner_vecs), desc.a_stride[1], desc.a_stride[0], desc.b_stride[1], desc.b_stride[0]);
        };
        // one streamed operand and a large output: write through L2
        const bool through = (ma == kFull) != (mb == kFull) && n * sizeof(S) >= kWriteThroughBytes && inner_vecs < (1ull << 28);
        bool launched = false;
        // a whole tensor plus one row whose length is a multiple of a wavefront of vectors
        // (up to what one launch of single-wavefront workgroups spans, 64 GiB of 16-bit output; beyond that the general kernels below)
        if (desc.ndim == 2 && inner_vecs % kWave == 0 && desc.shape[1] * (inner_vecs / kWave) < max_grid_1d(kWave) &&
            ((ma == kFull && mb == kRuns && desc.b_stride[1] == 0) || (ma == kRuns && mb == kFull && desc.a_stride[1] == 0))) {
            const bool swap = ma == kRuns;
            const u32x4 *full = static_cast<const u32x4 *>(swap ? b : a), *vec = static_cast<const u32x4 *>(swap ? a : b);
            u32x4 *pc = static_cast<u32x4 *>(c);
            const uint32_t tpr = static_cast<uint32_t>(inner_vecs / kWave);
            const unsigned g = static_cast<unsigned>(desc.shape[1] * tpr);
            const FastDiv by_row = fast_div(tpr);
            if (swap && through) add_rowvec_tiles<Op, true, true><<<g, kWave, 0, stream>>>(pc, full, vec, tpr, by_row);
            else if (swap) add_rowvec_tiles<Op, true, false><<<g, kWave, 0, stream>>>(pc, full, vec, tpr, by_row);
            else if (through) add_rowvec_tiles<Op, false, true><<<g, kWave, 0, stream>>>(pc, full, vec, tpr, by_row);
            else add_rowvec_tiles<Op, false, false><<<g, kWave, 0, stream>>>(pc, full, vec, tpr, by_row);
            return STATUS_SUCCESS;
        }
        // the same with more outer dimensions (see add_bcast_tiles)
        if (inner_vecs % kWave == 0 && nvec / kWave < max_grid_1d(kWave) && ((ma == kFull && mb == kRuns) || (ma == kRuns && mb == kFull))) {
            const bool swap = ma == kRuns;
            TileDims t;
            t.ndim = desc.ndim;
            bool fits = true;
            for (int k = 0; k < kAddMaxDims; ++k) {
                const bool used = k < desc.ndim;
                fits = fits && (!used || desc.shape[k] < kFastDivLimit);
                t.shape[k] = used ? static_cast<uint32_t>(desc.shape[k]) : 1;
                t.stride[k] = used ? (swap ? desc.a_stride[k] : desc.b_stride[k]) : 0;
                t.by_shape[k] = fast_div(t.shape[k]);
            }
            if (fits) {
                const u32x4 *full = static_cast<const u32x4 *>(swap ? b : a);
                const S *runs = static_cast<const S *>(swap ? a : b);
                u32x4 *pc = static_cast<u32x4 *>(c);
                const uint32_t tpr = static_cast<uint32_t>(inner_vecs / kWave);
                const unsigned g = static_cast<unsigned>(nvec / kWave);
                const FastDiv by_row = fast_div(tpr);
                if (swap && through) add_bcast_tiles<Op, true, true><<<g, kWave, 0, stream>>>(pc, full, runs, tpr, by_row, t);
                else if (swap) add_bcast_tiles<Op, true, false><<<g, kWave, 0, stream>>>(pc, full, runs, tpr, by_row, t);
                else if (through) add_bcast_tiles<Op, false, true><<<g, kWave, 0, stream>>>(pc, full, runs, tpr, by_row, t);
                else add_bcast_tiles<Op, false, false><<<g, kWave, 0, stream>>>(pc, full, runs, tpr, by_row, t);
                return STATUS_SUCCESS;
            }
        }
#define ADD_BCAST_CASE(MA, MB)                                        \
    if (ma == MA && mb == MB) {                                       \
        if (rows_form && through) go_rows(add_bcast_rows<Op, MA, MB, true>);  \
        else if (rows_form) go_rows(add_bcast_rows<Op, MA, MB, false>); \
        else if (small) go(add_bcast_vec<Op, uint32_t, MA, MB>);      \
        else go(add_bcast_vec<Op, uint64_t, MA, MB>);                 \
        launched = true;                                              \
    }
        ADD_BCAST_CASE(kFull, kRuns)
        ADD_BCAST_CASE(kFull, kStill)
        ADD_BCAST_CASE(kRuns, kFull)
        ADD_BCAST_CASE(kRuns, kRuns)
        ADD_BCAST_CASE(kRuns, kStill)
        ADD_BCAST_CASE(kStill, kFull)
        ADD_BCAST_CASE(kStill, kRuns)
        ADD_BCAST_CASE(kStill, kStill)
#undef ADD_BCAST_CASE
        if (launched) return STATUS_SUCCESS;
        // two full operands that did not merge into one flat range cannot reach
        // this point; if a new layout ever does, the element form below handles it
    }
    {
        const unsigned grid = grid_for(ceil_div(n, static_cast<uint64_t>(Op::kPerVec)), kBlock, cus, 0);
        if (small) {
            add_bcast_scalar<Op, uint32_t><<<grid, kBlock, 0, stream>>>(static_cast<S *>(c), static_cast<const S *>(a),
                                                                        static_cast<const S *>(b), d, n, fast_div(static_cast<uint32_t>(desc.shape[0])));
        } else {
            add_bcast_scalar<Op, uint64_t><<<grid, kBlock, 0, stream>>>(static_cast<S *>(c), static_cast<const S *>(a),
                                                                        static_cast<const S *>(b), d, n, FastDiv{});
        }
    }
    return STATUS_SUCCESS;
}

}// namespace

// Stage 4 of Add (reference src/ops/add/cuda/add.cu:104-120 for the NVIDIA
// device): bind the descriptor's GPU, enqueue on the caller's stream, return
// without waiting.
infiniopStatus_t amdAdd(AddAmdDescriptor_t desc, void *c, void const *a, void const *b, void *stream) {
    if (desc->total == 0) {
        return STATUS_SUCCESS;
    }
    if (c == nullptr || a == nullptr || b == nullptr) {
        return STATUS_BAD_PARAM;
    }
    AMD_CHECK_HIP(hipSetDevice(desc->device_id), STATUS_BAD_DEVICE);
    hipStream_t s = static_cast<hipStream_t>(stream);
    infiniopStatus_t st;
    switch (desc->elem) {
        case amd::Elem::F16:
            st = launch_add<Add16<amd::F16Ref>>(*desc, c, a, b, s);
            break;
        case amd::Elem::BF16:
            st = launch_add<Add16<amd::BF16Rne>>(*desc, c, a, b, s);
            break;
        case amd::Elem::F32:
            st = launch_add<Add32>(*desc, c, a, b, s);
            break;
        default:
            return STATUS_BAD_TENSOR_DTYPE;
    }
    AMD_CHECK_HIP(hipGetLastError(), STATUS_EXECUTION_FAILED);
    return st;
}
