// Device code of CausalSoftmax on gfx950 and its launch, one instantiation per element type; the two
// element types are compiled in translation units of their own (causal_softmax_amd.hip, causal_softmax_f16.hip).
// Include from .hip files only.
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
#ifndef INFINIOP_AMD_CAUSAL_SOFTMAX_KERNELS_H
#define INFINIOP_AMD_CAUSAL_SOFTMAX_KERNELS_H

#include "../../../devices/amd/kernel_amd.h"
#include "causal_softmax_amd.h"
#include <algorithm>

// Internal linkage: each including translation unit owns its copies.
namespace causal_softmax_kernels {
namespace {

using namespace amd;

// expf(d) for d <= 0 through the hardware exp2: d * log2(e) is formed as an
// unevaluated sum hi + lo (one fused multiply-add recovers the rounding error
// of the product, a second term carries the rest of log2(e)), exp2 takes hi
// and lo enters as the first-order factor (1 + lo * ln 2).  About 9 VALU slots
// against about 12 for the library routine, and no range checks: the caller
// guarantees -126 <= d <= 0, where everything is finite and normal.
__device__ __forceinline__ float exp_nonpositive(float d) {
    constexpr float kL2e = 1.44269502162933349609375f;    // log2(e) rounded to fp32
    constexpr float kL2eLo = 1.92596299112661746e-8f;     // log2(e) - kL2e
    constexpr float kLn2 = 0.693147182464599609375f;
    const float hi = d * kL2e;
    const float lo = __builtin_fmaf(d, kL2eLo, __builtin_fmaf(d, kL2e, -hi));
    const float e = __builtin_amdgcn_exp2f(hi);
    return __builtin_fmaf(e, lo * kLn2, e);
}
constexpr float kLeanExpLimit = -126.0f;

// The library exponential for the rare arguments outside that range (-inf,
// very long tails, NaN), eight at a time through memory.  Deliberately not
// inlined, and deliberately fed through a small array of its own: a call per
// element inside the kernels would make every value that is live across it
// compete for the few registers a callee preserves, and the common path would
// pay for that with half its occupancy.
__device__ __attribute__((noinline)) void exp_any8(float *v, float mx) {
    for (int e = 0; e < 8; ++e) v[e] = expf(v[e] - mx);
}

// One workgroup of BS lanes per row; lane l owns vectors l, l+BS, ... (NV of
// them, 8 elements each), so total <= 8*BS*NV.  A workgroup takes one row at a
// time and starts the next one only after it has stored the last: that keeps
// the register count low enough for three to five wavefronts per SIMD, and it
// is those other wavefronts that cover a row's load latency and arithmetic.
// (A form that kept the next row's loads in flight needed twice the registers
// and measured 3-30 % slower at every row length from 1024 to 32768 columns.
// Sending only the next row's loads out in front of this row's stores, once
// this row's vectors are dead, took 6-16 more registers and moved rows of
// 1000-16384 columns by -4 to +3 %.)
// Loads are unconditional: a lane whose vector lies in the masked part
// re-reads the row's last kept vector, which the memory pipeline merges into
// one request.  (Leaving out the load instructions that lie wholly in the
// masked part, behind wavefront-uniform branches: -3 to +2 %.)
// RAGGED: rows that do not all start on 128-byte boundaries - the scores of an
// attention over a number of keys that is no multiple of 64 - of at least 16
// elements.  Two things change.
// (1) The vectors are the whole 16-byte aligned ones inside the row (its
// body), as many as the workgroup has room for.  The up to 7 elements in front
// of the first of them and the up to 56 behind the last are taken one each by
// the lanes of the first wavefront, with 2-byte loads and stores, and enter
// the maximum, the sum and the quotients beside those lanes' vectors: about 25
// more vector instructions per row and nothing else.  So a row of 4100
// elements is still one wavefront's: 512 vectors and 4 elements.  (Taking the two 16-byte vectors that
// overlap the row's ends instead, and masking what is not the row's, cost
// 25-40 % at 1000-4000 elements; 16-byte accesses at 2-byte alignment, which
// gfx950 also serves, were 3-4 times slower still.)
// (2) Lanes take the vectors rotated by the body's distance from a 128-byte
// boundary (slot s holds vector s - shift, the first `shift` slots the last
// vectors the workgroup has room for), so that the 1 KiB a wavefront loads or
// stores with one instruction is made of whole 128-byte lines.  Without that,
// measured on MI355X: [32, 4088, 4088] fp16 360 us against 260 us for
// [32, 4032, 4032], [128, 1000, 1000] 83 us against 65 us for [128, 960, 960].
template<typename T, int BS, int NV, bool THROUGH, bool RAGGED>
__global__ __launch_bounds__(BS) __attribute__((amdgpu_waves_per_eu(BS == 512 && NV == 8 ? 4 : 1)))// 512 x 8: two workgroups per compute unit
void causal_softmax_rows(uint16_t *y, uint64_t rows, uint32_t seq, uint32_t total,
                                                          int64_t stride_b, int64_t stride_i, FastDiv by_seq) {
    AMD_ARGS_NOW(y, rows, seq, total, stride_b, stride_i, arg_pair(by_seq), gridDim.x);
    constexpr int WAVES = BS / kWave;
    // the form held to 128 registers has none to spare for the packed comparisons' second pair of accumulators
    constexpr bool kPacked = T::kPackedMinMax && !(BS == 512 && NV == 8);
    __shared__ float red[4 * WAVES];// two slot sets for the maxima, two for the sums
    // the same form, RAGGED: the first wavefront's end elements wait in LDS while the exponentials of the vectors are formed
    constexpr bool kStashEnds = RAGGED && BS == 512 && NV == 8;
    __shared__ float ends[kStashEnds ? kWave : 1];
    const float neg_inf = -__builtin_inff();

    struct Row {
        uint16_t *ptr;  // the row's first element
        uint32_t keep;  // columns kept, 1..total
        uint32_t head;  // elements in front of the body, 0..7; 0 unless RAGGED
        uint32_t nvec;  // vectors of the body
        uint32_t shift; // 16-byte vectors between the 128-byte boundary in front of the body and the body; 0 unless RAGGED
    };
    // the vector of the body that this lane holds in its slot k
    auto vector_at = [&](const Row &row, int k) {
        const uint32_t s = k * BS + threadIdx.x - row.shift;// shift < 8: only slot 0 can fall in front of the body
        return RAGGED && k == 0 && static_cast<int32_t>(s) < 0 ? s + NV * BS : s;
    };
    // Global row r = b*seq + i.  All workgroups work on neighbouring rows at
    // any one time (measured: faster than giving each matrix of the batch its
    // own workgroups); (b, i) is advanced by the constant hop without dividing.
    const uint32_t hop = gridDim.x;
    const uint32_t hop_b = fast_quotient(hop, by_seq), hop_i = hop - hop_b * seq;// the grid is far below 2^31 rows (see FastDiv)
    uint64_t b = fast_quotient(blockIdx.x, by_seq);
    uint32_t i = blockIdx.x - static_cast<uint32_t>(b) * seq;
    auto here = [&]() {
        uint16_t *ptr = y + static_cast<int64_t>(b) * stride_b + static_cast<int64_t>(i) * stride_i;
        if constexpr (RAGGED) {
            const uint32_t head = (8u - static_cast<uint32_t>(reinterpret_cast<uintptr_t>(ptr) & 15u) / 2) & 7u;
            const uint32_t shift = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(ptr + head) & 127u) / 16;
            const uint32_t whole = (total - head) / 8;
            return Row{ptr, total - seq + i + 1, head, whole < NV * BS ? whole : NV * BS, shift};
        } else {
            return Row{ptr, total - seq + i + 1, 0u, total / 8, 0u};
        }
    };
    auto advance = [&]() {
        b += hop_b;
        i += hop_i;
        if (i >= seq) {
            i -= seq;
            ++b;
        }
    };
    // kept columns of the body: all of them when !RAGGED, possibly none otherwise
    auto kept_in_body = [&](const Row &row) {
        if constexpr (!RAGGED) return row.keep;
        const uint32_t past_head = row.keep > row.head ? row.keep - row.head : 0u;
        return past_head < row.nvec * 8 ? past_head : row.nvec * 8;
    };
    auto load_row = [&](const Row &row, u32x4(&dst)[NV]) {
        const uint32_t keep = kept_in_body(row);
        const uint32_t last_vec = RAGGED && keep == 0 ? 0u : (keep - 1) / 8;
        const uint16_t *body = row.ptr + row.head;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = vector_at(row, k);
            dst[k] = ld16_stream(body + static_cast<uint64_t>(v < last_vec ? v : last_vec) * 8);
        }
    };
    // The one vector of a row that straddles the mask (when the kept length is
    // not a multiple of 8) is dealt with apart from the others, inside
    // wavefront-uniform branches that are taken once per row: its kept
    // elements enter the maximum and minimum one by one, the exponentials of
    // its masked elements (whatever they came to) are replaced by zero before
    // the sum, and its masked outputs are forced to zero before the store (a
    // row that turned to NaN would otherwise leak into them).  Everything else
    // runs without a per-element test.
    auto finish_row = [&](const Row &row, const u32x4(&cur)[NV], int phase) {
        const uint32_t keep = kept_in_body(row), nvec = row.nvec;
        const uint32_t keep_vecs = (keep + 7) / 8;
        const uint32_t tail = keep & 7u;// kept elements of the straddling vector, 0 when there is none
        // RAGGED: lanes 0-7 of the workgroup hold the elements in front of the body, lanes 8-63 those behind it
        [[maybe_unused]] uint32_t end_col = 0;// this lane's column of the row, if end_mine
        [[maybe_unused]] bool end_mine = false, end_kept = false;
        [[maybe_unused]] float end_x = 0.0f;
        if constexpr (RAGGED) {
            const uint32_t t = threadIdx.x;
            end_col = t < 8 ? t : row.head + nvec * 8 + (t - 8);
            end_mine = t < 8 ? t < row.head : (t < kWave && end_col < total);
            end_kept = end_mine && end_col < row.keep;
            if (end_kept) end_x = T::one(row.ptr[end_col]);
        }
        float mx = neg_inf, mn = __builtin_inff();
        [[maybe_unused]] typename T::pair mx2, mn2;
        if constexpr (kPacked) mx2 = T::splat(neg_inf), mn2 = T::splat(__builtin_inff());
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = vector_at(row, k);
            const bool straddles = tail != 0 && v + 1 == keep_vecs;
            if (__builtin_amdgcn_ballot_w64(straddles) != 0) {
                if (straddles) {
                    float b[8];
                    widen8<T>(cur[k], b);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        if (static_cast<uint32_t>(e) < tail) mx = fmaxf(mx, b[e]), mn = fminf(mn, b[e]);
                    }
                }
            }
            if (v >= keep_vecs || straddles) continue;// wholly masked: nothing to reduce, zeros are stored below
            if constexpr (kPacked) {
                const uint32_t w[4] = {cur[k].x, cur[k].y, cur[k].z, cur[k].w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    mx2 = T::max2(mx2, T::as_pair(w[i]));
                    mn2 = T::min2(mn2, T::as_pair(w[i]));
                }
            } else {
                float b[8];
                widen8<T>(cur[k], b);
#pragma unroll
                for (int e = 0; e < 8; ++e) mx = fmaxf(mx, b[e]), mn = fminf(mn, b[e]);
            }
        }
        if constexpr (kPacked) {
            mx = fmaxf(mx, fmaxf(T::first(mx2), T::second(mx2)));
            mn = fminf(mn, fminf(T::first(mn2), T::second(mn2)));
        }
        if constexpr (RAGGED) {
            if (end_kept) mx = fmaxf(mx, end_x), mn = fminf(mn, end_x);
            if constexpr (kStashEnds) {
                if (threadIdx.x < kWave) ends[threadIdx.x] = end_x;// read back by the same lane, behind the barrier below
            }
        }
        mx = block_max<WAVES>(mx, red, phase);

        // d = x - max <= 0.  Anything below the lean exponential's range (-inf
        // inputs, very long tails) sends the wavefront through the library
        // routine; NaN passes through either form as NaN.  The smallest d of
        // this lane is its minimum less the row's maximum.
        const float lowest = mn - mx;// +inf - max for a lane without kept elements: passes the test below
        const bool lean = __builtin_amdgcn_ballot_w64(!(lowest >= kLeanExpLimit)) == 0;
        float f[NV][8];
        float part = 0.0f;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = vector_at(row, k);
            if (v >= keep_vecs) continue;
            widen8<T>(cur[k], f[k]);
            if (lean) {
#pragma unroll
                for (int e = 0; e < 8; ++e) f[k][e] = exp_nonpositive(f[k][e] - mx);
            } else {
                float slow[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) slow[e] = f[k][e];
                exp_any8(slow, mx);
#pragma unroll
                for (int e = 0; e < 8; ++e) f[k][e] = slow[e];
            }
            const bool straddles = tail != 0 && v + 1 == keep_vecs;
            if (__builtin_amdgcn_ballot_w64(straddles) != 0) {
                if (straddles) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) f[k][e] = static_cast<uint32_t>(e) < tail ? f[k][e] : 0.0f;
                }
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) part += f[k][e];
        }
        // (The end elements' exponential and store come after the vectors': placed in front of them, to shorten
        // the life of their registers, they cost [32, 4095, 4095] fp16 285 -> 562 us, [32, 1024, 4099] 85 -> 148 us.)
        [[maybe_unused]] float end_f = 0.0f;
        if constexpr (RAGGED) {
            if (threadIdx.x < kWave) {
                if constexpr (kStashEnds) end_x = ends[threadIdx.x];
                if (lean) {
                    end_f = exp_nonpositive(end_x - mx);
                } else {
                    float slow[8] = {end_x, mx, mx, mx, mx, mx, mx, mx};
                    exp_any8(slow, mx);
                    end_f = slow[0];
                }
                end_f = end_kept ? end_f : 0.0f;
                part += end_f;
            }
        }
        const float sum = block_sum<WAVES>(part, red + 2 * WAVES, phase);
        const float rcp = 1.0f / sum;
        const StreamOut<THROUGH> out(row.ptr + row.head);// the row is the same for every lane of the workgroup
        // e / sum: one residual step makes the quotient correctly rounded in all but rare cases
        auto quotient = [&](float e) {
            const float q = e * rcp;
            return __builtin_fmaf(__builtin_fmaf(-sum, q, e), rcp, q);
        };

#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = vector_at(row, k);
            u32x4 packed{0, 0, 0, 0};
            if (v < keep_vecs) {
                float o[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = quotient(f[k][e]);
                packed = narrow8_unit_range<T>(o);
                const bool straddles = tail != 0 && v + 1 == keep_vecs;
                if (__builtin_amdgcn_ballot_w64(straddles) != 0) {
                    if (straddles) {// its masked tail is zero whatever the row turned into
                        uint32_t w[4] = {packed.x, packed.y, packed.z, packed.w};
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            if (static_cast<uint32_t>(e) >= tail) w[e / 2] &= (e & 1) ? 0x0000FFFFu : 0xFFFF0000u;
                        }
                        packed = u32x4{w[0], w[1], w[2], w[3]};
                    }
                }
            }
            if (v < nvec) out.st16(v * 16, packed);
        }
        if constexpr (RAGGED) {
            if (end_mine) row.ptr[end_col] = end_kept ? static_cast<uint16_t>(T::narrow2_fast(quotient(end_f), 0.0f) & 0xFFFFu) : uint16_t{0};
        }
    };

    uint64_t r = blockIdx.x;
    if (r >= rows) return;
    int phase = 0;// alternates the LDS slots, so that one barrier per reduction is enough
    while (true) {
        u32x4 x[NV];
        const Row row = here();
        load_row(row, x);
        finish_row(row, x, phase);
        phase ^= 1;
        r += hop;
        if (r >= rows) return;
        advance();
    }
}

// Rows of up to 512 elements: P lanes per row, NV vectors per lane (vector
// sub + k * P for lane sub of the row), 64 / P consecutive rows of one matrix
// per wavefront (the host takes this form when the matrix has a multiple of
// 64 / P rows, so a wavefront never straddles two matrices).  A row of the
// other kernel costs its wavefront about 220 vector instructions however short
// it is and whatever part of it the mask keeps; here the fixed part of that is
// shared by 2, 4 or 8 rows, and with two vectors per lane (rows of 257-512
// elements, two to a wavefront) the second vector costs nothing while both
// rows keep 256 columns or fewer.  The arithmetic is causal_softmax_rows', the
// kept length being a per-lane value; the sums are the same trees, one per
// vector index k, added in the order the whole-wavefront tree adds its halves
// (see segment_sum).
template<typename T, int P, int NV, bool THROUGH, bool RAGGED, bool ON16 = false>
__global__ __launch_bounds__(kWave) void causal_softmax_short(uint16_t *y, uint64_t groups, uint32_t seq, uint32_t total,
                                                              int64_t stride_b, int64_t stride_i, FastDiv by_groups_per_matrix,
                                                              uint32_t groups_per_matrix) {
    static_assert((NV >= 1 && NV <= 3 && P * NV <= kWave) || (P == 32 && NV == 4),
                  "up to three vector indices, added as the whole-wavefront tree adds them; or two rows of 65-128 vectors, added as a wavefront of its own adds a row's two vectors per lane");
    AMD_ARGS_NOW(y, groups, seq, total, stride_b, stride_i, arg_pair(by_groups_per_matrix), groups_per_matrix, gridDim.x);
    constexpr uint32_t RPW = kWave / P;// rows per wavefront
    const uint32_t sub = threadIdx.x % P, rr = threadIdx.x / P;
    // ON16: RAGGED rows that all start on 16-byte boundaries.  They keep the streaming hint; on rows that do not,
    // where neighbouring accesses share lines, it costs ([2048, 504, 504] fp16 305 with, 339 us without;
    // [2048, 333, 333] 170 with, 159 without).
    constexpr bool on_16 = ON16;
    const float neg_inf = -__builtin_inff();
    for (uint64_t g = blockIdx.x; g < groups; g += gridDim.x) {
        // group g of RPW rows: matrix b, rows i0 .. i0 + RPW - 1 (fewer than 2^31 groups, see FastDiv)
        const uint32_t b = fast_quotient(static_cast<uint32_t>(g), by_groups_per_matrix);
        const uint32_t i0 = (static_cast<uint32_t>(g) - b * groups_per_matrix) * RPW;
        uint16_t *base = y + static_cast<int64_t>(b) * stride_b + static_cast<int64_t>(i0) * stride_i;// the same for every lane unless RAGGED
        // RAGGED: rows at any 2-byte boundary and of any length.  The vectors are the row's groups of 8 elements from
        // its first element on, moved as 16 bytes at whatever boundary they lie on (gfx950 serves such accesses, at
        // a fraction of the aligned rate); the up to 7 elements behind the last whole group are taken one each by the
        // row's first lanes.  (Whole 16-byte aligned vectors inside the row instead, with the up to 7 elements in
        // front of them taken one by one as well, measured the same where the mask cuts rows short and 15 % slower
        // where it does not: [16384, 64, 250] fp16 224 against 192 us, [4096, 250, 250] 190 against 189.)  All per lane
        // here, and so is the row itself: a wavefront takes RPW consecutive rows of the whole tensor, whichever matrices
        // they lie in (the host passes the divisor of seq and the number of rows in place of the groups' figures), the
        // lanes behind the last row repeat it without storing.
        // What this form costs against rows in whole lines, from the counters ([4096, 250, 250] against [4096, 256, 256],
        // fp16, per launch): 1.27 times the bytes fetched (415 against 328 MB: a kept part that neither starts nor ends on
        // a line boundary brings in two partial lines per row instead of one), 1.14 times the vector instructions, 1.29
        // times the busy cycles.  (With aligned vectors and end elements at both ends: one end element per lane
        // instead of two, end loads issued unconditionally beside the vector loads, 32-bit row offsets for equally
        // spaced rows, the end stores left out altogether - each within 2 %, [8192, 120, 120] 13 % slower.)
        // Nor is it the arithmetic that these rows wait for: with the exponential cut to one multiply and the
        // hardware exp2, and the quotient to one multiply - a third of the vector instructions gone, at the price of
        // three times as many outputs one unit off the float64 quotient - [8192, 256, 256] took 276 against 274 us,
        // [4096, 250, 250] 190 against 190, [2048, 333, 333] 157 against 157; only [16384, 64, 256] (160 against 170)
        // and [65536, 64, 64] (168 against 178) moved.  Nor the memory latency: with the loads of a wavefront's next
        // group in flight during the work on this one (12 more registers, 6 wavefronts per SIMD in place of 7)
        // [8192, 256, 256] took 282 against 274 us, [4096, 250, 250] 184 against 189, [2048, 504, 504] 325 against 301,
        // [16384, 64, 250] 203 against 187.
        const uint32_t row_off = RAGGED ? 0u : rr * static_cast<uint32_t>(stride_i) * 2;// bytes from base to this lane's row
        struct Mine {
            uint16_t *row;       // the row's first element
            uint32_t row_keep;   // columns kept of the row
            uint32_t nvec;       // whole groups of 8 elements
            uint32_t keep;       // columns kept of those groups
            bool valid;
        };
        const Mine mine = [&]() {
            if constexpr (RAGGED) {
                const uint64_t r = g * RPW + rr;
                const bool valid = r < groups_per_matrix;
                const uint32_t rc = valid ? static_cast<uint32_t>(r) : groups_per_matrix - 1;
                const uint32_t rb = fast_quotient(rc, by_groups_per_matrix), ri = rc - rb * seq;
                uint16_t *row = y + static_cast<int64_t>(rb) * stride_b + static_cast<int64_t>(ri) * stride_i;
                const uint32_t row_keep = total - seq + ri + 1;
                const uint32_t nvec = total / 8;
                return Mine{row, row_keep, nvec, row_keep < nvec * 8 ? row_keep : nvec * 8, valid};
            } else {
                const uint32_t row_keep = total - seq + i0 + rr + 1;
                return Mine{base, row_keep, total / 8, row_keep, true};
            }
        }();
        const uint32_t row_keep = mine.row_keep, nvec = mine.nvec, keep = mine.keep;
        [[maybe_unused]] uint16_t *const row = mine.row;
        [[maybe_unused]] const bool valid = mine.valid;
        if constexpr (RAGGED) base = mine.row;
        const uint32_t keep_vecs = (keep + 7) / 8, tail = keep & 7u, last_vec = RAGGED && keep == 0 ? 0u : (keep - 1) / 8;
        u32x4 cur[NV];
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = sub + k * P;
            const uint8_t *at = reinterpret_cast<const uint8_t *>(base) + row_off + (v < last_vec ? v : last_vec) * 16;
            cur[k] = RAGGED && !on_16 ? ld16_any(at) : ld16_stream(at);
        }
        // the row's elements behind its whole groups (lane sub takes the sub-th of them)
        [[maybe_unused]] uint32_t col_t = 0;
        [[maybe_unused]] bool mine_t = false, kept_t = false;
        [[maybe_unused]] float x_t = 0.0f;
        if constexpr (RAGGED) {
            col_t = nvec * 8 + sub;
            mine_t = col_t < total;// P >= 8 lanes, at most 7 elements
            kept_t = mine_t && col_t < row_keep;
            if (kept_t) x_t = T::one(row[col_t]);
        }

        float mx = neg_inf, mn = __builtin_inff();
        float f[NV][8];
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = sub + k * P;
            if (k > 0 && __builtin_amdgcn_ballot_w64(v < keep_vecs) == 0) continue;// no row of this wavefront reaches that far
            const bool straddles = tail != 0 && v + 1 == keep_vecs;
            widen8<T>(cur[k], f[k]);
            if (__builtin_amdgcn_ballot_w64(straddles) != 0) {
                if (straddles) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        if (static_cast<uint32_t>(e) < tail) mx = fmaxf(mx, f[k][e]), mn = fminf(mn, f[k][e]);
                    }
                }
            }
            if (v < keep_vecs && !straddles) {// every element of this vector is kept
                if constexpr (T::kPackedMinMax) {
                    typename T::pair mx2 = T::as_pair(cur[k].x), mn2 = mx2;
                    const uint32_t w[3] = {cur[k].y, cur[k].z, cur[k].w};
#pragma unroll
                    for (int i = 0; i < 3; ++i) {
                        mx2 = T::max2(mx2, T::as_pair(w[i]));
                        mn2 = T::min2(mn2, T::as_pair(w[i]));
                    }
                    mx = fmaxf(mx, fmaxf(T::first(mx2), T::second(mx2)));
                    mn = fminf(mn, fminf(T::first(mn2), T::second(mn2)));
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) mx = fmaxf(mx, f[k][e]), mn = fminf(mn, f[k][e]);
                }
            }
        }
        if constexpr (RAGGED) {
            if (kept_t) mx = fmaxf(mx, x_t), mn = fminf(mn, x_t);
        }
        mx = segment_max<P>(mx);

        const float lowest = mn - mx;// +inf - max for a lane without kept elements: passes the test below
        const bool lean = __builtin_amdgcn_ballot_w64(!(lowest >= kLeanExpLimit)) == 0;
        [[maybe_unused]] float e_t = 0.0f;
        if constexpr (RAGGED) {
            if (lean) {
                e_t = exp_nonpositive(x_t - mx);
            } else {
                float slow[8] = {x_t, mx, mx, mx, mx, mx, mx, mx};
                exp_any8(slow, mx);
                e_t = slow[0];
            }
            e_t = kept_t ? e_t : 0.0f;
        }
        float tree[NV];
        // 32 x 4: a wavefront of its own (causal_softmax_rows, 64 lanes x 2 vectors) would give lane l the vectors l and
        // l + 64 and add their elements in one running sum; here they are lane sub's vectors k and k + 2
        [[maybe_unused]] float run[2] = {0.0f, 0.0f};
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = sub + k * P;
            tree[k] = 0.0f;
            if (k > 0 && __builtin_amdgcn_ballot_w64(v < keep_vecs) == 0) continue;// its sum would be an exact zero
            const bool straddles = tail != 0 && v + 1 == keep_vecs;
            if (v < keep_vecs) {
                if (lean) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) f[k][e] = exp_nonpositive(f[k][e] - mx);
                } else {
                    float slow[8];// an array of its own for the call: f stays in registers
#pragma unroll
                    for (int e = 0; e < 8; ++e) slow[e] = f[k][e];
                    exp_any8(slow, mx);
#pragma unroll
                    for (int e = 0; e < 8; ++e) f[k][e] = slow[e];
                }
            }
            if (__builtin_amdgcn_ballot_w64(straddles) != 0) {
                if (straddles) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) f[k][e] = static_cast<uint32_t>(e) < tail ? f[k][e] : 0.0f;
                }
            }
            if constexpr (NV == 4) {
                if (v < keep_vecs) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) run[k & 1] += f[k][e];
                }
                if constexpr (RAGGED) {
                    if (k == 0) run[0] += e_t;
                }
            } else {
                float part = 0.0f;
                if (v < keep_vecs) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) part += f[k][e];
                }
                if constexpr (RAGGED) {
                    if (k == 0) part += e_t;
                }
                tree[k] = segment_sum<P>(part);
            }
        }
        // the order in which the whole-wavefront tree adds these groups of lanes: upper to lower, pairwise
        float sum = tree[0];
        if constexpr (NV == 2) sum = tree[1] + tree[0];
        if constexpr (NV == 3) sum = tree[2] + (tree[1] + tree[0]);
        if constexpr (NV == 4) sum = segment_sum<P>(run[1]) + segment_sum<P>(run[0]);
        const float rcp = 1.0f / sum;

        const StreamOut<THROUGH> out(RAGGED ? y : base);// RAGGED: not used, every lane has a base of its own
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = sub + k * P;
            u32x4 packed{0, 0, 0, 0};
            if (k == 0 || __builtin_amdgcn_ballot_w64(v < keep_vecs) != 0) {
                const bool straddles = tail != 0 && v + 1 == keep_vecs;
                if (v < keep_vecs) {
                    float o[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float q = f[k][e] * rcp;
                        o[e] = __builtin_fmaf(__builtin_fmaf(-sum, q, f[k][e]), rcp, q);
                    }
                    packed = narrow8_unit_range<T>(o);
                }
                if (__builtin_amdgcn_ballot_w64(straddles) != 0) {
                    if (straddles) {// its masked tail is zero whatever the row turned into
                        uint32_t w[4] = {packed.x, packed.y, packed.z, packed.w};
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            if (static_cast<uint32_t>(e) >= tail) w[e / 2] &= (e & 1) ? 0x0000FFFFu : 0xFFFF0000u;
                        }
                        packed = u32x4{w[0], w[1], w[2], w[3]};
                    }
                }
            }
            if constexpr (RAGGED) {
                if (valid && v < nvec) {
                    if (on_16) st16_stream(base + v * 8, packed);
                    else st16_any(base + v * 8, packed);
                }
            } else {
                if (v < nvec) out.st16(row_off + v * 16, packed);
            }
        }
        if constexpr (RAGGED) {
            auto one = [&](float e) {
                const float q = e * rcp;
                return static_cast<uint16_t>(T::narrow2_fast(__builtin_fmaf(__builtin_fmaf(-sum, q, e), rcp, q), 0.0f) & 0xFFFFu);
            };
            if (valid && mine_t) row[col_t] = kept_t ? one(e_t) : uint16_t{0};
        }
    }
}

// Rows of more than 32 768 elements that the register kernels do not take:
// longer than 131 072 elements, or RAGGED - rows that do not start on 16-byte
// boundaries or whose length is no multiple of 8, which is what the scores of
// an attention over an arbitrary number of keys look like.  Two passes over
// the row with 16-byte accesses, UNROLL vectors per lane in flight at a time:
// the maximum (and the minimum, for the choice of exponential) together with
// the sum of the exponentials, then the quotients.  The first pass brings the
// row in from memory; the second finds most of it in L2 or in the Infinity
// Cache (the counters say 70 % at 65 536 elements: 1.15 times the algorithmic
// traffic), so the exponentials are formed twice.  (With the sum in a pass of
// its own, after the maximum: [64, 512, 65536] fp16 2163 us against 1691 us.)
// Masked vectors are written as zeros without being read.  One workgroup per
// row at a time.
// RAGGED: the vectors are the 16-byte aligned ones from the 128-byte boundary
// in front of the row (so that a wavefront's 1 KiB per instruction is whole
// lines) to the end of the row, so the first few hold elements of whatever
// lies in front of the row and the last up to 7 of what lies behind it (all
// inside the same 128 bytes as an element of the row, so reading them is safe).  Those foreign elements take
// no part in the reductions, and the two edge vectors are written element by
// element by the lane that owns them - the neighbouring bytes belong to other
// rows, which other workgroups are working on.  (16-byte accesses at 2-byte
// alignment, which gfx950 also serves, measured 3-4 times slower than this.)
template<typename T, int BS, bool THROUGH, bool RAGGED>
__global__ __launch_bounds__(BS) void causal_softmax_long(uint16_t *y, uint64_t rows, uint32_t seq, uint32_t total,
                                                          int64_t stride_b, int64_t stride_i, FastDiv by_seq) {
    AMD_ARGS_NOW(y, rows, seq, total, stride_b, stride_i, arg_pair(by_seq), gridDim.x);
    constexpr int WAVES = BS / kWave, UNROLL = 4;
    __shared__ float red[4 * WAVES];
    int phase = 0;
    for (uint64_t r = blockIdx.x; r < rows; r += gridDim.x, phase ^= 1) {
        const uint32_t b = fast_quotient(static_cast<uint32_t>(r), by_seq), i = static_cast<uint32_t>(r) - b * seq;// fewer than 2^31 rows (see FastDiv)
        uint16_t *row = y + static_cast<int64_t>(b) * stride_b + static_cast<int64_t>(i) * stride_i;
        // positions count from the 128-byte boundary at or in front of the row: the row is [lo, end), its kept part [lo, hi)
        const uint32_t lo = RAGGED ? static_cast<uint32_t>(reinterpret_cast<uintptr_t>(row) & 127u) / 2 : 0u;
        const uint16_t *base = row - lo;
        const uint32_t hi = lo + (total - seq + i + 1), end = lo + total;
        const uint32_t keep_vecs = (hi + 7) / 8, nvec = (end + 7) / 8;// vectors that hold kept elements; vectors that hold elements of the row
        const uint32_t kept_from = (lo + 7) / 8, kept_to = hi / 8;      // vectors [kept_from, kept_to) are kept entirely
        const uint32_t own_to = end / 8;                                // vectors [kept_from, own_to) belong to the row entirely

        // pass 1: maximum and minimum of the kept elements
        float mx = -__builtin_inff(), mn = __builtin_inff();
        // ... and the sum of the exponentials in the same sweep: each lane keeps the maximum of what it has seen so far
        // (own_max) and the sum of exp(x - own_max) (own_sum), rescaled when the maximum grows.  The sum only feeds the
        // denominator, so its exponentials are the plain v_exp_f32 of a rounded product (relative error below 2e-6
        // wherever a term matters, no range limits: -inf and underflow give 0).
        float own_max = -__builtin_inff(), own_sum = 0.0f;
        {
            constexpr float kL2e = 1.44269502162933349609375f;
            auto exp_rough = [&](float d) { return __builtin_amdgcn_exp2f(d * kL2e); };
            for (uint32_t v0 = threadIdx.x; v0 < keep_vecs; v0 += BS * UNROLL) {
                u32x4 x[UNROLL];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    const uint32_t v = v0 + u * BS;
                    x[u] = ld16(base + static_cast<uint64_t>(v < keep_vecs ? v : keep_vecs - 1) * 8);
                }
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    const uint32_t v = v0 + u * BS;
                    if (v >= keep_vecs) continue;
                    float f[8], low[8];
                    widen8<T>(x[u], f);
#pragma unroll
                    for (int e = 0; e < 8; ++e) low[e] = f[e];
                    const bool edge = v < kept_from || v >= kept_to;
                    if (__builtin_amdgcn_ballot_w64(edge) != 0) {
                        if (edge) {// what is not kept: -inf for the maximum and the sum, +inf for the minimum
#pragma unroll
                            for (int e = 0; e < 8; ++e) {
                                const uint32_t p = v * 8 + e;
                                const bool kept = p >= lo && p < hi;
                                f[e] = kept ? f[e] : -__builtin_inff();
                                low[e] = kept ? low[e] : __builtin_inff();
                            }
                        }
                    }
                    float top = f[0];
#pragma unroll
                    for (int e = 1; e < 8; ++e) top = fmaxf(top, f[e]);
#pragma unroll
                    for (int e = 0; e < 8; ++e) mn = fminf(mn, low[e]);
                    const float grown = fmaxf(own_max, top);
                    const float from = grown == -__builtin_inff() ? 0.0f : grown;// nothing finite yet: every term is exp(-inf) = 0
                    float add = 0.0f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) add += exp_rough(f[e] - from);
                    own_sum = own_sum * (own_max == grown ? 1.0f : exp_rough(own_max - grown)) + add;
                    own_max = grown;
                }
            }
            mx = own_max;
        }
        mx = block_max<WAVES>(mx, red, phase);
        const float lowest = mn - mx;
        const bool lean = __builtin_amdgcn_ballot_w64(!(lowest >= kLeanExpLimit)) == 0;

        // exp(x - max) of the elements of vector v, zero for those that are not kept
        auto exps = [&](u32x4 x, uint32_t v, float(&e8)[8]) {
            widen8<T>(x, e8);
            if (lean) {
#pragma unroll
                for (int e = 0; e < 8; ++e) e8[e] = exp_nonpositive(e8[e] - mx);
            } else {
                float slow[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) slow[e] = e8[e];
                exp_any8(slow, mx);
#pragma unroll
                for (int e = 0; e < 8; ++e) e8[e] = slow[e];
            }
            const bool edge = v < kept_from || v >= kept_to;
            if (__builtin_amdgcn_ballot_w64(edge) != 0) {
                if (edge) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const uint32_t p = v * 8 + e;
                        e8[e] = p >= lo && p < hi ? e8[e] : 0.0f;
                    }
                }
            }
        };

        // this lane's sum, brought from its own maximum to the row's (a lane that saw nothing finite holds 0), then the workgroup tree
        const float part = own_max == mx ? own_sum : own_sum * __builtin_amdgcn_exp2f((own_max - mx) * 1.44269502162933349609375f);
        const float sum = block_sum<WAVES>(part, red + 2 * WAVES, phase);
        const float rcp = 1.0f / sum;

        // pass 2: the quotients, and zeros behind them
        const StreamOut<THROUGH> out(const_cast<uint16_t *>(base));
        for (uint32_t v0 = threadIdx.x; v0 < nvec; v0 += BS * UNROLL) {
            u32x4 x[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const uint32_t v = v0 + u * BS;
                x[u] = ld16(base + static_cast<uint64_t>(v < keep_vecs ? v : keep_vecs - 1) * 8);
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                const uint32_t v = v0 + u * BS;
                u32x4 packed{0, 0, 0, 0};
                if (v < keep_vecs) {
                    float e8[8], o[8];
                    exps(x[u], v, e8);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float q = e8[e] * rcp;
                        o[e] = __builtin_fmaf(__builtin_fmaf(-sum, q, e8[e]), rcp, q);
                    }
                    packed = narrow8_unit_range<T>(o);
                    const bool edge = v < kept_from || v >= kept_to;
                    if (__builtin_amdgcn_ballot_w64(edge) != 0) {
                        if (edge) {// what is not kept is zero whatever the row turned into
                            uint32_t w[4] = {packed.x, packed.y, packed.z, packed.w};
#pragma unroll
                            for (int e = 0; e < 8; ++e) {
                                const uint32_t p = v * 8 + e;
                                if (!(p >= lo && p < hi)) w[e / 2] &= (e & 1) ? 0x0000FFFFu : 0xFFFF0000u;
                            }
                            packed = u32x4{w[0], w[1], w[2], w[3]};
                        }
                    }
                }
                const bool mine = v >= kept_from && v < own_to;// all sixteen bytes are the row's
                if (mine) out.st16(v * 16, packed);
                if constexpr (RAGGED) {
                    const bool shared = !mine && v < nvec;
                    if (__builtin_amdgcn_ballot_w64(shared) != 0) {
                        if (shared) {
                            const uint32_t w[4] = {packed.x, packed.y, packed.z, packed.w};
#pragma unroll
                            for (int e = 0; e < 8; ++e) {
                                const uint32_t p = v * 8 + e;
                                if (p >= lo && p < end) row[static_cast<int64_t>(p) - lo] = static_cast<uint16_t>(w[e / 2] >> (16 * (e & 1)));
                            }
                        }
                    }
                }
            }
        }
    }
}

// Rows of 32 769 to 131 072 elements on 16-byte boundaries: the row is read
// once and held in registers as raw 16-bit words - 12, 16 or 20 vectors per
// lane of a 512-lane workgroup up to 81 920 elements (two workgroups fit a
// compute unit, so one row's arithmetic runs under the other's loads and
// stores), 12, 14 or 16 vectors per lane of a 1024-lane workgroup beyond - and
// the three sweeps (the maximum, the sum, the quotients) widen it anew each
// time.  Holding the exponentials instead, as causal_softmax_rows does, would
// take twice the registers; forming them twice costs arithmetic, and at this
// length arithmetic is what the kernel is short of (at 100 % of the memory
// rate a compute unit has about 31 vector-instruction slots per element; the
// full-precision exponential takes 12 and would be needed twice).  So both
// sweeps use the hardware exp2 of one fused multiply-add,
// x * log2(e) - max * log2(e): relative error below 3e-6 where a term is not
// negligible, the same in the sum and in the quotient - well inside what the
// reference's own left-to-right fp32 sum of tens of thousands of terms leaves
// open (about 1e-5), and far below half a unit of either 16-bit format.  No
// range limits: -inf and underflow give 0, NaN stays NaN.
// Measured on MI355X, fp16, against the two-pass kernel above (which read 30 %
// of such rows a second time from memory), us:
//   [64, 512, 40000]   872 /  998     [64, 512, 65536]  1641 / 1677
//   [64, 256, 120000] 1561 / 1605     [64, 256, 131072] 1651 / 1723
// A row stride of 64 KiB or more that is a power of two costs every form here
// about a tenth: the rows that are in flight together then lie in the same
// memory channels and banks.  [64, 512, 65536] with each row 1 KiB further
// from the one before it: 1453 us (74 %) against 1641 us (65 %); [64, 512,
// 32768]: 764 against 815 us.  (Turning the order in which a workgroup's lanes
// take the row's vectors, by 1 KiB per row, changes nothing: 1647 us - the
// whole row is in flight at once either way.  Which rows are in flight
// together does matter, but not in a way a rule could be made of: workgroups
// taking row r * m mod rows instead of row r, for fourteen odd m from 3 to
// 12 289, ran [64, 512, 65536] in 1566 (m = 513) to 1800 us (m = 1025)
// against 1664, and [64, 512, 32768] in 796-814 against 799.)
template<typename T, int BS, int NV, bool THROUGH, bool TURN, bool RAGGED = false>
__global__ __launch_bounds__(BS) __attribute__((amdgpu_waves_per_eu(4)))
void causal_softmax_held(uint16_t *y, uint64_t rows, uint32_t seq, uint32_t total, int64_t stride_b, int64_t stride_i, FastDiv by_seq) {
    AMD_ARGS_NOW(y, rows, seq, total, stride_b, stride_i, arg_pair(by_seq), gridDim.x);
    constexpr int WAVES = BS / kWave;
    constexpr float kL2e = 1.44269502162933349609375f;
    __shared__ float red[4 * WAVES];
    const float neg_inf = -__builtin_inff();
    static_assert(!RAGGED || TURN, "rows at any 2-byte boundary are turned to line boundaries as well");
    int phase = 0;
    for (uint64_t r = blockIdx.x; r < rows; r += gridDim.x, phase ^= 1) {
        const uint32_t b = fast_quotient(static_cast<uint32_t>(r), by_seq), i = static_cast<uint32_t>(r) - b * seq;// fewer than 2^31 rows (see FastDiv)
        uint16_t *row = y + static_cast<int64_t>(b) * stride_b + static_cast<int64_t>(i) * stride_i;
        // RAGGED: rows at any 2-byte boundary and of any length.  The vectors are the whole 16-byte aligned ones
        // inside the row (its body); the up to 7 elements in front of them and the up to 7 behind are taken one each
        // by the first 16 lanes of the workgroup, with 2-byte accesses, and enter the maximum, the sum and the
        // quotients beside those lanes' vectors ([39, 512, 40001] fp16 614 us in two passes -> 5xx us).
        const uint32_t row_keep = total - seq + i + 1;
        uint32_t head = 0, nvec = total / 8, keep = row_keep;
        uint16_t *body = row;
        if constexpr (RAGGED) {
            head = (8u - static_cast<uint32_t>(reinterpret_cast<uintptr_t>(row) & 15u) / 2) & 7u;
            body = row + head;
            nvec = (total - head) / 8;
            const uint32_t past_head = row_keep > head ? row_keep - head : 0u;
            keep = past_head < nvec * 8 ? past_head : nvec * 8;
        }
        const uint32_t keep_vecs = (keep + 7) / 8, tail = keep & 7u, last_vec = RAGGED && keep == 0 ? 0u : (keep - 1) / 8;
        [[maybe_unused]] uint32_t end_col = 0;// this lane's column of the row, if end_mine
        [[maybe_unused]] bool end_mine = false, end_kept = false;
        [[maybe_unused]] float end_x = 0.0f, end_e = 0.0f;
        if constexpr (RAGGED) {
            const uint32_t t = threadIdx.x;
            end_col = t < 8 ? t : head + nvec * 8 + (t - 8);
            end_mine = t < 8 ? t < head : (t < 16 && end_col < total);
            end_kept = end_mine && end_col < row_keep;
            if (end_kept) end_x = T::one(row[end_col]);
        }
        // TURN: rows that start inside a 128-byte line.  Lanes take the vectors turned by the row's distance from
        // the line's start, the first few lanes of the first turn the last vectors there is room for, so that a
        // wavefront's 1 KiB per instruction is whole lines ([34, 512, 45000] fp16 657 -> 526 us, [47, 512, 33000]
        // 674 -> 585).  A form of its own: on rows in whole lines it costs 1-1.5 %, and the 20-vector form has no
        // register left for it.
        static_assert(!TURN || NV < 20, "no register left for the turn");
        [[maybe_unused]] const uint32_t turn = TURN ? static_cast<uint32_t>(reinterpret_cast<uintptr_t>(body) & 127u) / 16 : 0u;
        auto vector_at = [&](int k) {
            if constexpr (TURN) {
                const uint32_t s = static_cast<uint32_t>(k * BS + threadIdx.x) - turn;
                return k == 0 && static_cast<int32_t>(s) < 0 ? s + NV * BS : s;
            } else {
                return static_cast<uint32_t>(k * BS + threadIdx.x);
            }
        };
        u32x4 cur[NV];
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = vector_at(k);
            cur[k] = ld16_stream(body + static_cast<uint64_t>(v < last_vec ? v : last_vec) * 8);// masked vectors re-read the last kept one
        }
        // the maximum; the one vector that straddles the mask enters element by element
        float mx = neg_inf;
        [[maybe_unused]] typename T::pair mx2;
        if constexpr (T::kPackedMinMax) mx2 = T::splat(neg_inf);
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = vector_at(k);
            const bool straddles = tail != 0 && v + 1 == keep_vecs;
            if (__builtin_amdgcn_ballot_w64(straddles) != 0) {
                if (straddles) {
                    float f[8];
                    widen8<T>(cur[k], f);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        if (static_cast<uint32_t>(e) < tail) mx = fmaxf(mx, f[e]);
                    }
                }
            }
            if (v >= keep_vecs || straddles) continue;
            if constexpr (T::kPackedMinMax) {
                const uint32_t w[4] = {cur[k].x, cur[k].y, cur[k].z, cur[k].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) mx2 = T::max2(mx2, T::as_pair(w[j]));
            } else {
                float f[8];
                widen8<T>(cur[k], f);
#pragma unroll
                for (int e = 0; e < 8; ++e) mx = fmaxf(mx, f[e]);
            }
        }
        if constexpr (T::kPackedMinMax) mx = fmaxf(mx, fmaxf(T::first(mx2), T::second(mx2)));
        if constexpr (RAGGED) {
            if (end_kept) mx = fmaxf(mx, end_x);
        }
        mx = block_max<WAVES>(mx, red, phase);
        // exp(x - max) as exp2(x * log2(e) - max * log2(e)); a row whose maximum is +-inf goes the plain way (inf - inf must give NaN)
        const bool finite_max = __builtin_fabsf(mx) < __builtin_inff();
        const float m2 = mx * kL2e;
        auto exps = [&](u32x4 raw, float(&e8)[8]) {
            widen8<T>(raw, e8);
            if (finite_max) {
#pragma unroll
                for (int e = 0; e < 8; ++e) e8[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(e8[e], kL2e, -m2));
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) e8[e] = __builtin_amdgcn_exp2f((e8[e] - mx) * kL2e);
            }
        };
#pragma unroll
        for (int k = 0; k < NV; ++k) asm volatile("" : "+v"(cur[k]));// the sweeps widen the raw words anew: no widened copy is kept
        float part = 0.0f;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = vector_at(k);
            if (v >= keep_vecs) continue;
            float e8[8];
            exps(cur[k], e8);
            const bool straddles = tail != 0 && v + 1 == keep_vecs;
            if (__builtin_amdgcn_ballot_w64(straddles) != 0) {
                if (straddles) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) e8[e] = static_cast<uint32_t>(e) < tail ? e8[e] : 0.0f;
                }
            }
            part += ((e8[0] + e8[1]) + (e8[2] + e8[3])) + ((e8[4] + e8[5]) + (e8[6] + e8[7]));
        }
        if constexpr (RAGGED) {
            if (end_kept) end_e = __builtin_amdgcn_exp2f(finite_max ? __builtin_fmaf(end_x, kL2e, -m2) : (end_x - mx) * kL2e);
            part += end_e;// 0 for the lanes without a kept end element
        }
        const float sum = block_sum<WAVES>(part, red + 2 * WAVES, phase);
        const float rcp = 1.0f / sum;
#pragma unroll
        for (int k = 0; k < NV; ++k) asm volatile("" : "+v"(cur[k]));
        const StreamOut<THROUGH> out(body);
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const uint32_t v = vector_at(k);
            u32x4 packed{0, 0, 0, 0};
            if (v < keep_vecs) {
                float e8[8];
                exps(cur[k], e8);
#pragma unroll
                for (int e = 0; e < 8; ++e) e8[e] *= rcp;
                packed = narrow8_unit_range<T>(e8);
                const bool straddles = tail != 0 && v + 1 == keep_vecs;
                if (__builtin_amdgcn_ballot_w64(straddles) != 0) {
                    if (straddles) {// its masked tail is zero whatever the row turned into
                        uint32_t w[4] = {packed.x, packed.y, packed.z, packed.w};
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            if (static_cast<uint32_t>(e) >= tail) w[e / 2] &= (e & 1) ? 0x0000FFFFu : 0xFFFF0000u;
                        }
                        packed = u32x4{w[0], w[1], w[2], w[3]};
                    }
                }
            }
            if (v < nvec) out.st16(v * 16, packed);
        }
        if constexpr (RAGGED) {
            if (end_mine) row[end_col] = end_kept ? static_cast<uint16_t>(T::narrow2_fast(end_e * rcp, 0.0f) & 0xFFFFu) : uint16_t{0};
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

// ---- few long rows: a row split over several workgroups, two launches --------------
// Decoding over a long context is one query row per head: 64 rows of 131 072 columns keep 64 of 256 compute
// units busy at a workgroup per row.  Here workgroup (part, row) takes BS * 32 columns of the
// row - BS lanes x 4 vectors, held in registers.  The first launch leaves each part's maximum, minimum and sum
// of exp(x - maximum) over its kept columns in the workspace; the second reads the row's parts (the same few
// values in every workgroup of the row, combined in the same order), rescales the sums to the row's maximum and
// writes its own columns: exp(x - maximum) / sum, the exponentials and the quotient those of the other forms.
// Rows start on 16-byte boundaries and are whole vectors long (the host sees to it).
constexpr int kSplitVecs = 4;

template<typename T, int BS>
__global__ __launch_bounds__(BS) void causal_softmax_split_stats(const uint16_t *y, CausalSoftmaxPart *parts, uint32_t seq, uint32_t total,
                                                                           int64_t stride_b, int64_t stride_i, FastDiv by_seq) {
    AMD_ARGS_NOW(y, parts, seq, total, stride_b, stride_i, arg_pair(by_seq));
    constexpr int NV = kSplitVecs, WAVES = BS / kWave;
    constexpr uint32_t kColumns = BS * NV * 8;
    __shared__ float red[6 * WAVES];
    const uint32_t part = blockIdx.x, r = blockIdx.y;
    const uint32_t b = fast_quotient(r, by_seq), i = r - b * seq;
    const uint16_t *row = y + static_cast<int64_t>(b) * stride_b + static_cast<int64_t>(i) * stride_i;
    const uint32_t keep = total - seq + i + 1;
    const uint32_t from = part * kColumns;
    CausalSoftmaxPart *mine = parts + static_cast<size_t>(r) * gridDim.x + part;
    const float neg_inf = -__builtin_inff();
    if (from >= keep) {// nothing of this part is kept (uniform over the workgroup)
        if (threadIdx.x == 0) *mine = CausalSoftmaxPart{neg_inf, __builtin_inff(), 0.0f, 0.0f};
        return;
    }
    const uint32_t upto = keep - from < kColumns ? keep : from + kColumns;
    float f[NV][8];
    float mx = neg_inf, mn = __builtin_inff();
    u32x4 x[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const uint32_t c0 = from + (k * BS + threadIdx.x) * 8;
        x[k] = ld16_stream(row + (c0 < upto ? c0 : from));
    }
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const uint32_t c0 = from + (k * BS + threadIdx.x) * 8;
        widen8<T>(x[k], f[k]);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if (c0 + e < upto) mx = fmaxf(mx, f[k][e]), mn = fminf(mn, f[k][e]);
        }
    }
    mx = block_max<WAVES>(mx, red, 0);
    mn = -block_max<WAVES>(-mn, red + 2 * WAVES, 0);
    const bool lean = mn - mx >= kLeanExpLimit;// uniform; false for infinities and for a part without a finite element
    float sum = 0.0f;
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const uint32_t c0 = from + (k * BS + threadIdx.x) * 8;
        if (c0 >= upto) continue;
        if (lean) {
#pragma unroll
            for (int e = 0; e < 8; ++e) f[k][e] = exp_nonpositive(f[k][e] - mx);
        } else {
            float slow[8];// an array of its own for the call: f stays in registers
#pragma unroll
            for (int e = 0; e < 8; ++e) slow[e] = f[k][e];
            exp_any8(slow, mx);
#pragma unroll
            for (int e = 0; e < 8; ++e) f[k][e] = slow[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) sum += c0 + e < upto ? f[k][e] : 0.0f;
    }
    sum = block_sum<WAVES>(sum, red + 4 * WAVES, 0);
    if (threadIdx.x == 0) *mine = CausalSoftmaxPart{mx, mn, sum, 0.0f};
}

template<typename T, int BS>
__global__ __launch_bounds__(BS) void causal_softmax_split_apply(uint16_t *y, const CausalSoftmaxPart *parts, uint32_t seq, uint32_t total,
                                                                           int64_t stride_b, int64_t stride_i, FastDiv by_seq) {
    AMD_ARGS_NOW(y, parts, seq, total, stride_b, stride_i, arg_pair(by_seq));
    constexpr int NV = kSplitVecs;
    constexpr uint32_t kColumns = BS * NV * 8;
    const uint32_t part = blockIdx.x, r = blockIdx.y;
    const uint32_t b = fast_quotient(r, by_seq), i = r - b * seq;
    uint16_t *row = y + static_cast<int64_t>(b) * stride_b + static_cast<int64_t>(i) * stride_i;
    const uint32_t keep = total - seq + i + 1;
    const uint32_t from = part * kColumns;
    const uint32_t upto = from >= keep ? from : keep - from < kColumns ? keep : from + kColumns;
    u32x4 x[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) {// in flight while the row's parts are put together
        const uint32_t c0 = from + (k * BS + threadIdx.x) * 8;
        x[k] = c0 < upto ? ld16_stream(row + c0) : u32x4{0, 0, 0, 0};
    }
    // the row's maximum and its sum from its parts: lane p of every wavefront takes part p (at most 64 of them) and
    // the wavefront trees put them together - the same values in the same order in every workgroup of the row
    const CausalSoftmaxPart *of_row = parts + static_cast<size_t>(r) * gridDim.x;
    const float neg_inf = -__builtin_inff();
    const uint32_t lane = threadIdx.x & (kWave - 1);
    CausalSoftmaxPart q{neg_inf, __builtin_inff(), 0.0f, 0.0f};
    if (lane < gridDim.x) q = of_row[lane];
    const float top = wave_max(q.max);
    // a part at the row's maximum counts as it is (also where both are infinite); one without a kept or a
    // finite element counts nothing beside a finite maximum
    const float sum = wave_sum(q.max == top ? q.sum : q.max == neg_inf ? 0.0f : q.sum * expf(q.max - top));
    const float my_min = __shfl(q.min, static_cast<int>(part));
    const float rcp = 1.0f / sum;
    const bool lean = my_min - top >= kLeanExpLimit;// uniform over the workgroup
#pragma unroll
    for (int k = 0; k < NV; ++k) {
        const uint32_t c0 = from + (k * BS + threadIdx.x) * 8;
        if (c0 >= total) continue;
        u32x4 packed{0, 0, 0, 0};
        if (c0 < upto) {
            float f[8], o[8];
            widen8<T>(x[k], f);
            if (lean) {
#pragma unroll
                for (int e = 0; e < 8; ++e) f[e] = exp_nonpositive(f[e] - top);
            } else {
                exp_any8(f, top);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float q = f[e] * rcp;
                o[e] = c0 + e < upto ? __builtin_fmaf(__builtin_fmaf(-sum, q, f[e]), rcp, q) : 0.0f;
            }
            packed = narrow8_unit_range<T>(o);
            if (c0 + 8 > upto) {// the masked end of the straddling vector is zero whatever the row turned into
                uint32_t w[4] = {packed.x, packed.y, packed.z, packed.w};
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    if (c0 + e >= upto) w[e / 2] &= (e & 1) ? 0x0000FFFFu : 0xFFFF0000u;
                }
                packed = u32x4{w[0], w[1], w[2], w[3]};
            }
        }
        st16_stream(row + c0, packed);
    }
}

template<typename T>
void launch_causal_softmax(const CausalSoftmaxAmdDescriptor &d, void *data, CausalSoftmaxPart *parts, hipStream_t stream) {
    auto *py = static_cast<uint16_t *>(data);
    if (parts != nullptr) {// few long rows, and the caller brought the workspace: a row's parts on workgroups of their own
        const dim3 grid(causal_softmax_parts(d), static_cast<unsigned>(d.batch * d.seq));
        const FastDiv by = fast_div(static_cast<uint32_t>(d.seq));
#define CS_SPLIT(BS)                                                                                                                                          \
    do {                                                                                                                                                      \
        causal_softmax_split_stats<T, BS><<<grid, BS, 0, stream>>>(py, parts, static_cast<uint32_t>(d.seq), static_cast<uint32_t>(d.total), d.stride_b, d.stride_i, by); \
        causal_softmax_split_apply<T, BS><<<grid, BS, 0, stream>>>(py, parts, static_cast<uint32_t>(d.seq), static_cast<uint32_t>(d.total), d.stride_b, d.stride_i, by); \
    } while (0)
        if (causal_softmax_part_lanes(d) == 128) CS_SPLIT(128);
        else CS_SPLIT(512);
#undef CS_SPLIT
        return;
    }
    const uint64_t rows = d.batch * d.seq;
    const uint64_t nvec = d.total / 8;
    // Rows of up to 3072 elements are taken by single wavefronts (no barrier, no
    // LDS), longer ones by 128, 256 or 512 lanes (the ladder at the end of this function).  Measured on MI355X,
    // fp16 / bf16 (rows of 4096 with one wavefront):
    //   [32, 4096, 4096]   one workgroup per row 264 / 261-266 us (76 %), 256 workgroups per
    //                      compute unit 267 / 267-274, 64 per unit 293 / 292-299; 128 or 256
    //                      lanes per row 264-288 / 261-270
    //   [128, 2048, 2048]  one per row 261 / 258-266, 512 per unit 263 / 262-265
    //   [512, 1024, 1024]  one per row 262 / 253-264, 512 per unit 285 / 283-285
    //   [2048, 512, 512]   one per row 396 / 362, 512 per unit 361 / 332
    //   [8, 8192, 8192]    one per row 268 / 256-265, 64 per unit 272-274 / 270-274
    //   [2, 16384, 16384]  one per row 277-280, 64 per unit 282-284
    // so every row gets a workgroup of its own - the dispatcher then evens out
    // the causal triangle by itself - except rows of 512 elements and fewer,
    // where a workgroup's start costs as much as its row.  Those short rows are bound by
    // instruction issue, not by memory: about 220 vector instructions per row whatever part of
    // it the mask keeps, four cycles each on a 16-lane SIMD ([2048, 512, 512] fp16: 374 us =
    // 875 cycles per row and SIMD; the same bytes as [8192, 256, 256] take 735 us).  Asking
    // for 2 or 4 rows per wavefront before working on the first moved that by -5 to +2 %.
    const bool aligned = d.total % 8 == 0 && d.stride_i % 8 == 0 && d.stride_b % 8 == 0 && aligned16(data);
    const bool in_lines = aligned && d.stride_i % 64 == 0 && d.stride_b % 64 == 0 && (reinterpret_cast<uintptr_t>(data) & 127u) == 0;// rows start on 128-byte boundaries
    // Vectors per row that the kernel must have room for.  The ragged form takes up to 56 elements behind them one by one
    // (see causal_softmax_rows), which rows in whole lines also use when that spares them the next larger form.
    const auto form_of = [](uint64_t vectors) {// the vectors the launch shape for that many has room for (the ladder at the end of this function)
        for (const uint64_t room : {64, 128, 192, 256, 384, 512, 640, 768, 1024, 1280, 1536, 1792, 2048, 2560, 3072}) {
            if (vectors <= room) return room;
        }
        return uint64_t{4096};
    };
    const uint64_t spared = d.total <= 56 ? 1 : ceil_div(d.total - 56, 8);
    const bool ragged = !in_lines || form_of(spared) < form_of(nvec);
    const uint64_t cover = ragged ? spared : nvec;
    const uint64_t cap = cover <= 64 ? static_cast<uint64_t>(d.cu_count) * 512 : rows;
    const uint64_t limit = amd::max_grid_1d(1024);// the kernel strides over what the grid does not cover
    const unsigned grid = static_cast<unsigned>(std::min({rows, cap, limit}));

    const bool even = (reinterpret_cast<uintptr_t>(data) & 1u) == 0;// elements lie on 2-byte boundaries
    const bool vec_ok = even && cover <= 4096 && d.seq < (1ull << 31) && (!ragged || d.total >= 16);
    // Rows of more than 32 768 elements: held in registers as raw words up to 131 072 when they lie on 16-byte
    // boundaries (causal_softmax_held), two passes otherwise (causal_softmax_long; the element kernel took
    // 7230 us for [64, 512, 65536] fp16, 4194 us for [64, 512, 40000]).
    const uint64_t vecs = cover;
    const bool long_ok = even && cover > 4096 && d.total + 64 < (1ull << 31) && rows < kFastDivLimit;
    if (long_ok) {
        const bool thr = rows * d.total * sizeof(uint16_t) >= kWriteThroughBytes;
        const FastDiv by = fast_div(static_cast<uint32_t>(d.seq));
        if (nvec <= 16 * 1024) {// up to 131 072 elements: held in registers, read once (see causal_softmax_held)
            // rows off the 128-byte boundaries skip the 20-vector form, which has no turned variant; rows off the
            // 16-byte boundaries, or whose length is no multiple of 8, take the ragged one (its body is never longer)
            const uint64_t most_512 = in_lines ? 20 * 512 : 16 * 512;
            const unsigned lanes = nvec <= most_512 ? 512 : 1024;
            const unsigned g = static_cast<unsigned>(std::min<uint64_t>(rows, amd::max_grid_1d(lanes)));
#define CS_HELD_GO(BS, NV, TH, TURN, RG) causal_softmax_held<T, BS, NV, TH, TURN, RG><<<g, BS, 0, stream>>>(py, rows, static_cast<uint32_t>(d.seq), static_cast<uint32_t>(d.total), d.stride_b, d.stride_i, by)
#define CS_HELD(BS, NV)                                                              \
    do {                                                                             \
        if (thr && (in_lines || NV >= 20)) CS_HELD_GO(BS, NV, true, false, false);  \
        else if (thr && aligned) CS_HELD_GO(BS, NV, true, (NV < 20), false);         \
        else if (thr) CS_HELD_GO(BS, NV, true, (NV < 20), (NV < 20));                \
        else if (in_lines || NV >= 20) CS_HELD_GO(BS, NV, false, false, false);      \
        else if (aligned) CS_HELD_GO(BS, NV, false, (NV < 20), false);               \
        else CS_HELD_GO(BS, NV, false, (NV < 20), (NV < 20));                        \
    } while (0)
            if (nvec <= 12 * 512) CS_HELD(512, 12);
            else if (nvec <= 16 * 512) CS_HELD(512, 16);
            else if (nvec <= most_512) CS_HELD(512, 20);
            else if (nvec <= 12 * 1024) CS_HELD(1024, 12);
            else if (nvec <= 14 * 1024) CS_HELD(1024, 14);
            else CS_HELD(1024, 16);
#undef CS_HELD
#undef CS_HELD_GO
            return;
        }
        // a turn of the workgroup takes 4 vectors per lane: the lane count that covers the row in the fewest turns with the fewest idle lanes
        // ([64, 512, 40000] fp16: 512 lanes 996 us, 1024 lanes 1138 us; [64, 512, 65536]: 1752, 1684 us; [32, 512, 100000]: 1577, 1388 us)
        const int lanes = vecs < 8192 ? 512 : 1024;
        const unsigned g = static_cast<unsigned>(std::min<uint64_t>(rows, amd::max_grid_1d(1024)));
#define CS_LONG_GO(BS, TH, RG) causal_softmax_long<T, BS, TH, RG><<<g, BS, 0, stream>>>(py, rows, static_cast<uint32_t>(d.seq), static_cast<uint32_t>(d.total), d.stride_b, d.stride_i, by)
#define CS_LONG(BS)                                        \
    do {                                                   \
        if (!in_lines && thr) CS_LONG_GO(BS, true, true);  \
        else if (!in_lines) CS_LONG_GO(BS, false, true);   \
        else if (thr) CS_LONG_GO(BS, true, false);         \
        else CS_LONG_GO(BS, false, false);                 \
    } while (0)
        if (lanes == 512) CS_LONG(512);
        else CS_LONG(1024);
#undef CS_LONG
#undef CS_LONG_GO
        return;
    }
    if (!vec_ok) {
        causal_softmax_generic<T><<<grid, 256, 0, stream>>>(py, rows, d.seq, d.total, d.stride_b, d.stride_i);
        return;
    }
    const bool through = rows * d.total * sizeof(uint16_t) >= kWriteThroughBytes;
    const FastDiv by_seq = fast_div(static_cast<uint32_t>(d.seq));
    // Rows of up to 512 elements, several to a wavefront (see causal_softmax_short), when a matrix has a whole
    // number of such groups of rows and a group lies within reach of a 32-bit byte offset from its first row.
    // Measured on MI355X, fp16, one row per wavefront -> several:
    //   [2048, 512, 512]  374 -> 267 us (bf16 322 -> 260)   [8192, 256, 256]  700 -> 274 us
    //   [32768, 128, 128]  1385 -> 291 us                    [131072, 64, 64]  2765 -> 324 us
    // with 2048 wavefronts per compute unit striding over the groups (128 / 512 / 8192 per unit: 382 / 348 / 351 us
    // at 256 columns with 32 lanes per row).
    if ((aligned || d.total >= 16) && nvec <= 96 && rows < kFastDivLimit && d.stride_i >= 0 && static_cast<uint64_t>(d.stride_i) * 16 + d.total * 2 < (1ull << 31)) {
        // Lanes per row x vectors per lane: the pair that wastes the fewest lanes, the fewer lanes per row (more
        // rows per wavefront) when two waste the same, among those whose rows per wavefront divide the matrix's
        // row count.  More than one vector per lane spares the rows that the mask cuts short the work of the
        // vectors they do not reach.  Measured, fp16 (us):
        //   [2048, 512, 512]   32 x 2  265   16 x 4  274          [8192, 256, 256]   16 x 2  274   32 x 1  344   8 x 4  286
        //   [4096, 384, 384]   16 x 3  318   32 x 2  341          [32768, 128, 128]   8 x 2  296   16 x 1  344
        //   [16384, 192, 192]  16 x 2  338    8 x 3  339   32 x 1  516
        bool together = in_lines;// rows in whole lines: RPW rows of one matrix per wavefront; others: the ragged form, which measures
                                       // better for them also where they lie on 16-byte boundaries ([2048, 504, 504] fp16 345 against 411 us,
                                       // [8192, 120, 120] 89 against 164 us; in whole lines it is the other way round: [2048, 512, 512] 335 against 277 us)
        // (Contiguous rows at odd boundaries through LDS instead - a wavefront loads a run of 8 to 16 rows as the
        // aligned 16-byte vectors that it is, cuts the rows out of LDS with 16-byte LDS accesses and writes the run
        // back in whole vectors - measured level at best, fp16, us, rows addressed in memory / through LDS in chunks
        // of 8 / of 16 rows: [4096, 250, 250] 181 / 196 / 175, [2048, 333, 333] 160 / 192 / 201, [2048, 500, 500]
        // 342 / 326 / 521, [16384, 64, 250] 190 / 207 / 204; with the next run's loads issued before the work on
        // this one, 200 and more.  The three phases of a run follow each other within a wavefront, and LDS bounds
        // the wavefronts that can be in different phases.)
        unsigned lanes = 0, per_lane = 0;
        const auto pick = [&]() {
            for (const unsigned p : {8u, 16u, 32u}) {
                for (const unsigned v : {1u, 2u, 3u, 4u}) {
                    // (32 x 4: rows of 513-768 elements two to a wavefront.  Against a wavefront each - causal_softmax_rows,
                    // 64 x 2 - fp16, us: [2978, 520, 520] 569 / 638, [2427, 576, 576] 442 / 552, [1966, 640, 640] 426 / 515,
                    // [1365, 768, 768] 404 / 449; beyond, the wavefront each is level or ahead: [1333, 777, 777] 555 / 544,
                    // [1003, 896, 896] 417 / 416, [805, 1000, 1000] 461 / 457, [768, 1024, 1024] 389 / 376.)
                    const bool room = v == 4 ? p == 32 : p * v <= kWave;
                    const bool fits = p * v >= nvec && room && (!together || d.seq % (kWave / p) == 0);// ragged rows: any consecutive rows
                    if (fits && (lanes == 0 || p * v < lanes * per_lane)) lanes = p, per_lane = v;
                }
            }
        };
        pick();
        if (lanes == 0 && together && d.total >= 16) {// a matrix's rows do not fill wavefronts (seq = 1: decoding): any consecutive rows then
            together = false;
            pick();
        }
        if (lanes != 0) {
            const unsigned rpw = kWave / lanes;
            const uint64_t groups = ceil_div(rows, rpw);
            const uint32_t gpm = static_cast<uint32_t>(d.seq / rpw);
            const uint64_t capg = static_cast<uint64_t>(d.cu_count) * 2048;
            const unsigned g = static_cast<unsigned>(std::min(groups, capg));
#define CS_SHORT_GO(P, NV, TH, RG, ON16)                                                                                       \
    causal_softmax_short<T, P, NV, TH, RG, ON16><<<g, kWave, 0, stream>>>(py, groups, static_cast<uint32_t>(d.seq), static_cast<uint32_t>(d.total), \
                                                                          d.stride_b, d.stride_i, RG ? by_seq : fast_div(gpm), RG ? static_cast<uint32_t>(rows) : gpm)
#define CS_SHORT(P, NV)                                                                                                        \
    do {                                                                                                                       \
        if (through && together) CS_SHORT_GO(P, NV, true, false, false);                                                       \
        else if (through && aligned) CS_SHORT_GO(P, NV, true, true, true);                                                     \
        else if (through) CS_SHORT_GO(P, NV, true, true, false);                                                               \
        else if (together) CS_SHORT_GO(P, NV, false, false, false);                                                            \
        else if (aligned) CS_SHORT_GO(P, NV, false, true, true);                                                               \
        else CS_SHORT_GO(P, NV, false, true, false);                                                                           \
    } while (0)
            switch (lanes * 10 + per_lane) {
                case 81: CS_SHORT(8, 1); break;
                case 82: CS_SHORT(8, 2); break;
                case 83: CS_SHORT(8, 3); break;
                case 161: CS_SHORT(16, 1); break;
                case 162: CS_SHORT(16, 2); break;
                case 163: CS_SHORT(16, 3); break;
                case 321: CS_SHORT(32, 1); break;
                case 324: CS_SHORT(32, 4); break;
                default: CS_SHORT(32, 2); break;
            }
#undef CS_SHORT
#undef CS_SHORT_GO
            return;
        }
    }
#define CS_GO(BS, NV, TH, RG) \
    causal_softmax_rows<T, BS, NV, TH, RG><<<grid, BS, 0, stream>>>(py, rows, static_cast<uint32_t>(d.seq), static_cast<uint32_t>(d.total), d.stride_b, d.stride_i, by_seq)
#define CS_LAUNCH(BS, NV)                               \
    do {                                                \
        if (through && !ragged) CS_GO(BS, NV, true, false); \
        else if (through) CS_GO(BS, NV, true, true);    \
        else if (!ragged) CS_GO(BS, NV, false, false);  \
        else CS_GO(BS, NV, false, true);                \
    } while (0)
    // (Holding the one-wavefront form of 8 vectors to 128 registers as well, for four wavefronts per SIMD instead of
    // three, measured worse: [32, 4096, 4096] fp16 261 -> 301 us, [32, 4095, 4095] 285 -> 492 us.)
    // Rows of 16 385-32 768 elements: 512 lanes x 8 vectors, held to 128 registers so that a compute unit has two rows in
    // hand and one row's arithmetic overlaps the other's loads and stores.  1024 lanes x 4 vectors (one row per unit, its
    // phases strictly one after the other) measured, fp16: [64, 512, 20480] 644 -> 430 us (52 -> 77 %), [64, 512, 32768]
    // 945 -> 768 us, [2, 20480, 20480] 682 -> 454 us, [1, 32768, 32768] 723 -> 583 us.
    // (causal_softmax_held with 5, 6 or 8 raw vectors per lane, three or four workgroups per unit, on these rows:
    // [64, 512, 20480] 472 against 427 us, [64, 512, 24576] 578 against 527 us, [64, 512, 32768] 862 against 807 us.)
    // (A lane count taken from the launch, so that a row of 10240 elements gets 320 lanes x 4 vectors instead of
    // 512 x 4, measured worse, not better: [64, 512, 10240] fp16 364 against 237 us, [64, 512, 20480] 763
    // against 647 us - workgroups of 5, 10 or 12 wavefronts sit unevenly on a compute unit's four SIMDs.)
    // Rows that do not start on 128-byte boundaries, or are no multiple of 8 elements long, take the ragged form of the
    // same kernels.  Measured on MI355X, fp16, us (in brackets the element kernel, which used to take the unaligned ones,
    // and the plain form, which used to take those on 16-byte boundaries):
    //   [32, 4095, 4095]  285 (1033)   [32, 1024, 4099]  85 (392)   [64, 512, 1027]  24 (78)   [256, 128, 333]  18 (45)
    //   [32, 4088, 4088]  278 (360)    [32, 4100, 4104]  281 (450)  [32, 2048, 2056]  74 (100)  [128, 1000, 1000]  72 (83)
    // Lanes x vectors per lane: the tightest fit, with the fewer lanes where two fit equally.  Every shape that covers
    // the row was timed at 28 row lengths, square causal matrices [h, n, n] and chunks of 512 queries [h, 512, n], fp16
    // (us, this ladder against the powers of two - 64 x 8, 256 x 2, 256 x 4, 512 x 4, 512 x 8 - it replaces):
    //   n = 1536   75 /  77      2560  206 / 229     3500  285 / 323     5000  271 / 312     6144  257 / 272
    //   n = 9000  256 / 365     10240  256 / 331    12288  220 / 257    14000  204 / 228    20480  213 / 225   (square)
    //   n = 2560  167 / 179      5120  165 / 180     9216  160 / 207    10240  166 / 192    12288  171 / 183   (512 queries)
    // (512 lanes x 7 vectors is the one shape to stay away from: 354-611 us where 512 x 6 and 512 x 8 take 308-429.)
    const bool mostly_masked = d.seq * 2 > d.total;// a causal square: half of every matrix is masked
    if (cover <= 64) CS_LAUNCH(64, 1);
    else if (cover <= 128) CS_LAUNCH(64, 2);
    else if (cover <= 192) CS_LAUNCH(64, 3);
    else if (cover <= 256 && !ragged && !T::kPackedMinMax) CS_LAUNCH(128, 2);// bf16 rows of 2048 in whole lines: 257 against 269 us
                                                                              // (fp16 264 / 269 at seq 2048, 158 / 155 at seq 512; ragged 2047: 299 / 281)
    else if (cover <= 256) CS_LAUNCH(64, 4);
    else if (cover <= 384) CS_LAUNCH(64, 6);
    else if (cover <= 512 && mostly_masked) CS_LAUNCH(128, 4);// [33, 4000, 4000] 260 against 273 us with 256 x 2; [32, 4096, 4096] 259-261 either way
    else if (cover <= 512) CS_LAUNCH(256, 2);                 // [128, 512, 4096] 155 against 163 us with 128 x 4
    else if (cover <= 640) CS_LAUNCH(128, 5);
    else if (cover <= 768) CS_LAUNCH(256, 3);
    else if (cover <= 1024) CS_LAUNCH(256, 4);
    else if (cover <= 1280) CS_LAUNCH(256, 5);
    else if (cover <= 1536) CS_LAUNCH(256, 6);
    else if (cover <= 1792) CS_LAUNCH(256, 7);
    else if (cover <= 2048) CS_LAUNCH(256, 8);
    else if (cover <= 2560) CS_LAUNCH(512, 5);
    else if (cover <= 3072) CS_LAUNCH(512, 6);
    else CS_LAUNCH(512, 8);
#undef CS_LAUNCH
#undef CS_GO
}

}// namespace
}// namespace causal_softmax_kernels

#endif
