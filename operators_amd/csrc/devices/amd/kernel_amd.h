// Device-side building blocks for the gfx950 kernels: 128-bit global access,
// 16-bit <-> fp32 conversion with the reference's rounding, and wavefront /
// workgroup reductions for 64-wide wavefronts.  Include from .hip files only.
#ifndef INFINIOP_AMD_KERNEL_H
#define INFINIOP_AMD_KERNEL_H

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace amd {

constexpr int kWave = 64;// CDNA wavefront width

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// ---- kernel arguments, all at once -----------------------------------------
// A wavefront reads its kernel arguments with scalar loads, and the compiler
// places each load in the block that first uses the value: a kernel that
// tests one argument, leaves early on it, then tests a second before it
// reaches the rest pays three memory round trips in a row before its first
// vector load goes out.  The first wavefronts of every launch miss the scalar
// cache on each.  Measured on MI355X on a 42 MB copy: 8.41 us in that shape
// against 8.12 us with one round trip (13.01 against 12.49 us at 71 MB).
// AMD_ARGS_NOW(a, b, ...) at the top of a kernel names the arguments as
// scalar-register inputs of an empty asm statement, so all their loads are
// issued together in the entry block and waited for once.  Up to 30 values of
// 4 or 8 bytes (an asm statement takes no more; two statements would be
// waited for one after the other); it emits no instruction of its own.
#define AMD_ARG_IN(x) "s"(x)
#define AMD_ARGS_1(a) AMD_ARG_IN(a)
#define AMD_ARGS_2(a, ...) AMD_ARG_IN(a), AMD_ARGS_1(__VA_ARGS__)
#define AMD_ARGS_3(a, ...) AMD_ARG_IN(a), AMD_ARGS_2(__VA_ARGS__)
#define AMD_ARGS_4(a, ...) AMD_ARG_IN(a), AMD_ARGS_3(__VA_ARGS__)
#define AMD_ARGS_5(a, ...) AMD_ARG_IN(a), AMD_ARGS_4(__VA_ARGS__)
#define AMD_ARGS_6(a, ...) AMD_ARG_IN(a), AMD_ARGS_5(__VA_ARGS__)
#define AMD_ARGS_7(a, ...) AMD_ARG_IN(a), AMD_ARGS_6(__VA_ARGS__)
#define AMD_ARGS_8(a, ...) AMD_ARG_IN(a), AMD_ARGS_7(__VA_ARGS__)
#define AMD_ARGS_9(a, ...) AMD_ARG_IN(a), AMD_ARGS_8(__VA_ARGS__)
#define AMD_ARGS_10(a, ...) AMD_ARG_IN(a), AMD_ARGS_9(__VA_ARGS__)
#define AMD_ARGS_11(a, ...) AMD_ARG_IN(a), AMD_ARGS_10(__VA_ARGS__)
#define AMD_ARGS_12(a, ...) AMD_ARG_IN(a), AMD_ARGS_11(__VA_ARGS__)
#define AMD_ARGS_13(a, ...) AMD_ARG_IN(a), AMD_ARGS_12(__VA_ARGS__)
#define AMD_ARGS_14(a, ...) AMD_ARG_IN(a), AMD_ARGS_13(__VA_ARGS__)
#define AMD_ARGS_15(a, ...) AMD_ARG_IN(a), AMD_ARGS_14(__VA_ARGS__)
#define AMD_ARGS_16(a, ...) AMD_ARG_IN(a), AMD_ARGS_15(__VA_ARGS__)
#define AMD_ARGS_17(a, ...) AMD_ARG_IN(a), AMD_ARGS_16(__VA_ARGS__)
#define AMD_ARGS_18(a, ...) AMD_ARG_IN(a), AMD_ARGS_17(__VA_ARGS__)
#define AMD_ARGS_19(a, ...) AMD_ARG_IN(a), AMD_ARGS_18(__VA_ARGS__)
#define AMD_ARGS_20(a, ...) AMD_ARG_IN(a), AMD_ARGS_19(__VA_ARGS__)
#define AMD_ARGS_21(a, ...) AMD_ARG_IN(a), AMD_ARGS_20(__VA_ARGS__)
#define AMD_ARGS_22(a, ...) AMD_ARG_IN(a), AMD_ARGS_21(__VA_ARGS__)
#define AMD_ARGS_23(a, ...) AMD_ARG_IN(a), AMD_ARGS_22(__VA_ARGS__)
#define AMD_ARGS_24(a, ...) AMD_ARG_IN(a), AMD_ARGS_23(__VA_ARGS__)
#define AMD_ARGS_25(a, ...) AMD_ARG_IN(a), AMD_ARGS_24(__VA_ARGS__)
#define AMD_ARGS_26(a, ...) AMD_ARG_IN(a), AMD_ARGS_25(__VA_ARGS__)
#define AMD_ARGS_27(a, ...) AMD_ARG_IN(a), AMD_ARGS_26(__VA_ARGS__)
#define AMD_ARGS_28(a, ...) AMD_ARG_IN(a), AMD_ARGS_27(__VA_ARGS__)
#define AMD_ARGS_29(a, ...) AMD_ARG_IN(a), AMD_ARGS_28(__VA_ARGS__)
#define AMD_ARGS_30(a, ...) AMD_ARG_IN(a), AMD_ARGS_29(__VA_ARGS__)
#define AMD_ARGS_PICK(_1, _2, _3, _4, _5, _6, _7, _8, _9, _10, _11, _12, _13, _14, _15, _16, _17, _18, _19, _20, _21, _22, _23, _24, _25, _26, _27, _28, _29, _30, N, ...) N
#define AMD_ARGS_NAMES AMD_ARGS_30, AMD_ARGS_29, AMD_ARGS_28, AMD_ARGS_27, AMD_ARGS_26, AMD_ARGS_25, AMD_ARGS_24, AMD_ARGS_23, AMD_ARGS_22, AMD_ARGS_21, AMD_ARGS_20, AMD_ARGS_19, AMD_ARGS_18, AMD_ARGS_17, AMD_ARGS_16, AMD_ARGS_15, AMD_ARGS_14, AMD_ARGS_13, AMD_ARGS_12, AMD_ARGS_11, AMD_ARGS_10, AMD_ARGS_9, AMD_ARGS_8, AMD_ARGS_7, AMD_ARGS_6, AMD_ARGS_5, AMD_ARGS_4, AMD_ARGS_3, AMD_ARGS_2, AMD_ARGS_1
#define AMD_ARGS_CALL(pick, ...) pick(__VA_ARGS__)
#define AMD_ARGS_NOW(...) asm volatile("" ::AMD_ARGS_CALL(AMD_ARGS_PICK, __VA_ARGS__, AMD_ARGS_NAMES)(__VA_ARGS__))

// ---- division by a number the host knows -----------------------------------
// Division of n < 2^31 by a divisor 1 <= d < 2^31 known on the host, as a
// multiply, an add and a shift (Granlund and Montgomery's round-up form:
// shift = ceil(log2 d), mul = floor(2^32 (2^shift - d) / d) + 1,
// n / d = (hi32(n * mul) + n) >> shift; the sum stays below 2^32 because
// n < 2^31).  A run-time 32-bit division costs a kernel about 25 vector
// instructions and a reciprocal that the compiler hoists in front of the
// first load of every wavefront.
struct FastDiv {
    uint32_t mul, shift;
};
constexpr uint64_t kFastDivLimit = 1ull << 31;// operands and divisors must be below this
inline FastDiv fast_div(uint32_t d) {
    if (d == 0) return FastDiv{0, 0};// nothing to divide by: the caller has no work to launch
    uint32_t shift = 0;
    while ((1ull << shift) < d) ++shift;
    return FastDiv{static_cast<uint32_t>((((1ull << shift) - d) << 32) / d + 1), shift};
}
__host__ __device__ __forceinline__ uint32_t fast_quotient(uint32_t n, FastDiv d) {
    return (static_cast<uint32_t>((static_cast<uint64_t>(n) * d.mul) >> 32) + n) >> d.shift;// the high half of a 32 x 32 bit product: one instruction
}
// two 4-byte kernel arguments that lie side by side, as one operand of AMD_ARGS_NOW
__device__ __forceinline__ uint64_t arg_pair(uint32_t lo, uint32_t hi) { return lo | static_cast<uint64_t>(hi) << 32; }
__device__ __forceinline__ uint64_t arg_pair(FastDiv f) { return arg_pair(f.mul, f.shift); }

// ---- 128-bit global access ------------------------------------------------
// One lane moves 16 bytes; a wavefront moves 1 KiB per instruction.  Streaming
// operands are touched exactly once, so loads and stores carry the
// non-temporal hint and do not displace reusable lines (weights, tables) from
// L2.  Measured on MI355X at the 8192-token sizes: dropping the hint from the
// loads or from the stores costs about 3 % of bandwidth each.
__device__ __forceinline__ u32x4 ld16_stream(const void *p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
}
__device__ __forceinline__ void st16_stream(void *p, u32x4 v) {
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(p));
}
__device__ __forceinline__ u32x4 ld16(const void *p) {
    return *reinterpret_cast<const u32x4 *>(p);
}
// 16 bytes at any 2-byte boundary (gfx950 serves global accesses at any
// alignment, at a fraction of the aligned rate): for the kernels that take
// what the vector kernels refuse.
typedef u32x4 __attribute__((aligned(2))) u32x4_any;
typedef f32x4 __attribute__((aligned(4))) f32x4_any;
__device__ __forceinline__ u32x4 ld16_any(const void *p) {
    return *reinterpret_cast<const u32x4_any *>(p);
}
__device__ __forceinline__ void st16_any(void *p, u32x4 v) {
    *reinterpret_cast<u32x4_any *>(p) = v;
}
__device__ __forceinline__ f32x4 ld16f(const float *p) {
    return *reinterpret_cast<const f32x4 *>(p);
}

// Streaming stores of kernels that write one byte per byte they read
// (RMSNorm, RoPE, CausalSoftmax, Rearrange).  With THROUGH set the store
// carries the cache policy "sc1 nt" - written through L2 instead of waiting
// there for eviction - which HIP source can only express through a buffer
// store: the address is a wavefront-uniform base (kept in scalar registers as
// a buffer resource covering 4 GiB from there) plus a 32-bit byte offset per
// lane.  Measured on MI355X with a 128 MiB copy: 41.5 us against 42.3 us with
// plain "nt" stores (in place: 41.4 against 42.6).  Outputs that L2 can absorb
// are better left to it (a 16 MiB RoPE: 9.2 us with "nt", 9.9 us written
// through), so hosts choose THROUGH from the output size (kWriteThroughBytes
// in common_amd.h; a template parameter because a run-time flag costs the
// unrolled store sequences about 1 %).  Kernels that read two bytes per byte
// written (Add, SwiGLU) lose 2 % when writing through and keep st16_stream.
template<bool THROUGH>
struct StreamOut {
    __amdgpu_buffer_rsrc_t rsrc;
    // base must be the same for every lane of the wavefront
    __device__ __forceinline__ explicit StreamOut(void *base)
        : rsrc(__builtin_amdgcn_make_buffer_rsrc(base, 0, -1, 0x00020000)) {}
    __device__ __forceinline__ void st16(uint32_t byte_offset, u32x4 v) const {
        if constexpr (THROUGH) {
            __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, static_cast<int>(byte_offset), 0, /* sc1 | nt */ 16 | 2);
        } else {
            __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, static_cast<int>(byte_offset), 0, /* nt */ 2);
        }
    }
};

// ---- fp32 -> fp16 exactly as the reference's CPU path narrows --------------
// The reference truncates the mantissa (round toward zero), produces
// subnormals by a truncating shift, maps NaN to sign|0x7E00, +-Inf and any
// exponent >= 31 to sign|0x7C00, and does not guard exponents 16..30, whose
// bits spill upward and are cut to 16 bits
// (reference src/devices/cpu/common_cpu.cc:41-64).  This is that rule for any
// input, in integer arithmetic.
__device__ __forceinline__ uint32_t narrow_f16_any(float v) {
    const uint32_t u = __float_as_uint(v);
    const uint32_t s = (u >> 16) & 0x8000u;
    const int e = static_cast<int>((u >> 23) & 0xFFu) - 127;
    uint32_t m = u & 0x7FFFFFu;
    if (e >= 31) return (e == 128 && m != 0) ? (s | 0x7E00u) : (s | 0x7C00u);
    if (e >= -14) return (s | (static_cast<uint32_t>(e + 15) << 10) | (m >> 13)) & 0xFFFFu;
    if (e >= -24) {
        m = (m | 0x800000u) >> static_cast<uint32_t>(-14 - e);
        return s | (m >> 13);
    }
    return s;
}

// True when the hardware round-toward-zero pack gives the reference's bits:
// every finite |v| < 65536 (normal, subnormal or zero result).
__device__ __forceinline__ bool f16_fast_ok(float v) {
    return (__float_as_uint(v) & 0x7FFFFFFFu) < 0x47800000u;
}

// ---- element traits ---------------------------------------------------------
// widen2: the two 16-bit elements of one 32-bit word -> two floats (exact).
// narrow2: two floats -> one 32-bit word, with the type's rounding rule.
struct F16Ref {
    static constexpr bool kNeedsFixup = true;
    // two elements compared at once in their own format (v_pk_max_f16, v_pk_min_f16)
    static constexpr bool kPackedMinMax = true;
    typedef f16x2 pair;
    __device__ static __forceinline__ pair as_pair(uint32_t w) { return __builtin_bit_cast(f16x2, w); }
    __device__ static __forceinline__ pair splat(float v) { return f16x2{static_cast<_Float16>(v), static_cast<_Float16>(v)}; }
    __device__ static __forceinline__ pair max2(pair a, pair b) { return __builtin_elementwise_max(a, b); }
    __device__ static __forceinline__ pair min2(pair a, pair b) { return __builtin_elementwise_min(a, b); }
    __device__ static __forceinline__ float first(pair p) { return static_cast<float>(p.x); }
    __device__ static __forceinline__ float second(pair p) { return static_cast<float>(p.y); }
    __device__ static __forceinline__ float lo(uint32_t w) {
        return static_cast<float>(__builtin_bit_cast(f16x2, w).x);
    }
    __device__ static __forceinline__ float hi(uint32_t w) {
        return static_cast<float>(__builtin_bit_cast(f16x2, w).y);
    }
    __device__ static __forceinline__ float one(uint16_t h) {
        return static_cast<float>(__builtin_bit_cast(_Float16, h));
    }
    // v_cvt_pkrtz_f16_f32: round toward zero, subnormals kept.
    __device__ static __forceinline__ uint32_t narrow2_fast(float a, float b) {
        return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
    }
    __device__ static __forceinline__ uint32_t narrow2_any(float a, float b) {
        return narrow_f16_any(a) | (narrow_f16_any(b) << 16);
    }
    __device__ static __forceinline__ bool fast_ok(float v) { return f16_fast_ok(v); }
    __device__ static __forceinline__ uint16_t narrow1(float a) {
        return static_cast<uint16_t>(narrow_f16_any(a));
    }
};

// bf16 is this back end's extension (the reference accepts it in none of the
// four operators): exact widening, round-to-nearest-even narrowing
// (v_cvt_pk_bf16_f32 on gfx950); NaN stays NaN.
struct BF16Rne {
    static constexpr bool kNeedsFixup = false;
    static constexpr bool kPackedMinMax = false;// no packed bf16 comparison on this part
    typedef uint32_t pair;
    __device__ static __forceinline__ float lo(uint32_t w) { return __uint_as_float(w << 16); }
    __device__ static __forceinline__ float hi(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }
    __device__ static __forceinline__ float one(uint16_t h) {
        return __uint_as_float(static_cast<uint32_t>(h) << 16);
    }
    __device__ static __forceinline__ uint32_t narrow2_fast(float a, float b) {
        f32x2 v = {a, b};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
    }
    __device__ static __forceinline__ uint32_t narrow2_any(float a, float b) { return narrow2_fast(a, b); }
    __device__ static __forceinline__ bool fast_ok(float) { return true; }
    __device__ static __forceinline__ uint16_t narrow1(float a) {
        return __builtin_bit_cast(uint16_t, static_cast<__bf16>(a));
    }
};

// The integer rule applied to eight values.  Deliberately not inlined: it is
// reached only when a value leaves the hardware pack's exact domain, and one
// shared copy keeps the kernels that narrow several times small.
template<typename T>
__device__ __attribute__((noinline)) u32x4 narrow8_any(float r0, float r1, float r2, float r3, float r4, float r5, float r6, float r7) {
    u32x4 out;
    out.x = T::narrow2_any(r0, r1);
    out.y = T::narrow2_any(r2, r3);
    out.z = T::narrow2_any(r4, r5);
    out.w = T::narrow2_any(r6, r7);
    return out;
}

// Eight results -> one 128-bit word.  For fp16 the hardware pack is used when
// all eight are inside its exact domain; the test is made wave-uniform with a
// ballot so the rare integer path costs nothing when no lane needs it.
template<typename T>
__device__ __forceinline__ u32x4 narrow8(const float (&r)[8]) {
    u32x4 out;
    out.x = T::narrow2_fast(r[0], r[1]);
    out.y = T::narrow2_fast(r[2], r[3]);
    out.z = T::narrow2_fast(r[4], r[5]);
    out.w = T::narrow2_fast(r[6], r[7]);
    if constexpr (T::kNeedsFixup) {
        uint32_t worst = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t mag = __float_as_uint(r[i]) & 0x7FFFFFFFu;
            worst = mag > worst ? mag : worst;
        }
        if (__builtin_amdgcn_ballot_w64(worst >= 0x47800000u) != 0) {
            out = narrow8_any<T>(r[0], r[1], r[2], r[3], r[4], r[5], r[6], r[7]);
        }
    }
    return out;
}

// Eight results known to lie in [0, 1] (or to be NaN): the hardware pack alone.
// Nothing in that range reaches the magnitudes where the reference's
// conversion departs from round-toward-zero.
template<typename T>
__device__ __forceinline__ u32x4 narrow8_unit_range(const float (&r)[8]) {
    u32x4 out;
    out.x = T::narrow2_fast(r[0], r[1]);
    out.y = T::narrow2_fast(r[2], r[3]);
    out.z = T::narrow2_fast(r[4], r[5]);
    out.w = T::narrow2_fast(r[6], r[7]);
    return out;
}

template<typename T>
__device__ __forceinline__ void widen8(u32x4 v, float (&r)[8]) {
    r[0] = T::lo(v.x);
    r[1] = T::hi(v.x);
    r[2] = T::lo(v.y);
    r[3] = T::hi(v.y);
    r[4] = T::lo(v.z);
    r[5] = T::hi(v.z);
    r[6] = T::lo(v.w);
    r[7] = T::hi(v.w);
}

// ---- reductions -------------------------------------------------------------
// Sum over the 64 lanes of a wavefront with DPP cross-lane adds: four steps
// inside each row of 16 lanes, then row broadcasts 15 and 31; the total lands
// in lane 63 and is read back to every lane through an SGPR.
__device__ __forceinline__ float wave_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));// quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));// quad_perm [2,3,0,1]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, false));// row_half_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, false));// row_mirror
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xA, 0xF, false));// row_bcast:15 -> rows 1,3
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xC, 0xF, false));// row_bcast:31 -> rows 2,3
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Maximum over the 64 lanes of a wavefront, same lane pattern as wave_sum.
// Lanes the row broadcasts do not reach keep their own value (old = v).
__device__ __forceinline__ float wave_max(float v) {
    const auto step = [](float x, float other) { return fmaxf(x, other); };
    const int b0 = __builtin_bit_cast(int, v);
    v = step(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(b0, b0, 0xB1, 0xF, 0xF, false)));
    int b = __builtin_bit_cast(int, v);
    v = step(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(b, b, 0x4E, 0xF, 0xF, false)));
    b = __builtin_bit_cast(int, v);
    v = step(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(b, b, 0x141, 0xF, 0xF, false)));
    b = __builtin_bit_cast(int, v);
    v = step(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(b, b, 0x140, 0xF, 0xF, false)));
    b = __builtin_bit_cast(int, v);
    v = step(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(b, b, 0x142, 0xA, 0xF, false)));
    b = __builtin_bit_cast(int, v);
    v = step(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(b, b, 0x143, 0xC, 0xF, false)));
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Reductions over groups of P = 8, 16 or 32 neighbouring lanes (short rows that
// share a wavefront): the first steps of wave_sum and wave_max, stopped at the
// group's width; every lane of a group ends up with the group's result.  They
// combine the same values in the same order as the full trees do when the
// lanes beyond the row hold zeros (or -inf for the maximum), so a short row
// gets the bits it would get with a wavefront to itself.
template<int P>
__device__ __forceinline__ float segment_sum(float v) {
    static_assert(P == 8 || P == 16 || P == 32, "lanes per row");
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));// quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));// quad_perm [2,3,0,1]
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, false));// row_half_mirror
    if constexpr (P >= 16) {
        v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, false));// row_mirror
    }
    if constexpr (P == 32) v += __shfl_xor(v, 16);// the neighbouring row of 16 lanes
    return v;
}
template<int P>
__device__ __forceinline__ float segment_max(float v) {
    static_assert(P == 8 || P == 16 || P == 32, "lanes per row");
    int b = __builtin_bit_cast(int, v);
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(b, b, 0xB1, 0xF, 0xF, false)));
    b = __builtin_bit_cast(int, v);
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(b, b, 0x4E, 0xF, 0xF, false)));
    b = __builtin_bit_cast(int, v);
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(b, b, 0x141, 0xF, 0xF, false)));
    if constexpr (P >= 16) {
        b = __builtin_bit_cast(int, v);
        v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(b, b, 0x140, 0xF, 0xF, false)));
    }
    if constexpr (P == 32) v = fmaxf(v, __shfl_xor(v, 16));
    return v;
}

// Maximum over a workgroup; same slot discipline as block_sum below.
template<int WAVES>
__device__ __forceinline__ float block_max(float v, float *slots, int phase) {
    v = wave_max(v);
    if constexpr (WAVES == 1) {
        return v;
    } else {
        float *mine = slots + phase * WAVES;
        const int wave = threadIdx.x / kWave;
        if ((threadIdx.x & (kWave - 1)) == 0) mine[wave] = v;
        __syncthreads();
        float m = mine[0];
#pragma unroll
        for (int i = 1; i < WAVES; ++i) m = fmaxf(m, mine[i]);
        return m;
    }
}

// Sum over a workgroup of WAVES wavefronts.  `slots` is LDS with room for
// 2*WAVES floats; `phase` alternates 0/1 between consecutive calls so that one
// barrier per call is enough (a wave can only overwrite a slot set after every
// wave has passed the barrier that follows the previous use of the other set).
template<int WAVES>
__device__ __forceinline__ float block_sum(float v, float *slots, int phase) {
    v = wave_sum(v);
    if constexpr (WAVES == 1) {
        return v;
    } else {
        float *mine = slots + phase * WAVES;
        const int wave = threadIdx.x / kWave;
        if ((threadIdx.x & (kWave - 1)) == 0) mine[wave] = v;
        __syncthreads();
        float total = 0.0f;
#pragma unroll
        for (int i = 0; i < WAVES; ++i) total += mine[i];
        return total;
    }
}

}// namespace amd

#endif
