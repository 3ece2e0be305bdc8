/*
 * CPU oracle for the InfiniOperators memory-bound LLM path: Add, RMSNorm,
 * RoPE (rotary_embedding) and SwiGLU.
 *
 * THIS FILE IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It restates, in plain
 * C, the arithmetic of the reference's CPU back end so that the gfx950 kernels
 * can be checked against it on machines where the reference sources are not
 * present.  Nothing in the shipped library links or calls it; only the test
 * suite, the smoke check and the benchmark's CPU-baseline leg do.
 *
 * Every function names the reference lines it follows.  Paths are relative to
 * the reference checkout.
 *
 * Pinning status (what independently checks each function):
 *   oracle_f16_to_f32 / oracle_f32_to_f16   pinned  - all 65 536 fp16 codes
 *       against numpy's exact widening; >1e6 fp32 inputs against an ideal
 *       round-toward-zero narrowing built from numpy nextafter; hand probes
 *       for the overflow quirk; the compiled reference where it is available.
 *   oracle_add / oracle_rms_norm / oracle_rope / oracle_swiglu (fp16, and
 *       fp32 for add)                        pinned  - golden vectors written
 *       by the compiled reference, the compiled reference itself where it is
 *       available, plus closed forms (identity elements, constant rows,
 *       pos = 0, norm preservation, b = 0).
 *   oracle_causal_softmax (fp16)             pinned  - golden vectors written
 *       by the compiled reference, the compiled reference itself where it is
 *       available, a float64 softmax, rows summing to one, zeros above the
 *       diagonal.  (This operator is outside the four-operator hot path; it is
 *       the first of the operators that come next.)
 *   oracle_rearrange                         pinned  - golden vectors written by
 *       the compiled reference, the compiled reference itself, numpy's own
 *       strided assignment.  (Second operator beyond the hot path.)
 *   oracle_matmul (fp16, fp32)               pinned  - the compiled reference
 *       itself bit for bit (its own test shapes, row- and column-major
 *       operands, batches, beta != 0), a float64 product, identity and
 *       permutation matrices.  The MLP is the reference's composition of
 *       matmul, swiglu and matmul (src/ops/mlp/operator.cc:22-122), checked
 *       against the compiled reference's MLP bit for bit.
 *   oracle_random_sample (fp16)              pinned  - golden indices written by
 *       the compiled reference (its own nine test cases, ties, special
 *       values), the compiled reference itself on fresh inputs, an independent
 *       argsort/float64 model for tie-free logits, closed forms (tiny topp,
 *       random_val 0 and 1, flat distributions, greedy = argmax).
 *   bf16 variants of the operators           PARITY UNPINNED by the reference:
 *       no reference back end accepts bf16 for these operators.  The bf16
 *       arithmetic here is this project's extension (exact widening, the same
 *       fp32/fp64 formulas, round-to-nearest-even narrowing) and is pinned only
 *       against torch's CPU bf16 arithmetic and the same closed forms.
 *
 * Build with  -O2 -ffp-contract=off -fno-strict-aliasing  and without
 * -ffast-math / -march flags: the reference is compiled for baseline x86-64,
 * so a*b+c is always a separate multiply and add.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))

/* Status codes: include/status.h:4-14 of the reference. */
enum {
    ST_SUCCESS = 0,
    ST_EXECUTION_FAILED = 1,
    ST_BAD_PARAM = 2,
    ST_BAD_TENSOR_DTYPE = 3,
    ST_BAD_TENSOR_SHAPE = 4,
    ST_BAD_TENSOR_STRIDES = 5,
    ST_MEMORY_NOT_ALLOCATED = 6,
    ST_INSUFFICIENT_WORKSPACE = 7,
    ST_BAD_DEVICE = 8,
};

/* Data types as the 32-bit image of the reference's DataLayout bitfield
 * {packed:8, sign:1, size:7, mantissa:8, exponent:8}, include/data_type.h:4-46. */
#define DT_CODE(packed, sign, size, mant, exp) \
    ((uint32_t) (packed) | ((uint32_t) (sign) << 8) | ((uint32_t) (size) << 9) | ((uint32_t) (mant) << 16) | ((uint32_t) (exp) << 24))
#define DT_F16 DT_CODE(1, 1, 2, 10, 5)
#define DT_BF16 DT_CODE(1, 1, 2, 7, 8)
#define DT_F32 DT_CODE(1, 1, 4, 23, 8)
#define DT_U64 DT_CODE(1, 0, 8, 64, 0)

/* A tensor description with the reference's meaning (include/tensor.h:7-18):
 * strides are counted in elements. */
typedef struct {
    uint32_t dt;
    uint64_t ndim;
    const uint64_t *shape;
    const int64_t *strides;
} oracle_tensor;

static inline uint32_t bits_of(float f) {
    uint32_t u;
    memcpy(&u, &f, sizeof u);
    return u;
}
static inline float float_of(uint32_t u) {
    float f;
    memcpy(&f, &u, sizeof f);
    return f;
}

/* ------------------------------------------------------------------------ *
 * Scalar conversions
 * ------------------------------------------------------------------------ */

/* fp16 -> fp32, exact for every code.  Follows src/devices/cpu/common_cpu.cc:3-39:
 * Inf/NaN keep the payload shifted left by 13 (NaNs are NOT quieted), zeros keep
 * their sign, subnormals are renormalised. */
ORACLE_API float oracle_f16_to_f32(uint16_t h) {
    uint32_t s = ((uint32_t) h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1Fu;
    uint32_t m = h & 0x3FFu;
    if (e == 0x1Fu) {
        return float_of(s | 0x7F800000u | (m << 13));
    }
    if (e == 0) {
        if (m == 0) {
            return float_of(s);
        }
        /* subnormal: value = m * 2^-24; shift the leading one up to bit 10 */
        int32_t ue = -14;
        while (!(m & 0x400u)) {
            m <<= 1;
            --ue;
        }
        return float_of(s | ((uint32_t) (ue + 127) << 23) | ((m & 0x3FFu) << 13));
    }
    return float_of(s | ((e + 112u) << 23) | (m << 13));
}

/* fp32 -> fp16 as the reference does it, src/devices/cpu/common_cpu.cc:41-64:
 *  - the mantissa is TRUNCATED (round toward zero), never rounded;
 *  - unbiased exponent >= 31: NaN (exponent 128, mantissa != 0) -> sign|0x7E00,
 *    anything else -> sign|0x7C00;
 *  - unbiased exponent 16..30 is not guarded: (e+15)<<10 is OR-ed in as is and
 *    the 16-bit return type cuts it off, so e == 16 lands on an Inf/NaN
 *    pattern and larger e also sets bit 15;
 *  - unbiased exponent -24..-15 gives a subnormal by shifting, again truncating;
 *  - below that, a signed zero. */
ORACLE_API uint16_t oracle_f32_to_f16(float v) {
    uint32_t u = bits_of(v);
    uint32_t s = (u >> 16) & 0x8000u;
    int32_t e = (int32_t) ((u >> 23) & 0xFFu) - 127;
    uint32_t m = u & 0x7FFFFFu;
    if (e >= 31) {
        return (uint16_t) ((e == 128 && m != 0) ? (s | 0x7E00u) : (s | 0x7C00u));
    }
    if (e >= -14) {
        return (uint16_t) (s | ((uint32_t) (e + 15) << 10) | (m >> 13));
    }
    if (e >= -24) {
        m = (m | 0x800000u) >> (uint32_t) (-14 - e);
        return (uint16_t) (s | (m >> 13));
    }
    return (uint16_t) s;
}

/* bf16 extension (no reference counterpart): exact widening. */
ORACLE_API float oracle_bf16_to_f32(uint16_t h) {
    return float_of((uint32_t) h << 16);
}

/* bf16 extension: round to nearest, ties to even; every NaN becomes 0x7FC0
 * (the convention of torch's CPU conversion, which pins this function). */
ORACLE_API uint16_t oracle_f32_to_bf16(float v) {
    uint32_t u = bits_of(v);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) {
        return 0x7FC0u;
    }
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t) (u >> 16);
}

static inline float load16(uint32_t dt, const uint16_t *p) {
    return dt == DT_F16 ? oracle_f16_to_f32(*p) : oracle_bf16_to_f32(*p);
}
static inline void store16(uint32_t dt, uint16_t *p, float v) {
    *p = dt == DT_F16 ? oracle_f32_to_f16(v) : oracle_f32_to_bf16(v);
}

/* Array forms, used by the tests to sweep many values per call. */
ORACLE_API void oracle_f16_to_f32_array(float *dst, const uint16_t *src, uint64_t n) {
    for (uint64_t i = 0; i < n; ++i) dst[i] = oracle_f16_to_f32(src[i]);
}
ORACLE_API void oracle_f32_to_f16_array(uint16_t *dst, const float *src, uint64_t n) {
    for (uint64_t i = 0; i < n; ++i) dst[i] = oracle_f32_to_f16(src[i]);
}
ORACLE_API void oracle_bf16_to_f32_array(float *dst, const uint16_t *src, uint64_t n) {
    for (uint64_t i = 0; i < n; ++i) dst[i] = oracle_bf16_to_f32(src[i]);
}
ORACLE_API void oracle_f32_to_bf16_array(uint16_t *dst, const float *src, uint64_t n) {
    for (uint64_t i = 0; i < n; ++i) dst[i] = oracle_f32_to_bf16(src[i]);
}

/* ------------------------------------------------------------------------ *
 * Shape helpers shared by the create-time checks
 * ------------------------------------------------------------------------ */

/* src/ops/utils.h:174-188: "contiguous" means strides[i-1] == shape[i]*strides[i]
 * for every i >= 1.  The innermost stride itself is not examined, and a tensor
 * with no dimensions passes. */
static int ref_is_contiguous(const oracle_tensor *t) {
    for (uint64_t i = 1; i < t->ndim; ++i) {
        if (t->strides[i - 1] != (int64_t) t->shape[i] * t->strides[i]) {
            return 0;
        }
    }
    return 1;
}

/* src/ops/utils.h:85-121,141-143: numpy-style broadcast of a and b, right
 * aligned, must give exactly c's shape and c->ndim == max(a->ndim, b->ndim). */
static int ref_broadcast_ok(const oracle_tensor *a, const oracle_tensor *b, const oracle_tensor *c) {
    uint64_t rank = a->ndim > b->ndim ? a->ndim : b->ndim;
    if (rank != c->ndim) {
        return 0;
    }
    for (uint64_t i = 0; i < rank; ++i) {
        uint64_t da = i < rank - a->ndim ? 1 : a->shape[i - (rank - a->ndim)];
        uint64_t db = i < rank - b->ndim ? 1 : b->shape[i - (rank - b->ndim)];
        if (!(da == db || da == 1 || db == 1)) {
            return 0;
        }
        if ((da > db ? da : db) != c->shape[i]) {
            return 0;
        }
    }
    return 1;
}

/* ------------------------------------------------------------------------ *
 * Add
 * ------------------------------------------------------------------------ */

/* Create-time checks of src/ops/add/cpu/add_cpu.cc:18-35, in the reference's
 * order: shape, then strides, then dtype.  `allow_bf16` switches on this
 * project's bf16 extension; with 0 the answer is the reference's. */
ORACLE_API int oracle_add_check(const oracle_tensor *c, const oracle_tensor *a, const oracle_tensor *b, int allow_bf16) {
    if (!ref_broadcast_ok(a, b, c)) {
        return ST_BAD_TENSOR_SHAPE;
    }
    if (!ref_is_contiguous(a) || !ref_is_contiguous(b) || !ref_is_contiguous(c)) {
        return ST_BAD_TENSOR_STRIDES;
    }
    if (c->dt != DT_F16 && c->dt != DT_F32 && !(allow_bf16 && c->dt == DT_BF16)) {
        return ST_BAD_TENSOR_DTYPE;
    }
    if (c->dt != a->dt || c->dt != b->dt) {
        return ST_BAD_TENSOR_DTYPE;
    }
    return ST_SUCCESS;
}

/* c = a + b with broadcasting.  Follows src/ops/add/cpu/add_cpu.cc:37-101:
 * c is written in flat row-major order whatever its strides say; a and b are
 * read at sum(index[i] * stride[i]) where stride is the operand's own stride on
 * dimensions it has with c's extent, and 0 on dimensions it lacks or broadcasts.
 * fp16: widen both, add in fp32, narrow by truncation (add_cpu.cc:83);
 * fp32: a plain IEEE add (add_cpu.cc:85); bf16: extension.
 * Supports up to 16 dimensions (the reference has no limit). */
ORACLE_API int oracle_add(const oracle_tensor *c, const oracle_tensor *a, const oracle_tensor *b,
                          void *c_data, const void *a_data, const void *b_data) {
    enum { MAXD = 16 };
    uint64_t nd = c->ndim;
    if (nd > MAXD) {
        return ST_BAD_PARAM;
    }
    int64_t sa[MAXD], sb[MAXD];
    uint64_t idx[MAXD];
    uint64_t total = 1;
    for (uint64_t i = 0; i < nd; ++i) {
        uint64_t lack_a = nd - a->ndim, lack_b = nd - b->ndim;
        sa[i] = (i < lack_a || c->shape[i] != a->shape[i - lack_a]) ? 0 : a->strides[i - lack_a];
        sb[i] = (i < lack_b || c->shape[i] != b->shape[i - lack_b]) ? 0 : b->strides[i - lack_b];
        idx[i] = 0;
        total *= c->shape[i];
    }
    uint32_t dt = c->dt;
    if (dt != DT_F16 && dt != DT_F32 && dt != DT_BF16) {
        return ST_BAD_TENSOR_DTYPE;
    }
    for (uint64_t flat = 0; flat < total; ++flat) {
        int64_t ia = 0, ib = 0;
        for (uint64_t i = 0; i < nd; ++i) {
            ia += (int64_t) idx[i] * sa[i];
            ib += (int64_t) idx[i] * sb[i];
        }
        if (dt == DT_F32) {
            ((float *) c_data)[flat] = ((const float *) a_data)[ia] + ((const float *) b_data)[ib];
        } else {
            float x = load16(dt, (const uint16_t *) a_data + ia);
            float y = load16(dt, (const uint16_t *) b_data + ib);
            store16(dt, (uint16_t *) c_data + flat, x + y);
        }
        /* odometer step over c's shape, last dimension fastest (add_cpu.cc:5-12) */
        for (int64_t i = (int64_t) nd - 1; i >= 0; --i) {
            if (++idx[i] != c->shape[i]) {
                break;
            }
            idx[i] = 0;
        }
    }
    return ST_SUCCESS;
}

/* ------------------------------------------------------------------------ *
 * RMSNorm
 * ------------------------------------------------------------------------ */

/* Create-time checks of src/ops/rms_norm/cpu/rms_norm_cpu.cc:6-17: ranks and
 * extents only.  Data types are not examined at create time. */
ORACLE_API int oracle_rms_norm_check(const oracle_tensor *y, const oracle_tensor *x, const oracle_tensor *w) {
    if (y->ndim != 2 || x->ndim != 2 || w->ndim != 1) {
        return ST_BAD_TENSOR_SHAPE;
    }
    if (x->shape[0] != y->shape[0] || x->shape[1] != y->shape[1] || w->shape[0] != y->shape[1]) {
        return ST_BAD_TENSOR_SHAPE;
    }
    return ST_SUCCESS;
}

/* y[i][j] = x[i][j] * (mean_j x[i][j]^2 + eps)^-1/2 * w[j].
 * Follows src/ops/rms_norm/cpu/rms_norm_cpu.cc:46-86:
 *  - the sum of squares runs left to right in fp32 (:67-71);
 *  - k = pow((float)(sum/d + eps), -0.5) is a DOUBLE (std::pow(float, double)
 *    promotes), with sum/d and "+ eps" both done in fp32 first (:73);
 *  - each output is (k * x) * w evaluated in double, narrowed to fp32, then
 *    to 16 bits (:83);
 *  - w is read as fp16 when its type is F16 and as fp32 otherwise (:57-61,77-81).
 * The reference takes x's row stride from y's descriptor (:20); here both
 * strides are explicit arguments and the caller chooses.
 * dt: DT_F16 (reference) or DT_BF16 (extension; w may then also be bf16). */
ORACLE_API int oracle_rms_norm(uint32_t dt, uint32_t w_dt, uint64_t n, uint64_t d,
                               int64_t stride_y, int64_t stride_x, float eps,
                               void *y, const void *x, const void *w) {
    if (dt != DT_F16 && dt != DT_BF16) {
        return ST_BAD_TENSOR_DTYPE;
    }
    for (uint64_t i = 0; i < n; ++i) {
        const uint16_t *xr = (const uint16_t *) x + (int64_t) i * stride_x;
        uint16_t *yr = (uint16_t *) y + (int64_t) i * stride_y;
        float ss = 0.0f;
        for (uint64_t j = 0; j < d; ++j) {
            float v = load16(dt, xr + j);
            ss += v * v;
        }
        float mean_eps = ss / (float) d + eps;
        double k = pow((double) mean_eps, -0.5);
        for (uint64_t j = 0; j < d; ++j) {
            float v = load16(dt, xr + j);
            float g;
            if (w_dt == DT_F16 || w_dt == DT_BF16) {
                g = load16(w_dt, (const uint16_t *) w + j);
            } else {
                g = ((const float *) w)[j];
            }
            store16(dt, yr + j, (float) (k * (double) v * (double) g));
        }
    }
    return ST_SUCCESS;
}

/* ------------------------------------------------------------------------ *
 * RoPE
 * ------------------------------------------------------------------------ */

/* Create-time checks of src/ops/rotary_embedding/cpu/rotary_embedding_cpu.cc:47-90
 * in the reference's order: ranks, even head dim, extents, unit inner strides,
 * then data types (t F16, tables F32, pos U64).  `allow_bf16` admits bf16 t. */
ORACLE_API int oracle_rope_check(const oracle_tensor *t, const oracle_tensor *pos,
                                 const oracle_tensor *sin_t, const oracle_tensor *cos_t, int allow_bf16) {
    if (t->ndim != 3 || pos->ndim != 1 || sin_t->ndim != 2 || cos_t->ndim != 2) {
        return ST_BAD_TENSOR_SHAPE;
    }
    uint64_t nt = t->shape[0], dh = t->shape[2];
    if (dh % 2 != 0) {
        return ST_BAD_TENSOR_SHAPE;
    }
    if (pos->shape[0] != nt || sin_t->shape[1] != dh || cos_t->shape[1] != dh || sin_t->shape[0] != cos_t->shape[0]) {
        return ST_BAD_TENSOR_SHAPE;
    }
    if (t->strides[2] != 1 || pos->strides[0] != 1 || sin_t->strides[1] != 1 || cos_t->strides[1] != 1) {
        return ST_BAD_TENSOR_STRIDES;
    }
    if (t->dt != DT_F16 && !(allow_bf16 && t->dt == DT_BF16)) {
        return ST_BAD_TENSOR_DTYPE;
    }
    if (sin_t->dt != DT_F32 || cos_t->dt != DT_F32) {
        return ST_BAD_TENSOR_DTYPE;
    }
    if (pos->dt != DT_U64) {
        return ST_BAD_TENSOR_DTYPE;
    }
    return ST_SUCCESS;
}

/* In-place rotation of adjacent pairs.  Follows
 * src/ops/rotary_embedding/cpu/rotary_embedding_cpu.cc:16-44: for token i the
 * table rows start at pos[i]*dh (row stride is dh, never the descriptor's);
 * for pair k of head j
 *     t[2k]   = a*cos[2k]   - b*sin[2k]
 *     t[2k+1] = a*sin[2k+1] + b*cos[2k+1]
 * with a = t[2k], b = t[2k+1] widened to fp32, each product rounded to fp32
 * before the add/subtract, and four separate table reads per pair. */
ORACLE_API int oracle_rope(uint32_t dt, uint64_t nt, uint64_t nh, uint64_t dh,
                           int64_t stride_token, int64_t stride_head,
                           void *t, const uint64_t *pos, const float *sin_t, const float *cos_t) {
    if (dt != DT_F16 && dt != DT_BF16) {
        return ST_BAD_TENSOR_DTYPE;
    }
    if (!t || !pos || !sin_t || !cos_t) {
        return ST_BAD_PARAM;
    }
    for (uint64_t i = 0; i < nt; ++i) {
        const float *sr = sin_t + pos[i] * dh;
        const float *cr = cos_t + pos[i] * dh;
        for (uint64_t j = 0; j < nh; ++j) {
            uint16_t *p = (uint16_t *) t + (int64_t) i * stride_token + (int64_t) j * stride_head;
            for (uint64_t k = 0; k < dh / 2; ++k) {
                float a = load16(dt, p + 2 * k);
                float b = load16(dt, p + 2 * k + 1);
                float s0 = sr[2 * k], c0 = cr[2 * k];
                float s1 = sr[2 * k + 1], c1 = cr[2 * k + 1];
                float ac = a * c0, bs = b * s0;
                float as = a * s1, bc = b * c1;
                store16(dt, p + 2 * k, ac - bs);
                store16(dt, p + 2 * k + 1, as + bc);
            }
        }
    }
    return ST_SUCCESS;
}

/* ------------------------------------------------------------------------ *
 * SwiGLU
 * ------------------------------------------------------------------------ */

/* Create-time checks of src/ops/swiglu/cpu/swiglu_cpu.cc:7-37 in the
 * reference's order: ranks; c's dtype; unit inner strides; then a/b extents and
 * dtypes against c, which report BAD_PARAM.  `allow_bf16` admits bf16. */
ORACLE_API int oracle_swiglu_check(const oracle_tensor *c, const oracle_tensor *a, const oracle_tensor *b, int allow_bf16) {
    if (c->ndim != 2 || a->ndim != 2 || b->ndim != 2) {
        return ST_BAD_TENSOR_SHAPE;
    }
    if (c->dt != DT_F16 && !(allow_bf16 && c->dt == DT_BF16)) {
        return ST_BAD_TENSOR_DTYPE;
    }
    if (a->strides[1] != 1 || b->strides[1] != 1 || c->strides[1] != 1) {
        return ST_BAD_TENSOR_STRIDES;
    }
    if (a->shape[0] != c->shape[0] || a->shape[1] != c->shape[1] || a->dt != c->dt ||
        b->shape[0] != c->shape[0] || b->shape[1] != c->shape[1] || b->dt != c->dt) {
        return ST_BAD_PARAM;
    }
    return ST_SUCCESS;
}

/* c = a * (b / (1 + expf(-b))), src/ops/swiglu/cpu/swiglu_cpu.cc:49-72: b is
 * the gated operand.  All in fp32; expf is the float libm routine.  Each tensor
 * has its own row stride. */
ORACLE_API int oracle_swiglu(uint32_t dt, uint64_t n, uint64_t di,
                             int64_t stride_c, int64_t stride_a, int64_t stride_b,
                             void *c, const void *a, const void *b) {
    if (dt != DT_F16 && dt != DT_BF16) {
        return ST_BAD_TENSOR_DTYPE;
    }
    for (uint64_t i = 0; i < n; ++i) {
        const uint16_t *ar = (const uint16_t *) a + (int64_t) i * stride_a;
        const uint16_t *br = (const uint16_t *) b + (int64_t) i * stride_b;
        uint16_t *cr = (uint16_t *) c + (int64_t) i * stride_c;
        for (uint64_t j = 0; j < di; ++j) {
            float up = load16(dt, ar + j);
            float gate = load16(dt, br + j);
            float act = gate / (1.0f + expf(-gate));
            store16(dt, cr + j, up * act);
        }
    }
    return ST_SUCCESS;
}

/* ------------------------------------------------------------------------ *
 * Causal softmax (next operator after the four-operator path)
 * ------------------------------------------------------------------------ */

/* Create-time checks of src/ops/causal_softmax/cpu/causal_softmax_cpu.cc:6-15:
 * rank 2 or 3, then F16.  `allow_bf16` admits bf16; `unit_inner` additionally
 * demands a unit innermost stride, which the reference's GPU back end does
 * (cuda/causal_softmax.cc:22-24) and its CPU back end does not. */
ORACLE_API int oracle_causal_softmax_check(const oracle_tensor *y, int allow_bf16, int unit_inner) {
    if (y->ndim != 2 && y->ndim != 3) {
        return ST_BAD_TENSOR_SHAPE;
    }
    if (y->dt != DT_F16 && !(allow_bf16 && y->dt == DT_BF16)) {
        return ST_BAD_TENSOR_DTYPE;
    }
    if (unit_inner && y->strides[y->ndim - 1] != 1) {
        return ST_BAD_TENSOR_STRIDES;
    }
    return ST_SUCCESS;
}

/* In-place masked softmax over the last dimension, following
 * src/ops/causal_softmax/cpu/causal_softmax_cpu.cc:52-82.  Row i of a
 * [seq, total] matrix keeps columns j <= total - seq + i (computed in unsigned
 * 64-bit arithmetic, so for total < seq the early rows keep everything) and
 * gets exact zeros elsewhere; the maximum starts from column 0; the sum of
 * expf(x - max) runs left to right in fp32; each output is expf(x - max) / sum
 * recomputed, then narrowed. */
ORACLE_API int oracle_causal_softmax(uint32_t dt, uint64_t batch, uint64_t seq, uint64_t total,
                                     int64_t stride_b, int64_t stride_i, int64_t stride_j, void *data) {
    if (dt != DT_F16 && dt != DT_BF16) {
        return ST_BAD_TENSOR_DTYPE;
    }
    uint16_t *y = (uint16_t *) data;
    for (uint64_t b = 0; b < batch; ++b) {
        for (uint64_t i = 0; i < seq; ++i) {
            uint16_t *row = y + (int64_t) b * stride_b + (int64_t) i * stride_i;
            const uint64_t last = total - seq + i; /* wraps when total < seq, as in the reference */
            float mx = load16(dt, row);
            for (uint64_t j = 1; j < total; ++j) {
                if (j <= last) {
                    float v = load16(dt, row + (int64_t) j * stride_j);
                    mx = v > mx ? v : mx; /* std::max(a, b): b only if a < b */
                } else {
                    row[(int64_t) j * stride_j] = 0;
                }
            }
            float sum = 0.0f;
            for (uint64_t j = 0; j < total && j <= last; ++j) {
                sum += expf(load16(dt, row + (int64_t) j * stride_j) - mx);
            }
            for (uint64_t j = 0; j < total && j <= last; ++j) {
                float e = expf(load16(dt, row + (int64_t) j * stride_j) - mx) / sum;
                store16(dt, row + (int64_t) j * stride_j, e);
            }
        }
    }
    return ST_SUCCESS;
}

/* ------------------------------------------------------------------------ *
 * Rearrange (strided copy; second operator after the four-operator path)
 * ------------------------------------------------------------------------ */

/* Create-time checks of src/ops/rearrange/cpu/rearrange_cpu.cc:7-54 in the
 * reference's order: equal element types; equal, non-zero rank and equal
 * extents; unit innermost strides; for rank >= 4, dimensions 1..rank-3 must
 * nest inside their predecessor (shape[i]*stride[i] == stride[i-1]) in both
 * tensors. */
ORACLE_API int oracle_rearrange_check(const oracle_tensor *dst, const oracle_tensor *src) {
    if (dst->dt != src->dt) {
        return ST_BAD_TENSOR_DTYPE;
    }
    uint64_t nd = dst->ndim;
    if (src->ndim != nd || nd == 0) {
        return ST_BAD_TENSOR_SHAPE;
    }
    for (uint64_t i = 0; i < nd; ++i) {
        if (dst->shape[i] != src->shape[i]) {
            return ST_BAD_TENSOR_SHAPE;
        }
    }
    if (dst->strides[nd - 1] != 1 || src->strides[nd - 1] != 1) {
        return ST_BAD_TENSOR_STRIDES;
    }
    if (nd >= 4) {
        for (int64_t i = (int64_t) nd - 3; i >= 1; --i) {
            if ((int64_t) dst->shape[i] * dst->strides[i] != dst->strides[i - 1] ||
                (int64_t) src->shape[i] * src->strides[i] != src->strides[i - 1]) {
                return ST_BAD_TENSOR_STRIDES;
            }
        }
    }
    return ST_SUCCESS;
}

/* dst[index] = src[index] for every index, rows of the innermost dimension
 * moved as blocks of bytes (rearrange_cpu.cc:70-92).  Strides in elements of
 * elem_size bytes.  Up to 16 dimensions. */
ORACLE_API int oracle_rearrange(uint32_t elem_size, uint64_t ndim, const uint64_t *shape,
                                const int64_t *dst_strides, const int64_t *src_strides,
                                void *dst, const void *src) {
    if (ndim == 0 || ndim > 16) {
        return ST_BAD_TENSOR_SHAPE;
    }
    uint64_t rows = 1;
    for (uint64_t i = 0; i + 1 < ndim; ++i) {
        rows *= shape[i];
    }
    const uint64_t row_bytes = shape[ndim - 1] * elem_size;
    for (uint64_t r = 0; r < rows; ++r) {
        int64_t od = 0, os = 0;
        uint64_t rest = r;
        for (int64_t j = (int64_t) ndim - 2; j >= 0; --j) {
            uint64_t k = rest % shape[j];
            rest /= shape[j];
            od += (int64_t) k * dst_strides[j];
            os += (int64_t) k * src_strides[j];
        }
        memcpy((uint8_t *) dst + od * (int64_t) elem_size, (const uint8_t *) src + os * (int64_t) elem_size, row_bytes);
    }
    return ST_SUCCESS;
}

/* ------------------------------------------------------------------------ *
 * Matmul (third operator beyond the four-operator path, with the MLP that is
 * built on it)
 * ------------------------------------------------------------------------ */

/* c = alpha * a @ b + beta * c, src/ops/matmul/cpu/matmul_cpu.cc:47-82: per
 * output element a running fp32 sum over k of widened products, in index
 * order; then f32_to_f16(alpha * sum) when beta == 0 (c is not read), else
 * f32_to_f16(beta * c + alpha * sum).  fp32 data: beta * c + alpha * sum
 * always.  Each operand: `batch` matrices `*_sb` elements apart (0 when the
 * operand has one matrix for every batch), element (i, j) at i * rs + j * cs.
 * The reference's transposition trick (blas.h:100-106) changes the order in
 * which outputs are visited, not what is computed for any of them. */
ORACLE_API int oracle_matmul(uint32_t dt, uint64_t batch, uint64_t m, uint64_t n, uint64_t k,
                             int64_t c_sb, int64_t c_rs, int64_t c_cs,
                             int64_t a_sb, int64_t a_rs, int64_t a_cs,
                             int64_t b_sb, int64_t b_rs, int64_t b_cs,
                             float alpha, float beta, void *c, const void *a, const void *b) {
    if (dt != DT_F16 && dt != DT_F32 && dt != DT_BF16) {
        return ST_BAD_TENSOR_DTYPE;
    }
    for (uint64_t i = 0; i < batch; ++i) {
        for (uint64_t r = 0; r < m; ++r) {
            for (uint64_t q = 0; q < n; ++q) {
                const int64_t oc = (int64_t) i * c_sb + (int64_t) r * c_rs + (int64_t) q * c_cs;
                float sum = 0;
                for (uint64_t t = 0; t < k; ++t) {
                    const int64_t oa = (int64_t) i * a_sb + (int64_t) r * a_rs + (int64_t) t * a_cs;
                    const int64_t ob = (int64_t) i * b_sb + (int64_t) t * b_rs + (int64_t) q * b_cs;
                    if (dt == DT_F32) {
                        sum += ((const float *) a)[oa] * ((const float *) b)[ob];
                    } else {
                        sum += load16(dt, (const uint16_t *) a + oa) * load16(dt, (const uint16_t *) b + ob);
                    }
                }
                if (dt == DT_F32) {
                    float *pc = (float *) c + oc;
                    *pc = beta * (*pc) + alpha * sum;
                } else {
                    uint16_t *pc = (uint16_t *) c + oc;
                    if (beta == 0) {
                        store16(dt, pc, alpha * sum);
                    } else {
                        store16(dt, pc, beta * load16(dt, pc) + alpha * sum);
                    }
                }
            }
        }
    }
    return ST_SUCCESS;
}

/* ------------------------------------------------------------------------ *
 * RandomSample (fourth operator beyond the four-operator path)
 * ------------------------------------------------------------------------ */

/* Create-time checks of src/ops/random_sample/cpu/random_sample.cc:7-33 in the
 * reference's order: probs of rank 1; probs F16; result U64; result refused
 * only when it is neither of rank 1 nor has a first extent of 1.  A result
 * with no dimensions (whose first extent the reference reads anyway) counts
 * as a scalar here and passes. */
ORACLE_API int oracle_random_sample_check(const oracle_tensor *result, const oracle_tensor *probs, int allow_bf16) {
    if (probs->ndim != 1) {
        return ST_BAD_TENSOR_SHAPE;
    }
    if (probs->dt != DT_F16 && !(allow_bf16 && probs->dt == DT_BF16)) {
        return ST_BAD_TENSOR_DTYPE;
    }
    if (result->dt != DT_U64) {
        return ST_BAD_TENSOR_DTYPE;
    }
    if (result->ndim != 1 && result->ndim != 0 && result->shape[0] != 1) {
        return ST_BAD_TENSOR_SHAPE;
    }
    return ST_SUCCESS;
}

/* src/ops/random_sample/cpu/random_sample.cc:47-171.  `logits` and `order`
 * are the caller's scratch of voc entries each (the reference carves them out
 * of its workspace).  Returns 1 when result[0] was written, 0 when it was
 * left alone (the last loop of the sampling form found no entry, which
 * happens for random_val >= 1 or NaN probabilities).
 *
 * Sampling form (topp > 0 and topk > 1): a partial selection sort moves the
 * topk largest codes to the front in descending order - position i is swapped
 * with every later position holding a strictly greater value, and the value
 * written back goes through f16 -> f32 -> f16; then every entry becomes
 * f32_to_f16(expf((x - max) / temperature) / sum), the sum running in fp32
 * over the array in its permuted order; a running fp32 sum over the first
 * topk entries finds where it reaches topp; random_val is scaled by the sum
 * of the kept prefix and the first entry whose running sum exceeds it wins.
 * Greedy form (otherwise): the first index holding the maximum.
 * dt = BF16 is this project's extension (the reference accepts F16 only):
 * exact widening, the same arithmetic, round-to-nearest-even where the
 * reference truncates to fp16.  PARITY UNPINNED by the reference. */
ORACLE_API int oracle_random_sample(uint32_t dt, uint64_t *result, const uint16_t *probs, int voc, float random_val, float topp,
                                    int topk, float temperature, uint16_t *logits, uint64_t *order) {
    if (dt != DT_F16 && dt != DT_BF16) {
        return -ST_BAD_TENSOR_DTYPE;
    }
    memcpy(logits, probs, (size_t) voc * sizeof(uint16_t));
    if (!(topp > 0 && topk > 1)) {
        float m = load16(dt, logits + 0);
        int index = 0;
        for (int j = 1; j < voc; ++j) {
            if (m < load16(dt, logits + j)) {
                m = load16(dt, logits + j);
                index = j;
            }
        }
        result[0] = (uint64_t) index;
        return 1;
    }
    if (topk > voc) {
        topk = voc;
    }
    for (int i = 0; i < voc; ++i) {
        order[i] = (uint64_t) i;
    }
    for (int i = 0; i < topk; ++i) {
        for (int j = i + 1; j < voc; ++j) {
            if (load16(dt, logits + i) < load16(dt, logits + j)) {
                const float held = load16(dt, logits + i);
                logits[i] = logits[j];
                store16(dt, logits + j, held);
                const int t = (int) order[i];
                order[i] = order[j];
                order[j] = (uint64_t) t;
            }
        }
    }
    const float top = load16(dt, logits + 0);
    float total = 0.0f;
    for (int i = 0; i < voc; ++i) {
        total += expf((load16(dt, logits + i) - top) / temperature);
    }
    for (int i = 0; i < voc; ++i) {
        store16(dt, logits + i, expf((load16(dt, logits + i) - top) / temperature) / total);
    }
    float run = 0.0f;
    int end;
    for (end = 0; end < topk; ++end) {
        run += load16(dt, logits + end);
        if (run >= topp) {
            break;
        }
    }
    if (end < topk - 1) {
        end += 1;
    } else {
        end = topk;
    }
    float kept = 0.0f;
    for (int i = 0; i < end; ++i) {
        kept += load16(dt, logits + i);
    }
    random_val *= kept;
    kept = 0.0f;
    for (int i = 0; i < end; ++i) {
        kept += load16(dt, logits + i);
        if (random_val < kept) {
            result[0] = order[i];
            return 1;
        }
    }
    return 0;
}
