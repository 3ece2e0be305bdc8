// gfx950 Matmul for the shape decoding gives the scores of an attention:
// few queries against very many keys,
//     c[i, j] = alpha * sum_k a[i, k] * b[k, j] + beta * c[i, j]
// in the descriptor's column-major terms with n <= 16 columns (the queries of
// one K/V head), m in the tens of thousands (the keys), k = head_dim, every
// row of a (a key) and every column of b (a query) contiguous along k.  The
// product is bound by reading a once, and this kernel does just that.
// Measured on MI355X, bf16, 8 K/V heads of [8 x head_dim] x [head_dim x 32768],
// us, this kernel / the library GEMM: head_dim 32: 5.5 / 17.6, 64: 9.5 / 17.7,
// 128: 15.8 / 25.6, 256: 29.7 / 40.6, 512: 55.6 / 73.8 (4.3-4.8 TB/s from 128
// on); 128 at 4096 keys 5.9 / 18, at 131072 keys 57 / 59.
//
// A wavefront takes 16 x TILES rows of a per turn.  Lane l holds 16 bytes of row
// l % 16 of each tile per step of 32 along k (8 elements from k = 32 s +
// 8 (l / 16) on), and the same 16 bytes of column l % 16 of b - loaded once,
// zeros for the columns b does not have.  Two v_mfma_f32_16x16x16 per step
// multiply them: the matrix unit's k index within an instruction is a label
// that a and b only have to agree on, so the first takes each lane's elements
// 0-3 and the second its elements 4-7.  The accumulator leaves lane l with rows
// 4 (l / 16) .. + 3 of the tile for column l % 16: four consecutive elements of
// c's column, one 8-byte store.  fp32 accumulation, alpha and beta applied in
// fp32, one rounding to nearest even into the element type - as the library
// GEMM does it.
#include "../../../devices/amd/kernel_amd.h"
#include "matmul_amd.h"

namespace {

using namespace amd;

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 h16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template<bool BF>
__device__ __forceinline__ f32x4 mma(uint32_t a0, uint32_t a1, uint32_t b0, uint32_t b1, f32x4 acc) {
    const u32x2 a{a0, a1}, b{b0, b1};
    if constexpr (BF) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), acc, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(h16x4, a), __builtin_bit_cast(h16x4, b), acc, 0, 0, 0);
    }
}

template<bool BF>
__device__ __forceinline__ float widen(uint16_t h) {
    if constexpr (BF) return BF16Rne::one(h);
    else return static_cast<float>(__builtin_bit_cast(_Float16, h));
}
template<bool BF>
__device__ __forceinline__ uint16_t narrow(float v) {// round to nearest even
    if constexpr (BF) return BF16Rne::narrow1(v);
    else return __builtin_bit_cast(uint16_t, static_cast<_Float16>(v));
}

constexpr int kSkinnyLanes = 256;

// GROUPS turns of KS steps of 32 along k.  TILES x KS 16-byte loads per lane are in flight together.
template<bool BF, int KS, int TILES, int GROUPS>
__global__ __launch_bounds__(kSkinnyLanes) void matmul_skinny(uint16_t *c, const uint16_t *a, const uint16_t *b, uint32_t m, uint32_t n,
                                                              int64_t lda, int64_t ldb, int64_t ldc, int64_t batch_a, int64_t batch_b,
                                                              int64_t batch_c, float alpha, float beta, uint32_t c_in_eights) {
    AMD_ARGS_NOW(c, a, b, m, n, lda, ldb, ldc, batch_a, batch_b, batch_c, alpha, beta, c_in_eights);
    const uint32_t lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const uint32_t of16 = lane & 15u, quad = lane >> 4;
    const uint32_t row0 = (blockIdx.x * (kSkinnyLanes / kWave) + wave) * (16u * TILES);
    if (row0 >= m) return;// uniform over the wavefront; there is no barrier below
    a += static_cast<int64_t>(blockIdx.y) * batch_a;
    b += static_cast<int64_t>(blockIdx.y) * batch_b;
    c += static_cast<int64_t>(blockIdx.y) * batch_c;

    f32x4 acc[TILES];
#pragma unroll
    for (int t = 0; t < TILES; ++t) acc[t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll 1
    for (int g = 0; g < GROUPS; ++g) {
        u32x4 x[TILES][KS];
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
            const uint32_t row = row0 + t * 16 + of16;
            // rows past the end repeat the last one; nothing of them is stored
            const uint16_t *at = a + static_cast<int64_t>(row < m ? row : m - 1) * lda + g * (KS * 32) + quad * 8;
#pragma unroll
            for (int s = 0; s < KS; ++s) x[t][s] = ld16_stream(at + s * 32);
        }
        u32x4 q[KS];
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            q[s] = u32x4{0, 0, 0, 0};
            if (of16 < n) q[s] = *reinterpret_cast<const u32x4 *>(b + static_cast<int64_t>(of16) * ldb + g * (KS * 32) + s * 32 + quad * 8);
        }
#pragma unroll
        for (int t = 0; t < TILES; ++t) {
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                acc[t] = mma<BF>(x[t][s].x, x[t][s].y, q[s].x, q[s].y, acc[t]);
                acc[t] = mma<BF>(x[t][s].z, x[t][s].w, q[s].z, q[s].w, acc[t]);
            }
        }
    }
#pragma unroll
    for (int t = 0; t < TILES; ++t) {
        const uint32_t first = row0 + t * 16 + quad * 4;// this lane's four rows of c, column of16
        if (of16 >= n || first >= m) continue;
        uint16_t *out = c + static_cast<int64_t>(of16) * ldc + first;
        const float r[4] = {acc[t].x, acc[t].y, acc[t].z, acc[t].w};
        uint16_t h[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float v = alpha * r[e];
            if (beta != 0.0f && first + e < m) v += beta * widen<BF>(out[e]);// (beta = 0: c is not read, as in a BLAS library)
            h[e] = narrow<BF>(v);
        }
        if (c_in_eights && first + 4 <= m) {
            *reinterpret_cast<u32x2 *>(out) = u32x2{h[0] | (static_cast<uint32_t>(h[1]) << 16), h[2] | (static_cast<uint32_t>(h[3]) << 16)};
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (first + e < m) out[e] = h[e];
            }
        }
    }
}

template<bool BF, int KS, int GROUPS>
void launch(const MatmulAmdDescriptor &d, void *c, const void *a, const void *b, bool c_in_eights, hipStream_t stream) {
    constexpr int TILES = 4;
    const uint32_t rows_per_group = (kSkinnyLanes / kWave) * 16 * TILES;
    const dim3 grid(static_cast<unsigned>((d.m + rows_per_group - 1) / rows_per_group), static_cast<unsigned>(d.batch));
    matmul_skinny<BF, KS, TILES, GROUPS><<<grid, kSkinnyLanes, 0, stream>>>(
        static_cast<uint16_t *>(c), static_cast<const uint16_t *>(a), static_cast<const uint16_t *>(b), static_cast<uint32_t>(d.m),
        static_cast<uint32_t>(d.n), d.a.row_stride, d.b.col_stride, d.c.col_stride, d.a.stride, d.b.stride, d.c.stride, d.alpha, d.beta,
        c_in_eights ? 1u : 0u);
}

}// namespace

// a, b, c: the operands of the descriptor's column-major problem (already exchanged where the descriptor says so).
// False: the call is not of this shape; nothing was launched.
bool amd_matmul_skinny(const MatmulAmdDescriptor &d, void *c, const void *a, const void *b, hipStream_t stream) {
    const bool sixteen_bit = d.elem == amd::Elem::F16 || d.elem == amd::Elem::BF16;
    if (!sixteen_bit || d.n < 1 || d.n > 16 || d.m < 1024 || d.k < 32 || d.k > 512 || d.k % 32 != 0 || d.batch > 65535) return false;
    // rows of a and columns of b contiguous along k, c's columns contiguous; 16-byte loads
    if (d.a.col_stride != 1 || d.b.row_stride != 1 || d.c.row_stride != 1) return false;
    if (d.a.row_stride % 8 != 0 || d.b.col_stride % 8 != 0 || d.a.stride % 8 != 0 || d.b.stride % 8 != 0) return false;
    if (d.a.row_stride < d.k || d.b.col_stride < d.k || d.c.col_stride < d.m) return false;// (also rules out negative strides)
    if (!amd::aligned16(a) || !amd::aligned16(b)) return false;
    if (d.m > 0x7FFFFFF0ll) return false;
    const bool c_in_eights = (reinterpret_cast<uintptr_t>(c) & 7u) == 0 && d.c.col_stride % 4 == 0 && d.c.stride % 4 == 0;
    const bool bf = d.elem == amd::Elem::BF16;
#define SKINNY(STEPS, KS, GROUPS)                                          \
    case STEPS:                                                            \
        if (bf) launch<true, KS, GROUPS>(d, c, a, b, c_in_eights, stream); \
        else launch<false, KS, GROUPS>(d, c, a, b, c_in_eights, stream);   \
        break
    // head widths of 256 and more in turns of 128: with all of k in registers at once the compiler needs every one
    // of them (8 x [8 x 256] x [256 x 32768] bf16: 49.5 us that way, 29.7 in two turns; 512: 64.9 and 55.6)
    switch (d.k / 32) {
        SKINNY(1, 1, 1);
        SKINNY(2, 2, 1);
        SKINNY(3, 3, 1);
        SKINNY(4, 4, 1);
        SKINNY(5, 5, 1);
        SKINNY(6, 6, 1);
        SKINNY(7, 7, 1);
        SKINNY(8, 4, 2);
        SKINNY(12, 4, 3);
        SKINNY(16, 4, 4);
        default: return false;
    }
#undef SKINNY
    return true;
}
