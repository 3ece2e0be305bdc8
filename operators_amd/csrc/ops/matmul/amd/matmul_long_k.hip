// gfx950 Matmul for the other product of an attention while decoding: the
// weights of few queries times the values of very many keys,
//     c[i, j] = alpha * sum_k a[i, k] * b[k, j] + beta * c[i, j]
// in the descriptor's column-major terms with m = head_dim rows (8 to 256, a
// power of two), n <= 8 columns (the queries of one K/V head) and k in the
// thousands to hundreds of thousands (the keys); a's columns (a key's values)
// and b's columns (a query's weights over the keys) are contiguous.  The
// library GEMM runs this shape at 1-2 TB/s ([128 x 131072] x [131072 x 8] per
// K/V head, 8 heads, bf16: 152 us for 268 MB; 59 us at 32768 keys, 18 us at
// 4096); it is bound by reading a once.
//
// The same two launches serve a few tokens through a weight matrix (m = the
// layer's output width in the thousands: matmul_long_k_wide below).
//
// Two launches.  The first splits k into chunks, a workgroup of 256 lanes
// each: m / 8 lanes cover a column of a (16 bytes, 8 rows, per lane), so a
// wavefront takes 512 / m pairs of neighbouring columns per step; a lane
// interleaves its two columns into (k, k + 1) pairs per row and multiplies
// them with v_dot2 by the matching pairs of b's n columns, which the workgroup
// staged in LDS beforehand (32 bytes per pair of k: eight columns of b, zeros
// for those it does not have); 64 fp32 accumulators per lane.  At the end the
// lanes that share rows add up through shuffles and LDS, and the workgroup
// leaves its m x 8 partial sums in the workspace.  The second launch adds a
// column's partial sums in ascending order of the chunks, applies alpha and
// beta in fp32 and rounds once, to nearest even, into the element type.
#include "../../../devices/amd/kernel_amd.h"
#include "matmul_amd.h"
#include <algorithm>

namespace {

using namespace amd;

typedef _Float16 h16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 b16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32_any __attribute__((aligned(2)));

template<bool BF>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
    if constexpr (BF) return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b16x2, a), __builtin_bit_cast(b16x2, b), acc, false);
    else return __builtin_amdgcn_fdot2(__builtin_bit_cast(h16x2, a), __builtin_bit_cast(h16x2, b), acc, false);
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

constexpr int kLanes = 256, kColumnsOfB = 8;

// chunk: columns of a (values of k) per workgroup, a multiple of 2 * steps' worth; lanes_per_column = m / 8, a power of two.
template<bool BF>
__global__ __launch_bounds__(kLanes) void matmul_long_k_partial(float *partial, const uint16_t *a, const uint16_t *b, uint32_t m, uint32_t n,
                                                                uint32_t k, uint32_t chunk, uint32_t lpc_shift, int64_t lda, int64_t ldb,
                                                                int64_t batch_a, int64_t batch_b) {
    AMD_ARGS_NOW(partial, a, b, m, n, k, chunk, lpc_shift, lda, ldb, batch_a, batch_b);
    extern __shared__ __attribute__((aligned(16))) uint32_t staged[];// [pair of k][column of b]: b[2p, j] | b[2p + 1, j] << 16
    const uint32_t tid = threadIdx.x;
    const uint32_t k0 = blockIdx.x * chunk;
    const uint32_t here = k - k0 < chunk ? k - k0 : chunk;// columns of a in this chunk (the host launches no empty chunk)
    a += static_cast<int64_t>(blockIdx.y) * batch_a;
    b += static_cast<int64_t>(blockIdx.y) * batch_b;

    const uint32_t pairs = (here + 1) / 2;
    const uint32_t lanes_per_column = 1u << lpc_shift;
    const uint32_t sub = tid & (lanes_per_column - 1);// which 8 rows of a
    const uint32_t slot = tid >> lpc_shift;           // which pair of columns within a step
    const uint32_t pairs_per_step = kLanes >> lpc_shift;
    constexpr int AHEAD = 2;// steps per set of registers; two sets take turns, so loads are in flight while the arrived ones are worked on
    const uint16_t *mine = a + static_cast<int64_t>(k0) * lda + sub * 8;
    const auto fetch = [&](uint32_t p0, u32x4(&lo)[AHEAD], u32x4(&hi)[AHEAD]) {
#pragma unroll
        for (int s = 0; s < AHEAD; ++s) {
            const uint32_t p = p0 + s * pairs_per_step + slot;
            const uint32_t c0 = 2 * p, c1 = 2 * p + 1;
            // a column past the end is the chunk's last one again, and is not used
            lo[s] = ld16_stream(mine + static_cast<int64_t>(c0 < here ? c0 : here - 1) * lda);
            hi[s] = ld16_stream(mine + static_cast<int64_t>(c1 < here ? c1 : here - 1) * lda);
        }
    };
    // the first loads of a go out before b's share of the chunk is staged
    u32x4 lo0[AHEAD], hi0[AHEAD], lo1[AHEAD], hi1[AHEAD];
    fetch(0, lo0, hi0);

    // b's share of the chunk into LDS, pairs along k
    for (uint32_t w = tid; w < pairs * kColumnsOfB; w += kLanes) {
        const uint32_t j = w / pairs, p = w - j * pairs;// a column of b at a time: neighbouring lanes read neighbouring words
        uint32_t word = 0;
        if (j < n) {
            const uint16_t *at = b + static_cast<int64_t>(j) * ldb + k0 + 2 * p;
            word = 2 * p + 1 < here ? *reinterpret_cast<const u32_any *>(at) : static_cast<uint32_t>(*at);
        }
        staged[p * kColumnsOfB + j] = word;
    }
    __syncthreads();

    float acc[kColumnsOfB][8];
#pragma unroll
    for (int j = 0; j < kColumnsOfB; ++j) {
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[j][e] = 0.0f;
    }
    const auto work = [&](uint32_t p0, const u32x4(&lo)[AHEAD], const u32x4(&hi)[AHEAD]) {
#pragma unroll
        for (int s = 0; s < AHEAD; ++s) {
            const uint32_t p = p0 + s * pairs_per_step + slot;
            if (p >= pairs) continue;// (nothing below crosses lanes)
            const bool has1 = 2 * p + 1 < here;// (column 2 p is there: p < pairs)
            const uint32_t x[4] = {lo[s].x, lo[s].y, lo[s].z, lo[s].w};
            const uint32_t y[4] = {has1 ? hi[s].x : 0u, has1 ? hi[s].y : 0u, has1 ? hi[s].z : 0u, has1 ? hi[s].w : 0u};
            uint32_t v[8];// row e of both columns: a[e, k] | a[e, k + 1] << 16
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[2 * i] = __builtin_amdgcn_perm(y[i], x[i], 0x05040100u);
                v[2 * i + 1] = __builtin_amdgcn_perm(y[i], x[i], 0x07060302u);
            }
            const u32x4 w0 = *reinterpret_cast<const u32x4 *>(staged + p * kColumnsOfB);
            const u32x4 w1 = *reinterpret_cast<const u32x4 *>(staged + p * kColumnsOfB + 4);
            const uint32_t w[kColumnsOfB] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
            for (int j = 0; j < kColumnsOfB; ++j) {
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[j][e] = dot2<BF>(v[e], w[j], acc[j][e]);
            }
        }
    };
    const uint32_t turn = pairs_per_step * AHEAD;
    for (uint32_t p0 = 0; p0 < pairs; p0 += 2 * turn) {
        fetch(p0 + turn, lo1, hi1);
        work(p0, lo0, hi0);
        fetch(p0 + 2 * turn, lo0, hi0);
        work(p0 + turn, lo1, hi1);
    }

    // the lanes of a wavefront that share rows (lanes sub, sub + lanes_per_column, ...), then the wavefronts through LDS
#pragma unroll 1
    for (uint32_t off = lanes_per_column; off < kWave; off <<= 1) {
#pragma unroll
        for (int j = 0; j < kColumnsOfB; ++j) {
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[j][e] += __shfl_xor(acc[j][e], static_cast<int>(off));
        }
    }
    __syncthreads();// everybody has read its last pairs of b: the staging area is free
    float *sums = reinterpret_cast<float *>(staged);// [wavefront or part of one][row group][column of b][row]
    const uint32_t lane = tid & (kWave - 1), wave = tid / kWave;
    // with more than 64 lanes per column (m = 1024 would be) this would not hold; m <= 256 means at most 32
    const uint32_t groups = lanes_per_column;// row groups of 8
    if (lane < groups) {
#pragma unroll
        for (int j = 0; j < kColumnsOfB; ++j) {
#pragma unroll
            for (int e = 0; e < 8; ++e) sums[((wave * groups + lane) * kColumnsOfB + j) * 8 + e] = acc[j][e];
        }
    }
    __syncthreads();
    float *out = partial + (static_cast<size_t>(blockIdx.y) * gridDim.x + blockIdx.x) * (static_cast<size_t>(m) * kColumnsOfB);
    for (uint32_t o = tid; o < m * kColumnsOfB; o += kLanes) {
        const uint32_t j = o / m, row = o - j * m;// partial[j][row]: a column of c contiguous
        const uint32_t g = row >> 3, e = row & 7u;
        float total = 0.0f;
#pragma unroll
        for (int wv = 0; wv < kLanes / kWave; ++wv) total += sums[((wv * groups + g) * kColumnsOfB + j) * 8 + e];
        out[o] = total;
    }
}

// The same product with many rows: a few tokens through a weight matrix while decoding (c^T = W^T x^T: m is the
// layer's output width, k its input width, the n columns are the tokens).  A workgroup is one wavefront, a lane
// takes 8 rows of a tile of 512 and every column of its chunk of k, so no two lanes share a row and nothing is
// added across lanes; the tokens' pairs along k come from LDS, the same 32 bytes for every lane.
constexpr int kWideRows = 512, kWideAhead = 4;

template<bool BF>
__global__ __launch_bounds__(kWave) void matmul_long_k_wide(float *partial, const uint16_t *a, const uint16_t *b, uint32_t m, uint32_t n,
                                                             uint32_t k, uint32_t chunk, uint32_t tiles, int64_t lda, int64_t ldb,
                                                             int64_t batch_a, int64_t batch_b) {
    AMD_ARGS_NOW(partial, a, b, m, n, k, chunk, tiles, lda, ldb, batch_a, batch_b);
    extern __shared__ __attribute__((aligned(16))) uint32_t staged[];// [pair of k][column of b]
    const uint32_t lane = threadIdx.x;
    const uint32_t ch = blockIdx.x / tiles, tile = blockIdx.x - ch * tiles;// neighbouring workgroups read neighbouring KiBs of the same columns
    const uint32_t chunks = gridDim.x / tiles;
    const uint32_t k0 = ch * chunk;
    const uint32_t here = k - k0 < chunk ? k - k0 : chunk;
    a += static_cast<int64_t>(blockIdx.y) * batch_a;
    b += static_cast<int64_t>(blockIdx.y) * batch_b;
    const uint32_t pairs = (here + 1) / 2;
    const uint32_t row0 = tile * kWideRows + lane * 8;
    const bool rows_here = row0 < m;// m is a multiple of 8: a lane's rows are all there or none is
    const uint16_t *mine = a + static_cast<int64_t>(k0) * lda + (rows_here ? row0 : 0);
    // Two sets of registers take turns: the loads of the next kWideAhead pairs of columns go out before the work on
    // the ones that have arrived, so a wavefront always has loads in flight.
    const auto fetch = [&](uint32_t p0, u32x4(&lo)[kWideAhead], u32x4(&hi)[kWideAhead]) {
#pragma unroll
        for (int s = 0; s < kWideAhead; ++s) {
            const uint32_t c0 = 2 * (p0 + s), c1 = c0 + 1;// a column past the end is the chunk's last one again, and is not used
            lo[s] = ld16_stream(mine + static_cast<int64_t>(c0 < here ? c0 : here - 1) * lda);
            hi[s] = ld16_stream(mine + static_cast<int64_t>(c1 < here ? c1 : here - 1) * lda);
        }
    };
    // the first loads of a go out before b's share of the chunk is staged
    u32x4 lo0[kWideAhead], hi0[kWideAhead], lo1[kWideAhead], hi1[kWideAhead];
    fetch(0, lo0, hi0);
    for (uint32_t w = lane; w < pairs * kColumnsOfB; w += kWave) {
        const uint32_t j = w / pairs, p = w - j * pairs;
        uint32_t word = 0;
        if (j < n) {
            const uint16_t *at = b + static_cast<int64_t>(j) * ldb + k0 + 2 * p;
            word = 2 * p + 1 < here ? *reinterpret_cast<const u32_any *>(at) : static_cast<uint32_t>(*at);
        }
        staged[p * kColumnsOfB + j] = word;
    }
    __syncthreads();

    float acc[kColumnsOfB][8];
#pragma unroll
    for (int j = 0; j < kColumnsOfB; ++j) {
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[j][e] = 0.0f;
    }
    const auto work = [&](uint32_t p0, const u32x4(&lo)[kWideAhead], const u32x4(&hi)[kWideAhead]) {
#pragma unroll
        for (int s = 0; s < kWideAhead; ++s) {
            const uint32_t p = p0 + s;
            if (p >= pairs) break;// uniform over the wavefront
            const bool has1 = 2 * p + 1 < here;
            const uint32_t x[4] = {lo[s].x, lo[s].y, lo[s].z, lo[s].w};
            const uint32_t y[4] = {has1 ? hi[s].x : 0u, has1 ? hi[s].y : 0u, has1 ? hi[s].z : 0u, has1 ? hi[s].w : 0u};
            uint32_t v[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[2 * i] = __builtin_amdgcn_perm(y[i], x[i], 0x05040100u);
                v[2 * i + 1] = __builtin_amdgcn_perm(y[i], x[i], 0x07060302u);
            }
            const u32x4 w0 = *reinterpret_cast<const u32x4 *>(staged + p * kColumnsOfB);
            const u32x4 w1 = *reinterpret_cast<const u32x4 *>(staged + p * kColumnsOfB + 4);
            const uint32_t w[kColumnsOfB] = {w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w};
#pragma unroll
            for (int j = 0; j < kColumnsOfB; ++j) {
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[j][e] = dot2<BF>(v[e], w[j], acc[j][e]);
            }
        }
    };
    for (uint32_t p0 = 0; p0 < pairs; p0 += 2 * kWideAhead) {
        fetch(p0 + kWideAhead, lo1, hi1);
        work(p0, lo0, hi0);
        fetch(p0 + 2 * kWideAhead, lo0, hi0);
        work(p0 + kWideAhead, lo1, hi1);
    }
    if (!rows_here) return;
    float *out = partial + (static_cast<size_t>(blockIdx.y) * chunks + ch) * (static_cast<size_t>(m) * kColumnsOfB) + row0;
#pragma unroll
    for (int j = 0; j < kColumnsOfB; ++j) {
        if (static_cast<uint32_t>(j) >= n) break;// the sums of columns b does not have are never read
        f32x4 *at = reinterpret_cast<f32x4 *>(out + static_cast<size_t>(j) * m);
        at[0] = f32x4{acc[j][0], acc[j][1], acc[j][2], acc[j][3]};
        at[1] = f32x4{acc[j][4], acc[j][5], acc[j][6], acc[j][7]};
    }
}

template<bool BF>
__global__ __launch_bounds__(256) void matmul_long_k_combine(uint16_t *c, const float *partial, uint32_t m, uint32_t n, uint32_t chunks,
                                                             int64_t ldc, int64_t batch_c, float alpha, float beta) {
    const uint32_t o = blockIdx.x * 256 + threadIdx.x;
    if (o >= m * n) return;
    const uint32_t j = o / m, row = o - j * m;
    const float *at = partial + static_cast<size_t>(blockIdx.y) * chunks * (static_cast<size_t>(m) * kColumnsOfB) + static_cast<size_t>(j) * m + row;
    // in ascending order of the chunks, eight loads in flight at a time (one after the other they took 32 us for 128 chunks)
    const size_t hop = static_cast<size_t>(m) * kColumnsOfB;
    float total = 0.0f;
    uint32_t ch = 0;
    for (; ch + 8 <= chunks; ch += 8) {
        float part[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) part[i] = at[(ch + i) * hop];
#pragma unroll
        for (int i = 0; i < 8; ++i) total += part[i];
    }
    for (; ch < chunks; ++ch) total += at[ch * hop];
    uint16_t *out = c + static_cast<int64_t>(blockIdx.y) * batch_c + static_cast<int64_t>(j) * ldc + row;
    float v = alpha * total;
    if (beta != 0.0f) v += beta * widen<BF>(*out);// (beta = 0: c is not read, as in a BLAS library)
    *out = narrow<BF>(v);
}

struct Plan {
    int kind;// 0: not a shape for these kernels, 1: up to 256 rows (a workgroup covers them all), 2: many rows (tiles of 512)
    uint32_t chunk, chunks, tiles;
};

// Columns of a per workgroup, few rows: the largest of 1024, 512, 256 that still gives the chip 512 workgroups, else 128.  A
// workgroup works through its chunk in turns of 128 columns, a memory latency each, and ends with a sum over its
// lanes that costs as much as a turn or two.  Measured, 8 batches of [128 x k] x [k x 8] bf16, both launches, us,
// chunks of 128 / 256 / 512 / 1024 / 2048: k = 4096: 11.1 / 11.6 / 14.7 / 22.4 / 36.1; 32768: 41.9 / 29.8 / 25.2 /
// 28.4 / 43.7; 131072: 141 / 93.0 / 73.6 / 62.6 / 64.9.
Plan plan_of(const MatmulAmdDescriptor &d) {
    const Plan none{0, 0, 0, 0};
    const bool sixteen_bit = d.elem == amd::Elem::F16 || d.elem == amd::Elem::BF16;
    if (!sixteen_bit || d.n < 1 || d.n > kColumnsOfB || d.k < 1024 || d.k > 0x7FFFFFF0ll || d.batch < 1 || d.batch > 65535) return none;
    // columns of a and of b contiguous, c's columns contiguous; 16-byte loads of a
    if (d.a.row_stride != 1 || d.b.row_stride != 1 || d.c.row_stride != 1) return none;
    if (d.a.col_stride % 8 != 0 || d.a.stride % 8 != 0 || d.a.col_stride < d.m || d.b.col_stride < d.k || d.c.col_stride < d.m) return none;
    if (d.m >= 8 && d.m <= 256 && (d.m & (d.m - 1)) == 0) {
        uint32_t chunk = 128;
        for (const uint32_t c : {1024u, 512u, 256u}) {
            if (static_cast<uint64_t>(d.batch) * ((d.k + c - 1) / c) >= 512) {
                chunk = c;
                break;
            }
        }
        return Plan{1, chunk, static_cast<uint32_t>((d.k + chunk - 1) / chunk), 1};
    }
    // Many rows: about 1024 wavefronts in all, chunks of 256 columns and more (a chunk leaves 32 bytes of partial
    // sums per row and column of b behind).  Measured against the BLAS library, bf16, us, 1 / 8 columns of b:
    // [8192 x 28672]: 81 / 91 against 127 / 132; [22016 x 4096]: 36 / 42 against 52 / 52; [10240 x 8192]: 36 / 42
    // against 49 / 50; [8192 x 8192]: 38 / 42 against 43 / 44; [57344 x 8192], 1 / 4 / 8 columns: 153 / 161 / 172
    // against 158 / 165 / 166 - the library reads that one at 5.7 TB/s, and keeps it from five columns of b on
    // (fewer, longer chunks there - 512 or 768 wavefronts - take 238 and 160 us).  (Room for 16 columns of b - 128
    // accumulators per lane - took 211 registers and 528 bytes of scratch and ran 9-10 times slower than the
    // library on every shape: 9 to 16 columns stay with the library.)
    if (d.m >= 1024 && d.m % 8 == 0 && d.m <= 0x7FFFFFF0ll && d.m * kColumnsOfB < (1ll << 31)) {
        const uint32_t tiles = static_cast<uint32_t>((d.m + kWideRows - 1) / kWideRows);
        if (tiles >= 64 && d.n > 4) return none;
        uint64_t chunks = 1024 / (static_cast<uint64_t>(tiles) * d.batch);
        if (chunks < 1) chunks = 1;
        uint64_t chunk = (d.k + chunks - 1) / chunks;
        if (chunk < 256) chunk = 256;
        chunk = (chunk + 15) / 16 * 16;
        if (chunk > 2048) chunk = 2048;// 32 KiB of LDS for b's share
        chunks = (d.k + chunk - 1) / chunk;
        if (static_cast<uint64_t>(tiles) * chunks > 0x7FFFFFFFull) return none;
        return Plan{2, static_cast<uint32_t>(chunk), static_cast<uint32_t>(chunks), tiles};
    }
    return none;
}

}// namespace

// Bytes of workspace with which amd_matmul_long_k serves the descriptor's shape; 0: not a shape for it.
uint64_t amd_matmul_long_k_workspace(const MatmulAmdDescriptor &d) {
    const Plan p = plan_of(d);
    if (p.kind == 0) return 0;
    return static_cast<uint64_t>(d.batch) * p.chunks * d.m * kColumnsOfB * sizeof(float);
}

namespace {

template<bool BF>
void launch_long_k(const MatmulAmdDescriptor &d, const Plan &p, float *partial, void *c, const void *a, const void *b, hipStream_t stream) {
    const auto *pa = static_cast<const uint16_t *>(a);
    const auto *pb = static_cast<const uint16_t *>(b);
    const uint32_t m = static_cast<uint32_t>(d.m), n = static_cast<uint32_t>(d.n), k = static_cast<uint32_t>(d.k);
    if (p.kind == 1) {
        uint32_t lpc_shift = 0;
        while ((8u << lpc_shift) < m) ++lpc_shift;
        const size_t lds = std::max<size_t>(static_cast<size_t>(p.chunk / 2) * kColumnsOfB * sizeof(uint32_t),
                                            static_cast<size_t>(kLanes / kWave) * (m / 8) * kColumnsOfB * 8 * sizeof(float));
        matmul_long_k_partial<BF><<<dim3(p.chunks, static_cast<unsigned>(d.batch)), kLanes, lds, stream>>>(
            partial, pa, pb, m, n, k, p.chunk, lpc_shift, d.a.col_stride, d.b.col_stride, d.a.stride, d.b.stride);
    } else {
        const size_t lds = static_cast<size_t>((p.chunk + 1) / 2) * kColumnsOfB * sizeof(uint32_t);
        matmul_long_k_wide<BF><<<dim3(p.tiles * p.chunks, static_cast<unsigned>(d.batch)), kWave, lds, stream>>>(
            partial, pa, pb, m, n, k, p.chunk, p.tiles, d.a.col_stride, d.b.col_stride, d.a.stride, d.b.stride);
    }
    const dim3 grid2(static_cast<unsigned>((d.m * d.n + 255) / 256), static_cast<unsigned>(d.batch));
    matmul_long_k_combine<BF><<<grid2, 256, 0, stream>>>(static_cast<uint16_t *>(c), partial, m, n, p.chunks, d.c.col_stride, d.c.stride,
                                                         d.alpha, d.beta);
}

}// namespace

// a, b, c: the operands of the descriptor's column-major problem.  False: not of this shape, or the workspace is
// missing or short; nothing was launched.
bool amd_matmul_long_k(const MatmulAmdDescriptor &d, void *workspace, uint64_t workspace_size, void *c, const void *a, const void *b,
                       hipStream_t stream) {
    const Plan p = plan_of(d);
    const uint64_t need = amd_matmul_long_k_workspace(d);
    if (p.kind == 0 || workspace == nullptr || workspace_size < need || !amd::aligned16(workspace) || !amd::aligned16(a)) return false;
    if ((reinterpret_cast<uintptr_t>(b) & 1u) != 0 || (reinterpret_cast<uintptr_t>(c) & 1u) != 0) return false;
    if (d.elem == amd::Elem::BF16) launch_long_k<true>(d, p, static_cast<float *>(workspace), c, a, b, stream);
    else launch_long_k<false>(d, p, static_cast<float *>(workspace), c, a, b, stream);
    return true;
}
