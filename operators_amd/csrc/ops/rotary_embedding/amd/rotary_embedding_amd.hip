// gfx950 kernels for RoPE and their launch.
//
// Arithmetic contract (reference
// src/ops/rotary_embedding/cpu/rotary_embedding_cpu.cc:16-44): for token i the
// table rows start at pos[i]*head_dim; for pair k of every head, with
// a = t[2k], b = t[2k+1] widened to fp32,
//     t[2k]   = narrow( a*cos[2k]   - b*sin[2k]   )
//     t[2k+1] = narrow( a*sin[2k+1] + b*cos[2k+1] )
// each product rounded to fp32 on its own (the CPU build has no fused
// multiply-add), four distinct table reads per pair.  Only IEEE multiply,
// add and the reference's truncating narrowing are involved, so fp16 results
// are bit-identical to the CPU's.  bf16 (extension) rounds to nearest even.
//
// t is read and written exactly once through arbitrary token/head strides;
// the table rows of a token are fetched once per lane, through the caches, and
// reused for every head that lane rotates.  (Staging the rows in LDS with one
// head per lane was measured on MI355X and is slower: 52.7 against 48.9 us at
// q = [8192, 64, 128] bf16.)  One pass, one tile per workgroup, in dispatch
// order: workgroups that loop over tiles with the next tile's loads in flight
// were measured at every shape of the benchmark and are never faster.
#include "../../../devices/amd/kernel_amd.h"
#include "rotary_embedding_amd.h"

// Products must not be fused into the add/subtract that follows them.
#pragma clang fp contract(off)

namespace {

using namespace amd;

constexpr int kBlock = 256;
constexpr int kHeadsPerLane = 4;// 2 and 4 measure within 2 % of each other on MI355X; 1 and 8 are slower

// The token of the wavefront's first lane, as a wavefront-uniform value: lanes
// are numbered in item order, so it is the smallest token the wavefront
// touches, and the base address of the wavefront's buffer stores.
template<typename Idx>
__device__ __forceinline__ Idx first_lane(Idx v) {
    if constexpr (sizeof(Idx) == 4) {
        return static_cast<Idx>(__builtin_amdgcn_readfirstlane(static_cast<int>(v)));
    } else {
        const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(static_cast<uint32_t>(v))));
        const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(static_cast<uint32_t>(v >> 32))));
        return static_cast<Idx>((static_cast<uint64_t>(hi) << 32) | lo);
    }
}

// One lane = one 8-element column group `cv` of up to HPT heads of one token.
// Work items are numbered (token, head group g, cv) with cv fastest, so the
// lanes of a wavefront cover consecutive 16-byte pieces of consecutive heads.
// Lane (g, cv) rotates heads g, g+G, g+2G, ... (G = number of head groups):
// at every step the wavefront's accesses are again to neighbouring heads.
//
// rope_vec is the general form of this map - any item count (Idx may be 64
// bits wide), head counts that HPT does not divide - and serves what
// rope_once below does not take.  BUFST: results are written through L2 by
// buffer stores relative to the wavefront's first token (see StreamOut).
template<typename T, typename Idx, int HPT, bool BUFST>
__global__ __launch_bounds__(kBlock) void rope_vec(uint16_t *t, const uint64_t *pos, const float *sin_t, const float *cos_t,
                                                   uint64_t total_items, Idx items_per_token, Idx vecs_per_head, Idx groups,
                                                   uint32_t heads, uint32_t head_dim, int64_t stride_token, int64_t stride_head) {
    const uint64_t item64 = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (item64 >= total_items) return;
    const Idx item = static_cast<Idx>(item64);
    const Idx token = item / items_per_token;
    const Idx rem = item - token * items_per_token;
    const Idx g = rem / vecs_per_head;
    const Idx cv = rem - g * vecs_per_head;

    uint16_t *base = t + static_cast<int64_t>(token) * stride_token + static_cast<int64_t>(cv) * 8;
    const Idx token0 = BUFST ? first_lane(token) : token;
    const StreamOut<true> out(t + static_cast<int64_t>(token0) * stride_token);
    const uint32_t off = static_cast<uint32_t>(token - token0) * static_cast<uint32_t>(stride_token) * 2 + static_cast<uint32_t>(cv) * 16;

    u32x4 tv[HPT];
#pragma unroll
    for (int i = 0; i < HPT; ++i) {
        const uint32_t h = static_cast<uint32_t>(g) + i * static_cast<uint32_t>(groups);
        if (h < heads) tv[i] = ld16_stream(base + static_cast<int64_t>(h) * stride_head);
    }

    const uint64_t row = pos[token] * head_dim + static_cast<uint64_t>(cv) * 8;
    const f32x4 s_lo = ld16f(sin_t + row), s_hi = ld16f(sin_t + row + 4);
    const f32x4 c_lo = ld16f(cos_t + row), c_hi = ld16f(cos_t + row + 4);
    const float sn[8] = {s_lo.x, s_lo.y, s_lo.z, s_lo.w, s_hi.x, s_hi.y, s_hi.z, s_hi.w};
    const float cs[8] = {c_lo.x, c_lo.y, c_lo.z, c_lo.w, c_hi.x, c_hi.y, c_hi.z, c_hi.w};

#pragma unroll
    for (int i = 0; i < HPT; ++i) {
        const uint32_t h = static_cast<uint32_t>(g) + i * static_cast<uint32_t>(groups);
        if (h < heads) {
            float f[8], r[8];
            widen8<T>(tv[i], f);
#pragma unroll
            for (int k = 0; k < 8; k += 2) {
                const float a = f[k], b = f[k + 1];
                const float ac = a * cs[k], bs = b * sn[k];
                const float as = a * sn[k + 1], bc = b * cs[k + 1];
                r[k] = ac - bs;
                r[k + 1] = as + bc;
            }
            if constexpr (BUFST) {
                out.st16(off + h * static_cast<uint32_t>(stride_head) * 2, narrow8<T>(r));
            } else {
                st16_stream(base + static_cast<int64_t>(h) * stride_head, narrow8<T>(r));
            }
        }
    }
}

// One pass, one tile of BS work items per workgroup, in the order the
// dispatcher hands workgroups out.  UNI: a token's work items are a multiple
// of BS, so a workgroup lies inside one token and its position is one load
// from a uniform address, asked for before the data and waited for alone
// (vector loads return in order).  Otherwise every lane loads its token's
// position itself, after the data loads: asked for first, the position delays
// the data behind it (k [8192, 8, 128] bf16 with 4 heads per lane: 10.6 us
// position first, 8.7 us position last).  Positions fetched per wavefront
// through the scalar unit, so that the table loads can follow the data loads
// at once, measured the same as that (k 8.8 us, [4096, 32, 128] fp16 13.2 us):
// in a tensor of this size the strided rows bound the time (a strided copy of
// k's rows takes 9.4 us, a dense one 8.2 us).
// The head count is a multiple of HPT (every lane's heads exist): nothing is
// predicated, so no load can sink into a branch behind the wait for another.
template<typename T, int BS, int HPT, bool BUFST, bool UNI>
__global__ __launch_bounds__(BS) void rope_once(uint16_t *__restrict__ t, const uint64_t *__restrict__ pos,
                                                const float *__restrict__ sin_t, const float *__restrict__ cos_t,
                                                uint32_t total_items, uint32_t items_per_token, uint32_t vecs_per_head, uint32_t groups,
                                                uint32_t head_dim, int64_t stride_token, int64_t stride_head, FastDiv by_token,
                                                FastDiv by_head) {
    AMD_ARGS_NOW(t, pos, sin_t, cos_t, total_items, items_per_token, vecs_per_head, groups, head_dim, stride_token, stride_head,
                 arg_pair(by_token), arg_pair(by_head));
    // fewer than 2^31 work items: the two divisions are multiplications (see FastDiv)
    uint32_t token, rem;
    if constexpr (UNI) {
        const uint32_t item0 = blockIdx.x * BS;
        token = fast_quotient(item0, by_token);
        rem = item0 - token * items_per_token + threadIdx.x;
    } else {
        const uint32_t item = blockIdx.x * BS + threadIdx.x;
        if (item >= total_items) return;
        token = fast_quotient(item, by_token);
        rem = item - token * items_per_token;
    }
    const uint32_t g = fast_quotient(rem, by_head);
    const uint32_t cv = rem - g * vecs_per_head;
    uint64_t p;
    if constexpr (UNI) p = pos[token];

    uint16_t *base = t + static_cast<int64_t>(token) * stride_token + static_cast<int64_t>(cv) * 8;
    u32x4 tv[HPT];
#pragma unroll
    for (int i = 0; i < HPT; ++i) {
        const uint32_t h = g + i * groups;
        tv[i] = ld16_stream(base + static_cast<int64_t>(h) * stride_head);
    }
    if constexpr (!UNI) p = pos[token];
    __builtin_amdgcn_sched_barrier(0);// the data loads leave before anything waits for the position

    const uint64_t row = p * head_dim + static_cast<uint64_t>(cv) * 8;
    const f32x4 s_lo = ld16f(sin_t + row), s_hi = ld16f(sin_t + row + 4);
    const f32x4 c_lo = ld16f(cos_t + row), c_hi = ld16f(cos_t + row + 4);
    const float sn[8] = {s_lo.x, s_lo.y, s_lo.z, s_lo.w, s_hi.x, s_hi.y, s_hi.z, s_hi.w};
    const float cs[8] = {c_lo.x, c_lo.y, c_lo.z, c_lo.w, c_hi.x, c_hi.y, c_hi.z, c_hi.w};

    // buffer stores address from the wavefront's first token
    const uint32_t token0 = UNI || !BUFST ? token : first_lane(token);
    const StreamOut<true> out(t + static_cast<int64_t>(token0) * stride_token);
    const uint32_t off = (token - token0) * static_cast<uint32_t>(stride_token) * 2 + cv * 16;
#pragma unroll
    for (int i = 0; i < HPT; ++i) {
        const uint32_t h = g + i * groups;
        float f[8], r[8];
        widen8<T>(tv[i], f);
#pragma unroll
        for (int k = 0; k < 8; k += 2) {
            const float a = f[k], b = f[k + 1];
            const float ac = a * cs[k], bs = b * sn[k];
            const float as = a * sn[k + 1], bc = b * cs[k + 1];
            r[k] = ac - bs;
            r[k + 1] = as + bc;
        }
        if constexpr (BUFST) {
            out.st16(off + h * static_cast<uint32_t>(stride_head) * 2, narrow8<T>(r));
        } else {
            st16_stream(base + static_cast<int64_t>(h) * stride_head, narrow8<T>(r));
        }
    }
}

// Any even head_dim, any strides and alignment.  A lane takes 8 consecutive
// elements (4 pairs) of one head: a whole group moves as 16 bytes at whatever
// 2-byte boundary it lies on, with its 2 x 8 table values as 16-byte loads at
// their 4-byte boundary (gfx950 serves such accesses, at a fraction of the
// aligned rate); a head's last, partial group pair by pair.  [8192, 64, 128]
// bf16 one element into its buffer: 119 us with one lane per pair.
template<typename T>
__global__ __launch_bounds__(kBlock) void rope_pairs(uint16_t *t, const uint64_t *pos, const float *sin_t, const float *cos_t,
                                                     uint64_t total_groups, uint64_t heads, uint64_t head_dim,
                                                     int64_t stride_token, int64_t stride_head) {
    const uint64_t per_head = (head_dim + 7) / 8;
    const uint64_t step = static_cast<uint64_t>(gridDim.x) * kBlock;
    for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x; i < total_groups; i += step) {
        const uint64_t th = i / per_head, col = (i - th * per_head) * 8;
        const uint64_t token = th / heads, h = th - token * heads;
        uint16_t *p = t + static_cast<int64_t>(token) * stride_token + static_cast<int64_t>(h) * stride_head + col;
        const uint64_t row = pos[token] * head_dim + col;
        if (col + 8 <= head_dim) {
            float f[8], r[8];
            widen8<T>(ld16_any(p), f);
            const f32x4 s_lo = *reinterpret_cast<const f32x4_any *>(sin_t + row), s_hi = *reinterpret_cast<const f32x4_any *>(sin_t + row + 4);
            const f32x4 c_lo = *reinterpret_cast<const f32x4_any *>(cos_t + row), c_hi = *reinterpret_cast<const f32x4_any *>(cos_t + row + 4);
            const float sn[8] = {s_lo.x, s_lo.y, s_lo.z, s_lo.w, s_hi.x, s_hi.y, s_hi.z, s_hi.w};
            const float cs[8] = {c_lo.x, c_lo.y, c_lo.z, c_lo.w, c_hi.x, c_hi.y, c_hi.z, c_hi.w};
#pragma unroll
            for (int k = 0; k < 8; k += 2) {
                const float a = f[k], b = f[k + 1];
                const float ac = a * cs[k], bs = b * sn[k];
                const float as = a * sn[k + 1], bc = b * cs[k + 1];
                r[k] = ac - bs;
                r[k + 1] = as + bc;
            }
            st16_any(p, narrow8<T>(r));
        } else {
            for (uint64_t k = 0; col + k < head_dim; k += 2) {
                const float a = T::one(p[k]), b = T::one(p[k + 1]);
                const float ac = a * cos_t[row + k], bs = b * sin_t[row + k];
                const float as = a * sin_t[row + k + 1], bc = b * cos_t[row + k + 1];
                p[k] = T::narrow1(ac - bs);
                p[k + 1] = T::narrow1(as + bc);
            }
        }
    }
}

template<typename T, typename Idx>
void launch_vec(const RoPEAmdDescriptor &d, uint16_t *t, const uint64_t *pos, const float *sn, const float *cs, hipStream_t stream) {
    const uint64_t vph = d.head_dim / 8;
    // Large outputs are written through L2 with buffer stores, which address
    // 32 bits from the first token of a wavefront (it spans at most 64 tokens).
    const bool bufst = d.tokens * d.heads * d.head_dim * sizeof(uint16_t) >= kWriteThroughBytes &&
                       d.stride_token >= 0 && d.stride_head >= 0 &&
                       static_cast<uint64_t>(d.stride_token) < (1ull << 23) &&
                       d.heads * static_cast<uint64_t>(d.stride_head) < (1ull << 30) && d.head_dim < (1ull << 24);

    // Heads per lane.  Every lane fetches the 64 bytes of table values of its
    // column group whatever the number of heads it rotates with them, so few
    // heads per lane multiply the table traffic through L2, and many heads per
    // lane leave few lanes.  Measured on MI355X (us; one pass, 256 lanes; "uni"
    // = a token's lanes fill whole workgroups):
    //   heads per lane                          2          4          8        16
    //   q [8192,64,128] bf16, 128 MiB        43.6 uni   43.3 uni   46.2      46.4
    //   k [8192,8,128] bf16, 16 MiB          10.9        8.7        8.7       -
    //   [4096,32,128] fp16, 32 MiB, random   14.0 uni   14.2       13.2      12.9
    //   positions
    // (q with workgroups looping over tokens with prefetch: 45.5; workgroups of
    // 64 or 128 lanes: the same or worse at every shape.)  So: tensors that
    // keep the memory system busy for tens of microseconds take the layout in
    // which a token fills a workgroup; smaller ones, whose time is mostly
    // launch and latency, put as many heads on a lane as divide the count.
    const bool large = d.tokens * d.heads * d.head_dim * sizeof(uint16_t) >= kWriteThroughBytes;
    int hpt = 1;
    if (large) {
        for (int cand : {8, 4, 2}) {// the most heads per lane that still leave a workgroup's worth of lanes per token
            if (d.heads % cand == 0 && (d.heads / cand) * vph >= kBlock) {
                hpt = cand;
                break;
            }
        }
    }
    if (hpt == 1) {
        for (int cand : {16, 8, 4, 2}) {
            if (d.heads % cand == 0 && (large ? cand <= 8 : true)) {
                hpt = cand;
                break;
            }
        }
    }
    const uint64_t groups = d.heads / hpt;
    const uint64_t ipt = groups * vph;
    const uint64_t total = d.tokens * ipt;
    if (sizeof(Idx) == 4 && total < (1ull << 31)) {
        const bool uni = ipt % kBlock == 0;
        const unsigned grid = static_cast<unsigned>(ceil_div(total, kBlock));
        const bool b1 = bufst && static_cast<uint64_t>(kWave) * static_cast<uint64_t>(d.stride_token) * 2 +
                                         d.heads * static_cast<uint64_t>(d.stride_head) * 2 < (1ull << 31);
#define ROPE_ONCE_GO(HPT, B, U)                                                                                              \
    rope_once<T, kBlock, HPT, B, U><<<grid, kBlock, 0, stream>>>(t, pos, sn, cs, static_cast<uint32_t>(total),                \
                                                                 static_cast<uint32_t>(ipt), static_cast<uint32_t>(vph),      \
                                                                 static_cast<uint32_t>(groups), static_cast<uint32_t>(d.head_dim), \
                                                                 d.stride_token, d.stride_head, fast_div(static_cast<uint32_t>(ipt)), \
                                                                 fast_div(static_cast<uint32_t>(vph)))
#define ROPE_ONCE_BU(HPT)                                \
    do {                                                 \
        if (b1 && uni) ROPE_ONCE_GO(HPT, true, true);    \
        else if (b1) ROPE_ONCE_GO(HPT, true, false);     \
        else if (uni) ROPE_ONCE_GO(HPT, false, true);    \
        else ROPE_ONCE_GO(HPT, false, false);            \
    } while (0)
        if (hpt == 16) ROPE_ONCE_BU(16);
        else if (hpt == 8) ROPE_ONCE_BU(8);
        else if (hpt == 4) ROPE_ONCE_BU(4);
        else if (hpt == 2) ROPE_ONCE_BU(2);
        else ROPE_ONCE_BU(1);
#undef ROPE_ONCE_BU
#undef ROPE_ONCE_GO
        return;
    }
    // more work items than 32 bits index: the general form, lanes find their token by division
    {
        const int h2 = d.heads >= kHeadsPerLane ? kHeadsPerLane : (d.heads >= 2 ? 2 : 1);
        const uint64_t g2 = ceil_div(d.heads, h2);
        const uint64_t ipt2 = g2 * vph, total2 = d.tokens * ipt2;
        const unsigned grid = static_cast<unsigned>(ceil_div(total2, kBlock));
#define ROPE_LAUNCH(HPT)                                                                                                          \
    rope_vec<T, Idx, HPT, false><<<grid, kBlock, 0, stream>>>(t, pos, sn, cs, total2, static_cast<Idx>(ipt2), static_cast<Idx>(vph), \
                                                              static_cast<Idx>(g2), static_cast<uint32_t>(d.heads),                \
                                                              static_cast<uint32_t>(d.head_dim), d.stride_token, d.stride_head)
        if (h2 == 4) ROPE_LAUNCH(4);
        else if (h2 == 2) ROPE_LAUNCH(2);
        else ROPE_LAUNCH(1);
#undef ROPE_LAUNCH
    }
}

template<typename T>
void launch_rope(const RoPEAmdDescriptor &d, void *t, const void *pos_ids, const void *sin_table, const void *cos_table, hipStream_t stream) {
    auto *pt = static_cast<uint16_t *>(t);
    auto *pos = static_cast<const uint64_t *>(pos_ids);
    auto *sn = static_cast<const float *>(sin_table);
    auto *cs = static_cast<const float *>(cos_table);

    const uint64_t elems = d.tokens * d.heads * d.head_dim;
    const bool vec_ok = d.head_dim % 8 == 0 && d.stride_token % 8 == 0 && d.stride_head % 8 == 0 &&
                        aligned16(t) && aligned16(sin_table) && aligned16(cos_table) &&
                        d.heads < (1ull << 31) && d.head_dim < (1ull << 31) && elems / 8 < (1ull << 38);
    if (!vec_ok) {
        const uint64_t groups = d.tokens * d.heads * ceil_div(d.head_dim, 8);
        const uint64_t want = ceil_div(groups, kBlock), cap = max_grid_1d(kBlock);
        rope_pairs<T><<<static_cast<unsigned>(want < cap ? want : cap), kBlock, 0, stream>>>(
            pt, pos, sn, cs, groups, d.heads, d.head_dim, d.stride_token, d.stride_head);
        return;
    }
    if (elems / 8 < (1ull << 31)) launch_vec<T, uint32_t>(d, pt, pos, sn, cs, stream);
    else launch_vec<T, uint64_t>(d, pt, pos, sn, cs, stream);
}

}// namespace

// Stage 4 of RoPE.  Null data pointers are a bad parameter, as in
// rotary_embedding_cpu.cc:119-120.  The workspace is unused (its size is 0).
// pos_ids are not checked against the table length, as in the reference: a
// position beyond the table is the caller's error.
infiniopStatus_t amdRoPE(RoPEAmdDescriptor_t desc, void *, uint64_t, void *t, void const *pos_ids,
                         void const *sin_table, void const *cos_table, void *stream) {
    if (t == nullptr || pos_ids == nullptr || sin_table == nullptr || cos_table == nullptr) {
        return STATUS_BAD_PARAM;
    }
    if (desc->tokens == 0 || desc->heads == 0 || desc->head_dim == 0) {
        return STATUS_SUCCESS;
    }
    AMD_CHECK_HIP(hipSetDevice(desc->device_id), STATUS_BAD_DEVICE);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (desc->elem) {
        case amd::Elem::F16:
            launch_rope<amd::F16Ref>(*desc, t, pos_ids, sin_table, cos_table, s);
            break;
        case amd::Elem::BF16:
            launch_rope<amd::BF16Rne>(*desc, t, pos_ids, sin_table, cos_table, s);
            break;
        default:
            return STATUS_BAD_TENSOR_DTYPE;
    }
    AMD_CHECK_HIP(hipGetLastError(), STATUS_EXECUTION_FAILED);
    return STATUS_SUCCESS;
}
