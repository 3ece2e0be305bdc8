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
// q = [8192, 64, 128] bf16.)
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
// BUFST: results are written through L2 by buffer stores relative to the
// wavefront's first token (see StreamOut); the host selects it for large
// outputs when strides are non-negative and the 64 tokens a wavefront can span
// fit a 32-bit byte offset.
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

// The same lane-to-data map as rope_vec, as a looping kernel: a workgroup
// walks tiles of kBlock work items and always has the next tile's loads (t
// and table rows) in flight while it rotates and stores the current one.  All
// loads are unconditional - items or heads past the end are redirected to the
// last valid one and simply not stored - so the compiler can count the loads
// in flight and wait for the current tile only.
template<typename T, int HPT>
struct RopeTile {
    u32x4 tv[HPT];
    f32x4 s_lo, s_hi, c_lo, c_hi;
    uint16_t *base;
    uint16_t *out_base;// wavefront-uniform: the first lane's token
    uint32_t off;      // this lane's byte offset from out_base, head 0
    uint32_t g;
    bool live;
};

template<typename T, typename Idx, int HPT, bool BUFST>
__global__ __launch_bounds__(kBlock) void rope_vec_loop(uint16_t *t, const uint64_t *pos, const float *sin_t, const float *cos_t,
                                                        uint64_t total_items, Idx items_per_token, Idx vecs_per_head, Idx groups,
                                                        uint32_t heads, uint32_t head_dim, int64_t stride_token, int64_t stride_head) {
    const uint64_t tiles = (total_items + kBlock - 1) / kBlock;
    auto fetch = [&](uint64_t tile, RopeTile<T, HPT> &r) {
        const uint64_t item64 = tile * kBlock + threadIdx.x;
        r.live = item64 < total_items;
        const Idx item = static_cast<Idx>(r.live ? item64 : total_items - 1);
        const Idx token = item / items_per_token;
        const Idx rem = item - token * items_per_token;
        const Idx g = rem / vecs_per_head;
        const Idx cv = rem - g * vecs_per_head;
        r.g = static_cast<uint32_t>(g);
        r.base = t + static_cast<int64_t>(token) * stride_token + static_cast<int64_t>(cv) * 8;
        if constexpr (BUFST) {
            const Idx token0 = first_lane(token);
            r.out_base = t + static_cast<int64_t>(token0) * stride_token;
            r.off = static_cast<uint32_t>(token - token0) * static_cast<uint32_t>(stride_token) * 2 + static_cast<uint32_t>(cv) * 16;
        }
#pragma unroll
        for (int i = 0; i < HPT; ++i) {
            uint32_t h = r.g + i * static_cast<uint32_t>(groups);
            h = h < heads ? h : heads - 1;
            r.tv[i] = ld16_stream(r.base + static_cast<int64_t>(h) * stride_head);
        }
        const uint64_t row = pos[token] * head_dim + static_cast<uint64_t>(cv) * 8;
        r.s_lo = ld16f(sin_t + row), r.s_hi = ld16f(sin_t + row + 4);
        r.c_lo = ld16f(cos_t + row), r.c_hi = ld16f(cos_t + row + 4);
    };
    auto rotate = [&](const RopeTile<T, HPT> &r) {
        const float sn[8] = {r.s_lo.x, r.s_lo.y, r.s_lo.z, r.s_lo.w, r.s_hi.x, r.s_hi.y, r.s_hi.z, r.s_hi.w};
        const float cs[8] = {r.c_lo.x, r.c_lo.y, r.c_lo.z, r.c_lo.w, r.c_hi.x, r.c_hi.y, r.c_hi.z, r.c_hi.w};
        const StreamOut<true> out(BUFST ? r.out_base : t);
#pragma unroll
        for (int i = 0; i < HPT; ++i) {
            const uint32_t h = r.g + i * static_cast<uint32_t>(groups);
            float f[8], o[8];
            widen8<T>(r.tv[i], f);
#pragma unroll
            for (int k = 0; k < 8; k += 2) {
                const float a = f[k], b = f[k + 1];
                const float ac = a * cs[k], bs = b * sn[k];
                const float as = a * sn[k + 1], bc = b * cs[k + 1];
                o[k] = ac - bs;
                o[k + 1] = as + bc;
            }
            const u32x4 packed = narrow8<T>(o);
            if (r.live && h < heads) {
                if constexpr (BUFST) {
                    out.st16(r.off + h * static_cast<uint32_t>(stride_head) * 2, packed);
                } else {
                    st16_stream(r.base + static_cast<int64_t>(h) * stride_head, packed);
                }
            }
        }
    };

    uint64_t tile = blockIdx.x;
    if (tile >= tiles) return;
    const uint64_t hop = gridDim.x;
    RopeTile<T, HPT> a, b;
    fetch(tile, a);
    while (true) {
        if (tile + hop >= tiles) {
            rotate(a);
            break;
        }
        fetch(tile + hop, b);
        rotate(a);
        tile += hop;
        if (tile + hop >= tiles) {
            rotate(b);
            break;
        }
        fetch(tile + hop, a);
        rotate(b);
        tile += hop;
    }
}

// One token per tile: when a token's work items fill a workgroup exactly
// (heads / HPT * head_dim / 8 == kBlock), a lane's head group and column group
// never change, the token is the same for the whole workgroup, and its
// position and table rows are found with scalar loads and scalar arithmetic.
// Nothing is predicated.  Workgroups loop over tokens with the next token's
// loads in flight, as rope_vec_loop does.
template<typename T, int HPT>
struct RopeTokenTile {
    u32x4 tv[HPT];
    f32x4 s_lo, s_hi, c_lo, c_hi;
    uint16_t *base;// the token's row: wavefront-uniform
};

template<typename T, int HPT, bool BUFST>
__global__ __launch_bounds__(kBlock) void rope_token_loop(uint16_t *__restrict__ t, const uint64_t *__restrict__ pos,
                                                          const float *__restrict__ sin_t, const float *__restrict__ cos_t,
                                                          uint64_t tokens, uint32_t vecs_per_head, uint32_t groups, uint32_t head_dim,
                                                          int64_t stride_token, int64_t stride_head) {
    const uint32_t g = threadIdx.x / vecs_per_head;
    const uint32_t cv = threadIdx.x - g * vecs_per_head;
    int64_t lane_off[HPT];// elements from the token's row to this lane's vector of head g + i * groups
#pragma unroll
    for (int i = 0; i < HPT; ++i) lane_off[i] = static_cast<int64_t>(g + i * groups) * stride_head + static_cast<int64_t>(cv) * 8;

    auto fetch = [&](uint64_t token, RopeTokenTile<T, HPT> &r) {
        r.base = t + static_cast<int64_t>(token) * stride_token;
#pragma unroll
        for (int i = 0; i < HPT; ++i) r.tv[i] = ld16_stream(r.base + lane_off[i]);
        const uint64_t row = pos[token] * head_dim;
        const float *sp = sin_t + row + cv * 8, *cp = cos_t + row + cv * 8;
        r.s_lo = ld16f(sp), r.s_hi = ld16f(sp + 4);
        r.c_lo = ld16f(cp), r.c_hi = ld16f(cp + 4);
    };
    auto rotate = [&](const RopeTokenTile<T, HPT> &r) {
        const float sn[8] = {r.s_lo.x, r.s_lo.y, r.s_lo.z, r.s_lo.w, r.s_hi.x, r.s_hi.y, r.s_hi.z, r.s_hi.w};
        const float cs[8] = {r.c_lo.x, r.c_lo.y, r.c_lo.z, r.c_lo.w, r.c_hi.x, r.c_hi.y, r.c_hi.z, r.c_hi.w};
        const StreamOut<true> out(r.base);
#pragma unroll
        for (int i = 0; i < HPT; ++i) {
            float f[8], o[8];
            widen8<T>(r.tv[i], f);
#pragma unroll
            for (int k = 0; k < 8; k += 2) {
                const float a = f[k], b = f[k + 1];
                const float ac = a * cs[k], bs = b * sn[k];
                const float as = a * sn[k + 1], bc = b * cs[k + 1];
                o[k] = ac - bs;
                o[k + 1] = as + bc;
            }
            if constexpr (BUFST) {
                out.st16(static_cast<uint32_t>(lane_off[i]) * 2, narrow8<T>(o));
            } else {
                st16_stream(r.base + lane_off[i], narrow8<T>(o));
            }
        }
    };

    uint64_t token = blockIdx.x;
    if (token >= tokens) return;
    const uint64_t hop = gridDim.x;
    RopeTokenTile<T, HPT> a, b;
    fetch(token, a);
    while (true) {
        if (token + hop >= tokens) {
            rotate(a);
            break;
        }
        fetch(token + hop, b);
        rotate(a);
        token += hop;
        if (token + hop >= tokens) {
            rotate(b);
            break;
        }
        fetch(token + hop, a);
        rotate(b);
        token += hop;
    }
}

// Any even head_dim, any strides and alignment: one lane per pair.
template<typename T>
__global__ __launch_bounds__(kBlock) void rope_pairs(uint16_t *t, const uint64_t *pos, const float *sin_t, const float *cos_t,
                                                     uint64_t total_pairs, uint64_t heads, uint64_t head_dim,
                                                     int64_t stride_token, int64_t stride_head) {
    const uint64_t half = head_dim / 2;
    const uint64_t step = static_cast<uint64_t>(gridDim.x) * kBlock;
    for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * kBlock + threadIdx.x; i < total_pairs; i += step) {
        const uint64_t k = i % half;
        const uint64_t th = i / half;
        const uint64_t h = th % heads, token = th / heads;
        uint16_t *p = t + static_cast<int64_t>(token) * stride_token + static_cast<int64_t>(h) * stride_head + 2 * k;
        const uint64_t row = pos[token] * head_dim + 2 * k;
        const float a = T::one(p[0]), b = T::one(p[1]);
        const float ac = a * cos_t[row], bs = b * sin_t[row];
        const float as = a * sin_t[row + 1], bc = b * cos_t[row + 1];
        p[0] = T::narrow1(ac - bs);
        p[1] = T::narrow1(as + bc);
    }
}

template<typename T, typename Idx>
void launch_vec(const RoPEAmdDescriptor &d, uint16_t *t, const uint64_t *pos, const float *sn, const float *cs, hipStream_t stream) {
    const uint64_t vph = d.head_dim / 8;
    const int hpt = d.heads >= kHeadsPerLane ? kHeadsPerLane : (d.heads >= 2 ? 2 : 1);
    const uint64_t groups = ceil_div(d.heads, hpt);
    const uint64_t ipt = groups * vph;
    const uint64_t total = d.tokens * ipt;
    const unsigned grid = static_cast<unsigned>(ceil_div(total, kBlock));
    // Large outputs are written through L2 with buffer stores, which address
    // 32 bits from the first token of a wavefront (it spans at most 64 tokens).
    const bool bufst = d.tokens * d.heads * d.head_dim * sizeof(uint16_t) >= kWriteThroughBytes &&
                       d.stride_token >= 0 && d.stride_head >= 0 &&
                       static_cast<uint64_t>(d.stride_token) < (1ull << 23) &&
                       d.heads * static_cast<uint64_t>(d.stride_head) < (1ull << 30) && d.head_dim < (1ull << 24);
    // Enough tiles to keep every compute unit looping: the prefetching form.
    // Measured on MI355X (256 compute units): q [8192,64,128] bf16, 8192 tiles,
    // 47.0 us looping with 2 workgroups per unit against 48.5 us one tile per
    // workgroup; [4096,32,128] fp16, 2048 tiles, 14.1 us (4 per unit) against
    // 16.8 us; k [8192,8,128], 1024 tiles, is faster one tile per workgroup
    // (9.7 against 10.5 us) and stays on rope_vec (with two heads per lane, and
    // so twice the workgroups, it takes 10.8 us).  Workgroups of 64 or 128
    // lanes, one tile each, measure the same as 256 for all three shapes, and
    // so does a 2-D grid with the token in blockIdx.y (position and table base
    // then come through scalar loads): 47.3 us for q.  With table loads and
    // arithmetic removed the looping form takes 44.7 us for q, so they cost
    // 1.7 us; an out-of-place copy of the same strided rows takes 41.9 us.
    // A token per tile, when some number of heads per lane makes a token fill a
    // workgroup exactly and there are tokens enough to loop over.  Measured on
    // MI355X: q [8192,64,128] bf16 45.1 us with 2 workgroups per compute unit
    // (46.3 with 4, 45.9 with 8) against 46.4 us for rope_vec_loop, whose lanes
    // recompute token, head group and column for every tile; [4096,32,128]
    // fp16 (2 heads per lane) 14.1 us either way.
    if (sizeof(Idx) == 4 && d.tokens >= 8ull * d.cu_count) {
        int h2 = 0;
        for (int cand : {4, 2, 8}) {// not 1: a lane that rotates one head loads four table vectors for it ([32768,32,64]: 62 us against 47)
            if (h2 == 0 && d.heads % cand == 0 && (d.heads / cand) * vph == kBlock) h2 = cand;
        }
        if (h2 != 0) {
            const uint64_t cap2 = static_cast<uint64_t>(d.cu_count) * 2;
            const unsigned g2 = static_cast<unsigned>(d.tokens < cap2 ? d.tokens : cap2);
            const bool b2 = bufst && d.heads * static_cast<uint64_t>(d.stride_head) < (1ull << 30);
#define ROPE_TL(HPT, B) rope_token_loop<T, HPT, B><<<g2, kBlock, 0, stream>>>(t, pos, sn, cs, d.tokens, static_cast<uint32_t>(vph), static_cast<uint32_t>(d.heads / HPT), static_cast<uint32_t>(d.head_dim), d.stride_token, d.stride_head)
            if (b2) { if (h2 == 4) ROPE_TL(4, true); else if (h2 == 2) ROPE_TL(2, true); else ROPE_TL(8, true); }
            else { if (h2 == 4) ROPE_TL(4, false); else if (h2 == 2) ROPE_TL(2, false); else ROPE_TL(8, false); }
#undef ROPE_TL
            return;
        }
    }
    if (grid >= 8u * static_cast<unsigned>(d.cu_count)) {
        const uint64_t per_cu = grid >= 16u * static_cast<unsigned>(d.cu_count) ? 2 : 4;
        const uint64_t cap = static_cast<uint64_t>(d.cu_count) * per_cu;
        const unsigned lgrid = static_cast<unsigned>(grid < cap ? grid : cap);
#define ROPE_LAUNCH_LOOP(HPT, B)                                                                                                    \
    rope_vec_loop<T, Idx, HPT, B><<<lgrid, kBlock, 0, stream>>>(t, pos, sn, cs, total, static_cast<Idx>(ipt), static_cast<Idx>(vph), \
                                                                static_cast<Idx>(groups), static_cast<uint32_t>(d.heads),           \
                                                                static_cast<uint32_t>(d.head_dim), d.stride_token, d.stride_head)
        if (bufst) {
            if (hpt == 4) ROPE_LAUNCH_LOOP(4, true);
            else if (hpt == 2) ROPE_LAUNCH_LOOP(2, true);
            else ROPE_LAUNCH_LOOP(1, true);
        } else {
            if (hpt == 4) ROPE_LAUNCH_LOOP(4, false);
            else if (hpt == 2) ROPE_LAUNCH_LOOP(2, false);
            else ROPE_LAUNCH_LOOP(1, false);
        }
#undef ROPE_LAUNCH_LOOP
        return;
    }
#define ROPE_LAUNCH(HPT, B)                                                                                                   \
    rope_vec<T, Idx, HPT, B><<<grid, kBlock, 0, stream>>>(t, pos, sn, cs, total, static_cast<Idx>(ipt), static_cast<Idx>(vph), \
                                                          static_cast<Idx>(groups), static_cast<uint32_t>(d.heads),           \
                                                          static_cast<uint32_t>(d.head_dim), d.stride_token, d.stride_head)
    if (bufst) {
        if (hpt == 4) ROPE_LAUNCH(4, true);
        else if (hpt == 2) ROPE_LAUNCH(2, true);
        else ROPE_LAUNCH(1, true);
    } else {
        if (hpt == 4) ROPE_LAUNCH(4, false);
        else if (hpt == 2) ROPE_LAUNCH(2, false);
        else ROPE_LAUNCH(1, false);
    }
#undef ROPE_LAUNCH
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
        const uint64_t pairs = elems / 2;
        const uint64_t want = ceil_div(pairs, kBlock), cap = static_cast<uint64_t>(d.cu_count) * 64;
        rope_pairs<T><<<static_cast<unsigned>(want < cap ? want : cap), kBlock, 0, stream>>>(
            pt, pos, sn, cs, pairs, d.heads, d.head_dim, d.stride_token, d.stride_head);
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
