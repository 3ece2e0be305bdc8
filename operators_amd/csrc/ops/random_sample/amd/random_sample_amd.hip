// RandomSample on gfx950.
//
// The reference's CPU path (src/ops/random_sample/cpu/random_sample.cc:47-171)
// sorts the topk largest logits to the front with a selection sort, turns the
// logits into fp16 probabilities, keeps the sorted prefix whose running sum
// reaches topp and draws from it with random_val.  What is reproduced here is
// that arithmetic - fp32 (x - max) / temperature, expf, division by the sum,
// truncation to fp16, the running fp32 sums in sorted order, every comparison -
// not the sort.  A vocabulary is 64-300 KiB: no work for the memory system, a
// latency chain for a sort.  So nothing is sorted:
//  * the key of the topk-th largest logit is found by a radix select over the
//    16-bit codes (four passes of 4 bits; counters in registers or packed
//    fields summed over the wavefront with DPP adds, no atomics on hot bins);
//  * the at most topk candidates are compacted into LDS and ranked there by
//    (logit descending, index ascending), one candidate per lane;
//  * the first wavefront forms the sequential running sums once, as a
//    branch-free chain with the addends in registers, and takes the top-p and
//    random_val decisions with ballots over them.
// That is the form for up to 256 candidates (topk after clamping) when the
// caller hands over the workspace the descriptor asks for and there are 4096
// logits or more: a first launch spreads the pass over the logits over up to
// 48 workgroups, each of which drops everything that cannot be in the overall
// topk, and a second launch of one workgroup finishes from the few hundred
// survivors (6.9 + 10.3 us for 32 000 logits, 9.7 + 14.0 us for 151 936).
// (One workgroup can do all of it from the logits alone - topk_full, which the
// second launch falls back to when a list overflows - but takes several times
// as long: one compute unit's instruction rate is the limit.)
// More candidates than that - any number, the reference has no limit - and
// every call without the workspace are not ranked at all: the running sums
// are formed over a histogram of the keys (further down).
//
// Two things differ from the CPU path and are visible to a caller:
//  * equal logits: the CPU's selection sort leaves equal values in an order
//    that depends on its swap history; here they are ordered by ascending
//    index.  The logit at the returned index is the same either way, which is
//    what the reference's own test accepts (operatorspy/tests/random_sample.py:
//    `indices == ans or data[indices] == data[ans]`);
//  * the softmax denominator is summed as a tree (and, in the two-launch form,
//    per workgroup relative to the workgroup's own maximum, then rescaled), not
//    left to right, so a probability can differ in its last fp16 bit in rare
//    cases.
// NaN logits: the greedy form treats them as the CPU does (never greater than
// anything; one in front wins); the sampling form ranks them below -Inf.
#include "../../../devices/amd/kernel_amd.h"
#include "random_sample_amd.h"
#include <mutex>

namespace {

using namespace amd;

constexpr int BS = 1024;
constexpr int WAVES = BS / kWave;
constexpr int KMAX = kRandomSampleMaxTopk;
constexpr uint32_t kNoKey = 0xFFFFFFFFu;// marks a slot past the end of the logits

// Code of +Inf: everything above it (sign aside) is a NaN.
template<typename T>
constexpr uint32_t kInfCode = 0x7C00u;
template<>
constexpr uint32_t kInfCode<BF16Rne> = 0x7F80u;

// Order-preserving 16-bit key of an fp16 or bf16 code (both are sign-magnitude):
// a greater value has a greater key, -0 and +0 share one, NaN is the smallest.
template<typename T>
__device__ __forceinline__ uint32_t key_of(uint32_t h) {
    if ((h & 0x7FFFu) > kInfCode<T>) return 0u;
    if (h == 0x8000u) h = 0u;
    return (h & 0x8000u) ? (h ^ 0xFFFFu) : (h | 0x8000u);
}
template<typename T>
__device__ __forceinline__ float value_of_key(uint32_t k) {
    const uint32_t h = (k & 0x8000u) ? (k & 0x7FFFu) : (k ^ 0xFFFFu);
    return T::one(static_cast<uint16_t>(h));
}

// The eight codes starting at element `base` (a multiple of 8): one 128-bit
// load when they all exist and the array is 16-byte aligned, element loads
// otherwise; slots past the end read as 0 and are flagged in `n`.
template<bool VEC>
__device__ __forceinline__ int load_codes(const uint16_t *p, uint32_t voc, uint32_t base, uint32_t (&h)[8]) {
    if (base >= voc) {
#pragma unroll
        for (int e = 0; e < 8; ++e) h[e] = 0;
        return 0;
    }
    if (VEC && base + 8 <= voc) {
        const u32x4 v = ld16(p + base);
        h[0] = v.x & 0xFFFFu, h[1] = v.x >> 16, h[2] = v.y & 0xFFFFu, h[3] = v.y >> 16;
        h[4] = v.z & 0xFFFFu, h[5] = v.z >> 16, h[6] = v.w & 0xFFFFu, h[7] = v.w >> 16;
        return 8;
    }
    const int n = voc - base < 8u ? static_cast<int>(voc - base) : 8;
#pragma unroll
    for (int e = 0; e < 8; ++e) h[e] = e < n ? p[base + e] : 0u;
    return n;
}

// A pass of `lanes` lanes over the logits [begin, end) (begin a multiple of
// 8): lane `me` takes the 8-logit vectors me, me + lanes, ... of the range and
// calls body(base, codes, n) for each (n < 8 only for the vector that holds
// the end).  With a 16-byte aligned array the loads of U vectors are issued
// together before the first is used: a workgroup that walks a few hundred KB
// alone is bound by the latency of each round of loads, not by bandwidth
// (151 936 logits, 1024 lanes: 19 rounds of one load against 3 rounds of 8).
template<bool VEC, int U, typename F>
__device__ __forceinline__ void sweep_logits(const uint16_t *probs, uint32_t begin, uint32_t end, uint32_t me, uint32_t lanes, F &&body) {
    if constexpr (VEC) {
        const uint32_t full = begin + (end - begin) / 8u * 8u;// end of the whole vectors
        if (full > begin) {
            const uint32_t last = full - 8u;
            for (uint32_t base0 = begin + me * 8u; base0 < full; base0 += lanes * 8u * U) {
                u32x4 v[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const uint32_t b = base0 + static_cast<uint32_t>(u) * lanes * 8u;
                    v[u] = ld16(probs + (b < full ? b : last));// a vector past the range re-reads the last one and is dropped below
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const uint32_t b = base0 + static_cast<uint32_t>(u) * lanes * 8u;
                    if (b < full) {
                        const uint32_t h[8] = {v[u].x & 0xFFFFu, v[u].x >> 16, v[u].y & 0xFFFFu, v[u].y >> 16,
                                               v[u].z & 0xFFFFu, v[u].z >> 16, v[u].w & 0xFFFFu, v[u].w >> 16};
                        body(b, h, 8);
                    }
                }
            }
        }
        if (full < end && me == ((full - begin) / 8u) % lanes) {// the partial vector, by the lane whose turn it is
            uint32_t h[8];
            const int n = static_cast<int>(end - full);
#pragma unroll
            for (int e = 0; e < 8; ++e) h[e] = e < n ? probs[full + e] : 0u;
            body(full, h, n);
        }
    } else {
        for (uint32_t base = begin + me * 8u; base < end; base += lanes * 8u) {
            uint32_t h[8];
            const int n = end - base < 8u ? static_cast<int>(end - base) : 8;
#pragma unroll
            for (int e = 0; e < 8; ++e) h[e] = e < n ? probs[base + e] : 0u;
            body(base, h, n);
        }
    }
}

// Sum over the 64 lanes with DPP adds (the lane pattern of amd::wave_sum):
// four steps inside each row of 16 lanes, then row broadcasts 15 and 31; the
// total lands in lane 63 and is read back to every lane through an SGPR.
__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t v) {
    int x = static_cast<int>(v);
    x += __builtin_amdgcn_update_dpp(0, x, 0xB1, 0xF, 0xF, false); // quad_perm [1,0,3,2]
    x += __builtin_amdgcn_update_dpp(0, x, 0x4E, 0xF, 0xF, false); // quad_perm [2,3,0,1]
    x += __builtin_amdgcn_update_dpp(0, x, 0x141, 0xF, 0xF, false);// row_half_mirror
    x += __builtin_amdgcn_update_dpp(0, x, 0x140, 0xF, 0xF, false);// row_mirror
    x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xA, 0xF, false);// row_bcast:15 -> rows 1, 3
    x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xC, 0xF, false);// row_bcast:31 -> rows 2, 3
    return static_cast<uint32_t>(__builtin_amdgcn_readlane(x, 63));
}
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const uint32_t other = __shfl_xor(v, o);
        v = other > v ? other : v;
    }
    return v;
}
__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const unsigned long long other = __shfl_xor(v, o);
        v = other > v ? other : v;
    }
    return v;
}
// Inclusive prefix sum over the lanes of a wavefront with DPP adds: shifts by
// 1, 2, 4 and 8 lanes inside each row of 16, then the last lane of row 0 and
// of row 2 onto the rows that follow (row_bcast:15 for rows 1 and 3), then the
// last lane of row 1 onto rows 2 and 3 (row_bcast:31).  Lanes a shift does not
// reach add zero.
__device__ __forceinline__ uint32_t wave_scan_u32(uint32_t v) {
    int x = static_cast<int>(v);
    x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xF, 0xF, false);// row_shr:1
    x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xF, 0xF, false);// row_shr:2
    x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xF, 0xF, false);// row_shr:4
    x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xF, 0xF, false);// row_shr:8
    x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xA, 0xF, false);// row_bcast:15 -> rows 1, 3
    x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xC, 0xF, false);// row_bcast:31 -> rows 2, 3
    return static_cast<uint32_t>(x);
}

// Greedy form (random_sample.cc:127-148): the first index holding the maximum,
// where NaN is never greater than anything and a NaN in front is never beaten.
template<typename T, bool VEC>
__global__ __launch_bounds__(BS) void random_sample_greedy(uint64_t *result, const uint16_t *probs, uint32_t voc) {
    AMD_ARGS_NOW(result, probs, voc);
    __shared__ unsigned long long best_of[WAVES];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    unsigned long long best = 0;
    for (uint32_t base = tid * 8u; base < voc; base += BS * 8u) {
        uint32_t h[8];
        const int n = load_codes<VEC>(probs, voc, base, h);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if (e < n) {
                // greater key first, then the lower index
                const unsigned long long c = (static_cast<unsigned long long>(key_of<T>(h[e])) << 32) | (0xFFFFFFFFu - (base + e));
                best = c > best ? c : best;
            }
        }
    }
    best = wave_max_u64(best);
    if (lane == 0) best_of[wave] = best;
    __syncthreads();
    if (tid == 0) {
#pragma unroll
        for (int w = 1; w < WAVES; ++w) best = best_of[w] > best ? best_of[w] : best;
        const uint32_t first = probs[0];
        const bool first_is_nan = (first & 0x7FFFu) > kInfCode<T>;
        result[0] = first_is_nan ? 0ull : static_cast<unsigned long long>(0xFFFFFFFFu - static_cast<uint32_t>(best));
    }
}

// LDS of the sampling kernels.
struct TopkShared {
    uint32_t wave_cnt[2][WAVES * 16];// per-wavefront digit counts of one select pass (two sets, used in turn)
    uint32_t digit_cnt[16];          // their totals
    uint32_t wave_key[WAVES];        // per-wavefront maximum key
    uint32_t scan_tot[2][WAVES][2];  // per-wavefront (greater, equal) counts of one compaction step
    float sum_slots[WAVES];
    unsigned long long cand[KMAX];   // key << 32 | ~index
    float sorted_p[KMAX];            // probabilities, widened, in descending order of logit
    uint32_t sorted_i[KMAX];         // their indices
};

// One step of a radix select over 16-bit keys: digit_cnt holds how many of the
// entries that share `prefix` have each value of the next 4-bit digit; walk
// down from 15 to the digit that contains the entry of rank `want`.
__device__ __forceinline__ void choose_digit(const uint32_t *digit_cnt, uint32_t &prefix, uint32_t &want) {
    uint32_t above = 0, chosen = 0;
    bool found = false;
#pragma unroll
    for (int d = 15; d >= 0; --d) {
        const uint32_t c = digit_cnt[d];
        if (!found) {
            if (above + c >= want) {
                chosen = d;
                found = true;
            } else {
                above += c;
            }
        }
    }
    want -= above;
    prefix = (prefix << 4) | chosen;
}

// Rank the `count` candidates of sh.cand (greater logit first, then the lower
// index), turn the first topk of them into fp16 probabilities and walk the
// running sums of random_sample.cc:97-125 in their order.  Ends with the
// result written, or left alone when no running sum exceeds the limit.
template<typename T>
__device__ __forceinline__ void rank_and_draw(TopkShared &sh, uint64_t *result, uint32_t count, uint32_t topk, float top,
                                              float total, float random_val, float topp, float temperature) {
    const int tid = threadIdx.x;
    if (static_cast<uint32_t>(tid) < count) {
        const unsigned long long mine = sh.cand[tid];
        uint32_t rank = 0;
        for (uint32_t j = 0; j < count; ++j) rank += sh.cand[j] > mine ? 1u : 0u;
        if (rank < topk) {
            const float x = value_of_key<T>(static_cast<uint32_t>(mine >> 32));
            const float p = expf((x - top) / temperature) / total;
            sh.sorted_p[rank] = T::one(T::narrow1(p));
            sh.sorted_i[rank] = 0xFFFFFFFFu - static_cast<uint32_t>(mine);
        }
    }
    __syncthreads();
    // The reference walks the sorted probabilities three times with a running
    // fp32 sum that starts from zero each time: to find where it reaches topp,
    // to total the kept prefix, to find where it exceeds random_val times that
    // total.  All three see the same sequence of partial sums, and those have
    // to be formed by sequential additions to round as the reference's do.
    // So the first wavefront forms them once, 64 at a time, in a branch-free
    // chain - the addends come out of a register by constant lane number, lane
    // i keeps the i-th partial sum - and takes the two decisions with ballots
    // over the stored sums.  (A loop that adds, compares and branches per
    // entry costs 47 ns per entry here: 4.7 us for topk = 50.)
    if (tid < kWave) {
        float run = 0.0f, kept = 0.0f;
        uint32_t end = topk;
        bool stopped = false;
        for (uint32_t c0 = 0; c0 < topk && !stopped; c0 += kWave) {
            const bool live = c0 + tid < topk;
            const float p = live ? sh.sorted_p[c0 + tid] : 0.0f;
            float mine = 0.0f;
#pragma unroll
            for (int i = 0; i < kWave; ++i) {
                run += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, p), i));
                mine = tid == i ? run : mine;
            }
            if (live) sh.sorted_p[c0 + tid] = mine;// from here on the array holds the partial sums
            const unsigned long long reached = __builtin_amdgcn_ballot_w64(live && mine >= topp);
            if (reached != 0) {
                const int at = __builtin_ctzll(reached);
                end = c0 + at;
                kept = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mine), at));
                stopped = true;
            }
        }
        // the sum of the kept prefix: the partial sum at the entry where the
        // walk stopped (that entry is the last one kept, or the last of all),
        // or the sum of all topk entries when it never stopped
        if (!stopped) kept = run;
        end = end + 1 < topk ? end + 1 : topk;
        const float limit = random_val * kept;
        for (uint32_t c0 = 0; c0 < end; c0 += kWave) {
            const bool live = c0 + tid < end;
            const float upto = live ? sh.sorted_p[c0 + tid] : 0.0f;
            const unsigned long long above = __builtin_amdgcn_ballot_w64(live && limit < upto);
            if (above != 0) {
                if (tid == 0) result[0] = sh.sorted_i[c0 + __builtin_ctzll(above)];
                break;
            }
        }
    }
}

// Sampling form (random_sample.cc:47-126), everything by one workgroup from
// the logits themselves.  topk is already clamped to [2, min(voc, KMAX)].
template<typename T, bool VEC>
__device__ __attribute__((noinline)) void topk_full(TopkShared &sh, uint64_t *result, const uint16_t *probs, uint32_t voc,
                                          float random_val, float topp, uint32_t topk, float temperature) {
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t step = BS * 8u;

    // ---- radix select: the key of the topk-th largest logit ----------------
    uint32_t prefix = 0;   // the digits chosen so far
    uint32_t want = topk;  // rank looked for among the elements that share them
    uint32_t key_max = 0;
#pragma unroll 1
    for (int shift = 12; shift >= 0; shift -= 4) {
        // Per-lane digit counts.  An element adds a one to an 8-bit field (digit
        // d: field d & 3 of word d >> 2), four conditional adds instead of
        // sixteen; a lane adds at most eight ones per round, so the fields are
        // emptied into full-width counters every 31 rounds.
        uint32_t cnt[16], packed[4] = {0, 0, 0, 0};
#pragma unroll
        for (int d = 0; d < 16; ++d) cnt[d] = 0;
        const auto unpack = [&]() {
#pragma unroll
            for (int d = 0; d < 16; ++d) cnt[d] += (packed[d >> 2] >> (8 * (d & 3))) & 0xFFu;
#pragma unroll
            for (int w = 0; w < 4; ++w) packed[w] = 0;
        };
        uint32_t since = 0;
        for (uint32_t base = tid * 8u; base < voc; base += step) {
            uint32_t h[8];
            const int n = load_codes<VEC>(probs, voc, base, h);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t k = e < n ? key_of<T>(h[e]) : kNoKey;
                if (shift == 12 && e < n) key_max = k > key_max ? k : key_max;
                const bool in = (k >> (shift + 4)) == prefix;// never true for kNoKey: prefix < 2^12
                const uint32_t digit = (k >> shift) & 15u;
                const uint32_t one = in ? 1u << (8u * (digit & 3u)) : 0u;
                const uint32_t word = digit >> 2;
#pragma unroll
                for (int w = 0; w < 4; ++w) packed[w] += word == static_cast<uint32_t>(w) ? one : 0u;
            }
            if (++since == 31) {
                unpack();
                since = 0;
            }
        }
        unpack();
        uint32_t mine = 0;
#pragma unroll
        for (int d = 0; d < 16; ++d) {
            const uint32_t t = wave_sum_u32(cnt[d]);
            if (lane == d) mine = t;
        }
        if (lane < 16) sh.wave_cnt[0][wave * 16 + lane] = mine;
        if (shift == 12) {
            const uint32_t m = wave_max_u32(key_max);
            if (lane == 0) sh.wave_key[wave] = m;
        }
        __syncthreads();
        if (tid < 16) {
            uint32_t t = 0;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) t += sh.wave_cnt[0][w * 16 + tid];
            sh.digit_cnt[tid] = t;
        }
        __syncthreads();
        choose_digit(sh.digit_cnt, prefix, want);
    }
    const uint32_t key_k = prefix;          // key of the topk-th largest
    const uint32_t need_eq = want;          // how many of its equals belong to the topk
    const uint32_t n_greater = topk - want; // elements with a greater key
#pragma unroll
    for (int w = 0; w < WAVES; ++w) key_max = sh.wave_key[w] > key_max ? sh.wave_key[w] : key_max;
    const float top = value_of_key<T>(key_max);

    // ---- compaction in index order, and the softmax denominator ------------
    float part = 0.0f;
    uint32_t run_gt = 0, run_eq = 0;
    int buf = 0;
    const uint32_t rounds = (voc + step - 1) / step;
#pragma unroll 1
    for (uint32_t r = 0; r < rounds; ++r, buf ^= 1) {
        const uint32_t base = r * step + tid * 8u;
        uint32_t h[8], k[8];
        const int n = load_codes<VEC>(probs, voc, base, h);
        uint32_t c_gt = 0, c_eq = 0;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            k[e] = e < n ? key_of<T>(h[e]) : kNoKey;
            if (e < n) {
                part += expf((T::one(static_cast<uint16_t>(h[e])) - top) / temperature);
                c_gt += k[e] > key_k ? 1u : 0u;
                c_eq += k[e] == key_k ? 1u : 0u;
            }
        }
        const uint32_t inc_gt = wave_scan_u32(c_gt), inc_eq = wave_scan_u32(c_eq);
        if (lane == kWave - 1) {
            sh.scan_tot[buf][wave][0] = inc_gt;
            sh.scan_tot[buf][wave][1] = inc_eq;
        }
        __syncthreads();
        uint32_t at_gt = run_gt + inc_gt - c_gt, at_eq = run_eq + inc_eq - c_eq;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const uint32_t g = sh.scan_tot[buf][w][0], q = sh.scan_tot[buf][w][1];
            if (w < wave) at_gt += g, at_eq += q;
            run_gt += g, run_eq += q;
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if (e < n) {
                const unsigned long long c = (static_cast<unsigned long long>(k[e]) << 32) | (0xFFFFFFFFu - (base + e));
                if (k[e] > key_k) {
                    sh.cand[at_gt++] = c;
                } else if (k[e] == key_k) {
                    if (at_eq < need_eq) sh.cand[n_greater + at_eq] = c;
                    ++at_eq;
                }
            }
        }
    }
    part = wave_sum(part);
    if (lane == 0) sh.sum_slots[wave] = part;
    __syncthreads();// candidates and partial sums are in LDS
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) total += sh.sum_slots[w];
    rank_and_draw<T>(sh, result, topk, topk, top, total, random_val, topp, temperature);
}

// ---- more candidates than LDS ranks: sampling without a sorted list -----------
// The reference keeps any topk up to the vocabulary size (random_sample.cc:
// 67-74 only clamps it).  Beyond 256 candidates nothing is compacted or
// ranked.  Equal logits have equal probabilities, so the sorted sequence the
// reference walks is fully described by how often every 16-bit code occurs: a
// histogram over the ordered keys, walked from the largest key down, adding
// each key's probability as many times as the key occurs - the same fp32
// running sums, the same comparisons:
//   1. the largest key and the softmax denominator, part by part (see
//      part_max_and_sum);
//   2. walk 1 finds where the running sum reaches topp (or the topk-th entry)
//      and with it the sum of the kept prefix; walk 2 finds the entry whose
//      running sum exceeds random_val times that sum.  A walk takes the key
//      space in ranges of kWideBins keys from the top: the counts of the
//      range's keys into LDS, every occupied key's probability in parallel,
//      then the first wavefront goes through them in order.  Walks stop as
//      soon as their question is answered - for ordinary top-p values within
//      the first range - and the second walk starts on the range the first
//      one left in LDS;
//   3. the answer is "occurrence r of key K": every wavefront counts K in its
//      contiguous sixteenth of the logits, and the wavefront whose part holds
//      occurrence r goes through it once more in order.  Equal logits are
//      thereby ordered by ascending index, as in the other form.
// With the workspace, two launches before the one workgroup that draws take
// what can be spread over the chip: the counts of all 65 536 keys (cleared,
// then one atomic add per logit) and every part's maximum and sum; the walks
// then read a range's counts instead of passing over the logits, and once a
// walk has left the first range it steps over whole ranges in which nothing
// can happen (wide_range_totals) - a top-p of 1 with top-k off, plain
// sampling from the whole distribution, costs little more than a peaked one.
// Without the workspace the one workgroup counts a range at a time itself.
// 151 936 fp16 logits, top-k off, MI355X, with the workspace: 54 us at top-p
// 0.9 (4.5 clear + 17.7 count + 28.8 draw), 112 us at top-p 1; without:
// 87 us and 0.41 ms.  (Before the measures described here and below: 223 us
// and 5.9 ms.)
// The additions need not be made one by one.  An fp16 probability is a whole
// number of units of 2^-24 (the spacing of fp16 subnormals), and so is every
// sum of them; below 1.0 an fp32 holds any such number exactly (at most 24
// significant bits).  Up to a running sum of 1.0, therefore, no addition of
// the reference's chain rounds, the chain's value after any number of entries
// is the plain integer sum of their units, and the walk can take 64 keys at a
// time: a prefix sum of count * units over the lanes, a ballot for the first
// key at which the comparison turns, one integer division for the entry
// inside that key.  Only a running sum that passes 1.0 (one-hot
// distributions; bf16 probabilities, which are finer than 2^-24, always) is
// continued one entry at a time, as the reference adds.  On its own this
// took 151 936 logits with top-k off from 223 to 123 us at top-p 0.9, from 760
// to 131 us at top-p 0.99 and from 5.9 ms to 0.47 ms for a distribution so
// flat that the walk covers the whole vocabulary.
constexpr int kWideBins = 4096;
constexpr int kWideRanges = static_cast<int>(kRandomSampleKeys) / kWideBins;
constexpr uint32_t kOneUnits = 1u << 24;     // 1.0 in units of 2^-24
constexpr uint32_t kManyUnits = 1u << 25;    // stands for "more than 1.0" in a prefix sum of 64 terms

// Probabilities of T as whole units of 2^-24: fp16 only.
template<typename T> struct ExactUnits { static constexpr bool value = false; };
template<> struct ExactUnits<F16Ref> { static constexpr bool value = true; };

// The smallest running sum, in units, for which a walk's comparison holds:
// MODE 0 asks run >= threshold, MODE 1 asks threshold < run.
template<int MODE>
__device__ __forceinline__ uint32_t walk_threshold_units(float threshold) {
    if (!(threshold == threshold)) return 0xFFFFFFFFu;// NaN compares false with everything
    const double t = static_cast<double>(threshold) * 16777216.0;
    if (MODE == 0) {
        if (t <= 0.0) return 0u;
        return t > 4.0e9 ? 0xFFFFFFFFu : static_cast<uint32_t>(ceil(t));
    }
    if (t < 0.0) return 0u;
    return t >= 4.0e9 ? 0xFFFFFFFFu : static_cast<uint32_t>(floor(t)) + 1u;
}

struct WideShared {
    uint32_t hist[kWideBins];
    float p_of[kWideBins];
    uint32_t wave_key[WAVES];
    float sum_slots[WAVES];
    uint32_t wave_tot[WAVES];
    uint32_t part_key[kRandomSampleMaxGroups];// per part of the logits: its largest key and its
    float part_sum[kRandomSampleMaxGroups];   // sum of expf((x - its largest) / temperature)
    // state of a walk, written by the first wavefront
    uint32_t done, found, entry, key, occurrence;
    float run;
    uint32_t n;
    uint32_t exact;// the running sum is still a whole number of units of 2^-24, at most 1.0
    int64_t range_top;// the key range hist and p_of describe now, by its top key; -1: none
    // per range of kWideBins keys from the top: what all its entries add to the running sum, in units (kManyUnits:
    // more than the exact walk handles), and how many entries it has; filled on demand
    unsigned long long range_sum[kWideRanges];
    uint32_t range_units[kWideRanges], range_count[kWideRanges];
    uint32_t ranges_known;
};

// What every range of keys adds to the running sum and to the entry count,
// from the counts of all keys (split form, exact units only).  A walk that has
// left the first range behind asks for this once and then steps over every
// range in which nothing can happen - a top-p of 1 sends the first walk
// through the whole vocabulary only to learn the sum - instead of fetching
// and walking it.  Lane l takes the 64 keys from 64 * l up (they lie in at
// most two ranges); a key's probability is formed exactly as the walk forms
// it, except that keys so far below the top that it must truncate to zero
// (expf(d) / total < 2^-24, the smallest fp16) are not exponentiated.
template<typename T>
__device__ __attribute__((noinline)) void wide_range_totals(WideShared &sh, const uint32_t *counts, uint32_t key_max, float top, float total,
                                                          float temperature) {
    const uint32_t tid = threadIdx.x;
    if (tid < static_cast<uint32_t>(kWideRanges)) {
        sh.range_sum[tid] = 0;
        sh.range_count[tid] = 0;
    }
    __syncthreads();
    const uint32_t k0 = tid * 64u;
    if (k0 <= key_max) {
        const float zero_below = logf(total) - 17.0f;
        const uint32_t r_far = (key_max - k0) / kWideBins;// the range of the lowest key; the highest is in it or in the one before
        unsigned long long sum_far = 0, sum_near = 0;
        uint32_t cnt_far = 0, cnt_near = 0;
#pragma unroll 1
        for (int half = 0; half < 2; ++half) {// 32 keys' counts in flight at a time: the calling kernel has 128 registers a lane
        u32x4 c[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) c[i] = *reinterpret_cast<const u32x4 *>(counts + k0 + 32 * half + 4 * i);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t four[4] = {c[i].x, c[i].y, c[i].z, c[i].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t k = k0 + 32 * half + 4 * i + j, n = four[j];
                if (n != 0 && k <= key_max) {
                    const float d = (value_of_key<T>(k) - top) / temperature;
                    uint32_t units = 0;
                    if (!(d < zero_below)) {
                        const float p = T::one(T::narrow1(expf(d) / total));
                        units = p <= 1.0f ? static_cast<uint32_t>(p * 16777216.0f) : kManyUnits;
                    }
                    unsigned long long add = static_cast<unsigned long long>(n) * units;
                    add = add > kManyUnits ? kManyUnits : add;
                    if ((key_max - k) / kWideBins == r_far) sum_far += add, cnt_far += n;
                    else sum_near += add, cnt_near += n;
                }
            }
        }
        }
        if (cnt_far != 0) {
            atomicAdd(&sh.range_sum[r_far], sum_far);
            atomicAdd(&sh.range_count[r_far], cnt_far);
        }
        if (cnt_near != 0) {// r_far >= 1 here
            atomicAdd(&sh.range_sum[r_far - 1], sum_near);
            atomicAdd(&sh.range_count[r_far - 1], cnt_near);
        }
    }
    __syncthreads();
    if (tid < static_cast<uint32_t>(kWideRanges)) sh.range_units[tid] = sh.range_sum[tid] > kManyUnits ? kManyUnits : static_cast<uint32_t>(sh.range_sum[tid]);
    if (tid == 0) sh.ranges_known = 1;
    __syncthreads();
}

// One walk over the sorted sequence.  MODE 0: stop at the first entry whose
// running sum reaches `threshold` (found = 1, entry = its rank), or after
// `limit_n` entries.  MODE 1: stop at the first entry whose running sum
// exceeds `threshold` (found = 1, key/occurrence name it), or after `limit_n`.
// Leaves the running sum in sh.run.  All lanes call it.
template<typename T, bool VEC, int MODE>
__device__ __forceinline__ void wide_walk(WideShared &sh, const uint16_t *probs, uint32_t voc, const uint32_t *counts, uint32_t key_max,
                                          float top, float total, float temperature, float threshold, uint32_t limit_n) {
    const int tid = threadIdx.x, lane = tid & (kWave - 1);
    if (tid == 0) {
        sh.done = limit_n == 0 ? 1u : 0u;
        sh.found = 0;
        sh.run = 0.0f;
        sh.n = 0;
        sh.exact = ExactUnits<T>::value ? 1u : 0u;
    }
    const uint32_t thr = walk_threshold_units<MODE>(threshold);
    __syncthreads();
    for (int64_t hi = key_max; hi >= 0; hi -= kWideBins) {
        if (sh.done != 0) break;// uniform: written before the last barrier
        if (ExactUnits<T>::value && counts != nullptr && hi != static_cast<int64_t>(key_max) && sh.exact != 0) {
            // past the first range, with every key's count at hand: step over this range if nothing happens in it
            if (sh.ranges_known == 0) wide_range_totals<T>(sh, counts, key_max, top, total, temperature);
            const int r = static_cast<int>((static_cast<int64_t>(key_max) - hi) / kWideBins);
            const uint32_t adds = sh.range_units[r], entries = sh.range_count[r];
            const uint32_t units_run = static_cast<uint32_t>(sh.run * 16777216.0f), n = sh.n;
            if (adds < kManyUnits && units_run + adds <= kOneUnits && units_run + adds < thr && n + entries < limit_n) {
                __syncthreads();// everyone has read the state
                if (tid == 0) {
                    sh.run = static_cast<float>(units_run + adds) * (1.0f / 16777216.0f);
                    sh.n = n + entries;
                }
                __syncthreads();
                continue;
            }
        }
        if (sh.range_top != hi) {// uniform; the second walk finds the first walk's last range still there
            __syncthreads();// everyone has read range_top
            if (tid == 0) sh.range_top = hi;
            if (counts != nullptr) {// counted by an earlier launch: key k's count is counts[k]
                for (int b = tid; b < kWideBins; b += BS) sh.hist[b] = static_cast<int64_t>(b) <= hi ? counts[hi - b] : 0u;
            } else {
                for (int b = tid; b < kWideBins; b += BS) sh.hist[b] = 0;
                __syncthreads();
                sweep_logits<VEC, 8>(probs, 0, voc, tid, BS, [&](uint32_t, const uint32_t(&h)[8], int n) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        if (e < n) {
                            const uint32_t below = static_cast<uint32_t>(hi) - key_of<T>(h[e]);// wraps for keys above the range
                            if (below < static_cast<uint32_t>(kWideBins)) atomicAdd(&sh.hist[below], 1u);
                        }
                    }
                });
            }
            __syncthreads();
            for (int b = tid; b < kWideBins; b += BS) {
                float p = 0.0f;
                if (sh.hist[b] != 0 && static_cast<int64_t>(b) <= hi) {
                    const float x = value_of_key<T>(static_cast<uint32_t>(hi - b));
                    p = T::one(T::narrow1(expf((x - top) / temperature) / total));
                }
                sh.p_of[b] = p;
            }
            __syncthreads();
        }
        if (tid < kWave) {
            float run = sh.run;
            uint32_t n = sh.n;
            bool done = false;
            bool exact = sh.exact != 0;
            uint32_t units_run = exact ? static_cast<uint32_t>(run * 16777216.0f) : 0u;// exact: see above
            for (int b0 = 0; b0 < kWideBins && !done; b0 += kWave) {
                const uint32_t c = sh.hist[b0 + lane];
                const float p = sh.p_of[b0 + lane];
                int from = 0;// first lane of this chunk still to be taken one entry at a time
                if (exact && __builtin_amdgcn_ballot_w64(c != 0 && !(p <= 1.0f)) != 0) {
                    // a probability that is no number of units (NaN from NaN logits or a zero temperature): the
                    // reference's own additions and comparisons decide, one entry at a time
                    exact = false;
                    run = static_cast<float>(units_run) * (1.0f / 16777216.0f);
                }
                if (exact) {
                    // 64 keys at once.  A key takes min(its count, what the entry limit leaves).
                    const uint32_t room = limit_n - n;
                    const uint32_t cnt_incl = wave_scan_u32(c), cnt_excl = cnt_incl - c;
                    const uint32_t take = cnt_excl >= room ? 0u : (c < room - cnt_excl ? c : room - cnt_excl);
                    const uint32_t units = static_cast<uint32_t>(p * 16777216.0f);
                    const uint64_t all = static_cast<uint64_t>(take) * units;
                    const uint32_t mine = all > kManyUnits ? kManyUnits : static_cast<uint32_t>(all);
                    const uint32_t sum_incl = wave_scan_u32(mine), sum_excl = sum_incl - mine;
                    const uint32_t reach = units_run + sum_incl;// below 2^32: 2^24 + 64 * 2^25
                    const bool turns = take != 0 && (reach >= thr || reach > kOneUnits);
                    const unsigned long long where = __builtin_amdgcn_ballot_w64(turns);
                    if (where == 0) {// nothing happens in these 64 keys
                        const uint32_t counted = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(cnt_incl), kWave - 1));
                        n += counted < room ? counted : room;
                        units_run += static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(sum_incl), kWave - 1));
                        if (n >= limit_n) done = true;
                        continue;
                    }
                    // The keys before it are taken whole (a key cut short by the entry limit is followed by
                    // keys that take nothing, and those never turn).
                    const int j = __builtin_ctzll(where);
                    n += static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(cnt_excl), j));
                    units_run += static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(sum_excl), j));
                    const uint32_t tj = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(take), j));
                    const uint32_t uj = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(units), j));
                    // entries of this key until the comparison holds: it is made after every addition, so at least one
                    uint64_t need = 1;
                    if (units_run < thr) need = uj == 0 ? ~0ull : (static_cast<uint64_t>(thr) - units_run + uj - 1) / uj;
                    if (need <= tj && units_run + need * uj <= kOneUnits) {
                        units_run += static_cast<uint32_t>(need) * uj;
                        if (lane == 0) {
                            sh.found = 1;
                            sh.entry = n + static_cast<uint32_t>(need) - 1;
                            sh.key = static_cast<uint32_t>(hi - (b0 + j));
                            sh.occurrence = static_cast<uint32_t>(need) - 1;
                        }
                        n += static_cast<uint32_t>(need);
                        done = true;
                        continue;
                    }
                    // the running sum passes 1.0 inside this key: from here on one entry at a time
                    exact = false;
                    run = static_cast<float>(units_run) * (1.0f / 16777216.0f);
                    from = j;
                }
                unsigned long long occupied = __builtin_amdgcn_ballot_w64(c != 0) & (~0ull << from);
                while (occupied != 0 && !done) {
                    const int j = __builtin_ctzll(occupied);
                    occupied &= occupied - 1;
                    const uint32_t cj = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(c), j));
                    const float pj = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, p), j));
                    const uint32_t take = cj < limit_n - n ? cj : limit_n - n;
                    if (__builtin_bit_cast(uint32_t, pj) == 0u) {
                        // adding +0 leaves the sum as it is: the comparison gives for every one of these entries
                        // what it gives for the first
                        if (take != 0 && (MODE == 0 ? run >= threshold : threshold < run)) {
                            if (lane == 0) {
                                sh.found = 1;
                                sh.entry = n;
                                sh.key = static_cast<uint32_t>(hi - (b0 + j));
                                sh.occurrence = 0;
                            }
                            ++n;
                            done = true;
                        } else {
                            n += take;
                        }
                    } else {
                        for (uint32_t i = 0; i < take; ++i) {
                            run += pj;
                            ++n;
                            if (MODE == 0 ? run >= threshold : threshold < run) {
                                if (lane == 0) {
                                    sh.found = 1;
                                    sh.entry = n - 1;
                                    sh.key = static_cast<uint32_t>(hi - (b0 + j));
                                    sh.occurrence = i;
                                }
                                done = true;
                                break;
                            }
                        }
                    }
                    if (n >= limit_n) done = true;
                }
            }
            if (exact) run = static_cast<float>(units_run) * (1.0f / 16777216.0f);
            if (lane == 0) sh.exact = exact ? 1u : 0u;
            if (lane == 0) {
                sh.run = run;
                sh.n = n;
                sh.done = done ? 1u : 0u;
            }
        }
        __syncthreads();
    }
}

// The softmax denominator is formed part by part: the logits are cut into
// `groups` parts of 2048 * vecs, each part's sum is taken relative to the
// part's own largest logit by 256 lanes (sequentially per lane, then the
// wavefront tree, then the four wavefronts in order), and the parts are
// rescaled to the overall maximum and added in a fixed order.  The split form
// gives every part to a workgroup of its own in an earlier launch; one
// workgroup alone takes four parts at a time, 256 lanes each - the same
// arithmetic in the same order, so both forms get the same denominator, to
// the bit, and with it the same probabilities and the same draw.
template<typename T, bool VEC>
__device__ __forceinline__ void part_max_and_sum(const uint16_t *probs, uint32_t voc, uint32_t start, uint32_t vecs, float temperature,
                                                 bool active, uint32_t t, uint32_t *key_slots, float *sum_slots,
                                                 uint32_t &key_max, float &sum) {
    constexpr uint32_t PL = kRandomSamplePartLanes;
    const uint32_t lane = t & (kWave - 1), w = t / kWave;
    uint32_t km = 0;
    if (active) {
        for (uint32_t v = 0; v < vecs; ++v) {
            const uint32_t base = start + (v * PL + t) * 8u;
            if (base < voc) {
                uint32_t h[8];
                const int n = load_codes<VEC>(probs, voc, base, h);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    if (e < n) {
                        const uint32_t k = key_of<T>(h[e]);
                        km = k > km ? k : km;
                    }
                }
            }
        }
        km = wave_max_u32(km);
        if (lane == 0) key_slots[w] = km;
    }
    __syncthreads();
    float part = 0.0f;
    if (active) {
#pragma unroll
        for (uint32_t i = 0; i < PL / kWave; ++i) km = key_slots[i] > km ? key_slots[i] : km;
        const float top = value_of_key<T>(km);
        for (uint32_t v = 0; v < vecs; ++v) {
            const uint32_t base = start + (v * PL + t) * 8u;
            if (base < voc) {
                uint32_t h[8];
                const int n = load_codes<VEC>(probs, voc, base, h);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    if (e < n) part += expf((T::one(static_cast<uint16_t>(h[e])) - top) / temperature);
                }
            }
        }
        part = wave_sum(part);
        if (lane == 0) sum_slots[w] = part;
    }
    __syncthreads();
    key_max = km;
    sum = 0.0f;
    if (active) {
#pragma unroll
        for (uint32_t i = 0; i < PL / kWave; ++i) sum += sum_slots[i];
    }
}

// First launches of the split form: clear the counts, then one workgroup per
// part of the logits leaves its part's maximum and sum while further
// workgroups count every key.
__global__ __launch_bounds__(256) void random_sample_clear(u32x4 *counts) {
    counts[blockIdx.x * 256u + threadIdx.x] = u32x4{0, 0, 0, 0};
}

template<typename T, bool VEC>
__global__ __launch_bounds__(kRandomSamplePartLanes) void random_sample_count(RandomSamplePart *heads, uint32_t *counts, const uint16_t *probs,
                                                                                uint32_t voc, uint32_t groups, uint32_t vecs, float temperature) {
    AMD_ARGS_NOW(heads, counts, probs, voc, groups, vecs, temperature);
    __shared__ uint32_t key_slots[kRandomSamplePartLanes / kWave];
    __shared__ float sum_slots[kRandomSamplePartLanes / kWave];
    if (blockIdx.x >= groups) {
        // The workgroups behind the first `groups` only count: one vector of eight logits per lane, one atomic add
        // per logit.  It is the atomic adds that this launch waits for: 151 936 of them take 13 us however they are
        // spread (the sums alone: 4.8 us; counting inside the summing workgroups: 19.2 us in all; like this: 17.7).
        const uint32_t base = ((blockIdx.x - groups) * kRandomSamplePartLanes + threadIdx.x) * 8u;
        if (base < voc) {
            uint32_t h[8];
            const int n = load_codes<VEC>(probs, voc, base, h);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                if (e < n) atomicAdd(&counts[key_of<T>(h[e])], 1u);
            }
        }
        return;
    }
    uint32_t key_max;
    float sum;
    part_max_and_sum<T, VEC>(probs, voc, blockIdx.x * (kRandomSamplePartLanes * 8u * vecs), vecs, temperature, true, threadIdx.x,
                             key_slots, sum_slots, key_max, sum);
    if (threadIdx.x == 0) heads[blockIdx.x] = RandomSamplePart{0, key_max, sum, 0};
}

// SPLIT: the parts' maxima and sums come from `heads` and the counts of all
// keys from `counts`, both left by the launches above; otherwise this
// workgroup works them out itself (counts: a range of keys at a time, in LDS).
template<typename T, bool VEC, bool SPLIT>
__global__ __launch_bounds__(BS) void random_sample_wide(uint64_t *result, const uint16_t *probs, uint32_t voc,
                                                          float random_val, float topp, uint32_t topk, float temperature,
                                                          const RandomSamplePart *heads, const uint32_t *counts, uint32_t groups, uint32_t vecs) {
    AMD_ARGS_NOW(result, probs, voc, random_val, topp, topk, temperature, heads, counts, groups, vecs);
    __shared__ WideShared sh;
    __shared__ uint32_t key_slots[BS / kWave];
    __shared__ float sum_slots4[BS / kWave];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    if (tid == 0) {
        sh.range_top = -1;
        sh.ranges_known = 0;
    }

    if constexpr (SPLIT) {
        if (static_cast<uint32_t>(tid) < groups) {
            sh.part_key[tid] = heads[tid].key_max;
            sh.part_sum[tid] = heads[tid].sum;
        }
    } else {
        constexpr uint32_t PL = kRandomSamplePartLanes, SIDE = BS / PL;// parts taken side by side
        const uint32_t side = tid / PL, t = tid % PL;
        for (uint32_t g0 = 0; g0 < groups; g0 += SIDE) {
            const uint32_t g = g0 + side;
            uint32_t key_max;
            float sum;
            part_max_and_sum<T, VEC>(probs, voc, g * (PL * 8u * vecs), vecs, temperature, g < groups, t,
                                     key_slots + side * (PL / kWave), sum_slots4 + side * (PL / kWave), key_max, sum);
            if (g < groups && t == 0) {
                sh.part_key[g] = key_max;
                sh.part_sum[g] = sum;
            }
        }
    }
    __syncthreads();
    // the overall maximum and the denominator rescaled to it, in a fixed order (groups <= 48: one wavefront's work)
    uint32_t key_max = 0;
    for (uint32_t g = 0; g < groups; ++g) key_max = sh.part_key[g] > key_max ? sh.part_key[g] : key_max;
    const float top = value_of_key<T>(key_max);
    if (tid < kWave) {
        float part = 0.0f;
        if (static_cast<uint32_t>(tid) < groups) part = sh.part_sum[tid] * expf((value_of_key<T>(sh.part_key[tid]) - top) / temperature);
        part = wave_sum(part);
        if (tid == 0) sh.sum_slots[0] = part;
    }
    __syncthreads();
    const float total = sh.sum_slots[0];
    const uint32_t *const from = SPLIT ? counts : nullptr;

    // walk 1 (random_sample.cc:97-109): where the running sum reaches topp
    wide_walk<T, VEC, 0>(sh, probs, voc, from, key_max, top, total, temperature, topp, topk);
    const uint32_t stop = sh.found != 0 ? sh.entry : topk;// rank of the entry that reached topp
    const float kept = sh.run;                             // the sum up to and including it, or over all topk entries
    const uint32_t end = stop + 1 < topk ? stop + 1 : topk;
    __syncthreads();
    // walk 2 (random_sample.cc:112-125): the first of those `end` entries whose running sum exceeds random_val * kept
    wide_walk<T, VEC, 1>(sh, probs, voc, from, key_max, top, total, temperature, random_val * kept, end);
    if (sh.found == 0) return;// nothing exceeds it (random_val >= 1): the result stays as it is, as in the reference
    const uint32_t key = sh.key, occurrence = sh.occurrence;

    // Occurrence `occurrence` of `key` in index order.  Every wavefront takes one contiguous sixteenth of the
    // logits, 64 neighbouring vectors at a time, and counts the key in it; the wavefront whose part holds the
    // occurrence goes through its part once more, in order, and the lane that holds it writes the index.
    const uint32_t part_len = ((voc + WAVES - 1) / WAVES + 7u) & ~7u;// logits per wavefront, a multiple of 8
    const uint32_t first = static_cast<uint32_t>(wave) * part_len < voc ? static_cast<uint32_t>(wave) * part_len : voc;
    const uint32_t last = first + part_len < voc ? first + part_len : voc;
    uint32_t mine = 0;
    sweep_logits<VEC, 8>(probs, first, last, lane, kWave, [&](uint32_t, const uint32_t(&h)[8], int n) {
#pragma unroll
        for (int e = 0; e < 8; ++e) mine += (e < n && key_of<T>(h[e]) == key) ? 1u : 0u;
    });
    mine = wave_sum_u32(mine);
    if (lane == 0) sh.wave_tot[wave] = mine;
    __syncthreads();
    uint32_t before = 0;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) before += w < wave ? sh.wave_tot[w] : 0u;
    if (occurrence < before || occurrence >= before + mine) return;// uniform over the wavefront
    // in index order, 64 neighbouring vectors at a time; the loads of eight such rounds are issued together
    constexpr int U = 8;
    const uint32_t whole = first + (last - first) / 8u * 8u;// end of this part's whole vectors
    uint32_t seen = before;
    for (uint32_t base0 = first; base0 < whole; base0 += kWave * 8u * U) {
        u32x4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t base = base0 + (static_cast<uint32_t>(u) * kWave + lane) * 8u;
            const uint32_t at = base < whole ? base : first;// past the end: any vector of the part, dropped below
            if constexpr (VEC) {
                v[u] = ld16(probs + at);
            } else {
                v[u] = u32x4{probs[at] | (static_cast<uint32_t>(probs[at + 1]) << 16), probs[at + 2] | (static_cast<uint32_t>(probs[at + 3]) << 16),
                             probs[at + 4] | (static_cast<uint32_t>(probs[at + 5]) << 16), probs[at + 6] | (static_cast<uint32_t>(probs[at + 7]) << 16)};
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t base = base0 + (static_cast<uint32_t>(u) * kWave + lane) * 8u;
            const uint32_t h[8] = {v[u].x & 0xFFFFu, v[u].x >> 16, v[u].y & 0xFFFFu, v[u].y >> 16,
                                   v[u].z & 0xFFFFu, v[u].z >> 16, v[u].w & 0xFFFFu, v[u].w >> 16};
            uint32_t hits = 0;
#pragma unroll
            for (int e = 0; e < 8; ++e) hits += (base < whole && key_of<T>(h[e]) == key) ? 1u : 0u;
            const uint32_t upto = wave_scan_u32(hits);
            const uint32_t here = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(upto), kWave - 1));
            if (occurrence < seen + here) {// uniform: it is in this round
                uint32_t at = seen + upto - hits;// matches before this lane's vector
                if (occurrence >= at && occurrence < at + hits) {
                    for (int e = 0; e < 8; ++e) {
                        if (key_of<T>(h[e]) == key) {
                            if (at == occurrence) result[0] = base + e;
                            ++at;
                        }
                    }
                }
                return;
            }
            seen += here;
        }
    }
    // what is left is the vector that holds the end of the logits
    if (lane == 0) {
        for (uint32_t i = whole; i < last; ++i) {
            if (key_of<T>(probs[i]) == key) {
                if (seen == occurrence) {
                    result[0] = i;
                    return;
                }
                ++seen;
            }
        }
    }
}

// ---- the same in two launches, the first spread over the chip ---------------
// First launch: workgroup w of 256 lanes takes the logits
// [w * 2048 * vecs, (w + 1) * 2048 * vecs) and leaves in the workspace
//   * every element that can belong to the overall topk.  The topk-th largest
//     of the 256 lane maxima is a lower bound of the workgroup's own topk-th
//     largest element, and an element of the overall topk is among the topk
//     largest of its workgroup, so elements below that bound are dropped
//     without a sort: with topk = 50 about 55 of 2048 remain;
//   * its maximum and its sum of expf((x - maximum) / temperature), which the
//     second launch rescales to the overall maximum.
// Second launch: one workgroup selects the topk-th key among the survivors
// (radix select in LDS), ranks what is left and draws.  Whenever a list
// overflows - very many equal logits, topk close to 256 - it does the whole
// job itself from the logits (topk_full), so the answer never depends on the
// shortcut working.
template<typename T, bool VEC>
__global__ __launch_bounds__(kRandomSamplePartLanes) void random_sample_partial(RandomSamplePart *heads, unsigned long long *lists,
                                                                                  const uint16_t *probs, uint32_t voc,
                                                                                  uint32_t vecs, uint32_t topk, float temperature) {
    AMD_ARGS_NOW(heads, lists, probs, voc, vecs, topk, temperature);
    constexpr int PBS = kRandomSamplePartLanes, PW = PBS / kWave;
    __shared__ __attribute__((aligned(16))) uint32_t lane_rank_key[PBS];
    __shared__ uint32_t bound_slot, max_slot, data_lanes;
    __shared__ float sum_slots[PW];
    __shared__ uint32_t fill;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    const uint32_t start = blockIdx.x * (PBS * 8u * vecs);

    // lane maxima
    uint32_t lane_max = 0;
    bool has = false;
    for (uint32_t v = 0; v < vecs; ++v) {
        const uint32_t base = start + (v * PBS + tid) * 8u;
        if (base < voc) {
            uint32_t h[8];
            const int n = load_codes<VEC>(probs, voc, base, h);
            has = true;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t k = key_of<T>(h[e]);
                if (e < n) lane_max = k > lane_max ? k : lane_max;
            }
        }
    }
    // The topk-th largest lane maximum, by rank: every lane reads all 256
    // (one LDS round trip, 64 four-word reads) and counts those that beat its
    // own; the lane number breaks ties so the ranks are a permutation, and the
    // lane of rank topk - 1 holds the bound.  Lanes without data rank last;
    // with fewer than topk lanes holding data everything is kept.  (A
    // four-pass radix select over the 256 values, two barriers a pass, took
    // 3.9 us of this kernel's 7.5.)
    const uint32_t my_rank_key = has ? ((lane_max << 8) | (255u - static_cast<uint32_t>(tid))) + 1u : 0u;
    lane_rank_key[tid] = my_rank_key;
    if (tid == 0) {
        fill = 0;
        bound_slot = 0;
        data_lanes = PBS;
    }
    __syncthreads();
    uint32_t rank = 0;
    {
        const u32x4 *all = reinterpret_cast<const u32x4 *>(lane_rank_key);
#pragma unroll 8
        for (int j = 0; j < PBS / 4; ++j) {
            const u32x4 q = all[j];
            rank += (q.x > my_rank_key ? 1u : 0u) + (q.y > my_rank_key ? 1u : 0u) + (q.z > my_rank_key ? 1u : 0u) + (q.w > my_rank_key ? 1u : 0u);
        }
    }
    // what the ranks say besides the bound: rank 0 holds the workgroup's
    // maximum, and a lane without data is beaten by exactly the lanes with data
    if (has && rank == 0) max_slot = lane_max;
    if (!has) data_lanes = rank;// every such lane writes the same number
    if (has && rank == topk - 1) bound_slot = lane_max;
    __syncthreads();
    const bool keep_all = data_lanes < topk;// uniform over the workgroup
    const uint32_t bound = keep_all ? 0u : bound_slot;
    const uint32_t key_max = max_slot;
    const float top = value_of_key<T>(key_max);

    // survivors to the workspace, and the partial denominator
    float part = 0.0f;
    unsigned long long *list = lists + static_cast<size_t>(blockIdx.x) * kRandomSamplePartCap;
    for (uint32_t v = 0; v < vecs; ++v) {
        const uint32_t base = start + (v * PBS + tid) * 8u;
        uint32_t h[8], k[8];
        int n = 0;
        uint32_t c = 0;
        if (base < voc) {
            n = load_codes<VEC>(probs, voc, base, h);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                k[e] = e < n ? key_of<T>(h[e]) : kNoKey;
                if (e < n) {
                    const float x = T::one(static_cast<uint16_t>(h[e]));
                    // the maximum itself counts as expf(0) also when it is infinite
                    part += k[e] == key_max ? 1.0f : expf((x - top) / temperature);
                    c += k[e] >= bound ? 1u : 0u;
                }
            }
        }
        const uint32_t inc = wave_scan_u32(c);
        uint32_t at = 0;
        if (lane == kWave - 1 && inc != 0) at = atomicAdd(&fill, inc);
        at = __shfl(at, kWave - 1) + inc - c;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if (e < n && k[e] >= bound) {
                if (at < static_cast<uint32_t>(kRandomSamplePartCap)) {
                    list[at] = (static_cast<unsigned long long>(k[e]) << 32) | (0xFFFFFFFFu - (base + e));
                }
                ++at;
            }
        }
    }
    part = wave_sum(part);
    if (lane == 0) sum_slots[wave] = part;
    __syncthreads();
    if (tid == 0) {
        float total = 0.0f;
#pragma unroll
        for (int w = 0; w < PW; ++w) total += sum_slots[w];
        RandomSamplePart head;
        head.count = fill;
        head.key_max = key_max;
        head.sum = total;
        head.unused = 0;
        heads[blockIdx.x] = head;
    }
}

template<typename T, bool VEC>
__global__ __launch_bounds__(BS) void random_sample_merge(uint64_t *result, const uint16_t *probs, uint32_t voc, float random_val,
                                                           float topp, uint32_t topk, float temperature,
                                                           const RandomSamplePart *heads, const unsigned long long *lists,
                                                           uint32_t groups) {
    AMD_ARGS_NOW(result, probs, voc, random_val, topp, topk, temperature, heads, lists, groups);
    constexpr int CMAX = 4096, PER_LANE = CMAX / BS;
    __shared__ TopkShared sh;
    __shared__ unsigned long long pool[CMAX];
    __shared__ uint32_t offs[kRandomSampleMaxGroups + 1];
    __shared__ uint32_t g_key[kRandomSampleMaxGroups];
    __shared__ float g_sum[kRandomSampleMaxGroups];
    __shared__ uint32_t verdict[2];// [0]: lists usable, [1]: fill of sh.cand
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;

    // groups <= 48: the headers are one wavefront's work
    if (tid < kWave) {
        RandomSamplePart head{0, 0, 0.0f, 0};
        if (static_cast<uint32_t>(tid) < groups) head = heads[tid];
        const uint32_t upto = wave_scan_u32(head.count);
        const bool fits = __builtin_amdgcn_ballot_w64(head.count > static_cast<uint32_t>(kRandomSamplePartCap)) == 0;
        if (static_cast<uint32_t>(tid) < groups) {
            offs[tid + 1] = upto;
            g_key[tid] = head.key_max;
            g_sum[tid] = head.sum;
        }
        const uint32_t all = __shfl(upto, kWave - 1);
        if (tid == 0) {
            offs[0] = 0;
            verdict[0] = (fits && all <= static_cast<uint32_t>(CMAX) && all >= topk) ? 1u : 0u;
            verdict[1] = 0;
        }
    }
    __syncthreads();
    if (verdict[0] == 0) {// uniform over the workgroup
        topk_full<T, VEC>(sh, result, probs, voc, random_val, topp, topk, temperature);
        return;
    }
    const uint32_t count = offs[groups];

    // the overall maximum and the denominator rescaled to it, in a fixed order
    uint32_t key_max = 0;
    for (uint32_t w = 0; w < groups; ++w) key_max = g_key[w] > key_max ? g_key[w] : key_max;
    const float top = value_of_key<T>(key_max);
    float part = 0.0f;
    if (static_cast<uint32_t>(tid) < groups) {
        part = g_sum[tid] * expf((value_of_key<T>(g_key[tid]) - top) / temperature);
    }
    part = wave_sum(part);// groups <= 64: all of them sit in the first wavefront
    if (tid == 0) sh.sum_slots[0] = part;

    // the survivors into LDS
    for (uint32_t w = wave; w < groups; w += WAVES) {
        const uint32_t from = offs[w], n = offs[w + 1] - from;
        for (uint32_t j = lane; j < n; j += kWave) pool[from + j] = lists[static_cast<size_t>(w) * kRandomSamplePartCap + j];
    }
    __syncthreads();
    const float total = sh.sum_slots[0];

    // radix select of the topk-th key among them
    uint32_t keys[PER_LANE];
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i) {
        const uint32_t at = tid + i * BS;
        keys[i] = at < count ? static_cast<uint32_t>(pool[at] >> 32) : kNoKey;
    }
    uint32_t prefix = 0, want = topk, ties = 0;
#pragma unroll 1
    for (int shift = 12; shift >= 0; shift -= 4) {
        // Counting: a lane's entry becomes a one in an 8-bit field - digit d in
        // field d & 3 of word d >> 2 - and four DPP wave sums add the fields of
        // all 64 lanes at once (a field holds at most 64); lane d then picks
        // its field.  A wavefront skips the slots in which none of its entries
        // shares the prefix any more (with a few hundred survivors most
        // wavefronts hold one live slot or none).  One ballot and population
        // count per digit and slot, the first form, took 1.5 us a pass.
        uint32_t mine = 0;
#pragma unroll
        for (int i = 0; i < PER_LANE; ++i) {
            const bool in = (keys[i] >> (shift + 4)) == prefix;
            if (__builtin_amdgcn_ballot_w64(in) == 0) continue;
            const uint32_t digit = (keys[i] >> shift) & 15u;
            const uint32_t one = in ? 1u << (8u * (digit & 3u)) : 0u;
            const uint32_t word = digit >> 2;
            const uint32_t s0 = wave_sum_u32(word == 0 ? one : 0u), s1 = wave_sum_u32(word == 1 ? one : 0u);
            const uint32_t s2 = wave_sum_u32(word == 2 ? one : 0u), s3 = wave_sum_u32(word == 3 ? one : 0u);
            const uint32_t lw = static_cast<uint32_t>(lane) >> 2;
            const uint32_t sel = lw == 0 ? s0 : lw == 1 ? s1 : lw == 2 ? s2 : s3;
            mine += (sel >> (8u * (static_cast<uint32_t>(lane) & 3u))) & 0xFFu;// lanes past 15 hold nothing of use
        }
        // one barrier a pass: every wavefront totals the columns itself (lane d
        // the column of digit d) and walks them through lane reads; the two
        // sets of counters take turns, so a wavefront that is a pass ahead
        // never overwrites what a slower one still reads
        uint32_t *set = sh.wave_cnt[(shift >> 2) & 1];
        if (lane < 16) set[wave * 16 + lane] = mine;
        __syncthreads();
        uint32_t column = 0;
        if (lane < 16) {
#pragma unroll
            for (int w = 0; w < WAVES; ++w) column += set[w * 16 + lane];
        }
        uint32_t above = 0, chosen = 0, chosen_count = 0;
        bool found = false;
#pragma unroll
        for (int d = 15; d >= 0; --d) {
            const uint32_t c = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(column), d));
            if (!found) {
                if (above + c >= want) {
                    chosen = d;
                    chosen_count = c;
                    found = true;
                } else {
                    above += c;
                }
            }
        }
        want -= above;
        prefix = (prefix << 4) | chosen;
        if (shift == 0) ties = chosen_count;
    }
    // everything above the topk-th key plus every entry equal to it
    const uint32_t kept = topk - want + ties;
    if (kept > static_cast<uint32_t>(KMAX)) {// uniform: more equal logits at the boundary than LDS ranks
        __syncthreads();
        topk_full<T, VEC>(sh, result, probs, voc, random_val, topp, topk, temperature);
        return;
    }
#pragma unroll
    for (int i = 0; i < PER_LANE; ++i) {
        if (keys[i] != kNoKey && keys[i] >= prefix) sh.cand[atomicAdd(&verdict[1], 1u)] = pool[tid + i * BS];
    }
    __syncthreads();
    rank_and_draw<T>(sh, result, kept, topk, top, total, random_val, topp, temperature);
}

struct RandomSampleCall {
    uint64_t *result;
    const uint16_t *probs;
    uint32_t voc;
    float random_val, topp;
    uint32_t topk;
    float temperature;
    void *workspace;// what a first launch leaves for the drawing workgroup goes here; null: one workgroup does the whole call
    uint32_t groups, vecs;
};

// form 2: sampling, 1: greedy, 0: nothing to launch.  Sampling with up to
// kRandomSamplePartTopk candidates and the workspace ranks them in LDS
// (candidate lists from a first launch); with more candidates it walks the
// histogram of keys (counts from two launches before it); without the
// workspace one workgroup walks the histogram whatever the candidate count -
// measured against the one-workgroup ranking form (topk_full, still what the
// second launch of the list form falls back to), top-k 50, MI355X: 13.9
// against 18.1 us at 512 logits, 29.6 against 57.1 us at 32 000, 94.9 against
// 211.5 us at 151 936.
template<typename T, bool VEC>
void launch_random_sample(const RandomSampleCall &c, int form, hipStream_t s) {
    auto *heads = static_cast<RandomSamplePart *>(c.workspace);
    if (form == 1) {
        random_sample_greedy<T, VEC><<<1, BS, 0, s>>>(c.result, c.probs, c.voc);
    } else if (form == 2 && (c.topk > static_cast<uint32_t>(kRandomSamplePartTopk) || heads == nullptr)) {
        if (heads != nullptr) {
            auto *counts = reinterpret_cast<uint32_t *>(heads + kRandomSampleMaxGroups);
            random_sample_clear<<<kRandomSampleKeys / (256 * 4), 256, 0, s>>>(reinterpret_cast<u32x4 *>(counts));
            const unsigned counting = static_cast<unsigned>(amd::ceil_div(c.voc, kRandomSamplePartLanes * 8u));
            random_sample_count<T, VEC><<<c.groups + counting, kRandomSamplePartLanes, 0, s>>>(heads, counts, c.probs, c.voc, c.groups, c.vecs, c.temperature);
            random_sample_wide<T, VEC, true><<<1, BS, 0, s>>>(c.result, c.probs, c.voc, c.random_val, c.topp, c.topk, c.temperature,
                                                              heads, counts, c.groups, c.vecs);
        } else {
            random_sample_wide<T, VEC, false><<<1, BS, 0, s>>>(c.result, c.probs, c.voc, c.random_val, c.topp, c.topk, c.temperature,
                                                               nullptr, nullptr, c.groups, c.vecs);
        }
    } else if (form == 2) {
        auto *lists = reinterpret_cast<unsigned long long *>(heads + kRandomSampleMaxGroups);
        random_sample_partial<T, VEC><<<c.groups, kRandomSamplePartLanes, 0, s>>>(heads, lists, c.probs, c.voc, c.vecs, c.topk, c.temperature);
        random_sample_merge<T, VEC><<<1, BS, 0, s>>>(c.result, c.probs, c.voc, c.random_val, c.topp, c.topk, c.temperature, heads, lists, c.groups);
    }
}

// ---- the library's own candidate lists ----------------------------------------
// For callers that cannot hand over a workspace they allocated: the two-launch
// form's lists in a fixed array in device memory, one copy per GPU, held until
// the process ends.  Host code never uses the array's name as an address (on
// the host it is only a handle for the symbol): the address on a GPU is asked
// for once, with that GPU current, and kept; a descriptor takes it when it is
// made, so the call path holds no lock and asks the runtime nothing.
constexpr uint64_t kScratchListBytes = kRandomSampleMaxGroups * sizeof(RandomSamplePart) +
                                       static_cast<uint64_t>(kRandomSampleMaxGroups) * kRandomSamplePartCap * sizeof(uint64_t);
constexpr uint64_t kScratchCountBytes = kRandomSampleMaxGroups * sizeof(RandomSamplePart) + static_cast<uint64_t>(kRandomSampleKeys) * sizeof(uint32_t);
constexpr uint64_t kScratchBytes = kScratchListBytes > kScratchCountBytes ? kScratchListBytes : kScratchCountBytes;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxGpus = 64;
std::mutex scratch_lock;
void *scratch_on_gpu[kMaxGpus];// null until asked for

}// namespace

// The address of a GPU's copy: asked for once per GPU, with that GPU current, at the creation of a descriptor.
infiniopStatus_t amdRandomSampleScratch(int device_id, void **address) {
    if (device_id < 0 || device_id >= kMaxGpus) {
        return STATUS_BAD_DEVICE;
    }
    std::lock_guard<std::mutex> guard(scratch_lock);
    if (scratch_on_gpu[device_id] == nullptr) {
        AMD_CHECK_HIP(hipSetDevice(device_id), STATUS_BAD_DEVICE);
        void *ptr = nullptr;
        AMD_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), STATUS_EXECUTION_FAILED);
        if (ptr == nullptr) {
            return STATUS_EXECUTION_FAILED;
        }
        scratch_on_gpu[device_id] = ptr;
    }
    *address = scratch_on_gpu[device_id];
    return STATUS_SUCCESS;
}

// RandomSample without a caller-provided workspace and without any allocation:
// what the first launches leave for the drawing workgroup lives in this
// library's own array on the GPU.  Same results as amdRandomSample with a
// workspace.  Nothing in the array has to be cleared between calls by the host
// (the first launch writes every header and every list entry the last one
// reads; the counts of the histogram form are cleared by a kernel of the call
// itself).  All calls on one GPU
// share the array: two of them in flight at once, on any streams, race.
infiniopStatus_t amdRandomSampleNoAlloc(RandomSampleAmdDescriptor_t desc, void *result, void const *probs, float random_val,
                                        float topp, int topk, float temperature, void *stream) {
    if (result == nullptr || probs == nullptr) {
        return STATUS_BAD_PARAM;
    }
    if (desc->voc > kRandomSampleNoAllocMaxVoc) {
        std::fprintf(stderr, "infiniop[amd-gpu]: RandomSampleNoAlloc serves at most %u logits, the descriptor has %u; "
                             "use infiniopRandomSample with a workspace\n", kRandomSampleNoAllocMaxVoc, desc->voc);
        return STATUS_BAD_PARAM;
    }
    if (amdRandomSampleWorkspaceBytes(*desc) > kScratchBytes) {
        std::fprintf(stderr, "infiniop[amd-gpu]: RandomSampleNoAlloc: the lists of %u logits need %llu bytes, the library holds %llu\n",
                     desc->voc, static_cast<unsigned long long>(amdRandomSampleWorkspaceBytes(*desc)), static_cast<unsigned long long>(kScratchBytes));
        return STATUS_BAD_PARAM;
    }
    if (desc->scratch == nullptr) {// the runtime did not give the array's address when the descriptor was made
        return STATUS_EXECUTION_FAILED;
    }
    return amdRandomSample(desc, desc->scratch, kScratchBytes, result, probs, random_val, topp, topk, temperature, stream);
}

// Stage 4 of RandomSample.  With topp > 0 and topk > 1 it samples, otherwise
// it returns the first index of the maximum, as the reference does
// (random_sample.cc:160-166).  The workspace carries what a first launch
// spread over the chip leaves for the workgroup that draws: candidate lists
// for up to 256 candidates, a count per key for more.  Without it (null, too
// small for the form the call takes, misaligned) and for small vocabularies
// one workgroup does the whole call, with the same result.
infiniopStatus_t amdRandomSample(RandomSampleAmdDescriptor_t desc, void *workspace, uint64_t workspace_size, void *result,
                                 void const *probs, float random_val, float topp, int topk, float temperature, void *stream) {
    if (result == nullptr || probs == nullptr) {
        return STATUS_BAD_PARAM;
    }
    const bool sample = topp > 0 && topk > 1;
    uint32_t k = 0;
    if (sample) {
        k = static_cast<uint32_t>(topk) > desc->voc ? desc->voc : static_cast<uint32_t>(topk);
    }
    AMD_CHECK_HIP(hipSetDevice(desc->device_id), STATUS_BAD_DEVICE);
    hipStream_t s = static_cast<hipStream_t>(stream);
    // what the form this call takes needs of the workspace (16-byte aligned: the counts are cleared 16 bytes at a time)
    const uint64_t needs = k <= static_cast<uint32_t>(kRandomSamplePartTopk) ? amdRandomSampleListBytes(*desc) : amdRandomSampleHistogramBytes(*desc);
    const bool split = sample && k >= 2 && desc->groups != 0 && workspace != nullptr && workspace_size >= needs &&
                       (reinterpret_cast<uintptr_t>(workspace) & 15u) == 0;
    // the parts the denominator is formed in: the first launch's workgroups, or as many of one vector per lane for
    // vocabularies too small to be split
    const uint32_t groups = desc->groups != 0 ? desc->groups : static_cast<uint32_t>(amd::ceil_div(desc->voc, kRandomSamplePartLanes * 8u));
    const uint32_t vecs = desc->groups != 0 ? desc->vecs : 1u;
    const RandomSampleCall call{static_cast<uint64_t *>(result), static_cast<const uint16_t *>(probs), desc->voc, random_val, topp, k,
                                temperature, split ? workspace : nullptr, groups, vecs};
    // greedy unless sampling; a vocabulary of one logit has one candidate of
    // probability 1, which wins unless random_val >= 1, as in the reference's loops
    const int form = (sample && k >= 2) ? 2 : (!sample || random_val < 1.0f) ? 1 : 0;
    const bool vec = amd::aligned16(probs);
    if (desc->elem == amd::Elem::F16) {
        if (vec) launch_random_sample<amd::F16Ref, true>(call, form, s);
        else launch_random_sample<amd::F16Ref, false>(call, form, s);
    } else {
        if (vec) launch_random_sample<amd::BF16Rne, true>(call, form, s);
        else launch_random_sample<amd::BF16Rne, false>(call, form, s);
    }
    AMD_CHECK_HIP(hipGetLastError(), STATUS_EXECUTION_FAILED);
    return STATUS_SUCCESS;
}
