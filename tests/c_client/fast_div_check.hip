// Host-side check of the multiply-and-shift division the kernels use for
// divisors the host knows (FastDiv in devices/amd/kernel_amd.h): the quotient
// must equal n / d for every divisor and operand below 2^31.  Compiled with
// hipcc and run on the CPU by tests/test_fast_div.py; prints "ok <count>".
#include "devices/amd/kernel_amd.h"
#include <cstdio>
#include <cstdint>

static uint64_t state = 0x9E3779B97F4A7C15ull;
static uint32_t next31() {// xorshift64*, top bits
    state ^= state >> 12;
    state ^= state << 25;
    state ^= state >> 27;
    return static_cast<uint32_t>((state * 0x2545F4914F6CDD1Dull) >> 33);
}

int main() {
    const uint32_t limit = static_cast<uint32_t>(amd::kFastDivLimit - 1);// largest operand and divisor
    uint64_t checked = 0;
    auto check = [&](uint32_t d) {
        const amd::FastDiv f = amd::fast_div(d);
        const uint32_t edge[] = {0, 1, d - 1, d, d + 1 <= limit ? d + 1 : d, limit, limit - 1, limit / d * d, limit / d * d ? limit / d * d - 1 : 0};
        for (uint32_t n : edge) {
            if (n <= limit && amd::fast_quotient(n, f) != n / d) { printf("wrong: %u / %u\n", n, d); return false; }
        }
        for (int i = 0; i < 64; ++i) {
            const uint32_t n = next31();
            if (amd::fast_quotient(n, f) != n / d) { printf("wrong: %u / %u\n", n, d); return false; }
        }
        checked += 73;
        return true;
    };
    for (uint32_t d = 1; d <= 70000; ++d) if (!check(d)) return 1;               // every small divisor: row lengths, head counts, sequence lengths
    for (int s = 0; s < 31; ++s) for (int o = -2; o <= 2; ++o) {                   // around the powers of two
        const int64_t d = (int64_t(1) << s) + o;
        if (d >= 1 && d <= limit && !check(static_cast<uint32_t>(d))) return 1;
    }
    for (int i = 0; i < 200000; ++i) { const uint32_t d = next31(); if (d >= 1 && !check(d)) return 1; }  // anything
    if (!check(limit)) return 1;
    // one small divisor against every operand in a range that crosses many multiples
    const amd::FastDiv f7 = amd::fast_div(7), f80 = amd::fast_div(80);
    for (uint32_t n = limit - 3000000; n <= limit && n >= limit - 3000000; ++n) {
        if (amd::fast_quotient(n, f7) != n / 7 || amd::fast_quotient(n, f80) != n / 80) { printf("wrong at %u\n", n); return 1; }
        if (n == limit) break;
    }
    printf("ok %llu\n", static_cast<unsigned long long>(checked));
    return 0;
}
