// Fixed-point accumulator words of the atomic split reductions. No HIP types: the
// functions are constexpr (host and device in HIP, plain C++ elsewhere), so the same
// header is unit-tested in a host build.
#pragma once

namespace exl3 {

// Accumulator word of the atomic split reductions: count << 56 | sum, the count an
// unsigned 8-bit number (up to 255 contributors), the sum a signed fixed-point number
// with 20 fraction bits. A partial sum is clamped to +-2^18 (fp16 ends at 65504, so a
// clamped total still rounds to infinity, as the unclamped one would); a partial sum
// that is not finite contributes 2^47 instead, more than 255 clamped partial sums can
// add up to (255 * 2^38 < 2^46), so the total is recognised and becomes NaN: a
// non-finite input gives a non-finite output, as in the partial-row reduction.
constexpr float kFixScale = 1048576.f;  // 2^20
constexpr float kFixClamp = 262144.f;   // 2^18
constexpr long long kFixPoison = 1ll << 47;
constexpr long long kFixPoisonFrom = 1ll << 46;

constexpr unsigned long long fix_word(float v) {
    long long fixed = kFixPoison;
    if (v - v == 0.f) {  // finite (NaN and the infinities keep the poison value)
        v = v < -kFixClamp ? -kFixClamp : (v > kFixClamp ? kFixClamp : v);
        fixed = (long long)((double)v * (double)kFixScale);
    }
    return (1ull << 56) + (unsigned long long)fixed;
}
constexpr int fix_count(unsigned long long w) {
    return (int)((w + (1ull << 55)) >> 56);
}
constexpr float fix_value(unsigned long long w) {
    const unsigned long long c = (w + (1ull << 55)) >> 56;
    const long long fixed = (long long)(w - (c << 56));
    if (fixed >= kFixPoisonFrom) return __builtin_nanf("");
    return (float)((double)fixed * (1.0 / (double)kFixScale));
}

}  // namespace exl3
