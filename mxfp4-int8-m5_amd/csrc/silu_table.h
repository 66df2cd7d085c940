// silu(g) = bf16(g * sigmoid(g)) for every bf16 gate value g, with each step rounded to bf16 exactly as the
// SwiGLU epilogue computes it (e = bf16(exp|g|), y = bf16(1 / bf16(1 + e)), sigmoid = g < 0 ? y : bf16(1 - y)).
// The gate has only 65536 possible values, so the epilogue's ~60 instructions per output become one 2-byte load;
// the table is evaluated by the compiler from the functions below (plain IEEE single-precision operations, the same
// sequence as swiglu_bf16 / exp_pos in scmx_common.h), so it cannot drift from them.
#pragma once
#include <cstdint>

namespace scmx {
namespace silu_ce {

constexpr float from_bits(uint32_t u) { return __builtin_bit_cast(float, u); }
constexpr uint32_t to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }
constexpr uint16_t to_bf16(float f) {   // round to nearest even; NaN stays NaN
    uint32_t u = to_bits(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return uint16_t((u >> 16) | 0x40u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return uint16_t(u >> 16);
}
constexpr float round_bf16(float f) { return from_bits(uint32_t(to_bf16(f)) << 16); }
constexpr float rint_pos(float x) {   // round half to even for 0 <= x < 2^23
    int i = int(x);
    const float fr = x - float(i);
    if (fr > 0.5f || (fr == 0.5f && (i & 1))) ++i;
    return float(i);
}
constexpr float exp_pos(float a) {
    a = (a < 89.0f) ? a : 89.0f;
    const float n = rint_pos(a * 1.4426950408889634f);
    const float r = (a - n * 0.693145751953125f) - n * 1.428606765330187e-06f;
    float p = 1.0f / 5040.0f;
    p = p * r + 1.0f / 720.0f;
    p = p * r + 1.0f / 120.0f;
    p = p * r + 1.0f / 24.0f;
    p = p * r + 1.0f / 6.0f;
    p = p * r + 0.5f;
    p = p * r + 1.0f;
    p = p * r + 1.0f;
    const int ni = int(n), h = ni >> 1;
    return (p * from_bits(uint32_t(h + 127) << 23)) * from_bits(uint32_t(ni - h + 127) << 23);
}
constexpr uint16_t silu_bits(uint16_t gb) {
    const float g = from_bits(uint32_t(gb) << 16);
    if ((gb & 0x7FFFu) > 0x7F80u) return gb | 0x40u;   // NaN gate
    const float e = round_bf16(exp_pos(g < 0.0f ? -g : g));
    const float y = round_bf16(1.0f / round_bf16(1.0f + e));
    const float sig = (g < 0.0f) ? y : round_bf16(1.0f - y);
    return to_bf16(g * sig);
}

struct Table {
    uint16_t v[65536];
};
constexpr Table make() {
    Table t{};
    for (uint32_t i = 0; i < 65536; ++i) t.v[i] = silu_bits(uint16_t(i));
    return t;
}

}  // namespace silu_ce
}  // namespace scmx
