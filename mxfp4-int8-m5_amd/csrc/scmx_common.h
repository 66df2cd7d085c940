// Device-side helpers shared by the SC-MXFP4 W4A8 kernels (gfx950 / CDNA4, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/scmx.h"

namespace scmx {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int WAVE = 64;

// ---- weight format as the kernels see it -----------------------------------------------------------------------
// lut_lo / lut_hi: the 8 code magnitudes as bytes (index 0..3 / 4..7); mult[]: up to 16 multipliers as bytes.
// pow2 = 1 when mult[i] == 1 << i, so the multiplier is a shift.
struct DevFormat {
    uint32_t lut_lo, lut_hi;
    uint32_t mult[4];
    int32_t block;      // weights per block along K
    int32_t block_log2;
    int32_t bc_bits;    // 1, 2, 4 or 8
    int32_t pow2;
    int32_t e8m0;       // 1: the block-code bytes are E8M0 exponents of a standard MXFP4 tensor (block 32, bc_bits 8)
};

// Host: validate a caller's format and build the device view.  Returns 0 or SCMX_ERR_FORMAT.
int make_dev_format(const scmx_format* f, DevFormat* out);
inline bool is_default_format(const DevFormat& d) {
    return d.lut_lo == 0x03020100u && d.lut_hi == 0x0C080604u && d.block == 32 && d.bc_bits == 2 && d.pow2;
}
// The same codebook and power-of-two shifts on 16-element blocks (one 2-bit code per two code words).
inline bool is_pow2_block16_format(const DevFormat& d) {
    return d.lut_lo == 0x03020100u && d.lut_hi == 0x0C080604u && d.block == 16 && d.bc_bits == 2 && d.pow2;
}

// The same codebook on 16-element blocks with 4-bit block codes whose multipliers are consecutive integers
// (mult[i] = mult[0] + i, unused entries 0): the "B16/M<lo>..<hi>" members of the family.  A block's multiplier is then
// its code plus mult[0], no table needed.
inline bool is_block16_range_format(const DevFormat& d) {
    if (!(d.lut_lo == 0x03020100u && d.lut_hi == 0x0C080604u && d.block == 16 && d.bc_bits == 4) || d.pow2) return false;
    const uint32_t m0 = d.mult[0] & 0xFFu;
    bool ended = false;
    for (uint32_t i = 0; i < 16; ++i) {
        const uint32_t m = (d.mult[i >> 2] >> (8 * (i & 3))) & 0xFFu;
        if (m == 0) ended = true;
        else if (ended || m != m0 + i) return false;
    }
    return m0 >= 1;
}

// Standard MXFP4 read in place: one E8M0 byte per 32-block instead of a block code.  A row's lowest exponent is
// carried by its scale, wscale = 2^(lowest - 128), so the block's shift is byte - (exponent field of wscale + 1).
inline bool is_mxfp4_e8m0_format(const DevFormat& d) { return d.e8m0 != 0; }

// Compute units of the current device (queried once per device).
int device_cus();

// Thread-local error text behind scmx_last_error().
void set_error(const char* fmt, ...);
int check_launch(const char* what);

// ---- bf16 ------------------------------------------------------------------------------------------------------
__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float(uint32_t(b) << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {   // round to nearest even; NaN stays NaN
    __bf16 h = (__bf16)f;
    return __builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ float round_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }

// ---- deterministic FP32 exp for a >= 0: IEEE multiply / add / rint only (no FMA contraction) ------------------
__device__ __forceinline__ float exp_pos(float a) {
    a = (a < 89.0f) ? a : 89.0f;
    const float n = rintf(__fmul_rn(a, 1.4426950408889634f));
    const float r = __fsub_rn(__fsub_rn(a, __fmul_rn(n, 0.693145751953125f)), __fmul_rn(n, 1.428606765330187e-06f));
    float p = 1.0f / 5040.0f;
    p = __fadd_rn(__fmul_rn(p, r), 1.0f / 720.0f);
    p = __fadd_rn(__fmul_rn(p, r), 1.0f / 120.0f);
    p = __fadd_rn(__fmul_rn(p, r), 1.0f / 24.0f);
    p = __fadd_rn(__fmul_rn(p, r), 1.0f / 6.0f);
    p = __fadd_rn(__fmul_rn(p, r), 0.5f);
    p = __fadd_rn(__fmul_rn(p, r), 1.0f);
    p = __fadd_rn(__fmul_rn(p, r), 1.0f);
    const int ni = (int)n, h = ni >> 1;
    const float s1 = __uint_as_float(uint32_t(h + 127) << 23);
    const float s2 = __uint_as_float(uint32_t(ni - h + 127) << 23);
    return __fmul_rn(__fmul_rn(p, s1), s2);
}

// SwiGLU on bf16 values with every operation rounded to bf16 (gate g, up u given as FP32 holding bf16 values).
__device__ __forceinline__ uint16_t swiglu_bf16(float g, float u) {
    const float e = round_bf16(exp_pos(fabsf(g)));
    const float y = round_bf16(__fdiv_rn(1.0f, round_bf16(__fadd_rn(1.0f, e))));
    const float sig = (g < 0.0f) ? y : round_bf16(__fsub_rn(1.0f, y));
    const float silu = round_bf16(__fmul_rn(g, sig));
    return f32_to_bf16(__fmul_rn(silu, u));
}

// Device address (current device) of the 65536-entry table silu[g] = bf16(g * sigmoid(g)) over bf16 gate bit patterns,
// built at compile time from the same operation sequence as swiglu_bf16; NULL if the symbol cannot be resolved.
const uint16_t* silu_table_device();
__device__ __forceinline__ uint16_t swiglu_lut(const uint16_t* __restrict__ table, float g, float u) {
    return f32_to_bf16(__fmul_rn(bf16_to_f32(table[f32_to_bf16(g)]), u));
}

// ---- 4-bit code decode -----------------------------------------------------------------------------------------
// v_perm_b32: byte i of the result is byte sel[i] of the 8-byte value {hi, lo} (selector 0..3 -> lo, 4..7 -> hi).
__device__ __forceinline__ uint32_t perm(uint32_t hi, uint32_t lo, uint32_t sel) {
    return __builtin_amdgcn_perm(hi, lo, sel);
}

// Per-byte two's-complement negation of bytes in 0..127: (0x80 - x) ^ 0x80 never borrows across bytes.
__device__ __forceinline__ uint32_t neg_bytes(uint32_t x) { return (0x80808080u - x) ^ 0x80808080u; }

// The four lookup registers of one block: magnitudes already multiplied by the block multiplier, and their
// negations.  mag * mult <= 127 per byte, so the 32-bit multiply / shift never carries across bytes.
struct BlockLut {
    uint32_t p_lo, p_hi, n_lo, n_hi;
};
__device__ __forceinline__ BlockLut scaled_lut_shift(uint32_t lut_lo, uint32_t lut_hi, uint32_t shift) {
    BlockLut t;
    t.p_lo = lut_lo << shift;
    t.p_hi = lut_hi << shift;
    t.n_lo = neg_bytes(t.p_lo);
    t.n_hi = neg_bytes(t.p_hi);
    return t;
}
__device__ __forceinline__ BlockLut scaled_lut_mul(uint32_t lut_lo, uint32_t lut_hi, uint32_t mult) {
    BlockLut t;
    t.p_lo = lut_lo * mult;
    t.p_hi = lut_hi * mult;
    t.n_lo = neg_bytes(t.p_lo);
    t.n_hi = neg_bytes(t.p_hi);
    return t;
}

// Four codes held in the low nibbles' positions of `sel4` bytes (bits 0..2 index, bit 3 sign) -> four INT8.
// A selector byte of 12 makes v_perm_b32 return 0x00, so perm(.., 0xFF.., (c & 8) | 4) is 0xFF for non-negative
// codes and 0x00 for negative ones; v_bfi then picks the positive or the negated magnitude per byte.
__device__ __forceinline__ uint32_t decode4(uint32_t c4, const BlockLut& t) {
    const uint32_t sel = c4 & 0x07070707u;
    const uint32_t pos = perm(t.p_hi, t.p_lo, sel);
    const uint32_t neg = perm(t.n_hi, t.n_lo, sel);
    const uint32_t keep = perm(0x000000FFu, 0u, (c4 & 0x08080808u) | 0x04040404u);
    return (pos & keep) | (neg & ~keep);
}

// One packed word (elements k..k+7, element i in bits 4i..4i+3) -> INT8 elements 0..3 in `a`, 4..7 in `b`.
__device__ __forceinline__ void decode_word(uint32_t w, const BlockLut& t, uint32_t& a, uint32_t& b) {
    const uint32_t s = w >> 4;
    // bytes of w: (c1c0, c3c2, c5c4, c7c6); bytes of s: (c2c1, c4c3, c6c5, 0c7): interleave to put code i in byte i
    const uint32_t c03 = perm(s, w, 0x05010400u);   // (w.b0, s.b0, w.b1, s.b1) -> low nibbles c0 c1 c2 c3
    const uint32_t c47 = perm(s, w, 0x07030602u);   // (w.b2, s.b2, w.b3, s.b3) -> low nibbles c4 c5 c6 c7
    a = decode4(c03, t);
    b = decode4(c47, t);
}

// The same word decoded without restoring element order: `e` holds elements 0,2,4,6 and `o` elements 1,3,5,7.
// Cheaper by two instructions; usable when the other operand of the dot product is permuted the same way.
__device__ __forceinline__ void decode_word_split(uint32_t w, const BlockLut& t, uint32_t& e, uint32_t& o) {
    e = decode4(w, t);
    o = decode4(w >> 4, t);
}

// The published format (E2M1 codes, power-of-two block multipliers) through the FP4 conversion instruction:
// v_cvt_scalef32_pk_f16_fp4 turns the two codes of one byte into two half-precision values, sign included, times a
// power-of-two scale; with scale = 2^(shift + 1) these are the INT8 embedding q (|q| <= 96) exactly.  Adding 1536
// puts q into the low mantissa bits (1536 + q lies in [1024, 2048), where half precision steps by 1), so the low
// byte of each half is q in two's complement; one byte permute gathers four of them.
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float fp4_scale(uint32_t shift) { return __uint_as_float((128u + shift) << 23); }
// Lowest E8M0 exponent of a row of a standard MXFP4 tensor, recovered from its scale 2^(lowest - 128) (lowest >= 1).
__device__ __forceinline__ uint32_t e8m0_row_min(float wscale) { return ((__float_as_uint(wscale) >> 23) & 0xFFu) + 1u; }
__device__ __forceinline__ void decode_word_fp4(uint32_t w, float scale, uint32_t& a, uint32_t& b) {
    const half2_t bias = half2_t{_Float16(1536.0f), _Float16(1536.0f)};
    const half2_t q0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, scale, 0) + bias;
    const half2_t q1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, scale, 1) + bias;
    const half2_t q2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, scale, 2) + bias;
    const half2_t q3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, scale, 3) + bias;
    a = perm(__builtin_bit_cast(uint32_t, q1), __builtin_bit_cast(uint32_t, q0), 0x06040200u);
    b = perm(__builtin_bit_cast(uint32_t, q3), __builtin_bit_cast(uint32_t, q2), 0x06040200u);
}

// The same with an integer multiplier per call (m = the multiplier in both halves): code value x multiplier.
__device__ __forceinline__ void decode_word_fp4_mul(uint32_t w, half2_t m, uint32_t& a, uint32_t& b) {
    const half2_t bias = half2_t{_Float16(1536.0f), _Float16(1536.0f)};
    const half2_t q0 = __builtin_elementwise_fma(half2_t(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 2.0f, 0)), m, bias);
    const half2_t q1 = __builtin_elementwise_fma(half2_t(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 2.0f, 1)), m, bias);
    const half2_t q2 = __builtin_elementwise_fma(half2_t(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 2.0f, 2)), m, bias);
    const half2_t q3 = __builtin_elementwise_fma(half2_t(__builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, 2.0f, 3)), m, bias);
    a = perm(__builtin_bit_cast(uint32_t, q1), __builtin_bit_cast(uint32_t, q0), 0x06040200u);
    b = perm(__builtin_bit_cast(uint32_t, q3), __builtin_bit_cast(uint32_t, q2), 0x06040200u);
}

// Block code of block `blk` in a row whose block codes start at `row_bc`.
__device__ __forceinline__ uint32_t block_code(const uint8_t* row_bc, uint32_t blk, int bc_bits) {
    const uint32_t per_byte = 8u / bc_bits;
    return (row_bc[blk / per_byte] >> (bc_bits * (blk % per_byte))) & ((1u << bc_bits) - 1u);
}
__device__ __forceinline__ uint32_t mult_of(const DevFormat& f, uint32_t bc) {
    return f.pow2 ? (1u << bc) : ((f.mult[bc >> 2] >> (8 * (bc & 3))) & 0xFFu);
}

// ---- wave reductions (butterfly, every lane ends with the result) ----------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = __fadd_rn(v, __shfl_xor(v, off, WAVE));
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, WAVE));
    return v;
}
__device__ __forceinline__ int wave_sum_i32(int v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, WAVE);
    return v;
}

// Per-head RMSNorm of one q or k head held by one wave: the lane holds the bf16-valued elements per*lane ..
// per*lane + per - 1 of the head in yv and their sum of squares in ss; nv receives the normalised values (bf16-valued).
__device__ __forceinline__ void head_norm(const float* yv, float ss, int per, int lane, int d,
                                          const uint16_t* __restrict__ w, float eps, float* nv) {
    ss = wave_sum(ss);
    const float inv = __fdiv_rn(1.0f, sqrtf(__fadd_rn(__fdiv_rn(ss, float(d)), eps)));
    for (int i = 0; i < per; ++i)
        nv[i] = round_bf16(__fmul_rn(bf16_to_f32(w[per * lane + i]), round_bf16(__fmul_rn(yv[i], inv))));
}
// The rotary embedding of such a head (sn / cs: the d / 2 sines and cosines of the row's position; sn == nullptr: no
// rotation).  emit(i, value) receives the bf16 result of element per*lane + i.
template <typename Emit>
__device__ __forceinline__ void head_rope(const float* nv, int per, int lane, int d, const float* sn, const float* cs,
                                          Emit&& emit) {
    for (int i = 0; i < per; ++i) {
        float v = nv[i];
        if (sn) {
            // element e = per*lane + i pairs with e +- d/2, held by lane +- 32 at the same i
            const float other = __shfl_xor(v, 32, WAVE);
            const int e = (per * lane + i) % (d / 2);
            v = lane < 32 ? __fsub_rn(__fmul_rn(v, cs[e]), __fmul_rn(other, sn[e]))
                          : __fadd_rn(__fmul_rn(v, cs[e]), __fmul_rn(other, sn[e]));
        }
        emit(i, f32_to_bf16(v));
    }
}
// Both in sequence.  Shared by the row kernel and the fused decode attention so that both give the same bits.
template <typename Emit>
__device__ __forceinline__ void head_norm_rope(const float* yv, float ss, int per, int lane, int d,
                                               const uint16_t* __restrict__ w, float eps, const float* sn,
                                               const float* cs, Emit&& emit) {
    float nv[8];
    head_norm(yv, ss, per, lane, d, w, eps, nv);
    head_rope(nv, per, lane, d, sn, cs, emit);
}

// Symmetric INT8 code of v at inverse scale qi: clamp(rint(v * qi), +-127).
__device__ __forceinline__ int quant_code(float v, float qi) {
    float r = rintf(__fmul_rn(v, qi));
    r = fminf(fmaxf(r, -127.0f), 127.0f);
    return (int)r;
}

}  // namespace scmx
