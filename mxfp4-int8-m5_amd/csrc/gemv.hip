// Decode GEMV on packed SC-MXFP4 weights: y[b, n] = epi(xs[b] * ws[n] * sum_k xq[b, k] * q[n, k]).
//
// One activation row is bandwidth-bound and needs no MFMA: a wave owns R consecutive weight rows and walks K in steps
// of 64 blocks; each lane
// loads 16 bytes of codes (one run of 32 weights) per row per step, so a wave reads 1 KiB of contiguous weights
// per load instruction.  With one activation row the codes go through the FP4 conversion instruction (two codes ->
// two half-precision values, sign and block scale included) and v_dot2c_f32_f16 against the activations staged in
// LDS as half precision: all values are small integers, so the FP32 partial sums are exact.  With several rows, or
// another weight format, codes are decoded to INT8 four at a time with byte-permute lookups and accumulated with
// v_dot4_i32_i8 against INT8 activations in LDS (bytes of every 8-group stored as elements 0,2,4,6,1,3,5,7 so the
// decode needs no re-interleave).  Either way the totals are the GEMM's INT32 accumulators and the epilogues are
// the GEMM's.  `BATCH` activation rows share one pass over the weights; for the published format they go through
// gemv_mfma_kernel below, which hands the dot products to the 4x4x4 INT8 MFMA so that the vector work per weight
// does not grow with the number of rows.
#include "scmx_common.h"

namespace scmx {

// Cache policy of the weight loads: the non-temporal hint.  A GEMV reads every code word exactly once, so nothing is
// gained by keeping the lines; marked as streaming they leave room for the activations and scales that are re-read
// (lm_head batch 1: 31.0 -> 29.3 us).
constexpr int W_STREAM = 2;
// From this many weight rows on a layer has enough 16-row groups to keep every CU busy with the half-precision MFMA kernel.
constexpr int HMFMA_MIN_ROWS = 32768;

struct GemvArgs {
    const void* x;            // pro 0: int8 [rows, K]; pro 1, 2: bf16 [rows, K]
    const float* xscale;      // pro 0
    const uint32_t* codes;
    const uint8_t* bcodes;
    const float* wscale;
    const uint16_t* res;
    uint16_t* out;
    const uint16_t* nw;       // pro 2: RMSNorm weight
    float eps;
    int epi, pro, N, K, bc_row_bytes;
    const int32_t* eidx;      // MoE: expert of each slot
    int n_eidx, xstride, shared_expert;
    DevFormat fmt;
};

__device__ __forceinline__ void store_perm8(int8_t* dst, const int q[8]) {
    const uint32_t e = (uint32_t(q[0]) & 0xFFu) | ((uint32_t(q[2]) & 0xFFu) << 8) | ((uint32_t(q[4]) & 0xFFu) << 16) |
                       ((uint32_t(q[6]) & 0xFFu) << 24);
    const uint32_t o = (uint32_t(q[1]) & 0xFFu) | ((uint32_t(q[3]) & 0xFFu) << 8) | ((uint32_t(q[5]) & 0xFFu) << 16) |
                       ((uint32_t(q[7]) & 0xFFu) << 24);
    *reinterpret_cast<u32x2*>(dst) = u32x2{e, o};
}

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));

// Eight INT8 codes as eight half-precision values (exact), in element order, 16 bytes.
__device__ __forceinline__ void store_half8(int8_t* dst, const int q[8]) {
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const h2 p = h2{_Float16(float(q[2 * i])), _Float16(float(q[2 * i + 1]))};
        o[i] = __builtin_bit_cast(uint32_t, p);
    }
    *reinterpret_cast<u32x4*>(dst) = o;
}

// Eight INT8 codes in element order, 8 bytes.
__device__ __forceinline__ void store_plain8(int8_t* dst, const int q[8]) {
    u32x2 o = u32x2{0u, 0u};
#pragma unroll
    for (int i = 0; i < 8; ++i) o[i >> 2] |= (uint32_t(q[i]) & 0xFFu) << (8 * (i & 3));
    *reinterpret_cast<u32x2*>(dst) = o;
}

enum { X_PERM8 = 0, X_HALF = 1, X_PLAIN8 = 2 };

// Stage one activation row into LDS and return its scale: permuted INT8 (8 bytes per 8-group), or with F16 the codes
// as half-precision values in element order (16 bytes per 8-group).  `red` holds 66 floats.
// `pre` (valid when have_pre): the thread's 16 bytes of the row, x[8 tid .. 8 tid + 7], loaded by the caller BEFORE it
// requested its first weights.  Loads return in order, so a row read after the weight prefetch could only be used once
// those weights had arrived; read first, the row is quantized while the weights are still on their way.
// KEEP: rows of up to 8 * NT * KEEP values are read once and stay in registers between the maximum and the rounding.
template <int NT, int XMODE, int KEEP = 1>
__device__ float stage_row(const GemvArgs& a, int row, int8_t* sx, float* red, u32x4 pre = u32x4{0u, 0u, 0u, 0u},
                           bool have_pre = false) {
    constexpr bool F16 = XMODE == X_HALF;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int K = a.K;
    if (a.pro == 0) {
        const u32x2* src = reinterpret_cast<const u32x2*>(reinterpret_cast<const int8_t*>(a.x) + size_t(row) * K);
        for (int c = tid; c < K / 8; c += NT) {
            const u32x2 v = src[c];
            if (F16) {
                int q[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) q[i] = int(int8_t(v[i >> 2] >> (8 * (i & 3))));
                store_half8(sx + 16 * c, q);
            } else if (XMODE == X_PLAIN8) {
                *reinterpret_cast<u32x2*>(sx + 8 * c) = v;
            } else {
                *reinterpret_cast<u32x2*>(sx + 8 * c) = u32x2{perm(v[1], v[0], 0x06040200u), perm(v[1], v[0], 0x07050301u)};
            }
        }
        return a.xscale[row];
    }
    const uint16_t* xr = reinterpret_cast<const uint16_t*>(a.x) + size_t(row) * K;
    float inv = 1.0f;
    if (a.pro == 2) {
        // sum of squares: K/4 virtual threads of 4 values, 64 virtual threads per wave_sum, then one wave_sum over
        // the per-group partials (at most 64 groups: K <= 16384)
        for (int g = wave; g < (K / 4 + 63) / 64; g += NT / 64) {
            const int v = 64 * g + lane;
            float ss = 0.0f;
            if (v < K / 4) {
                const u32x2 p = *reinterpret_cast<const u32x2*>(xr + 4 * v);
                const float x0 = __uint_as_float(p[0] << 16), x1 = __uint_as_float(p[0] & 0xFFFF0000u);
                const float x2 = __uint_as_float(p[1] << 16), x3 = __uint_as_float(p[1] & 0xFFFF0000u);
                ss = __fadd_rn(ss, __fmul_rn(x0, x0));
                ss = __fadd_rn(ss, __fmul_rn(x1, x1));
                ss = __fadd_rn(ss, __fmul_rn(x2, x2));
                ss = __fadd_rn(ss, __fmul_rn(x3, x3));
            }
            ss = wave_sum(ss);
            if (lane == 0) red[g] = ss;
        }
        __syncthreads();
        if (wave == 0) {
            const float tot = wave_sum(lane < (K / 4 + 63) / 64 ? red[lane] : 0.0f);
            if (lane == 0) red[64] = __fdiv_rn(1.0f, sqrtf(__fadd_rn(__fdiv_rn(tot, float(K)), a.eps)));
        }
        __syncthreads();
        inv = red[64];
        __syncthreads();
    }
    // eight values per thread and step, from one 16-byte load (and one of the norm weight for pro 2)
    auto values = [&](int c, float (&v)[8]) {
        const u32x4 p = (have_pre && c == int(threadIdx.x)) ? pre : *reinterpret_cast<const u32x4*>(xr + 8 * c);
        u32x4 q = u32x4{0u, 0u, 0u, 0u};
        if (a.pro == 2) q = *reinterpret_cast<const u32x4*>(a.nw + 8 * c);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float xv = __uint_as_float(i & 1 ? (p[i >> 1] & 0xFFFF0000u) : (p[i >> 1] << 16));
            if (a.pro == 2) {
                const float wv = __uint_as_float(i & 1 ? (q[i >> 1] & 0xFFFF0000u) : (q[i >> 1] << 16));
                v[i] = round_bf16(__fmul_rn(wv, round_bf16(__fmul_rn(xv, inv))));
            } else {
                v[i] = xv;
            }
        }
    };
    // KEEP = 1 where many waves per CU matter (more costs a wave of occupancy: the first weight loads are in flight too);
    // 3 for narrow layers with long rows, whose second pass over the row would be a second round trip to memory.
    const bool keep = K <= 8 * NT * KEEP;
    float kept[KEEP][8];
    float amax = 0.0f;
    if (keep) {
#pragma unroll
        for (int j = 0; j < KEEP; ++j) {
            const int c = tid + j * NT;
            if (c < K / 8) {
                values(c, kept[j]);
#pragma unroll
                for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(kept[j][i]));
            }
        }
    } else {
        for (int c = tid; c < K / 8; c += NT) {
            float v[8];
            values(c, v);
#pragma unroll
            for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
        }
    }
    amax = wave_max(amax);
    if (lane == 0) red[wave] = amax;
    __syncthreads();
    amax = 0.0f;
    for (int w = 0; w < NT / 64; ++w) amax = fmaxf(amax, red[w]);
    const float s = __fdiv_rn(amax, 127.0f);
    const float qi = s > 0.0f ? __fdiv_rn(1.0f, s) : 0.0f;
    const auto emit = [&](int c, const float (&v)[8]) {
        int q[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = quant_code(v[i], qi);
        if (F16) store_half8(sx + 16 * c, q);
        else if (XMODE == X_PLAIN8) store_plain8(sx + 8 * c, q);
        else store_perm8(sx + 8 * c, q);
    };
    if (keep) {
#pragma unroll
        for (int j = 0; j < KEEP; ++j) {
            const int c = tid + j * NT;
            if (c < K / 8) emit(c, kept[j]);
        }
    } else {
        for (int c = tid; c < K / 8; c += NT) {
            float v[8];
            values(c, v);
            emit(c, v);
        }
    }
    __syncthreads();   // `red` is reused by the next row
    return s;
}

// The same staging done by ONE wave (every lane of the wave calls it): with several activation rows each wave of the
// workgroup takes rows of its own, so the rows are staged side by side instead of one after another and no workgroup
// barrier is needed in between.  Same arithmetic in the same order as stage_row (maxima are order-free; the sum of
// squares is formed by the same virtual threads, butterflies and partials), hence the same bits.  K <= 16384.
// `pre` (valid when have_pre, K <= 512 * WAVE_PRE): the lane's chunks x[8 (lane + 64 j) ..], loaded before the first weights.
template <int WAVE_PRE>
struct WavePre {
    u32x4 v[WAVE_PRE];
};
template <int XMODE, int WAVE_PRE>
__device__ float stage_row_wave(const GemvArgs& a, int row, int8_t* sx, const WavePre<WAVE_PRE>& pre, bool have_pre) {
    constexpr bool F16 = XMODE == X_HALF;
    const int lane = threadIdx.x & 63;
    const int K = a.K;
    if (a.pro == 0) {
        const u32x2* src = reinterpret_cast<const u32x2*>(reinterpret_cast<const int8_t*>(a.x) + size_t(row) * K);
        for (int c = lane; c < K / 8; c += 64) {
            const u32x2 v = src[c];
            if (F16) {
                int q[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) q[i] = int(int8_t(v[i >> 2] >> (8 * (i & 3))));
                store_half8(sx + 16 * c, q);
            } else if (XMODE == X_PLAIN8) {
                *reinterpret_cast<u32x2*>(sx + 8 * c) = v;
            } else {
                *reinterpret_cast<u32x2*>(sx + 8 * c) = u32x2{perm(v[1], v[0], 0x06040200u), perm(v[1], v[0], 0x07050301u)};
            }
        }
        return a.xscale[row];
    }
    const uint16_t* xr = reinterpret_cast<const uint16_t*>(a.x) + size_t(row) * K;
    float inv = 1.0f;
    if (a.pro == 2) {
        const int groups = (K / 4 + 63) / 64;
        float mine = 0.0f;   // lane g keeps the partial of group g
        for (int g = 0; g < groups; ++g) {
            const int v = 64 * g + lane;
            float ss = 0.0f;
            if (v < K / 4) {
                const u32x2 p = *reinterpret_cast<const u32x2*>(xr + 4 * v);
                const float x0 = __uint_as_float(p[0] << 16), x1 = __uint_as_float(p[0] & 0xFFFF0000u);
                const float x2 = __uint_as_float(p[1] << 16), x3 = __uint_as_float(p[1] & 0xFFFF0000u);
                ss = __fadd_rn(ss, __fmul_rn(x0, x0));
                ss = __fadd_rn(ss, __fmul_rn(x1, x1));
                ss = __fadd_rn(ss, __fmul_rn(x2, x2));
                ss = __fadd_rn(ss, __fmul_rn(x3, x3));
            }
            ss = wave_sum(ss);
            if (lane == g) mine = ss;
        }
        const float tot = wave_sum(lane < groups ? mine : 0.0f);
        inv = __fdiv_rn(1.0f, sqrtf(__fadd_rn(__fdiv_rn(tot, float(K)), a.eps)));
    }
    auto values = [&](int c, u32x4 p, float (&v)[8]) {
        u32x4 q = u32x4{0u, 0u, 0u, 0u};
        if (a.pro == 2) q = *reinterpret_cast<const u32x4*>(a.nw + 8 * c);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float xv = __uint_as_float(i & 1 ? (p[i >> 1] & 0xFFFF0000u) : (p[i >> 1] << 16));
            if (a.pro == 2) {
                const float wv = __uint_as_float(i & 1 ? (q[i >> 1] & 0xFFFF0000u) : (q[i >> 1] << 16));
                v[i] = round_bf16(__fmul_rn(wv, round_bf16(__fmul_rn(xv, inv))));
            } else {
                v[i] = xv;
            }
        }
    };
    const auto emit = [&](int c, const float (&v)[8], float qi) {
        int q[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) q[i] = quant_code(v[i], qi);
        if (F16) store_half8(sx + 16 * c, q);
        else if (XMODE == X_PLAIN8) store_plain8(sx + 8 * c, q);
        else store_perm8(sx + 8 * c, q);
    };
    float amax = 0.0f;
    if (have_pre) {   // the row is in registers: one pass
#pragma unroll
        for (int j = 0; j < WAVE_PRE; ++j)
            if (lane + 64 * j < K / 8) {
                float v[8];
                values(lane + 64 * j, pre.v[j], v);
#pragma unroll
                for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
            }
    } else {
        for (int c = lane; c < K / 8; c += 64) {
            float v[8];
            values(c, *reinterpret_cast<const u32x4*>(xr + 8 * c), v);
#pragma unroll
            for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
        }
    }
    amax = wave_max(amax);
    const float s = __fdiv_rn(amax, 127.0f);
    const float qi = s > 0.0f ? __fdiv_rn(1.0f, s) : 0.0f;
    if (have_pre) {
#pragma unroll
        for (int j = 0; j < WAVE_PRE; ++j)
            if (lane + 64 * j < K / 8) {
                float v[8];
                values(lane + 64 * j, pre.v[j], v);
                emit(lane + 64 * j, v, qi);
            }
    } else {
        for (int c = lane; c < K / 8; c += 64) {
            float v[8];
            values(c, *reinterpret_cast<const u32x4*>(xr + 8 * c), v);
            emit(c, v, qi);
        }
    }
    return s;
}

// The lane's chunks of activation row `row` for stage_row_wave, requested now (prologue 1 only, K <= 512 * WAVE_PRE).
template <int WAVE_PRE>
__device__ __forceinline__ bool wave_prefetch_row(const GemvArgs& a, int row, bool valid, WavePre<WAVE_PRE>& pre) {
    const int lane = threadIdx.x & 63;
    const bool ok = valid && a.pro == 1 && a.K <= 512 * WAVE_PRE;
    if (ok) {
        const uint16_t* xr = reinterpret_cast<const uint16_t*>(a.x) + size_t(row) * a.K;
#pragma unroll
        for (int j = 0; j < WAVE_PRE; ++j)
            if (lane + 64 * j < a.K / 8) pre.v[j] = *reinterpret_cast<const u32x4*>(xr + 8 * (lane + 64 * j));
    }
    return ok;
}
// The thread's chunk of activation row `row` for the workgroup-wide stage_row (prologue 1 only, K <= 8 * NT).
template <int NT>
__device__ __forceinline__ bool block_prefetch_row(const GemvArgs& a, int row, u32x4& pre) {
    const bool ok = a.pro == 1 && a.K <= 8 * NT;
    if (ok && int(threadIdx.x) < a.K / 8)
        pre = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(a.x) + size_t(row) * a.K + 8 * threadIdx.x);
    return ok;
}

// Wave sum with DPP adds (one VALU instruction per step): quad swaps, half-row and row mirrors, then the two row
// broadcasts.  The total is valid in lane 63 only.
__device__ __forceinline__ int wave_sum_to_lane63(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, false);    // quad_perm [1,0,3,2]
    v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, false);    // quad_perm [2,3,0,1]
    v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, false);   // row_half_mirror
    v += __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, false);   // row_mirror
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false);   // row_bcast15 into rows 1 and 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false);   // row_bcast31 into rows 2 and 3
    return v;
}

// Value of `v` in lane (lane ^ OFF): DPP moves where the pattern exists, the LDS crossbar otherwise.
template <int OFF>
__device__ __forceinline__ int xor_lane(int v) {
    if (OFF == 1) return __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, false);    // quad_perm [1,0,3,2]
    if (OFF == 2) return __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, false);    // quad_perm [2,3,0,1]
    if (OFF == 4) return __builtin_amdgcn_ds_swizzle(v, 0x101F);                      // bit mode: xor 4
    if (OFF == 8) return __builtin_amdgcn_update_dpp(0, v, 0x128, 0xF, 0xF, false);   // row_ror:8
    if (OFF == 16) return __builtin_amdgcn_ds_swizzle(v, 0x401F);                     // bit mode: xor 16
    return __shfl_xor(v, 32, WAVE);
}

// Wave totals of NV per-lane values in 6 exchange steps (offsets 1, 2, 4, 8, 16, 32).  While more than one value is
// left, a step halves the set: lanes whose bit is clear keep the lower half and receive the partner's partials of
// it, the others the upper half; the remaining steps are plain sums.  Lane L ends with the total of value index
// bitreverse(L mod NV) over log2(NV) bits; every lane with the same L mod NV holds the same total.
template <int NV, int OFF = 1>
__device__ __forceinline__ int select_reduce(int (&v)[NV], int lane) {
    if constexpr (NV > 1) {
        const bool up = (lane & OFF) != 0;
        int h[NV / 2];
#pragma unroll
        for (int i = 0; i < NV / 2; ++i) {
            const int keep = up ? v[i + NV / 2] : v[i];
            const int send = up ? v[i] : v[i + NV / 2];
            h[i] = keep + xor_lane<OFF>(send);
        }
        if constexpr (OFF < 32) return select_reduce<NV / 2, OFF * 2>(h, lane);
        else return h[0];
    } else {
        int t = v[0];
        if constexpr (OFF <= 1) t += xor_lane<1>(t);
        if constexpr (OFF <= 2) t += xor_lane<2>(t);
        if constexpr (OFF <= 4) t += xor_lane<4>(t);
        if constexpr (OFF <= 8) t += xor_lane<8>(t);
        if constexpr (OFF <= 16) t += xor_lane<16>(t);
        if constexpr (OFF <= 32) t += xor_lane<32>(t);
        return t;
    }
}

// MODE 0: any format, byte-permute decode + v_dot4_i32_i8.  MODE 1: the published format with the same arithmetic
// (lookup tables are constants).  MODE 2: the published format through the FP4 conversion
// instruction: v_cvt_scalef32_pk_f16_fp4 turns two codes into two half-precision values, sign and block scale
// included, and v_dot2c_f32_f16 multiplies them with the activations held as half precision.  Every value is an
// integer below 2^11 and every partial sum one below 2^24, so the FP32 sums are exact and equal the integer ones.
template <int BATCH, int R, int MODE, int KEEP = 1>
__global__ __launch_bounds__(256) void gemv_kernel(const GemvArgs a) {
    constexpr int NT = 256;
    constexpr int NV = R * BATCH;
    // MODE 0: any member of the format family (table decode); 1: published format, integer dot products; 2: published
    // format through the FP4 conversion; 3: the same codebook and shifts on 16-element blocks through the FP4 conversion
    constexpr bool DEFAULT_FMT = MODE != 0;
    // conversion; 4: that codebook on 16-element blocks with 4-bit codes for consecutive integer multipliers
    constexpr bool FP4 = MODE >= 2;
    constexpr bool B16 = MODE == 3;
    constexpr bool B16M = MODE == 4;
    // 5: a standard MXFP4 tensor in place -- the FP4 conversion with one E8M0 byte per 32-block instead of a 2-bit code
    constexpr bool E8 = MODE == 5;
    constexpr int XB = FP4 ? 2 : 1;                    // bytes per staged activation
    extern __shared__ __attribute__((aligned(16))) int8_t smem[];
    const int K = a.K, N = a.N;
    int8_t* sx = smem;                                                   // [BATCH][K] staged activations
    const int Kp = (K + 2047) & ~2047;                                    // row pitch: whole 64-chunk slices, zero padded
    float* red = reinterpret_cast<float*>(smem + size_t(BATCH) * Kp * XB);   // 68 floats + BATCH scales
    float* sxs = red + 68;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: row bases stay in scalar registers

    // MoE: one slot per blockIdx.y, its own expert and (xstride = 1) its own input row
    const int slot = blockIdx.y;
    int expert = 0, xrow0 = 0;
    if (a.eidx) {
        expert = (a.shared_expert >= 0 && slot == a.n_eidx) ? a.shared_expert : a.eidx[slot];
        xrow0 = slot * a.xstride;
    }
    const size_t erow = size_t(expert) * N;
    const int orow0 = a.eidx ? slot : 0;
    const int nchunk = K / 32;   // 16-byte code groups per row
    const int groups = N / R;
    // Waves walk the row groups with a grid stride, so the staged activations serve many rows.  The work of a wave is
    // a sequence of items (row group, 64-chunk slice of K); the weights of the next item are loaded into a second
    // register set before the current item is decoded, so every wave always has loads in flight.
    struct Item {
        u32x4 w[R];
        uint32_t bc[R];
        uint32_t rmin[E8 ? R : 1];   // E8: the rows' lowest exponent bytes (from their scales; wave-uniform)
    };
    const int g_stride = gridDim.x * (NT / 64);
    const int CI = (nchunk + 63) / 64;                 // items per row group
    // Buffer loads: the row group's base sits in a scalar resource descriptor, the row offset in a scalar operand and
    // the lane's chunk offset in one vector register, so a load costs no vector address arithmetic; reads past the
    // group's last row return zero.
    auto load_item = [&](Item& it, int g, uint32_t c) {
        const uint32_t cc = min(c, uint32_t(nchunk - 1));
        const uint8_t* crow = reinterpret_cast<const uint8_t*>(a.codes) + (erow + size_t(g) * R) * (K / 2);   // uniform
        const uint8_t* brow = a.bcodes + (erow + size_t(g) * R) * a.bc_row_bytes;
        const __amdgpu_buffer_rsrc_t rc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(crow), 0, R * (K / 2), 0x00020000);
        const __amdgpu_buffer_rsrc_t rb =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(brow), 0, R * a.bc_row_bytes, 0x00020000);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            it.w[r] = __builtin_amdgcn_raw_buffer_load_b128(rc, int(16u * cc), r * (K / 2), W_STREAM);
            // the byte with the chunk's block codes: 4 blocks per byte = 4 chunks of 32 weights, or 2 with 16-blocks
            if (DEFAULT_FMT) it.bc[r] = __builtin_amdgcn_raw_buffer_load_b8(rb, int(cc >> ((B16M || E8) ? 0 : B16 ? 1 : 2)), r * a.bc_row_bytes, 0);
            if constexpr (E8) it.rmin[E8 ? r : 0] = e8m0_row_min(a.wscale[erow + size_t(g) * R + r]);
        }
    };
    auto compute_item = [&](const Item& it, int g, uint32_t c_in, int (&acc)[NV]) {
        const uint32_t c = c_in;   // lanes past the row end read activations from the zero padding in LDS
        const u32x4(&w)[R] = it.w;
        const uint32_t(&bc)[R] = it.bc;
        const uint8_t* brow = a.bcodes + (erow + size_t(g) * R) * a.bc_row_bytes;
        (void)brow;
        if constexpr (FP4) {
            float part[R][BATCH];
            float part2[B16M ? R : 1][BATCH];   // integer multipliers: words 2-3 (the chunk's second block) summed apart
            float scale[R][2];   // 2^(shift + 1) of words 0-1 and 2-3: the codes are E2M1 values, the INT8 embedding is twice the value
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (B16M) {
                    scale[r][0] = scale[r][1] = 2.0f;
#pragma unroll
                    for (int b = 0; b < BATCH; ++b) part2[r][b] = 0.0f;
                } else if (E8) {
                    scale[r][0] = scale[r][1] = __uint_as_float(((128u + bc[r] - it.rmin[E8 ? r : 0]) & 0xFFu) << 23);
                } else if (B16) {
                    scale[r][0] = __uint_as_float((128u + ((bc[r] >> (4 * (c & 1))) & 3u)) << 23);
                    scale[r][1] = __uint_as_float((128u + ((bc[r] >> (4 * (c & 1) + 2)) & 3u)) << 23);
                } else {
                    scale[r][0] = scale[r][1] = __uint_as_float((128u + ((bc[r] >> (2 * (c & 3))) & 3u)) << 23);
                }
#pragma unroll
                for (int b = 0; b < BATCH; ++b) part[r][b] = 0.0f;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                h8 xv[BATCH];   // the 8 activations of word j
#pragma unroll
                for (int b = 0; b < BATCH; ++b)
                    xv[b] = *reinterpret_cast<const h8*>(sx + (size_t(b) * Kp + 32u * c + 8u * j) * 2);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const uint32_t wj = w[r][j];
                    const h2 q0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(wj, scale[r][j >> 1], 0);
                    const h2 q1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(wj, scale[r][j >> 1], 1);
                    const h2 q2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(wj, scale[r][j >> 1], 2);
                    const h2 q3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(wj, scale[r][j >> 1], 3);
#pragma unroll
                    for (int b = 0; b < BATCH; ++b) {
                        float& dst = (B16M && j >= 2) ? part2[B16M ? r : 0][b] : part[r][b];
                        float p = dst;
                        p = __builtin_amdgcn_fdot2(q0, __builtin_shufflevector(xv[b], xv[b], 0, 1), p, false);
                        p = __builtin_amdgcn_fdot2(q1, __builtin_shufflevector(xv[b], xv[b], 2, 3), p, false);
                        p = __builtin_amdgcn_fdot2(q2, __builtin_shufflevector(xv[b], xv[b], 4, 5), p, false);
                        p = __builtin_amdgcn_fdot2(q3, __builtin_shufflevector(xv[b], xv[b], 6, 7), p, false);
                        dst = p;
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int m0 = int(a.fmt.mult[0] & 0xFFu);
                const int mlo = m0 + int(bc[r] & 15u), mhi = m0 + int((bc[r] >> 4) & 15u);
#pragma unroll
                for (int b = 0; b < BATCH; ++b) {
                    if (B16M)
                        acc[r * BATCH + b] += int(part[r][b]) * mlo + int(part2[r][b]) * mhi;
                    else
                        acc[r * BATCH + b] += int(part[r][b]);
                }
            }
            return;
        }
            u32x4 xv[BATCH][2];
#pragma unroll
            for (int b = 0; b < BATCH; ++b) {
                xv[b][0] = *reinterpret_cast<const u32x4*>(sx + size_t(b) * Kp + 32u * c);
                xv[b][1] = *reinterpret_cast<const u32x4*>(sx + size_t(b) * Kp + 32u * c + 16);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                int part[BATCH];
#pragma unroll
                for (int b = 0; b < BATCH; ++b) part[b] = 0;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t wj = w[r][j];
                    uint32_t e, o;
                    if (DEFAULT_FMT) {
                        const BlockLut t = scaled_lut_shift(0x03020100u, 0x0C080604u, 0u);   // folds to constants
                        decode_word_split(wj, t, e, o);
                    } else {
                        const uint32_t blk = uint32_t(32 * c + 8 * j) >> a.fmt.block_log2;
                        const uint32_t code = block_code(brow + r * a.bc_row_bytes, blk, a.fmt.bc_bits);
                        const BlockLut t = scaled_lut_mul(a.fmt.lut_lo, a.fmt.lut_hi, mult_of(a.fmt, code));
                        decode_word_split(wj, t, e, o);
                    }
#pragma unroll
                    for (int b = 0; b < BATCH; ++b) {
                        part[b] = __builtin_amdgcn_sdot4(int(e), int(xv[b][j >> 1][2 * (j & 1)]), part[b], false);
                        part[b] = __builtin_amdgcn_sdot4(int(o), int(xv[b][j >> 1][2 * (j & 1) + 1]), part[b], false);
                    }
                }
                const uint32_t sh = DEFAULT_FMT ? (bc[r] >> (2 * (c & 3))) & 3u : 0u;
#pragma unroll
                for (int b = 0; b < BATCH; ++b) acc[r * BATCH + b] += part[b] << sh;
            }

    };
    auto finish = [&](int g, int (&acc)[NV]) {
        const int n0 = g * R;
        if (a.epi != SCMX_EPI_SWIGLU) {
            // one output per lane: lane L < NV ends with the total of value index bitreverse(L), r * BATCH + b
            const int tot = select_reduce<NV>(acc, lane);
            if (lane < NV) {
                constexpr int LOG = NV == 1 ? 0 : NV == 2 ? 1 : NV == 4 ? 2 : NV == 8 ? 3 : NV == 16 ? 4 : NV == 32 ? 5 : 6;
                const int idx = LOG == 0 ? 0 : int(__builtin_bitreverse32(uint32_t(lane)) >> (32 - (LOG == 0 ? 1 : LOG)));
                const int r = idx / BATCH, b = idx % BATCH;
                const float y = __fmul_rn(__fmul_rn(float(tot), sxs[b]), a.wscale[erow + n0 + r]);
                const size_t o = size_t(orow0 + b) * N + n0 + r;
                if (a.epi == SCMX_EPI_SCALE)
                    a.out[o] = f32_to_bf16(y);
                else
                    a.out[o] = f32_to_bf16(__fadd_rn(bf16_to_f32(a.res[o]), round_bf16(y)));
            }
            return;
        }
        // SwiGLU needs four rows in one lane: totals land in lane 63, which applies the epilogue
#pragma unroll
        for (int i = 0; i < NV; ++i) acc[i] = wave_sum_to_lane63(acc[i]);
        if (lane == 63) {
            float wsr[R];
#pragma unroll
            for (int r = 0; r < R; ++r) wsr[r] = a.wscale[erow + n0 + r];
#pragma unroll
            for (int b = 0; b < BATCH; ++b) {
                const float xsb = sxs[b];
                const size_t orow = size_t(orow0 + b);
                float y[R];
#pragma unroll
                for (int r = 0; r < R; ++r) y[r] = __fmul_rn(__fmul_rn(float(acc[r * BATCH + b]), xsb), wsr[r]);
                if (a.epi == SCMX_EPI_SCALE) {
                    if (R == 8 && (N & 7) == 0) {   // 8 consecutive outputs: one 16-byte store
                        u32x4 o;
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            o[r] = uint32_t(f32_to_bf16(y[(2 * r) % R])) | (uint32_t(f32_to_bf16(y[(2 * r + 1) % R])) << 16);
                        *reinterpret_cast<u32x4*>(a.out + orow * N + n0) = o;
                    } else {
#pragma unroll
                        for (int r = 0; r < R; ++r) a.out[orow * N + n0 + r] = f32_to_bf16(y[r]);
                    }
                } else if (a.epi == SCMX_EPI_RES) {
#pragma unroll
                    for (int r = 0; r < R; ++r) {
                        const float rv = bf16_to_f32(a.res[orow * N + n0 + r]);
                        a.out[orow * N + n0 + r] = f32_to_bf16(__fadd_rn(rv, round_bf16(y[r])));
                    }
                } else if (R % 4 == 0) {   // SwiGLU of rows (g, g, u, u)
#pragma unroll
                    for (int r = 0; r < R; r += 4) {
                        uint16_t* o = a.out + orow * (N / 2) + (n0 + r) / 2;
                        o[0] = swiglu_bf16(round_bf16(y[r]), round_bf16(y[(r + 2) % R]));
                        o[1] = swiglu_bf16(round_bf16(y[(r + 1) % R]), round_bf16(y[(r + 3) % R]));
                    }
                }
            }
        }
    };

    // ---- driver ---------------------------------------------------------------------------------------------------
    // NB register sets hold the wave's current item and the NB - 1 after it.  All are requested before the
    // activations are staged, so the first weights are already on their way while the workgroup quantizes its input.
    // a third set costs occupancy and measured slower on wide layers; the long-row variant for narrow layers (KEEP > 1)
    // has few waves per CU anyway and three items per row, so it requests all of a row's codes at once
    constexpr int NB = KEEP > 1 ? 3 : 2;
    const auto advance = [&](int& gi, int& cidx) {
        if (++cidx == CI) {
            cidx = 0;
            gi += g_stride;
        }
    };
    Item buf[NB];
    int gq[NB], cq[NB];   // the item each set holds
    gq[0] = blockIdx.x * (NT / 64) + wave;
    cq[0] = 0;
#pragma unroll
    for (int i = 1; i < NB; ++i) {
        gq[i] = gq[i - 1];
        cq[i] = cq[i - 1];
        advance(gq[i], cq[i]);
    }
    // the first activation row is requested before the weights: memory returns a wave's loads in order
    u32x4 xpre = u32x4{0u, 0u, 0u, 0u};
    const bool have_pre = block_prefetch_row<NT>(a, xrow0, xpre);
#pragma unroll
    for (int i = 0; i < NB; ++i)
        if (gq[i] < groups) load_item(buf[i], gq[i], lane + 64u * cq[i]);

#pragma unroll
    for (int b = 0; b < BATCH; ++b) {
        const float s = stage_row<NT, FP4 ? X_HALF : X_PERM8, KEEP>(a, xrow0 + b, sx + size_t(b) * Kp * XB, red, xpre, have_pre && b == 0);
        for (int c = K * XB / 4 + tid; c < Kp * XB / 4; c += NT) reinterpret_cast<uint32_t*>(sx + size_t(b) * Kp * XB)[c] = 0u;
        if (tid == 0) sxs[b] = s;
    }
    __syncthreads();
    if (gq[0] >= groups) return;
    int acc[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) acc[i] = 0;
    bool more = true;
    while (more) {
#pragma unroll
        for (int i = 0; i < NB; ++i) {   // consume set i, then refill it with the item after the newest one in flight
            if (gq[i] >= groups) {
                more = false;
                break;
            }
            compute_item(buf[i], gq[i], lane + 64u * cq[i], acc);
            if (cq[i] == CI - 1) {
                finish(gq[i], acc);
#pragma unroll
                for (int v = 0; v < NV; ++v) acc[v] = 0;
            }
            gq[i] = gq[(i + NB - 1) % NB];
            cq[i] = cq[(i + NB - 1) % NB];
            advance(gq[i], cq[i]);
            if (gq[i] < groups) load_item(buf[i], gq[i], lane + 64u * cq[i]);
        }
    }
}

// Several activation rows against the published format: the dot products go to the matrix pipe.
// v_mfma_i32_4x4x4_16b_i8 multiplies, in each of 16 blocks of 4 lanes, a 4x4 INT8 matrix of activations (lane i of the
// block: 4 consecutive k of activation row i) with one of weights (lane j: the same 4 k of weight row j) and adds the
// 4x4 INT32 result (lane j, register r = activation row r, weight row j).  A wave owns 4 consecutive weight rows;
// lane (block b, j) loads four 16-byte runs of row j (chunks b, b+16, b+32, b+48 of the 64-chunk slice), decodes
// them with the FP4 conversion and feeds 8 MFMAs per run; the 16 blocks cover different k, so a row group ends with a
// sum over the blocks.  Vector work per weight no longer grows with the number of activation rows.
template <int BATCH>
__global__ __launch_bounds__(256) void gemv_mfma_kernel(const GemvArgs a) {
    constexpr int NT = 256;
    constexpr int NSET = BATCH > 4 ? 2 : 1;    // MFMA accumulators: activation rows 0..3 and 4..7
    constexpr int XR = 4 * NSET;               // activation rows as the MFMA sees them (zero rows pad BATCH up)
    extern __shared__ __attribute__((aligned(16))) int8_t smem[];
    const int K = a.K, N = a.N;
    const int Kp = (K + 2047) & ~2047;
    int8_t* sx = smem;                                                   // [XR][Kp] INT8 in element order
    float* red = reinterpret_cast<float*>(smem + size_t(XR) * Kp);      // 68 floats + BATCH scales
    float* sxs = red + 68;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int blk = lane >> 2, j = lane & 3;
    const int nchunk = K / 32, groups = N / 4;
    const int CI = (nchunk + 63) / 64;
    const int g_stride = gridDim.x * (NT / 64);

    struct Item {
        u32x4 w[4];   // runs blk, blk + 16, blk + 32, blk + 48 of the slice, weight row j
        u32x4 bc;     // the slice's 16 block-code bytes of row j
    };
    const auto load_item = [&](Item& it, int g, int ci) {
        const uint8_t* crow = reinterpret_cast<const uint8_t*>(a.codes) + size_t(g) * 4 * (K / 2);   // uniform
        const uint8_t* brow = a.bcodes + size_t(g) * 4 * a.bc_row_bytes;
        const __amdgpu_buffer_rsrc_t rc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(crow), 0, 4 * (K / 2), 0x00020000);
        const __amdgpu_buffer_rsrc_t rb =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(brow), 0, 4 * a.bc_row_bytes, 0x00020000);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = min(ci * 64 + blk + 16 * i, nchunk - 1);   // past the row: any valid run (its activations are 0)
            it.w[i] = __builtin_amdgcn_raw_buffer_load_b128(rc, j * (K / 2) + 16 * c, 0, W_STREAM);
        }
        it.bc = __builtin_amdgcn_raw_buffer_load_b128(rb, j * a.bc_row_bytes, ci * 16, 0);   // out of range reads 0
    };
    v4i acc[NSET], acc2[NSET];   // two accumulation chains per set: consecutive MFMAs do not wait for each other
    const auto compute_item = [&](const Item& it, int ci) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t c = uint32_t(ci * 64 + blk + 16 * i);
            // block code of run c: byte blk / 4 of dword i of the slice's 16 bytes, bits 2 * (blk % 4)
            const float scale = fp4_scale((it.bc[i] >> (2 * blk)) & 3u);
            u32x4 xv[NSET][2];
#pragma unroll
            for (int s = 0; s < NSET; ++s) {
                xv[s][0] = *reinterpret_cast<const u32x4*>(sx + size_t(4 * s + j) * Kp + 32u * c);
                xv[s][1] = *reinterpret_cast<const u32x4*>(sx + size_t(4 * s + j) * Kp + 32u * c + 16);
            }
#pragma unroll
            for (int wd = 0; wd < 4; ++wd) {
                uint32_t qa, qb;
                decode_word_fp4(it.w[i][wd], scale, qa, qb);
#pragma unroll
                for (int s = 0; s < NSET; ++s) {
                    acc[s] = __builtin_amdgcn_mfma_i32_4x4x4i8(int(xv[s][wd >> 1][2 * (wd & 1)]), int(qa), acc[s], 0, 0, 0);
                    acc2[s] = __builtin_amdgcn_mfma_i32_4x4x4i8(int(xv[s][wd >> 1][2 * (wd & 1) + 1]), int(qb), acc2[s], 0, 0, 0);
                }
            }
        }
    };
    const auto finish = [&](int g) {
        // Totals over the 16 blocks (lane bits 2..5).  The first exchange steps also halve the set of values a lane
        // carries, so a lane ends with one total: that of activation row `brow`, weight row j.
        constexpr int NV = 4 * NSET;
        int vals[NV];
#pragma unroll
        for (int s = 0; s < NSET; ++s)
#pragma unroll
            for (int r = 0; r < 4; ++r) vals[4 * s + r] = acc[s][r] + acc2[s][r];
        const int tot = select_reduce<NV, 4>(vals, lane);
        const int brow = NSET == 1 ? 2 * (blk & 1) + ((blk >> 1) & 1)
                                   : 4 * (blk & 1) + 2 * ((blk >> 1) & 1) + ((blk >> 2) & 1);
        const bool emit = brow < BATCH && (blk >> (NSET == 1 ? 2 : 3)) == 0;   // one of the lanes that hold this total
        const int n = g * 4 + j;
        float y = 0.0f;
        if (emit) y = __fmul_rn(__fmul_rn(float(tot), sxs[brow]), a.wscale[n]);
        if (a.epi == SCMX_EPI_SWIGLU) {   // rows (g, g, u, u): lanes j = 0, 1 pair with j + 2
            const float yb = round_bf16(y);
            const float up = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(yb), 0x4E, 0xF, 0xF, false));
            if (emit && j < 2) a.out[size_t(brow) * (N / 2) + (g * 4) / 2 + j] = swiglu_bf16(yb, up);
        } else if (emit) {
            const size_t o = size_t(brow) * N + n;
            if (a.epi == SCMX_EPI_SCALE) a.out[o] = f32_to_bf16(y);
            else a.out[o] = f32_to_bf16(__fadd_rn(bf16_to_f32(a.res[o]), round_bf16(y)));
        }
    };

    const auto advance = [&](int& gi, int& cidx) {
        if (++cidx == CI) {
            cidx = 0;
            gi += g_stride;
        }
    };
    Item buf[2];
    int gq[2], cq[2];
    gq[0] = blockIdx.x * (NT / 64) + wave;
    cq[0] = 0;
    gq[1] = gq[0];
    cq[1] = 0;
    advance(gq[1], cq[1]);
#pragma unroll
    for (int i = 0; i < 2; ++i)
        if (gq[i] < groups) load_item(buf[i], gq[i], cq[i]);
    const WavePre<1> xpre = {};   // (no early request here: the extra registers would cost this kernel a wave of occupancy)

    for (int b = wave; b < XR; b += NT / 64) {   // a wave per activation row, side by side (rows beyond the batch are zero)
        if (b < BATCH) {
            const float s = stage_row_wave<X_PLAIN8>(a, b, sx + size_t(b) * Kp, xpre, false);
            for (int c = K / 4 + lane; c < Kp / 4; c += 64) reinterpret_cast<uint32_t*>(sx + size_t(b) * Kp)[c] = 0u;
            if (lane == 0) sxs[b] = s;
        } else {
            for (int c = lane; c < Kp / 4; c += 64) reinterpret_cast<uint32_t*>(sx + size_t(b) * Kp)[c] = 0u;
        }
    }
    __syncthreads();
    if (gq[0] >= groups) return;
#pragma unroll
    for (int s = 0; s < NSET; ++s) acc[s] = acc2[s] = v4i{0, 0, 0, 0};
    bool more = true;
    while (more) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            if (gq[i] >= groups) {
                more = false;
                break;
            }
            compute_item(buf[i], cq[i]);
            if (cq[i] == CI - 1) {
                finish(gq[i]);
#pragma unroll
                for (int s = 0; s < NSET; ++s) acc[s] = acc2[s] = v4i{0, 0, 0, 0};
            }
            gq[i] = gq[1 - i];
            cq[i] = cq[1 - i];
            advance(gq[i], cq[i]);
            if (gq[i] < groups) load_item(buf[i], gq[i], cq[i]);
        }
    }
}

// Wide layers in the published format, any batch up to 8: the dot products as half-precision MFMAs.
// v_cvt_scalef32_pk_f16_fp4 turns a code word into four half-precision pairs, sign and block scale included, which IS the
// 8-value operand of v_mfma_f32_16x16x32_f16; the activations sit in LDS as half precision (integers up to 127).  Every
// product is an integer below 2^14 and an accumulator is converted to INT32 and cleared before its sum can reach 2^24
// (at most 16 MFMAs x 32 products of at most 127 * 96 per chain between two conversions), so the FP32 sums are exact and
// the totals are the GEMM's INT32 accumulators.  A wave owns 16 consecutive weight rows: lane (row r = l % 16, group
// c = l / 16) loads 16 bytes of codes (one 32-weight block) per load, load i of a 512-wide piece of K covering
// k = 128 i + 32 c .. + 31, and feeds each of its four code words to one MFMA whose other operand is the activations of
// the same 8 k (lane column l % 16 = batch row, columns beyond the batch repeat row 0 and are never stored).  The MFMA
// sums over the four lane groups, so no cross-lane reduction is left: lane (column b, group c) ends with the totals of
// batch row b and weight rows 4 c .. 4 c + 3, which is also the unit of the SwiGLU epilogue.
// Per 8 weights and lane: 4 conversions, one 16-byte LDS read, one MFMA.
typedef float f4 __attribute__((ext_vector_type(4)));
// SPLIT (narrow layers): one row group per workgroup, the waves take the 512-wide pieces of K in turn (wave, wave + 4, ...)
// and their INT32 partial totals meet in LDS: the layer's few rows are spread over 4 x N / 16 waves with one or a few
// pieces each instead of N / 16 waves walking all of K.
// E8: a standard MXFP4 tensor in place -- the piece's 16 blocks bring 16 E8M0 bytes per row instead of 4 code bytes.
template <int BATCH, int POL, bool SPLIT, int WAVE_PRE, bool E8 = false>
__global__ __launch_bounds__(256, (E8 && WAVE_PRE <= 4) ? 4 : 1) void gemv_hmfma_kernel(const GemvArgs a) {
    constexpr int NT = 256;
    extern __shared__ __attribute__((aligned(16))) int8_t smem[];
    const int K = a.K, N = a.N;
    const int Kp = (K + 511) & ~511;                  // whole pieces of 512, zero padded
    const int pitch = Kp * 2 + 16;                     // bytes per staged row: the 16 spreads the batch rows over the banks
    int8_t* sx = smem;
    float* red = reinterpret_cast<float*>(smem + size_t(BATCH) * pitch);   // 68 floats + BATCH scales
    float* sxs = red + 68;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, c = lane >> 4;
    // Codes are loaded coalesced (an instruction reads 256 contiguous bytes of each of 4 rows) and turned into the MFMA
    // layout (lane = row, four lanes per row) through a wave-private LDS slot of 16 rows x 256 bytes; rows are 272 bytes
    // apart so that the 16 rows a read pass touches fall into different banks.
    constexpr int WPITCH = 272;
    int8_t* slot = reinterpret_cast<int8_t*>(sxs + ((BATCH + 3) & ~3)) + size_t(wave) * 16 * WPITCH;
    const int groups = N / 16;
    const int CI = Kp / 512;                           // pieces per row group
    const int g_stride = gridDim.x * (NT / 64);
    const int brow = r < BATCH ? r : 0;                // the batch row this lane's MFMA column reads
    // E8, wide layers (E8T; at least 3 pieces per row group): a row group's exponent bytes, 16 rows x K / 32, are at most
    // 1 KiB -- ONE wave-wide 16-byte load per row group instead of a strided 4-byte load per piece (whose 16 cache lines per
    // instruction cost the batch-4 output head a quarter of its rate).  They wait in registers (`e8n`) until the group's
    // first piece is multiplied, then sit in a wave-private LDS tile of 16 rows x 80 bytes (conflict-free 4-byte reads).
    constexpr bool E8T = E8 && !SPLIT;
    constexpr int EPITCH = 80;
    int8_t* e8tile = reinterpret_cast<int8_t*>(sxs + ((BATCH + 3) & ~3)) + size_t(NT / 64) * 16 * WPITCH + size_t(wave) * 16 * EPITCH;
    [[maybe_unused]] u32x4 e8n = u32x4{0u, 0u, 0u, 0u};
    [[maybe_unused]] uint32_t rmin_next = 0, rmin_cur = 0;

    struct Item {
        u32x4 w[4];     // loads i = 0..3 of the piece: the 32-weight block 4 i + c of row r
        uint32_t bc;    // the piece's four block-code bytes of row r (byte i: blocks 4 i .. 4 i + 3)
        uint32_t rmin;  // E8: the row's lowest exponent byte (bc then holds the exponent bytes of blocks 4 c .. 4 c + 3)
    };
    const auto load_item = [&](Item& it, int g, int ci) {
        const uint8_t* crow = reinterpret_cast<const uint8_t*>(a.codes) + size_t(g) * 16 * (K / 2);   // uniform
        const uint8_t* brw = a.bcodes + size_t(g) * 16 * a.bc_row_bytes;
        const __amdgpu_buffer_rsrc_t rc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(crow), 0, 16 * (K / 2), 0x00020000);
        const __amdgpu_buffer_rsrc_t rb =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(brw), 0, 16 * a.bc_row_bytes, 0x00020000);
#pragma unroll
        for (int i = 0; i < 4; ++i)   // rows 4 i .. 4 i + 3: lane l reads 16 bytes at byte 16 (l % 16) of row 4 i + l / 16
            it.w[i] = __builtin_amdgcn_raw_buffer_load_b128(rc, (4 * i + c) * (K / 2) + 16 * r, ci * 256, POL);
        if constexpr (E8T) {
            if (ci == 0) {   // the first piece of a row group brings the group's exponent bytes and lowest exponents
                e8n = __builtin_amdgcn_raw_buffer_load_b128(rb, r * a.bc_row_bytes + 16 * c, 0, 0);
                rmin_next = e8m0_row_min(a.wscale[size_t(g) * 16 + r]);
            }
        } else if constexpr (E8) {
            it.bc = __builtin_amdgcn_raw_buffer_load_b32(rb, r * a.bc_row_bytes + 4 * c, ci * 16, 0);
            it.rmin = e8m0_row_min(a.wscale[size_t(g) * 16 + r]);
        } else {
            it.bc = __builtin_amdgcn_raw_buffer_load_b32(rb, r * a.bc_row_bytes, ci * 4, 0);
        }
    };
    f4 acc0, acc1;     // two chains: consecutive MFMAs do not wait for each other
    int tot[4];
    const auto flush = [&]() {
#pragma unroll
        for (int i = 0; i < 4; ++i) tot[i] += int(acc0[i]) + int(acc1[i]);
        acc0 = acc1 = f4{0.0f, 0.0f, 0.0f, 0.0f};
    };
    // Which of the piece's 16 blocks a lane multiplies is free (the MFMA sums over the four lane groups): group c takes
    // blocks 4 i + c, or with E8M0 bytes blocks 4 c + i, whose four exponent bytes are one aligned 4-byte load.
    const auto compute_item = [&](const Item& it, int ci) {
        const int8_t* xrow = sx + size_t(brow) * pitch + (size_t(ci) * 512 + (E8 ? 128 : 32) * c) * 2;
#pragma unroll
        for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(slot + (4 * i + c) * WPITCH + 16 * r) = it.w[i];
        u32x4 wt[4];   // row r, blocks 4 i + c (E8: 4 c + i): bytes 64 i + 16 c (64 c + 16 i) of the row's 256
#pragma unroll
        for (int i = 0; i < 4; ++i)
            wt[i] = *reinterpret_cast<const u32x4*>(slot + r * WPITCH + (E8 ? 64 * c + 16 * i : 64 * i + 16 * c));
        uint32_t ebytes = it.bc, elow = it.rmin;
        if constexpr (E8T) {
            if (ci == 0) {
                *reinterpret_cast<u32x4*>(e8tile + r * EPITCH + 16 * c) = e8n;
                rmin_cur = rmin_next;
            }
            ebytes = *reinterpret_cast<const uint32_t*>(e8tile + r * EPITCH + 16 * ci + 4 * c);   // blocks 4 c .. 4 c + 3 of the piece
            elow = rmin_cur;
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float scale = E8 ? fp4_scale((((ebytes >> (8 * i)) & 0xFFu) - elow) & 0x7Fu)
                                   : fp4_scale((it.bc >> (8 * i + 2 * c)) & 3u);
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const uint32_t w = wt[i][d];
                const h2 q0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, scale, 0);
                const h2 q1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, scale, 1);
                const h2 q2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, scale, 2);
                const h2 q3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w, scale, 3);
                const h8 wv = h8{q0[0], q0[1], q1[0], q1[1], q2[0], q2[1], q3[0], q3[1]};
                const h8 xv = *reinterpret_cast<const h8*>(xrow + ((E8 ? 32 : 128) * i + 8 * d) * 2);
                if (d & 1) acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(wv, xv, acc1, 0, 0, 0);
                else acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(wv, xv, acc0, 0, 0, 0);
            }
        }
        flush();   // 8 MFMAs per chain and piece: far below the 43 that keep a chain exact
    };
    const auto finish = [&](int g) {
        if (r >= BATCH) return;
        const int n = g * 16 + 4 * c;
        const f4 ws = *reinterpret_cast<const f4*>(a.wscale + n);
        const float xs = sxs[r];
        float y[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) y[i] = __fmul_rn(__fmul_rn(float(tot[i]), xs), ws[i]);
        if (a.epi == SCMX_EPI_SWIGLU) {   // rows (g, g, u, u)
            const uint16_t o0 = swiglu_bf16(round_bf16(y[0]), round_bf16(y[2]));
            const uint16_t o1 = swiglu_bf16(round_bf16(y[1]), round_bf16(y[3]));
            *reinterpret_cast<uint32_t*>(a.out + size_t(r) * (N / 2) + n / 2) = uint32_t(o0) | (uint32_t(o1) << 16);
            return;
        }
        const size_t o = size_t(r) * N + n;
        if (a.epi == SCMX_EPI_RES) {
            const u32x2 rr = *reinterpret_cast<const u32x2*>(a.res + o);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float rv = __uint_as_float(i & 1 ? (rr[i >> 1] & 0xFFFF0000u) : (rr[i >> 1] << 16));
                y[i] = __fadd_rn(rv, round_bf16(y[i]));
            }
        }
        *reinterpret_cast<u32x2*>(a.out + o) = u32x2{uint32_t(f32_to_bf16(y[0])) | (uint32_t(f32_to_bf16(y[1])) << 16),
                                                      uint32_t(f32_to_bf16(y[2])) | (uint32_t(f32_to_bf16(y[3])) << 16)};
    };

    const auto advance = [&](int& gi, int& cidx) {
        if (SPLIT) {
            cidx += NT / 64;
            if (cidx >= CI) gi = groups;   // this wave's pieces are done
        } else if (++cidx == CI) {
            cidx = 0;
            gi += g_stride;
        }
    };
    constexpr int NB = 3;   // pieces in flight per wave: 3 x 4 KiB
    Item buf[NB];
    int gq[NB], cq[NB];
    gq[0] = SPLIT ? (wave < CI ? int(blockIdx.x) : groups) : int(blockIdx.x * (NT / 64) + wave);
    cq[0] = SPLIT ? wave : 0;
#pragma unroll
    for (int i = 1; i < NB; ++i) {
        gq[i] = gq[i - 1];
        cq[i] = cq[i - 1];
        advance(gq[i], cq[i]);
    }
    // activations are requested before the weights: memory returns a wave's loads in order
    u32x4 xpre1 = u32x4{0u, 0u, 0u, 0u};
    constexpr int RPW = BATCH > 4 ? 2 : 1;   // activation rows per wave
    WavePre<WAVE_PRE> xpre[RPW];
    bool have_pre = false;
    if (BATCH == 1) {
        have_pre = block_prefetch_row<NT>(a, 0, xpre1);
    } else {
#pragma unroll
        for (int j = 0; j < RPW; ++j) have_pre = wave_prefetch_row(a, wave + 4 * j, wave + 4 * j < BATCH, xpre[j]);
        have_pre = a.pro == 1 && a.K <= 512 * WAVE_PRE;
    }
#pragma unroll
    for (int i = 0; i < NB; ++i)
        if (gq[i] < groups) load_item(buf[i], gq[i], cq[i]);

    if (BATCH == 1) {   // one row: the whole workgroup stages it
        const float s = stage_row<NT, X_HALF>(a, 0, sx, red, xpre1, have_pre);
        for (int i = K / 2 + tid; i < Kp / 2; i += NT) reinterpret_cast<uint32_t*>(sx)[i] = 0u;
        if (tid == 0) sxs[0] = s;
    } else {            // several rows: a wave per row, side by side
#pragma unroll
        for (int j = 0; j < RPW; ++j) {
            const int b = wave + 4 * j;
            if (b >= BATCH) break;
            const float s = stage_row_wave<X_HALF>(a, b, sx + size_t(b) * pitch, xpre[j], have_pre);
            for (int i = K / 2 + lane; i < Kp / 2; i += 64) reinterpret_cast<uint32_t*>(sx + size_t(b) * pitch)[i] = 0u;
            if (lane == 0) sxs[b] = s;
        }
    }
    __syncthreads();
    if (!SPLIT && gq[0] >= groups) return;
    acc0 = acc1 = f4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int i = 0; i < 4; ++i) tot[i] = 0;
    bool more = true;
    while (more) {
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            if (gq[i] >= groups) {
                more = false;
                break;
            }
            compute_item(buf[i], cq[i]);
            if (!SPLIT && cq[i] == CI - 1) {
                finish(gq[i]);
#pragma unroll
                for (int v = 0; v < 4; ++v) tot[v] = 0;
            }
            gq[i] = gq[(i + NB - 1) % NB];
            cq[i] = cq[(i + NB - 1) % NB];
            advance(gq[i], cq[i]);
            if (gq[i] < groups) load_item(buf[i], gq[i], cq[i]);
        }
    }
    if constexpr (SPLIT) {   // every wave of the workgroup arrives here: partial totals through the waves' LDS slots
        *reinterpret_cast<v4i*>(slot + 16 * lane) = v4i{tot[0], tot[1], tot[2], tot[3]};
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int w = 1; w < NT / 64; ++w) {
                const v4i o = *reinterpret_cast<const v4i*>(slot + size_t(w) * 16 * WPITCH + 16 * lane);
#pragma unroll
                for (int i = 0; i < 4; ++i) tot[i] += o[i];
            }
            finish(blockIdx.x);
        }
    }
}

template <int BATCH, int R>
static void launch_gemv(const GemvArgs& a, int slots, int dflt, hipStream_t s) {
    // enough workgroups to fill the chip (4 waves each), but no more than the ~24 waves per CU that can be resident:
    // waves loop
    const int groups = a.N / R;
    const int want = (groups + 3) / 4;
    const int cap = max(1, 1536 / slots);
    const int rounds = (want + cap - 1) / cap;                      // row groups each wave walks through
    const dim3 grid((want + rounds - 1) / rounds, slots), block(256);   // ... the same number for every wave
    // one activation row: the FP4-conversion path (activations staged as half precision) is the faster one; with
    // more rows sharing the weight stream its extra LDS reads cost more than the integer dot products
    // dflt: 1 = the published format, 2 = its 16-block variant (fast path for one activation row only), 0 = other
    // 3 = the 16-block family members with consecutive integer multipliers (likewise)
    // 4 = a standard MXFP4 tensor in place (E8M0 bytes; the FP4-conversion path whatever the batch)
    const int mode = dflt == 4 ? 5 : dflt == 1 ? (BATCH == 1 ? 2 : 1) : (dflt >= 2 && BATCH == 1) ? dflt + 1 : 0;
    const size_t smem = size_t(BATCH) * ((a.K + 2047) & ~2047) * (mode >= 2 ? 2 : 1) + (68 + BATCH) * sizeof(float);
    auto go = [&](auto kernel) {
        if (smem > 64 * 1024)
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(smem));
        kernel<<<grid, block, smem, s>>>(a);
    };
    // one activation row longer than a pass of the workgroup on a narrow layer: keep the whole row in registers (one trip
    // to memory for it instead of two; down_proj 2048 x 6144)
    const bool long_row = BATCH == 1 && R == 1 && a.pro != 0 && a.K > 2048 && a.K <= 6144;
    if (mode == 5 && long_row) go(gemv_kernel<BATCH, R, 5, (BATCH == 1 && R == 1) ? 3 : 1>);
    else if (mode == 5) go(gemv_kernel<BATCH, R, 5>);
    else if (mode == 2 && long_row) go(gemv_kernel<BATCH, R, 2, (BATCH == 1 && R == 1) ? 3 : 1>);
    else if (mode == 2) go(gemv_kernel<BATCH, R, 2>);
    else if (mode == 3) go(gemv_kernel<BATCH, R, 3>);
    else if (mode == 4) go(gemv_kernel<BATCH, R, 4>);
    else if (mode == 1) go(gemv_kernel<BATCH, R, 1>);
    else go(gemv_kernel<BATCH, R, 0>);
}

template <int BATCH>
static void launch_gemv_mfma(const GemvArgs& a, hipStream_t s) {
    const int groups = a.N / 4;
    const int want = (groups + 3) / 4;
    const int rounds = (want + 1279) / 1280;   // 5 waves per SIMD are resident
    const dim3 grid((want + rounds - 1) / rounds), block(256);
    const size_t smem = size_t(BATCH > 4 ? 8 : 4) * ((a.K + 2047) & ~2047) + (68 + BATCH) * sizeof(float);
    if (smem > 64 * 1024)
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(gemv_mfma_kernel<BATCH>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, int(smem));
    gemv_mfma_kernel<BATCH><<<grid, block, smem, s>>>(a);
}

template <int BATCH, bool E8 = false>
static void launch_gemv_hmfma(const GemvArgs& a, bool split, hipStream_t s) {
    const int groups = a.N / 16;
    const int want = (groups + 3) / 4;
    const int rounds = (want + 1535) / 1536;   // 6 waves per SIMD are resident
    const dim3 grid(split ? groups : (want + rounds - 1) / rounds), block(256);
    const size_t smem = size_t(BATCH) * (((a.K + 511) & ~511) * 2 + 16) + (68 + ((BATCH + 3) & ~3)) * sizeof(float) + 4 * 16 * 272 +
                        (E8 ? 4 * 16 * 80 : 0);
    auto go = [&](auto kernel) {
        if (smem > 64 * 1024)
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, int(smem));
        kernel<<<grid, block, smem, s>>>(a);
    };
    // the early request of the activation rows holds K / 512 chunks per lane: 4 for K <= 2048, 12 up to 6144
    if (!split) go(gemv_hmfma_kernel<BATCH, W_STREAM, false, 4, E8>);
    else if (a.K <= 2048) go(gemv_hmfma_kernel<BATCH, W_STREAM, true, 4, E8>);
    else go(gemv_hmfma_kernel<BATCH, W_STREAM, true, 12, E8>);
}

template <int BATCH>
static void launch_gemv_rows(const GemvArgs& a, int slots, int dflt, hipStream_t s) {
    // wide layers in the published format: half-precision MFMA dot products (whole row groups of 16, pieces of 512)
    // (several activation rows, K up to 2048: beyond that its half-precision activations cost too much LDS)
    if (BATCH > 1 && dflt == 4 && !a.eidx && a.N % 16 == 0 && a.K % 512 == 0 && a.K <= 8192 && size_t(BATCH) * a.K <= 32768 &&
        uintptr_t(a.bcodes) % 4 == 0) {   // the same two kernels reading E8M0 bytes (4 per lane and piece, one aligned load)
        // wide layers: the form that loads a row group's exponent bytes at once needs 3 pieces per group (K >= 1536)
        if (a.N >= HMFMA_MIN_ROWS && a.K <= 2048 && a.K >= 1536) return launch_gemv_hmfma<BATCH, true>(a, false, s);
        return launch_gemv_hmfma<BATCH, true>(a, true, s);
    }
    // (both half-precision MFMA kernels read a row's block codes of a piece with one 4-byte load: aligned codes only)
    const bool bc4 = uintptr_t(a.bcodes) % 4 == 0;
    if (BATCH > 1 && dflt == 1 && bc4 && !a.eidx && a.N % 16 == 0 && a.K % 512 == 0 && a.K <= 2048 && a.N >= HMFMA_MIN_ROWS)
        return launch_gemv_hmfma<BATCH>(a, false, s);
    // narrow layers with several activation rows: the same kernel with K split over the waves of a workgroup
    // (batch 1 measured no faster this way than with the per-row kernels: qkv 4.70 against 4.40 us, down 7.32 against 6.34)
    if (BATCH > 1 && dflt == 1 && bc4 && !a.eidx && a.N % 16 == 0 && a.K % 512 == 0 && a.K <= 8192 && a.N < HMFMA_MIN_ROWS &&
        size_t(BATCH) * a.K <= 32768)
        return launch_gemv_hmfma<BATCH>(a, true, s);
    if (BATCH > 1 && dflt == 1 && bc4 && !a.eidx && a.N % 4 == 0 && a.K % 512 == 0)
        return launch_gemv_mfma<BATCH>(a, s);
    // more rows per wave = more loads in flight per lane; fewer = more waves for narrow layers
    const long rows = long(a.N) * slots;
    constexpr int RMAX = BATCH == 1 ? 4 : BATCH == 2 ? 4 : BATCH == 4 ? 2 : 1;   // keeps several waves per SIMD resident
    if (a.epi == SCMX_EPI_SWIGLU) return launch_gemv<BATCH, 4>(a, slots, dflt, s);
    if (RMAX >= 4 && rows >= 16384 && a.N % 4 == 0) return launch_gemv<BATCH, RMAX >= 4 ? 4 : 1>(a, slots, dflt, s);
    if (RMAX >= 2 && rows >= 4096 && a.N % 2 == 0) return launch_gemv<BATCH, RMAX >= 2 ? 2 : 1>(a, slots, dflt, s);
    return launch_gemv<BATCH, 1>(a, slots, dflt, s);
}

}  // namespace scmx

using namespace scmx;

extern "C" int scmx_gemv(const scmx_format* fmt, const void* x, const float* xscale, const uint32_t* codes,
                         const uint8_t* bcodes, const float* wscale, const uint16_t* res, uint16_t* out, int epi,
                         int pro, const uint16_t* nw, float eps, int batch, int N, int K, const int32_t* eidx,
                         int n_eidx, int xstride, int shared_expert, void* stream) {
    DevFormat f;
    if (int rc = make_dev_format(fmt, &f)) return rc;
    if (!x || !codes || !bcodes || !wscale || !out || (pro == 0 && !xscale) || (pro == 2 && !nw) ||
        (epi == SCMX_EPI_RES && !res)) {
        set_error("gemv: null pointer argument");
        return SCMX_ERR_ARG;
    }
    if (epi < 1 || epi > 3 || pro < 0 || pro > 2) {
        set_error("gemv: epilogue %d / prologue %d unknown", epi, pro);
        return SCMX_ERR_ARG;
    }
    if (N <= 0 || N > (1 << 30) || K <= 0 || K > (1 << 20) || K % 128 || K % f.block || (K / f.block * f.bc_bits) % 8 ||
        (epi == SCMX_EPI_SWIGLU && N % 4)) {
        set_error("gemv: need N <= 2^30, K <= 2^20, K %% 128 == 0, whole block-code bytes per row, N %% 4 == 0 for SwiGLU (N=%d K=%d)", N, K);
        return SCMX_ERR_ARG;
    }
    if (pro == 2 && K > 16384) {   // the norm's sum of squares is formed from at most 64 partials of 256 values
        set_error("gemv: the RMSNorm prologue takes K <= 16384 (K=%d)", K);
        return SCMX_ERR_ARG;
    }
    if (uintptr_t(codes) % 16 || uintptr_t(x) % 16 || (pro == 2 && uintptr_t(nw) % 16)) {
        set_error("gemv: codes, x and nw must be 16-byte aligned");
        return SCMX_ERR_ARG;
    }
    int slots = 1;
    if (eidx) {
        if (batch != 1 || n_eidx < 0 || n_eidx > 65534 || (xstride != 0 && xstride != 1)) {
            set_error("gemv: the expert-gather form takes batch 1, at most 65534 slots, xstride 0 or 1");
            return SCMX_ERR_ARG;
        }
        slots = n_eidx + (shared_expert >= 0 ? 1 : 0);
        if (slots == 0) return SCMX_OK;
    }
    if (!(batch == 1 || batch == 2 || batch == 4 || batch == 8)) {
        set_error("gemv: batch %d not in {1,2,4,8}", batch);
        return SCMX_ERR_ARG;
    }
    if (size_t(batch) * ((K + 2047) & ~2047) * 2 + 80 * sizeof(float) > 160 * 1024) {
        set_error("gemv: batch * K = %zu activations exceed what one workgroup can stage (80 Ki)", size_t(batch) * K);
        return SCMX_ERR_ARG;
    }
    GemvArgs a = {};
    a.x = x; a.xscale = xscale; a.codes = codes; a.bcodes = bcodes; a.wscale = wscale; a.res = res; a.out = out;
    a.nw = nw; a.eps = eps; a.epi = epi; a.pro = pro; a.N = N; a.K = K;
    a.bc_row_bytes = K / f.block * f.bc_bits / 8;
    a.eidx = eidx; a.n_eidx = n_eidx; a.xstride = xstride; a.shared_expert = eidx ? shared_expert : -1;
    a.fmt = f;
    const int dflt = is_mxfp4_e8m0_format(f)    ? 4
                     : is_default_format(f)       ? 1
                     : is_pow2_block16_format(f)  ? 2
                     : is_block16_range_format(f) ? 3
                                                  : 0;
    hipStream_t s = (hipStream_t)stream;
    switch (batch) {
        case 1: launch_gemv_rows<1>(a, slots, dflt, s); break;
        case 2: launch_gemv_rows<2>(a, slots, dflt, s); break;
        case 4: launch_gemv_rows<4>(a, slots, dflt, s); break;
        default: launch_gemv_rows<8>(a, slots, dflt, s); break;
    }
    return check_launch("gemv");
}
