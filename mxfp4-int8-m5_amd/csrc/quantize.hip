// SC-MXFP4 weight quantizer on the device: float weights -> packed codes, block codes and row scales.
//
// Restates, in float64 exactly as the host procedure computes it, sim/mx_int8.py:39-109 (block exponent search,
// spread constraint, E2M1 rounding, INT8 embedding) followed by the packing of sim/make_testcase.py:26-44 and
// e2e/sc_format.py:93-111.  One workgroup quantizes one row; a lane holds one weight, a group of BLOCK lanes one
// block.
//
// Bit-exactness rests on three things: every quantity is a float64 (weights arrive as float32 or bf16, both exact
// in float64); scaling by block steps is a multiplication by a power of two (exact); and the squared error of a
// block is summed in the order of the host's pairwise reduction over BLOCK contiguous values: eight running sums
// r[j] = ((a[j] + a[8+j]) + a[16+j]) + a[24+j], then ((r0+r1)+(r2+r3)) + ((r4+r5)+(r6+r7)).  The candidate
// comparison is a strict "<" on those sums, so a different order could flip a near tie.
#include <climits>

#include "scmx_common.h"

namespace scmx {

constexpr int QNT = 256;
constexpr int MAX_SPREAD = 3;   // sim/mx_int8.py:18

__device__ __forceinline__ double pow2_f64(int e) { return __longlong_as_double((long long)(1023 + e) << 52); }

// Index of the E2M1 level nearest to |x| (saturating at 6); a midpoint goes to the lower level (sim/mx_int8.py:23-25).
__device__ __forceinline__ int e2m1_index(double x) {
    const double a = fmin(fabs(x), 6.0);
    return int(a > 0.25) + int(a > 0.75) + int(a > 1.25) + int(a > 1.75) + int(a > 2.5) + int(a > 3.5) + int(a > 5.0);
}
__device__ __forceinline__ double e2m1_level(int idx) {   // 0, .5, 1, 1.5, 2, 3, 4, 6
    return idx <= 4 ? 0.5 * idx : (idx == 5 ? 3.0 : (idx == 6 ? 4.0 : 6.0));
}

// Squared error of the block this lane belongs to when quantized at exponent e (sim/mx_int8.py:34-36), summed in the
// host's order; every lane of the block returns the same value.
template <int BLOCK>
__device__ __forceinline__ double block_sq_err(double b, int e) {
    const double x = b * pow2_f64(-e);
    const double lv = e2m1_level(e2m1_index(x));
    const double v = x < 0.0 ? -lv : lv;
    const double d = v * pow2_f64(e) - b;
    const double sq = d * d;
    double r = sq + __shfl_down(sq, 8, BLOCK);
    if (BLOCK == 32) {
        r = r + __shfl_down(sq, 16, BLOCK);
        r = r + __shfl_down(sq, 24, BLOCK);
    }
    r = r + __shfl_xor(r, 1, BLOCK);
    r = r + __shfl_xor(r, 2, BLOCK);
    r = r + __shfl_xor(r, 4, BLOCK);
    return __shfl(r, 0, BLOCK);
}

template <bool MAXOP>
__device__ __forceinline__ int wg_reduce(int v, int* red) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const int o = __shfl_xor(v, off, WAVE);
        v = MAXOP ? max(v, o) : min(v, o);
    }
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    int r = red[0];
#pragma unroll
    for (int i = 1; i < QNT / 64; ++i) r = MAXOP ? max(r, red[i]) : min(r, red[i]);
    return r;
}

template <int BLOCK, bool BF16>
__global__ __launch_bounds__(QNT) void quantize_sc_kernel(const void* __restrict__ w, uint32_t* __restrict__ codes,
                                                         uint8_t* __restrict__ bcodes, float* __restrict__ wscale,
                                                         int K) {
    extern __shared__ int s_e[];   // K / BLOCK block exponents, then 4 ints of reduction scratch
    const int nb = K / BLOCK;
    int* red = s_e + nb;
    const size_t row = blockIdx.x;
    const int tid = threadIdx.x;
    constexpr int EMPTY = INT_MIN;   // an all-zero block: the host's -inf
    auto weight = [&](int k) -> double {
        if (BF16) return double(bf16_to_f32(reinterpret_cast<const uint16_t*>(w)[row * K + k]));
        return double(reinterpret_cast<const float*>(w)[row * K + k]);
    };

    // ---- pass 1: exponent of every block (sim/mx_int8.py:39-65, rule "search") ------------------------------------
    // QNT is a multiple of BLOCK and K a multiple of BLOCK, so a block is entirely inside or outside the row.
    for (int k0 = 0; k0 < K; k0 += QNT) {
        const int k = k0 + tid;
        const bool in = k < K;
        const double b = in ? weight(k) : 0.0;
        double amax = fabs(b);
#pragma unroll
        for (int off = BLOCK / 2; off >= 1; off >>= 1) amax = fmax(amax, __shfl_xor(amax, off, BLOCK));
        // floor(log2 amax) of a float32-born value is its binary exponent
        const int e0 = amax > 0.0 ? int((__double_as_longlong(amax) >> 52) & 0x7FF) - 1023 - 2 : 0;
        double best = block_sq_err<BLOCK>(b, e0);
        int chosen = e0;
        double t = block_sq_err<BLOCK>(b, e0 - 1);
        if (t < best) {
            best = t;
            chosen = e0 - 1;
        }
        t = block_sq_err<BLOCK>(b, e0 + 1);
        if (t < best) chosen = e0 + 1;
        if (in && tid % BLOCK == 0) s_e[k / BLOCK] = amax > 0.0 ? chosen : EMPTY;
    }
    __syncthreads();

    // ---- row constraint (sim/mx_int8.py:68-81) and the row's lowest exponent (sim/mx_int8.py:92-109) ---------------
    int top = EMPTY;
    for (int i = tid; i < nb; i += QNT) top = max(top, s_e[i]);
    top = wg_reduce<true>(top, red);
    if (top == EMPTY) top = 0;   // all-zero row
    const int floor_e = top - MAX_SPREAD;
    int lo = INT_MAX;
    for (int i = tid; i < nb; i += QNT) lo = min(lo, max(s_e[i], floor_e));
    lo = wg_reduce<false>(lo, red);

    // ---- pass 2: codes (sim/make_testcase.py:36-39, e2e/sc_format.py:72-73) ---------------------------------------
    for (int k0 = 0; k0 < K; k0 += QNT) {
        const int k = k0 + tid;
        const bool in = k < K;
        uint32_t c = 0;
        if (in) {
            const int e = max(s_e[k / BLOCK], floor_e);
            const double x = weight(k) * pow2_f64(-e);
            const int idx = e2m1_index(x);
            c = uint32_t(idx) | ((x < 0.0 && idx > 0) ? 8u : 0u);
        }
        c <<= 4 * (tid & 7);
        c |= __shfl_xor(c, 1, 8);
        c |= __shfl_xor(c, 2, 8);
        c |= __shfl_xor(c, 4, 8);
        if (in && (tid & 7) == 0) codes[(row * K + k) >> 3] = c;
    }
    // block codes: shift = e - lo in 0..3, 2 bits each, four blocks per byte (e2e/sc_format.py:14)
    for (int j = tid; j < nb / 4; j += QNT) {
        uint32_t byte = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) byte |= uint32_t(max(s_e[4 * j + i], floor_e) - lo) << (2 * i);
        bcodes[row * (nb / 4) + j] = uint8_t(byte);
    }
    if (tid == 0) wscale[row] = float(pow2_f64(lo - 1));   // 2^(E_lo - 1), sim/mx_int8.py:101
}

// ---- the integer-exact format family: w = base[row] * mult[block] * sign * code ------------------------------------
// Restates sim/formats.py:64-107 in float32, as the host computes it: the largest row base is
// peak / (largest multiplier * largest code); 8 bases per octave below it are tried in descending order, each with
// the per-block multiplier of least squared error (first minimum), and a candidate replaces the best so far only
// when its total error over the row is strictly smaller.  Block errors and row totals are summed in the order of
// the host's pairwise reduction.  One workgroup per row, one lane per weight.
struct FamilyArgs {
    float cb[8];      // code magnitudes
    float cut[7];     // midpoints between neighbouring magnitudes
    float mult[16];
    int n_mult, bc_bits;
};

// numpy's pairwise sum of n contiguous float32 values (n <= 128: eight strided running sums, a fixed tree, then the
// n % 8 tail; longer inputs are split in two at a multiple of 8 below the middle).
__device__ float np_pairwise_sum(const float* a, int n) {
    if (n < 8) {
        float r = 0.0f;
        for (int i = 0; i < n; ++i) r = __fadd_rn(r, a[i]);
        return r;
    }
    if (n <= 128) {
        float r[8];
        for (int j = 0; j < 8; ++j) r[j] = a[j];
        int i = 8;
        for (; i < n - (n % 8); i += 8)
            for (int j = 0; j < 8; ++j) r[j] = __fadd_rn(r[j], a[i + j]);
        float res = __fadd_rn(__fadd_rn(__fadd_rn(r[0], r[1]), __fadd_rn(r[2], r[3])),
                              __fadd_rn(__fadd_rn(r[4], r[5]), __fadd_rn(r[6], r[7])));
        for (; i < n; ++i) res = __fadd_rn(res, a[i]);
        return res;
    }
    int n2 = n / 2;
    n2 -= n2 % 8;
    return __fadd_rn(np_pairwise_sum(a, n2), np_pairwise_sum(a + n2, n - n2));
}

__device__ __forceinline__ int family_index(const FamilyArgs& f, float x) {   // nearest code, ties to the lower one
    const float a = fminf(fabsf(x), f.cb[7]);
    int idx = 0;
#pragma unroll
    for (int i = 0; i < 7; ++i) idx += int(a > f.cut[i]);
    return idx;
}

template <int BLOCK, bool BF16>
__global__ __launch_bounds__(QNT) void quantize_family_kernel(const void* __restrict__ w, uint32_t* __restrict__ codes,
                                                             uint8_t* __restrict__ bcodes, float* __restrict__ wscale,
                                                             int K, const FamilyArgs f) {
    extern __shared__ float s_f[];   // 8 x nb block errors, 8 totals, 8 reduction slots, then 8 x nb multiplier indices
    const int nb = K / BLOCK;
    float* s_err = s_f;
    float* s_tot = s_f + 8 * nb;
    float* s_red = s_tot + 8;
    uint8_t* s_mi = reinterpret_cast<uint8_t*>(s_red + 8);
    __shared__ int s_best;
    const size_t row = blockIdx.x;
    const int tid = threadIdx.x;
    auto weight = [&](int k) -> float {
        if (BF16) return bf16_to_f32(reinterpret_cast<const uint16_t*>(w)[row * K + k]);
        return reinterpret_cast<const float*>(w)[row * K + k];
    };
    // row peak
    float peak = 0.0f;
    for (int k = tid; k < K; k += QNT) peak = fmaxf(peak, fabsf(weight(k)));
    peak = wave_max(peak);
    if ((tid & 63) == 0) s_red[tid >> 6] = peak;
    __syncthreads();
    peak = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
    if (peak == 0.0f) peak = 1.0f;
    const float top = __fdiv_rn(peak, __fmul_rn(f.mult[f.n_mult - 1], f.cb[7]));
    // 2^(-j/8) rounded to float32: the candidate ladder of one octave
    const float ladder[8] = {1.0f, 0.9170040488243103f, 0.8408964276313782f, 0.7711054086685181f, 0.7071067690849304f,
                             0.6484197974205017f, 0.5946035385131836f, 0.5452538728713989f};

    // ---- per candidate base and block: the best multiplier and its error ------------------------------------------
    for (int k0 = 0; k0 < K; k0 += QNT) {
        const int k = k0 + tid;
        const bool in = k < K;
        const float wv = in ? weight(k) : 0.0f;
#pragma unroll 1
        for (int j = 0; j < 8; ++j) {
            const float base = __fmul_rn(top, ladder[j]);
            float best = 0.0f;
            int best_i = 0;
            for (int i = 0; i < f.n_mult; ++i) {
                const float sc = __fmul_rn(base, f.mult[i]);
                const float x = __fdiv_rn(wv, sc);
                const float lv = f.cb[family_index(f, x)];
                const float v = x > 0.0f ? lv : (x < 0.0f ? -lv : 0.0f * lv);
                const float d = __fsub_rn(__fmul_rn(v, sc), wv);
                const float sq = __fmul_rn(d, d);
                float r = __fadd_rn(sq, __shfl_down(sq, 8, BLOCK));
                if (BLOCK == 32) {
                    r = __fadd_rn(r, __shfl_down(sq, 16, BLOCK));
                    r = __fadd_rn(r, __shfl_down(sq, 24, BLOCK));
                }
                r = __fadd_rn(r, __shfl_xor(r, 1, BLOCK));
                r = __fadd_rn(r, __shfl_xor(r, 2, BLOCK));
                r = __fadd_rn(r, __shfl_xor(r, 4, BLOCK));
                r = __shfl(r, 0, BLOCK);
                if (i == 0 || r < best) {
                    best = r;
                    best_i = i;
                }
            }
            if (in && tid % BLOCK == 0) {
                s_err[j * nb + k / BLOCK] = best;
                s_mi[j * nb + k / BLOCK] = uint8_t(best_i);
            }
        }
    }
    __syncthreads();
    if (tid < 8) s_tot[tid] = np_pairwise_sum(s_err + tid * nb, nb);
    __syncthreads();
    if (tid == 0) {
        float best = __builtin_inff();
        int bj = 0;
        for (int j = 0; j < 8; ++j)
            if (s_tot[j] < best) {
                best = s_tot[j];
                bj = j;
            }
        s_best = bj;
    }
    __syncthreads();
    const int bj = s_best;
    const float base = __fmul_rn(top, ladder[bj]);
    const bool dead = base == 0.0f;   // a vanishing row underflows its base: it is exactly zero (e2e/pack_format.py:55-58)

    // ---- codes ----------------------------------------------------------------------------------------------------
    for (int k0 = 0; k0 < K; k0 += QNT) {
        const int k = k0 + tid;
        const bool in = k < K;
        uint32_t c = 0;
        if (in && !dead) {
            const float sc = __fmul_rn(base, f.mult[s_mi[bj * nb + k / BLOCK]]);
            const float x = __fdiv_rn(weight(k), sc);
            const int idx = family_index(f, x);
            c = uint32_t(idx) | ((x < 0.0f && f.cb[idx] > 0.0f) ? 8u : 0u);
        }
        c <<= 4 * (tid & 7);
        c |= __shfl_xor(c, 1, 8);
        c |= __shfl_xor(c, 2, 8);
        c |= __shfl_xor(c, 4, 8);
        if (in && (tid & 7) == 0) codes[(row * K + k) >> 3] = c;
    }
    // block codes: index into the multiplier table, bc_bits each (e2e/sc_format.py:14); a dead row takes multiplier 1
    const int per_byte = 8 / f.bc_bits;
    int one = 0;
    for (int i = 0; i < f.n_mult; ++i)
        if (f.mult[i] == 1.0f) one = i;
    for (int b = tid; b < nb / per_byte; b += QNT) {
        uint32_t byte = 0;
        for (int i = 0; i < per_byte; ++i)
            byte |= uint32_t(dead ? one : s_mi[bj * nb + b * per_byte + i]) << (f.bc_bits * i);
        bcodes[row * (nb / per_byte) + b] = uint8_t(byte);
    }
    if (tid == 0) wscale[row] = base;
}

}  // namespace scmx

using namespace scmx;

extern "C" int scmx_quantize_family(const scmx_format* fmt, const void* w, int w_is_bf16, int64_t N, int K,
                                    uint32_t* codes, uint8_t* bcodes, float* wscale, void* stream) {
    DevFormat df;
    if (int rc = make_dev_format(fmt, &df)) return rc;
    if (!w || !codes || !bcodes || !wscale || N < 0 || N > 0x7FFFFFFF || K <= 0) {
        set_error("quantize_family: null pointer or bad shape (N=%lld K=%d)", (long long)N, K);
        return SCMX_ERR_ARG;
    }
    const int block = fmt->block, per_byte = 8 / fmt->bc_bits;
    if ((block != 16 && block != 32) || K % (block * per_byte) || K > 16384) {
        set_error("quantize_family: block must be 16 or 32 and K a multiple of %d blocks, at most 16384 (block=%d K=%d)",
                  per_byte, block, K);
        return SCMX_ERR_ARG;
    }
    FamilyArgs f = {};
    for (int i = 0; i < 8; ++i) f.cb[i] = float(fmt->code_mag[i]);
    for (int i = 0; i < 7; ++i) {
        if (fmt->code_mag[i + 1] < fmt->code_mag[i]) {
            set_error("quantize_family: code magnitudes must ascend");
            return SCMX_ERR_FORMAT;
        }
        f.cut[i] = (f.cb[i + 1] + f.cb[i]) / 2.0f;
    }
    for (int i = 0; i < fmt->n_mult; ++i) {
        if (i && fmt->mult[i] <= fmt->mult[i - 1]) {
            set_error("quantize_family: block multipliers must ascend");
            return SCMX_ERR_FORMAT;
        }
        f.mult[i] = float(fmt->mult[i]);
    }
    f.n_mult = fmt->n_mult;
    f.bc_bits = fmt->bc_bits;
    if (N == 0) return SCMX_OK;
    const int nb = K / block;
    const size_t smem = size_t(8 * nb + 16) * sizeof(float) + size_t(8 * nb);
    const dim3 grid((unsigned)N), wg(QNT);
    hipStream_t st = (hipStream_t)stream;
    if (block == 32) {
        if (w_is_bf16) quantize_family_kernel<32, true><<<grid, wg, smem, st>>>(w, codes, bcodes, wscale, K, f);
        else quantize_family_kernel<32, false><<<grid, wg, smem, st>>>(w, codes, bcodes, wscale, K, f);
    } else {
        if (w_is_bf16) quantize_family_kernel<16, true><<<grid, wg, smem, st>>>(w, codes, bcodes, wscale, K, f);
        else quantize_family_kernel<16, false><<<grid, wg, smem, st>>>(w, codes, bcodes, wscale, K, f);
    }
    return check_launch("quantize_family");
}

extern "C" int scmx_quantize_sc(const void* w, int w_is_bf16, int64_t N, int K, int block, uint32_t* codes,
                                uint8_t* bcodes, float* wscale, void* stream) {
    if (!w || !codes || !bcodes || !wscale || N < 0 || K <= 0) {
        set_error("quantize_sc: null pointer or bad shape (N=%lld K=%d)", (long long)N, K);
        return SCMX_ERR_ARG;
    }
    if ((block != 16 && block != 32) || K % (4 * block) || K > 131072) {
        set_error("quantize_sc: block must be 16 or 32 and K a multiple of 4 blocks, at most 131072 (block=%d K=%d)",
                  block, K);
        return SCMX_ERR_ARG;
    }
    if (N > 0x7FFFFFFF) {
        set_error("quantize_sc: more than 2^31 - 1 rows");
        return SCMX_ERR_ARG;
    }
    if (N == 0) return SCMX_OK;
    const dim3 grid((unsigned)N), wg(QNT);
    const size_t smem = (size_t(K / block) + 4) * sizeof(int);
    hipStream_t st = (hipStream_t)stream;
    if (block == 32) {
        if (w_is_bf16) quantize_sc_kernel<32, true><<<grid, wg, smem, st>>>(w, codes, bcodes, wscale, K);
        else quantize_sc_kernel<32, false><<<grid, wg, smem, st>>>(w, codes, bcodes, wscale, K);
    } else {
        if (w_is_bf16) quantize_sc_kernel<16, true><<<grid, wg, smem, st>>>(w, codes, bcodes, wscale, K);
        else quantize_sc_kernel<16, false><<<grid, wg, smem, st>>>(w, codes, bcodes, wscale, K);
    }
    return check_launch("quantize_sc");
}
