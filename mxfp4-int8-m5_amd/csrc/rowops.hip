// Row kernels around the GEMMs (memory-bound, one workgroup per token row): RMSNorm + INT8 quantization, residual
// epilogue, SwiGLU + quantization, the q/k/v splits with head norms, the MoE token sort and the weighted combine.
//
// Reduction order (fixed, so results do not depend on the launch shape): a row's sum of squares is formed by K/4
// virtual threads of 4 consecutive values summed in order, 64 virtual threads per butterfly wave sum, and one more
// butterfly over the per-group partials.
#include <type_traits>

#include "scmx_common.h"

namespace scmx {

constexpr int NT = 256;

// 1 / sqrt(mean(x^2) + eps) of a bf16 row; every thread of the workgroup calls it.  red: >= 65 floats of LDS.
__device__ float block_inv_rms(const uint16_t* xr, int K, float eps, float* red) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int groups = (K / 4 + 63) / 64;
    for (int g = wave; g < groups; g += NT / 64) {
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
        const float tot = wave_sum(lane < groups ? red[lane] : 0.0f);
        if (lane == 0) red[64] = __fdiv_rn(1.0f, sqrtf(__fadd_rn(__fdiv_rn(tot, float(K)), eps)));
    }
    __syncthreads();
    const float inv = red[64];
    __syncthreads();
    return inv;
}

// Per-token INT8 of a row given as bf16 bit patterns in memory (global or LDS): codes to qrow, scale to *xs.
__device__ void block_quant_row(const uint16_t* v, int K, int8_t* qrow, float* xs, float* red) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float amax = 0.0f;
    for (int c = tid; c < K / 4; c += NT) {
        const u32x2 p = *reinterpret_cast<const u32x2*>(v + 4 * c);
        amax = fmaxf(amax, fabsf(__uint_as_float(p[0] << 16)));
        amax = fmaxf(amax, fabsf(__uint_as_float(p[0] & 0xFFFF0000u)));
        amax = fmaxf(amax, fabsf(__uint_as_float(p[1] << 16)));
        amax = fmaxf(amax, fabsf(__uint_as_float(p[1] & 0xFFFF0000u)));
    }
    amax = wave_max(amax);
    if (lane == 0) red[wave] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float s = __fdiv_rn(amax, 127.0f);
    const float qi = s > 0.0f ? __fdiv_rn(1.0f, s) : 0.0f;
    for (int c = tid; c < K / 4; c += NT) {
        const u32x2 p = *reinterpret_cast<const u32x2*>(v + 4 * c);
        const int q0 = quant_code(__uint_as_float(p[0] << 16), qi), q1 = quant_code(__uint_as_float(p[0] & 0xFFFF0000u), qi);
        const int q2 = quant_code(__uint_as_float(p[1] << 16), qi), q3 = quant_code(__uint_as_float(p[1] & 0xFFFF0000u), qi);
        *reinterpret_cast<uint32_t*>(qrow + 4 * c) = (uint32_t(q0) & 0xFFu) | ((uint32_t(q1) & 0xFFu) << 8) |
                                                     ((uint32_t(q2) & 0xFFu) << 16) | ((uint32_t(q3) & 0xFFu) << 24);
    }
    if (tid == 0) *xs = s;
    __syncthreads();
}

__device__ void block_zero_row(int8_t* qrow, float* xs, uint16_t* xn, int K) {
    for (int c = threadIdx.x; c < K / 4; c += NT) {
        *reinterpret_cast<uint32_t*>(qrow + 4 * c) = 0u;
        if (xn) *reinterpret_cast<u32x2*>(xn + 4 * c) = u32x2{0u, 0u};
    }
    if (threadIdx.x == 0) *xs = 0.0f;
}

// y = bf16(w * bf16(x * inv)) for a row, written as bf16 bits to `dst` (LDS) and optionally to xn (global).
__device__ void block_norm_row(const uint16_t* xr, const uint16_t* w, float inv, uint16_t* dst, uint16_t* xn, int K) {
    for (int c = threadIdx.x; c < K / 4; c += NT) {
        const u32x2 p = *reinterpret_cast<const u32x2*>(xr + 4 * c);
        const u32x2 q = *reinterpret_cast<const u32x2*>(w + 4 * c);
        uint16_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float xv = __uint_as_float(i & 1 ? (p[i >> 1] & 0xFFFF0000u) : (p[i >> 1] << 16));
            const float wv = __uint_as_float(i & 1 ? (q[i >> 1] & 0xFFFF0000u) : (q[i >> 1] << 16));
            o[i] = f32_to_bf16(__fmul_rn(wv, round_bf16(__fmul_rn(xv, inv))));
        }
        const u32x2 r = u32x2{uint32_t(o[0]) | (uint32_t(o[1]) << 16), uint32_t(o[2]) | (uint32_t(o[3]) << 16)};
        *reinterpret_cast<u32x2*>(dst + 4 * c) = r;
        if (xn) *reinterpret_cast<u32x2*>(xn + 4 * c) = r;
    }
    __syncthreads();
}

// ---- rmsnorm_quant(_n) -----------------------------------------------------------------------------------------
__global__ __launch_bounds__(NT) void rmsnorm_quant_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                                           float eps, int8_t* __restrict__ xq, float* __restrict__ xs,
                                                           uint16_t* __restrict__ xn, int M, int K) {
    extern __shared__ __attribute__((aligned(16))) uint16_t srow[];   // K bf16 + 72 floats
    float* red = reinterpret_cast<float*>(srow + K);
    const int row = blockIdx.x;
    int8_t* qrow = xq + size_t(row) * K;
    uint16_t* nrow = xn ? xn + size_t(row) * K : nullptr;
    if (row >= M) return block_zero_row(qrow, xs + row, nrow, K);
    const uint16_t* xr = x + size_t(row) * K;
    const float inv = block_inv_rms(xr, K, eps, red);
    block_norm_row(xr, w, inv, srow, nrow, K);
    block_quant_row(srow, K, qrow, xs + row, red);
}

// The same with the row in registers: one wave per row, lane l owns the 16-byte pieces l, l + 64, ... (CH of them,
// K = 512 * CH), four rows per workgroup, no LDS and no workgroup barrier.  The sum of squares is taken in the order of
// block_inv_rms, so both kernels give the same bits: there, thread (wave g, lane t) adds the squares of elements
// 256 g + 4 t .. + 3 in sequence, a butterfly over lane distances 32 ... 1 gives the sum of group g, and a second
// butterfly over the group sums (zeros beyond the last group) gives the total.  Here piece l + 64 j holds the
// elements of lanes 2 (l % 32) and 2 (l % 32) + 1 of group 2 j + l / 32: the two four-element sums stay apart through
// the butterfly over lane distances 16 ... 1 (= 32 ... 2 there) and are added last (= distance 1); lane l then picks
// up the sum of group l and the second butterfly runs as it does there.
// BLK: xq leaves in the blocked layout of the dense GEMM (32 x 32 blocks in MFMA operand order, Mp % 32 == 0): eight
// rows per workgroup, whose codes meet in LDS -- the 16 bytes of row r, k 16 c ... at slot c * 8 + (r + c / 2) % 8 -- and
// are stored as whole 128-byte lines (8 rows x 16 bytes are adjacent in a block).  Same codes and scales.
template <int CH, bool BLK = false>
__global__ __launch_bounds__(BLK ? 512 : 256) void rmsnorm_quant_wave_kernel(const uint16_t* __restrict__ x,
                                                                             const uint16_t* __restrict__ w, float eps,
                                                                             int8_t* __restrict__ xq, float* __restrict__ xs,
                                                                             uint16_t* __restrict__ xn, int M, int Mp) {
    constexpr int K = 512 * CH, RPW = BLK ? 8 : 4;
    __shared__ u32x2 tile[BLK ? CH * 64 * 8 : 1];
    const int wid = threadIdx.x >> 6, row0 = blockIdx.x * RPW, row = row0 + wid, lane = threadIdx.x & 63;
    auto gather_store = [&]() {   // BLK: after every wave's codes are in LDS
        __syncthreads();
        int8_t* const blk = xq + (size_t(row0 >> 5) * size_t(K >> 5)) * 1024;
        const u32x4* t16 = reinterpret_cast<const u32x4*>(tile);
#pragma unroll
        for (int j = 0; j < CH / 2 + CH % 2; ++j) {   // K / 16 pieces x 8 rows of 16 bytes, 512 per pass
            const int idx = int(threadIdx.x) + 512 * j, c = idx >> 3, r = idx & 7;
            if (CH % 2 == 0 || c < K / 16)
                *reinterpret_cast<u32x4*>(blk + size_t(c >> 1) * 1024 + (c & 1) * 512 + ((row0 + r) & 31) * 16) =
                    t16[c * 8 + ((r + (c >> 1)) & 7)];
        }
    };
    // piece p (8 codes) of this wave's row: half p % 2 of the 16-byte slot of chunk p / 2
    auto slot = [&](int p) { return ((p >> 1) * 8 + ((wid + (p >> 2)) & 7)) * 2 + (p & 1); };
    if (!BLK && row >= Mp) return;
    u32x2* qrow = reinterpret_cast<u32x2*>(xq + size_t(row) * K);
    u32x4* nrow = xn ? reinterpret_cast<u32x4*>(xn + size_t(row) * K) : nullptr;
    if (row >= M) {
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            if (BLK) tile[slot(lane + 64 * j)] = u32x2{0u, 0u}; else qrow[lane + 64 * j] = u32x2{0u, 0u};
            if (nrow) nrow[lane + 64 * j] = u32x4{0u, 0u, 0u, 0u};
        }
        if (lane == 0) xs[row] = 0.0f;
        if (BLK) gather_store();
        return;
    }
    const u32x4* xrow = reinterpret_cast<const u32x4*>(x + size_t(row) * K);
    const u32x4* wrow = reinterpret_cast<const u32x4*>(w);
    u32x4 v[CH], wv[CH];
#pragma unroll
    for (int j = 0; j < CH; ++j) v[j] = xrow[lane + 64 * j];
#pragma unroll
    for (int j = 0; j < CH; ++j) wv[j] = wrow[lane + 64 * j];
    auto lo = [](uint32_t u) { return __uint_as_float(u << 16); };
    auto hi = [](uint32_t u) { return __uint_as_float(u & 0xFFFF0000u); };
    float r = 0.0f;   // lane l < 2 CH: the sum of group l
#pragma unroll
    for (int j = 0; j < CH; ++j) {
        float a = __fmul_rn(lo(v[j][0]), lo(v[j][0]));
        a = __fadd_rn(a, __fmul_rn(hi(v[j][0]), hi(v[j][0])));
        a = __fadd_rn(a, __fmul_rn(lo(v[j][1]), lo(v[j][1])));
        a = __fadd_rn(a, __fmul_rn(hi(v[j][1]), hi(v[j][1])));
        float b = __fmul_rn(lo(v[j][2]), lo(v[j][2]));
        b = __fadd_rn(b, __fmul_rn(hi(v[j][2]), hi(v[j][2])));
        b = __fadd_rn(b, __fmul_rn(lo(v[j][3]), lo(v[j][3])));
        b = __fadd_rn(b, __fmul_rn(hi(v[j][3]), hi(v[j][3])));
#pragma unroll
        for (int off = 16; off >= 1; off >>= 1) {
            a = __fadd_rn(a, __shfl_xor(a, off, WAVE));
            b = __fadd_rn(b, __shfl_xor(b, off, WAVE));
        }
        const float mine = __fadd_rn(a, b);                 // group 2 j + lane / 32
        const float other = __shfl_xor(mine, 32, WAVE);     // the other group of this j
        const float even = lane < 32 ? mine : other, odd = lane < 32 ? other : mine;
        if ((lane >> 1) == j) r = (lane & 1) ? odd : even;
    }
    const float tot = wave_sum(r);
    const float inv = __fdiv_rn(1.0f, sqrtf(__fadd_rn(__fdiv_rn(tot, float(K)), eps)));
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < CH; ++j) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float n0 = round_bf16(__fmul_rn(lo(wv[j][e]), round_bf16(__fmul_rn(lo(v[j][e]), inv))));
            const float n1 = round_bf16(__fmul_rn(hi(wv[j][e]), round_bf16(__fmul_rn(hi(v[j][e]), inv))));
            amax = fmaxf(amax, fmaxf(fabsf(n0), fabsf(n1)));
            v[j][e] = (__float_as_uint(n0) >> 16) | (__float_as_uint(n1) & 0xFFFF0000u);
        }
        if (nrow) nrow[lane + 64 * j] = v[j];
    }
    amax = wave_max(amax);
    const float s = __fdiv_rn(amax, 127.0f);
    const float qi = s > 0.0f ? __fdiv_rn(1.0f, s) : 0.0f;
#pragma unroll
    for (int j = 0; j < CH; ++j) {
        uint32_t o[2] = {0u, 0u};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int q0 = quant_code(lo(v[j][e]), qi);
            const int q1 = quant_code(hi(v[j][e]), qi);
            o[e >> 1] |= (uint32_t(q0) & 0xFFu) << (16 * (e & 1));
            o[e >> 1] |= (uint32_t(q1) & 0xFFu) << (16 * (e & 1) + 8);
        }
        if (BLK) tile[slot(lane + 64 * j)] = u32x2{o[0], o[1]}; else qrow[lane + 64 * j] = u32x2{o[0], o[1]};
    }
    if (lane == 0) xs[row] = s;
    if (BLK) gather_store();
}

// ---- res_norm_quant / res_epilogue -----------------------------------------------------------------------------
__global__ __launch_bounds__(NT) void res_norm_quant_kernel(const int32_t* __restrict__ acc, const float* __restrict__ xscale,
                                                            const float* __restrict__ wscale, const uint16_t* __restrict__ res,
                                                            const uint16_t* __restrict__ w, float eps, uint16_t* __restrict__ h,
                                                            int8_t* __restrict__ xq, float* __restrict__ xs, int K) {
    extern __shared__ __attribute__((aligned(16))) uint16_t srow[];   // 2 K bf16 + 72 floats
    uint16_t* hrow_s = srow;
    uint16_t* nrow_s = srow + K;
    float* red = reinterpret_cast<float*>(srow + 2 * K);
    const int row = blockIdx.x;
    const float xsr = xscale[row];
    for (int c = threadIdx.x; c < K / 4; c += NT) {
        const v4i a4 = *reinterpret_cast<const v4i*>(acc + size_t(row) * K + 4 * c);
        const f32x4 w4 = *reinterpret_cast<const f32x4*>(wscale + 4 * c);
        const u32x2 r2 = *reinterpret_cast<const u32x2*>(res + size_t(row) * K + 4 * c);
        uint16_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float y = round_bf16(__fmul_rn(__fmul_rn(float(a4[i]), xsr), w4[i]));
            const float rv = __uint_as_float(i & 1 ? (r2[i >> 1] & 0xFFFF0000u) : (r2[i >> 1] << 16));
            o[i] = f32_to_bf16(__fadd_rn(rv, y));
        }
        const u32x2 r = u32x2{uint32_t(o[0]) | (uint32_t(o[1]) << 16), uint32_t(o[2]) | (uint32_t(o[3]) << 16)};
        *reinterpret_cast<u32x2*>(hrow_s + 4 * c) = r;
        *reinterpret_cast<u32x2*>(h + size_t(row) * K + 4 * c) = r;
    }
    __syncthreads();
    if (!xq) return;
    const float inv = block_inv_rms(hrow_s, K, eps, red);
    block_norm_row(hrow_s, w, inv, nrow_s, nullptr, K);
    block_quant_row(nrow_s, K, xq + size_t(row) * K, xs + row, red);
}

// ---- swiglu_quant ----------------------------------------------------------------------------------------------
__global__ __launch_bounds__(NT) void swiglu_quant_kernel(const int32_t* __restrict__ acc, const float* __restrict__ xscale,
                                                          const float* __restrict__ wscale, int8_t* __restrict__ xq,
                                                          float* __restrict__ xs, int F,
                                                          const uint16_t* __restrict__ silu) {
    extern __shared__ __attribute__((aligned(16))) uint16_t srow[];   // F bf16 + 72 floats
    float* red = reinterpret_cast<float*>(srow + F);
    const int row = blockIdx.x;
    const float xsr = xscale[row];
    const int32_t* ar = acc + size_t(row) * 2 * F;
    for (int c = threadIdx.x; c < F / 4; c += NT) {
        const v4i g4 = *reinterpret_cast<const v4i*>(ar + 4 * c);
        const v4i u4 = *reinterpret_cast<const v4i*>(ar + F + 4 * c);
        const f32x4 wg = *reinterpret_cast<const f32x4*>(wscale + 4 * c);
        const f32x4 wu = *reinterpret_cast<const f32x4*>(wscale + F + 4 * c);
        uint16_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float g = __fmul_rn(__fmul_rn(float(g4[i]), xsr), wg[i]);
            const float u = round_bf16(__fmul_rn(__fmul_rn(float(u4[i]), xsr), wu[i]));
            o[i] = swiglu_lut(silu, g, u);   // table over the bf16 value of the gate
        }
        *reinterpret_cast<u32x2*>(srow + 4 * c) =
            u32x2{uint32_t(o[0]) | (uint32_t(o[1]) << 16), uint32_t(o[2]) | (uint32_t(o[3]) << 16)};
    }
    __syncthreads();
    block_quant_row(srow, F, xq + size_t(row) * F, xs + row, red);
}

// ---- Qwen3 q/k/v split with per-head RMSNorm: one wave per head, d/64 consecutive values per lane ---------------
// With inv_freq != NULL the kernel also rotates q and k (pairs (i, i + d/2) of a head, angle = position * inv_freq[i])
// and writes k and v at rows pos .. pos+L-1 of caches [hk, kv_rows, d] instead of dense [hk, L, d] outputs.
struct RopeArgs {
    const float* inv_freq;   // [d / 2] or NULL
    const int64_t* pos_dev;  // optional device-resident position of row 0 (read when non-NULL), else pos0
    int64_t pos0;
    int kv_rows;             // rows per head of the k / v destinations
    int q_token_major;       // q as [L, hq, d] instead of [hq, L, d]
};

__global__ __launch_bounds__(NT) void qkv_headnorm_kernel(const int32_t* __restrict__ acc, const float* __restrict__ xscale,
                                                          const float* __restrict__ wscale, const uint16_t* __restrict__ y,
                                                          const uint16_t* __restrict__ qn, const uint16_t* __restrict__ kn,
                                                          float eps, uint16_t* __restrict__ q, uint16_t* __restrict__ k,
                                                          uint16_t* __restrict__ v, int L, int hq, int hk, int d,
                                                          const RopeArgs rope) {
    const int row = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int heads = hq + 2 * hk, ntot = heads * d, per = d / 64;
    const int64_t pos = rope.inv_freq ? (rope.pos_dev ? rope.pos_dev[0] : rope.pos0) + row : row;
    const int kv_rows = rope.inv_freq ? rope.kv_rows : L;
    // the d / 2 rotation angles of this row are the same for every head: one sine / cosine each per workgroup
    __shared__ float s_sin[256], s_cos[256];
    if (rope.inv_freq) {
        for (int i = threadIdx.x; i < d / 2; i += NT) sincosf(float(pos) * rope.inv_freq[i], &s_sin[i], &s_cos[i]);
        __syncthreads();
    }
    // blockIdx.y strides over groups of NT / 64 heads (one per wave): a single row still fills many CUs.  A wave takes
    // its heads U at a time with all their loads issued first, so one memory latency covers U heads.
    constexpr int U = 4;
    const int stride = gridDim.y * (NT / 64);
    for (int g0 = blockIdx.y * (NT / 64) + wave; g0 < heads; g0 += U * stride) {
        float yv[U][8];   // per <= 8 (d <= 512)
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int g = g0 + u * stride;
            if (g >= heads) break;
            if (!acc && per == 2) {   // head dim 128: the lane's two values in one 32-bit load
                const uint32_t w = *reinterpret_cast<const uint32_t*>(y + size_t(row) * ntot + g * d + 2 * lane);
                yv[u][0] = __uint_as_float(w << 16);
                yv[u][1] = __uint_as_float(w & 0xFFFF0000u);
                continue;
            }
            for (int i = 0; i < per; ++i) {
                const int c = g * d + per * lane + i;
                if (acc)
                    yv[u][i] = round_bf16(__fmul_rn(__fmul_rn(float(acc[size_t(row) * ntot + c]), xscale[row]), wscale[c]));
                else
                    yv[u][i] = bf16_to_f32(y[size_t(row) * ntot + c]);
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int g = g0 + u * stride;
            if (g >= heads) break;
            float ss = 0.0f;
            for (int i = 0; i < per; ++i) ss = __fadd_rn(ss, __fmul_rn(yv[u][i], yv[u][i]));
            uint16_t* out;
            int hh;
            if (g < hq) { out = q; hh = g; } else if (g < hq + hk) { out = k; hh = g - hq; } else { out = v; hh = g - hq - hk; }
            uint16_t* o = g >= hq              ? out + (size_t(hh) * kv_rows + size_t(pos)) * d + per * lane
                          : rope.q_token_major ? out + (size_t(row) * hq + hh) * d + per * lane
                                               : out + (size_t(hh) * L + row) * d + per * lane;
            uint32_t pair = 0;   // per == 2: both results leave in one 32-bit store
            auto emit = [&](int i, uint16_t b) {
                if (per != 2) { o[i] = b; return; }
                pair |= uint32_t(b) << (16 * i);
                if (i == 1) *reinterpret_cast<uint32_t*>(o) = pair;
            };
            if (g < hq + hk) {
                head_norm_rope(yv[u], ss, per, lane, d, g < hq ? qn : kn, eps, rope.inv_freq ? s_sin : nullptr, s_cos, emit);
            } else {
                for (int i = 0; i < per; ++i) emit(i, f32_to_bf16(yv[u][i]));
            }
        }
    }
}

// The same for head dim 128 and bf16 input on many rows: sixteen lanes per head with eight consecutive values each
// (16-byte loads and stores, sixteen heads per pass of a workgroup) instead of a wave per head with two.  The sum of
// squares is taken in the order of the kernel above, so both give the same bits: that one adds the squares of values
// (2l, 2l + 1) in lane l and then runs a butterfly over lane distances 32, 16, 8, 4, 2, 1; here the lane keeps the four
// pair sums of its eight values apart through the butterfly over group-lane distances 8, 4, 2, 1 (= 32 ... 4 there) and
// joins them last, (p0 + p2) + (p1 + p3) (= distances 2 and 1).
__global__ __launch_bounds__(NT) void qkv_headnorm128_kernel(const uint16_t* __restrict__ y, const uint16_t* __restrict__ qn,
                                                             const uint16_t* __restrict__ kn, float eps,
                                                             uint16_t* __restrict__ q, uint16_t* __restrict__ k,
                                                             uint16_t* __restrict__ v, int L, int hq, int hk,
                                                             const RopeArgs rope) {
    constexpr int d = 128, U = 2, GROUPS = NT / 16;
    const int row = blockIdx.x, grp = threadIdx.x >> 4, j = threadIdx.x & 15;
    const int heads = hq + 2 * hk, ntot = heads * d;
    const int64_t pos = rope.inv_freq ? (rope.pos_dev ? rope.pos_dev[0] : rope.pos0) + row : row;
    const int kv_rows = rope.inv_freq ? rope.kv_rows : L;
    __shared__ float s_sin[d / 2], s_cos[d / 2];
    if (rope.inv_freq) {
        if (threadIdx.x < d / 2) sincosf(float(pos) * rope.inv_freq[threadIdx.x], &s_sin[threadIdx.x], &s_cos[threadIdx.x]);
        __syncthreads();
    }
    for (int g0 = grp; g0 < heads; g0 += U * GROUPS) {
        u32x4 raw[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int g = g0 + u * GROUPS;
            if (g < heads) raw[u] = *reinterpret_cast<const u32x4*>(y + size_t(row) * ntot + g * d + 8 * j);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int g = g0 + u * GROUPS;
            if (g >= heads) break;
            uint16_t* out;
            int hh;
            if (g < hq) { out = q; hh = g; } else if (g < hq + hk) { out = k; hh = g - hq; } else { out = v; hh = g - hq - hk; }
            uint16_t* o = g >= hq              ? out + (size_t(hh) * kv_rows + size_t(pos)) * d + 8 * j
                          : rope.q_token_major ? out + (size_t(row) * hq + hh) * d + 8 * j
                                               : out + (size_t(hh) * L + row) * d + 8 * j;
            if (g >= hq + hk) {   // v: as it is
                *reinterpret_cast<u32x4*>(o) = raw[u];
                continue;
            }
            float x[8], p[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                x[2 * i] = __uint_as_float(raw[u][i] << 16);
                x[2 * i + 1] = __uint_as_float(raw[u][i] & 0xFFFF0000u);
                p[i] = __fadd_rn(__fmul_rn(x[2 * i], x[2 * i]), __fmul_rn(x[2 * i + 1], x[2 * i + 1]));
            }
#pragma unroll
            for (int off = 8; off >= 1; off >>= 1)
#pragma unroll
                for (int i = 0; i < 4; ++i) p[i] = __fadd_rn(p[i], __shfl_xor(p[i], off, 16));
            const float ss = __fadd_rn(__fadd_rn(p[0], p[2]), __fadd_rn(p[1], p[3]));
            const float inv = __fdiv_rn(1.0f, sqrtf(__fadd_rn(__fdiv_rn(ss, float(d)), eps)));
            const u32x4 wr = *reinterpret_cast<const u32x4*>((g < hq ? qn : kn) + 8 * j);
            u32x4 res;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const float wv = __uint_as_float(i & 1 ? (wr[i >> 1] & 0xFFFF0000u) : (wr[i >> 1] << 16));
                float nv = round_bf16(__fmul_rn(wv, round_bf16(__fmul_rn(x[i], inv))));
                if (rope.inv_freq) {   // element 8 j + i pairs with the one 64 away, eight group lanes off
                    const float other = __shfl_xor(nv, 8, 16);
                    const int e = (8 * j + i) & 63;
                    nv = j < 8 ? __fsub_rn(__fmul_rn(nv, s_cos[e]), __fmul_rn(other, s_sin[e]))
                               : __fadd_rn(__fmul_rn(nv, s_cos[e]), __fmul_rn(other, s_sin[e]));
                }
                const uint32_t b = f32_to_bf16(nv);
                if (i & 1) res[i >> 1] |= b << 16; else res[i >> 1] = b;
            }
            *reinterpret_cast<u32x4*>(o) = res;
        }
    }
}

// ---- OLMoE q/k/v split with RMSNorm over the full h*d width ------------------------------------------------------
__global__ __launch_bounds__(NT) void qkv_fullnorm_kernel(const uint16_t* __restrict__ y, const uint16_t* __restrict__ qn,
                                                          const uint16_t* __restrict__ kn, float eps, uint16_t* __restrict__ q,
                                                          uint16_t* __restrict__ k, uint16_t* __restrict__ v, int L, int h,
                                                          int d) {
    extern __shared__ __attribute__((aligned(16))) uint16_t srow[];   // W bf16 + 72 floats
    const int W = h * d, row = blockIdx.x;
    float* red = reinterpret_cast<float*>(srow + W);
    for (int part = 0; part < 3; ++part) {
        const uint16_t* yr = y + size_t(row) * 3 * W + size_t(part) * W;
        uint16_t* out = part == 0 ? q : (part == 1 ? k : v);
        const uint16_t* src = yr;
        if (part < 2) {
            const float inv = block_inv_rms(yr, W, eps, red);
            block_norm_row(yr, part == 0 ? qn : kn, inv, srow, nullptr, W);
            src = srow;
        }
        for (int c = threadIdx.x; c < W / 4; c += NT) {
            const int col = 4 * c, hh = col / d, dd = col % d;
            *reinterpret_cast<u32x2*>(out + (size_t(hh) * L + row) * d + dd) = *reinterpret_cast<const u32x2*>(src + col);
        }
        __syncthreads();
    }
}

// ---- MoE: counting sort of the token-expert assignments, one workgroup ------------------------------------------
__global__ __launch_bounds__(1024) void route_sort_kernel(const int32_t* __restrict__ inds, int R, int topk, int E, int tm,
                                                          int32_t* __restrict__ pos, int32_t* __restrict__ tok,
                                                          int32_t* __restrict__ esorted, int32_t* __restrict__ off,
                                                          int32_t* __restrict__ tstart) {
    __shared__ uint32_t cnt[1024], cur[1024], tl[1024];
    const int tid = threadIdx.x;
    cnt[tid] = 0;
    __syncthreads();
    for (int i = tid; i < R; i += 1024) atomicAdd(&cnt[min(max(inds[i], 0), E - 1)], 1u);
    __syncthreads();
    // exclusive prefix sums of the counts and of the per-expert tile counts (Hillis-Steele over 1024 entries)
    const uint32_t c = tid < E ? cnt[tid] : 0u;
    uint32_t so = c, st = (c + tm - 1) / tm;
    const uint32_t t0 = st;
    cur[tid] = so;
    tl[tid] = st;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {
        const uint32_t ao = tid >= d ? cur[tid - d] : 0u, at = tid >= d ? tl[tid - d] : 0u;
        __syncthreads();
        so += ao;
        st += at;
        cur[tid] = so;
        tl[tid] = st;
        __syncthreads();
    }
    if (tid < E) {
        off[tid] = int32_t(so - c);
        tstart[tid] = int32_t(st - t0);
    }
    if (tid == E - 1) {
        off[E] = int32_t(so);
        tstart[E] = int32_t(st);
    }
    __syncthreads();
    cur[tid] = so - c;   // next free row of each expert
    __syncthreads();
    for (int i = tid; i < R; i += 1024) {
        const int e = min(max(inds[i], 0), E - 1);
        const uint32_t p = atomicAdd(&cur[e], 1u);
        pos[i] = int32_t(p);
        tok[p] = i / topk;
        esorted[p] = e;
    }
    for (int p = R + tid; p < R + tm; p += 1024) tok[p] = 0;   // padding rows gather token 0
}

// ---- MoE: the same counting sort over several workgroups, three launches -------------------------------------------
// Workgroup g owns assignments [g * 1024, (g + 1) * 1024), the last one also the tail of fewer than 1024.  Its
// per-expert counts, and later its per-expert first rows, are parked in pos[g * 1024 + e] (E <= 1024), i.e. inside the
// part of `pos` that only this workgroup writes in the last pass, so no extra memory is needed and no workgroup reads
// what another one may already have overwritten.
constexpr int RS_CHUNK = 1024;

__global__ __launch_bounds__(RS_CHUNK) void route_count_kernel(const int32_t* __restrict__ inds, int R, int E,
                                                               int32_t* __restrict__ pos) {
    __shared__ uint32_t cnt[1024];
    const int tid = threadIdx.x;
    const int end = blockIdx.x == gridDim.x - 1 ? R : (blockIdx.x + 1) * RS_CHUNK;   // the last one takes the tail
    cnt[tid] = 0;
    __syncthreads();
    for (int i = blockIdx.x * RS_CHUNK + tid; i < end; i += RS_CHUNK) atomicAdd(&cnt[min(max(inds[i], 0), E - 1)], 1u);
    __syncthreads();
    if (tid < E) pos[blockIdx.x * RS_CHUNK + tid] = int32_t(cnt[tid]);
}

// One workgroup: thread e turns the G counts of expert e into exclusive prefixes (the rows of the expert taken by
// earlier workgroups), then the experts' totals are scanned into off / tstart as in the single-workgroup kernel.
__global__ __launch_bounds__(1024) void route_scan_kernel(int G, int E, int tm, int32_t* __restrict__ pos,
                                                          int32_t* __restrict__ off, int32_t* __restrict__ tstart) {
    __shared__ uint32_t cur[1024], tl[1024];
    const int tid = threadIdx.x;
    uint32_t c = 0;
    if (tid < E) {
        int g = 0;
        for (; g + 8 <= G; g += 8) {
            uint32_t v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = uint32_t(pos[(g + u) * RS_CHUNK + tid]);
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                pos[(g + u) * RS_CHUNK + tid] = int32_t(c);
                c += v[u];
            }
        }
        for (; g < G; ++g) {
            const uint32_t v = uint32_t(pos[g * RS_CHUNK + tid]);
            pos[g * RS_CHUNK + tid] = int32_t(c);
            c += v;
        }
    }
    uint32_t so = c, st = (c + tm - 1) / tm;
    const uint32_t t0 = st;
    cur[tid] = so;
    tl[tid] = st;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {
        const uint32_t ao = tid >= d ? cur[tid - d] : 0u, at = tid >= d ? tl[tid - d] : 0u;
        __syncthreads();
        so += ao;
        st += at;
        cur[tid] = so;
        tl[tid] = st;
        __syncthreads();
    }
    if (tid < E) {
        off[tid] = int32_t(so - c);
        tstart[tid] = int32_t(st - t0);
    }
    if (tid == E - 1) {
        off[E] = int32_t(so);
        tstart[E] = int32_t(st);
    }
}

__global__ __launch_bounds__(RS_CHUNK) void route_place_kernel(const int32_t* __restrict__ inds, int R, int topk, int E,
                                                               int tm, const int32_t* __restrict__ off,
                                                               int32_t* __restrict__ pos, int32_t* __restrict__ tok,
                                                               int32_t* __restrict__ esorted) {
    __shared__ uint32_t cur[1024];
    const int tid = threadIdx.x;
    const int end = blockIdx.x == gridDim.x - 1 ? R : (blockIdx.x + 1) * RS_CHUNK;
    if (tid < E) cur[tid] = uint32_t(off[tid]) + uint32_t(pos[blockIdx.x * RS_CHUNK + tid]);
    __syncthreads();   // the parked prefixes are in LDS before any pos[i] of this range is written
    for (int i = blockIdx.x * RS_CHUNK + tid; i < end; i += RS_CHUNK) {
        const int e = min(max(inds[i], 0), E - 1);
        const uint32_t p = atomicAdd(&cur[e], 1u);
        pos[i] = int32_t(p);
        tok[p] = i / topk;
        esorted[p] = e;
    }
    if (blockIdx.x == 0)
        for (int p = R + tid; p < R + tm; p += RS_CHUNK) tok[p] = 0;   // padding rows gather token 0
}

// ---- MoE: weighted combine of the top-k expert outputs, sequential in bf16 ---------------------------------------
// W = elements per thread and pass: 8 (16-byte loads) where K and the pointers allow, else 4.
template <int W>
__global__ __launch_bounds__(NT) void moe_combine_kernel(const uint16_t* __restrict__ y, const int32_t* __restrict__ pos,
                                                         const uint16_t* __restrict__ scores, const uint16_t* __restrict__ sscore,
                                                         const uint16_t* __restrict__ res, const uint16_t* __restrict__ w,
                                                         float eps, uint16_t* __restrict__ h, int8_t* __restrict__ xq,
                                                         float* __restrict__ xs, int M, int K, int topk) {
    extern __shared__ __attribute__((aligned(16))) uint16_t srow[];   // 2 K bf16 + 72 floats
    uint16_t* hrow_s = srow;
    uint16_t* nrow_s = srow + K;
    float* red = reinterpret_cast<float*>(srow + 2 * K);
    using vec = typename std::conditional<W == 8, u32x4, u32x2>::type;
    const int row = blockIdx.x;
    const int nsc = sscore ? topk - 1 : topk;
    for (int c = threadIdx.x; c < K / W; c += NT) {
        const vec r2 = *reinterpret_cast<const vec*>(res + size_t(row) * K + W * c);
        vec o = r2;
        if (row < M) {
            float acc[W];
#pragma unroll
            for (int i = 0; i < W; ++i) acc[i] = 0.0f;
            // the slots' rows are requested eight at a time, then added in slot order
            for (int j0 = 0; j0 < topk; j0 += 8) {
                vec y2[8];
                float sc[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int j = j0 + u;
                    if (j < topk) {
                        const int p = pos[row * topk + j];
                        sc[u] = bf16_to_f32((sscore && j == topk - 1) ? sscore[row] : scores[row * nsc + j]);
                        y2[u] = *reinterpret_cast<const vec*>(y + size_t(p) * K + W * c);
                    }
                }
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    if (j0 + u >= topk) break;
#pragma unroll
                    for (int i = 0; i < W; ++i) {
                        const float yv = __uint_as_float(i & 1 ? (y2[u][i >> 1] & 0xFFFF0000u) : (y2[u][i >> 1] << 16));
                        acc[i] = round_bf16(__fadd_rn(round_bf16(__fmul_rn(yv, sc[u])), acc[i]));
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < W / 2; ++i) {
                const float lo = __fadd_rn(__uint_as_float(r2[i] << 16), acc[2 * i]);
                const float hi = __fadd_rn(__uint_as_float(r2[i] & 0xFFFF0000u), acc[2 * i + 1]);
                o[i] = uint32_t(f32_to_bf16(lo)) | (uint32_t(f32_to_bf16(hi)) << 16);
            }
        }
        *reinterpret_cast<vec*>(hrow_s + W * c) = o;
        *reinterpret_cast<vec*>(h + size_t(row) * K + W * c) = o;
    }
    __syncthreads();
    if (!xq) return;
    const float inv = block_inv_rms(hrow_s, K, eps, red);
    block_norm_row(hrow_s, w, inv, nrow_s, nullptr, K);
    block_quant_row(nrow_s, K, xq + size_t(row) * K, xs + row, red);
}

static bool row_shape_ok(const char* who, int rows, int K, int max_k) {
    if (rows < 0 || K <= 0 || K % 4 || K > max_k) {
        set_error("%s: need rows >= 0 and K %% 4 == 0, K <= %d (rows=%d K=%d)", who, max_k, rows, K);
        return false;
    }
    return true;
}

// ---- router: softmax over the experts, the k largest, renormalisation, shared-expert gate --------------------------
// One wave per token.  Lane l holds experts l, l + 64, ...; probabilities are bf16(e_j / sum e) with
// e_j = 1 / exp(min(max - x_j, 80)) (exp_pos: IEEE operations only, so a host restatement gives the same bits), the sum
// taken per lane in rising j and then by the butterfly wave_sum.  The k winners are found by k wave-wide maxima over
// the key (probability bits << 16 | 65535 - j): largest probability first, equal ones by rising expert index.
constexpr int ROUTE_MAX_E = 1024;
// PER = experts per lane the kernel is built for (64 * PER >= E): slots past E cost what live ones do, so the launch picks
// the smallest of 1, 2, 4, 8, 16 that covers E.  The arithmetic of the live slots does not depend on PER.
template <int PER>
__global__ __launch_bounds__(NT) void route_topk_kernel(const uint16_t* __restrict__ logits,
                                                        const uint16_t* __restrict__ shared_logit, int M, int E, int topk,
                                                        int renorm, int32_t* __restrict__ inds,
                                                        uint16_t* __restrict__ scores) {
    static_assert(PER >= 1 && 64 * PER <= ROUTE_MAX_E, "experts per lane");
    const int lane = threadIdx.x & 63, t = blockIdx.x * (NT / 64) + (threadIdx.x >> 6);
    if (t >= M) return;   // wave-uniform
    const int stride = topk + (shared_logit ? 1 : 0);
    const uint16_t* row = logits + size_t(t) * E;
    float x[PER];
    float mx = -3.0e38f;
#pragma unroll
    for (int c = 0; c < PER; ++c) {
        const int j = 64 * c + lane;
        x[c] = j < E ? bf16_to_f32(row[j]) : 0.0f;
        if (j < E) mx = fmaxf(mx, x[c]);
    }
    mx = wave_max(mx);
    float part = 0.0f;
#pragma unroll
    for (int c = 0; c < PER; ++c) {
        const int j = 64 * c + lane;
        x[c] = j < E ? __fdiv_rn(1.0f, exp_pos(fminf(__fsub_rn(mx, x[c]), 80.0f))) : 0.0f;
        if (64 * c < E) part = __fadd_rn(part, x[c]);
    }
    const float total = wave_sum(part);
    uint32_t key[PER];
#pragma unroll
    for (int c = 0; c < PER; ++c) {
        const int j = 64 * c + lane;
        key[c] = j < E ? (uint32_t(f32_to_bf16(__fdiv_rn(x[c], total))) << 16) | uint32_t(0xFFFF - j) : 0u;
    }
    uint32_t mine = 0;      // lane s keeps the winner of round s
    float tot = 0.0f;
    for (int s = 0; s < topk; ++s) {
        uint32_t best = 0;
#pragma unroll
        for (int c = 0; c < PER; ++c) best = max(best, key[c]);
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) best = max(best, uint32_t(__shfl_xor(int(best), off, WAVE)));
#pragma unroll
        for (int c = 0; c < PER; ++c)
            if (key[c] == best) key[c] = 0;    // keys are distinct (they carry the expert index)
        if (lane == s) mine = best;
        tot = __fadd_rn(tot, bf16_to_f32(uint16_t(best >> 16)));
    }
    if (lane < topk) {
        const uint16_t pb = uint16_t(mine >> 16);
        inds[size_t(t) * stride + lane] = 0xFFFF - int(mine & 0xFFFFu);
        scores[size_t(t) * stride + lane] = renorm ? f32_to_bf16(__fdiv_rn(bf16_to_f32(pb), round_bf16(tot))) : pb;
    }
    if (shared_logit && lane == 0) {
        const float g = bf16_to_f32(shared_logit[t]);
        const float y = __fdiv_rn(1.0f, __fadd_rn(1.0f, exp_pos(fminf(fabsf(g), 80.0f))));
        inds[size_t(t) * stride + topk] = E;
        scores[size_t(t) * stride + topk] = f32_to_bf16(g < 0.0f ? y : __fsub_rn(1.0f, y));
    }
}

}  // namespace scmx

using namespace scmx;

extern "C" {

int scmx_rmsnorm_quant_blocked(const uint16_t* x, const uint16_t* w, float eps, int8_t* xq, float* xs, uint16_t* xn, int M,
                               int Mp, int K, void* stream) {
    if (!x || !w || !xq || !xs || Mp < M || Mp % 32 || !row_shape_ok("rmsnorm_quant_blocked", M, K, 4096) || K % 512 ||
        (uintptr_t(x) | uintptr_t(w) | uintptr_t(xn) | uintptr_t(xq)) % 16) {
        if (!(x && w && xq && xs) || Mp < M || Mp % 32 || K % 512 || (uintptr_t(x) | uintptr_t(w) | uintptr_t(xn) | uintptr_t(xq)) % 16)
            set_error("rmsnorm_quant_blocked: need M <= Mp with Mp %% 32 == 0 (Mp = %d), K %% 512 == 0 and K <= 4096 (K = %d), "
                      "16-byte aligned operands", Mp, K);
        return SCMX_ERR_ARG;
    }
    if (Mp == 0) return SCMX_OK;
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid(unsigned(Mp) / 8u), block(512);
    switch (K / 512) {
        case 1: rmsnorm_quant_wave_kernel<1, true><<<grid, block, 0, st>>>(x, w, eps, xq, xs, xn, M, Mp); break;
        case 2: rmsnorm_quant_wave_kernel<2, true><<<grid, block, 0, st>>>(x, w, eps, xq, xs, xn, M, Mp); break;
        case 3: rmsnorm_quant_wave_kernel<3, true><<<grid, block, 0, st>>>(x, w, eps, xq, xs, xn, M, Mp); break;
        case 4: rmsnorm_quant_wave_kernel<4, true><<<grid, block, 0, st>>>(x, w, eps, xq, xs, xn, M, Mp); break;
        case 5: rmsnorm_quant_wave_kernel<5, true><<<grid, block, 0, st>>>(x, w, eps, xq, xs, xn, M, Mp); break;
        case 6: rmsnorm_quant_wave_kernel<6, true><<<grid, block, 0, st>>>(x, w, eps, xq, xs, xn, M, Mp); break;
        case 7: rmsnorm_quant_wave_kernel<7, true><<<grid, block, 0, st>>>(x, w, eps, xq, xs, xn, M, Mp); break;
        default: rmsnorm_quant_wave_kernel<8, true><<<grid, block, 0, st>>>(x, w, eps, xq, xs, xn, M, Mp); break;
    }
    return check_launch("rmsnorm_quant_blocked");
}

int scmx_rmsnorm_quant(const uint16_t* x, const uint16_t* w, float eps, int8_t* xq, float* xs, uint16_t* xn, int M,
                       int Mp, int K, void* stream) {
    if (!x || !w || !xq || !xs || Mp < M || !row_shape_ok("rmsnorm_quant", M, K, 16384)) {
        if (!(x && w && xq && xs) || Mp < M) set_error("rmsnorm_quant: null pointer or Mp < M");
        return SCMX_ERR_ARG;
    }
    if (Mp == 0) return SCMX_OK;
    hipStream_t st = (hipStream_t)stream;
    if (K % 512 == 0 && (uintptr_t(x) | uintptr_t(w) | uintptr_t(xn)) % 16 == 0 && uintptr_t(xq) % 8 == 0) {
        // rows of up to 4096 elements stay in registers (one wave per row)
        const dim3 wgrid((unsigned(Mp) + 3u) / 4u), block(256);
        switch (K / 512) {
            case 1: rmsnorm_quant_wave_kernel<1><<<wgrid, block, 0, st>>>(x, w, eps, xq, xs, xn, M, Mp); return check_launch("rmsnorm_quant");
            case 2: rmsnorm_quant_wave_kernel<2><<<wgrid, block, 0, st>>>(x, w, eps, xq, xs, xn, M, Mp); return check_launch("rmsnorm_quant");
            case 3: rmsnorm_quant_wave_kernel<3><<<wgrid, block, 0, st>>>(x, w, eps, xq, xs, xn, M, Mp); return check_launch("rmsnorm_quant");
            case 4: rmsnorm_quant_wave_kernel<4><<<wgrid, block, 0, st>>>(x, w, eps, xq, xs, xn, M, Mp); return check_launch("rmsnorm_quant");
            case 5: rmsnorm_quant_wave_kernel<5><<<wgrid, block, 0, st>>>(x, w, eps, xq, xs, xn, M, Mp); return check_launch("rmsnorm_quant");
            case 6: rmsnorm_quant_wave_kernel<6><<<wgrid, block, 0, st>>>(x, w, eps, xq, xs, xn, M, Mp); return check_launch("rmsnorm_quant");
            case 7: rmsnorm_quant_wave_kernel<7><<<wgrid, block, 0, st>>>(x, w, eps, xq, xs, xn, M, Mp); return check_launch("rmsnorm_quant");
            case 8: rmsnorm_quant_wave_kernel<8><<<wgrid, block, 0, st>>>(x, w, eps, xq, xs, xn, M, Mp); return check_launch("rmsnorm_quant");
            default: break;
        }
    }
    rmsnorm_quant_kernel<<<dim3(Mp), dim3(NT), size_t(K) * 2 + 72 * 4, st>>>(x, w, eps, xq, xs, xn, M, K);
    return check_launch("rmsnorm_quant");
}

int scmx_res_norm_quant(const int32_t* acc, const float* xscale, const float* wscale, const uint16_t* res,
                        const uint16_t* w, float eps, uint16_t* h, int8_t* xq, float* xs, int Mp, int K, void* stream) {
    if (!acc || !xscale || !wscale || !res || !h || (xq && (!w || !xs)) || !row_shape_ok("res_norm_quant", Mp, K, 8192)) {
        if (!(acc && xscale && wscale && res && h) || (xq && (!w || !xs))) set_error("res_norm_quant: null pointer argument");
        return SCMX_ERR_ARG;
    }
    if (Mp == 0) return SCMX_OK;
    res_norm_quant_kernel<<<dim3(Mp), dim3(NT), size_t(K) * 4 + 72 * 4, (hipStream_t)stream>>>(acc, xscale, wscale, res, w,
                                                                                                  eps, h, xq, xs, K);
    return check_launch("res_norm_quant");
}

int scmx_swiglu_quant(const int32_t* acc, const float* xscale, const float* wscale, int8_t* xq, float* xs, int Mp, int F,
                      void* stream) {
    if (!acc || !xscale || !wscale || !xq || !xs || !row_shape_ok("swiglu_quant", Mp, F, 16384)) {
        if (!(acc && xscale && wscale && xq && xs)) set_error("swiglu_quant: null pointer argument");
        return SCMX_ERR_ARG;
    }
    if (Mp == 0) return SCMX_OK;
    const uint16_t* silu = silu_table_device();
    if (!silu) {
        set_error("swiglu_quant: the SiLU table could not be located on the device");
        return SCMX_ERR_LAUNCH;
    }
    swiglu_quant_kernel<<<dim3(Mp), dim3(NT), size_t(F) * 2 + 72 * 4, (hipStream_t)stream>>>(acc, xscale, wscale, xq, xs, F,
                                                                                            silu);
    return check_launch("swiglu_quant");
}

// few rows (decode): spread the heads over workgroups; many rows: one workgroup per row
static dim3 headnorm_grid(int L, int heads) {
    const int groups = (heads + NT / 64 - 1) / (NT / 64);
    return dim3(L, L >= 256 ? 1 : groups);
}

// Many rows of bf16 input with head dim 128 and 16-byte aligned operands take the kernel with 16-byte accesses (a few rows
// are spread over more workgroups by the general one).
static bool headnorm128_fits(const int32_t* acc, const uint16_t* y, const uint16_t* qn, const uint16_t* kn, const uint16_t* q,
                             const uint16_t* k, const uint16_t* v, int L, int d) {
    return !acc && d == 128 && L >= 16 &&
           (uintptr_t(y) | uintptr_t(qn) | uintptr_t(kn) | uintptr_t(q) | uintptr_t(k) | uintptr_t(v)) % 16 == 0;
}

int scmx_qkv_headnorm(const int32_t* acc, const float* xscale, const float* wscale, const uint16_t* y,
                      const uint16_t* qn, const uint16_t* kn, float eps, uint16_t* q, uint16_t* k, uint16_t* v, int L,
                      int hq, int hk, int d, void* stream) {
    if ((!acc && !y) || (acc && (!xscale || !wscale)) || !qn || !kn || !q || !k || !v) {
        set_error("qkv_headnorm: null pointer argument");
        return SCMX_ERR_ARG;
    }
    if (L < 0 || hq < 1 || hk < 1 || hq > 65536 || hk > 65536 || d % 64 || d < 64 || d > 512) {
        set_error("qkv_headnorm: need 1..65536 heads and a head dim that is a multiple of 64 in 64..512 (hq=%d hk=%d d=%d)", hq, hk, d);
        return SCMX_ERR_ARG;
    }
    if (L == 0) return SCMX_OK;
    if (headnorm128_fits(acc, y, qn, kn, q, k, v, L, d)) {
        qkv_headnorm128_kernel<<<dim3(L), dim3(NT), 0, (hipStream_t)stream>>>(y, qn, kn, eps, q, k, v, L, hq, hk,
                                                                               RopeArgs{nullptr, nullptr, 0, 0, 0});
        return check_launch("qkv_headnorm");
    }
    qkv_headnorm_kernel<<<headnorm_grid(L, hq + 2 * hk), dim3(NT), 0, (hipStream_t)stream>>>(
        acc, xscale, wscale, y, qn, kn, eps, q, k, v, L, hq, hk, d, RopeArgs{nullptr, nullptr, 0, 0, 0});
    return check_launch("qkv_headnorm");
}

int scmx_qkv_headnorm_rope(const int32_t* acc, const float* xscale, const float* wscale, const uint16_t* y,
                           const uint16_t* qn, const uint16_t* kn, float eps, uint16_t* q, uint16_t* kcache,
                           uint16_t* vcache, int L, int hq, int hk, int d, const float* inv_freq,
                           const int64_t* pos_dev, int64_t pos0, int cache_rows, int q_token_major, void* stream) {
    if ((!acc && !y) || (acc && (!xscale || !wscale)) || !qn || !kn || !q || !kcache || !vcache || !inv_freq) {
        set_error("qkv_headnorm_rope: null pointer argument");
        return SCMX_ERR_ARG;
    }
    if (L < 0 || hq < 1 || hk < 1 || hq > 65536 || hk > 65536 || d % 64 || d < 64 || d > 512) {
        set_error("qkv_headnorm_rope: need 1..65536 heads and a head dim that is a multiple of 64 in 64..512 (hq=%d hk=%d d=%d)", hq, hk, d);
        return SCMX_ERR_ARG;
    }
    if (cache_rows < L || (!pos_dev && (pos0 < 0 || pos0 > int64_t(cache_rows) - L))) {
        set_error("qkv_headnorm_rope: rows %lld..%lld do not fit a cache of %d rows", (long long)pos0,
                  (long long)(pos0 + L), cache_rows);
        return SCMX_ERR_ARG;
    }
    if (L == 0) return SCMX_OK;
    if (headnorm128_fits(acc, y, qn, kn, q, kcache, vcache, L, d)) {
        qkv_headnorm128_kernel<<<dim3(L), dim3(NT), 0, (hipStream_t)stream>>>(
            y, qn, kn, eps, q, kcache, vcache, L, hq, hk, RopeArgs{inv_freq, pos_dev, pos0, cache_rows, q_token_major});
        return check_launch("qkv_headnorm_rope");
    }
    qkv_headnorm_kernel<<<headnorm_grid(L, hq + 2 * hk), dim3(NT), 0, (hipStream_t)stream>>>(
        acc, xscale, wscale, y, qn, kn, eps, q, kcache, vcache, L, hq, hk, d, RopeArgs{inv_freq, pos_dev, pos0, cache_rows, q_token_major});
    return check_launch("qkv_headnorm_rope");
}

int scmx_qkv_fullnorm(const uint16_t* y, const uint16_t* qn, const uint16_t* kn, float eps, uint16_t* q, uint16_t* k,
                      uint16_t* v, int L, int h, int d, void* stream) {
    if (!y || !qn || !kn || !q || !k || !v) {
        set_error("qkv_fullnorm: null pointer argument");
        return SCMX_ERR_ARG;
    }
    if (L < 0 || h < 1 || d < 4 || d % 4 || d > 16384 || h > 16384 / d) {
        set_error("qkv_fullnorm: need L >= 0, h >= 1, d %% 4 == 0 and h * d <= 16384 (L=%d h=%d d=%d)", L, h, d);
        return SCMX_ERR_ARG;
    }
    if (L == 0) return SCMX_OK;
    qkv_fullnorm_kernel<<<dim3(L), dim3(NT), size_t(h) * d * 2 + 72 * 4, (hipStream_t)stream>>>(y, qn, kn, eps, q, k, v, L,
                                                                                                 h, d);
    return check_launch("qkv_fullnorm");
}

int scmx_route_topk(const uint16_t* logits, const uint16_t* shared_logit, int M, int n_experts, int topk, int renorm,
                    int32_t* inds, uint16_t* scores, void* stream) {
    if (!logits || !inds || !scores || M < 0 || n_experts < 1 || n_experts > ROUTE_MAX_E || topk < 1 || topk > 64 ||
        topk > n_experts) {
        set_error("route_topk: null pointer, n_experts (%d) outside 1..%d or topk (%d) outside 1..min(64, n_experts)",
                  n_experts, ROUTE_MAX_E, topk);
        return SCMX_ERR_ARG;
    }
    if (M == 0) return SCMX_OK;
    const dim3 grid((unsigned(M) + NT / 64 - 1) / (NT / 64)), block(NT);
    hipStream_t st = (hipStream_t)stream;
    const auto launch = [&](auto per_tag) {
        route_topk_kernel<decltype(per_tag)::value><<<grid, block, 0, st>>>(logits, shared_logit, M, n_experts, topk, renorm,
                                                                           inds, scores);
    };
    if (n_experts <= 64) launch(std::integral_constant<int, 1>{});
    else if (n_experts <= 128) launch(std::integral_constant<int, 2>{});
    else if (n_experts <= 256) launch(std::integral_constant<int, 4>{});
    else if (n_experts <= 512) launch(std::integral_constant<int, 8>{});
    else launch(std::integral_constant<int, 16>{});
    return check_launch("route_topk");
}

int scmx_route_sort(const int32_t* inds, int M, int topk, int n_experts, int tm, int32_t* pos, int32_t* tok,
                    int32_t* esorted, int32_t* off, int32_t* tstart, void* stream) {
    if (!inds || !pos || !tok || !esorted || !off || !tstart || M < 0 || topk < 1 || tm < 1 || n_experts < 1 ||
        n_experts > 1024) {
        set_error("route_sort: null pointer, or n_experts (%d) outside 1..1024", n_experts);
        return SCMX_ERR_ARG;
    }
    const long long R = (long long)M * topk;
    if (R > 0x7FFFFFFF - tm) {
        set_error("route_sort: M * topk = %lld beyond 32-bit row indices", R);
        return SCMX_ERR_ARG;
    }
    hipStream_t st = (hipStream_t)stream;
    const int G = int(R / RS_CHUNK);   // whole chunks; the last workgroup also takes the tail
    if (G < 4) {   // small inputs: one launch of one workgroup beats three launches
        route_sort_kernel<<<dim3(1), dim3(1024), 0, st>>>(inds, int(R), topk, n_experts, tm, pos, tok, esorted, off, tstart);
        return check_launch("route_sort");
    }
    route_count_kernel<<<dim3(G), dim3(RS_CHUNK), 0, st>>>(inds, int(R), n_experts, pos);
    route_scan_kernel<<<dim3(1), dim3(1024), 0, st>>>(G, n_experts, tm, pos, off, tstart);
    route_place_kernel<<<dim3(G), dim3(RS_CHUNK), 0, st>>>(inds, int(R), topk, n_experts, tm, off, pos, tok, esorted);
    return check_launch("route_sort");
}

int scmx_moe_combine(const uint16_t* y, const int32_t* pos, const uint16_t* scores, const uint16_t* sscore,
                     const uint16_t* res, const uint16_t* w, float eps, uint16_t* h, int8_t* xq, float* xs, int M, int Mp,
                     int K, int topk, void* stream) {
    if (!y || !pos || !scores || !res || !h || (xq && (!w || !xs)) || Mp < M || topk < 1 || topk > 65536 ||
        !row_shape_ok("moe_combine", M, K, 8192)) {
        if (!(y && pos && scores && res && h) || (xq && (!w || !xs)) || Mp < M || topk < 1 || topk > 65536)
            set_error("moe_combine: null pointer argument, Mp < M or topk outside 1..65536");
        return SCMX_ERR_ARG;
    }
    if (Mp == 0) return SCMX_OK;
    if (K % 8 == 0 && (uintptr_t(y) | uintptr_t(res) | uintptr_t(h)) % 16 == 0)
        moe_combine_kernel<8><<<dim3(Mp), dim3(NT), size_t(K) * 4 + 72 * 4, (hipStream_t)stream>>>(y, pos, scores, sscore, res,
                                                                                                    w, eps, h, xq, xs, M, K, topk);
    else
        moe_combine_kernel<4><<<dim3(Mp), dim3(NT), size_t(K) * 4 + 72 * 4, (hipStream_t)stream>>>(y, pos, scores, sscore, res,
                                                                                                    w, eps, h, xq, xs, M, K, topk);
    return check_launch("moe_combine");
}

}  // extern "C"
