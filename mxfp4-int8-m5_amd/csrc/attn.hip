// Single-token attention against a KV cache (decode): out[h] = softmax(q[h] . K^T * scale) V for every query head.
//
// The linear layers are the product here; this kernel exists so that a decode step is a fixed, short sequence of
// launches that a HIP graph can replay: it reads the number of valid cache rows from device memory, so the same
// captured launch serves every position.  One workgroup per query head.  A row of K or V (d bf16 values) is read by
// d / 8 lanes, 16 bytes each; such a lane group walks every (groups)-th row with a running maximum, sum and
// weighted value chunk (one pass over K and V, both rows of a step in flight together), and the groups' partial
// results are merged through LDS.  Accumulation is float32, the output bf16.
#include "scmx_common.h"

namespace scmx {

constexpr int ANT = 256;

template <int D>
__global__ __launch_bounds__(ANT) void attn_decode_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ kc,
                                                         const uint16_t* __restrict__ vc,
                                                         const int64_t* __restrict__ pos_dev, int n0,
                                                         uint16_t* __restrict__ out, int hq, int hk, int rows, float scale) {
    constexpr int LPR = D / 8;              // lanes per cache row
    constexpr int GROUPS = ANT / LPR;       // lane groups per workgroup, each walking its own rows
    __shared__ float s_m[GROUPS], s_l[GROUPS], s_acc[GROUPS][D];
    const int n = min(rows, pos_dev ? int(pos_dev[0]) + 1 : n0);
    const int head = blockIdx.x, kvh = head / (hq / hk);
    const int tid = threadIdx.x, grp = tid / LPR, c = tid % LPR;
    const uint16_t* kbase = kc + size_t(kvh) * rows * D + 8 * c;
    const uint16_t* vbase = vc + size_t(kvh) * rows * D + 8 * c;

    float qv[8];
    {
        const u32x4 w = *reinterpret_cast<const u32x4*>(q + size_t(head) * D + 8 * c);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            qv[2 * i] = __uint_as_float(w[i] << 16) * scale;
            qv[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u) * scale;
        }
    }
    float m = -3.0e38f, l = 0.0f;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    // Every lane of the workgroup runs the same number of trips (rows beyond n are skipped by predication), so the
    // cross-lane sums below always see whole groups.
    const int trips = (n + GROUPS - 1) / GROUPS;
    constexpr int UN = 4;   // rows in flight per lane group: the K and V rows of UN steps are requested together
    for (int t0 = 0; t0 < trips; t0 += UN) {
        u32x4 kw[UN], vw[UN];
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int j = (t0 + u) * GROUPS + grp;
            const size_t ro = size_t(j < n ? j : 0) * D;
            kw[u] = *reinterpret_cast<const u32x4*>(kbase + ro);
            vw[u] = *reinterpret_cast<const u32x4*>(vbase + ro);
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const bool ok = (t0 + u) * GROUPS + grp < n;
            float s = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                s += qv[2 * i] * __uint_as_float(kw[u][i] << 16) + qv[2 * i + 1] * __uint_as_float(kw[u][i] & 0xFFFF0000u);
#pragma unroll
            for (int off = LPR / 2; off >= 1; off >>= 1) s += __shfl_xor(s, off, WAVE);
            if (ok) {
                const float mn = fmaxf(m, s);
                const float alpha = __expf(m - mn), p = __expf(s - mn);
                l = l * alpha + p;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc[2 * i] = acc[2 * i] * alpha + p * __uint_as_float(vw[u][i] << 16);
                    acc[2 * i + 1] = acc[2 * i + 1] * alpha + p * __uint_as_float(vw[u][i] & 0xFFFF0000u);
                }
                m = mn;
            }
        }
    }
    if (c == 0) {
        s_m[grp] = m;
        s_l[grp] = l;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) s_acc[grp][8 * c + i] = acc[i];
    __syncthreads();
    // merge the groups: element e of the output by thread e
    for (int e = tid; e < D; e += ANT) {
        float mx = s_m[0];
#pragma unroll
        for (int g = 1; g < GROUPS; ++g) mx = fmaxf(mx, s_m[g]);
        float num = 0.0f, den = 0.0f;
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
            const float w = __expf(s_m[g] - mx);   // groups that saw no row have l = 0 and contribute nothing
            num += w * s_acc[g][e];
            den += w * s_l[g];
        }
        out[size_t(head) * D + e] = f32_to_bf16(num / den);
    }
}

}  // namespace scmx

using namespace scmx;

extern "C" int scmx_attn_decode(const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache, const int64_t* pos_dev,
                                int n, uint16_t* out, int hq, int hk, int d, int cache_rows, float scale, void* stream) {
    if (!q || !kcache || !vcache || !out || hq < 1 || hk < 1 || hq % hk || cache_rows < 1) {
        set_error("attn_decode: null pointer or bad head counts (hq=%d hk=%d)", hq, hk);
        return SCMX_ERR_ARG;
    }
    if (d != 64 && d != 128 && d != 256) {
        set_error("attn_decode: head dim must be 64, 128 or 256 (d=%d)", d);
        return SCMX_ERR_ARG;
    }
    if (!pos_dev && (n < 1 || n > cache_rows)) {
        set_error("attn_decode: %d valid rows outside 1..%d", n, cache_rows);
        return SCMX_ERR_ARG;
    }
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid(hq), wg(ANT);
    if (d == 64)
        attn_decode_kernel<64><<<grid, wg, 0, st>>>(q, kcache, vcache, pos_dev, n, out, hq, hk, cache_rows, scale);
    else if (d == 128)
        attn_decode_kernel<128><<<grid, wg, 0, st>>>(q, kcache, vcache, pos_dev, n, out, hq, hk, cache_rows, scale);
    else
        attn_decode_kernel<256><<<grid, wg, 0, st>>>(q, kcache, vcache, pos_dev, n, out, hq, hk, cache_rows, scale);
    return check_launch("attn_decode");
}
