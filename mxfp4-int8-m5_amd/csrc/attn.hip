// Single-token attention against a KV cache (decode): out[h] = softmax(q[h] . K^T * scale) V for every query head.
//
// The linear layers are the product here; this kernel exists so that a decode step is a fixed, short sequence of
// launches that a HIP graph can replay: it reads the number of valid cache rows from device memory, so the same
// captured launch serves every position.  One workgroup per query head.  A row of K or V (d bf16 values) is read by
// d / 8 lanes, 16 bytes each; such a lane group walks every (groups)-th row with a running maximum, sum and
// weighted value chunk (one pass over K and V, both rows of a step in flight together), and the groups' partial
// results are merged through LDS.  Accumulation is float32, the output bf16.  For long contexts the rows of a head
// are cut into several ranges, one workgroup each (16 workgroups alone read a long cache at a fraction of the memory
// bandwidth), and a small second kernel merges the ranges' results.
#include "scmx_common.h"

namespace scmx {

constexpr int ANT = 512;
constexpr int ATTN_SINGLE_MAX = 512;   // rows up to which a split launch falls back to one workgroup per head

// What the fused variant needs besides the attention operands: the token's q|k|v row as the qkv projection wrote it,
// the per-head norm weights and the rotary frequencies.
struct QkvArgs {
    const uint16_t* y;        // bf16 [(hq + 2 hk) * d]: q heads, k heads, v heads
    const uint16_t* qn;       // bf16 [d]
    const uint16_t* kn;       // bf16 [d]
    const float* inv_freq;    // [d / 2]
    float eps;
};

// FUSED: the workgroup first normalises and rotates its own q head and its KV head's new k (as the row kernel
// qkv_headnorm_kernel does, same arithmetic), keeps them and the new v in LDS, and attends over the cache rows below
// the position plus that new row; the first query head of every KV group appends the new k and v to the cache.  No
// workgroup reads what another writes in the same launch.
template <int D, bool FUSED>
__global__ __launch_bounds__(ANT) void attn_decode_kernel(const uint16_t* __restrict__ q, uint16_t* __restrict__ kc,
                                                         uint16_t* __restrict__ vc,
                                                         const int64_t* __restrict__ pos_dev, int n0,
                                                         uint16_t* __restrict__ out, int hq, int hk, int rows, float scale,
                                                         const QkvArgs x, float* __restrict__ partial) {
    constexpr int LPR = D / 8;              // lanes per cache row
    constexpr int GROUPS = ANT / LPR;       // lane groups per workgroup, each walking its own rows
    __shared__ float s_m[GROUPS], s_l[GROUPS], s_acc[GROUPS][D];
    __shared__ float s_sin[FUSED ? D / 2 : 1], s_cos[FUSED ? D / 2 : 1];
    __shared__ __attribute__((aligned(16))) uint16_t s_new[FUSED ? 3 : 1][D];   // this token's q, k, v (bf16)
    const int head = blockIdx.x, kvh = head / (hq / hk);
    const int tid = threadIdx.x, grp = tid / LPR, c = tid % LPR;
    // A device-resident position outside the cache (the host cannot see it) touches no cache row: the output is
    // zero and nothing is appended.
    const int64_t n64 = pos_dev ? pos_dev[0] + 1 : int64_t(n0);
    if (n64 < 1 || n64 > rows) {
        if (blockIdx.y == 0)
            for (int e = tid; e < D; e += ANT) out[size_t(head) * D + e] = 0;
        return;
    }
    const int n = int(n64);
    const uint16_t* kbase = kc + size_t(kvh) * rows * D + 8 * c;
    const uint16_t* vbase = vc + size_t(kvh) * rows * D + 8 * c;

    // gridDim.y > 1: the valid rows are cut into gridDim.y equal ranges, one per workgroup of a head; every workgroup
    // leaves its unnormalised result, maximum and sum in `partial` and a second kernel merges them.
    // A context of at most ATTN_SINGLE_MAX rows is read fastest by one workgroup per head: range 0 then takes all of
    // it and writes the output, the other workgroups leave at once and the merge kernel finds nothing to do.
    const bool single = gridDim.y == 1 || n <= ATTN_SINGLE_MAX;
    if (single && blockIdx.y > 0) return;
    const int nsplit = single ? 1 : int(gridDim.y);
    const int chunk = (n + nsplit - 1) / nsplit;
    const int row0 = int(blockIdx.y) * chunk, row1 = min(n, row0 + chunk);   // this workgroup's rows [row0, row1)
    // Every lane of the workgroup runs the same number of trips (rows beyond row1 are skipped by predication), so the
    // cross-lane sums below always see whole groups.
    const int trips = (max(row1 - row0, 0) + GROUPS - 1) / GROUPS;
    constexpr int UN = 4;   // rows in flight per lane group: the K and V rows of UN steps are requested together
    u32x4 kw[UN], vw[UN];
    auto load_trip = [&](int t0) {
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const int j = row0 + (t0 + u) * GROUPS + grp;
            const size_t ro = size_t(j < row1 ? j : 0) * D;
            kw[u] = *reinterpret_cast<const u32x4*>(kbase + ro);
            vw[u] = *reinterpret_cast<const u32x4*>(vbase + ro);
        }
    };
    load_trip(0);   // on their way while the fused variant prepares q and the new row

    if (FUSED) {
        constexpr int PER = D / 64;
        const int lane = tid & 63, wave = tid >> 6;
        const int newrow = n - 1;   // the position of the token being decoded
        // wave 3 computes the row's sines and cosines while waves 0 / 1 / 2 fetch and normalise the q / k / v head
        float nv[PER];
        const int g = wave == 0 ? head : (wave == 1 ? hq + kvh : hq + hk + kvh);
        if (wave == 3) {
            for (int i = lane; i < D / 2; i += 64) sincosf(float(int64_t(newrow)) * x.inv_freq[i], &s_sin[i], &s_cos[i]);
        } else {
            float yv[PER];
            float ss = 0.0f;
#pragma unroll
            for (int i = 0; i < PER; ++i) {
                yv[i] = bf16_to_f32(x.y[size_t(g) * D + PER * lane + i]);
                ss = __fadd_rn(ss, __fmul_rn(yv[i], yv[i]));
            }
            if (wave < 2) {
                head_norm(yv, ss, PER, lane, D, wave == 0 ? x.qn : x.kn, x.eps, nv);
            } else {
#pragma unroll
                for (int i = 0; i < PER; ++i) nv[i] = yv[i];
            }
        }
        __syncthreads();
        if (wave < 3) {
            const bool append = wave > 0 && head % (hq / hk) == 0 && blockIdx.y == 0;
            uint16_t* dst = (wave == 1 ? kc : vc) + (size_t(kvh) * rows + newrow) * D + PER * lane;
            auto emit = [&](int i, uint16_t b) {
                s_new[wave][PER * lane + i] = b;
                if (append) dst[i] = b;
            };
            head_rope(nv, PER, lane, D, wave < 2 ? s_sin : nullptr, s_cos, emit);   // v passes through unrotated
        }
        __syncthreads();
    }

    float qv[8];
    {
        const u32x4 w = FUSED ? *reinterpret_cast<const u32x4*>(&s_new[0][8 * c])
                              : *reinterpret_cast<const u32x4*>(q + size_t(head) * D + 8 * c);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            qv[2 * i] = __uint_as_float(w[i] << 16) * scale;
            qv[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u) * scale;
        }
    }
    float m = -3.0e38f, l = 0.0f;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int t0 = 0; t0 < trips; t0 += UN) {
        if (t0 > 0) load_trip(t0);
        if (FUSED) {   // the new row comes from LDS, not from the cache being appended to
#pragma unroll
            for (int u = 0; u < UN; ++u)
                if (row0 + (t0 + u) * GROUPS + grp == n - 1) {
                    kw[u] = *reinterpret_cast<const u32x4*>(&s_new[1][8 * c]);
                    vw[u] = *reinterpret_cast<const u32x4*>(&s_new[2][8 * c]);
                }
        }
#pragma unroll
        for (int u = 0; u < UN; ++u) {
            const bool ok = row0 + (t0 + u) * GROUPS + grp < row1;
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
        if (single) {
            out[size_t(head) * D + e] = f32_to_bf16(num / den);
        } else {   // num and den are relative to mx; a range without rows leaves mx = -3e38, den = 0
            float* pw = partial + (size_t(head) * gridDim.y + blockIdx.y) * (D + 2);
            pw[e] = num;
            if (e == 0) {
                pw[D] = mx;
                pw[D + 1] = den;
            }
        }
    }
}

// Merge of the per-range results of one head: out = sum_s w_s num_s / sum_s w_s den_s with w_s = exp(m_s - max m).
template <int D>
__global__ __launch_bounds__(D) void attn_merge_kernel(const float* __restrict__ partial, uint16_t* __restrict__ out,
                                                     int splits, const int64_t* __restrict__ pos_dev, int n0, int rows) {
    const int64_t n64 = pos_dev ? pos_dev[0] + 1 : int64_t(n0);
    if (n64 <= ATTN_SINGLE_MAX || n64 > rows) return;   // range 0 wrote the output itself (zeros for a position outside the cache)
    const int head = blockIdx.x, e = threadIdx.x;
    const float* pw = partial + size_t(head) * splits * (D + 2);
    float mx = -3.0e38f;
    for (int s = 0; s < splits; ++s) mx = fmaxf(mx, pw[s * (D + 2) + D]);
    float num = 0.0f, den = 0.0f;
    for (int s = 0; s < splits; ++s) {
        const float w = __expf(pw[s * (D + 2) + D] - mx);
        num += w * pw[s * (D + 2) + e];
        den += w * pw[s * (D + 2) + D + 1];
    }
    out[size_t(head) * D + e] = f32_to_bf16(num / den);
}

template <bool FUSED>
static void launch_attn(int d, hipStream_t st, const uint16_t* q, uint16_t* kc, uint16_t* vc, const int64_t* pos_dev, int n,
                        uint16_t* out, int hq, int hk, int rows, float scale, const QkvArgs& x, float* partial, int splits) {
    const dim3 grid(hq, splits), wg(ANT);
    if (d == 64) {
        attn_decode_kernel<64, FUSED><<<grid, wg, 0, st>>>(q, kc, vc, pos_dev, n, out, hq, hk, rows, scale, x, partial);
        if (splits > 1) attn_merge_kernel<64><<<dim3(hq), dim3(64), 0, st>>>(partial, out, splits, pos_dev, n, rows);
    } else if (d == 128) {
        attn_decode_kernel<128, FUSED><<<grid, wg, 0, st>>>(q, kc, vc, pos_dev, n, out, hq, hk, rows, scale, x, partial);
        if (splits > 1) attn_merge_kernel<128><<<dim3(hq), dim3(128), 0, st>>>(partial, out, splits, pos_dev, n, rows);
    } else {
        attn_decode_kernel<256, FUSED><<<grid, wg, 0, st>>>(q, kc, vc, pos_dev, n, out, hq, hk, rows, scale, x, partial);
        if (splits > 1) attn_merge_kernel<256><<<dim3(hq), dim3(256), 0, st>>>(partial, out, splits, pos_dev, n, rows);
    }
}

// The row ranges of a split launch: `workspace` holds splits * hq * (d + 2) floats.
static int check_split(const char* who, const float* workspace, int splits) {
    if (splits < 1 || splits > 64 || (splits > 1 && (!workspace || uintptr_t(workspace) % 4))) {
        set_error("%s: splits must be 1..64 and need a float workspace of splits * hq * (d + 2) entries", who);
        return SCMX_ERR_ARG;
    }
    return SCMX_OK;
}

}  // namespace scmx

using namespace scmx;

static int check_attn(const char* who, int hq, int hk, int d, int cache_rows) {
    if (hq < 1 || hk < 1 || hq > 65535 || hq % hk || cache_rows < 1) {
        set_error("%s: bad head counts or cache size (hq=%d hk=%d rows=%d)", who, hq, hk, cache_rows);
        return SCMX_ERR_ARG;
    }
    if (d != 64 && d != 128 && d != 256) {
        set_error("%s: head dim must be 64, 128 or 256 (d=%d)", who, d);
        return SCMX_ERR_ARG;
    }
    return SCMX_OK;
}

extern "C" int scmx_attn_decode(const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache, const int64_t* pos_dev,
                                int n, uint16_t* out, int hq, int hk, int d, int cache_rows, float scale,
                                float* workspace, int splits, void* stream) {
    if (!q || !kcache || !vcache || !out) {
        set_error("attn_decode: null pointer argument");
        return SCMX_ERR_ARG;
    }
    if (int rc = check_attn("attn_decode", hq, hk, d, cache_rows)) return rc;
    if (uintptr_t(q) % 16 || uintptr_t(kcache) % 16 || uintptr_t(vcache) % 16) {
        set_error("attn_decode: q and the caches must be 16-byte aligned");
        return SCMX_ERR_ARG;
    }
    if (!pos_dev && (n < 1 || n > cache_rows)) {
        set_error("attn_decode: %d valid rows outside 1..%d", n, cache_rows);
        return SCMX_ERR_ARG;
    }
    if (int rc = check_split("attn_decode", workspace, splits)) return rc;
    launch_attn<false>(d, (hipStream_t)stream, q, const_cast<uint16_t*>(kcache), const_cast<uint16_t*>(vcache), pos_dev, n,
                       out, hq, hk, cache_rows, scale, QkvArgs{}, workspace, splits);
    return check_launch("attn_decode");
}

extern "C" int scmx_attn_decode_qkv(const uint16_t* y, const uint16_t* qn, const uint16_t* kn, float eps,
                                    const float* inv_freq, const int64_t* pos_dev, int64_t pos0, uint16_t* kcache,
                                    uint16_t* vcache, uint16_t* out, int hq, int hk, int d, int cache_rows, float scale,
                                    float* workspace, int splits, void* stream) {
    if (!y || !qn || !kn || !inv_freq || !kcache || !vcache || !out) {
        set_error("attn_decode_qkv: null pointer argument");
        return SCMX_ERR_ARG;
    }
    if (int rc = check_attn("attn_decode_qkv", hq, hk, d, cache_rows)) return rc;
    if (uintptr_t(kcache) % 16 || uintptr_t(vcache) % 16) {
        set_error("attn_decode_qkv: caches must be 16-byte aligned");
        return SCMX_ERR_ARG;
    }
    if (!pos_dev && (pos0 < 0 || pos0 >= cache_rows)) {
        set_error("attn_decode_qkv: position %lld outside a cache of %d rows", (long long)pos0, cache_rows);
        return SCMX_ERR_ARG;
    }
    if (int rc = check_split("attn_decode_qkv", workspace, splits)) return rc;
    launch_attn<true>(d, (hipStream_t)stream, nullptr, kcache, vcache, pos_dev, int(pos0) + 1, out, hq, hk, cache_rows, scale,
                      QkvArgs{y, qn, kn, inv_freq, eps}, workspace, splits);
    return check_launch("attn_decode_qkv");
}
