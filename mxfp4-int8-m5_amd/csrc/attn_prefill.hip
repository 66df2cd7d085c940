// Causal attention of a block of L new tokens against a KV cache that already holds `off` earlier rows (prefill):
// out[i] = softmax(q[i] . K[0 .. off+i]^T * scale) V[0 .. off+i] per query head, grouped-query sharing of the KV heads.
//
// The linear layers are the product here; this kernel exists because the attention between them is a third of the
// prefill time with the array library's kernel.  One workgroup of eight waves owns 128 consecutive queries of one head:
// four blocks of 32 queries times two halves of the keys.  The keys are walked in pairs of 64-key tiles with a running
// maximum and sum (one pass over K and V); wave (block, half) multiplies the pair's tile `half`, and the two halves
// of a block are merged through LDS at the end.  Splitting the keys inside the workgroup halves the longest serial
// chain (the last query tile sees every key) and puts two waves on every SIMD, and eight waves share what is staged.
//
// Everything is computed transposed, so that no operand has to change lanes between the two matrix products:
//   S^T = K Q^T    (v_mfma_f32_32x32x16_bf16: rows = keys, columns = queries, contraction over the head dimension)
//   O^T = V^T P^T  (rows = head dimension, columns = queries, contraction over keys)
// A lane's column of an accumulator tile is one query (lane % 32), so the softmax statistics of a query live in two
// lanes (lane, lane ^ 32), the rescaling of O^T is a per-lane multiply, and the S^T accumulators, converted to bf16,
// already are the column operand of the second product: register 4g + r of a 32 x 32 tile holds key 8g + 4h + r
// (h = lane / 32), so the 16-key slice s takes g = 2s, 2s + 1, and V^T is read with the same key order.
// K tiles sit in LDS row by row (272-byte rows: conflict-free 16-byte fragment reads), V tiles transposed (a row per
// head-dimension index, 144 bytes), written as pairs of keys so that a wave's LDS stores cover distinct words; inside
// every 16-key slice the middle two groups of four keys change places, which puts the 8 keys of a lane half (4h + r
// and 8 + 4h + r) next to each other: one 16-byte read per fragment.
// Pairs of tiles are double-buffered in LDS and the global loads of the pair after the next one are in flight in
// registers while the current one is multiplied: one barrier per pair.  Query tiles are launched last to first (the last one sees the most keys).
#include "scmx_common.h"

namespace scmx {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int FA_NT = 512;                  // eight waves: (query block, key half)
constexpr int FA_BM = 128, FA_BN = 64, FA_D = 128;
constexpr int FA_KROW = FA_D * 2 + 16;      // bytes per K row in LDS
constexpr int FA_VROW = FA_BN * 2 + 16;     // bytes per V^T row in LDS
constexpr int FA_KBYTES = FA_BN * FA_KROW;
constexpr int FA_VBYTES = FA_D * FA_VROW;

__global__ __launch_bounds__(FA_NT) void attn_prefill_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ kc,
                                                             const uint16_t* __restrict__ vc, uint16_t* __restrict__ out,
                                                             int L, int off, int hq, int hk, int rows, float scale_log2) {
    __shared__ __attribute__((aligned(16))) uint8_t smem[2][2][FA_KBYTES + FA_VBYTES];   // [buffer][tile of the pair]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, ln = lane & 31, h = lane >> 5;
    const int num_qt = (L + FA_BM - 1) / FA_BM;
    const int qt = num_qt - 1 - int(blockIdx.x);
    const int head = blockIdx.y, kvh = head / (hq / hk);
    const int qb = wave & 3, kh = wave >> 2;   // query block and key half of this wave
    const int q0 = qt * FA_BM, qw0 = q0 + qb * 32;
    const int n = off + L;   // valid cache rows

    // this lane's query as the column operand of S^T: 8 consecutive head-dimension values per 16-wide slice
    bf16x8 qf[FA_D / 16];
    {
        const uint16_t* qp = q + (size_t(min(qw0 + ln, L - 1)) * hq + head) * FA_D + 8 * h;
#pragma unroll
        for (int s = 0; s < FA_D / 16; ++s) qf[s] = *reinterpret_cast<const bf16x8*>(qp + 16 * s);
    }
    f32x16 o[FA_D / 32];
#pragma unroll
    for (int db = 0; db < FA_D / 32; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[db][r] = 0.0f;
    float m = -1.0e30f, l = 0.0f;

    const int kv_end = off + min(q0 + FA_BM, L);   // the tile's last query sees keys [0, kv_end)
    const int ntile = (kv_end + FA_BN - 1) / FA_BN;
    const uint16_t* kb = kc + size_t(kvh) * rows * FA_D;
    const uint16_t* vb = vc + size_t(kvh) * rows * FA_D;

    const int npair = (ntile + 1) / 2;

    // staging of a pair of tiles: K as 16-byte pieces (tile = c / 1024, key = c / 16 % 64, piece = c % 16), V as pairs of
    // keys (tile = c / 512, pair = c % 32, piece = c / 32 % 16)
    constexpr int KJ = 2 * FA_BN * 16 / FA_NT, VJ = 2 * (FA_BN / 2) * 16 / FA_NT;
    u32x4 kr[KJ], va[VJ], vb2[VJ];
    auto load_pair = [&](int i) {
#pragma unroll
        for (int j = 0; j < KJ; ++j) {
            const int c = tid + FA_NT * j;
            const int key = min((2 * i + c / 1024) * FA_BN + (c / 16) % FA_BN, n - 1);
            kr[j] = *reinterpret_cast<const u32x4*>(kb + size_t(key) * FA_D + (c % 16) * 8);
        }
#pragma unroll
        for (int j = 0; j < VJ; ++j) {
            const int c = tid + FA_NT * j;
            const int key = (2 * i + c / 512) * FA_BN + 2 * (c % 32);
            const int piece = (c / 32) % 16;
            va[j] = *reinterpret_cast<const u32x4*>(vb + size_t(min(key, n - 1)) * FA_D + piece * 8);
            vb2[j] = *reinterpret_cast<const u32x4*>(vb + size_t(min(key + 1, n - 1)) * FA_D + piece * 8);
        }
    };
    auto store_pair = [&](int buf) {
#pragma unroll
        for (int j = 0; j < KJ; ++j) {
            const int c = tid + FA_NT * j;
            *reinterpret_cast<u32x4*>(smem[buf][c / 1024] + ((c / 16) % FA_BN) * FA_KROW + (c % 16) * 16) = kr[j];
        }
#pragma unroll
        for (int j = 0; j < VJ; ++j) {
            const int c = tid + FA_NT * j;
            uint8_t* vs = smem[buf][c / 512] + FA_KBYTES;
            const int pair = c % 32, piece = (c / 32) % 16;
            const int kk = 2 * pair;   // first key of the pair; its place in the row: bits 2 and 3 of the key index swapped
            const int place = (kk & ~12) | ((kk & 4) << 1) | ((kk & 8) >> 1);
#pragma unroll
            for (int i = 0; i < 8; ++i) {   // head-dimension index piece * 8 + i: the two keys' values side by side
                const uint32_t w = perm(vb2[j][i / 2], va[j][i / 2], (i & 1) ? 0x07060302u : 0x05040100u);
                *reinterpret_cast<uint32_t*>(vs + (piece * 8 + i) * FA_VROW + place * 2) = w;
            }
        }
    };

    load_pair(0);
    store_pair(0);
    if (npair > 1) load_pair(1);
    __syncthreads();
    for (int i = 0; i < npair; ++i) {
        const int t = 2 * i + kh;
        const int kv0 = t * FA_BN;
        if (kv0 <= off + qw0 + 31) {   // some key of the tile is visible to some query of this wave
            const uint8_t* ks = smem[i & 1][kh];
            const uint8_t* vs = smem[i & 1][kh] + FA_KBYTES;
            f32x16 sacc[2];
#pragma unroll
            for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                for (int r = 0; r < 16; ++r) sacc[blk][r] = 0.0f;
#pragma unroll
            for (int s = 0; s < FA_D / 16; ++s)   // the two key blocks are independent accumulation chains: alternate them
#pragma unroll
                for (int blk = 0; blk < 2; ++blk) {
                    const bf16x8 a = *reinterpret_cast<const bf16x8*>(ks + (blk * 32 + ln) * FA_KROW + 32 * s + 16 * h);
                    sacc[blk] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[s], sacc[blk], 0, 0, 0);
                }
            // running maximum of the raw scores; tiles that reach past the wave's first query are masked first
            if (kv0 + FA_BN - 1 > off + qw0) {
                const int limit = off + qw0 + ln - kv0;   // keys with tile index <= limit are visible to this query
#pragma unroll
                for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                    for (int g = 0; g < 4; ++g)
#pragma unroll
                        for (int r = 0; r < 4; ++r)
                            if (blk * 32 + 8 * g + 4 * h + r > limit) sacc[blk][4 * g + r] = -1.0e30f;
            }
            float mx = -1.0e30f;
#pragma unroll
            for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sacc[blk][r]);
            mx = fmaxf(mx, __shfl_xor(mx, 32, WAVE));
            const float mn = fmaxf(m, mx);               // in units of raw scores; the softmax scale enters the exponent
            const float alpha = __builtin_amdgcn_exp2f((m - mn) * scale_log2);
            const float shift = mn * scale_log2;
            m = mn;
            float ls = 0.0f;
            bf16x8 pb[FA_BN / 16];   // P^T as the column operand: slice s holds registers g = 2s, 2s + 1 of its block
#pragma unroll
            for (int blk = 0; blk < 2; ++blk)
#pragma unroll
                for (int g = 0; g < 4; ++g)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[blk][4 * g + r], scale_log2, -shift));
                        ls += p;
                        pb[blk * 2 + g / 2][(g & 1) * 4 + r] = (__bf16)p;
                    }
            l = l * alpha + ls;
            const bool rescale = __builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0;   // no query's maximum moved: skip
            if (rescale) {
#pragma unroll
                for (int db = 0; db < FA_D / 32; ++db)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o[db][r] *= alpha;
            }
#pragma unroll
            for (int s = 0; s < FA_BN / 16; ++s)   // four independent chains (head-dimension blocks) per key slice
#pragma unroll
                for (int db = 0; db < FA_D / 32; ++db) {
                    // keys 16s + 4h + (0..3) and 16s + 8 + 4h + (0..3) of head-dimension row db * 32 + ln
                    const bf16x8 a = *reinterpret_cast<const bf16x8*>(vs + (db * 32 + ln) * FA_VROW + 32 * s + 16 * h);
                    o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[s], o[db], 0, 0, 0);
                }
        }
        if (i + 1 < npair) {   // the other buffer was last read one barrier ago
            store_pair((i + 1) & 1);
            if (i + 2 < npair) load_pair(i + 2);   // the registers are free again
        }
        __syncthreads();
    }

    // merge the two key halves of every query block: the second half parks its state in LDS, the first one folds it in
    float* park = reinterpret_cast<float*>(&smem[0][0][0]) + qb * (FA_D / 32 * 16 + 2) * 64;
    if (kh == 1) {
#pragma unroll
        for (int db = 0; db < FA_D / 32; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) park[(db * 16 + r) * 64 + lane] = o[db][r];
        park[(FA_D / 32 * 16) * 64 + lane] = m;
        park[(FA_D / 32 * 16 + 1) * 64 + lane] = l;
    }
    __syncthreads();
    if (kh == 1) return;
    {
        const float m2 = park[(FA_D / 32 * 16) * 64 + lane], l2 = park[(FA_D / 32 * 16 + 1) * 64 + lane];
        const float mn = fmaxf(m, m2);
        const float a1 = __builtin_amdgcn_exp2f((m - mn) * scale_log2), a2 = __builtin_amdgcn_exp2f((m2 - mn) * scale_log2);
        l = l * a1 + l2 * a2;
#pragma unroll
        for (int db = 0; db < FA_D / 32; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[db][r] = o[db][r] * a1 + park[(db * 16 + r) * 64 + lane] * a2;
    }
    l += __shfl_xor(l, 32, WAVE);
    const float inv = 1.0f / l;
    const int query = qw0 + ln;
    if (query < L) {
        uint16_t* op = out + (size_t(query) * hq + head) * FA_D;
#pragma unroll
        for (int db = 0; db < FA_D / 32; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                u32x2 w;
                w[0] = uint32_t(f32_to_bf16(o[db][4 * g] * inv)) | (uint32_t(f32_to_bf16(o[db][4 * g + 1] * inv)) << 16);
                w[1] = uint32_t(f32_to_bf16(o[db][4 * g + 2] * inv)) | (uint32_t(f32_to_bf16(o[db][4 * g + 3] * inv)) << 16);
                *reinterpret_cast<u32x2*>(op + db * 32 + 8 * g + 4 * h) = w;
            }
    }
}

}  // namespace scmx

using namespace scmx;

extern "C" int scmx_attn_prefill(const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache, uint16_t* out, int L,
                                 int off, int hq, int hk, int d, int cache_rows, float scale, void* stream) {
    if (!q || !kcache || !vcache || !out) {
        set_error("attn_prefill: null pointer argument");
        return SCMX_ERR_ARG;
    }
    if (hq < 1 || hk < 1 || hq > 65535 || hq % hk || d != FA_D) {
        set_error("attn_prefill: need hq %% hk == 0 and head dim %d (hq=%d hk=%d d=%d)", FA_D, hq, hk, d);
        return SCMX_ERR_ARG;
    }
    if (!(scale > 0.0f)) {   // the running maximum is kept on the unscaled scores
        set_error("attn_prefill: scale must be positive");
        return SCMX_ERR_ARG;
    }
    if (L < 0 || off < 0 || int64_t(off) + L > cache_rows) {
        set_error("attn_prefill: rows %d..%lld do not fit a cache of %d rows", off, (long long)off + L, cache_rows);
        return SCMX_ERR_ARG;
    }
    if (uintptr_t(q) % 16 || uintptr_t(kcache) % 16 || uintptr_t(vcache) % 16 || uintptr_t(out) % 8) {
        set_error("attn_prefill: q / caches must be 16-byte aligned, out 8-byte");
        return SCMX_ERR_ARG;
    }
    if (L == 0) return SCMX_OK;
    const dim3 grid((L + FA_BM - 1) / FA_BM, hq), block(FA_NT);
    attn_prefill_kernel<<<grid, block, 0, (hipStream_t)stream>>>(q, kcache, vcache, out, L, off, hq, hk, cache_rows,
                                                                 scale * 1.4426950408889634f);
    return check_launch("attn_prefill");
}
