// W4A8 GEMM on CDNA4 INT8 MFMA: dense prefill and grouped mixture-of-experts.
//
// One workgroup computes a BM x BN tile of  acc[m, n] = sum_k xq[m, k] * q[n, k]  in INT32.  Per K step of BK the
// workgroup stages BM x BK activation bytes and BN x BK weight bytes in LDS; the weight bytes are produced in
// registers from the packed 4-bit codes (16 bytes of codes = one run of 32 weights per thread) right before they
// are written to LDS, so the INT8 form of the weights exists only there.  Waves then read 16-byte operand
// fragments and issue v_mfma_i32_32x32x32_i8 with the weights as the row operand: each lane ends up with groups
// of 4 consecutive output columns n of one token row m, which is the unit every epilogue works on.
// LDS is double buffered: global loads for step i+1 are issued before the MFMAs of step i, decoded and stored
// after them, with one barrier per step.
#include "scmx_common.h"

namespace scmx {

struct GemmArgs {
    const int8_t* xq;        // activations INT8 [rows, K]
    const float* xscale;     // [rows]
    const int32_t* gather;   // optional: logical row r reads xq[gather[r]], xscale[gather[r]]
    const uint32_t* codes;   // packed weights [E][N*K/8]
    const uint8_t* bcodes;   // [E][N][bc_row_bytes]
    const int8_t* wq;        // INT8 weights [E*N, K] when the tile is fed from unpacked weights
    const float* wscale;     // [E][N]
    const uint16_t* res;     // [M, N] residual (epilogue 2)
    void* out;
    int M, N, K;             // M = number of logical rows (R for the grouped GEMM)
    int bc_row_bytes;
    int epi;
    const int32_t* off;      // grouped: expert segment offsets [E+1]; dense: NULL
    const int32_t* tstart;   // grouped: first row tile of each expert [E+1]
    int n_experts;
    DevFormat fmt;
};

constexpr int PAD = 16;  // LDS row padding in bytes: consecutive rows start 4 banks apart modulo 64

enum { B_INT8 = 0, B_PACKED_DEFAULT = 1, B_PACKED_GENERIC = 2 };

template <int BM, int BN, int BK, int WGM, int WGN, int BMODE>
__global__ __launch_bounds__(WGM* WGN * 64) void gemm_kernel(const GemmArgs a) {
    constexpr int NT = WGM * WGN * 64;
    constexpr int RS = BK + PAD;             // LDS row stride in bytes
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int MI = WTM / 32, NI = WTN / 32;
    static_assert(WTM % 32 == 0 && WTN % 32 == 0 && BK % 32 == 0, "tile must be whole 32x32x32 MFMAs");
    constexpr int A_CHUNKS = BM * BK / 16;   // 16-byte pieces of the activation tile
    constexpr int A_PER = (A_CHUNKS + NT - 1) / NT;
    constexpr int B_CHUNKS = BMODE == B_INT8 ? BN * BK / 16 : BN * BK / 32;   // 16 bytes of INT8 or of codes
    constexpr int B_PER = (B_CHUNKS + NT - 1) / NT;

    __shared__ __attribute__((aligned(16))) int8_t sA[2][BM * RS];
    __shared__ __attribute__((aligned(16))) int8_t sB[2][BN * RS];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WGM, wn = wave / WGM;

    // ---- which tile ------------------------------------------------------------------------------------------
    const int num_n = (a.N + BN - 1) / BN;
    int m0, n0, row_end, expert = 0;
    if (a.tstart) {   // grouped: row tiles of BM inside expert segments
        const int slot = blockIdx.x / num_n;
        n0 = (blockIdx.x % num_n) * BN;
        const int E = a.n_experts;
        if (slot >= a.tstart[E]) return;
        int lo = 0, hi = E;   // largest e with tstart[e] <= slot
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (a.tstart[mid] <= slot) lo = mid; else hi = mid;
        }
        expert = lo;
        m0 = a.off[expert] + (slot - a.tstart[expert]) * BM;
        row_end = a.off[expert + 1];
    } else {
        const int num_m = (a.M + BM - 1) / BM;
        int pid = blockIdx.x;
        const int total = num_m * num_n;
        if ((total & 7) == 0) pid = (pid & 7) * (total >> 3) + (pid >> 3);   // neighbours in tile order share an XCD
        n0 = (pid / num_m) * BN;
        m0 = (pid % num_m) * BM;
        row_end = a.M;
    }
    const int K = a.K;

    // ---- per-thread staging assignments (fixed over the K loop) ------------------------------------------------
    const int8_t* a_src[A_PER];
    int a_dst[A_PER];
#pragma unroll
    for (int j = 0; j < A_PER; ++j) {
        const int c = tid + j * NT;
        const int row = c / (BK / 16), kc = c % (BK / 16);
        int gr = min(m0 + row, a.M - 1);
        if (a.gather) gr = a.gather[gr];
        a_src[j] = a.xq + size_t(gr) * K + kc * 16;
        a_dst[j] = row * RS + kc * 16;
    }
    const uint8_t* b_src[B_PER];
    const uint8_t* b_bc[B_PER];
    int b_dst[B_PER], b_k[B_PER];
#pragma unroll
    for (int j = 0; j < B_PER; ++j) {
        const int c = tid + j * NT;
        if (BMODE == B_INT8) {
            const int row = c / (BK / 16), kc = c % (BK / 16);
            const int gn = min(n0 + row, a.N - 1);
            b_src[j] = reinterpret_cast<const uint8_t*>(a.wq) + (size_t(expert) * a.N + gn) * K + kc * 16;
            b_dst[j] = row * RS + kc * 16;
            b_bc[j] = nullptr;
            b_k[j] = 0;
        } else {
            const int row = c / (BK / 32), kb = c % (BK / 32);
            const int gn = min(n0 + row, a.N - 1);
            b_src[j] = reinterpret_cast<const uint8_t*>(a.codes) + (size_t(expert) * a.N + gn) * (K / 2) + kb * 16;
            b_bc[j] = a.bcodes + (size_t(expert) * a.N + gn) * a.bc_row_bytes;
            b_dst[j] = row * RS + kb * 32;
            b_k[j] = kb * 32;
        }
    }

    u32x4 ra[A_PER], rb[B_PER];
    uint32_t rbc[B_PER];

    auto load_global = [&](int k0) {
#pragma unroll
        for (int j = 0; j < A_PER; ++j)
            if (A_CHUNKS % NT == 0 || tid + j * NT < A_CHUNKS)
                ra[j] = *reinterpret_cast<const u32x4*>(a_src[j] + k0);
#pragma unroll
        for (int j = 0; j < B_PER; ++j)
            if (B_CHUNKS % NT == 0 || tid + j * NT < B_CHUNKS) {
                if (BMODE == B_INT8) {
                    rb[j] = *reinterpret_cast<const u32x4*>(b_src[j] + k0);
                } else {
                    rb[j] = *reinterpret_cast<const u32x4*>(b_src[j] + (k0 >> 1));
                    if (BMODE == B_PACKED_DEFAULT) {   // 32-blocks, 2-bit codes: 4 blocks per byte
                        const uint32_t blk = uint32_t(k0 + b_k[j]) >> 5;
                        rbc[j] = (uint32_t(b_bc[j][blk >> 2]) >> (2 * (blk & 3))) & 3u;
                    }
                }
            }
    };

    auto store_lds = [&](int buf, int k0) {
#pragma unroll
        for (int j = 0; j < A_PER; ++j)
            if (A_CHUNKS % NT == 0 || tid + j * NT < A_CHUNKS)
                *reinterpret_cast<u32x4*>(&sA[buf][a_dst[j]]) = ra[j];
#pragma unroll
        for (int j = 0; j < B_PER; ++j)
            if (B_CHUNKS % NT == 0 || tid + j * NT < B_CHUNKS) {
                if (BMODE == B_INT8) {
                    *reinterpret_cast<u32x4*>(&sB[buf][b_dst[j]]) = rb[j];
                } else {
                    uint32_t o[8];
                    if (BMODE == B_PACKED_DEFAULT) {
                        const BlockLut t = scaled_lut_shift(0x03020100u, 0x0C080604u, rbc[j]);
#pragma unroll
                        for (int w = 0; w < 4; ++w) decode_word(rb[j][w], t, o[2 * w], o[2 * w + 1]);
                    } else {
#pragma unroll
                        for (int w = 0; w < 4; ++w) {
                            const uint32_t blk = uint32_t(k0 + b_k[j] + 8 * w) >> a.fmt.block_log2;
                            const uint32_t bc = block_code(b_bc[j], blk, a.fmt.bc_bits);
                            const BlockLut t = scaled_lut_mul(a.fmt.lut_lo, a.fmt.lut_hi, mult_of(a.fmt, bc));
                            decode_word(rb[j][w], t, o[2 * w], o[2 * w + 1]);
                        }
                    }
                    *reinterpret_cast<u32x4*>(&sB[buf][b_dst[j]]) = u32x4{o[0], o[1], o[2], o[3]};
                    *reinterpret_cast<u32x4*>(&sB[buf][b_dst[j] + 16]) = u32x4{o[4], o[5], o[6], o[7]};
                }
            }
    };

    v16i acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    // fragment addresses: lane l supplies row l % 32 and the 16 k-bytes of half l / 32 of a 32-wide k slice
    const int frag_off = (lane & 31) * RS + (lane >> 5) * 16;
    const int a_frag = (wm * WTM) * RS + frag_off;
    const int b_frag = (wn * WTN) * RS + frag_off;

    auto mma = [&](int buf) {
#pragma unroll
        for (int kk = 0; kk < BK / 32; ++kk) {
            v4i fa[MI], fb[NI];
#pragma unroll
            for (int i = 0; i < MI; ++i)
                fa[i] = *reinterpret_cast<const v4i*>(&sA[buf][a_frag + i * 32 * RS + kk * 32]);
#pragma unroll
            for (int j = 0; j < NI; ++j)
                fb[j] = *reinterpret_cast<const v4i*>(&sB[buf][b_frag + j * 32 * RS + kk * 32]);
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[j], fa[i], acc[i][j], 0, 0, 0);
        }
    };

    const int KT = K / BK;
    load_global(0);
    store_lds(0, 0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
        const int cur = kt & 1;
        const bool more = kt + 1 < KT;
        if (more) load_global((kt + 1) * BK);
        mma(cur);
        if (more) store_lds(cur ^ 1, (kt + 1) * BK);
        __syncthreads();
    }

    // ---- epilogue: lane holds acc[i][j][4g + r] = (m = tile_m + i*32 + lane%32, n = tile_n + j*32 + 8g + 4(lane/32) + r)
    const int epi = a.epi;
    const int N = a.N;
    const float* ws = a.wscale + size_t(expert) * N;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        const int m = m0 + wm * WTM + i * 32 + (lane & 31);
        if (m >= row_end) continue;
        float xs = 0.0f;
        if (epi != SCMX_EPI_I32) xs = a.xscale[a.gather ? a.gather[m] : m];
#pragma unroll
        for (int j = 0; j < NI; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int n = n0 + wn * WTN + j * 32 + 8 * g + 4 * (lane >> 5);
                if (n >= N) continue;
                if (epi == SCMX_EPI_I32) {
                    *reinterpret_cast<v4i*>(reinterpret_cast<int32_t*>(a.out) + size_t(m) * N + n) =
                        v4i{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                    continue;
                }
                const f32x4 w4 = *reinterpret_cast<const f32x4*>(ws + n);
                float y[4];
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    y[r] = __fmul_rn(__fmul_rn(float(acc[i][j][4 * g + r]), xs), w4[r]);
                uint16_t* out = reinterpret_cast<uint16_t*>(a.out);
                if (epi == SCMX_EPI_SCALE) {
                    u32x2 o;
                    o[0] = uint32_t(f32_to_bf16(y[0])) | (uint32_t(f32_to_bf16(y[1])) << 16);
                    o[1] = uint32_t(f32_to_bf16(y[2])) | (uint32_t(f32_to_bf16(y[3])) << 16);
                    *reinterpret_cast<u32x2*>(out + size_t(m) * N + n) = o;
                } else if (epi == SCMX_EPI_RES) {
                    const u32x2 rr = *reinterpret_cast<const u32x2*>(a.res + size_t(m) * N + n);
                    uint16_t h[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const float rv = __uint_as_float(r & 1 ? (rr[r >> 1] & 0xFFFF0000u) : (rr[r >> 1] << 16));
                        h[r] = f32_to_bf16(__fadd_rn(rv, round_bf16(y[r])));
                    }
                    u32x2 o;
                    o[0] = uint32_t(h[0]) | (uint32_t(h[1]) << 16);
                    o[1] = uint32_t(h[2]) | (uint32_t(h[3]) << 16);
                    *reinterpret_cast<u32x2*>(out + size_t(m) * N + n) = o;
                } else {   // SwiGLU of (g, g, u, u)
                    const uint16_t s0 = swiglu_bf16(round_bf16(y[0]), round_bf16(y[2]));
                    const uint16_t s1 = swiglu_bf16(round_bf16(y[1]), round_bf16(y[3]));
                    *reinterpret_cast<uint32_t*>(out + size_t(m) * (N / 2) + n / 2) = uint32_t(s0) | (uint32_t(s1) << 16);
                }
            }
        }
    }
}

// ---- host dispatch ---------------------------------------------------------------------------------------------

template <int BM, int BN, int BK, int WGM, int WGN>
static void launch_tile(const GemmArgs& a, int bmode, int row_tiles, hipStream_t s) {
    const int num_n = (a.N + BN - 1) / BN;
    const dim3 grid(unsigned(row_tiles) * unsigned(num_n)), block(WGM * WGN * 64);
    if (bmode == B_INT8)
        gemm_kernel<BM, BN, BK, WGM, WGN, B_INT8><<<grid, block, 0, s>>>(a);
    else if (bmode == B_PACKED_DEFAULT)
        gemm_kernel<BM, BN, BK, WGM, WGN, B_PACKED_DEFAULT><<<grid, block, 0, s>>>(a);
    else
        gemm_kernel<BM, BN, BK, WGM, WGN, B_PACKED_GENERIC><<<grid, block, 0, s>>>(a);
}

// Dense: the largest tile that still gives every CU a workgroup.
static void launch_dense(const GemmArgs& a, int bmode, hipStream_t s) {
    const long cus = 256;
    auto tiles = [&](int bm, int bn) { return long((a.M + bm - 1) / bm) * ((a.N + bn - 1) / bn); };
    if (tiles(256, 128) >= cus) return launch_tile<256, 128, 128, 4, 2>(a, bmode, (a.M + 255) / 256, s);
    if (tiles(256, 64) >= cus) return launch_tile<256, 64, 128, 4, 2>(a, bmode, (a.M + 255) / 256, s);
    if (tiles(128, 128) >= cus) return launch_tile<128, 128, 128, 4, 2>(a, bmode, (a.M + 127) / 128, s);
    if (tiles(128, 64) >= cus) return launch_tile<128, 64, 128, 4, 2>(a, bmode, (a.M + 127) / 128, s);
    return launch_tile<64, 64, 128, 2, 2>(a, bmode, (a.M + 63) / 64, s);
}

static int check_gemm_common(const char* who, int M, int N, int K, int epi, bool need_scales, const void* xq,
                             const float* xscale, const float* wscale, const uint16_t* res, const void* out) {
    if (M < 0 || N <= 0 || K <= 0 || K % 128 || N % 4) {
        set_error("%s: need M >= 0, N %% 4 == 0 and K %% 128 == 0 (M=%d N=%d K=%d)", who, M, N, K);
        return SCMX_ERR_ARG;
    }
    if (epi < 0 || epi > 3) {
        set_error("%s: unknown epilogue %d", who, epi);
        return SCMX_ERR_ARG;
    }
    if (!xq || !out || (need_scales && epi != SCMX_EPI_I32 && (!xscale || !wscale)) || (epi == SCMX_EPI_RES && !res)) {
        set_error("%s: null pointer argument", who);
        return SCMX_ERR_ARG;
    }
    if (uintptr_t(xq) % 16 || uintptr_t(out) % 16 || uintptr_t(wscale) % 16 || uintptr_t(res) % 8) {
        set_error("%s: xq / out / wscale must be 16-byte aligned (res 8-byte)", who);
        return SCMX_ERR_ARG;
    }
    if (epi == SCMX_EPI_SWIGLU && N % 8) {
        set_error("%s: the SwiGLU epilogue needs N %% 8 == 0", who);
        return SCMX_ERR_ARG;
    }
    return SCMX_OK;
}

}  // namespace scmx

using namespace scmx;

extern "C" {

int scmx_mm_epi(const int8_t* xq, const int8_t* wq, const float* xscale, const float* wscale, const uint16_t* res,
                void* out, int epi, int M, int N, int K, void* stream) {
    if (int rc = check_gemm_common("mm_epi", M, N, K, epi, true, xq, xscale, wscale, res, out)) return rc;
    if (!wq || uintptr_t(wq) % 16) {
        set_error("mm_epi: wq must be non-null and 16-byte aligned");
        return SCMX_ERR_ARG;
    }
    if (M == 0) return SCMX_OK;
    GemmArgs a = {};
    a.xq = xq; a.xscale = xscale; a.wq = wq; a.wscale = wscale; a.res = res; a.out = out;
    a.M = M; a.N = N; a.K = K; a.epi = epi;
    launch_dense(a, B_INT8, (hipStream_t)stream);
    return check_launch("mm_epi");
}

int scmx_mm_i8_i32(const int8_t* xq, const int8_t* wq, int32_t* acc, int M, int N, int K, void* stream) {
    return scmx_mm_epi(xq, wq, nullptr, nullptr, nullptr, acc, SCMX_EPI_I32, M, N, K, stream);
}

int scmx_mm_w4a8(const scmx_format* fmt, const int8_t* xq, const float* xscale, const uint32_t* codes,
                 const uint8_t* bcodes, const float* wscale, const uint16_t* res, void* out, int epi, int M, int N,
                 int K, void* stream) {
    DevFormat f;
    if (int rc = make_dev_format(fmt, &f)) return rc;
    if (int rc = check_gemm_common("mm_w4a8", M, N, K, epi, true, xq, xscale, wscale, res, out)) return rc;
    if (!codes || !bcodes || uintptr_t(codes) % 16 || K % f.block || (K / f.block * f.bc_bits) % 8) {
        set_error("mm_w4a8: codes must be 16-byte aligned, K a multiple of the block with whole block-code bytes per row");
        return SCMX_ERR_ARG;
    }
    if (M == 0) return SCMX_OK;
    GemmArgs a = {};
    a.xq = xq; a.xscale = xscale; a.codes = codes; a.bcodes = bcodes; a.wscale = wscale; a.res = res; a.out = out;
    a.M = M; a.N = N; a.K = K; a.epi = epi; a.fmt = f;
    a.bc_row_bytes = K / f.block * f.bc_bits / 8;
    launch_dense(a, is_default_format(f) ? B_PACKED_DEFAULT : B_PACKED_GENERIC, (hipStream_t)stream);
    return check_launch("mm_w4a8");
}

size_t scmx_linear_w4a8_workspace(int M, int K) {
    const size_t q = (size_t(M) * size_t(K) + 255) & ~size_t(255);
    return q + size_t(M) * sizeof(float);
}

int scmx_linear_w4a8(const scmx_format* fmt, const uint16_t* x, const uint32_t* codes, const uint8_t* bcodes,
                     const float* wscale, const uint16_t* res, void* out, int epi, int M, int N, int K,
                     void* workspace, size_t workspace_bytes, void* stream) {
    if (M < 0 || K <= 0) {
        set_error("linear_w4a8: bad shape M=%d K=%d", M, K);
        return SCMX_ERR_ARG;
    }
    if (!workspace || workspace_bytes < scmx_linear_w4a8_workspace(M, K) || uintptr_t(workspace) % 256) {
        set_error("linear_w4a8: workspace must be 256-byte aligned and hold %zu bytes",
                  scmx_linear_w4a8_workspace(M, K));
        return SCMX_ERR_WORKSPACE;
    }
    int8_t* xq = reinterpret_cast<int8_t*>(workspace);
    float* xs = reinterpret_cast<float*>(xq + ((size_t(M) * size_t(K) + 255) & ~size_t(255)));
    if (int rc = scmx_act_quant(x, xq, xs, M, M, K, stream)) return rc;
    return scmx_mm_w4a8(fmt, xq, xs, codes, bcodes, wscale, res, out, epi, M, N, K, stream);
}

static int moe_common(const char* who, const int8_t* xq, const float* xscale, const int32_t* gather, int R,
                      const float* wscale, const int32_t* off, const int32_t* tstart, int n_experts, int tm, int N,
                      int K, int epi, void* out, GemmArgs* a) {
    if (epi == SCMX_EPI_RES) {
        set_error("%s: the grouped GEMM has no residual epilogue", who);
        return SCMX_ERR_ARG;
    }
    if (int rc = check_gemm_common(who, R, N, K, epi, true, xq, xscale, wscale, nullptr, out)) return rc;
    if (!off || !tstart || n_experts < 1 || !(tm == 64 || tm == 128)) {
        set_error("%s: need off / tstart, n_experts >= 1 and a row tile of 64 or 128 (got %d)", who, tm);
        return SCMX_ERR_ARG;
    }
    *a = GemmArgs{};
    a->xq = xq; a->xscale = xscale; a->gather = gather; a->wscale = wscale; a->out = out;
    a->M = R; a->N = N; a->K = K; a->epi = epi; a->off = off; a->tstart = tstart; a->n_experts = n_experts;
    return SCMX_OK;
}

static void launch_grouped(const GemmArgs& a, int bmode, int tm, hipStream_t s) {
    const int max_tiles = (a.M + tm - 1) / tm + a.n_experts;   // e2e/sc_moe.py:155
    if (tm == 128)
        launch_tile<128, 128, 128, 4, 2>(a, bmode, max_tiles, s);
    else
        launch_tile<64, 128, 128, 2, 4>(a, bmode, max_tiles, s);
}

int scmx_moe_mm(const scmx_format* fmt, const int8_t* xq, const float* xscale, const int32_t* gather, int R,
                const uint32_t* codes, const uint8_t* bcodes, const float* wscale, const int32_t* off,
                const int32_t* tstart, int n_experts, int tm, int N, int K, int epi, void* out, void* stream) {
    DevFormat f;
    if (int rc = make_dev_format(fmt, &f)) return rc;
    GemmArgs a;
    if (int rc = moe_common("moe_mm", xq, xscale, gather, R, wscale, off, tstart, n_experts, tm, N, K, epi, out, &a))
        return rc;
    if (!codes || !bcodes || uintptr_t(codes) % 16 || K % f.block || (K / f.block * f.bc_bits) % 8) {
        set_error("moe_mm: codes must be 16-byte aligned, K a multiple of the block with whole block-code bytes per row");
        return SCMX_ERR_ARG;
    }
    if (R == 0) return SCMX_OK;
    a.codes = codes; a.bcodes = bcodes; a.fmt = f;
    a.bc_row_bytes = K / f.block * f.bc_bits / 8;
    launch_grouped(a, is_default_format(f) ? B_PACKED_DEFAULT : B_PACKED_GENERIC, tm, (hipStream_t)stream);
    return check_launch("moe_mm");
}

int scmx_moe_mm_i8(const int8_t* xq, const float* xscale, const int32_t* gather, int R, const int8_t* wq,
                   const float* wscale, const int32_t* off, const int32_t* tstart, int n_experts, int tm, int N,
                   int K, int epi, void* out, void* stream) {
    GemmArgs a;
    if (int rc = moe_common("moe_mm_i8", xq, xscale, gather, R, wscale, off, tstart, n_experts, tm, N, K, epi, out, &a))
        return rc;
    if (!wq || uintptr_t(wq) % 16) {
        set_error("moe_mm_i8: wq must be non-null and 16-byte aligned");
        return SCMX_ERR_ARG;
    }
    if (R == 0) return SCMX_OK;
    a.wq = wq;
    launch_grouped(a, B_INT8, tm, (hipStream_t)stream);
    return check_launch("moe_mm_i8");
}

}  // extern "C"
