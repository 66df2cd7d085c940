// Library plumbing (errors, format validation) and the small memory-bound kernels: weight unpack, activation
// quantization, standard-MXFP4 scale conversion.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <atomic>

#include "scmx_common.h"

namespace scmx {

static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: %s", what, hipGetErrorString(e));
        return SCMX_ERR_LAUNCH;
    }
    return SCMX_OK;
}

// Compute units of the current device, asked once per device (256 on MI355X; the fallback when the query fails).
int device_cus() {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n <= 0) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

int make_dev_format(const scmx_format* f, DevFormat* out) {
    if (!f) {
        set_error("format is NULL");
        return SCMX_ERR_ARG;
    }
    const int b = f->block;
    if (!(b == 8 || b == 16 || b == 32 || b == 64 || b == 128)) {
        set_error("format: block %d not in {8,16,32,64,128}", b);
        return SCMX_ERR_FORMAT;
    }
    if (b == 32 && f->bc_bits == 8 && f->n_mult == 0) {   // standard MXFP4: E8M0 bytes in place of block codes
        const int mag[8] = {0, 1, 2, 3, 4, 6, 8, 12};
        for (int i = 0; i < 8; ++i)
            if (f->code_mag[i] != mag[i]) {
                set_error("format: the E8M0 form takes the E2M1 code magnitudes 0,1,2,3,4,6,8,12");
                return SCMX_ERR_FORMAT;
            }
        DevFormat d;
        memset(&d, 0, sizeof(d));
        d.lut_lo = 0x03020100u;
        d.lut_hi = 0x0C080604u;
        d.mult[0] = 0x08040201u;
        d.block = 32;
        d.block_log2 = 5;
        d.bc_bits = 8;
        d.pow2 = 1;
        d.e8m0 = 1;
        *out = d;
        return SCMX_OK;
    }
    if (!(f->bc_bits == 1 || f->bc_bits == 2 || f->bc_bits == 4 || f->bc_bits == 8) || f->n_mult < 1 ||
        f->n_mult > 16 || f->n_mult > (1 << f->bc_bits)) {
        set_error("format: bc_bits %d / n_mult %d unsupported (need bc_bits in {1,2,4,8}, n_mult <= min(16, 2^bc_bits))",
                  f->bc_bits, f->n_mult);
        return SCMX_ERR_FORMAT;
    }
    int mag_max = 0, mult_max = 0;
    for (int i = 0; i < 8; ++i) {
        if (f->code_mag[i] < 0 || f->code_mag[i] > 127) {
            set_error("format: code_mag[%d] = %d outside 0..127", i, f->code_mag[i]);
            return SCMX_ERR_FORMAT;
        }
        mag_max = f->code_mag[i] > mag_max ? f->code_mag[i] : mag_max;
    }
    for (int i = 0; i < f->n_mult; ++i) {
        if (f->mult[i] < 1 || f->mult[i] > 127) {
            set_error("format: mult[%d] = %d outside 1..127", i, f->mult[i]);
            return SCMX_ERR_FORMAT;
        }
        mult_max = f->mult[i] > mult_max ? f->mult[i] : mult_max;
    }
    if (mag_max * mult_max > 127) {
        set_error("format: max(code_mag) * max(mult) = %d does not fit INT8", mag_max * mult_max);
        return SCMX_ERR_FORMAT;
    }
    DevFormat d;
    memset(&d, 0, sizeof(d));
    for (int i = 0; i < 4; ++i) {
        d.lut_lo |= uint32_t(f->code_mag[i]) << (8 * i);
        d.lut_hi |= uint32_t(f->code_mag[4 + i]) << (8 * i);
    }
    d.pow2 = 1;
    for (int i = 0; i < f->n_mult; ++i) {
        d.mult[i >> 2] |= uint32_t(f->mult[i]) << (8 * (i & 3));
        if (f->mult[i] != (1 << i)) d.pow2 = 0;
    }
    d.block = b;
    d.block_log2 = b == 8 ? 3 : b == 16 ? 4 : b == 32 ? 5 : b == 64 ? 6 : 7;
    d.bc_bits = f->bc_bits;
    *out = d;
    return SCMX_OK;
}

// ---- unpack_i8: one thread per 16-byte group of codes (32 weights) ---------------------------------------------
__global__ __launch_bounds__(256) void unpack_i8_kernel(DevFormat f, const u32x4* __restrict__ codes,
                                                        const uint8_t* __restrict__ bcodes, u32x4* __restrict__ wq,
                                                        int64_t n_groups, int groups_per_row, int bc_row_bytes) {
    const int64_t g = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (g >= n_groups) return;
    const int64_t row = g / groups_per_row;
    const uint32_t k0 = uint32_t(g % groups_per_row) * 32u;
    const u32x4 w = codes[g];
    const uint8_t* row_bc = bcodes + row * bc_row_bytes;
    uint32_t o[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t bc = block_code(row_bc, (k0 + 8u * j) >> f.block_log2, f.bc_bits);
        const BlockLut t = scaled_lut_mul(f.lut_lo, f.lut_hi, mult_of(f, bc));
        decode_word(w[j], t, o[2 * j], o[2 * j + 1]);
    }
    wq[2 * g] = u32x4{o[0], o[1], o[2], o[3]};
    wq[2 * g + 1] = u32x4{o[4], o[5], o[6], o[7]};
}

// Fallback for K not a multiple of 32: one thread per code word (8 weights).
__global__ __launch_bounds__(256) void unpack_i8_word_kernel(DevFormat f, const uint32_t* __restrict__ codes,
                                                             const uint8_t* __restrict__ bcodes,
                                                             u32x2* __restrict__ wq, int64_t n_words,
                                                             int words_per_row, int bc_row_bytes) {
    const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (i >= n_words) return;
    const int64_t row = i / words_per_row;
    const uint32_t k0 = uint32_t(i % words_per_row) * 8u;
    const uint32_t bc = block_code(bcodes + row * bc_row_bytes, k0 >> f.block_log2, f.bc_bits);
    const BlockLut t = scaled_lut_mul(f.lut_lo, f.lut_hi, mult_of(f, bc));
    uint32_t a, b;
    decode_word(codes[i], t, a, b);
    wq[i] = u32x2{a, b};
}

// ---- act_quant: one workgroup per token row ---------------------------------------------------------------------
// Lanes read 8 bf16 (16 bytes) per step; the row maximum goes through LDS; the second sweep re-reads the row
// (cache hit) and writes 8 codes per lane.
__global__ __launch_bounds__(256) void act_quant_kernel(const uint16_t* __restrict__ x, int8_t* __restrict__ xq,
                                                        float* __restrict__ xs, int M, int K) {
    __shared__ float red[4];
    const int row = blockIdx.x, tid = threadIdx.x;
    u32x2* qrow = reinterpret_cast<u32x2*>(xq + size_t(row) * K);
    if (row >= M) {
        for (int c = tid; c < K / 8; c += 256) qrow[c] = u32x2{0u, 0u};
        if (tid == 0) xs[row] = 0.0f;
        return;
    }
    const u32x4* xrow = reinterpret_cast<const u32x4*>(x + size_t(row) * K);
    float amax = 0.0f;
    for (int c = tid; c < K / 8; c += 256) {
        const u32x4 v = xrow[c];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            amax = fmaxf(amax, fabsf(__uint_as_float(v[j] << 16)));
            amax = fmaxf(amax, fabsf(__uint_as_float(v[j] & 0xFFFF0000u)));
        }
    }
    amax = wave_max(amax);
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float s = __fdiv_rn(amax, 127.0f);
    const float qi = s > 0.0f ? __fdiv_rn(1.0f, s) : 0.0f;
    for (int c = tid; c < K / 8; c += 256) {
        const u32x4 v = xrow[c];
        uint32_t o[2] = {0u, 0u};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int q0 = quant_code(__uint_as_float(v[j] << 16), qi);
            const int q1 = quant_code(__uint_as_float(v[j] & 0xFFFF0000u), qi);
            o[j >> 1] |= (uint32_t(q0) & 0xFFu) << (16 * (j & 1));
            o[j >> 1] |= (uint32_t(q1) & 0xFFu) << (16 * (j & 1) + 8);
        }
        qrow[c] = u32x2{o[0], o[1]};
    }
    if (tid == 0) xs[row] = s;
}

// The same with the row held in registers: one wave per row, lane l owns the 16-byte pieces l, l + 64, ... (CH of
// them, K = 512 * CH), so the row is read once and the only reduction is inside the wave.  Four rows per workgroup.
// BLK: xq leaves in the blocked layout of the dense GEMM's large tiles (32 x 32 blocks in MFMA operand order, described at
// act_quant_blocked_kernel below; Mp % 32 == 0): eight rows per workgroup, whose codes meet in LDS -- the 16 bytes of row
// r, k 16 c ... at slot c * 8 + (r + c / 2) % 8 -- and are stored as whole 128-byte lines (8 rows x 16 bytes are adjacent
// in a block).  The loads stay what they are by rows: 16 contiguous bytes per lane.
template <int CH, bool BLK = false>
__global__ __launch_bounds__(BLK ? 512 : 256) void act_quant_wave_kernel(const uint16_t* __restrict__ x, int8_t* __restrict__ xq,
                                                                         float* __restrict__ xs, int M, int Mp) {
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
    if (row >= M) {
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            if (BLK) tile[slot(lane + 64 * j)] = u32x2{0u, 0u}; else qrow[lane + 64 * j] = u32x2{0u, 0u};
        }
        if (lane == 0) xs[row] = 0.0f;
        if (BLK) gather_store();
        return;
    }
    const u32x4* xrow = reinterpret_cast<const u32x4*>(x + size_t(row) * K);
    u32x4 v[CH];
#pragma unroll
    for (int j = 0; j < CH; ++j) v[j] = xrow[lane + 64 * j];
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < CH; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            amax = fmaxf(amax, fabsf(__uint_as_float(v[j][e] << 16)));
            amax = fmaxf(amax, fabsf(__uint_as_float(v[j][e] & 0xFFFF0000u)));
        }
    amax = wave_max(amax);
    const float s = __fdiv_rn(amax, 127.0f);
    const float qi = s > 0.0f ? __fdiv_rn(1.0f, s) : 0.0f;
#pragma unroll
    for (int j = 0; j < CH; ++j) {
        uint32_t o[2] = {0u, 0u};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int q0 = quant_code(__uint_as_float(v[j][e] << 16), qi);
            const int q1 = quant_code(__uint_as_float(v[j][e] & 0xFFFF0000u), qi);
            o[e >> 1] |= (uint32_t(q0) & 0xFFu) << (16 * (e & 1));
            o[e >> 1] |= (uint32_t(q1) & 0xFFu) << (16 * (e & 1) + 8);
        }
        if (BLK) tile[slot(lane + 64 * j)] = u32x2{o[0], o[1]}; else qrow[lane + 64 * j] = u32x2{o[0], o[1]};
    }
    if (lane == 0) xs[row] = s;
    if (BLK) gather_store();
}

// ---- act_quant into the blocked layout ---------------------------------------------------------------------------
// xq as the large dense GEMM tiles take it: blocks of 32 rows x 32 k (1 KB), block (m / 32, k / 32) at
// ((m / 32) * (K / 32) + k / 32) KB, and inside a block the 16 bytes of row r, k half h at (32 h + r) * 16 -- the order
// in which the 64 lanes of a wave hold a 32x32x32 MFMA operand, so that a wave fetches one block with one coalesced load.
// Rows of K = 512 ... 8192 in steps of 512 go through act_quant_wave_kernel<CH, true> above; this is the kernel for every
// other K % 32 == 0: one wave per row, eight rows per workgroup, the row read twice, every lane writing the 16 bytes of
// its own 16 elements.  Same codes and scales as act_quant_kernel: the row maximum does not depend on the order it is
// taken in.
__global__ __launch_bounds__(512) void act_quant_blocked_kernel(const uint16_t* __restrict__ x, int8_t* __restrict__ xq,
                                                                float* __restrict__ xs, int M, int Mp, int K) {
    const int row = blockIdx.x * 8 + (threadIdx.x >> 6), lane = threadIdx.x & 63;   // Mp % 32 == 0: whole groups of 8 rows
    const int pieces = K / 16;
    // piece c of the row (k = 16 c ...): k slice c / 2, half c % 2
    int8_t* const dst = xq + (size_t(row >> 5) * size_t(K >> 5)) * 1024 + size_t(row & 31) * 16;
    auto at = [&](int c) { return reinterpret_cast<u32x4*>(dst + size_t(c >> 1) * 1024 + (c & 1) * 512); };
    if (row >= M) {
        for (int c = lane; c < pieces; c += 64) *at(c) = u32x4{0u, 0u, 0u, 0u};
        if (lane == 0) xs[row] = 0.0f;
        return;
    }
    auto amax8 = [](const u32x4& v, float m) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            m = fmaxf(m, fabsf(__uint_as_float(v[e] << 16)));
            m = fmaxf(m, fabsf(__uint_as_float(v[e] & 0xFFFF0000u)));
        }
        return m;
    };
    auto codes8 = [](const u32x4& v, float qi) {
        uint32_t o[2] = {0u, 0u};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int q0 = quant_code(__uint_as_float(v[e] << 16), qi);
            const int q1 = quant_code(__uint_as_float(v[e] & 0xFFFF0000u), qi);
            o[e >> 1] |= (uint32_t(q0) & 0xFFu) << (16 * (e & 1));
            o[e >> 1] |= (uint32_t(q1) & 0xFFu) << (16 * (e & 1) + 8);
        }
        return u32x2{o[0], o[1]};
    };
    const u32x4* xrow = reinterpret_cast<const u32x4*>(x + size_t(row) * K);
    float amax = 0.0f;
    for (int c = lane; c < pieces; c += 64) amax = amax8(xrow[2 * c + 1], amax8(xrow[2 * c], amax));
    amax = wave_max(amax);
    const float s = __fdiv_rn(amax, 127.0f);
    const float qi = s > 0.0f ? __fdiv_rn(1.0f, s) : 0.0f;
    for (int c = lane; c < pieces; c += 64) {
        const u32x2 lo = codes8(xrow[2 * c], qi), hi = codes8(xrow[2 * c + 1], qi);
        *at(c) = u32x4{lo[0], lo[1], hi[0], hi[1]};
    }
    if (lane == 0) xs[row] = s;
}

// ---- rot_quant: randomized Hadamard rotation of every 32-wide block, then per-token INT8 ---------------------------
// Thread t owns 4 consecutive values; 8 consecutive lanes hold one block.  Butterfly order as in the host
// formulation: two stages inside the thread, then strides 1, 2, 4 across lanes (lower = lower + upper,
// upper = lower - upper); the result times 1/sqrt(32) is rounded to bf16 before the row maximum is taken.
__global__ __launch_bounds__(256) void rot_quant_kernel(const uint16_t* __restrict__ x, const float* __restrict__ signs,
                                                        int8_t* __restrict__ xq, float* __restrict__ xs, int M, int K) {
    __shared__ float red[4];
    constexpr int MAXJ = 8;   // K <= 8192
    const int row = blockIdx.x, tid = threadIdx.x;
    const int J = K / 1024, rem = K % 1024;   // whole sweeps of 256 threads x 4 values, then a partial one
    float v[MAXJ + 1][4];
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j <= MAXJ; ++j) {
        const int p = 4 * (j * 256 + tid);
        const bool in = j < J || (j == J && p < K);
        if (j > J || (j == J && rem == 0)) break;
        float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
        if (in && row < M) {
            const u32x2 w = *reinterpret_cast<const u32x2*>(x + size_t(row) * K + p);
            const f32x4 sg = *reinterpret_cast<const f32x4*>(signs + p);
            a0 = __fmul_rn(__uint_as_float(w[0] << 16), sg[0]);
            a1 = __fmul_rn(__uint_as_float(w[0] & 0xFFFF0000u), sg[1]);
            a2 = __fmul_rn(__uint_as_float(w[1] << 16), sg[2]);
            a3 = __fmul_rn(__uint_as_float(w[1] & 0xFFFF0000u), sg[3]);
        }
        float b[4] = {__fadd_rn(a0, a1), __fsub_rn(a0, a1), __fadd_rn(a2, a3), __fsub_rn(a2, a3)};
        float a[4] = {__fadd_rn(b[0], b[2]), __fadd_rn(b[1], b[3]), __fsub_rn(b[0], b[2]), __fsub_rn(b[1], b[3])};
#pragma unroll
        for (int h = 1; h < 8; h <<= 1)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float c = __shfl_xor(a[i], h, WAVE);
                a[i] = (tid & h) ? __fsub_rn(c, a[i]) : __fadd_rn(a[i], c);
            }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[j][i] = round_bf16(__fmul_rn(a[i], 0.17677669529663687f));
            if (in) amax = fmaxf(amax, fabsf(v[j][i]));
        }
    }
    amax = wave_max(amax);
    if ((tid & 63) == 0) red[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    const float s = __fdiv_rn(amax, 127.0f);
    const float qi = s > 0.0f ? __fdiv_rn(1.0f, s) : 0.0f;
#pragma unroll
    for (int j = 0; j <= MAXJ; ++j) {
        const int p = 4 * (j * 256 + tid);
        if (j > J || (j == J && rem == 0)) break;
        if (j < J || p < K) {
            uint32_t o = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) o |= (uint32_t(quant_code(v[j][i], qi)) & 0xFFu) << (8 * i);
            *reinterpret_cast<uint32_t*>(xq + size_t(row) * K + p) = o;
        }
    }
    if (tid == 0) xs[row] = row < M ? s : 0.0f;
}

// ---- standard MXFP4 -> block codes + row scale: one wave per row -----------------------------------------------
__global__ __launch_bounds__(256) void mxfp4_to_sc_kernel(const uint8_t* __restrict__ e8m0,
                                                          uint8_t* __restrict__ bcodes, float* __restrict__ wscale,
                                                          int32_t* __restrict__ status, int64_t N, int nb) {
    const int64_t row = int64_t(blockIdx.x) * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= N) return;
    const uint8_t* e = e8m0 + row * nb;
    int lo = 255, hi = 0;
    for (int b = lane; b < nb; b += 64) {
        lo = min(lo, int(e[b]));
        hi = max(hi, int(e[b]));
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        lo = min(lo, __shfl_xor(lo, off, WAVE));
        hi = max(hi, __shfl_xor(hi, off, WAVE));
    }
    if (hi - lo > 3 && lane == 0) atomicOr(status, 1);
    // exponent bytes 0 (a scale below every normal float's) and 255 (NaN in the MX specification) cannot be read in place
    if ((lo < 1 || hi > 254) && lane == 0) atomicOr(status, 2);
    for (int byte = lane; bcodes && byte < nb / 4; byte += 64) {
        uint32_t v = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) v |= (uint32_t(min(int(e[4 * byte + j]) - lo, 3))) << (2 * j);
        bcodes[row * (nb / 4) + byte] = uint8_t(v);
    }
    // wscale = 2^(lo - 127 - 1); exponents below the normal range give the exact subnormal (or zero) value
    if (lane == 0) wscale[row] = ldexpf(1.0f, lo - 128);
}

}  // namespace scmx

using namespace scmx;

extern "C" {

#ifndef SCMX_BUILD_ID
#define SCMX_BUILD_ID "unknown"
#endif
// "scmx <version> (gfx950) <source revision the library was built from>"
const char* scmx_version(void) { return "scmx 0.2 (gfx950) " SCMX_BUILD_ID; }
const char* scmx_last_error(void) { return g_err; }

void scmx_mxfp4_format(scmx_format* f) {
    scmx_default_format(f);
    f->bc_bits = 8;
    f->n_mult = 0;
    for (int i = 0; i < 16; ++i) f->mult[i] = 0;
}

void scmx_default_format(scmx_format* f) {
    memset(f, 0, sizeof(*f));
    f->block = 32;
    f->bc_bits = 2;
    f->n_mult = 4;
    const int mag[8] = {0, 1, 2, 3, 4, 6, 8, 12};
    for (int i = 0; i < 8; ++i) f->code_mag[i] = mag[i];
    for (int i = 0; i < 4; ++i) f->mult[i] = 1 << i;
}

int scmx_unpack_i8(const scmx_format* fmt, const uint32_t* codes, const uint8_t* bcodes, int8_t* wq, int64_t n_rows,
                   int64_t K, void* stream) {
    DevFormat f;
    if (int rc = make_dev_format(fmt, &f)) return rc;
    if (f.e8m0) {
        set_error("unpack_i8: the E8M0 form needs the row scales to place a block; convert with scmx_mxfp4_to_sc first");
        return SCMX_ERR_FORMAT;
    }
    if (!codes || !bcodes || !wq || n_rows < 0 || K <= 0 || K % f.block || (K / f.block * f.bc_bits) % 8) {
        set_error("unpack_i8: need non-null pointers, K (%lld) a multiple of block %d and whole block-code bytes per row",
                  (long long)K, f.block);
        return SCMX_ERR_ARG;
    }
    if (K > (int64_t(1) << 30) || n_rows > (int64_t(1) << 40) / K) {   // keeps every count below 2^40 and the grid below 2^32
        set_error("unpack_i8: %lld x %lld weights are more than one launch takes (2^40)", (long long)n_rows, (long long)K);
        return SCMX_ERR_ARG;
    }
    if (n_rows == 0) return SCMX_OK;
    const int bc_row_bytes = int(K / f.block * f.bc_bits / 8);
    hipStream_t s = (hipStream_t)stream;
    if (K % 32 == 0 && (uintptr_t(codes) % 16 == 0) && (uintptr_t(wq) % 16 == 0)) {
        const int64_t groups = n_rows * (K / 32);
        unpack_i8_kernel<<<dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, s>>>(
            f, (const u32x4*)codes, bcodes, (u32x4*)wq, groups, int(K / 32), bc_row_bytes);
    } else {
        if (uintptr_t(wq) % 8) {
            set_error("unpack_i8: output must be 8-byte aligned");
            return SCMX_ERR_ARG;
        }
        const int64_t words = n_rows * (K / 8);
        unpack_i8_word_kernel<<<dim3((unsigned)((words + 255) / 256)), dim3(256), 0, s>>>(
            f, codes, bcodes, (u32x2*)wq, words, int(K / 8), bc_row_bytes);
    }
    return check_launch("unpack_i8");
}

int scmx_act_quant_blocked(const uint16_t* x, int8_t* xq, float* xs, int M, int Mp, int K, void* stream) {
    if (!x || !xq || !xs || M < 0 || Mp < M || Mp % 32 || Mp > (1 << 30) || K <= 0 || K % 32 || uintptr_t(x) % 16 ||
        uintptr_t(xq) % 16) {
        set_error("act_quant_blocked: need M <= Mp <= 2^30 with Mp %% 32 == 0 (Mp = %d), K %% 32 == 0 (K = %d), x and xq "
                  "16-byte aligned", Mp, K);
        return SCMX_ERR_ARG;
    }
    if (Mp == 0) return SCMX_OK;
    const dim3 grid(unsigned(Mp) / 8u), block(512);
    hipStream_t st = (hipStream_t)stream;
    switch (K % 512 ? 0 : K / 512) {   // rows of up to 8192 elements stay in registers, loaded as by rows
        case 1: act_quant_wave_kernel<1, true><<<grid, block, 0, st>>>(x, xq, xs, M, Mp); break;
        case 2: act_quant_wave_kernel<2, true><<<grid, block, 0, st>>>(x, xq, xs, M, Mp); break;
        case 3: act_quant_wave_kernel<3, true><<<grid, block, 0, st>>>(x, xq, xs, M, Mp); break;
        case 4: act_quant_wave_kernel<4, true><<<grid, block, 0, st>>>(x, xq, xs, M, Mp); break;
        case 6: act_quant_wave_kernel<6, true><<<grid, block, 0, st>>>(x, xq, xs, M, Mp); break;
        case 8: act_quant_wave_kernel<8, true><<<grid, block, 0, st>>>(x, xq, xs, M, Mp); break;
        case 12: act_quant_wave_kernel<12, true><<<grid, block, 0, st>>>(x, xq, xs, M, Mp); break;
        case 16: act_quant_wave_kernel<16, true><<<grid, block, 0, st>>>(x, xq, xs, M, Mp); break;
        default: act_quant_blocked_kernel<<<grid, block, 0, st>>>(x, xq, xs, M, Mp, K); break;
    }
    return check_launch("act_quant_blocked");
}

int scmx_act_quant(const uint16_t* x, int8_t* xq, float* xs, int M, int Mp, int K, void* stream) {
    if (!x || !xq || !xs || M < 0 || Mp < M || Mp > (1 << 30) || K <= 0 || K % 8 || uintptr_t(x) % 16 || uintptr_t(xq) % 8) {
        set_error("act_quant: need M <= Mp <= 2^30, K %% 8 == 0 (K = %d), x 16-byte and xq 8-byte aligned", K);
        return SCMX_ERR_ARG;
    }
    if (Mp == 0) return SCMX_OK;
    const dim3 wgrid((unsigned(Mp) + 3u) / 4u), block(256);
    hipStream_t st = (hipStream_t)stream;
    switch (K % 512 ? 0 : K / 512) {   // rows of up to 8192 elements stay in registers
        case 1: act_quant_wave_kernel<1><<<wgrid, block, 0, st>>>(x, xq, xs, M, Mp); break;
        case 2: act_quant_wave_kernel<2><<<wgrid, block, 0, st>>>(x, xq, xs, M, Mp); break;
        case 3: act_quant_wave_kernel<3><<<wgrid, block, 0, st>>>(x, xq, xs, M, Mp); break;
        case 4: act_quant_wave_kernel<4><<<wgrid, block, 0, st>>>(x, xq, xs, M, Mp); break;
        case 6: act_quant_wave_kernel<6><<<wgrid, block, 0, st>>>(x, xq, xs, M, Mp); break;
        case 8: act_quant_wave_kernel<8><<<wgrid, block, 0, st>>>(x, xq, xs, M, Mp); break;
        case 12: act_quant_wave_kernel<12><<<wgrid, block, 0, st>>>(x, xq, xs, M, Mp); break;
        case 16: act_quant_wave_kernel<16><<<wgrid, block, 0, st>>>(x, xq, xs, M, Mp); break;
        default: act_quant_kernel<<<dim3(Mp), block, 0, st>>>(x, xq, xs, M, K); break;
    }
    return check_launch("act_quant");
}

int scmx_rot_quant(const uint16_t* x, const float* signs, int8_t* xq, float* xs, int M, int Mp, int K, void* stream) {
    if (!x || !signs || !xq || !xs || M < 0 || Mp < M || K <= 0 || K % 32 || K > 8192) {
        set_error("rot_quant: null pointer, Mp < M, or K not a multiple of 32 in 32..8192 (M=%d Mp=%d K=%d)", M, Mp, K);
        return SCMX_ERR_ARG;
    }
    if (uintptr_t(x) % 8 || uintptr_t(signs) % 16 || uintptr_t(xq) % 4) {
        set_error("rot_quant: x must be 8-byte, signs 16-byte, xq 4-byte aligned");
        return SCMX_ERR_ARG;
    }
    if (Mp == 0) return SCMX_OK;
    rot_quant_kernel<<<dim3(Mp), dim3(256), 0, (hipStream_t)stream>>>(x, signs, xq, xs, M, K);
    return check_launch("rot_quant");
}

int scmx_mxfp4_to_sc(const uint8_t* e8m0, uint8_t* bcodes, float* wscale, int32_t* status, int64_t N, int64_t K,
                     void* stream) {
    if (!e8m0 || !wscale || !status || N < 0 || N > (int64_t(1) << 32) || K <= 0 || K % 128 || K > (int64_t(1) << 30)) {
        set_error("mxfp4_to_sc: need non-null pointers, N <= 2^32 and K %% 128 == 0, K <= 2^30 (K = %lld)", (long long)K);
        return SCMX_ERR_ARG;
    }
    if (N == 0) return SCMX_OK;
    mxfp4_to_sc_kernel<<<dim3((unsigned)((N + 3) / 4)), dim3(256), 0, (hipStream_t)stream>>>(e8m0, bcodes, wscale,
                                                                                               status, N, int(K / 32));
    return check_launch("mxfp4_to_sc");
}

}  // extern "C"
