// W4A8 GEMM on CDNA4 INT8 MFMA: dense prefill and grouped mixture-of-experts.
//
// One workgroup computes a BM x BN tile of  acc[m, n] = sum_k xq[m, k] * q[n, k]  in INT32.  Per K step of BK the
// workgroup stages BM x BK activation bytes and BN x BK weight bytes in LDS; the weight bytes are produced in
// registers from the packed 4-bit codes (16 bytes of codes = one run of 32 weights per thread) right before they
// are written to LDS, so the INT8 form of the weights exists only there.  Waves then read 16-byte operand
// fragments and issue v_mfma_i32_32x32x32_i8 with the weights as the row operand: each lane ends up with groups
// of 4 consecutive output columns n of one token row m, which is the unit every epilogue works on.
// LDS holds three stages of the K loop; global loads run four steps ahead in two register sets, and the decode and
// LDS writes of step i+2 are issued between the MFMAs of step i, with one barrier per step.
#include <atomic>
#include <type_traits>

#include "scmx_common.h"

namespace scmx {

struct GemmArgs {
    const int8_t* xq;        // activations INT8 [rows, K] (blocked: 32 x 32 blocks in MFMA operand order, see AD)
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
    const uint16_t* silu;    // SwiGLU epilogue: lookup table over bf16 gate values
    const int32_t* tstart;   // grouped: first row tile of each expert [E+1]
    int n_experts;
    int blocked;             // dense: xq is in the blocked layout
    DevFormat fmt;
};

// B_PACKED_DEFAULT / B_PACKED_B16: the published codebook with power-of-two shifts on 32- / 16-element blocks (decoded
// with the FP4 conversion); B_PACKED_B16M: that codebook on 16-element blocks with 4-bit codes for consecutive integer
// multipliers (FP4 conversion, then one fused multiply-add); B_PACKED_GENERIC: any member of the format family (table
// decode).
// B_PACKED_E8M0: a standard MXFP4 tensor in place -- B_PACKED_DEFAULT's decode with the block's shift taken from its
// E8M0 byte minus the row's lowest one (which the row scale carries).
enum { B_INT8 = 0, B_PACKED_DEFAULT = 1, B_PACKED_GENERIC = 2, B_PACKED_B16 = 3, B_PACKED_B16M = 4, B_PACKED_E8M0 = 5 };

// FD = number of fragment register buffers: fragments are fetched FD - 1 k slices ahead of their MFMAs.
// SKIP (grouped launches): a row tile that ends inside its expert's segment multiplies only the 32-row blocks that hold
// valid rows.  The two waves that share a SIMD then own the same columns and different row halves of the tile, so that
// a half-empty tile halves the MFMA work of every SIMD instead of idling two of the four.
// PK (B_PACKED_DEFAULT / B_PACKED_B16, K steps of 128): the weights stay packed in LDS -- 64 bytes of codes per row and
// K step plus the step's block-code bytes -- and every wave decodes its own fragments after reading them.  Half the
// weight bytes through LDS in both directions, paid with one decode per wave row that shares the fragment.
// KG > 1 (small problems: fewer tiles than CUs): KG groups of WGM x WGN waves share the tile, each multiplies its own
// K / KG of the reduction out of LDS stages of its own, and the INT32 partial sums meet in LDS before the epilogue (exact:
// integer addition is associative).  A CU then runs KG times the waves on the same tile count.
// AD (dense, activations in the blocked layout): the activation tile does not pass through LDS; every wave loads the
// fragments of its own rows from memory, one coalesced 1 KB load per 32-row x 32-k block, two K steps ahead.  Waves must
// then not share rows (WGN = 1, or few column groups), and only the weight rows of a stage exist in LDS.
template <int BM, int BN, int BK, int WGM, int WGN, int BMODE, int OCC = 1, int FD = 2, bool SKIP = false, bool PK = false,
          int KG = 1, bool AD = false>
__global__ __launch_bounds__(WGM* WGN* KG * 64, OCC) void gemm_kernel(const GemmArgs a) {
    constexpr int NSTAGE = 3;   // LDS stages: one being read, one ready, one being written
    constexpr int NT = WGM * WGN * 64;   // threads of one K group
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int MI = WTM / 32, NI = WTN / 32;
    static_assert(WTM % 32 == 0 && WTN % 32 == 0 && (BK == 64 || BK == 128), "tile must be whole 32x32x32 MFMAs");
    constexpr int CPR = BK / 16;             // 16-byte chunks per LDS row
    constexpr int RPB = 256 / BK;            // rows per 256 bytes, i.e. per sweep of the 64 LDS banks
    constexpr int A_CHUNKS = AD ? 0 : BM * CPR;   // 16-byte pieces of the activation tile
    constexpr int A_PER = AD ? 1 : (A_CHUNKS + NT - 1) / NT;
    constexpr int A_BYTES = AD ? 0 : BM * BK;     // the activation rows of a stage
    // packed weights are staged in runs of 8 * WPC weights (WPC code words) per thread: 32 when that keeps every
    // thread busy, else 16
    constexpr int WPC = BN * BK / 32 >= NT ? 4 : 2;
    constexpr int B_CHUNKS = BMODE == B_INT8 ? BN * CPR : BN * BK / (8 * WPC);
    constexpr int B_PER = (B_CHUNKS + NT - 1) / NT;
    constexpr int BCB = BMODE == B_PACKED_B16 ? 2 : 1;   // PK: block-code bytes per weight row and K step
    static_assert(!PK || (BK == 128 && WPC == 4 && (BMODE == B_PACKED_DEFAULT || BMODE == B_PACKED_B16)),
                  "packed weights in LDS: K steps of 128, 16-byte runs, FP4-conversion formats");
    // bytes per stage: BM activation rows, then BN weight rows (PK: 64 code bytes each)
    constexpr int STAGE = A_BYTES + (PK ? BN * (BK / 2) : BN * BK);
    static_assert(STAGE % 16 == 0, "stages keep 16-byte alignment");

    // Rows are BK bytes with no padding; the 16-byte chunk c of row r sits at chunk c ^ ((r / RPB) % CPR), which
    // spreads the 16 rows a b128 fragment read touches per pass over all 64 banks.
    // The epilogue reuses the buffer for one [WTM x (row bytes + 16)] output tile per wave; when the bf16 tiles
    // need more than the stages and still fit the CU, the buffer is sized for them.
    constexpr int EPI_BYTES = WGM * WGN * WTM * (WTN * 2 + 16);
    static_assert(KG == 1 || (!PK && !SKIP), "K groups: staged dense tiles");
    static_assert(!AD || (!PK && !SKIP && KG == 1), "activation fragments from memory: staged dense tiles");
    constexpr int GROUP_BYTES = NSTAGE * STAGE;
    // after the K loop: group 0's output tiles (the widest epilogue's) from 0, then the other groups' partial sums
    constexpr int PART_BYTES = NT * MI * NI * 64;
    constexpr int PART_BASE = WGM * WGN * WTM * (WTN * 4 + 16);
    constexpr int KG_BYTES = PART_BASE + (KG - 1) * PART_BYTES > KG * GROUP_BYTES ? PART_BASE + (KG - 1) * PART_BYTES : KG * GROUP_BYTES;
    static_assert(KG == 1 || KG_BYTES <= 160 * 1024, "stages and partial sums fit the CU's LDS");
    constexpr int SMEM_BYTES =
        KG > 1 ? KG_BYTES : (EPI_BYTES > NSTAGE * STAGE && EPI_BYTES <= 150 * 1024) ? EPI_BYTES : NSTAGE * STAGE;
    __shared__ __attribute__((aligned(16))) int8_t smem[SMEM_BYTES];
    // scales of the tile's rows and columns, fetched before the K loop so that the epilogue does not start with a
    // round trip to memory
    __shared__ __attribute__((aligned(16))) float s_xs[BM], s_ws[BN];
    auto swz = [](int row, int chunk) { return row * BK + ((chunk ^ ((row / RPB) & (CPR - 1))) << 4); };
    // packed weight rows (64 bytes, 4 chunks): 4 rows per sweep of the banks, chunk c of row r at c ^ ((r / 4) % 4)
    auto swzp = [](int row, int chunk) { return row * (BK / 2) + ((chunk ^ ((row >> 2) & 3)) << 4); };

    const int kg = KG == 1 ? 0 : __builtin_amdgcn_readfirstlane(int(threadIdx.x) / NT);   // K group (wave-uniform)
    const int tid = KG == 1 ? int(threadIdx.x) : int(threadIdx.x) % NT, lane = tid & 63, wave = tid >> 6;
    int8_t* const sm = smem + kg * GROUP_BYTES;   // this group's stages
    const int wm = SKIP ? wave / WGN : wave % WGM, wn = SKIP ? wave % WGN : wave / WGM;

    // ---- which tile ------------------------------------------------------------------------------------------
    const int num_n = (a.N + BN - 1) / BN;
    int m0, n0, row_end, expert = 0;
    if (a.tstart) {   // grouped: row tiles of BM inside expert segments
        // Workgroup b runs on XCD b % 8: inside every chunk of 8 row tiles each XCD takes one row tile with all of
        // its column tiles, so an activation panel is fetched into one L2 only.
        const int j = blockIdx.x % (8 * num_n);
        const int slot = blockIdx.x / (8 * num_n) * 8 + (j & 7);
        n0 = (j >> 3) * BN;
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
        // Tile order: bands of 4 row tiles, inside a band column by column.  The 32 workgroups an XCD runs at once
        // then share 4 activation panels and 8 weight panels (what its L2 holds) however large M is.
        constexpr int GM = 4;
        const int band = pid / (GM * num_n), r = pid % (GM * num_n);
        const int rows_in_band = min(GM, num_m - band * GM);
        n0 = (r / rows_in_band) * BN;
        m0 = (band * GM + r % rows_in_band) * BM;
        row_end = a.M;
    }
    const int K = a.K;
    const int KL = K / KG;         // length of this group's part of the reduction
    const int kbase = kg * KL;     // and its first k (a multiple of 128)
    // 32-row blocks of this wave's tile that hold rows of the segment (wave-uniform)
    const int mi_active =
        SKIP ? __builtin_amdgcn_readfirstlane(min(MI, max(0, (row_end - (m0 + wm * WTM) + 31) / 32))) : MI;
    // The tile's scales are REQUESTED here, before the first operand loads, and stored to LDS after those have been
    // issued: memory returns a wave's loads in order, so scales requested first arrive first and their wait does not
    // cover the operand loads (fetched and stored up front they cost every tile two serial round trips to memory).
    constexpr int XS_PER = (BM + NT - 1) / NT, WS_PER = (BN + NT - 1) / NT;
    float xs_reg[XS_PER], ws_reg[WS_PER];
    int xs_row[XS_PER];
#pragma unroll
    for (int j = 0; j < XS_PER; ++j) {   // the scale's row: through the gather list when there is one (loaded with the
        const int m = m0 + tid + j * NT;   // operand rows' entries below, one wait for all of them)
        xs_row[j] = (a.xscale && tid + j * NT < BM && m < row_end) ? (a.gather ? a.gather[m] : m) : -1;
    }

    // ---- per-thread staging assignments (fixed over the K loop) ------------------------------------------------
    // Global operands are read with buffer loads: a per-thread byte offset fixed for the whole K loop plus a scalar
    // offset that advances with k, so the loop spends no vector instructions on addresses.
    const auto rsrc = [](const void* p, size_t bytes) {
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, int(bytes), 0x00020000);
    };
    const size_t erow = size_t(expert) * a.N;   // first weight row of this expert
    const __amdgpu_buffer_rsrc_t ra = rsrc(a.xq, 0xFFFFFFFFu);
    const __amdgpu_buffer_rsrc_t rb = BMODE == B_INT8 ? rsrc(a.wq + erow * K, size_t(a.N) * K)
                                                      : rsrc(reinterpret_cast<const uint8_t*>(a.codes) + erow * (K / 2), size_t(a.N) * (K / 2));
    const __amdgpu_buffer_rsrc_t rbc = rsrc(a.bcodes + erow * a.bc_row_bytes, size_t(a.N) * a.bc_row_bytes);
    int a_src[A_PER], a_dst[A_PER];
    uint32_t a_live = 0;   // SKIP: the chunks of rows inside the segment (the others are neither written to LDS nor used)
#pragma unroll
    for (int j = 0; j < A_PER; ++j) {
        if (AD) { a_src[j] = a_dst[j] = 0; continue; }
        const int c = tid + j * NT;
        const int row = c / CPR, kc = c % CPR;
        if (m0 + row < row_end) a_live |= 1u << j;
        int gr = min(m0 + row, row_end - 1);   // rows past the segment re-read its last row: one cache line, not a row each
        if (a.gather) gr = a.gather[gr];
        a_src[j] = int(uint32_t(gr) * uint32_t(K) + kc * 16 + kbase);
        a_dst[j] = swz(row, kc);
    }
    int b_src[B_PER], b_bc[B_PER], b_dst[B_PER], b_dst2[B_PER], b_k[B_PER];
    [[maybe_unused]] uint32_t b_rmin[B_PER];   // B_PACKED_E8M0: lowest exponent byte of the thread's weight row
#pragma unroll
    for (int j = 0; j < B_PER; ++j) {
        const int c = tid + j * NT;
        if (BMODE == B_INT8) {
            const int row = c / CPR, kc = c % CPR;
            const int gn = min(n0 + row, a.N - 1);
            b_src[j] = gn * K + kc * 16 + kbase;
            b_dst[j] = A_BYTES + swz(row, kc);
            b_dst2[j] = 0;
            b_bc[j] = 0;
            b_k[j] = 0;
        } else {
            constexpr int RUNS = BK / (8 * WPC);   // runs per tile row
            const int row = c / RUNS, kb = c % RUNS;
            const int gn = min(n0 + row, a.N - 1);
            b_src[j] = gn * (K / 2) + kb * 4 * WPC + kbase / 2;
            // the block-code byte of the run: 4 blocks per byte, i.e. 128 weights (one byte per K step at most) or 64
            // (two 4-bit codes per byte: 32)
            b_bc[j] = gn * a.bc_row_bytes + (BMODE == B_PACKED_B16      ? (kbase + kb * 8 * WPC) >> 6
                                             : BMODE == B_PACKED_B16M   ? (kbase + kb * 8 * WPC) >> 5
                                             : BMODE == B_PACKED_E8M0   ? (kbase + kb * 8 * WPC) >> 5
                                             : BMODE == B_PACKED_DEFAULT ? kbase >> 7
                                                                        : 0);
            if (BMODE == B_PACKED_E8M0) b_rmin[j] = e8m0_row_min(a.wscale[erow + gn]);
            if (PK) {   // the run's 16 code bytes as they are
                b_dst[j] = A_BYTES + swzp(row, kb);
                b_dst2[j] = 0;
            } else {
                b_dst[j] = A_BYTES + swz(row, kb * WPC / 2);
                b_dst2[j] = A_BYTES + swz(row, kb * WPC / 2 + 1);
            }
            b_k[j] = kb * 8 * WPC;
        }
    }

#pragma unroll
    for (int j = 0; j < XS_PER; ++j) xs_reg[j] = xs_row[j] >= 0 ? a.xscale[xs_row[j]] : 0.0f;
#pragma unroll
    for (int j = 0; j < WS_PER; ++j) {
        const int c = tid + j * NT;
        ws_reg[j] = (a.xscale && c < BN && n0 + c < a.N) ? a.wscale[size_t(expert) * a.N + n0 + c] : 0.0f;
    }

    // Two register sets hold the global loads of two K steps in flight.
    struct Staged {
        u32x4 a[A_PER], b[B_PER];
        uint8_t bc[B_PER];   // kept as loaded: widening it here would make the compiler wait for the load at once
    };
    Staged r0, r1;

    // Loads past the last K step re-read the last step (never consumed): every iteration issues the same loads, so
    // the wait before a register set is used covers exactly that set and not the younger one.
    // The loads of one K step are issued in NKK slices (activation chunks j with j % NKK == q in slice q, the
    // weight words in the last one) so that the K loop can spread them between its MFMAs.
    constexpr int NKK = BK / 32;
    auto load_slice = [&](Staged& r, int k0, int q) {
#pragma unroll
        for (int j = 0; j < A_PER; ++j)
            if (!AD && j % NKK == q && (A_CHUNKS % NT == 0 || tid + j * NT < A_CHUNKS))
                r.a[j] = __builtin_amdgcn_raw_buffer_load_b128(ra, a_src[j], k0, 0);
        if (q != NKK - 1) return;
#pragma unroll
        for (int j = 0; j < B_PER; ++j)
            if (B_CHUNKS % NT == 0 || tid + j * NT < B_CHUNKS) {
                if (BMODE == B_INT8) {
                    r.b[j] = __builtin_amdgcn_raw_buffer_load_b128(rb, b_src[j], k0, 0);
                } else {
                    if (WPC == 4) {
                        r.b[j] = __builtin_amdgcn_raw_buffer_load_b128(rb, b_src[j], k0 >> 1, 0);
                    } else {
                        const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rb, b_src[j], k0 >> 1, 0);
                        r.b[j][0] = v[0];
                        r.b[j][1] = v[1];
                    }
                    if (PK) continue;   // block codes go straight to the lanes that decode
                    if (BMODE == B_PACKED_DEFAULT)   // 32-blocks, 2-bit codes, 4 blocks per byte: keep the raw byte
                        r.bc[j] = __builtin_amdgcn_raw_buffer_load_b8(rbc, b_bc[j], k0 >> 7, 0);
                    if (BMODE == B_PACKED_B16)       // 16-blocks: a byte covers 64 weights
                        r.bc[j] = __builtin_amdgcn_raw_buffer_load_b8(rbc, b_bc[j], k0 >> 6, 0);
                    if (BMODE == B_PACKED_B16M)      // 16-blocks, 4-bit codes: 32 weights
                        r.bc[j] = __builtin_amdgcn_raw_buffer_load_b8(rbc, b_bc[j], k0 >> 5, 0);
                    if (BMODE == B_PACKED_E8M0)      // one exponent byte per 32 weights
                        r.bc[j] = __builtin_amdgcn_raw_buffer_load_b8(rbc, b_bc[j], k0 >> 5, 0);
                }
            }
    };
    auto load_global = [&](Staged& r, int k0) {
        k0 = min(k0, KL - BK);
#pragma unroll
        for (int q = 0; q < NKK; ++q) load_slice(r, k0, q);
    };

    // Staging work of one K step, cut into NKK slices so that it can be issued in the shadow of the MFMAs of the
    // step being multiplied: slice q writes the activation chunks j with j % NKK == q and decodes the weight code
    // words w with w * NKK / 4 == q; the last slice writes the decoded weights.
    auto stage_slice = [&](const Staged& r, int8_t* st, int k0, int q, uint32_t (&o)[B_PER][8]) {
        k0 += kbase;   // block indices below count from the row's first weight
#pragma unroll
        for (int j = 0; j < A_PER; ++j)
            if (!AD && j % NKK == q && (A_CHUNKS % NT == 0 || tid + j * NT < A_CHUNKS) && (!SKIP || ((a_live >> j) & 1u)))
                *reinterpret_cast<u32x4*>(st + a_dst[j]) = r.a[j];
#pragma unroll
        for (int j = 0; j < B_PER; ++j)
            if (B_CHUNKS % NT == 0 || tid + j * NT < B_CHUNKS) {
                if (BMODE == B_INT8) {
                    if (q == 0) *reinterpret_cast<u32x4*>(st + b_dst[j]) = r.b[j];
                } else if (PK) {
                    if (q == j % NKK) *reinterpret_cast<u32x4*>(st + b_dst[j]) = r.b[j];
                } else {
#pragma unroll
                    for (int w = 0; w < WPC; ++w) {
                        if (w * NKK / WPC != q) continue;
                        if (BMODE == B_PACKED_DEFAULT) {
                            const uint32_t blk = uint32_t(k0 + b_k[j]) >> 5;
                            decode_word_fp4(r.b[j][w], fp4_scale((uint32_t(r.bc[j]) >> (2 * (blk & 3))) & 3u), o[j][2 * w],
                                            o[j][2 * w + 1]);
                        } else if (BMODE == B_PACKED_E8M0) {   // the run lies inside one block
                            decode_word_fp4(r.b[j][w], fp4_scale((uint32_t(r.bc[j]) - b_rmin[j]) & 0x7Fu), o[j][2 * w],
                                            o[j][2 * w + 1]);
                        } else if (BMODE == B_PACKED_B16) {
                            const uint32_t blk = uint32_t(k0 + b_k[j] + 8 * w) >> 4;
                            decode_word_fp4(r.b[j][w], fp4_scale((uint32_t(r.bc[j]) >> (2 * (blk & 3))) & 3u), o[j][2 * w],
                                            o[j][2 * w + 1]);
                        } else if (BMODE == B_PACKED_B16M) {
                            const uint32_t blk = uint32_t(k0 + b_k[j] + 8 * w) >> 4;
                            const _Float16 m = _Float16(int(((uint32_t(r.bc[j]) >> (4 * (blk & 1))) & 15u) + (a.fmt.mult[0] & 0xFFu)));
                            decode_word_fp4_mul(r.b[j][w], half2_t{m, m}, o[j][2 * w], o[j][2 * w + 1]);
                        } else {
                            const uint32_t blk = uint32_t(k0 + b_k[j] + 8 * w) >> a.fmt.block_log2;
                            const uint32_t bc = block_code(a.bcodes + erow * a.bc_row_bytes + b_bc[j], blk, a.fmt.bc_bits);
                            const BlockLut t = scaled_lut_mul(a.fmt.lut_lo, a.fmt.lut_hi, mult_of(a.fmt, bc));
                            decode_word(r.b[j][w], t, o[j][2 * w], o[j][2 * w + 1]);
                        }
                    }
                    if (q == (WPC - 1) * NKK / WPC) {
                        *reinterpret_cast<u32x4*>(st + b_dst[j]) = u32x4{o[j][0], o[j][1], o[j][2], o[j][3]};
                        if (WPC == 4) *reinterpret_cast<u32x4*>(st + b_dst2[j]) = u32x4{o[j][4], o[j][5], o[j][6], o[j][7]};
                    }
                }
            }
    };
    auto store_lds = [&](const Staged& r, int stage, int k0) {
        k0 = min(k0, KL - BK);
        uint32_t o[B_PER][8];
#pragma unroll
        for (int q = 0; q < NKK; ++q) stage_slice(r, sm + stage * STAGE, k0, q, o);
    };

    v16i acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    // fragment addresses: lane l supplies row l % 32 and the 16 k-bytes of half l / 32 of a 32-wide k slice; tile
    // origins are multiples of 32 rows, so the swizzle term depends on the lane only
    const int lr = lane & 31, half = lane >> 5;
    const int sw = (lr / RPB) & (CPR - 1);
    int koff[NKK];
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) koff[kk] = ((2 * kk + half) ^ sw) << 4;
    const int a_frag = (wm * WTM + lr) * BK;
    const int b_frag = A_BYTES + (wn * WTN + lr) * BK;

    const int KT = KL / BK;
    // Pipeline.  Iteration kt: barrier; multiply step kt out of its LDS stage while the register set holding step
    // kt+2 is decoded and written into its stage, one slice per 32-wide k slice of MFMAs; then reissue that set's
    // global loads for step kt+4.  A stage is rewritten two barriers after its last read and readable one barrier
    // after it was written, so the first fragments of step kt+1 are fetched at the end of iteration kt, ahead of the
    // barrier that opens kt+1.  The stage indices are compile-time constants (the loop is unrolled over the
    // 3 stages x 2 register sets), which keeps every LDS address an immediate offset from a fixed register.
    [[maybe_unused]] uint32_t bcc[NI], bcn[NI];   // PK: block codes of the current / the next two K steps
    [[maybe_unused]] int bc_src[NI];
#pragma unroll
    for (int j = 0; j < NI; ++j) bc_src[j] = min(n0 + wn * WTN + j * 32 + lr, a.N - 1) * a.bc_row_bytes;
    // block codes of K steps s and s + 1 (s even); past the end the last pair of steps again (never consumed)
    auto load_bc = [&](int s, uint32_t (&f)[NI]) {
        const int so = min(s, (K / BK - 1) & ~1) * BCB;
#pragma unroll
        for (int j = 0; j < NI; ++j)
            f[j] = BCB == 2 ? uint32_t(__builtin_amdgcn_raw_buffer_load_b32(rbc, bc_src[j], so, 0))
                            : uint32_t(__builtin_amdgcn_raw_buffer_load_b16(rbc, bc_src[j], so, 0));
    };
    if constexpr (PK) load_bc(0, bcc);   // ahead of the operand loads, like the scales
    load_global(r0, 0);
    load_global(r1, BK);
    if (a.xscale) {   // published by the barrier that opens the K loop
#pragma unroll
        for (int j = 0; j < XS_PER; ++j)
            if (tid + j * NT < BM) s_xs[tid + j * NT] = xs_reg[j];
#pragma unroll
        for (int j = 0; j < WS_PER; ++j)
            if (tid + j * NT < BN) s_ws[tid + j * NT] = ws_reg[j];
    }
    store_lds(r0, 0, 0);
    store_lds(r1, 1, BK);
    load_global(r0, 2 * BK);
    // the two sets' loads stay apart, in the order the K loop issues them: its first copy has two predecessors (this code
    // and the loop's end) and waits for the fewer outstanding loads of the two -- interleaved here, that wait covered
    // the younger set as well, in every trip
    __builtin_amdgcn_sched_barrier(0);
    load_global(r1, 3 * BK);
    // ---- PK: fragments of packed weights ------------------------------------------------------------------------
    // The k positions of a 64-wide pair of MFMA slices are dealt so that a lane's packed codes are one 16-byte read:
    // lane half h supplies k = 64 kp + 32 h + 16 s + (0..15) to slice s of pair kp, i.e. 32 consecutive activation
    // bytes (two 16-byte reads) and 32 consecutive codes (one), the latter one 32-block or two 16-blocks.
    constexpr int NKP = NKK / 2;
    // Three things are in flight per wave: the MFMAs of pair p, the decode of pair p + 1 (its codes were read during
    // pair p - 1) and the LDS reads of pair p + 1's activations and pair p + 2's codes.
    // The block codes do not pass through LDS: the lane that decodes row n reads the codes of two K steps of that row
    // (2 * BCB bytes) from memory every second step, two steps ahead.
    [[maybe_unused]] v4i pa[2][2][MI];   // activation fragments [pair parity][slice][32-row block]
    [[maybe_unused]] v4i pw[2][NI];      // 32 codes per weight row as read from LDS [pair parity]
    [[maybe_unused]] v4i px[2][2][NI];   // decoded INT8 operands [pair parity][slice][32-column block]
    [[maybe_unused]] int koff_pa[NKP][2], koff_pw[NKP];
#pragma unroll
    for (int kp = 0; kp < NKP; ++kp) {
        koff_pa[kp][0] = ((4 * kp + 2 * half) ^ sw) << 4;
        koff_pa[kp][1] = ((4 * kp + 2 * half + 1) ^ sw) << 4;
        koff_pw[kp] = ((2 * kp + half) ^ ((lr >> 2) & 3)) << 4;
    }
    [[maybe_unused]] const int w_frag = A_BYTES + (wn * WTN + lr) * (BK / 2);
    auto load_pa = [&](const int8_t* src, int kp, v4i (&f)[2][MI]) {
#pragma unroll
        for (int i = 0; i < MI; ++i)
            if (!SKIP || i < mi_active) {
                f[0][i] = *reinterpret_cast<const v4i*>(src + a_frag + i * 32 * BK + koff_pa[kp][0]);
                f[1][i] = *reinterpret_cast<const v4i*>(src + a_frag + i * 32 * BK + koff_pa[kp][1]);
            }
    };
    auto load_pw = [&](const int8_t* src, int kp, v4i (&f)[NI]) {
        if (SKIP && mi_active == 0) return;
#pragma unroll
        for (int j = 0; j < NI; ++j) f[j] = *reinterpret_cast<const v4i*>(src + w_frag + j * 32 * (BK / 2) + koff_pw[kp]);
    };
    // 32 codes -> the INT8 operands of the pair's two slices; `odd` = the K step's parity (which half of the block codes)
    auto decode_pair = [&](const v4i (&f)[NI], const uint32_t (&bc)[NI], int odd, int kp, v4i (&x)[2][NI]) {
        if (SKIP && mi_active == 0) return;
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            float s0, s1;
            if (BMODE == B_PACKED_B16) {   // blocks 4 kp + 2 h and the next one of the step's 8
                const uint32_t t = bc[j] >> (16 * odd + 8 * kp + 4 * half);
                s0 = fp4_scale(t & 3u);
                s1 = fp4_scale((t >> 2) & 3u);
            } else {                       // block 2 kp + h of the step's 4
                s0 = s1 = fp4_scale((bc[j] >> (8 * odd + 4 * kp + 2 * half)) & 3u);
            }
            uint32_t o[8];
            decode_word_fp4(uint32_t(f[j][0]), s0, o[0], o[1]);
            decode_word_fp4(uint32_t(f[j][1]), s0, o[2], o[3]);
            decode_word_fp4(uint32_t(f[j][2]), s1, o[4], o[5]);
            decode_word_fp4(uint32_t(f[j][3]), s1, o[6], o[7]);
            x[0][j] = v4i{int(o[0]), int(o[1]), int(o[2]), int(o[3])};
            x[1][j] = v4i{int(o[4]), int(o[5]), int(o[6]), int(o[7])};
        }
    };
    auto iteration_pk = [&](auto step_tag, auto parity_tag, Staged& r, int kt) {
        constexpr int rd = decltype(step_tag)::value;
        constexpr int odd = decltype(parity_tag)::value;   // kt % 2
        constexpr int wr = (rd + 2) % NSTAGE;
        constexpr int nx = (rd + 1) % NSTAGE;
        __syncthreads();
        const int8_t* src = smem + rd * STAGE;
        const int8_t* nxt = smem + nx * STAGE;
        int8_t* dst = smem + wr * STAGE;
        const int k2 = min((kt + 2) * BK, K - BK);
        const int k4 = min((kt + 4) * BK, K - BK);
        uint32_t o[B_PER][8];
        if (!odd) load_bc(kt + 2, bcn);
#pragma unroll
        for (int kp = 0; kp < NKP; ++kp) {
            const int cur = kp % 2, oth = (kp + 1) % 2;   // NKP is even: pair 0 of every step has parity 0
            if (kp + 1 < NKP) {
                load_pa(src, kp + 1, pa[oth]);
                decode_pair(pw[oth], bcc, odd, kp + 1, px[oth]);
            } else {   // pair 0 of step kt + 1
                load_pa(nxt, 0, pa[oth]);
                if (odd) {
#pragma unroll
                    for (int j = 0; j < NI; ++j) bcc[j] = bcn[j];
                }
                decode_pair(pw[oth], bcc, 1 - odd, 0, px[oth]);
            }
            load_pw(nxt, kp, pw[cur]);   // pair kp + 2 = pair kp of the next step; pw[cur] was decoded a pair ago
#pragma unroll
            for (int sl = 0; sl < 2; ++sl) {
#pragma unroll
                for (int i = 0; i < MI; ++i) {
                    if (SKIP && i >= mi_active) continue;
#pragma unroll
                    for (int j = 0; j < NI; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(px[cur][sl][j], pa[cur][sl][i], acc[i][j], 0, 0, 0);
                }
                stage_slice(r, dst, k2, 2 * kp + sl, o);
            }
        }
        load_global(r, k4);
    };
    static_assert(!PK || NKP % 2 == 0, "the pair buffers return to phase 0 every K step");

    // Fragments are fetched FD - 1 k slices ahead of the MFMAs that use them, into FD rotating register buffers; the
    // slices fetched at the end of an iteration belong to the next step's stage.
    constexpr int AHEAD = FD - 1;
    static_assert(AHEAD >= 1 && AHEAD <= NKK, "fragment prefetch distance");
    [[maybe_unused]] v4i fa[FD][MI], fb[FD][NI];
    auto load_frags = [&](const int8_t* src, int kk, v4i (&xa)[MI], v4i (&xb)[NI]) {
        if (SKIP && mi_active == 0) return;
#pragma unroll
        for (int i = 0; i < MI; ++i)
            if (!AD && (!SKIP || i < mi_active)) xa[i] = *reinterpret_cast<const v4i*>(src + a_frag + i * 32 * BK + koff[kk]);
#pragma unroll
        for (int j = 0; j < NI; ++j) xb[j] = *reinterpret_cast<const v4i*>(src + b_frag + j * 32 * BK + koff[kk]);
    };
    // AD: the activations come in 32-row x 32-k blocks of 1 KB laid out as the MFMA takes them (lane l = row l % 32,
    // k half l / 32, 16 bytes each), block (m / 32, k / 32) at ((m / 32) * (K / 32) + k / 32) KB.  Every wave loads the
    // fragments of its own rows straight into registers, two K steps ahead, in three buffers that rotate with the LDS
    // stages: the activation tile never passes through LDS.
    [[maybe_unused]] v4i fad[NSTAGE][NKK][MI];
    [[maybe_unused]] int ad_src[MI];
    if constexpr (AD) {
        const int last_block = (a.M + 31) / 32 - 1;
#pragma unroll
        for (int i = 0; i < MI; ++i)
            ad_src[i] = int(uint32_t(min((m0 + wm * WTM) / 32 + i, last_block)) * uint32_t(K >> 5) * 1024u + uint32_t(lane) * 16u +
                            uint32_t(kbase) * 32u);
    }
    auto load_ad = [&](int buf, int k0) __attribute__((always_inline)) {
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk)
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(ra, ad_src[i] + kk * 1024, k0 * 32, 0);
                fad[buf][kk][i] = v4i{int(v[0]), int(v[1]), int(v[2]), int(v[3])};
            }
    };
    if constexpr (AD) {
        load_ad(0, 0);
        load_ad(1, min(BK, KL - BK));
    }
    __syncthreads();
    if constexpr (PK) {
        load_pa(smem, 0, pa[0]);
        load_pw(smem, 0, pw[0]);
        load_pw(smem, 1, pw[1]);
        decode_pair(pw[0], bcc, 0, 0, px[0]);
    } else {
#pragma unroll
        for (int q = 0; q < AHEAD; ++q) load_frags(sm, q, fa[q], fb[q]);
    }
    // The k slices of an iteration are fenced against each other for the scheduler: left alone, the compiler sinks every
    // LDS write of the step to its end, in front of the barrier (M = 8192: 442 -> 429 us over the four layers with the
    // fences on the 256x256 tile; M = 128 ... 1024 on the small tiles: 2-3 %).
    auto iteration_staged = [&](auto step_tag, auto stage_tag, Staged& r, int kt) __attribute__((always_inline)) {
        constexpr int rd = decltype(step_tag)::value;        // kt % 3: stage of step kt
        constexpr bool ST = decltype(stage_tag)::value;      // false in the last two steps: nothing left to stage
        constexpr int wr = (rd + 2) % NSTAGE;                // stage of step kt + 2
        constexpr int nx = (rd + 1) % NSTAGE;                // stage of step kt + 1
        constexpr int ph = (NKK * rd) % FD;                  // fragment buffer of slice 0 of this step (FD divides 6 * NKK)
        __syncthreads();
        const int8_t* src = sm + rd * STAGE;
        const int8_t* nxt = sm + nx * STAGE;
        int8_t* dst = sm + wr * STAGE;
        const int k2 = min((kt + 2) * BK, KL - BK);      // past the end: rewrites a stage nobody reads again
        const int k4 = min((kt + 4) * BK, KL - BK);
        uint32_t o[B_PER][8];
        if constexpr (AD && ST) load_ad(wr, k2);
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk) {
            if (kk + AHEAD < NKK)
                load_frags(src, kk + AHEAD, fa[(ph + kk + AHEAD) % FD], fb[(ph + kk + AHEAD) % FD]);
            else
                load_frags(nxt, kk + AHEAD - NKK, fa[(ph + kk + AHEAD) % FD], fb[(ph + kk + AHEAD) % FD]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                if (SKIP && i >= mi_active) continue;
#pragma unroll
                for (int j = 0; j < NI; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[(ph + kk) % FD][j], AD ? fad[rd][kk][i] : fa[(ph + kk) % FD][i],
                                                                      acc[i][j], 0, 0, 0);
            }
            if constexpr (ST) stage_slice(r, dst, k2, kk, o);
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (ST) load_global(r, k4);
    };
    auto iteration = [&](auto step_tag, auto parity_tag, Staged& r, int kt) __attribute__((always_inline)) {
        if constexpr (PK) iteration_pk(step_tag, parity_tag, r, kt); else iteration_staged(step_tag, std::true_type{}, r, kt);
    };
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    using S2 = std::integral_constant<int, 2>;
    // Whole trips of 6 steps run without an exit inside; the remaining steps are nested so that every copy of the
    // iteration has exactly one predecessor.  (With merging paths the compiler must assume the fewest outstanding
    // loads of any path when it places its waits, and ends up waiting for loads issued one step ago.)
    int kt = 0;
    using Even = std::integral_constant<int, 0>;
    using Odd = std::integral_constant<int, 1>;
    if constexpr (PK) {
        for (; kt + 6 <= KT; kt += 6) {   // kt stays even here: the parity of every copy is fixed
            iteration(S0{}, Even{}, r0, kt);
            iteration(S1{}, Odd{}, r1, kt + 1);
            iteration(S2{}, Even{}, r0, kt + 2);
            iteration(S0{}, Odd{}, r1, kt + 3);
            iteration(S1{}, Even{}, r0, kt + 4);
            iteration(S2{}, Odd{}, r1, kt + 5);
        }
        if (kt < KT) {
            iteration(S0{}, Even{}, r0, kt);
            if (kt + 1 < KT) {
                iteration(S1{}, Odd{}, r1, kt + 1);
                if (kt + 2 < KT) {
                    iteration(S2{}, Even{}, r0, kt + 2);
                    if (kt + 3 < KT) {
                        iteration(S0{}, Odd{}, r1, kt + 3);
                        if (kt + 4 < KT) iteration(S1{}, Even{}, r0, kt + 4);
                    }
                }
            }
        }
    } else {
        // The last two steps find their stages written and have nothing to stage or load: they run as copies without
        // that work.  Small wave tiles append them at each exit of the staged steps (one predecessor each); larger
        // ones, with few registers to spare for the copies that so many joins cost, select them by the stage reached;
        // the largest (128 accumulators, 256x256) keeps every step alike and stages past the end.
        constexpr bool INLINE_TAIL = MI * NI <= 2, NO_TAIL = MI * NI > 4;
        const int KM = NO_TAIL ? KT : max(KT - 2, 0);   // steps that stage step kt + 2
        auto last_two = [&](auto s_first, auto s_second) __attribute__((always_inline)) {
            iteration_staged(s_first, std::false_type{}, r0, 0);
            if (KT >= 2) iteration_staged(s_second, std::false_type{}, r0, 0);
        };
        auto tail = [&](auto s_first, auto s_second) __attribute__((always_inline)) {
            if constexpr (INLINE_TAIL) last_two(s_first, s_second);
        };
        for (; kt + 6 <= KM; kt += 6) {
            iteration(S0{}, Even{}, r0, kt);
            iteration(S1{}, Odd{}, r1, kt + 1);
            iteration(S2{}, Even{}, r0, kt + 2);
            iteration(S0{}, Odd{}, r1, kt + 3);
            iteration(S1{}, Even{}, r0, kt + 4);
            iteration(S2{}, Odd{}, r1, kt + 5);
        }
        if (kt < KM) {
            iteration(S0{}, Even{}, r0, kt);
            if (kt + 1 < KM) {
                iteration(S1{}, Odd{}, r1, kt + 1);
                if (kt + 2 < KM) {
                    iteration(S2{}, Even{}, r0, kt + 2);
                    if (kt + 3 < KM) {
                        iteration(S0{}, Odd{}, r1, kt + 3);
                        if (kt + 4 < KM) {
                            iteration(S1{}, Even{}, r0, kt + 4);
                            tail(S2{}, S0{});
                        } else {
                            tail(S1{}, S2{});
                        }
                    } else {
                        tail(S0{}, S1{});
                    }
                } else {
                    tail(S2{}, S0{});
                }
            } else {
                tail(S1{}, S2{});
            }
        } else {
            tail(S0{}, S1{});
        }
        if constexpr (!INLINE_TAIL && !NO_TAIL) {
            switch (KM % 3) {
                case 0: last_two(S0{}, S1{}); break;
                case 1: last_two(S1{}, S2{}); break;
                default: last_two(S2{}, S0{}); break;
            }
        }
    }

    // ---- epilogue ---------------------------------------------------------------------------------------------
    // Lane holds acc[i][j][4g + r] = (m = i*32 + lane%32, n = j*32 + 8g + 4(lane/32) + r) of its wave tile: 4 consecutive
    // columns of one row, the unit every epilogue works on.  Results go through a per-wave LDS tile so that global
    // stores are 16 bytes per lane over whole contiguous row segments.
    const int N = a.N;
    __syncthreads();   // every wave is done reading the staging buffers
    if constexpr (KG > 1) {   // the groups' partial sums meet in group 0 (register r of thread t at word r * NT + t)
        if (kg > 0) {
            int32_t* part = reinterpret_cast<int32_t*>(smem + PART_BASE + (kg - 1) * PART_BYTES);
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) part[((i * NI + j) * 16 + r) * NT + tid] = acc[i][j][r];
        }
        __syncthreads();
        if (kg > 0) return;
#pragma unroll
        for (int g = 1; g < KG; ++g) {
            const int32_t* other = reinterpret_cast<const int32_t*>(smem + PART_BASE + (g - 1) * PART_BYTES);
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) acc[i][j][r] += other[((i * NI + j) * 16 + r) * NT + tid];
        }
    }
    auto epilogue = [&](auto epi_tag) {
    constexpr int epi = decltype(epi_tag)::value;
    constexpr int esize = epi == SCMX_EPI_I32 ? 4 : 2;
    constexpr int ocols = epi == SCMX_EPI_SWIGLU ? WTN / 2 : WTN;     // output columns of the wave tile
    const int on = epi == SCMX_EPI_SWIGLU ? N / 2 : N;            // output row length
    constexpr int rowb = ocols * esize;                                // bytes per tile row
    constexpr int rsb = rowb + 16;                                     // padded LDS row stride
    constexpr bool fits = WGM * WGN * WTM * rsb <= SMEM_BYTES;   // per-wave tiles reuse the staging LDS
    int8_t* wtile = smem + (fits ? wave * (WTM * rsb) : 0);
    const int wm0 = m0 + wm * WTM, wn0 = n0 + wn * WTN;            // wave tile origin (input column index)
    const bool wide = fits && (size_t(on) * esize) % 16 == 0 && reinterpret_cast<uintptr_t>(a.out) % 16 == 0 &&
                      (epi != SCMX_EPI_RES || reinterpret_cast<uintptr_t>(a.res) % 16 == 0);

    float xsv[MI];
    f32x4 wsv[NI][4];
    if (epi != SCMX_EPI_I32) {
#pragma unroll
        for (int i = 0; i < MI; ++i) xsv[i] = s_xs[wm * WTM + i * 32 + lr];
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g)
                wsv[j][g] = *reinterpret_cast<const f32x4*>(&s_ws[wn * WTN + j * 32 + 8 * g + 4 * half]);
    }
    auto emit = [&](auto wide_tag) __attribute__((always_inline)) {
    constexpr bool W = decltype(wide_tag)::value;
#pragma unroll
    for (int i = 0; i < MI; ++i) {
        const int row = i * 32 + lr;
        const int m = wm0 + row;
        const float xs = epi != SCMX_EPI_I32 ? xsv[i] : 0.0f;
#pragma unroll
        for (int j = 0; j < NI; ++j) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int col = j * 32 + 8 * g + 4 * half;
                const int n = wn0 + col;
                if (epi == SCMX_EPI_I32) {
                    const v4i v = v4i{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                    if (W)
                        *reinterpret_cast<v4i*>(wtile + row * rsb + col * 4) = v;
                    else if (m < row_end && n < N)
                        *reinterpret_cast<v4i*>(reinterpret_cast<int32_t*>(a.out) + size_t(m) * N + n) = v;
                    continue;
                }
                const f32x4 w4 = wsv[j][g];
                float y[4];
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    y[r] = __fmul_rn(__fmul_rn(float(acc[i][j][4 * g + r]), xs), w4[r]);
                uint16_t* out = reinterpret_cast<uint16_t*>(a.out);
                if (epi == SCMX_EPI_SWIGLU) {   // (g, g, u, u) -> two outputs
                    const uint16_t s0 = swiglu_lut(a.silu, y[0], round_bf16(y[2]));
                    const uint16_t s1 = swiglu_lut(a.silu, y[1], round_bf16(y[3]));
                    const uint32_t o = uint32_t(s0) | (uint32_t(s1) << 16);
                    if (W)
                        *reinterpret_cast<uint32_t*>(wtile + row * rsb + col) = o;
                    else if (m < row_end && n < N)
                        *reinterpret_cast<uint32_t*>(out + size_t(m) * on + n / 2) = o;
                    continue;
                }
                u32x2 o;
                o[0] = uint32_t(f32_to_bf16(y[0])) | (uint32_t(f32_to_bf16(y[1])) << 16);
                o[1] = uint32_t(f32_to_bf16(y[2])) | (uint32_t(f32_to_bf16(y[3])) << 16);
                if (W) {
                    *reinterpret_cast<u32x2*>(wtile + row * rsb + col * 2) = o;   // the residual is added on the way out
                } else if (m < row_end && n < N) {
                    if (epi == SCMX_EPI_RES) {
                        const u32x2 rr = *reinterpret_cast<const u32x2*>(a.res + size_t(m) * N + n);
#pragma unroll
                        for (int r = 0; r < 2; ++r) {
                            const float lo = __fadd_rn(__uint_as_float(rr[r] << 16), __uint_as_float(o[r] << 16));
                            const float hi = __fadd_rn(__uint_as_float(rr[r] & 0xFFFF0000u), __uint_as_float(o[r] & 0xFFFF0000u));
                            o[r] = uint32_t(f32_to_bf16(lo)) | (uint32_t(f32_to_bf16(hi)) << 16);
                        }
                    }
                    *reinterpret_cast<u32x2*>(out + size_t(m) * N + n) = o;
                }
            }
        }
    }
    };
    if (wide) emit(std::true_type{}); else emit(std::false_type{});
    if (!wide) return;
    __builtin_amdgcn_wave_barrier();   // LDS operations of one wave complete in order: the tile is visible to its lanes

    // read the tile back 16 bytes per lane, whole rows at a time, and store
    constexpr int ppr = rowb / 16;                 // 16-byte pieces per tile row (2, 4, 8 or 16)
    constexpr int epp = 16 / esize;                // output elements per piece
    const int ocol0 = epi == SCMX_EPI_SWIGLU ? wn0 / 2 : wn0;
    // In batches of eight pieces per lane: all LDS reads (and residual loads) of a batch are in flight before the first
    // is used, instead of one round trip per piece.
    constexpr int NP = WTM * ppr / 64, NB = NP < 8 ? NP : 8;
    static_assert(WTM * ppr % 64 == 0 && NP % NB == 0, "whole batches of pieces per lane");
#pragma unroll 1
    for (int p0 = lane; p0 < WTM * ppr; p0 += 64 * NB) {
        u32x4 v[NB], rr[NB];
        bool ok[NB], full[NB];
        int8_t* dst[NB];
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const int p = p0 + 64 * i;
            const int row = p / ppr, pc = p % ppr;
            const int m = wm0 + row, c = ocol0 + pc * epp;
            ok[i] = m < row_end && c < on;
            full[i] = c + epp <= on;
            dst[i] = reinterpret_cast<int8_t*>(a.out) + (size_t(m) * on + c) * esize;
            v[i] = *reinterpret_cast<const u32x4*>(wtile + row * rsb + pc * 16);
            if (epi == SCMX_EPI_RES) {
                rr[i] = u32x4{0u, 0u, 0u, 0u};
                if (ok[i]) {
                    if (full[i]) {
                        rr[i] = *reinterpret_cast<const u32x4*>(a.res + size_t(m) * on + c);
                    } else {
                        const u32x2 r2 = *reinterpret_cast<const u32x2*>(a.res + size_t(m) * on + c);
                        rr[i][0] = r2[0];
                        rr[i][1] = r2[1];
                    }
                }
            }
        }
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            if (!ok[i]) continue;
            if (epi == SCMX_EPI_RES) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float lo = __fadd_rn(__uint_as_float(rr[i][r] << 16), __uint_as_float(v[i][r] << 16));
                    const float hi = __fadd_rn(__uint_as_float(rr[i][r] & 0xFFFF0000u), __uint_as_float(v[i][r] & 0xFFFF0000u));
                    v[i][r] = uint32_t(f32_to_bf16(lo)) | (uint32_t(f32_to_bf16(hi)) << 16);
                }
            }
            if (full[i])
                // streaming store: the tile is not read again by this kernel, and lines that never sit dirty in the L2
                // do not have to be written back when the kernel ends
                __builtin_nontemporal_store(v[i], reinterpret_cast<u32x4*>(dst[i]));
            else   // the row ends inside this piece: rows are multiples of 4 elements, so exactly half of it is valid
                *reinterpret_cast<u32x2*>(dst[i]) = u32x2{v[i][0], v[i][1]};
        }
    }
    };
    switch (a.epi) {
        case SCMX_EPI_I32: epilogue(std::integral_constant<int, SCMX_EPI_I32>{}); break;
        case SCMX_EPI_SCALE: epilogue(std::integral_constant<int, SCMX_EPI_SCALE>{}); break;
        case SCMX_EPI_RES: epilogue(std::integral_constant<int, SCMX_EPI_RES>{}); break;
        default: epilogue(std::integral_constant<int, SCMX_EPI_SWIGLU>{}); break;
    }
}

// ---- host dispatch ---------------------------------------------------------------------------------------------

template <int BM, int BN, int BK, int WGM, int WGN, int OCC = 1, int FD = 2, bool SKIP = false, bool PK = false, int KG = 1,
          bool AD = false>
static void launch_tile(const GemmArgs& a_in, int bmode, int row_tiles, hipStream_t s) {
    GemmArgs a = a_in;
    if (a.epi == SCMX_EPI_SWIGLU) a.silu = silu_table_device();
    const int num_n = (a.N + BN - 1) / BN;
    if (a.tstart) row_tiles = (row_tiles + 7) & ~7;   // grouped: whole chunks of 8 row-tile slots (spare slots exit at once)
    const dim3 grid(unsigned(row_tiles) * unsigned(num_n)), block(WGM * WGN * KG * 64);
    if constexpr (PK) {   // callers choose this tile for the two FP4-conversion formats only
        if (bmode == B_PACKED_DEFAULT)
            gemm_kernel<BM, BN, BK, WGM, WGN, B_PACKED_DEFAULT, OCC, FD, SKIP, true><<<grid, block, 0, s>>>(a);
        else
            gemm_kernel<BM, BN, BK, WGM, WGN, B_PACKED_B16, OCC, FD, SKIP, true><<<grid, block, 0, s>>>(a);
    } else {
        if (bmode == B_INT8)
            gemm_kernel<BM, BN, BK, WGM, WGN, B_INT8, OCC, FD, SKIP, false, KG, AD><<<grid, block, 0, s>>>(a);
        else if (bmode == B_PACKED_DEFAULT)
            gemm_kernel<BM, BN, BK, WGM, WGN, B_PACKED_DEFAULT, OCC, FD, SKIP, false, KG, AD><<<grid, block, 0, s>>>(a);
        else if (bmode == B_PACKED_B16)
            gemm_kernel<BM, BN, BK, WGM, WGN, B_PACKED_B16, OCC, FD, SKIP, false, KG, AD><<<grid, block, 0, s>>>(a);
        else if (bmode == B_PACKED_B16M)
            gemm_kernel<BM, BN, BK, WGM, WGN, B_PACKED_B16M, OCC, FD, SKIP, false, KG, AD><<<grid, block, 0, s>>>(a);
        else if (bmode == B_PACKED_E8M0)
            gemm_kernel<BM, BN, BK, WGM, WGN, B_PACKED_E8M0, OCC, FD, SKIP, false, KG, AD><<<grid, block, 0, s>>>(a);
        else
            gemm_kernel<BM, BN, BK, WGM, WGN, B_PACKED_GENERIC, OCC, FD, SKIP, false, KG, AD><<<grid, block, 0, s>>>(a);
    }
}

static int packed_mode(const DevFormat& f) {
    return is_mxfp4_e8m0_format(f)     ? B_PACKED_E8M0
           : is_default_format(f)      ? B_PACKED_DEFAULT
           : is_pow2_block16_format(f) ? B_PACKED_B16
           : is_block16_range_format(f) ? B_PACKED_B16M
                                        : B_PACKED_GENERIC;
}

// Dense: one launch, with the tile a cost model of the candidates below makes fastest.
// Which tile a dense problem runs on: the index into the candidate table below.  blocked: the activations are in the
// blocked layout, which four tiles read (their waves then load activation fragments straight from memory).
static int dense_choice(long M, long N, long K, bool blocked) {
    const long cus = device_cus();
    auto tiles = [&](int bm, int bn) { return long((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    // The tile is the one a small cost model makes fastest.  A launch runs its tiles in waves of (CUs x workgroups that
    // share a CU); a wave costs F + S per 128 of K and not less than W, all three measured per configuration and per
    // number of co-resident workgroups (four Qwen3-1.7B layer shapes and five others, K = 128 ... 6144, M = 64 ... 8192:
    // the choice is within 2.5 % of the fastest configuration on all 118), and a last wave that leaves CUs idle runs
    // faster (less contention for the L2s and HBM).  What the table encodes: 256x256 moves the fewest LDS bytes per MFMA
    // and pays where it fills the chip or saves a round; a mostly empty last round costs more than a narrower tile's
    // extra LDS traffic; the small tiles share a CU and lose less to a ragged tile count; with no more 64x64 tiles
    // than CUs two K groups per tile put eight waves on a CU, and with no more 64x32 tiles than CUs four K groups of two
    // waves do (a 2048-wide layer on up to 128 rows: 64 ... 128 tiles instead of 32 ... 64; down 14.4 -> 10.2-10.9 us).
    // (A 256x64 tile was never the fastest and is gone.)
    struct Cand {
        int bm, bn, occ;
        float f[3], s[3], w[3];   // per wave, by co-resident workgroups 1..occ: fixed us, us per 128 of K, least us
        float low, mid;           // a wave on half of the CUs or fewer / on three quarters of them costs this part of a full one
    };
    static const Cand cand[7] = {
        {256, 256, 1, {6.5f, 0, 0}, {1.9f, 0, 0}, {8.4f, 0, 0}, 0.70f, 0.835f},
        {256, 128, 1, {4.2f, 0, 0}, {0.94f, 0, 0}, {5.5f, 0, 0}, 0.74f, 0.78f},
        {128, 128, 1, {1.4f, 0, 0}, {0.62f, 0, 0}, {3.0f, 0, 0}, 0.86f, 0.97f},
        {128, 64, 2, {1.4f, 1.2f, 0}, {0.39f, 0.77f, 0}, {2.2f, 3.0f, 0}, 0.91f, 1.0f},
        {64, 64, 3, {0.85f, 0.6f, 0.6f}, {0.34f, 0.53f, 0.70f}, {1.9f, 2.3f, 2.7f}, 0.95f, 1.0f},
        {64, 64, 1, {1.1f, 0, 0}, {0.26f, 0, 0}, {2.0f, 0, 0}, 0.97f, 1.0f},   // two K groups
        {64, 32, 1, {1.26f, 0, 0}, {0.14f, 0, 0}, {2.0f, 0, 0}, 0.95f, 0.97f},  // four K groups
    };
    // the same tiles fed from blocked activations (fewer LDS bytes per MFMA: a shorter K step)
    static const Cand cand_blocked[4] = {
        {256, 256, 1, {6.8f, 0, 0}, {1.78f, 0, 0}, {8.4f, 0, 0}, 0.70f, 0.835f},
        {256, 128, 1, {3.8f, 0, 0}, {0.92f, 0, 0}, {5.5f, 0, 0}, 0.74f, 0.78f},
        {128, 128, 1, {2.8f, 0, 0}, {0.58f, 0, 0}, {3.0f, 0, 0}, 0.86f, 0.97f},
        // eight waves stacked along M on 64 columns: half the weight staging of the 128x128 tile per MFMA, no activation
        // row fetched twice (2048-wide layers at M = 1024 ... 2048: 13.7 -> 12.2 us, K = 6144: 30.8 -> 28.9)
        {256, 64, 1, {2.2f, 0, 0}, {0.55f, 0, 0}, {3.0f, 0, 0}, 0.86f, 0.97f},
    };
    const float steps = float(K) / 128.0f;
    int best = blocked ? 2 : 4;
    float best_t = 1e30f;
    for (int c = 0; c < (blocked ? 4 : 7); ++c) {
        const Cand& k = blocked ? cand_blocked[c] : cand[c];
        const long n = tiles(k.bm, k.bn);
        if (c == 5 && (n > cus || K % 256)) continue;
        if (c == 6 && (n > cus || K % 512)) continue;
        const long cap = cus * k.occ;
        const long full = n / cap, rest = n % cap;
        float t = float(full) * fmaxf(k.f[k.occ - 1] + steps * k.s[k.occ - 1], k.w[k.occ - 1]);
        if (rest) {
            const int r = int((rest + cus - 1) / cus);   // workgroups per CU in the last wave
            float w = fmaxf(k.f[r - 1] + steps * k.s[r - 1], k.w[r - 1]);
            if (r == 1) {   // CUs idle
                const float fill = float(rest) / float(cus);
                w *= fill <= 0.5f    ? k.low
                     : fill <= 0.75f ? k.low + (k.mid - k.low) * (fill - 0.5f) * 4.0f
                                     : k.mid + (1.0f - k.mid) * (fill - 0.75f) * 4.0f;
            }
            t += w;
        }
        if (t < best_t * 0.98f) {   // candidates run from the largest tile down: a tie goes to the larger one
            best_t = t;
            best = c;
        }
    }
    return best;
}

static void launch_dense(const GemmArgs& a, int bmode, hipStream_t s) {
    const int best = dense_choice(a.M, a.N, a.K, a.blocked != 0);
    if (a.blocked) {
        switch (best) {
            case 0: return launch_tile<256, 256, 64, 4, 2, 1, 2, false, false, 1, true>(a, bmode, (a.M + 255) / 256, s);
            case 1: return launch_tile<256, 128, 128, 8, 1, 1, 2, false, false, 1, true>(a, bmode, (a.M + 255) / 256, s);
            case 3: return launch_tile<256, 64, 128, 8, 1, 1, 2, false, false, 1, true>(a, bmode, (a.M + 255) / 256, s);
            default: return launch_tile<128, 128, 128, 4, 2, 1, 2, false, false, 1, true>(a, bmode, (a.M + 127) / 128, s);
        }
    }
    switch (best) {
        case 0: return launch_tile<256, 256, 64, 2, 4, 1, 2>(a, bmode, (a.M + 255) / 256, s);
        case 1: return launch_tile<256, 128, 128, 4, 2, 1, 3>(a, bmode, (a.M + 255) / 256, s);
        case 2: return launch_tile<128, 128, 128, 4, 2, 1, 3>(a, bmode, (a.M + 127) / 128, s);
        case 3: return launch_tile<128, 64, 128, 4, 2>(a, bmode, (a.M + 127) / 128, s);
        case 5: return launch_tile<64, 64, 128, 2, 2, 1, 2, false, false, 2>(a, bmode, (a.M + 63) / 64, s);
        case 6: return launch_tile<64, 32, 128, 2, 1, 1, 2, false, false, 4>(a, bmode, (a.M + 63) / 64, s);
        default: return launch_tile<64, 64, 128, 2, 2>(a, bmode, (a.M + 63) / 64, s);
    }
}

static int check_gemm_common(const char* who, int M, int N, int K, int epi, bool need_scales, const void* xq,
                             const float* xscale, const float* wscale, const uint16_t* res, const void* out) {
    if (M < 0 || N <= 0 || K <= 0 || K % 128 || N % 4) {
        set_error("%s: need M >= 0, N %% 4 == 0 and K %% 128 == 0 (M=%d N=%d K=%d)", who, M, N, K);
        return SCMX_ERR_ARG;
    }
    if (uint64_t(M) * uint64_t(K) > 0xFFFFFFFFull || uint64_t(N) * uint64_t(K) > 0x7FFFFFFFull) {
        set_error("%s: operands beyond the 32-bit offsets of the kernel (M*K = %llu, N*K = %llu)", who,
                  (unsigned long long)(uint64_t(M) * K), (unsigned long long)(uint64_t(N) * K));
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
    if (epi == SCMX_EPI_SWIGLU && !silu_table_device()) {
        set_error("%s: the SiLU table of the SwiGLU epilogue could not be located on the device", who);
        return SCMX_ERR_LAUNCH;
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

static int mm_w4a8(const scmx_format* fmt, const int8_t* xq, const float* xscale, const uint32_t* codes,
                   const uint8_t* bcodes, const float* wscale, const uint16_t* res, void* out, int epi, int M, int N,
                   int K, bool blocked, void* stream) {
    DevFormat f;
    if (int rc = make_dev_format(fmt, &f)) return rc;
    if (int rc = check_gemm_common("mm_w4a8", M, N, K, epi, true, xq, xscale, wscale, res, out)) return rc;
    if (!codes || !bcodes || uintptr_t(codes) % 16 || K % f.block || (K / f.block * f.bc_bits) % 8) {
        set_error("mm_w4a8: codes must be 16-byte aligned, K a multiple of the block with whole block-code bytes per row");
        return SCMX_ERR_ARG;
    }
    if (f.e8m0 && !wscale) {
        set_error("mm_w4a8: the E8M0 form decodes with the row scales; wscale must not be NULL");
        return SCMX_ERR_ARG;
    }
    if (M == 0) return SCMX_OK;
    GemmArgs a = {};
    a.xq = xq; a.xscale = xscale; a.codes = codes; a.bcodes = bcodes; a.wscale = wscale; a.res = res; a.out = out;
    a.M = M; a.N = N; a.K = K; a.epi = epi; a.fmt = f;
    a.bc_row_bytes = K / f.block * f.bc_bits / 8;
    a.blocked = blocked;
    launch_dense(a, packed_mode(f), (hipStream_t)stream);
    return check_launch("mm_w4a8");
}

int scmx_mm_w4a8(const scmx_format* fmt, const int8_t* xq, const float* xscale, const uint32_t* codes,
                 const uint8_t* bcodes, const float* wscale, const uint16_t* res, void* out, int epi, int M, int N,
                 int K, void* stream) {
    return mm_w4a8(fmt, xq, xscale, codes, bcodes, wscale, res, out, epi, M, N, K, false, stream);
}

int scmx_mm_w4a8_blocked(const scmx_format* fmt, const int8_t* xq, const float* xscale, const uint32_t* codes,
                         const uint8_t* bcodes, const float* wscale, const uint16_t* res, void* out, int epi, int M,
                         int N, int K, void* stream) {
    if (uintptr_t(xq) % 16) {
        set_error("mm_w4a8_blocked: xq must be 16-byte aligned");
        return SCMX_ERR_ARG;
    }
    if (M > 0 && K > 0 && ((uint64_t(M) + 31) & ~uint64_t(31)) * uint64_t(K) > 0xFFFFFFFFull) {
        set_error("mm_w4a8_blocked: the activations' whole 32-row blocks lie beyond the 32-bit offsets of the kernel (M=%d K=%d)", M, K);
        return SCMX_ERR_ARG;
    }
    return mm_w4a8(fmt, xq, xscale, codes, bcodes, wscale, res, out, epi, M, N, K, true, stream);
}

int scmx_mm_w4a8_prefers_blocked(int M, int N, int K) {
    return M > 0 && N > 0 && K > 0 && K % 128 == 0 && dense_choice(M, N, K, false) <= 2;
}

// The fused layer quantizes into whichever layout suits the shape: blocked where the row-layout model would run one of its
// three largest tiles (the blocked tiles then win), by rows otherwise.  Both layouts take (M rounded up to 32) x K bytes at most.
static int quantize_and_multiply(const scmx_format* fmt, const uint16_t* x, int8_t* xq, float* xs, bool room_for_blocks,
                                 const uint32_t* codes, const uint8_t* bcodes, const float* wscale, const uint16_t* res,
                                 void* out, int epi, int M, int N, int K, void* stream) {
    const long long Mp = (static_cast<long long>(M) + 31) & ~31LL;
    const bool blocked = room_for_blocks && Mp <= (1LL << 30) && uint64_t(Mp) * uint64_t(K > 0 ? K : 0) <= 0xFFFFFFFFull &&
                         scmx_mm_w4a8_prefers_blocked(M, N, K);
    if (blocked) {
        if (int rc = scmx_act_quant_blocked(x, xq, xs, M, int(Mp), K, stream)) return rc;
    } else {
        if (int rc = scmx_act_quant(x, xq, xs, M, M, K, stream)) return rc;
    }
    return mm_w4a8(fmt, xq, xs, codes, bcodes, wscale, res, out, epi, M, N, K, blocked, stream);
}

size_t scmx_linear_w4a8_workspace(int M, int K) {
    if (M <= 0 || K <= 0) return 0;
    const size_t Mp = (size_t(M) + 31) & ~size_t(31);   // whole 32-row blocks of the blocked layout
    const size_t q = (Mp * size_t(K) + 255) & ~size_t(255);
    return q + Mp * sizeof(float);
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
    const size_t Mp = (size_t(M) + 31) & ~size_t(31);
    float* xs = reinterpret_cast<float*>(xq + ((Mp * size_t(K) + 255) & ~size_t(255)));
    return quantize_and_multiply(fmt, x, xq, xs, true, codes, bcodes, wscale, res, out, epi, M, N, K, stream);
}

// ---- the dense layer for callers that cannot allocate ------------------------------------------------------------
// The INT8 activations and their scales, which scmx_linear_w4a8 keeps in the caller's workspace, live here in a fixed
// array of the library's device image (every GPU the library runs on holds its own copy until the process ends).
// `scratch` is a host-side stand-in in host code, not a device address: the address on the current device comes from
// hipGetSymbolAddress, once per device, and only that pointer is handed to kernels.
constexpr size_t STATIC_XQ_BYTES = size_t(16) << 20;   // M * K <= 16 Mi elements, e.g. 2048 x 8192 or 8192 x 2048
constexpr int STATIC_MAX_ROWS = 16384;                 // M <= 16384 scales
constexpr size_t STATIC_SCRATCH_BYTES = STATIC_XQ_BYTES + size_t(STATIC_MAX_ROWS) * sizeof(float);
static __device__ __align__(256) uint8_t scratch[STATIC_SCRATCH_BYTES];

// Device address of `scratch` on the current device (NULL with the error text set when it cannot be resolved).
static uint8_t* static_scratch_device() {
    static std::atomic<uint8_t*> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        set_error("linear_w4a8_static: no current device (or a device index beyond 63)");
        return nullptr;
    }
    uint8_t* p = cached[dev].load(std::memory_order_acquire);
    if (!p) {
        void* addr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&addr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !addr) {
            set_error("linear_w4a8_static: hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
            return nullptr;
        }
        p = reinterpret_cast<uint8_t*>(addr);
        cached[dev].store(p, std::memory_order_release);
    }
    return p;
}

int scmx_init(void) {
    if (!static_scratch_device()) return SCMX_ERR_LAUNCH;
    if (!silu_table_device()) {
        set_error("init: the SiLU table of the SwiGLU epilogue could not be located on the current device");
        return SCMX_ERR_LAUNCH;
    }
    return SCMX_OK;
}

size_t scmx_linear_w4a8_static_max_elements(void) { return STATIC_XQ_BYTES; }
int scmx_linear_w4a8_static_max_rows(void) { return STATIC_MAX_ROWS; }

int scmx_linear_w4a8_static(const scmx_format* fmt, const uint16_t* x, const uint32_t* codes, const uint8_t* bcodes,
                            const float* wscale, const uint16_t* res, void* out, int epi, int M, int N, int K,
                            void* stream) {
    if (M < 0 || K <= 0) {
        set_error("linear_w4a8_static: bad shape M=%d K=%d", M, K);
        return SCMX_ERR_ARG;
    }
    if (size_t(M) * size_t(K) > STATIC_XQ_BYTES || M > STATIC_MAX_ROWS) {
        set_error("linear_w4a8_static: M*K = %zu elements or M = %d rows beyond the built-in scratch (%zu elements, %d "
                  "rows); use scmx_linear_w4a8 with a workspace", size_t(M) * size_t(K), M, STATIC_XQ_BYTES,
                  STATIC_MAX_ROWS);
        return SCMX_ERR_WORKSPACE;
    }
    uint8_t* base = static_scratch_device();
    if (!base) return SCMX_ERR_LAUNCH;
    int8_t* xq = reinterpret_cast<int8_t*>(base);
    float* xs = reinterpret_cast<float*>(base + STATIC_XQ_BYTES);
    // every byte of xq and xs[M] that the GEMM reads is written by the quantization first (in the blocked layout: the
    // whole last 32-row block, rows past M as zeros): nothing has to start at zero, whatever the previous call left behind
    const size_t Mp = (size_t(M) + 31) & ~size_t(31);
    const bool room = Mp * size_t(K) <= STATIC_XQ_BYTES && Mp <= size_t(STATIC_MAX_ROWS);
    return quantize_and_multiply(fmt, x, xq, xs, room, codes, bcodes, wscale, res, out, epi, M, N, K, stream);
}

static int moe_common(const char* who, const int8_t* xq, const float* xscale, const int32_t* gather, int R,
                      const float* wscale, const int32_t* off, const int32_t* tstart, int n_experts, int tm, int N,
                      int K, int epi, void* out, GemmArgs* a) {
    if (epi == SCMX_EPI_RES) {
        set_error("%s: the grouped GEMM has no residual epilogue", who);
        return SCMX_ERR_ARG;
    }
    if (int rc = check_gemm_common(who, R, N, K, epi, true, xq, xscale, wscale, nullptr, out)) return rc;
    if (!off || !tstart || n_experts < 1 || n_experts > (1 << 20) || !(tm == 64 || tm == 128 || tm == 256)) {
        set_error("%s: need off / tstart, 1 <= n_experts <= 2^20 and a row tile of 64, 128 or 256 (got %d)", who, tm);
        return SCMX_ERR_ARG;
    }
    *a = GemmArgs{};
    a->xq = xq; a->xscale = xscale; a->gather = gather; a->wscale = wscale; a->out = out;
    a->M = R; a->N = N; a->K = K; a->epi = epi; a->off = off; a->tstart = tstart; a->n_experts = n_experts;
    return SCMX_OK;
}

static void launch_grouped(const GemmArgs& a, int bmode, int tm, hipStream_t s) {
    const int max_tiles = (a.M + tm - 1) / tm + a.n_experts;   // e2e/sc_moe.py:155
    if (tm == 256 && (a.N % 256 == 0 || a.N >= 1024))   // 256-wide column tiles: fewer LDS bytes per MFMA
        launch_tile<256, 256, 64, 2, 4, 1, 2, true>(a, bmode, max_tiles, s);
    else if (tm == 256)
        launch_tile<256, 128, 128, 4, 2, 1, 3>(a, bmode, max_tiles, s);
    else if (tm == 128)
        launch_tile<128, 128, 128, 4, 2, 1, 3>(a, bmode, max_tiles, s);
    else if ((bmode == B_PACKED_DEFAULT || bmode == B_PACKED_B16) && a.K % 256 == 0 && a.N % 256 == 0 &&
             reinterpret_cast<uintptr_t>(a.bcodes) % 4 == 0)
        // few rows per expert: the pass streams the expert weights, and what it pays per weight is the staging.  The
        // packed tile writes and reads half the weight bytes in LDS, its eight waves sit side by side along N (every
        // fragment is decoded once) and two workgroups share a CU (128 registers).  Its lanes read the block codes of two
        // K steps with one aligned 2- or 4-byte load, hence the conditions on K and on the pointer.
        launch_tile<64, 256, 128, 1, 8, 4, 2, false, true>(a, bmode, max_tiles, s);
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
    if (f.e8m0 && !wscale) {
        set_error("moe_mm: the E8M0 form decodes with the row scales; wscale must not be NULL");
        return SCMX_ERR_ARG;
    }
    if (R == 0) return SCMX_OK;
    a.codes = codes; a.bcodes = bcodes; a.fmt = f;
    a.bc_row_bytes = K / f.block * f.bc_bits / 8;
    launch_grouped(a, packed_mode(f), tm, (hipStream_t)stream);
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
