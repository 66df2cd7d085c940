// Host-side check of the C ABI (include/scmx.h), built with AddressSanitizer and UBSan on the host pass and run on a
// machine WITHOUT a GPU: every entry point is called with null pointers, bad shapes, unsupported formats, sizes at the
// 32-bit limits and seeded random integers.  Nothing can launch here, so a call either refuses its arguments
// (SCMX_ERR_ARG / _FORMAT / _WORKSPACE), has nothing to do (SCMX_OK for empty inputs) or fails at the launch
// (SCMX_ERR_LAUNCH); the pointers handed in are not memory and must never be dereferenced by host code.  Any sanitizer
// report aborts the program; a wrong status prints the case and makes the exit code 1.
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <random>

#include "../include/scmx.h"

extern "C" int hipGetDeviceCount(int* count);   // from the HIP runtime the library links against

static int failures = 0;
static long calls = 0;

static void expect(int rc, int want, const char* what) {
    ++calls;
    if (rc != want) {
        printf("FAIL %s: status %d, expected %d (%s)\n", what, rc, want, scmx_last_error());
        ++failures;
    }
}
// A call that passes the argument checks ends at the launch on a machine without a device (or has nothing to do).
static void expect_valid(int rc, const char* what) {
    ++calls;
    if (rc != SCMX_OK && rc != SCMX_ERR_LAUNCH) {
        printf("FAIL %s: plausible arguments refused with %d (%s)\n", what, rc, scmx_last_error());
        ++failures;
    }
}
static void expect_status(int rc, const char* what) {
    ++calls;
    if (rc > 0 || rc < SCMX_ERR_WORKSPACE) {
        printf("FAIL %s: undocumented status %d\n", what, rc);
        ++failures;
    }
    if (rc != SCMX_OK && !scmx_last_error()[0]) {
        printf("FAIL %s: status %d without a message\n", what, rc);
        ++failures;
    }
}

int main() {
    int devices = 0;
    if (hipGetDeviceCount(&devices) == 0 && devices > 0) {
        printf("a GPU is present: this check passes addresses that are not memory and is meant for machines without one\n");
        return 77;
    }
    // not memory: 256-byte aligned addresses that fault if host code touches them
    uint8_t* const P = reinterpret_cast<uint8_t*>(uintptr_t(0x7100000000ull));
    auto p = [&](int i) { return P + size_t(i) * (size_t(1) << 30); };
    const uint16_t* h[6];
    for (int i = 0; i < 6; ++i) h[i] = reinterpret_cast<const uint16_t*>(p(i));
    const int8_t* xq = reinterpret_cast<const int8_t*>(p(6));
    int8_t* oq = reinterpret_cast<int8_t*>(p(7));
    const float* f0 = reinterpret_cast<const float*>(p(8));
    const float* f1 = reinterpret_cast<const float*>(p(9));
    float* of = reinterpret_cast<float*>(p(10));
    const uint32_t* codes = reinterpret_cast<const uint32_t*>(p(11));
    const uint8_t* bc = p(12);
    uint8_t* obc = p(13);
    uint32_t* ocodes = reinterpret_cast<uint32_t*>(p(14));
    int32_t* oi[5];
    for (int i = 0; i < 5; ++i) oi[i] = reinterpret_cast<int32_t*>(p(15 + i));
    uint16_t* oh[3];
    for (int i = 0; i < 3; ++i) oh[i] = reinterpret_cast<uint16_t*>(p(20 + i));
    const int32_t* ci = reinterpret_cast<const int32_t*>(p(23));
    const int64_t* pos = nullptr;
    void* out = p(24);
    void* wsp = p(25);

    scmx_format fmt;
    scmx_default_format(&fmt);
    if (fmt.block != 32 || fmt.bc_bits != 2 || fmt.n_mult != 4 || fmt.code_mag[7] != 12 || fmt.mult[3] != 8) {
        printf("FAIL default format\n");
        ++failures;
    }
    if (!strstr(scmx_version(), "gfx950")) {
        printf("FAIL version string\n");
        ++failures;
    }
    if (scmx_linear_w4a8_workspace(2048, 2048) != size_t(2048) * 2048 + 4 * 2048 ||
        scmx_linear_w4a8_workspace(1, 128) != 32 * 128 + 4 * 32 || scmx_linear_w4a8_workspace(0, 128) != 0 ||
        scmx_linear_w4a8_static_max_elements() != (size_t(16) << 20) || scmx_linear_w4a8_static_max_rows() != 16384) {
        printf("FAIL workspace sizes\n");
        ++failures;
    }

    scmx_format mx;
    scmx_mxfp4_format(&mx);
    if (mx.block != 32 || mx.bc_bits != 8 || mx.n_mult != 0 || mx.code_mag[7] != 12 || mx.mult[0] != 0) {
        printf("FAIL MXFP4 in-place format\n");
        ++failures;
    }
    expect(scmx_unpack_i8(&mx, codes, bc, oq, 8, 128, nullptr), SCMX_ERR_FORMAT, "unpack_i8 of the in-place MXFP4 form");
    expect(scmx_mm_w4a8(&mx, xq, nullptr, codes, bc, nullptr, nullptr, out, 0, 4, 8, 128, nullptr), SCMX_ERR_ARG,
           "mm_w4a8 in-place MXFP4 without row scales");
    expect(scmx_mxfp4_to_sc(bc, nullptr, nullptr, oi[0], 8, 128, nullptr), SCMX_ERR_ARG, "mxfp4_to_sc null wscale");

    // ---- refused arguments --------------------------------------------------------------------------------------------
    expect(scmx_unpack_i8(nullptr, codes, bc, oq, 8, 128, nullptr), SCMX_ERR_ARG, "unpack_i8 null format");
    expect(scmx_unpack_i8(&fmt, nullptr, bc, oq, 8, 128, nullptr), SCMX_ERR_ARG, "unpack_i8 null codes");
    expect(scmx_unpack_i8(&fmt, codes, bc, oq, 8, 100, nullptr), SCMX_ERR_ARG, "unpack_i8 K off the block grain");
    expect(scmx_unpack_i8(&fmt, codes, bc, oq, -1, 128, nullptr), SCMX_ERR_ARG, "unpack_i8 negative rows");
    expect(scmx_act_quant(nullptr, oq, of, 4, 4, 128, nullptr), SCMX_ERR_ARG, "act_quant null x");
    expect(scmx_act_quant(h[0], oq, of, 5, 4, 128, nullptr), SCMX_ERR_ARG, "act_quant Mp < M");
    expect(scmx_act_quant(h[0], oq, of, 4, 4, 12, nullptr), SCMX_ERR_ARG, "act_quant K % 8");
    expect(scmx_act_quant_blocked(nullptr, oq, of, 4, 32, 128, nullptr), SCMX_ERR_ARG, "act_quant_blocked null x");
    expect(scmx_act_quant_blocked(h[0], oq, of, 4, 4, 128, nullptr), SCMX_ERR_ARG, "act_quant_blocked Mp % 32");
    expect(scmx_act_quant_blocked(h[0], oq, of, 40, 32, 128, nullptr), SCMX_ERR_ARG, "act_quant_blocked Mp < M");
    expect(scmx_act_quant_blocked(h[0], oq, of, 4, 32, 48, nullptr), SCMX_ERR_ARG, "act_quant_blocked K % 32");
    expect(scmx_mm_i8_i32(xq, xq, oi[0], 4, 8, 100, nullptr), SCMX_ERR_ARG, "mm_i8_i32 K % 128");
    expect(scmx_mm_i8_i32(xq, nullptr, oi[0], 4, 8, 128, nullptr), SCMX_ERR_ARG, "mm_i8_i32 null wq");
    expect(scmx_mm_i8_i32(xq, xq, oi[0], 65536, 8, 65536, nullptr), SCMX_ERR_ARG, "mm_i8_i32 M*K beyond 32-bit offsets");
    expect(scmx_mm_epi(xq, xq, nullptr, f1, nullptr, out, 1, 4, 8, 128, nullptr), SCMX_ERR_ARG, "mm_epi null xscale");
    expect(scmx_mm_epi(xq, xq, f0, f1, nullptr, out, 2, 4, 8, 128, nullptr), SCMX_ERR_ARG, "mm_epi residual epilogue without res");
    expect(scmx_mm_epi(xq, xq, f0, f1, nullptr, out, 3, 4, 12, 128, nullptr), SCMX_ERR_ARG, "mm_epi SwiGLU with N % 8");
    expect(scmx_mm_epi(xq, xq + 1, f0, f1, nullptr, out, 1, 4, 8, 128, nullptr), SCMX_ERR_ARG, "mm_epi misaligned wq");
    expect(scmx_mm_w4a8(&fmt, xq, f0, codes, bc, f1, nullptr, out, 7, 4, 8, 128, nullptr), SCMX_ERR_ARG, "mm_w4a8 unknown epilogue");
    expect(scmx_mm_w4a8(&fmt, xq, f0, codes, bc, f1, nullptr, out, 1, 4, 6, 128, nullptr), SCMX_ERR_ARG, "mm_w4a8 N % 4");
    expect(scmx_mm_w4a8_blocked(&fmt, xq, f0, codes, bc, f1, nullptr, out, 1, 4, 6, 128, nullptr), SCMX_ERR_ARG, "mm_w4a8_blocked N % 4");
    expect(scmx_mm_w4a8_blocked(&fmt, xq, f0, codes, bc, f1, nullptr, out, 1, 4, 8, 192, nullptr), SCMX_ERR_ARG, "mm_w4a8_blocked K % 128");
    expect(scmx_mm_w4a8_blocked(&fmt, nullptr, f0, codes, bc, f1, nullptr, out, 1, 4, 8, 128, nullptr), SCMX_ERR_ARG, "mm_w4a8_blocked null xq");
    expect(scmx_mm_w4a8(&fmt, xq, f0, codes, nullptr, f1, nullptr, out, 1, 4, 8, 128, nullptr), SCMX_ERR_ARG, "mm_w4a8 null bcodes");
    {
        scmx_format bad = fmt;
        bad.bc_bits = 3;
        expect(scmx_mm_w4a8(&bad, xq, f0, codes, bc, f1, nullptr, out, 1, 4, 8, 128, nullptr), SCMX_ERR_FORMAT, "format bc_bits 3");
        bad = fmt;
        bad.block = 12;
        expect(scmx_gemv(&bad, xq, f0, codes, bc, f1, nullptr, oh[0], 1, 0, nullptr, 0.0f, 1, 8, 128, nullptr, 0, 0, -1, nullptr),
               SCMX_ERR_FORMAT, "format block 12");
        bad = fmt;
        bad.mult[3] = 16;   // 12 * 16 does not fit INT8
        expect(scmx_unpack_i8(&bad, codes, bc, oq, 8, 128, nullptr), SCMX_ERR_FORMAT, "format product beyond 127");
        bad = fmt;
        bad.n_mult = 5;     // more multipliers than 2-bit codes address
        expect(scmx_unpack_i8(&bad, codes, bc, oq, 8, 128, nullptr), SCMX_ERR_FORMAT, "format n_mult beyond 2^bc_bits");
        bad = fmt;
        bad.code_mag[2] = -1;
        expect(scmx_unpack_i8(&bad, codes, bc, oq, 8, 128, nullptr), SCMX_ERR_FORMAT, "format negative magnitude");
    }
    expect(scmx_linear_w4a8(&fmt, h[0], codes, bc, f1, nullptr, out, 1, 4, 8, 128, wsp, 16, nullptr), SCMX_ERR_WORKSPACE,
           "linear_w4a8 small workspace");
    expect(scmx_linear_w4a8(&fmt, h[0], codes, bc, f1, nullptr, out, 1, 4, 8, 128, nullptr, 1 << 20, nullptr), SCMX_ERR_WORKSPACE,
           "linear_w4a8 null workspace");
    expect(scmx_linear_w4a8(&fmt, h[0], codes, bc, f1, nullptr, out, 1, -4, 8, 128, wsp, 1 << 20, nullptr), SCMX_ERR_ARG,
           "linear_w4a8 negative M");
    expect(scmx_linear_w4a8_static(&fmt, h[0], codes, bc, f1, nullptr, out, 1, 8192, 128, 2176, nullptr), SCMX_ERR_WORKSPACE,
           "linear_w4a8_static M*K beyond the scratch");
    expect(scmx_linear_w4a8_static(&fmt, h[0], codes, bc, f1, nullptr, out, 1, 16385, 128, 128, nullptr), SCMX_ERR_WORKSPACE,
           "linear_w4a8_static rows beyond the scratch");
    expect(scmx_linear_w4a8_static(&fmt, h[0], codes, bc, f1, nullptr, out, 1, 4, 128, 0, nullptr), SCMX_ERR_ARG,
           "linear_w4a8_static K = 0");
    expect(scmx_rmsnorm_quant(h[0], nullptr, 1e-6f, oq, of, nullptr, 4, 4, 128, nullptr), SCMX_ERR_ARG, "rmsnorm_quant null weight");
    expect(scmx_rmsnorm_quant(h[0], h[1], 1e-6f, oq, of, nullptr, 4, 4, 130, nullptr), SCMX_ERR_ARG, "rmsnorm_quant K % 8");
    expect(scmx_rmsnorm_quant_blocked(h[0], h[1], 1e-6f, oq, of, nullptr, 4, 4, 512, nullptr), SCMX_ERR_ARG, "rmsnorm_quant_blocked Mp % 32");
    expect(scmx_rmsnorm_quant_blocked(h[0], h[1], 1e-6f, oq, of, nullptr, 4, 32, 768, nullptr), SCMX_ERR_ARG, "rmsnorm_quant_blocked K % 512");
    expect(scmx_rmsnorm_quant_blocked(h[0], h[1], 1e-6f, oq, of, nullptr, 4, 32, 8192, nullptr), SCMX_ERR_ARG, "rmsnorm_quant_blocked K > 4096");
    expect(scmx_res_norm_quant(nullptr, f0, f1, h[0], h[1], 1e-6f, oh[0], oq, of, 4, 128, nullptr), SCMX_ERR_ARG,
           "res_norm_quant null acc");
    expect(scmx_swiglu_quant(ci, f0, f1, nullptr, of, 4, 128, nullptr), SCMX_ERR_ARG, "swiglu_quant null xq");
    expect(scmx_qkv_headnorm(nullptr, f0, f1, nullptr, h[1], h[2], 1e-6f, oh[0], oh[1], oh[2], 4, 4, 2, 64, nullptr), SCMX_ERR_ARG,
           "qkv_headnorm neither acc nor y");
    expect(scmx_qkv_headnorm(nullptr, f0, f1, h[0], h[1], h[2], 1e-6f, oh[0], oh[1], oh[2], 4, 4, 3, 96, nullptr), SCMX_ERR_ARG,
           "qkv_headnorm head dim 96");
    expect(scmx_qkv_headnorm_rope(nullptr, f0, f1, h[0], h[1], h[2], 1e-6f, oh[0], oh[1], oh[2], 4, 4, 2, 64, f0, pos, 62, 64, 0,
                                  nullptr),
           SCMX_ERR_ARG, "qkv_headnorm_rope rows past the cache");
    expect(scmx_attn_decode(h[0], h[1], h[2], pos, 5, oh[0], 4, 2, 96, 64, 0.1f, nullptr, 1, nullptr), SCMX_ERR_ARG,
           "attn_decode head dim 96");
    expect(scmx_attn_decode(h[0], h[1], h[2], pos, 5, oh[0], 4, 2, 128, 64, 0.1f, nullptr, 4, nullptr), SCMX_ERR_ARG,
           "attn_decode splits without workspace");
    expect(scmx_attn_decode(h[0], h[1], h[2], pos, 65, oh[0], 4, 2, 128, 64, 0.1f, nullptr, 1, nullptr), SCMX_ERR_ARG,
           "attn_decode more valid rows than the cache");
    expect(scmx_attn_decode(h[0] + 1, h[1], h[2], pos, 5, oh[0], 4, 2, 128, 64, 0.1f, nullptr, 1, nullptr), SCMX_ERR_ARG,
           "attn_decode misaligned q");
    expect(scmx_attn_decode_qkv(h[0], h[1], h[2], 1e-6f, f0, pos, 64, oh[0], oh[1], oh[2], 4, 2, 128, 64, 0.1f, nullptr, 1, nullptr),
           SCMX_ERR_ARG, "attn_decode_qkv position outside the cache");
    expect(scmx_attn_prefill(h[0], h[1], h[2], oh[0], 8, 0, 4, 2, 64, 64, 0.1f, nullptr), SCMX_ERR_ARG, "attn_prefill head dim 64");
    expect(scmx_attn_prefill(h[0], h[1], h[2], oh[0], 60, 8, 4, 2, 128, 64, 0.1f, nullptr), SCMX_ERR_ARG,
           "attn_prefill rows past the cache");
    expect(scmx_qkv_fullnorm(h[0], h[1], h[2], 1e-6f, oh[0], oh[1], nullptr, 4, 4, 64, nullptr), SCMX_ERR_ARG, "qkv_fullnorm null v");
    expect(scmx_gemv(&fmt, xq, nullptr, codes, bc, f1, nullptr, oh[0], 1, 0, nullptr, 0.0f, 1, 8, 128, nullptr, 0, 0, -1, nullptr),
           SCMX_ERR_ARG, "gemv prologue 0 without xscale");
    expect(scmx_gemv(&fmt, xq, f0, codes, bc, f1, nullptr, oh[0], 1, 0, nullptr, 0.0f, 3, 8, 128, nullptr, 0, 0, -1, nullptr),
           SCMX_ERR_ARG, "gemv batch 3");
    expect(scmx_gemv(&fmt, xq, f0, codes, bc, f1, nullptr, oh[0], 2, 0, nullptr, 0.0f, 1, 8, 128, nullptr, 0, 0, -1, nullptr),
           SCMX_ERR_ARG, "gemv residual epilogue without res");
    expect(scmx_gemv(&fmt, h[0], nullptr, codes, bc, f1, nullptr, oh[0], 1, 2, nullptr, 1e-6f, 1, 8, 128, nullptr, 0, 0, -1, nullptr),
           SCMX_ERR_ARG, "gemv prologue 2 without norm weight");
    expect(scmx_gemv(&fmt, xq, f0, codes, bc, f1, nullptr, oh[0], 1, 0, nullptr, 0.0f, 2, 8, 128, ci, 2, 1, -1, nullptr), SCMX_ERR_ARG,
           "gemv expert gather with batch 2");
    expect(scmx_route_topk(h[0], nullptr, 4, 2000, 8, 1, oi[0], oh[0], nullptr), SCMX_ERR_ARG, "route_topk 2000 experts");
    expect(scmx_route_topk(h[0], nullptr, 4, 4, 8, 1, oi[0], oh[0], nullptr), SCMX_ERR_ARG, "route_topk k > E");
    expect(scmx_route_topk(h[0], nullptr, 4, 128, 65, 1, oi[0], oh[0], nullptr), SCMX_ERR_ARG, "route_topk k > 64");
    expect(scmx_route_sort(ci, 4, 8, 2000, 64, oi[0], oi[1], oi[2], oi[3], oi[4], nullptr), SCMX_ERR_ARG, "route_sort 2000 experts");
    expect(scmx_route_sort(ci, 1 << 30, 8, 64, 64, oi[0], oi[1], oi[2], oi[3], oi[4], nullptr), SCMX_ERR_ARG,
           "route_sort M*topk beyond 32 bits");
    expect(scmx_moe_mm(&fmt, xq, f0, nullptr, 100, codes, bc, f1, ci, ci, 4, 96, 8, 128, 1, out, nullptr), SCMX_ERR_ARG,
           "moe_mm row tile 96");
    expect(scmx_moe_mm(&fmt, xq, f0, nullptr, 100, codes, bc, f1, ci, ci, 4, 64, 8, 128, 2, out, nullptr), SCMX_ERR_ARG,
           "moe_mm residual epilogue");
    expect(scmx_moe_mm(&fmt, xq, f0, nullptr, 100, codes, bc, f1, nullptr, ci, 4, 64, 8, 128, 1, out, nullptr), SCMX_ERR_ARG,
           "moe_mm null off");
    expect(scmx_moe_mm_i8(xq, f0, nullptr, 100, nullptr, f1, ci, ci, 4, 64, 8, 128, 1, out, nullptr), SCMX_ERR_ARG, "moe_mm_i8 null wq");
    expect(scmx_moe_combine(h[0], ci, h[1], nullptr, h[2], nullptr, 0.0f, oh[0], oq, of, 4, 4, 128, 8, nullptr), SCMX_ERR_ARG,
           "moe_combine quantization without norm weight");
    expect(scmx_moe_combine(h[0], ci, h[1], nullptr, h[2], nullptr, 0.0f, oh[0], nullptr, nullptr, 5, 4, 128, 8, nullptr), SCMX_ERR_ARG,
           "moe_combine Mp < M");
    expect(scmx_rot_quant(h[0], f0, oq, of, 4, 4, 100, nullptr), SCMX_ERR_ARG, "rot_quant K % 32");
    expect(scmx_rot_quant(h[0], f0, oq, of, 4, 4, 16384, nullptr), SCMX_ERR_ARG, "rot_quant K > 8192");
    expect(scmx_mxfp4_to_sc(bc, obc, of, nullptr, 4, 128, nullptr), SCMX_ERR_ARG, "mxfp4_to_sc null status");
    expect(scmx_mxfp4_to_sc(bc, obc, of, oi[0], 4, 100, nullptr), SCMX_ERR_ARG, "mxfp4_to_sc K % 128");
    expect(scmx_quantize_sc(f0, 0, 4, 96, 32, ocodes, obc, of, nullptr), SCMX_ERR_ARG, "quantize_sc K % (4 block)");
    expect(scmx_quantize_sc(f0, 0, 4, 128, 24, ocodes, obc, of, nullptr), SCMX_ERR_ARG, "quantize_sc block 24");
    expect(scmx_quantize_sc(f0, 0, 4, 262144, 32, ocodes, obc, of, nullptr), SCMX_ERR_ARG, "quantize_sc K > 131072");
    expect(scmx_quantize_family(&fmt, f0, 0, 4, 32768, ocodes, obc, of, nullptr), SCMX_ERR_ARG, "quantize_family K > 16384");
    expect(scmx_quantize_family(nullptr, f0, 0, 4, 128, ocodes, obc, of, nullptr), SCMX_ERR_ARG, "quantize_family null format");

    // ---- nothing to do --------------------------------------------------------------------------------------------------
    expect(scmx_mm_w4a8(&fmt, xq, f0, codes, bc, f1, nullptr, out, 1, 0, 8, 128, nullptr), SCMX_OK, "mm_w4a8 M = 0");
    expect(scmx_mm_epi(xq, xq, f0, f1, nullptr, out, 1, 0, 8, 128, nullptr), SCMX_OK, "mm_epi M = 0");
    expect(scmx_act_quant(h[0], oq, of, 0, 0, 128, nullptr), SCMX_OK, "act_quant no rows");
    expect(scmx_moe_mm(&fmt, xq, f0, nullptr, 0, codes, bc, f1, ci, ci, 4, 64, 8, 128, 1, out, nullptr), SCMX_OK, "moe_mm R = 0");
    expect(scmx_route_topk(h[0], nullptr, 0, 64, 8, 1, oi[0], oh[0], nullptr), SCMX_OK, "route_topk M = 0");
    expect(scmx_qkv_fullnorm(h[0], h[1], h[2], 1e-6f, oh[0], oh[1], oh[2], 0, 4, 64, nullptr), SCMX_OK, "qkv_fullnorm L = 0");

    // ---- plausible arguments: accepted, and stopped by the missing device at the earliest ---------------------------------
    expect_valid(scmx_unpack_i8(&fmt, codes, bc, oq, 4096, 2048, nullptr), "unpack_i8");
    expect_valid(scmx_act_quant(h[0], oq, of, 2048, 2048, 2048, nullptr), "act_quant");
    expect_valid(scmx_act_quant(h[0], oq, of, 7, 128, 1000, nullptr), "act_quant ragged K");
    expect_valid(scmx_act_quant_blocked(h[0], oq, of, 2048, 2048, 2048, nullptr), "act_quant_blocked");
    expect_valid(scmx_act_quant_blocked(h[0], oq, of, 7, 32, 96, nullptr), "act_quant_blocked short rows");
    expect_valid(scmx_mm_i8_i32(xq, xq, oi[0], 2048, 4096, 2048, nullptr), "mm_i8_i32");
    for (int epi = 0; epi <= 3; ++epi)
        expect_valid(scmx_mm_w4a8(&fmt, xq, f0, codes, bc, f1, h[0], out, epi, 2048, 12288, 2048, nullptr), "mm_w4a8");
    expect_valid(scmx_mm_w4a8(&fmt, xq, f0, codes, bc, f1, nullptr, out, 1, 1, 4, 128, nullptr), "mm_w4a8 smallest");
    for (int epi = 0; epi <= 3; ++epi)
        expect_valid(scmx_mm_w4a8_blocked(&fmt, xq, f0, codes, bc, f1, h[0], out, epi, 2048, 12288, 2048, nullptr), "mm_w4a8_blocked");
    expect_valid(scmx_mm_w4a8_blocked(&fmt, xq, f0, codes, bc, f1, nullptr, out, 1, 1, 4, 128, nullptr), "mm_w4a8_blocked smallest");
    expect_valid(scmx_mm_w4a8(&fmt, xq, f0, codes, bc, f1, nullptr, out, 1, 8192, 2048, 6144, nullptr), "mm_w4a8 M = 8192");
    expect_valid(scmx_linear_w4a8(&fmt, h[0], codes, bc, f1, nullptr, out, 1, 2048, 4096, 2048, wsp,
                                  scmx_linear_w4a8_workspace(2048, 2048), nullptr),
                 "linear_w4a8");
    expect_valid(scmx_linear_w4a8_static(&fmt, h[0], codes, bc, f1, nullptr, out, 1, 2048, 4096, 2048, nullptr), "linear_w4a8_static");
    expect_valid(scmx_rmsnorm_quant(h[0], h[1], 1e-6f, oq, of, oh[0], 200, 256, 2048, nullptr), "rmsnorm_quant");
    expect_valid(scmx_rmsnorm_quant_blocked(h[0], h[1], 1e-6f, oq, of, oh[0], 200, 256, 2048, nullptr), "rmsnorm_quant_blocked");
    expect_valid(scmx_res_norm_quant(ci, f0, f1, h[0], h[1], 1e-6f, oh[0], oq, of, 256, 2048, nullptr), "res_norm_quant");
    expect_valid(scmx_swiglu_quant(ci, f0, f1, oq, of, 256, 6144, nullptr), "swiglu_quant");
    expect_valid(scmx_qkv_headnorm(nullptr, f0, f1, h[0], h[1], h[2], 1e-6f, oh[0], oh[1], oh[2], 200, 16, 8, 128, nullptr),
                 "qkv_headnorm");
    expect_valid(scmx_qkv_headnorm_rope(nullptr, f0, f1, h[0], h[1], h[2], 1e-6f, oh[0], oh[1], oh[2], 200, 16, 8, 128, f0, pos, 0, 512,
                                        1, nullptr),
                 "qkv_headnorm_rope");
    expect_valid(scmx_attn_decode(h[0], h[1], h[2], pos, 300, oh[0], 16, 8, 128, 512, 0.088f, nullptr, 1, nullptr), "attn_decode");
    expect_valid(scmx_attn_decode(h[0], h[1], h[2], pos, 3000, oh[0], 16, 8, 128, 4096, 0.088f, of, 8, nullptr), "attn_decode split");
    expect_valid(scmx_attn_decode_qkv(h[0], h[1], h[2], 1e-6f, f0, pos, 300, oh[0], oh[1], oh[2], 16, 8, 128, 512, 0.088f, nullptr, 1,
                                      nullptr),
                 "attn_decode_qkv");
    expect_valid(scmx_attn_prefill(h[0], h[1], h[2], oh[0], 2048, 0, 16, 8, 128, 2048, 0.088f, nullptr), "attn_prefill");
    expect_valid(scmx_qkv_fullnorm(h[0], h[1], h[2], 1e-6f, oh[0], oh[1], oh[2], 100, 16, 128, nullptr), "qkv_fullnorm");
    for (int batch : {1, 2, 4, 8})
        for (int pro = 0; pro <= 2; ++pro)
            expect_valid(scmx_gemv(&fmt, pro ? (const void*)h[0] : (const void*)xq, pro ? nullptr : f0, codes, bc, f1, h[1], oh[0],
                                   1 + pro % 2, pro, pro == 2 ? h[2] : nullptr, 1e-6f, batch, 151936, 2048, nullptr, 0, 0, -1, nullptr),
                         "gemv");
    expect_valid(scmx_gemv(&fmt, xq, f0, codes, bc, f1, nullptr, oh[0], 3, 0, nullptr, 0.0f, 1, 1024, 2048, ci, 8, 0, 256, nullptr),
                 "gemv expert slots");
    expect_valid(scmx_route_topk(h[0], h[1], 2048, 256, 8, 1, oi[0], oh[0], nullptr), "route_topk");
    expect_valid(scmx_route_sort(ci, 4096, 8, 64, 256, oi[0], oi[1], oi[2], oi[3], oi[4], nullptr), "route_sort");
    expect_valid(scmx_route_sort(ci, 10, 2, 8, 64, oi[0], oi[1], oi[2], oi[3], oi[4], nullptr), "route_sort small");
    for (int tm : {64, 128, 256})
        expect_valid(scmx_moe_mm(&fmt, xq, f0, ci, 32768, codes, bc, f1, ci, ci, 64, tm, 2048, 2048, 3, out, nullptr), "moe_mm");
    expect_valid(scmx_moe_mm_i8(xq, f0, nullptr, 600, xq, f1, ci, ci, 8, 64, 256, 512, 0, out, nullptr), "moe_mm_i8");
    expect_valid(scmx_moe_combine(h[0], ci, h[1], nullptr, h[2], h[3], 1e-5f, oh[0], oq, of, 200, 256, 2048, 8, nullptr), "moe_combine");
    expect_valid(scmx_rot_quant(h[0], f0, oq, of, 17, 128, 1536, nullptr), "rot_quant");
    expect_valid(scmx_mxfp4_to_sc(bc, obc, of, oi[0], 4096, 2048, nullptr), "mxfp4_to_sc");
    expect_valid(scmx_quantize_sc(f0, 0, 12288, 2048, 32, ocodes, obc, of, nullptr), "quantize_sc");
    expect_valid(scmx_quantize_sc(h[0], 1, 512, 2048, 16, ocodes, obc, of, nullptr), "quantize_sc bf16, 16-blocks");
    expect_valid(scmx_quantize_family(&fmt, f0, 0, 2048, 2048, ocodes, obc, of, nullptr), "quantize_family");

    // ---- seeded random integers, extremes included: any documented status, never undefined behaviour -----------------------
    std::mt19937 rng(12345);
    const int pool[] = {-2147483647 - 1, -1, 0, 1, 2, 3, 4, 7, 8, 16, 31, 32, 64, 100, 127, 128, 129, 255, 256, 512, 1000, 1024,
                        2048, 4096, 6144, 8192, 16384, 32768, 65536, 131072, 151936, 1 << 20, 1 << 24, 1 << 30, 2147483647};
    auto r = [&]() { return pool[rng() % (sizeof(pool) / sizeof(pool[0]))]; };
    auto maybe = [&](const void* q) { return (rng() % 8) ? q : nullptr; };
    for (int it = 0; it < 4000; ++it) {
        scmx_format f = fmt;
        if (rng() % 4 == 0) {
            f.block = r();
            f.bc_bits = int(rng() % 10);
            f.n_mult = r();
            f.code_mag[rng() % 8] = r();
            f.mult[rng() % 16] = r();
        }
        expect_status(scmx_unpack_i8(&f, (const uint32_t*)maybe(codes), bc, oq, r(), r(), nullptr), "fuzz unpack_i8");
        expect_status(scmx_act_quant((const uint16_t*)maybe(h[0]), oq, of, r(), r(), r(), nullptr), "fuzz act_quant");
        expect_status(scmx_act_quant_blocked((const uint16_t*)maybe(h[0]), oq, of, r(), r(), r(), nullptr), "fuzz act_quant_blocked");
        expect_status(scmx_mm_epi(xq, (const int8_t*)maybe(xq), f0, f1, (const uint16_t*)maybe(h[0]), out, int(rng() % 6) - 1, r(), r(), r(),
                                  nullptr),
                      "fuzz mm_epi");
        expect_status(scmx_mm_w4a8(&f, xq, f0, codes, bc, f1, (const uint16_t*)maybe(h[0]), out, int(rng() % 6) - 1, r(), r(), r(), nullptr),
                      "fuzz mm_w4a8");
        expect_status(scmx_mm_w4a8_blocked(&f, xq, f0, codes, bc, f1, (const uint16_t*)maybe(h[0]), out, int(rng() % 6) - 1, r(), r(), r(),
                                           nullptr),
                      "fuzz mm_w4a8_blocked");
        const int lm = r(), lk = r();
        expect_status(scmx_linear_w4a8(&f, h[0], codes, bc, f1, nullptr, out, 1, lm, r(), lk, wsp,
                                       (rng() % 2) ? scmx_linear_w4a8_workspace(lm, lk) : size_t(r()), nullptr),
                      "fuzz linear_w4a8");
        expect_status(scmx_linear_w4a8_static(&f, h[0], codes, bc, f1, nullptr, out, 1, r(), r(), r(), nullptr), "fuzz linear_w4a8_static");
        expect_status(scmx_rmsnorm_quant(h[0], h[1], 1e-6f, oq, of, (uint16_t*)maybe(oh[0]), r(), r(), r(), nullptr), "fuzz rmsnorm_quant");
        expect_status(scmx_rmsnorm_quant_blocked(h[0], h[1], 1e-6f, oq, of, (uint16_t*)maybe(oh[0]), r(), r(), r(), nullptr), "fuzz rmsnorm_quant_blocked");
        expect_status(scmx_res_norm_quant(ci, f0, f1, h[0], h[1], 1e-6f, oh[0], (int8_t*)maybe(oq), of, r(), r(), nullptr),
                      "fuzz res_norm_quant");
        expect_status(scmx_swiglu_quant(ci, f0, f1, oq, of, r(), r(), nullptr), "fuzz swiglu_quant");
        expect_status(scmx_qkv_headnorm((const int32_t*)maybe(ci), f0, f1, (const uint16_t*)maybe(h[0]), h[1], h[2], 1e-6f, oh[0], oh[1],
                                        oh[2], r(), r(), r(), r(), nullptr),
                      "fuzz qkv_headnorm");
        expect_status(scmx_qkv_headnorm_rope(nullptr, f0, f1, h[0], h[1], h[2], 1e-6f, oh[0], oh[1], oh[2], r(), r(), r(), r(), f0, pos,
                                             int64_t(r()) * (rng() % 3), r(), int(rng() % 2), nullptr),
                      "fuzz qkv_headnorm_rope");
        expect_status(scmx_attn_decode(h[0], h[1], h[2], pos, r(), oh[0], r(), r(), r(), r(), 0.1f, (float*)maybe(of), r(), nullptr),
                      "fuzz attn_decode");
        expect_status(scmx_attn_decode_qkv(h[0], h[1], h[2], 1e-6f, f0, pos, int64_t(r()) * (rng() % 3), oh[0], oh[1], oh[2], r(), r(), r(),
                                           r(), 0.1f, (float*)maybe(of), r(), nullptr),
                      "fuzz attn_decode_qkv");
        expect_status(scmx_attn_prefill(h[0], h[1], h[2], oh[0], r(), r(), r(), r(), r(), r(), 0.1f, nullptr), "fuzz attn_prefill");
        expect_status(scmx_qkv_fullnorm(h[0], h[1], h[2], 1e-6f, oh[0], oh[1], oh[2], r(), r(), r(), nullptr), "fuzz qkv_fullnorm");
        expect_status(scmx_gemv(&f, xq, (const float*)maybe(f0), codes, bc, f1, (const uint16_t*)maybe(h[1]), oh[0], int(rng() % 6) - 1,
                                int(rng() % 5) - 1, (const uint16_t*)maybe(h[2]), 1e-6f, r(), r(), r(), (const int32_t*)maybe(ci), r(), r(),
                                r(), nullptr),
                      "fuzz gemv");
        expect_status(scmx_route_topk(h[0], (const uint16_t*)maybe(h[1]), r(), r(), r(), int(rng() % 2), oi[0], oh[0], nullptr),
                      "fuzz route_topk");
        expect_status(scmx_route_sort(ci, r(), r(), r(), r(), oi[0], oi[1], oi[2], oi[3], oi[4], nullptr), "fuzz route_sort");
        expect_status(scmx_moe_mm(&f, xq, f0, (const int32_t*)maybe(ci), r(), codes, bc, f1, ci, ci, r(), r(), r(), r(), int(rng() % 6) - 1,
                                  out, nullptr),
                      "fuzz moe_mm");
        expect_status(scmx_moe_mm_i8(xq, f0, nullptr, r(), xq, f1, ci, ci, r(), r(), r(), r(), int(rng() % 6) - 1, out, nullptr),
                      "fuzz moe_mm_i8");
        expect_status(scmx_moe_combine(h[0], ci, h[1], (const uint16_t*)maybe(h[4]), h[2], (const uint16_t*)maybe(h[3]), 1e-5f, oh[0],
                                       (int8_t*)maybe(oq), of, r(), r(), r(), r(), nullptr),
                      "fuzz moe_combine");
        expect_status(scmx_rot_quant(h[0], f0, oq, of, r(), r(), r(), nullptr), "fuzz rot_quant");
        expect_status(scmx_mxfp4_to_sc(bc, obc, of, oi[0], r(), r(), nullptr), "fuzz mxfp4_to_sc");
        expect_status(scmx_quantize_sc(f0, int(rng() % 2), r(), r(), r(), ocodes, obc, of, nullptr), "fuzz quantize_sc");
        expect_status(scmx_quantize_family(&f, f0, int(rng() % 2), r(), r(), ocodes, obc, of, nullptr), "fuzz quantize_family");
        (void)scmx_linear_w4a8_workspace(r(), r());
    }
    printf("%ld calls, %d failure(s)\n", calls, failures);
    return failures ? 1 : 0;
}
