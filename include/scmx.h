/* scmx — C ABI of the MI355X (gfx950) SC-MXFP4 W4A8 linear-layer engine.
 *
 * Every entry point enqueues HIP kernels on the caller's stream and returns at once (stream-ordered, no implicit
 * synchronisation).  Pointers are DEVICE pointers unless stated otherwise; the library never allocates or frees
 * device memory and keeps no state between calls (beyond the per-device address of its constant SiLU lookup table,
 * looked up once), so it is reentrant.  Return value: 0 on success, a negative
 * SCMX_ERR_* code otherwise, with a message available from scmx_last_error() (thread-local).
 *
 * Each declaration names the function of the reference (shinyoungkang1/mxfp4-int8-m5) it replaces, as file:line.
 * `T` tensors are bfloat16 (uint16_t bit patterns) — the model dtype the reference runs with.
 *
 * Weight storage (e2e/sc_format.py:4-15): per row n of an [N, K] matrix
 *   codes   uint32 [N*K/8]   8 four-bit codes per word, element k = 8j+i in bits 4i..4i+3; code = sign<<3 | idx
 *   bcodes  uint8  [N, K*bc_bits/(8*block)]  block b in bits bc_bits*(b % per_byte) of byte b / per_byte
 *   wscale  float  [N]
 * decoding to the INT8 operand q[n,k] = +-code_mag[idx] * mult[bcode[n, k/block]], W = wscale[n] * q.
 */
#ifndef SCMX_H
#define SCMX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SCMX_OK 0
#define SCMX_ERR_ARG (-1)      /* bad shape, null pointer, misaligned pointer */
#define SCMX_ERR_FORMAT (-2)   /* weight format outside what the kernels decode */
#define SCMX_ERR_LAUNCH (-3)   /* HIP reported an error at launch */
#define SCMX_ERR_WORKSPACE (-4)/* caller-provided workspace too small */

/* Epilogues of the GEMM / GEMV (e2e/sc_kernels.py:73-78, e2e/sc_moe.py:10). */
#define SCMX_EPI_I32 0     /* INT32 accumulators */
#define SCMX_EPI_SCALE 1   /* T(acc * xscale[m] * wscale[n]) */
#define SCMX_EPI_RES 2     /* T(res + T(acc * xscale[m] * wscale[n])) */
#define SCMX_EPI_SWIGLU 3  /* rows interleaved g,g,u,u: swiglu(T(g), T(u)) -> [M, N/2] */

/* Weight format descriptor: the fields of sc_format.Format (e2e/sc_format.py:26-37), passed per call instead of
 * the reference's process-global F.DEFAULT (e2e/sc_kernels.py:471-473). */
typedef struct scmx_format {
    int32_t block;        /* weights per block along K: 8, 16, 32, 64 or 128 */
    int32_t bc_bits;      /* bits per block code: 1, 2, 4 or 8 */
    int32_t n_mult;       /* entries used in mult[], <= 16 and <= 2^bc_bits */
    int32_t code_mag[8];  /* magnitude of code index 0..7; max(code_mag) * max(mult) <= 127 */
    int32_t mult[16];     /* integer block multipliers */
} scmx_format;

const char* scmx_version(void);
const char* scmx_last_error(void);

/* Optional set-up for the CURRENT device: looks up the device addresses of the library's two device-resident objects (the
 * SiLU table of the SwiGLU epilogue and the built-in scratch of scmx_linear_w4a8_static) so that no later call has to.
 * Those look-ups are runtime calls outside any stream (the first one may load the code object); every entry point
 * performs them on first use, which is fine in eager code but must not happen while a stream is being captured into a HIP
 * graph: call scmx_init() once per device (or make one eager call of the entry points you capture) before capturing.
 * Idempotent, thread-safe, allocates nothing.  No counterpart in the reference (mx.compile needs no such step). */
int scmx_init(void);

/* Fill `f` with the published SC-MXFP4 format: block 32, magnitudes 2 x E2M1, multipliers 1,2,4,8, 2-bit codes
 * (sc_format.DEFAULT, e2e/sc_format.py:63). */
void scmx_default_format(scmx_format* f);

/* Fill `f` with the descriptor of a STANDARD MXFP4 tensor read in place (block 32, bc_bits 8, n_mult 0): `codes` are the
 * tensor's E2M1 nibble bytes (two codes per byte, even k low), `bcodes` its E8M0 scale bytes [N, K/32], one per
 * 32-block, exactly as e2e/fused_qwen38.py:319-334 lays them out; `wscale` [N] = 2^(lowest exponent byte of the row -
 * 128), which scmx_mxfp4_to_sc writes (with bcodes = NULL it writes nothing else).  A block decodes with shift = byte -
 * lowest, so a row's bytes must lie in 1..254 and span at most 3 (scmx_mxfp4_to_sc reports otherwise).  Accepted by
 * scmx_gemv, scmx_mm_w4a8, scmx_linear_w4a8(_static) and scmx_moe_mm; scmx_unpack_i8 takes the converted form only. */
void scmx_mxfp4_format(scmx_format* f);

/* ---- dense prefill ------------------------------------------------------------------------------------------ */

/* Packed weights -> INT8 [n_rows, K].  Replaces unpack_i8, e2e/sc_kernels.py:34-50,480-483 (and unpack_experts,
 * e2e/sc_moe.py:203-206, with n_rows = E*N). */
int scmx_unpack_i8(const scmx_format* fmt, const uint32_t* codes, const uint8_t* bcodes, int8_t* wq,
                   int64_t n_rows, int64_t K, void* stream);

/* Per-token symmetric INT8 of x T[M, K]: xq int8 [Mp, K], xs float [Mp]; rows >= M are zero with scale 0.
 * Replaces act_quant, e2e/sc_kernels.py:200-229,554-563. */
int scmx_act_quant(const uint16_t* x, int8_t* xq, float* xs, int M, int Mp, int K, void* stream);

/* scmx_act_quant (e2e/sc_kernels.py:200-229) writing xq in the BLOCKED layout that scmx_mm_w4a8_blocked reads: blocks
 * of 32 rows x 32 k (1 KB each), block (m / 32, k / 32) at byte ((m / 32) * (K / 32) + k / 32) * 1024, and inside a block
 * the 16 bytes xq[m, 16 j .. 16 j + 15] (j = k / 16) at ((j % 2) * 32 + m % 32) * 16.  Same codes and scales as
 * scmx_act_quant.  Mp % 32 == 0, K % 32 == 0; xq holds Mp * K bytes, rows >= M are zero with scale 0. */
int scmx_act_quant_blocked(const uint16_t* x, int8_t* xq, float* xs, int M, int Mp, int K, void* stream);

/* INT8 [M,K] x INT8 [N,K]^T -> INT32 [M,N] on INT8 MFMA.  Replaces mm_i8_i32, e2e/sc_kernels.py:53-71,486-495. */
int scmx_mm_i8_i32(const int8_t* xq, const int8_t* wq, int32_t* acc, int M, int N, int K, void* stream);

/* The same GEMM with the scaling epilogue applied in registers; `res` T[M,N] is read by SCMX_EPI_RES only.
 * out: T[M,N] (epi 1,2), T[M,N/2] (epi 3).  Replaces mm_epi, e2e/sc_kernels.py:79-115,498-508. */
int scmx_mm_epi(const int8_t* xq, const int8_t* wq, const float* xscale, const float* wscale, const uint16_t* res,
                void* out, int epi, int M, int N, int K, void* stream);

/* mm_epi reading the PACKED weights: each workgroup unpacks its weight tile into LDS as exact INT8 and feeds the
 * INT8 MFMA from there, so no INT8 copy of the weights is ever written (the in-kernel unpack of
 * e2e/sc_moe.py:42-69 applied to the dense path; replaces the unpack_i8 + mm_epi pair of
 * e2e/fused_qwen3.py:161-172).  epi 0 writes INT32 [M,N]. */
int scmx_mm_w4a8(const scmx_format* fmt, const int8_t* xq, const float* xscale, const uint32_t* codes,
                 const uint8_t* bcodes, const float* wscale, const uint16_t* res, void* out, int epi, int M, int N,
                 int K, void* stream);

/* scmx_mm_w4a8 on activations in the blocked layout of scmx_act_quant_blocked (xq: ceil(M / 32) * 32 rows, 16-byte
 * aligned): the waves of the large tiles load their activation fragments straight from memory, and only the weights
 * pass through LDS.  Same results as scmx_mm_w4a8 (same integers, same epilogues).  Meant for prefill-sized M: every
 * shape runs, on 128x128 tiles at least.  The same pair of reference calls as scmx_mm_w4a8 (e2e/fused_qwen3.py:161-172). */
int scmx_mm_w4a8_blocked(const scmx_format* fmt, const int8_t* xq, const float* xscale, const uint32_t* codes,
                         const uint8_t* bcodes, const float* wscale, const uint16_t* res, void* out, int epi, int M,
                         int N, int K, void* stream);

/* 1 when a dense problem of this shape runs faster from blocked activations (it is large enough for the tiles that read
 * them), 0 when the row layout is the one to quantize into; what scmx_linear_w4a8 decides by.  No device work. */
int scmx_mm_w4a8_prefers_blocked(int M, int N, int K);

/* Whole dense W4A8 linear on a bf16 input: activation quantization prologue + scmx_mm_w4a8, one call (the activations
 * are quantized into the blocked layout when the shape runs on a tile that reads it).
 * workspace must hold scmx_linear_w4a8_workspace(M, K) bytes (the INT8 activations and their scales). */
size_t scmx_linear_w4a8_workspace(int M, int K);
int scmx_linear_w4a8(const scmx_format* fmt, const uint16_t* x, const uint32_t* codes, const uint8_t* bcodes,
                     const float* wscale, const uint16_t* res, void* out, int epi, int M, int N, int K,
                     void* workspace, size_t workspace_bytes, void* stream);

/* scmx_linear_w4a8 for callers that cannot allocate device memory or provide a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): the INT8 activations and their scales are kept in a
 * fixed array inside the library's device image instead of a workspace, so the call allocates nothing and takes no
 * scratch argument.  No counterpart in the reference.  Limits: M * K <= scmx_linear_w4a8_static_max_elements()
 * (16 Mi) and M <= scmx_linear_w4a8_static_max_rows() (16384); larger shapes return SCMX_ERR_WORKSPACE.  Same results as
 * scmx_linear_w4a8.  All calls on one GPU share that GPU's array: calls that overlap on one GPU (different streams
 * or threads) race and must be serialised by the caller; each GPU holds 16.06 MiB for it until the process ends.
 * Under graph capture: call scmx_init() (or this entry point once, eagerly) on the device before the capture begins. */
size_t scmx_linear_w4a8_static_max_elements(void);
int scmx_linear_w4a8_static_max_rows(void);
int scmx_linear_w4a8_static(const scmx_format* fmt, const uint16_t* x, const uint32_t* codes, const uint8_t* bcodes,
                            const float* wscale, const uint16_t* res, void* out, int epi, int M, int N, int K,
                            void* stream);

/* ---- row kernels of the model integrations -------------------------------------------------------------------- */

/* RMSNorm(x, w, eps) then per-token INT8; xn (optional, may be NULL) receives the normalized T rows [Mp, K].
 * Replaces rmsnorm_quant / rmsnorm_quant_n, e2e/sc_kernels.py:123-174,383-386,527-533,619-626. */
int scmx_rmsnorm_quant(const uint16_t* x, const uint16_t* w, float eps, int8_t* xq, float* xs, uint16_t* xn, int M,
                       int Mp, int K, void* stream);

/* scmx_rmsnorm_quant writing xq in the blocked layout of scmx_act_quant_blocked (for scmx_mm_w4a8_blocked); xn stays by
 * rows.  Same codes and scales.  Mp % 32 == 0, K % 512 == 0, K <= 4096, 16-byte aligned operands.  The same reference
 * function (e2e/sc_kernels.py:123-174,527-533). */
int scmx_rmsnorm_quant_blocked(const uint16_t* x, const uint16_t* w, float eps, int8_t* xq, float* xs, uint16_t* xn, int M,
                               int Mp, int K, void* stream);

/* h = res + T(acc*xscale*wscale) written to h; then, when xq != NULL, RMSNorm(h, w, eps) + INT8.
 * Replaces res_norm_quant (e2e/sc_kernels.py:177-189,536-544) and res_epilogue (:191-197,547-551). */
int scmx_res_norm_quant(const int32_t* acc, const float* xscale, const float* wscale, const uint16_t* res,
                        const uint16_t* w, float eps, uint16_t* h, int8_t* xq, float* xs, int Mp, int K,
                        void* stream);

/* acc INT32 [Mp, 2F] (gate | up) -> per-token INT8 [Mp, F] of swiglu(T(gate), T(up)).
 * Replaces swiglu_quant, e2e/sc_kernels.py:279-315,585-594. */
int scmx_swiglu_quant(const int32_t* acc, const float* xscale, const float* wscale, int8_t* xq, float* xs, int Mp,
                      int F, void* stream);

/* Qwen3 q/k/v split with per-head RMSNorm of q and k, head-major outputs [heads, L, d].  Input is either the INT32
 * accumulators with their scales (acc != NULL; qkv_epilogue_headnorm, e2e/sc_kernels.py:333-356,597-606) or the T
 * GEMM output y (qkv_headnorm_y, :359-380,609-616). */
int scmx_qkv_headnorm(const int32_t* acc, const float* xscale, const float* wscale, const uint16_t* y,
                      const uint16_t* qn, const uint16_t* kn, float eps, uint16_t* q, uint16_t* k, uint16_t* v,
                      int L, int hq, int hk, int d, void* stream);

/* scmx_qkv_headnorm followed by the rotary embedding of q and k (pairs (i, i + d/2) of a head, angle = position *
 * inv_freq[i], inv_freq f32 [d/2]) and the append to the KV cache: q -> [hq, L, d] (q_token_major != 0: [L, hq, d],
 * the layout from which an attention output needs no transpose before the o projection); k, v -> rows pos..pos+L-1 of
 * caches [hk, cache_rows, d].  pos = *pos_dev when pos_dev != NULL (a device-resident position, so that a captured
 * graph can be replayed for every token), else pos0.  With pos_dev the caller guarantees *pos_dev + L <= cache_rows.
 * Fuses what the model integrations do with array ops after qkv_headnorm_y: at.rope(q), at.rope(k),
 * cache.update_and_fetch(k, v) (e2e/fused_qwen3.py:216-221). */
int scmx_qkv_headnorm_rope(const int32_t* acc, const float* xscale, const float* wscale, const uint16_t* y,
                           const uint16_t* qn, const uint16_t* kn, float eps, uint16_t* q, uint16_t* kcache,
                           uint16_t* vcache, int L, int hq, int hk, int d, const float* inv_freq,
                           const int64_t* pos_dev, int64_t pos0, int cache_rows, int q_token_major, void* stream);

/* Single-token attention against a KV cache: out bf16 [hq * d] = softmax(q . K^T * scale) V per query head, q bf16
 * [hq, d], caches bf16 [hk, cache_rows, d] of which the first n rows are valid; n = *pos_dev + 1 when pos_dev != NULL
 * (device-resident position, for graph replay; a value outside 0 .. cache_rows - 1 gives an all-zero output and
 * touches no cache row).  q and the caches 16-byte aligned.  d in {64, 128, 256}.  Takes the place of the
 * array library's scaled-dot-product attention at L = 1 in the decode step (e2e/decode.py:1-5, e2e/fused_qwen3.py:
 * 216-222), so that the step is a fixed launch sequence.  splits > 1 (at most 64; for long contexts): the valid rows
 * are cut into `splits` ranges, one workgroup per head and range, and a second launch merges the ranges' results out of
 * `workspace`, float [splits * hq * (d + 2)]; splits == 1 needs no workspace (NULL). */
int scmx_attn_decode(const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache, const int64_t* pos_dev, int n,
                     uint16_t* out, int hq, int hk, int d, int cache_rows, float scale, float* workspace, int splits,
                     void* stream);

/* scmx_qkv_headnorm_rope at L = 1 and scmx_attn_decode in one launch: y bf16 [(hq + 2 hk) * d] is the token's q|k|v
 * row from the qkv projection; per-head RMSNorm of q and k, rotary embedding at position p (*pos_dev, or pos0 when
 * pos_dev is NULL), append of k and v to row p of the caches, attention over rows 0..p (a device-resident p outside
 * 0 .. cache_rows - 1 appends nothing and gives an all-zero output).  Same bits as the two calls
 * (with the same `splits`; workspace / splits as for scmx_attn_decode).
 * One launch less per block of the batch-1 decode step (e2e/decode.py:51-82; the array ops it stands for are
 * e2e/fused_qwen3.py:216-222). */
int scmx_attn_decode_qkv(const uint16_t* y, const uint16_t* qn, const uint16_t* kn, float eps, const float* inv_freq,
                         const int64_t* pos_dev, int64_t pos0, uint16_t* kcache, uint16_t* vcache, uint16_t* out,
                         int hq, int hk, int d, int cache_rows, float scale, float* workspace, int splits,
                         void* stream);

/* Causal attention of L new tokens against a KV cache that holds `off` earlier rows followed by the L new ones:
 * q bf16 [L, hq, d] (token-major, as scmx_qkv_headnorm_rope writes it with q_token_major), caches bf16
 * [hk, cache_rows, d], out bf16 [L, hq * d]; query i attends to cache rows 0 .. off + i.  d = 128.  float32
 * accumulation, bf16 probabilities.  Takes the place of the array library's scaled-dot-product attention in the
 * prefill (e2e/fused_qwen3.py:216-222); no counterpart among the reference's own kernels. */
int scmx_attn_prefill(const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache, uint16_t* out, int L, int off,
                      int hq, int hk, int d, int cache_rows, float scale, void* stream);

/* OLMoE q/k/v split with RMSNorm over the full h*d width.  Replaces qkv_fullnorm_y, e2e/sc_kernels.py:390-423,
 * 629-637. */
int scmx_qkv_fullnorm(const uint16_t* y, const uint16_t* qn, const uint16_t* kn, float eps, uint16_t* q,
                      uint16_t* k, uint16_t* v, int L, int h, int d, void* stream);

/* ---- decode --------------------------------------------------------------------------------------------------- */

/* W4A8 GEMV on packed weights, `batch` input rows sharing one weight stream (batch 1, 2, 4 or 8; the reference has
 * batch 1).
 *   pro 0: xq int8 [batch, K] + xscale [batch];  pro 1: x T[batch, K] quantized in the kernel;
 *   pro 2: RMSNorm(x, nw, eps) then INT8 in the kernel.
 *   eidx != NULL (MoE): `slots` output rows, slot j uses expert eidx[j] (or `shared_expert` for the slot after the
 *   n_eidx routed ones when shared_expert >= 0) and input row j * xstride; batch must be 1.
 * out: T[slots or batch, N] (epi 1, 2), T[.., N/2] (epi 3).  Replaces gemv, e2e/sc_decode.py:19-183,208-238. */
int scmx_gemv(const scmx_format* fmt, const void* x, const float* xscale, const uint32_t* codes,
              const uint8_t* bcodes, const float* wscale, const uint16_t* res, uint16_t* out, int epi, int pro,
              const uint16_t* nw, float eps, int batch, int N, int K, const int32_t* eidx, int n_eidx, int xstride,
              int shared_expert, void* stream);

/* ---- mixture of experts ----------------------------------------------------------------------------------------- */

/* Router: bf16 logits [M, n_experts] -> the topk experts of largest softmax probability per token and their scores.
 * Probabilities are bf16(softmax in float32); scores are those probabilities, divided by their sum (bf16) when
 * renorm != 0.  inds int32 / scores bf16 [M, topk], slots by falling probability, equal ones by rising expert index
 * (the reference leaves both to argpartition).  shared_logit != NULL (bf16 [M], the shared expert's gate logit): one
 * more slot per token, rows become [M, topk + 1] with inds = n_experts and score = bf16(sigmoid(shared_logit)).
 * n_experts <= 1024, topk <= min(64, n_experts).  Replaces route, e2e/fused_olmoe.py:183-192 (softmax, argpartition,
 * take_along_axis, optional renormalisation) and e2e/fused_qwen35.py:171-180 (renormalised, shared expert as the
 * last slot with its sigmoid gate); the router's linear layer stays the caller's. */
int scmx_route_topk(const uint16_t* logits, const uint16_t* shared_logit, int M, int n_experts, int topk, int renorm,
                    int32_t* inds, uint16_t* scores, void* stream);

/* Counting sort of the M*topk token-expert assignments by expert: pos [R], tok [R+tm], esorted [R], off [E+1],
 * tstart [E+1] (tile starts for row tiles of tm).  Replaces route_sort, e2e/sc_moe.py:114-155. */
int scmx_route_sort(const int32_t* inds, int M, int topk, int n_experts, int tm, int32_t* pos, int32_t* tok,
                    int32_t* esorted, int32_t* off, int32_t* tstart, void* stream);

/* Grouped W4A8 GEMM over expert segments: rows [off[e], off[e+1]) of the sorted activations use expert e's packed
 * weights (codes [E, N*K/8], bcodes [E, N, ..], wscale [E, N]).  When `gather` != NULL, sorted row r reads
 * xq[gather[r]] and xscale[gather[r]] (the xq[tok] gather of e2e/fused_olmoe.py:230 folded into the A-tile load);
 * otherwise xq / xscale are already in sorted order.  tm = 64, 128 or 256 is the row tile `tstart` was built for.
 * out: INT32 [R,N] (epi 0), T[R,N] (1), T[R,N/2] (3).
 * Replaces moe_mm, e2e/sc_moe.py:19-92,169-185. */
int scmx_moe_mm(const scmx_format* fmt, const int8_t* xq, const float* xscale, const int32_t* gather, int R,
                const uint32_t* codes, const uint8_t* bcodes, const float* wscale, const int32_t* off,
                const int32_t* tstart, int n_experts, int tm, int N, int K, int epi, void* out, void* stream);

/* The two-pass variant on pre-unpacked INT8 weights [E*N, K].  Replaces moe_mm_i8, e2e/sc_moe.py:95-107,188-200. */
int scmx_moe_mm_i8(const int8_t* xq, const float* xscale, const int32_t* gather, int R, const int8_t* wq,
                   const float* wscale, const int32_t* off, const int32_t* tstart, int n_experts, int tm, int N,
                   int K, int epi, void* out, void* stream);

/* h[t] = res[t] + sum_j T(T(y[pos[t,j]] * score[t,j]) + acc) accumulated sequentially in T; rows >= M copy res.
 * sscore != NULL: the last slot's score comes from sscore[t] and scores is [M, topk-1] (moe_combine_split).
 * When xq != NULL also RMSNorm(h, w, eps) + INT8.  Replaces moe_combine / moe_combine_split,
 * e2e/fused_olmoe.py:34-97. */
int scmx_moe_combine(const uint16_t* y, const int32_t* pos, const uint16_t* scores, const uint16_t* sscore,
                     const uint16_t* res, const uint16_t* w, float eps, uint16_t* h, int8_t* xq, float* xs, int M,
                     int Mp, int K, int topk, void* stream);

/* Randomized Hadamard rotation of every 32-wide block of x T[M, K] (signs f32 [K], +-1; FP32 butterflies, result times
 * 1/sqrt(32) rounded to T), then per-token INT8 as scmx_act_quant.  K % 32 == 0, K <= 8192.
 * Replaces rot_quant, e2e/sc_kernels.py:231-275,571-582. */
int scmx_rot_quant(const uint16_t* x, const float* signs, int8_t* xq, float* xs, int M, int Mp, int K, void* stream);

/* ---- standard MXFP4 interchange --------------------------------------------------------------------------------- */

/* Standard MXFP4 rows (E2M1 nibbles + one E8M0 byte per 32-block, e8m0 [N, K/32]) -> block codes and row scales of
 * the default format: shift = e8m0 - min over the row, wscale = 2^(min - 128).  The nibble bytes are used as the
 * code words unchanged.  status[0] (cleared by the caller) gets bit 0 set when some row's exponents span more than 3 (not
 * INT8-embeddable) and bit 1 when a row holds the bytes 0 or 255 (fine for the converted form, not for reading the
 * tensor in place).  bcodes may
 * be NULL: then only the row scales are written, which is all that the in-place form (scmx_mxfp4_format) needs.
 * Device form of the map in e2e/fused_qwen38.py:319-334 (inverse direction) and e2e/gptq_pack.py:29-47. */
int scmx_mxfp4_to_sc(const uint8_t* e8m0, uint8_t* bcodes, float* wscale, int32_t* status, int64_t N, int64_t K,
                     void* stream);

/* ---- offline quantizer ------------------------------------------------------------------------------------------ */

/* Float weights w [N, K] (float32, or bf16 when w_is_bf16 != 0) -> SC-MXFP4 in the packed layout with `block`-wide
 * blocks (32 = the published format, 16 = its 16-block power-of-two sibling): codes u32 [N*K/8], bcodes u8
 * [N, K/(4*block)] (2-bit shifts), wscale f32 [N] = 2^(E_lo - 1).  Per block the exponent floor(log2 amax) - 2 is
 * tried against its two neighbours (-1 first, then +1, strict improvement of the float64 squared error), rows are
 * constrained to an exponent spread of 3, values are rounded to E2M1 with ties to the lower magnitude.  Bit-identical
 * to the host procedure: sim/mx_int8.py:39-109 (block_exponents "search", constrain_spread, dequant_mx, embed_int8),
 * sim/make_testcase.py:26-44 (pack), e2e/sc_format.py:105-111 (quantize).  K % (4*block) == 0, K <= 131072. */
int scmx_quantize_sc(const void* w, int w_is_bf16, int64_t N, int K, int block, uint32_t* codes, uint8_t* bcodes,
                     float* wscale, void* stream);

/* The quantizer of the integer-exact format family w = base[row] * mult[block] * sign * code (float32 decisions): the
 * largest row base is peak / (max mult * max code); 8 bases per octave below it are tried in descending order, each
 * with the per-block multiplier of least squared error, and the first strictly best total wins.  fmt gives block (16
 * or 32), the ascending code magnitudes and multipliers and the block-code width; outputs in fmt's packed layout
 * with wscale = the row base.  Bit-identical to the host procedure sim/formats.py:64-107 (quantize_mx) followed by
 * e2e/pack_format.py:44-76 (pack_matrix / pack_parts).  K a multiple of 8 / bc_bits blocks, at most 16384. */
int scmx_quantize_family(const scmx_format* fmt, const void* w, int w_is_bf16, int64_t N, int K, uint32_t* codes,
                         uint8_t* bcodes, float* wscale, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SCMX_H */
