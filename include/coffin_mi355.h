/*
 * C ABI of the MI355X (gfx950) quantized-linear kernels.
 *
 * This is the whole boundary between the host adapter and the device code:
 * plain device pointers, sizes and a HIP stream, `int` status out.  Each entry
 * point names the reference interface it stands in for (paths relative to the
 * MuWinds/coffin tree).  The reference binds its kernels with pybind11 and
 * torch types; a maintainer replaces those bindings with the ctypes stub in
 * coffin_amd/_native.py.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer valid on the current HIP device;
 *   - bf16 tensors are passed as `const void*` / `void*` (16-bit patterns);
 *   - all tensors are dense row-major unless a leading dimension is given;
 *   - `stream` is a hipStream_t (NULL = the legacy default stream; callers on
 *     torch pass torch.cuda.current_stream().cuda_stream);
 *   - nothing synchronises, allocates or reads device memory on the host;
 *   - return 0 on success, otherwise one of CMI_E_* and a message retrievable
 *     with cmi_last_error() (thread-local).
 */
#ifndef COFFIN_MI355_H
#define COFFIN_MI355_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CMI_OK 0
#define CMI_E_ARG 1         /* null pointer, non-positive size, misalignment */
#define CMI_E_UNSUPPORTED 2 /* shape outside what the kernels are built for   */
#define CMI_E_HIP 3         /* a HIP runtime call failed                       */

/* ABI version; bumped when a signature changes. */
int cmi_abi_version(void);

/* Kernel-selection override for tests and tuning; no counterpart in the reference.
 *   "gemm_tile"     0 (the library chooses) | 64 | 128 | 192 | 256 | 320 (tile along n) | 6464 (64 x 64)
 *                   | 128192 (128 n x 192 m) | 321 (the 256 x 320 tile walked weight tile by weight
 *                   tile: what the library runs where it chooses that tile; 320 names the older
 *                   two-stage kernel) | 322 (321 as one workgroup per CU that walks its tiles one
 *                   after the other; measures the same as 321 and is never the library's choice):
 *                   block tile of cmi_gemm_w8a8 / cmi_gemm_w4a8 (non-zero also
 *                   bypasses their few-row routes);
 *   "gemv_wholerow" -1 (the library chooses) | 0 (never) | 1: the one-wavefront-per-weight-row
 *                   kernel of cmi_gemv_w8a16;
 *   "w4_decode_waves" 0 (the library chooses) | 4 | 16: wavefronts per workgroup of the W4A8
 *                   decode GEMV (one bf16 or quantised row);
 *   "w4_decode_chain" 0 (the library chooses) | 1 (never) | lanes + 100 * split + 10000 * waves: the
 *                   W4A8 decode kernel that keeps the fp32 chain in registers, with `lanes` (8, 16)
 *                   lanes per weight row, `split` (1, 2, 4, 8) wavefronts sharing a row and `waves`
 *                   (4, 8, 16) wavefronts per workgroup, wherever the shape fits that arrangement
 *                   (a combination that is not built, or a shape it does not fit, leaves the
 *                   choice to the library).
 * The environment variables CMI_GEMM_TILE and CMI_GEMV_WHOLEROW give the initial values; they are
 * read once, at the first call that needs them.  Unknown names or values: CMI_E_ARG.  Every choice
 * gives the same bits. */
int cmi_set_option(const char *name, int value);

/* Message for the last non-zero status returned on this thread ("" if none). */
const char *cmi_last_error(void);

/* Per-token symmetric int8 quantisation, x bf16 [M,K] -> q int8 [M,K], s fp32 [M]:
 *   s = max(amax_k |x|, 1e-5) / 127 ;  q = clamp(rne(x / s), -127, 127)
 * with an IEEE fp32 division.  Replaces Ops.kv_quant
 * (backends/protocol.py:252-258, spec backends/reference/__init__.py:367-390)
 * and the native quant_act_i8 (backends/corex/kernels/w8a8.cu:75-107,
 * bound at backends/corex/kernels/w8a8.cu:213-240). */
int cmi_quant_act_i8(const void *x, int8_t *q, float *s, int M, int K, void *stream);

/* int8 weight-only GEMV, 1 <= M <= 16:
 *   y[m,n] = bf16( ws[n] * sum_k wq[n,k] * x[m,k] ),  fp32 accumulation,
 * wq int8 [N,K], ws fp32 [N], x bf16 [M,K], y bf16 [M,N].  K % 16 == 0.
 * Row m of a batched call is bit-identical to the M=1 call on x[m].
 * Replaces gemv_nk_i8 / gemv_nk_i8_m (backends/corex/kernels/gemv.cu:838-990,
 * called from backends/corex/__init__.py:424,533) and gemv_w8a16*
 * (backends/hip/kernels/gemv_int8.cu:61-212). */
int cmi_gemv_w8a16(const int8_t *wq, const float *ws, const void *x, void *y,
                   int M, int N, int K, void *stream);

/* The same product for a batch with the sums on the matrix pipe
 * (v_mfma_f32_16x16x32_bf16; int8 -> bf16 is exact), 1 <= M <= 16,
 * K % 128 == 0 (else CMI_E_UNSUPPORTED: use cmi_gemv_w8a16); also
 * up to 64 rows (up to K = 10240 the weight is still read once, the rows go through in chunks
 * of 16 with the 16-row arithmetic; longer weight rows are read once per 16 activation rows).
 * 2-3 times faster than cmi_gemv_w8a16 at 8-16 rows.  A row's bits depend on K
 * only, not on the rows it travels with, but differ from cmi_gemv_w8a16's in
 * the last place (fp32 summation order): for callers without the
 * "batched row == single-row call" obligation of static-batch decode
 * (models/qwen35/batch.py:19-22) -- speculative verify, whose entry may use a
 * path of its own (backends/protocol.py:152-155), and short prefill chunks.
 * Stands where gemv_nk_i8_m is used for those callers
 * (backends/corex/__init__.py:495-546). */
int cmi_gemv_w8a16_mfma(const int8_t *wq, const float *ws, const void *x, void *y,
                        int M, int N, int K, void *stream);

/* int8 weight-only projection of any number of rows, with the kernel family named by the caller:
 *   CMI_FAMILY_DOT   cmi_gemv_w8a16, 16 rows per launch: row m carries the bits of the single-row call
 *                    (what static-batch decode owes its users, models/qwen35/batch.py:19-22);
 *   CMI_FAMILY_MFMA  cmi_gemv_w8a16_mfma, 64 rows per launch (K % 128 == 0, else
 *                    CMI_E_UNSUPPORTED and nothing is launched): 1.5-2.8 times faster at 4-16 rows,
 *                    slower at one row; a row's bits depend on K only.
 * The rule holds inside either family as long as every call on a weight -- single rows included --
 * names the same one, so the family is a property of a weight (or of a deployment), not of a call
 * site.  Stands where linear / linear_m / linear_m_verify reach gemv_nk_i8 / gemv_nk_i8_m
 * (backends/corex/__init__.py:396-425,495-546). */
#define CMI_FAMILY_DOT 0
#define CMI_FAMILY_MFMA 1
int cmi_linear_w8a16(const int8_t *wq, const float *ws, const void *x, void *y, int M, int N, int K,
                     int family, void *stream);

/* Identity of the capture `stream` is recording into: 0 when it is not capturing, a positive
 * number that differs between captures while it is, -1 when the runtime cannot say.  No
 * counterpart in the reference; the adapter uses it to keep decisions taken at capture time
 * (which scratch a captured kernel reads) from leaking between graphs. */
long long cmi_stream_capture_id(void *stream);

/* One-time re-layout of a W4A8Weight for the device kernels.
 *   in : packed u8 [ceil(Kp/2), N] (low nibble = even k, code = q+8; Kp = K rounded up to whole
 *        groups, pad code 8) and scale fp32 [ceil(K/gs), N]   (w4a8_weights.py:14-20,28-53)
 *   out: w4 u8 [N, Kd/2] with, inside every 32-bit word, nibble 2i = code of
 *        k0+i and nibble 2i+1 = code of k0+4+i (k0 = 8*word index), and
 *        ws fp32 [N, Kd/gs];  Kd = cmi_w4_device_k(K, gs) >= K: K rounded up to whole groups and
 *        whole 128-element steps, the padding holding code 8 and scale 0.
 * gs in {64, 128, 256} (else CMI_E_UNSUPPORTED), any K >= 1.  Plays the role of the load-time
 * repack a backend may do at its own cost (backends/protocol.py:118-126,
 * backends/corex/pack.py:323-359).  The kernels below that take quantised rows (cmi_gemv_w4a8,
 * cmi_gemm_w4a8) are called with K = Kd and rows padded with zeros to Kd; the entries that take bf16
 * rows (cmi_linear_w4a8_bf16*, cmi_embed_rows_w4) take the logical K and do that themselves. */
int cmi_w4_device_k(int K, int gs);  /* 0 when the group size is not one the kernels take */
int cmi_w4_repack(const uint8_t *packed, const float *scale, uint8_t *w4, float *ws,
                  int N, int K, int gs, void *stream);

/* W4A8 GEMV, 1 <= M <= 16 (up to 128 when K <= 10240 and gs == 128), on the re-laid-out weight;
 * K % gs == 0, gs in {64, 128, 256} (the fast kernels are built for 128, the others take a general one):
 *   sum_g = sum_{k in g} xq[m,k]*(code-8)           (int32, exact)
 *   total = fma((float)sum_g, ws[n,g], total)        (g ascending, from 0)
 *   y[m,n] = bf16(total * xs[m])
 * Replaces w4a8_gemv = w4a8_dot + w4a8_finish
 * (backends/corex/kernels/w4a8.cu:56-195, called from
 * backends/corex/__init__.py:649).  group_acc (nullable) receives the int32
 * sums as [M, K/gs, N] for parity checks. */
int cmi_gemv_w4a8(const uint8_t *w4, const float *ws, const int8_t *xq, const float *xs,
                  void *y, int32_t *group_acc, int M, int N, int K, int gs, void *stream);

/* int4 weight-only GEMV on *unquantised* bf16 activations (W4A16), one activation row, on the
 * re-laid-out weight:
 *   y[n] = bf16( sum_g ws[n,g] * sum_{k in g} (code - 8) * x[k] ),  fp32 sums in an order that
 * depends on K only.  K % 128 == 0, gs == 128, K <= 32768 (a wavefront keeps its weight row in
 * registers).  This is what the reference's torch
 * path computes for an int4 weight (backends/reference/__init__.py:93-95 with
 * w4a8_weights.py:96-99: no activation quantisation) up to fp32 summation order, and stands where
 * gemv_kn_w4 is bound (backends/corex/kernels/gemv.cu:1918-1930, 1935-1975). */
int cmi_gemv_w4a16(const uint8_t *w4, const float *ws, const void *x, void *y, int N, int K,
                   int gs, void *stream);

/* cmi_gemv_w4a8 with the activation quantiser folded in, 1 <= M <= 4: x is bf16
 * [M,K]; every workgroup quantises it on the fly with the arithmetic of
 * cmi_quant_act_i8 (same bits), so one launch replaces quant_act_i8 + w4a8_gemv
 * on the decode path (backends/corex/__init__.py:640-649 issues the two).
 * xq_out / xs_out (nullable; xq_out 8-byte aligned) receive the int8 rows and
 * scales the kernel used, for parity checks.  Shapes the fused kernel does not
 * take return CMI_E_UNSUPPORTED: quantise and call cmi_gemv_w4a8 then. */
int cmi_gemv_w4a8_bf16(const uint8_t *w4, const float *ws, const void *x, void *y,
                       int32_t *group_acc, int8_t *xq_out, float *xs_out, int M, int N, int K,
                       int gs, void *stream);

/* W8A8 GEMM with fused epilogue:
 *   acc[m,n] = sum_k xq[m,k]*wq[n,k]  (int32) ; y[m,n] = bf16((float)acc*xs[m]*ws[n])
 * xq int8 [M,K], wq int8 [N,K], y bf16 with row stride ldy >= N.  K % 16 == 0
 * (K % 128 == 0 for the pipelined kernels; other K take a generic one).
 * acc_out (nullable) receives the int32 accumulators as [M,N].
 * Up to 16 rows (K % 128 == 0, K <= 10240) the weight is read once, GEMV style
 * (and once per 128 rows for batches up to 256 rows where that is cheaper than the tile pipeline):
 * the place of w8a8_dp4a_nk on the verify path (backends/corex/__init__.py:450-494).
 * Replaces w8a8_gemm + w8a8_epilogue (backends/corex/kernels/w8a8.cu:195-211,
 * 289-336) and w8a8_gemm_tcu (backends/corex/kernels/w8a8_tcu.cu:276-384),
 * called from backends/corex/__init__.py:1587-1608. */
int cmi_gemm_w8a8(const int8_t *xq, const int8_t *wq, const float *xs, const float *ws,
                  void *y, int32_t *acc_out, int M, int N, int K, int ldy, void *stream);

/* W4A8 GEMM on the re-laid-out weight; same arithmetic as cmi_gemv_w4a8 for
 * any M.  K % 128 == 0 and K % gs == 0, gs in {64, 128, 256} (the tile-count and few-row routes
 * are built for 128; other group sizes take the two-stage tile kernel).  Replaces w4a8_gemm_tcu
 * (backends/corex/kernels/w8a8_tcu.cu:453-574, called from
 * backends/corex/__init__.py:647). group_acc as in cmi_gemv_w4a8. */
int cmi_gemm_w4a8(const uint8_t *w4, const float *ws, const int8_t *xq, const float *xs,
                  void *y, int32_t *group_acc, int M, int N, int K, int gs, void *stream);

/* Whole projections from bf16 activations, one call each: the per-token quantiser into a
 * caller's workspace, then the integer kernels on the quantised rows; same bits as the separate
 * calls.  `workspace` is device memory, 16-byte aligned, of at least
 * cmi_linear_workspace_bytes(M, K) bytes (xq int8 [M,K], then xs fp32 [M], each rounded up to
 * 256 bytes); its contents after the call are the quantised rows and scales the kernels used.
 *   cmi_linear_w8a8_bf16: cmi_quant_act_i8 + cmi_gemm_w8a8 -- what _w8a8_rows issues
 *     (backends/corex/__init__.py:1557-1609: quant_act_i8 into private scratch, then the GEMM).
 *   cmi_linear_w4a8_bf16: what _w4_rows issues (backends/corex/__init__.py:576-651: quant_act_i8
 *     into private scratch, then w4a8_gemv or w4a8_gemm_tcu by row count); the GEMV that
 *     quantises by itself (cmi_gemv_w4a8_bf16) is taken where it is the faster route, the GEMV
 *     entry up to 16 rows, the GEMM entry beyond.  K is the logical row length (any K >= 1, gs in
 *     {64, 128, 256}); the workspace is sized for the padded one,
 *     cmi_linear_workspace_bytes(M, cmi_w4_device_k(K, gs)). */
size_t cmi_linear_workspace_bytes(int M, int K);
/* A workspace of cmi_linear_w8a8_workspace_bytes(M, N, K) bytes -- the above plus, for 17..256 rows,
 * 256 arrival counters and 8 MiB of partial tiles (16 MiB for 257..1024 rows of a projection of at
 * most 128 tiles of 128 x 128 and K >= 2048) -- lets cmi_linear_w8a8_bf16 split K over the idle
 * CUs where a projection is few tiles and many K steps (same bits: the partial sums are
 * integers); with the smaller workspace it does not split.  No counterpart in the reference. */
size_t cmi_linear_w8a8_workspace_bytes(int M, int N, int K);
int cmi_linear_w8a8_bf16(const void *x, const int8_t *wq, const float *ws, void *y, int M, int N,
                         int K, int ldy, void *workspace, size_t workspace_bytes, void *stream);
int cmi_linear_w4a8_bf16(const uint8_t *w4, const float *ws, const void *x, void *y, int M, int N,
                         int K, int gs, void *workspace, size_t workspace_bytes, void *stream);

/* cmi_linear_w4a8_bf16 without the workspace argument, for callers that cannot allocate device
 * memory: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * No counterpart in the reference (its adapters allocate their scratch through torch).  The
 * quantised rows and scales go through a fixed array inside the library -- 8 MiB + 64 KiB per
 * GPU, held until the process ends -- so M <= 16384 and M*K <= 8 MiB (8388608), otherwise
 * CMI_E_UNSUPPORTED and nothing is launched.  The call itself allocates and frees nothing.  All
 * calls on one GPU share that array: calls that overlap on one GPU (different streams or
 * threads) race and must be ordered by the caller.  Same bits as cmi_linear_w4a8_bf16. */
int cmi_linear_w4a8_bf16_static(const uint8_t *w4, const float *ws, const void *x, void *y, int M,
                                int N, int K, int gs, void *stream);

/* silu_mul and silu_mul_quant (backends/protocol.py:265-278; native form
 * backends/corex/kernels/attn.cu:594-641, adapter backends/corex/__init__.py:1038-1071):
 *   out[m,k] = bf16( float(bf16(silu(gate[m,k]))) * float(up[m,k]) ),  silu(g) = g / (1 + exp(-g)) in fp32
 *   out_q, out_s = cmi_quant_act_i8(out)      (absmax over the stored bf16 values: same bits as
 *                                              silu_mul followed by the quantiser)
 * gate, up: bf16 [M,K] with row pitches ld_gate, ld_up (elements; the two halves of a fused
 * gate_up projection have pitch 2K); out: bf16 with row pitch ld_out, may alias `up`, nullable
 * when only the quantised row is wanted; out_q int8 [M,K] dense and out_s fp32 [M], nullable
 * together (then this is silu_mul). */
int cmi_silu_mul_quant(const void *gate, const void *up, void *out, int8_t *out_q, float *out_s,
                       int M, int K, int64_t ld_gate, int64_t ld_up, int64_t ld_out, void *stream);

/* RMSNorm with the gain applied, optionally written as bf16 (y, pitch ld_y, nullable) and / or
 * quantised per row (out_q int8 [M,N] dense + out_s fp32 [M], nullable together); the
 * quantised row equals cmi_quant_act_i8 of the bf16 row bit for bit.  Arithmetic of
 * backends/reference/__init__.py:169-198:
 *   scale = 1 / sqrt(mean_k x^2 + eps)   (the mean correctly rounded to fp32)
 *   y = bf16( float(bf16(x * scale)) * float(w) )          x bf16 [M,N] pitch ld_x, w bf16 [N]
 * Stands where rms_norm_i8 is bound (backends/corex/kernels/norm.cu:310-350). */
int cmi_rms_norm_i8(const void *x, const void *w, void *y, int8_t *out_q, float *out_s, int M,
                    int N, int64_t ld_x, int64_t ld_y, float eps, void *stream);

/* The same after the residual add of backends/reference/__init__.py:224-250:
 * x = bf16(x + add) is written back to x (the residual stream), then normalised as above.
 * Stands where add_rms_norm_i8 is bound (backends/corex/kernels/norm.cu:257-308). */
int cmi_add_rms_norm_i8(void *x, const void *add, const void *w, void *y, int8_t *out_q,
                        float *out_s, int M, int N, int64_t ld_x, int64_t ld_add, int64_t ld_y,
                        float eps, void *stream);

/* Embedding lookup on a quantized weight: rows `ids` (int64 [T]) dequantised to bf16 [T,K].
 *   int8: out[t,k] = bf16(float(wq[id,k]) * ws[id])         (ops/embed.py:64-81, int8_weights.py:359)
 *   int4: out[t,k] = bf16(float(code-8) * ws[id,k/gs])      (w4a8_weights.py:84-94), on the
 *         re-laid-out weight of cmi_w4_repack (any K; gs in {64, 128, 256})
 * An id outside [0, N) gives a row of bf16 NaN (a device-side range error cannot be returned
 * without synchronising). */
int cmi_embed_rows_i8(const int8_t *wq, const float *ws, const int64_t *ids, void *out, int T,
                      int N, int K, void *stream);
int cmi_embed_rows_w4(const uint8_t *w4, const float *ws, const int64_t *ids, void *out, int T,
                      int N, int K, int gs, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* COFFIN_MI355_H */
