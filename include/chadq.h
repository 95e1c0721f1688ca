/*
 * chadq.h — C ABI of libchadq.so: quantized-weight matrix products on MI355X (gfx950).
 *
 * This is the drop-in boundary for one path only: unpacking packed int8/int4 weights
 * with their scales, fused dequantisation, and the GEMV (decode) / GEMM (prefill, MoE
 * expert) products on them.
 *
 * Reference interface replaced: none exists.  The reference snapshot
 * (happycube/chadslab) has no numpy-gemma/ or reclank/ runtime, no op table, no IR
 * interpreter and no FFI layer (its top level is README, ancientARMS/, hsv2.c, kaggle/,
 * m++/, m6502/, notebooks/, nv-fansetup/, ppmproc.cxx, sand/, talks/), so no entry
 * point below can cite a reference file:line.  Each one instead cites the closed form
 * of the benchmark configuration it computes; the Python operator layer in
 * chadslab_amd/ops.py is what a numpy runtime's `x @ dequant(W).T` call sites would
 * bind to.
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer owned by the caller.  The library allocates no
 *    device memory and does no host<->device copies.
 *  - `stream` is a hipStream_t passed as void* (NULL = the null stream).  Launches are
 *    asynchronous on that stream.
 *  - Return value: 0 on success, a negative chadq_status otherwise; the message for
 *    the calling thread's last failure is chadq_last_error().  No C++ exception crosses
 *    this boundary.
 *  - Formats (this build's choices where the configuration text is silent):
 *      int8 per-row : W int8 [N,K] row-major, scale fp32 [N];  w = W[n,k] * scale[n]
 *      int4 group-32: Wp uint8 [N,K/2] row-major, byte j of a row = (u[2j]) | (u[2j+1] << 4),
 *                     u = q + 8 in [0,15]; scale fp16 [N,K/32]; w = (u - 8) * scale[n,k/32]
 *      bf16 / fp16 values travel as uint16_t bit patterns.
 */
#ifndef CHADQ_H
#define CHADQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum chadq_status {
    CHADQ_OK = 0,
    CHADQ_ERR_NULL = -1,      /* a required pointer is NULL */
    CHADQ_ERR_SHAPE = -2,     /* a dimension is non-positive or breaks a divisibility rule */
    CHADQ_ERR_ALIGN = -3,     /* a pointer is not aligned as the entry point requires */
    CHADQ_ERR_WORKSPACE = -4, /* workspace missing or too small */
    CHADQ_ERR_HIP = -5,       /* a HIP call failed; the message names it */
    CHADQ_ERR_DEVICE = -6     /* the current device is not gfx950 */
} chadq_status;

/* Library version, major*10000 + minor*100 + patch. */
int chadq_version(void);

/* Message for the last failure on the calling thread ("" if none). Never NULL. */
const char *chadq_last_error(void);

/* Name of the gfx architecture the kernels were compiled for ("gfx950"). */
const char *chadq_arch(void);

/* ---- unpack / dequantise (parity and tooling entry points) -------------------------- */

/* nbytes packed bytes -> 2*nbytes int8 values in [-8,7] (low nibble first). Bit-exact. */
int chadq_unpack_i4(const uint8_t *wp, int8_t *q, int64_t nbytes, void *stream);

/* 2*nbytes int8 values in [-8,7] -> nbytes packed bytes; inverse of chadq_unpack_i4. */
int chadq_pack_i4(const int8_t *q, uint8_t *wp, int64_t nbytes, void *stream);

/* w[n,k] = (u[n,k]-8) * float(scale[n,k/32]) as fp32 [N,K]; exact (no rounding occurs). K%32==0. */
int chadq_dequant_i4g32(const uint8_t *wp, const uint16_t *scale_f16, float *w, int N, int K, void *stream);

/* w[n,k] = W[n,k] * scale[n] as fp32 [N,K]. */
int chadq_dequant_i8row(const int8_t *w8, const float *scale, float *w, int N, int K, void *stream);

/* ---- decode GEMV (benchmark configs 0 and 1) ----------------------------------------- */

/*
 * y[m,n] = sum_g float(scale[n,g]) * sum_{k in g} x[m,k] * (u[n,k]-8)      (config 1)
 * x bf16 [M,K], y fp32 [M,N], 1 <= M <= 16, K % 32 == 0.  wp and x 16-byte aligned.
 * HBM-bound: each packed weight byte and each scale is read once for all M <= 16 activation rows (the matrix-core
 * kernels; the fallback for K % 256 != 0 or unaligned scales reads them once per pair of rows).
 */
int chadq_gemv_i4g32(const uint16_t *x_bf16, const uint8_t *wp, const uint16_t *scale_f16, float *y, int M, int N,
                     int K, void *stream);

/*
 * Split-K form of the M = 1 product for matrices with few rows and long K (a down projection): y_parts fp32
 * [ksplit, N], part s = the sum over k in [s*K/ksplit, (s+1)*K/ksplit); the caller adds the parts
 * (chadq_add_rmsnorm_bf16 does).  K % (ksplit*4096) == 0; x, wp and scale 16-byte aligned.
 */
int chadq_gemv_i4g32_splitk(const uint16_t *x_bf16, const uint8_t *wp, const uint16_t *scale_f16, float *y_parts, int N,
                            int K, int ksplit, void *stream);

/*
 * chadq_gemv_i4g32_splitk with the GeGLU of a gated FFN folded in: the activation is formed inside the kernel as
 * x[k] = bf16( gelu_tanh(gu[k]) * gu[K + k] ) from gu fp32 [2K] (what chadq_geglu_bf16 would write).  gu 16-byte aligned.
 */
int chadq_gemv_i4g32_splitk_geglu(const float *gu, const uint8_t *wp, const uint16_t *scale_f16, float *y_parts, int N, int K,
                                  int ksplit, void *stream);

/*
 * chadq_add_rmsnorm_bf16 folded into the M = 1 product that consumes it: r = res + delta[0] + ... + delta[n_delta-1]
 * (fp32, in order; delta fp32 [n_delta, K], n_delta <= 4), x = bf16( r / sqrt(mean(r^2) + eps) * norm_w ),
 * y[n] = the int4 group-32 product of x with row n; r is written to res_out, which must be a different buffer
 * than res (other workgroups still read res while the first one writes).  K a multiple of 256, K <= 2048;
 * every array 16-byte aligned.
 */
int chadq_gemv_i4g32_addnorm(const float *res, const float *delta, int n_delta, const float *norm_w, float eps, float *res_out,
                             const uint8_t *wp, const uint16_t *scale_f16, float *y, int N, int K, void *stream);

/*
 * chadq_gemv_i4g32_addnorm for the gate/up projection of a GeGLU FFN whose matrix holds the two rows of a feature next
 * to each other (row 2i = gate of feature i, row 2i+1 = up): instead of the N sums the kernel writes
 * h[i] = bf16( gelu_tanh(y[2i]) * y[2i+1] ), N/2 values - what chadq_geglu_bf16 would make of them - so that the
 * down projection reads a bf16 vector and no fp32 gate/up vector is written.  N even; otherwise as above.
 */
int chadq_gemv_i4g32_addnorm_geglu(const float *res, const float *delta, int n_delta, const float *norm_w, float eps,
                                   float *res_out, const uint8_t *wp, const uint16_t *scale_f16, uint16_t *h_bf16, int N, int K,
                                   void *stream);

/*
 * y[m,n] = scale[n] * sum_k x[m,k] * W[n,k]                                 (config 0)
 * x fp32 [M,K], W int8 [N,K], scale fp32 [N], y fp32 [M,N], 1 <= M <= 16, K % 16 == 0.
 * K % 128 == 0: the weights are read once for all M rows, on the int8 matrix core; per activation row and block of
 * 2048 k the activations are held in fixed point (three 8-bit digits, a power-of-two scale from the block's largest
 * |x|), the integer sums are exact.  Bound: |y[m,n] - exact| <= |scale[n]| * sum over blocks b of
 * 2^-21 * max_{k in b}|x[m,k]| * sum_{k in b}|W[n,k]| (+ the fp32 rounding of the block sums).  For activations of one
 * order of magnitude that is 1e-6 relative; ONE outlier in a block costs the block's small elements their low bits,
 * also in output rows whose weight at the outlier is zero - call chadq_gemv_i8row_fp32 where that matters.  Integer
 * activations below 2^20 whose sums stay below 2^24 give exact results; a non-finite activation makes its row NaN;
 * a row's result does not depend on M.  Other K: fp32 arithmetic as in chadq_gemv_i8row_fp32.
 */
int chadq_gemv_i8row(const float *x, const int8_t *w8, const float *scale, float *y, int M, int N, int K,
                     void *stream);

/*
 * The same product with fp32 arithmetic on every element, whatever K: x[m,k] * float(W[n,k]) accumulated in fp32, the
 * row scale applied to the sum; the weights are streamed once per pair of activation rows (M = 1, 2: the speed of
 * chadq_gemv_i8row within a few per cent; M = 8: four passes).  Same argument rules.  An activation's error does not
 * depend on its neighbours; non-finite activations behave as IEEE arithmetic has them (inf * W is an infinity, inf * 0 a NaN).
 */
int chadq_gemv_i8row_fp32(const float *x, const int8_t *w8, const float *scale, float *y, int M, int N, int K,
                          void *stream);

/* ---- prefill dequant-GEMM (benchmark config 2) ---------------------------------------- */

/*
 * y[m,n] = bf16_rne( sum_k x[m,k] * w[n,k] ), w as in chadq_dequant_i4g32 rounded to bf16
 * for the MFMA, fp32 accumulate.  x bf16 [M,K], y bf16 [M,N].  K % 32 == 0, any M >= 1.
 */
int chadq_gemm_i4g32_bf16(const uint16_t *x_bf16, const uint8_t *wp, const uint16_t *scale_f16, uint16_t *y_bf16,
                          int M, int N, int K, void *stream);

/* Same with int8 weights and one fp32 scale per output row (scale applied in fp32 after the MFMA). */
int chadq_gemm_i8row_bf16(const uint16_t *x_bf16, const int8_t *w8, const float *scale, uint16_t *y_bf16, int M,
                          int N, int K, void *stream);

/* ---- mixture-of-experts FFN (benchmark config 3) ---------------------------------------- */

/*
 * softmax over E experts per token, then the top_k experts by logit (lowest index wins ties).
 * idx int32 [T,top_k], w fp32 [T,top_k] = their probabilities, divided by their sum if renorm != 0.
 * E <= 16, top_k <= min(E, 8).
 */
int chadq_moe_route(const float *logits, int32_t *idx, float *w, int T, int E, int top_k, int renorm, void *stream);

/* Device pointers of one expert's int4 group-32 weights: gate and up are [F,H], down is [H,F]. */
typedef struct chadq_moe_expert_i4g32 {
    const uint8_t *wg;
    const uint16_t *sg;
    const uint8_t *wu;
    const uint16_t *su;
    const uint8_t *wd;
    const uint16_t *sd;
} chadq_moe_expert_i4g32;

/* Bytes of device workspace chadq_moe_ffn_i4g32 needs for these sizes (0 if the sizes are invalid). */
size_t chadq_moe_ffn_i4g32_workspace_bytes(int T, int H, int F, int E, int top_k);

/*
 * y[t] = bf16( sum_j w[t,j] * Wd_e ( bf16( silu(Wg_e x_t) * (Wu_e x_t) ) ) ),  e = idx[t,j] from chadq_moe_route.
 * x bf16 [T,H], logits fp32 [T,E], y bf16 [T,H].  `experts` is a HOST array of E structs holding device pointers.
 * H % 32 == 0, F % 32 == 0.  Runs entirely on `stream`; no host synchronisation, nothing allocated.
 */
int chadq_moe_ffn_i4g32(const uint16_t *x_bf16, const float *logits, const chadq_moe_expert_i4g32 *experts,
                        uint16_t *y_bf16, int T, int H, int F, int E, int top_k, int renorm, void *workspace,
                        size_t workspace_bytes, void *stream);

/*
 * Tile order of int4 group-32 weights: a load-time repack for the experts of chadq_moe_ffn_i4g32_tiled.  The row-major
 * container (wp [N,K/2], scale [N,K/32]) stays the interchange format; the tiled arrays have the same sizes.
 *   packed: unit (b = n/32, c = k/256) is 4096 contiguous bytes at ((b*(K/256)) + c) * 4096; inside it the 16-byte
 *           piece (one scale group) of row r = n%32 and group g = (k%256)/32 sits at (g*32 + r) * 16.
 *   scales: block (b, c) is 512 contiguous bytes at ((b*(K/256)) + c) * 512; the scale of row r and group g sits at
 *           ((g%2)*32 + r) * 8 + (g/2) * 2.
 * N % 32 == 0, K % 256 == 0, all arrays 16-byte aligned, input and output distinct.  unrepack is the exact inverse.
 * No reference counterpart (the snapshot has no quantized containers): a layout of this build, in FORMAT.md.
 */
int chadq_repack_i4g32_tiles(const uint8_t *wp, const uint16_t *scale_f16, uint8_t *wp_tiles, uint16_t *scale_tiles, int N, int K,
                             void *stream);
int chadq_unrepack_i4g32_tiles(const uint8_t *wp_tiles, const uint16_t *scale_tiles, uint8_t *wp, uint16_t *scale_f16, int N, int K,
                               void *stream);

/*
 * chadq_moe_ffn_i4g32 on experts whose six arrays are in tile order: same arguments, same workspace.  Each load of the
 * expert kernel then reads 1 KiB of consecutive memory straight into registers, and the arithmetic is fp16 instead of
 * bf16: activations (and the gated intermediate h, after its bf16 rounding) are scaled per row by a power of two into
 * fp16's range - exact for bf16 inputs of any magnitude, the factor is undone on the fp32 result - and a weight enters
 * the matrix core as fp16(u * scale), the zero point as a separate exact term per scale group.  The results agree with
 * chadq_moe_ffn_i4g32 within rounding (they are the closer of the two to a float64 evaluation: fp16 keeps 3 more bits
 * of the dequantised weight than bf16), not bit for bit.  About 20 % faster at 256 tokens x 8 experts of 14336 x 4096.
 * H % 256 == 0 and F % 256 == 0; scales must be below 64 in magnitude (1024 * scale has to be a finite fp16);
 * T * top_k * max(H, F) < 2^30.
 */
int chadq_moe_ffn_i4g32_tiled(const uint16_t *x_bf16, const float *logits, const chadq_moe_expert_i4g32 *experts,
                              uint16_t *y_bf16, int T, int H, int F, int E, int top_k, int renorm, void *workspace,
                              size_t workspace_bytes, void *stream);

/* ---- decode-step pieces around the GEMVs (benchmark config 4), batch 1 ------------------- */
/* The position and the current token live in device memory so that one captured HIP graph serves every step.
 * The kernels clamp pos[0] to [0, max_ctx-1] and token[0] to [0, V-1] so that nothing is addressed out of bounds, and
 * report nothing when they do: a step past the end of the cache overwrites its last row and rotates by the wrong
 * angle.  Keeping pos + steps <= max_ctx is the caller's job (QuantDecoder.feed / generate check it on the host). */

/* x[d] fp32 = dequantised row token[0] (clamped to [0,V-1]) of the tied int4 group-32 table [V,d]. */
int chadq_embed_i4g32(const int32_t *token, const uint8_t *wp, const uint16_t *scale_f16, float *x, int d, int V,
                      void *stream);

/*
 * res[d] += delta[0][d] + ... + delta[n_delta-1][d] (delta fp32 [n_delta, d]; nothing is added or written if delta is
 * NULL or n_delta is 0); y[d] = bf16( res / sqrt(mean(res^2) + eps) * w ).
 */
int chadq_add_rmsnorm_bf16(float *res, const float *delta, int n_delta, const float *w, uint16_t *y_bf16, int d, float eps,
                           void *stream);

/*
 * qkv fp32 = [hq*dh | dh | dh].  Rotate-half RoPE (given base) at position pos[0] on q and k; q_out fp32 [hq*dh];
 * row pos[0] of the bf16 caches kcache/vcache [max_ctx,dh] receives k and v.  pos[0] is clamped to [0,max_ctx-1]
 * here and in chadq_attn_decode_mqa, so a runaway position cannot address outside the cache.
 */
int chadq_rope_kv_write(const float *qkv, const int32_t *pos, float *q_out, uint16_t *kcache_bf16,
                        uint16_t *vcache_bf16, int hq, int dh, int max_ctx, float base, void *stream);

/* Floats of workspace chadq_attn_decode_mqa needs for a cache of max_ctx rows. */
size_t chadq_attn_decode_mqa_workspace_floats(int hq, int dh, int max_ctx);

/*
 * Multi-query decode attention over cache rows 0..pos[0]: out bf16 [hq*dh] = softmax(q k^T / sqrt(dh)) v per head,
 * all heads sharing one K/V.  hq <= 8, dh <= 256 and a multiple of 8, max_ctx <= 65536; q and kcache 16-byte aligned.
 */
int chadq_attn_decode_mqa(const float *q, const uint16_t *kcache_bf16, const uint16_t *vcache_bf16, const int32_t *pos,
                          float *workspace, uint16_t *out_bf16, int hq, int dh, int max_ctx, void *stream);

/* table fp32 [max_ctx, dh/2, 2] = (cos, sin) of p * base^(-2j/dh): the rotation angles chadq_rope_kv_write computes. */
int chadq_rope_table(float *table, int dh, int max_ctx, float base, void *stream);

/* Floats of workspace chadq_attn_decode_mqa_fused needs. */
size_t chadq_attn_decode_mqa_fused_workspace_floats(int hq, int dh, int max_ctx);

/*
 * chadq_rope_kv_write and chadq_attn_decode_mqa with the rotation and the cache write folded into the attention
 * kernel: rotates q and k of qkv (angles from rope_table), writes row pos[0] of both caches, attends over rows
 * 0..pos[0] and writes out bf16 [hq*dh].  qkv fp32 = [hq*dh | dh | dh].
 * hq <= 8, dh <= 256 and a multiple of 16, max_ctx <= 65536; qkv, rope_table and kcache 16-byte aligned.
 * Both caches must be readable over all max_ctx rows: for hq = 8, dh = 256 and max_ctx <= 8192 the kernel asks for its
 * rows before it has read pos[0], clamped to the cache only; rows behind pos[0] never reach a result (whatever they
 * hold, NaN included) and are never written.
 */
int chadq_attn_decode_mqa_fused(const float *qkv, const int32_t *pos, const float *rope_table, uint16_t *kcache_bf16,
                                uint16_t *vcache_bf16, float *workspace, uint16_t *out_bf16, int hq, int dh, int max_ctx,
                                void *stream);

/*
 * chadq_attn_decode_mqa_fused followed by the output projection that consumes its result, y = Wo * out with Wo an int4
 * group-32 matrix [N, hq*dh] (wp / scale_f16 as for chadq_gemv_i4g32), in two launches instead of three: the
 * combination of the split-context partials happens inside the projection.  The projection is split over K by pairs
 * of heads: y_parts fp32 [hq/2, N] receives one partial vector per pair and the caller (or the n_delta argument of
 * chadq_gemv_i4g32_addnorm / _addnorm_geglu / chadq_add_rmsnorm_bf16) adds them, in order.  The attention vector itself
 * is rounded to bf16 as chadq_attn_decode_mqa_fused rounds it, but is not written anywhere.
 * y_parts must be ordinary device memory (hipMalloc): the first kernel clears it, and in the second the two heads of a
 * pair add their products into it with hardware float atomics - two addends on a cleared value, so the result is the
 * same bits whichever arrives first.
 * dh = 256 and hq in {2, 4, 6, 8} (CHADQ_ERR_SHAPE otherwise: use the two separate calls), max_ctx <= 65536, N >= 1;
 * qkv, rope_table, kcache, workspace and wp 16-byte aligned.  Workspace as chadq_attn_decode_mqa_fused_workspace_floats.
 * The reference has no counterpart: its numpy runtime would call the attention and the projection one after the other.
 */
int chadq_attn_decode_mqa_fused_oproj_i4g32(const float *qkv, const int32_t *pos, const float *rope_table, uint16_t *kcache_bf16,
                                            uint16_t *vcache_bf16, float *workspace, const uint8_t *wp,
                                            const uint16_t *scale_f16, float *y_parts, int hq, int dh, int max_ctx, int N,
                                            void *stream);

/*
 * chadq_attn_decode_mqa_fused for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments minus the
 * workspace, same kernels, same results bit for bit: the split-context partials live in a 2,113,536-byte array inside
 * the library's device code (one per GPU, held until the process ends), which covers max_ctx <= 8192 at hq <= 8,
 * dh <= 256; a larger max_ctx returns CHADQ_ERR_WORKSPACE.  Calls no hipMalloc / hipFree.  The array's address on a
 * device is looked up (hipGetSymbolAddress) by the first call of ANY entry point of this library on that device, which
 * therefore has to happen outside a stream capture (a repack, a warm-up step, chadq_rope_table all do); this entry
 * point itself only reads the stored address.  Every call on a GPU shares that GPU's array: one call at a time per
 * GPU - calls that overlap on one GPU (two streams, or two graphs replayed concurrently) race on it silently.
 */
int chadq_attn_decode_mqa_fused_static(const float *qkv, const int32_t *pos, const float *rope_table, uint16_t *kcache_bf16,
                                       uint16_t *vcache_bf16, uint16_t *out_bf16, int hq, int dh, int max_ctx, void *stream);

/* h[F] = bf16( gelu_tanh(gu[i]) * gu[F+i] ). */
int chadq_geglu_bf16(const float *gu, uint16_t *h_bf16, int F, void *stream);

/*
 * token[0] = argmax of v[0..n) (lowest index wins ties; NaN never wins; 0 if every value is NaN); pos[0] += 1 if
 * advance != 0.
 * scratch: 256 floats followed by 256 int32 (2048 bytes).
 */
int chadq_argmax_f32(const float *v, int n, void *scratch, int32_t *token, int32_t *pos, int advance, void *stream);

/*
 * A greedy decoder's last two calls and the next step's first in two launches: y = W x as chadq_gemv_i4g32 with M = 1
 * (W the int4 group-32 output table [N, K]), token[0] = argmax of y by the rules of chadq_argmax_f32, pos[0] += 1 if
 * advance != 0, and - next_x != NULL - next_x fp32 [K] = row token[0] of the same table, as chadq_embed_i4g32 would
 * write it (tied input and output embeddings: the vector the next step starts from).
 * For N >= 8192, K <= 2048 and a multiple of 256, N*K/2 < 2^31 and 16-byte aligned scales, every workgroup of the GEMV
 * leaves the largest of its 64 sums beside y and the second launch reads those candidates, not y; other shapes run the
 * separate kernels (same results).  scratch: chadq_gemv_i4g32_argmax_scratch_bytes(N, K) bytes.
 * x and wp 16-byte aligned.  The reference has no counterpart: its numpy runtime would call the
 * three operations one after the other.
 */
size_t chadq_gemv_i4g32_argmax_scratch_bytes(int N, int K);
int chadq_gemv_i4g32_argmax(const uint16_t *x_bf16, const uint8_t *wp, const uint16_t *scale_f16, float *y, int N, int K,
                            void *scratch, int32_t *token, int32_t *pos, int advance, float *next_x, void *stream);

/*
 * Top-k sampling.  Candidates: the k largest of v[0..n), larger first, lower index first among equals (NaN is never
 * a candidate).  p_j = exp((v_j - v_0) / temperature) in that order; token[0] = the first candidate whose running
 * sum of p exceeds u[0] * (sum of p), u[0] in [0, 1) read from device memory at run time (so a captured graph draws
 * afresh on every replay once the caller has rewritten it).  k = 1 is argmax.  pos[0] += 1 if advance != 0.
 * 1 <= k <= min(64, n), n <= 786432, temperature > 0.  workspace: 49152 bytes.
 */
int chadq_sample_topk_f32(const float *v, int n, int k, float temperature, const float *u, void *workspace, int32_t *token,
                          int32_t *pos, int advance, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* CHADQ_H */
