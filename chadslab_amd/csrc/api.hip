// extern "C" surface of libchadq.so: argument checks, error messages, dispatch.  No allocation, no copies.
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "chadq_common.h"

namespace chadq {

static thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

void clear_error() { g_err[0] = '\0'; }

int hip_check(hipError_t e, const char *what) {
    if (e == hipSuccess) return 0;
    return fail(CHADQ_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

int attn_mqa_fused_static_init(int dev);

int check_device() {
    static int ok_mask[64] = {0};  // 0 unknown, 1 ok, -1 wrong arch; benign race: idempotent values
    int dev = 0;
    CHADQ_HIP(hipGetDevice(&dev));
    if (dev >= 0 && dev < 64 && ok_mask[dev] == 1) return 0;
    hipDeviceProp_t prop;
    CHADQ_HIP(hipGetDeviceProperties(&prop, dev));
    const bool ok = strncmp(prop.gcnArchName, "gfx950", 6) == 0;
    if (!ok) {
        if (dev >= 0 && dev < 64) ok_mask[dev] = -1;
        return fail(CHADQ_ERR_DEVICE, "device %d is %s; libchadq is built for gfx950 only", dev, prop.gcnArchName);
    }
    // first entry-point call on this device: look up the address of the attention scratch array now, so that
    // chadq_attn_decode_mqa_fused_static itself never has to (it may be called under graph capture, where the lookup
    // is not allowed)
    int rc = attn_mqa_fused_static_init(dev);
    if (rc != 0) return rc;
    if (dev >= 0 && dev < 64) ok_mask[dev] = 1;
    return 0;
}

// kernels' launch functions (one per source file)
int unpack_i4_launch(const uint8_t *, int8_t *, int64_t, hipStream_t);
int pack_i4_launch(const int8_t *, uint8_t *, int64_t, hipStream_t);
int dequant_i4g32_launch(const uint8_t *, const uint16_t *, float *, int, int, hipStream_t);
int dequant_i8row_launch(const int8_t *, const float *, float *, int, int, hipStream_t);
int gemv_i4g32_dispatch(const uint16_t *, const uint8_t *, const uint16_t *, float *, int, int, int, hipStream_t);
int gemv_i4g32_mfma_dispatch(const uint16_t *, const uint8_t *, const uint16_t *, float *, int, int, int, hipStream_t);
int gemv_i8row_dispatch(const float *, const int8_t *, const float *, float *, int, int, int, bool, hipStream_t);
int gemm_i4g32_bf16_dispatch(const uint16_t *, const uint8_t *, const uint16_t *, uint16_t *, int, int, int,
                             hipStream_t);
int gemm_i8row_bf16_dispatch(const uint16_t *, const int8_t *, const float *, uint16_t *, int, int, int,
                             hipStream_t);

size_t moe_workspace_bytes(int, int, int, int, int);
int moe_route_launch(const float *, int32_t *, float *, int, int, int, int, hipStream_t);
int moe_ffn_i4g32_launch(const uint16_t *, const float *, const chadq_moe_expert_i4g32 *, uint16_t *, int, int, int, int, int,
                         int, void *, bool, hipStream_t);
bool moe_ffn_tiled_ok(int, int);
int repack_i4g32_tiles_launch(const uint8_t *, const uint16_t *, uint8_t *, uint16_t *, int, int, bool, hipStream_t);

int embed_launch(const int32_t *, const uint8_t *, const uint16_t *, float *, int, int, hipStream_t);
int add_rmsnorm_launch(float *, const float *, int, const float *, uint16_t *, int, float, hipStream_t);
int gemv_i4g32_splitk_launch(const uint16_t *, const uint8_t *, const uint16_t *, float *, int, int, int, hipStream_t);
int gemv_i4g32_splitk_geglu_launch(const float *, const uint8_t *, const uint16_t *, float *, int, int, int, hipStream_t);
int gemv_i4g32_addnorm_launch(const float *, const float *, int, const float *, float, float *, const uint8_t *, const uint16_t *,
                              float *, int, int, hipStream_t);
int gemv_i4g32_addnorm_geglu_launch(const float *, const float *, int, const float *, float, float *, const uint8_t *, const uint16_t *,
                                    uint16_t *, int, int, hipStream_t);
int rope_kv_launch(const float *, const int32_t *, float *, uint16_t *, uint16_t *, int, int, int, float, hipStream_t);
int attn_mqa_launch(const float *, const uint16_t *, const uint16_t *, const int32_t *, float *, uint16_t *, int, int, int,
                    hipStream_t);
int geglu_launch(const float *, uint16_t *, int, hipStream_t);
int rope_table_launch(float *, int, int, float, hipStream_t);
int attn_mqa_fused_launch(const float *, const int32_t *, const float *, uint16_t *, uint16_t *, float *, uint16_t *, int, int, int,
                          hipStream_t);
bool attn_mqa_fused_oproj_ok(int hq, int dh);
int attn_mqa_fused_oproj_launch(const float *, const int32_t *, const float *, uint16_t *, uint16_t *, float *, const uint8_t *,
                                const uint16_t *, float *, int, int, int, int, hipStream_t);
int attn_mqa_fused_static_launch(const float *, const int32_t *, const float *, uint16_t *, uint16_t *, uint16_t *, int, int, int,
                                 hipStream_t);
int attn_mqa_fused_static_max_ctx();
int argmax_launch(const float *, int, float *, int32_t *, int32_t *, int32_t *, int, hipStream_t);
int argmax_embed_launch(const float *, bool, float *, int32_t *, int, int, int32_t *, int32_t *, int, const uint8_t *, const uint16_t *,
                        float *, int, hipStream_t);
bool gemv_i4g32_argmax_ok(const uint16_t *, int, int);
int gemv_i4g32_argmax_launch(const uint16_t *, const uint8_t *, const uint16_t *, float *, int, int, float *, int32_t *, int *,
                             hipStream_t);
int sample_topk_launch(const float *, int, int, float, const float *, float *, int32_t *, int32_t *, int32_t *, int, hipStream_t);

}  // namespace chadq

using namespace chadq;

#define ENTER()                     \
    clear_error();                  \
    {                               \
        int _d = check_device();    \
        if (_d != 0) return _d;     \
    }                               \
    hipStream_t st = (hipStream_t)stream

extern "C" {

int chadq_version(void) { return 100; }

const char *chadq_last_error(void) { return g_err; }

const char *chadq_arch(void) { return "gfx950"; }

int chadq_unpack_i4(const uint8_t *wp, int8_t *q, int64_t nbytes, void *stream) {
    ENTER();
    CHADQ_REQUIRE(nbytes >= 0, CHADQ_ERR_SHAPE, "chadq_unpack_i4: nbytes=%lld is negative", (long long)nbytes);
    if (nbytes == 0) return 0;
    CHADQ_REQUIRE(wp && q, CHADQ_ERR_NULL, "chadq_unpack_i4: null pointer");
    return unpack_i4_launch(wp, q, nbytes, st);
}

int chadq_pack_i4(const int8_t *q, uint8_t *wp, int64_t nbytes, void *stream) {
    ENTER();
    CHADQ_REQUIRE(nbytes >= 0, CHADQ_ERR_SHAPE, "chadq_pack_i4: nbytes=%lld is negative", (long long)nbytes);
    if (nbytes == 0) return 0;
    CHADQ_REQUIRE(wp && q, CHADQ_ERR_NULL, "chadq_pack_i4: null pointer");
    return pack_i4_launch(q, wp, nbytes, st);
}

int chadq_dequant_i4g32(const uint8_t *wp, const uint16_t *scale_f16, float *w, int N, int K, void *stream) {
    ENTER();
    CHADQ_REQUIRE(N >= 0 && K >= 0 && K % 32 == 0, CHADQ_ERR_SHAPE, "chadq_dequant_i4g32: N=%d K=%d (K %% 32 != 0?)", N, K);
    if (N == 0 || K == 0) return 0;
    CHADQ_REQUIRE(wp && scale_f16 && w, CHADQ_ERR_NULL, "chadq_dequant_i4g32: null pointer");
    CHADQ_REQUIRE(aligned16(wp) && aligned16(w), CHADQ_ERR_ALIGN, "chadq_dequant_i4g32: wp and w must be 16-byte aligned");
    return dequant_i4g32_launch(wp, scale_f16, w, N, K, st);
}

int chadq_dequant_i8row(const int8_t *w8, const float *scale, float *w, int N, int K, void *stream) {
    ENTER();
    CHADQ_REQUIRE(N >= 0 && K >= 0, CHADQ_ERR_SHAPE, "chadq_dequant_i8row: N=%d K=%d", N, K);
    if (N == 0 || K == 0) return 0;
    CHADQ_REQUIRE(w8 && scale && w, CHADQ_ERR_NULL, "chadq_dequant_i8row: null pointer");
    return dequant_i8row_launch(w8, scale, w, N, K, st);
}

int chadq_gemv_i4g32(const uint16_t *x_bf16, const uint8_t *wp, const uint16_t *scale_f16, float *y, int M, int N,
                     int K, void *stream) {
    ENTER();
    CHADQ_REQUIRE(M >= 1 && M <= 16, CHADQ_ERR_SHAPE, "chadq_gemv_i4g32: M=%d outside [1,16] (use chadq_gemm_i4g32_bf16)", M);
    CHADQ_REQUIRE(N >= 0 && K >= 32 && K % 32 == 0, CHADQ_ERR_SHAPE, "chadq_gemv_i4g32: N=%d K=%d (K must be a positive multiple of 32)", N, K);
    if (N == 0) return 0;
    CHADQ_REQUIRE(x_bf16 && wp && scale_f16 && y, CHADQ_ERR_NULL, "chadq_gemv_i4g32: null pointer");
    CHADQ_REQUIRE(aligned16(x_bf16) && aligned16(wp), CHADQ_ERR_ALIGN, "chadq_gemv_i4g32: x and wp must be 16-byte aligned");
    return gemv_i4g32_mfma_dispatch(x_bf16, wp, scale_f16, y, M, N, K, st);
}

int chadq_gemv_i4g32_splitk(const uint16_t *x_bf16, const uint8_t *wp, const uint16_t *scale_f16, float *y_parts, int N,
                            int K, int ksplit, void *stream) {
    ENTER();
    CHADQ_REQUIRE(N >= 1 && K >= 4096 && ksplit >= 1 && ksplit <= 64 && K % (ksplit * 4096) == 0, CHADQ_ERR_SHAPE,
                  "chadq_gemv_i4g32_splitk: N=%d K=%d ksplit=%d (K must be a multiple of ksplit*4096)", N, K, ksplit);
    CHADQ_REQUIRE((int64_t)N * (K / 2) < ((int64_t)1 << 31), CHADQ_ERR_SHAPE,
                  "chadq_gemv_i4g32_splitk: N*K/2 = %lld bytes exceeds 2^31", (long long)N * (K / 2));
    CHADQ_REQUIRE(x_bf16 && wp && scale_f16 && y_parts, CHADQ_ERR_NULL, "chadq_gemv_i4g32_splitk: null pointer");
    CHADQ_REQUIRE(aligned16(x_bf16) && aligned16(wp) && aligned16(scale_f16), CHADQ_ERR_ALIGN,
                  "chadq_gemv_i4g32_splitk: x, wp and scale must be 16-byte aligned");
    return gemv_i4g32_splitk_launch(x_bf16, wp, scale_f16, y_parts, N, K, ksplit, st);
}

int chadq_gemv_i4g32_splitk_geglu(const float *gu, const uint8_t *wp, const uint16_t *scale_f16, float *y_parts, int N, int K,
                                  int ksplit, void *stream) {
    ENTER();
    CHADQ_REQUIRE(N >= 1 && K >= 4096 && ksplit >= 1 && ksplit <= 64 && K % (ksplit * 4096) == 0, CHADQ_ERR_SHAPE,
                  "chadq_gemv_i4g32_splitk_geglu: N=%d K=%d ksplit=%d (K must be a multiple of ksplit*4096)", N, K, ksplit);
    CHADQ_REQUIRE((int64_t)N * (K / 2) < ((int64_t)1 << 31), CHADQ_ERR_SHAPE,
                  "chadq_gemv_i4g32_splitk_geglu: N*K/2 = %lld bytes exceeds 2^31", (long long)N * (K / 2));
    CHADQ_REQUIRE(gu && wp && scale_f16 && y_parts, CHADQ_ERR_NULL, "chadq_gemv_i4g32_splitk_geglu: null pointer");
    CHADQ_REQUIRE(aligned16(gu) && aligned16(wp) && aligned16(scale_f16), CHADQ_ERR_ALIGN,
                  "chadq_gemv_i4g32_splitk_geglu: gu, wp and scale must be 16-byte aligned");
    return gemv_i4g32_splitk_geglu_launch(gu, wp, scale_f16, y_parts, N, K, ksplit, st);
}

int chadq_gemv_i4g32_addnorm(const float *res, const float *delta, int n_delta, const float *norm_w, float eps, float *res_out,
                             const uint8_t *wp, const uint16_t *scale_f16, float *y, int N, int K, void *stream) {
    ENTER();
    CHADQ_REQUIRE(N >= 1 && K >= 256 && K <= 2048 && K % 256 == 0 && n_delta >= 0 && n_delta <= 4, CHADQ_ERR_SHAPE,
                  "chadq_gemv_i4g32_addnorm: N=%d K=%d n_delta=%d (K a multiple of 256 up to 2048, n_delta <= 4)", N, K, n_delta);
    CHADQ_REQUIRE((int64_t)N * (K / 2) < ((int64_t)1 << 31), CHADQ_ERR_SHAPE,
                  "chadq_gemv_i4g32_addnorm: N*K/2 = %lld bytes exceeds 2^31", (long long)N * (K / 2));
    CHADQ_REQUIRE(res && norm_w && res_out && wp && scale_f16 && y && (delta || n_delta == 0), CHADQ_ERR_NULL,
                  "chadq_gemv_i4g32_addnorm: null pointer");
    CHADQ_REQUIRE(res != res_out, CHADQ_ERR_SHAPE, "chadq_gemv_i4g32_addnorm: res_out must not be res");
    CHADQ_REQUIRE(aligned16(res) && aligned16(delta) && aligned16(norm_w) && aligned16(res_out) && aligned16(wp) &&
                      aligned16(scale_f16),
                  CHADQ_ERR_ALIGN, "chadq_gemv_i4g32_addnorm: every array must be 16-byte aligned");
    return gemv_i4g32_addnorm_launch(res, delta, delta ? n_delta : 0, norm_w, eps, res_out, wp, scale_f16, y, N, K, st);
}

int chadq_gemv_i4g32_addnorm_geglu(const float *res, const float *delta, int n_delta, const float *norm_w, float eps,
                                   float *res_out, const uint8_t *wp, const uint16_t *scale_f16, uint16_t *h_bf16, int N, int K,
                                   void *stream) {
    ENTER();
    CHADQ_REQUIRE(N >= 2 && N % 2 == 0 && K >= 256 && K <= 2048 && K % 256 == 0 && n_delta >= 0 && n_delta <= 4, CHADQ_ERR_SHAPE,
                  "chadq_gemv_i4g32_addnorm_geglu: N=%d K=%d n_delta=%d (N even, K a multiple of 256 up to 2048, n_delta <= 4)", N, K,
                  n_delta);
    CHADQ_REQUIRE((int64_t)N * (K / 2) < ((int64_t)1 << 31), CHADQ_ERR_SHAPE,
                  "chadq_gemv_i4g32_addnorm_geglu: N*K/2 = %lld bytes exceeds 2^31", (long long)N * (K / 2));
    CHADQ_REQUIRE(res && norm_w && res_out && wp && scale_f16 && h_bf16 && (delta || n_delta == 0), CHADQ_ERR_NULL,
                  "chadq_gemv_i4g32_addnorm_geglu: null pointer");
    CHADQ_REQUIRE(res != res_out, CHADQ_ERR_SHAPE, "chadq_gemv_i4g32_addnorm_geglu: res_out must not be res");
    CHADQ_REQUIRE(aligned16(res) && aligned16(delta) && aligned16(norm_w) && aligned16(res_out) && aligned16(wp) &&
                      aligned16(scale_f16),
                  CHADQ_ERR_ALIGN, "chadq_gemv_i4g32_addnorm_geglu: every array must be 16-byte aligned");
    return gemv_i4g32_addnorm_geglu_launch(res, delta, delta ? n_delta : 0, norm_w, eps, res_out, wp, scale_f16, h_bf16, N, K, st);
}

static int gemv_i8row_entry(const char *name, bool fp32_only, const float *x, const int8_t *w8, const float *scale, float *y, int M,
                           int N, int K, hipStream_t st) {
    CHADQ_REQUIRE(M >= 1 && M <= 16, CHADQ_ERR_SHAPE, "%s: M=%d outside [1,16]", name, M);
    CHADQ_REQUIRE(N >= 0 && K >= 16 && K % 16 == 0, CHADQ_ERR_SHAPE, "%s: N=%d K=%d (K must be a positive multiple of 16)", name, N, K);
    if (N == 0) return 0;
    CHADQ_REQUIRE(x && w8 && scale && y, CHADQ_ERR_NULL, "%s: null pointer", name);
    CHADQ_REQUIRE(aligned16(x) && aligned16(w8), CHADQ_ERR_ALIGN, "%s: x and w8 must be 16-byte aligned", name);
    return gemv_i8row_dispatch(x, w8, scale, y, M, N, K, fp32_only, st);
}

int chadq_gemv_i8row(const float *x, const int8_t *w8, const float *scale, float *y, int M, int N, int K,
                     void *stream) {
    ENTER();
    return gemv_i8row_entry("chadq_gemv_i8row", false, x, w8, scale, y, M, N, K, st);
}

int chadq_gemv_i8row_fp32(const float *x, const int8_t *w8, const float *scale, float *y, int M, int N, int K,
                          void *stream) {
    ENTER();
    return gemv_i8row_entry("chadq_gemv_i8row_fp32", true, x, w8, scale, y, M, N, K, st);
}

int chadq_gemm_i4g32_bf16(const uint16_t *x_bf16, const uint8_t *wp, const uint16_t *scale_f16, uint16_t *y_bf16,
                          int M, int N, int K, void *stream) {
    ENTER();
    CHADQ_REQUIRE(M >= 0 && N >= 0 && K >= 32 && K % 32 == 0, CHADQ_ERR_SHAPE, "chadq_gemm_i4g32_bf16: M=%d N=%d K=%d (K must be a positive multiple of 32)", M, N, K);
    if (M == 0 || N == 0) return 0;
    CHADQ_REQUIRE(x_bf16 && wp && scale_f16 && y_bf16, CHADQ_ERR_NULL, "chadq_gemm_i4g32_bf16: null pointer");
    CHADQ_REQUIRE(aligned16(x_bf16) && aligned16(wp), CHADQ_ERR_ALIGN, "chadq_gemm_i4g32_bf16: x and wp must be 16-byte aligned");
    return gemm_i4g32_bf16_dispatch(x_bf16, wp, scale_f16, y_bf16, M, N, K, st);
}

int chadq_gemm_i8row_bf16(const uint16_t *x_bf16, const int8_t *w8, const float *scale, uint16_t *y_bf16, int M,
                          int N, int K, void *stream) {
    ENTER();
    CHADQ_REQUIRE(M >= 0 && N >= 0 && K >= 16 && K % 16 == 0, CHADQ_ERR_SHAPE, "chadq_gemm_i8row_bf16: M=%d N=%d K=%d (K must be a positive multiple of 16)", M, N, K);
    if (M == 0 || N == 0) return 0;
    CHADQ_REQUIRE(x_bf16 && w8 && scale && y_bf16, CHADQ_ERR_NULL, "chadq_gemm_i8row_bf16: null pointer");
    CHADQ_REQUIRE(aligned16(x_bf16) && aligned16(w8), CHADQ_ERR_ALIGN, "chadq_gemm_i8row_bf16: x and w8 must be 16-byte aligned");
    return gemm_i8row_bf16_dispatch(x_bf16, w8, scale, y_bf16, M, N, K, st);
}

static bool moe_sizes_ok(int T, int H, int F, int E, int top_k) {
    return T >= 1 && H >= 32 && F >= 32 && H % 32 == 0 && F % 32 == 0 && E >= 1 && E <= 16 && top_k >= 1 && top_k <= 8 &&
           top_k <= E;
}

int chadq_moe_route(const float *logits, int32_t *idx, float *w, int T, int E, int top_k, int renorm, void *stream) {
    ENTER();
    CHADQ_REQUIRE(T >= 0 && E >= 1 && E <= 16 && top_k >= 1 && top_k <= 8 && top_k <= E, CHADQ_ERR_SHAPE,
                  "chadq_moe_route: T=%d E=%d top_k=%d (E <= 16, top_k <= min(E, 8))", T, E, top_k);
    if (T == 0) return 0;
    CHADQ_REQUIRE(logits && idx && w, CHADQ_ERR_NULL, "chadq_moe_route: null pointer");
    return moe_route_launch(logits, idx, w, T, E, top_k, renorm, st);
}

size_t chadq_moe_ffn_i4g32_workspace_bytes(int T, int H, int F, int E, int top_k) {
    if (!moe_sizes_ok(T, H, F, E, top_k)) return 0;
    return moe_workspace_bytes(T, H, F, E, top_k);
}

static int moe_ffn_entry(const char *name, bool tiled, const uint16_t *x_bf16, const float *logits,
                         const chadq_moe_expert_i4g32 *experts, uint16_t *y_bf16, int T, int H, int F, int E, int top_k, int renorm,
                         void *workspace, size_t workspace_bytes, hipStream_t st) {
    CHADQ_REQUIRE(moe_sizes_ok(T, H, F, E, top_k), CHADQ_ERR_SHAPE,
                  "%s: T=%d H=%d F=%d E=%d top_k=%d (H, F multiples of 32; E <= 16; top_k <= min(E, 8))", name, T, H, F, E, top_k);
    CHADQ_REQUIRE(!tiled || moe_ffn_tiled_ok(H, F), CHADQ_ERR_SHAPE, "%s: H=%d and F=%d must be multiples of 256", name, H, F);
    // the tile-order kernel addresses its activation matrices with 32-bit byte offsets
    CHADQ_REQUIRE(!tiled || (size_t)T * top_k * (size_t)(H > F ? H : F) < ((size_t)1 << 30), CHADQ_ERR_SHAPE,
                  "%s: T * top_k * max(H, F) = %zu must stay below 2^30", name, (size_t)T * top_k * (size_t)(H > F ? H : F));
    CHADQ_REQUIRE(x_bf16 && logits && experts && y_bf16, CHADQ_ERR_NULL, "%s: null pointer", name);
    for (int e = 0; e < E; ++e)
        CHADQ_REQUIRE(experts[e].wg && experts[e].sg && experts[e].wu && experts[e].su && experts[e].wd && experts[e].sd,
                      CHADQ_ERR_NULL, "%s: expert %d has a null weight pointer", name, e);
    const size_t need = moe_workspace_bytes(T, H, F, E, top_k);
    CHADQ_REQUIRE(workspace && workspace_bytes >= need, CHADQ_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", name,
                  need, workspace ? workspace_bytes : (size_t)0);
    CHADQ_REQUIRE(aligned16(x_bf16) && aligned16(workspace) && aligned16(y_bf16), CHADQ_ERR_ALIGN,
                  "%s: x, y and workspace must be 16-byte aligned", name);
    return moe_ffn_i4g32_launch(x_bf16, logits, experts, y_bf16, T, H, F, E, top_k, renorm, workspace, tiled, st);
}

int chadq_moe_ffn_i4g32(const uint16_t *x_bf16, const float *logits, const chadq_moe_expert_i4g32 *experts,
                        uint16_t *y_bf16, int T, int H, int F, int E, int top_k, int renorm, void *workspace,
                        size_t workspace_bytes, void *stream) {
    ENTER();
    return moe_ffn_entry("chadq_moe_ffn_i4g32", false, x_bf16, logits, experts, y_bf16, T, H, F, E, top_k, renorm, workspace,
                         workspace_bytes, st);
}

int chadq_moe_ffn_i4g32_tiled(const uint16_t *x_bf16, const float *logits, const chadq_moe_expert_i4g32 *experts,
                              uint16_t *y_bf16, int T, int H, int F, int E, int top_k, int renorm, void *workspace,
                              size_t workspace_bytes, void *stream) {
    ENTER();
    return moe_ffn_entry("chadq_moe_ffn_i4g32_tiled", true, x_bf16, logits, experts, y_bf16, T, H, F, E, top_k, renorm, workspace,
                         workspace_bytes, st);
}

static int repack_entry(const char *name, bool to_tiles, const uint8_t *wp_in, const uint16_t *sc_in, uint8_t *wp_out,
                        uint16_t *sc_out, int N, int K, hipStream_t st) {
    CHADQ_REQUIRE(N >= 0 && K >= 0 && N % 32 == 0 && K % 256 == 0, CHADQ_ERR_SHAPE, "%s: N=%d must be a multiple of 32, K=%d of 256",
                  name, N, K);
    if (N == 0 || K == 0) return 0;
    CHADQ_REQUIRE(wp_in && sc_in && wp_out && sc_out, CHADQ_ERR_NULL, "%s: null pointer", name);
    CHADQ_REQUIRE(wp_in != wp_out && sc_in != sc_out, CHADQ_ERR_SHAPE, "%s: input and output must be different buffers", name);
    CHADQ_REQUIRE(aligned16(wp_in) && aligned16(sc_in) && aligned16(wp_out) && aligned16(sc_out), CHADQ_ERR_ALIGN,
                  "%s: all four arrays must be 16-byte aligned", name);
    return repack_i4g32_tiles_launch(wp_in, sc_in, wp_out, sc_out, N, K, to_tiles, st);
}

int chadq_repack_i4g32_tiles(const uint8_t *wp, const uint16_t *scale_f16, uint8_t *wp_tiles, uint16_t *scale_tiles, int N, int K,
                             void *stream) {
    ENTER();
    return repack_entry("chadq_repack_i4g32_tiles", true, wp, scale_f16, wp_tiles, scale_tiles, N, K, st);
}

int chadq_unrepack_i4g32_tiles(const uint8_t *wp_tiles, const uint16_t *scale_tiles, uint8_t *wp, uint16_t *scale_f16, int N, int K,
                               void *stream) {
    ENTER();
    return repack_entry("chadq_unrepack_i4g32_tiles", false, wp_tiles, scale_tiles, wp, scale_f16, N, K, st);
}

int chadq_embed_i4g32(const int32_t *token, const uint8_t *wp, const uint16_t *scale_f16, float *x, int d, int V, void *stream) {
    ENTER();
    CHADQ_REQUIRE(d >= 32 && d % 32 == 0 && V >= 1, CHADQ_ERR_SHAPE,
                  "chadq_embed_i4g32: d=%d must be a positive multiple of 32, V=%d positive", d, V);
    CHADQ_REQUIRE(token && wp && scale_f16 && x, CHADQ_ERR_NULL, "chadq_embed_i4g32: null pointer");
    return embed_launch(token, wp, scale_f16, x, d, V, st);
}

int chadq_add_rmsnorm_bf16(float *res, const float *delta, int n_delta, const float *w, uint16_t *y_bf16, int d, float eps,
                           void *stream) {
    ENTER();
    CHADQ_REQUIRE(d >= 1 && n_delta >= 0 && n_delta <= 64, CHADQ_ERR_SHAPE, "chadq_add_rmsnorm_bf16: d=%d n_delta=%d", d, n_delta);
    CHADQ_REQUIRE(res && w && y_bf16 && (delta || n_delta == 0), CHADQ_ERR_NULL, "chadq_add_rmsnorm_bf16: null pointer");
    return add_rmsnorm_launch(res, delta, delta ? n_delta : 0, w, y_bf16, d, eps, st);
}

int chadq_rope_kv_write(const float *qkv, const int32_t *pos, float *q_out, uint16_t *kcache_bf16,
                        uint16_t *vcache_bf16, int hq, int dh, int max_ctx, float base, void *stream) {
    ENTER();
    CHADQ_REQUIRE(hq >= 1 && dh >= 2 && dh % 2 == 0 && max_ctx >= 1, CHADQ_ERR_SHAPE,
                  "chadq_rope_kv_write: hq=%d dh=%d max_ctx=%d", hq, dh, max_ctx);
    CHADQ_REQUIRE(qkv && pos && q_out && kcache_bf16 && vcache_bf16, CHADQ_ERR_NULL, "chadq_rope_kv_write: null pointer");
    return rope_kv_launch(qkv, pos, q_out, kcache_bf16, vcache_bf16, hq, dh, max_ctx, base, st);
}

size_t chadq_attn_decode_mqa_workspace_floats(int hq, int dh, int max_ctx) {
    if (hq < 1 || dh < 1 || max_ctx < 1) return 0;
    return (size_t)((max_ctx + 31) / 32) * hq * (dh + 2);
}

int chadq_attn_decode_mqa(const float *q, const uint16_t *kcache_bf16, const uint16_t *vcache_bf16, const int32_t *pos,
                          float *workspace, uint16_t *out_bf16, int hq, int dh, int max_ctx, void *stream) {
    ENTER();
    CHADQ_REQUIRE(hq >= 1 && hq <= 8 && dh >= 8 && dh <= 256 && dh % 8 == 0 && max_ctx >= 1 && max_ctx <= 65536,
                  CHADQ_ERR_SHAPE,
                  "chadq_attn_decode_mqa: hq=%d dh=%d max_ctx=%d (hq <= 8, dh <= 256 and a multiple of 8, max_ctx <= 65536)", hq,
                  dh, max_ctx);
    CHADQ_REQUIRE(q && kcache_bf16 && vcache_bf16 && pos && workspace && out_bf16, CHADQ_ERR_NULL,
                  "chadq_attn_decode_mqa: null pointer");
    CHADQ_REQUIRE(aligned16(kcache_bf16) && aligned16(q), CHADQ_ERR_ALIGN,
                  "chadq_attn_decode_mqa: q and kcache must be 16-byte aligned");
    return attn_mqa_launch(q, kcache_bf16, vcache_bf16, pos, workspace, out_bf16, hq, dh, max_ctx, st);
}

int chadq_rope_table(float *table, int dh, int max_ctx, float base, void *stream) {
    ENTER();
    CHADQ_REQUIRE(dh >= 2 && dh % 2 == 0 && max_ctx >= 1 && base > 0.f, CHADQ_ERR_SHAPE, "chadq_rope_table: dh=%d max_ctx=%d", dh,
                  max_ctx);
    CHADQ_REQUIRE(table, CHADQ_ERR_NULL, "chadq_rope_table: null pointer");
    return rope_table_launch(table, dh, max_ctx, base, st);
}

size_t chadq_attn_decode_mqa_fused_workspace_floats(int hq, int dh, int max_ctx) {
    if (hq < 1 || dh < 1 || max_ctx < 1) return 0;
    return (size_t)((max_ctx + 31) / 32) * hq * (dh + 2);
}

int chadq_attn_decode_mqa_fused(const float *qkv, const int32_t *pos, const float *rope_table, uint16_t *kcache_bf16,
                                uint16_t *vcache_bf16, float *workspace, uint16_t *out_bf16, int hq, int dh, int max_ctx,
                                void *stream) {
    ENTER();
    CHADQ_REQUIRE(hq >= 1 && hq <= 8 && dh >= 16 && dh <= 256 && dh % 16 == 0 && max_ctx >= 1 && max_ctx <= 65536, CHADQ_ERR_SHAPE,
                  "chadq_attn_decode_mqa_fused: hq=%d dh=%d max_ctx=%d (hq <= 8, dh <= 256 and a multiple of 16, max_ctx <= 65536)",
                  hq, dh, max_ctx);
    CHADQ_REQUIRE(qkv && pos && rope_table && kcache_bf16 && vcache_bf16 && workspace && out_bf16, CHADQ_ERR_NULL,
                  "chadq_attn_decode_mqa_fused: null pointer");
    CHADQ_REQUIRE(aligned16(qkv) && aligned16(rope_table) && aligned16(kcache_bf16), CHADQ_ERR_ALIGN,
                  "chadq_attn_decode_mqa_fused: qkv, rope_table and kcache must be 16-byte aligned");
    return attn_mqa_fused_launch(qkv, pos, rope_table, kcache_bf16, vcache_bf16, workspace, out_bf16, hq, dh, max_ctx, st);
}

int chadq_attn_decode_mqa_fused_oproj_i4g32(const float *qkv, const int32_t *pos, const float *rope_table, uint16_t *kcache_bf16,
                                            uint16_t *vcache_bf16, float *workspace, const uint8_t *wp,
                                            const uint16_t *scale_f16, float *y_parts, int hq, int dh, int max_ctx, int N,
                                            void *stream) {
    ENTER();
    CHADQ_REQUIRE(attn_mqa_fused_oproj_ok(hq, dh) && max_ctx >= 1 && max_ctx <= 65536 && N >= 1, CHADQ_ERR_SHAPE,
                  "chadq_attn_decode_mqa_fused_oproj_i4g32: hq=%d dh=%d max_ctx=%d N=%d (dh = 256, hq one of 2, 4, 6, 8, "
                  "max_ctx <= 65536)", hq, dh, max_ctx, N);
    CHADQ_REQUIRE(qkv && pos && rope_table && kcache_bf16 && vcache_bf16 && workspace && wp && scale_f16 && y_parts, CHADQ_ERR_NULL,
                  "chadq_attn_decode_mqa_fused_oproj_i4g32: null pointer");
    CHADQ_REQUIRE(aligned16(qkv) && aligned16(rope_table) && aligned16(kcache_bf16) && aligned16(workspace) && aligned16(wp),
                  CHADQ_ERR_ALIGN,
                  "chadq_attn_decode_mqa_fused_oproj_i4g32: qkv, rope_table, kcache, workspace and wp must be 16-byte aligned");
    return attn_mqa_fused_oproj_launch(qkv, pos, rope_table, kcache_bf16, vcache_bf16, workspace, wp, scale_f16, y_parts, hq, dh,
                                       max_ctx, N, st);
}

int chadq_attn_decode_mqa_fused_static(const float *qkv, const int32_t *pos, const float *rope_table, uint16_t *kcache_bf16,
                                       uint16_t *vcache_bf16, uint16_t *out_bf16, int hq, int dh, int max_ctx, void *stream) {
    ENTER();
    CHADQ_REQUIRE(hq >= 1 && hq <= 8 && dh >= 16 && dh <= 256 && dh % 16 == 0 && max_ctx >= 1, CHADQ_ERR_SHAPE,
                  "chadq_attn_decode_mqa_fused_static: hq=%d dh=%d max_ctx=%d (hq <= 8, dh <= 256 and a multiple of 16)", hq, dh, max_ctx);
    CHADQ_REQUIRE(max_ctx <= attn_mqa_fused_static_max_ctx(), CHADQ_ERR_WORKSPACE,
                  "chadq_attn_decode_mqa_fused_static: max_ctx=%d exceeds the %d rows the built-in scratch covers "
                  "(use chadq_attn_decode_mqa_fused with a workspace)", max_ctx, attn_mqa_fused_static_max_ctx());
    CHADQ_REQUIRE(qkv && pos && rope_table && kcache_bf16 && vcache_bf16 && out_bf16, CHADQ_ERR_NULL,
                  "chadq_attn_decode_mqa_fused_static: null pointer");
    CHADQ_REQUIRE(aligned16(qkv) && aligned16(rope_table) && aligned16(kcache_bf16), CHADQ_ERR_ALIGN,
                  "chadq_attn_decode_mqa_fused_static: qkv, rope_table and kcache must be 16-byte aligned");
    return attn_mqa_fused_static_launch(qkv, pos, rope_table, kcache_bf16, vcache_bf16, out_bf16, hq, dh, max_ctx, st);
}

int chadq_geglu_bf16(const float *gu, uint16_t *h_bf16, int F, void *stream) {
    ENTER();
    CHADQ_REQUIRE(F >= 1, CHADQ_ERR_SHAPE, "chadq_geglu_bf16: F=%d", F);
    CHADQ_REQUIRE(gu && h_bf16, CHADQ_ERR_NULL, "chadq_geglu_bf16: null pointer");
    return geglu_launch(gu, h_bf16, F, st);
}

int chadq_argmax_f32(const float *v, int n, void *scratch, int32_t *token, int32_t *pos, int advance, void *stream) {
    ENTER();
    CHADQ_REQUIRE(n >= 1, CHADQ_ERR_SHAPE, "chadq_argmax_f32: n=%d", n);
    CHADQ_REQUIRE(v && scratch && token && (pos || !advance), CHADQ_ERR_NULL, "chadq_argmax_f32: null pointer");
    float *pv = reinterpret_cast<float *>(scratch);
    int32_t *pi = reinterpret_cast<int32_t *>(pv + 256);
    return argmax_launch(v, n, pv, pi, token, pos, advance, st);
}

// candidates of the GEMV's workgroups: at least 24 rows each (four 8-row tiles that may use 6 of their rows)
static size_t gemv_argmax_candidates(int N) {
    const size_t wgs = ((size_t)(N + 5) / 6 + 3) / 4;
    return wgs > 256 ? wgs : 256;
}

size_t chadq_gemv_i4g32_argmax_scratch_bytes(int N, int K) {
    (void)K;
    return N >= 1 ? 8 * gemv_argmax_candidates(N) : 0;
}

int chadq_gemv_i4g32_argmax(const uint16_t *x_bf16, const uint8_t *wp, const uint16_t *scale_f16, float *y, int N, int K,
                            void *scratch, int32_t *token, int32_t *pos, int advance, float *next_x, void *stream) {
    ENTER();
    CHADQ_REQUIRE(N >= 1 && K >= 32 && K % 32 == 0, CHADQ_ERR_SHAPE,
                  "chadq_gemv_i4g32_argmax: N=%d K=%d (K must be a positive multiple of 32)", N, K);
    CHADQ_REQUIRE(x_bf16 && wp && scale_f16 && y && scratch && token && (pos || !advance), CHADQ_ERR_NULL,
                  "chadq_gemv_i4g32_argmax: null pointer");
    CHADQ_REQUIRE(aligned16(x_bf16) && aligned16(wp), CHADQ_ERR_ALIGN, "chadq_gemv_i4g32_argmax: x and wp must be 16-byte aligned");
    const size_t cap = gemv_argmax_candidates(N);
    float *pv = reinterpret_cast<float *>(scratch);
    int32_t *pi = reinterpret_cast<int32_t *>(pv + cap);
    if (gemv_i4g32_argmax_ok(scale_f16, N, K)) {
        int n_cand = 0;
        int rc = gemv_i4g32_argmax_launch(x_bf16, nullptr, scale_f16, y, N, K, pv, pi, &n_cand, st);  // the grid only
        if (rc != 0) return rc;
        CHADQ_REQUIRE(n_cand >= 1 && (size_t)n_cand <= cap, CHADQ_ERR_SHAPE,
                      "chadq_gemv_i4g32_argmax: %d workgroups for %zu candidate slots", n_cand, cap);
        rc = gemv_i4g32_argmax_launch(x_bf16, wp, scale_f16, y, N, K, pv, pi, &n_cand, st);
        if (rc != 0) return rc;
        return argmax_embed_launch(y, false, pv, pi, n_cand, N, token, pos, advance, wp, scale_f16, next_x, K, st);
    }
    const int rc = gemv_i4g32_mfma_dispatch(x_bf16, wp, scale_f16, y, 1, N, K, st);
    if (rc != 0) return rc;
    return argmax_embed_launch(y, true, pv, pi, 256, N, token, pos, advance, wp, scale_f16, next_x, K, st);
}

int chadq_sample_topk_f32(const float *v, int n, int k, float temperature, const float *u, void *workspace, int32_t *token,
                          int32_t *pos, int advance, void *stream) {
    ENTER();
    CHADQ_REQUIRE(n >= 1 && n <= 96 * 8192, CHADQ_ERR_SHAPE, "chadq_sample_topk_f32: n=%d (1..786432)", n);
    CHADQ_REQUIRE(k >= 1 && k <= 64 && k <= n, CHADQ_ERR_SHAPE, "chadq_sample_topk_f32: k=%d (1..min(64, n))", k);
    CHADQ_REQUIRE(temperature > 0.f && temperature < INFINITY, CHADQ_ERR_SHAPE, "chadq_sample_topk_f32: temperature %g", (double)temperature);
    CHADQ_REQUIRE(v && u && workspace && token && (pos || !advance), CHADQ_ERR_NULL, "chadq_sample_topk_f32: null pointer");
    float *cv = reinterpret_cast<float *>(workspace);
    int32_t *ci = reinterpret_cast<int32_t *>(cv + 96 * 64);
    return sample_topk_launch(v, n, k, temperature, u, cv, ci, token, pos, advance, st);
}

}  // extern "C"
