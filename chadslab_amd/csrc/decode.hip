// The non-GEMV pieces of a Gemma-2B-shaped decode step (benchmark config 4), batch 1.  All of them are tiny
// next to the weight stream; they exist so that the whole step stays on the GPU and can be replayed from a
// HIP graph.  The position is read from device memory (`pos`), so one captured graph serves every step.
//
// Model conventions (the configuration text fixes shapes only; these are this build's plain choices):
//   RMSNorm: y = x / sqrt(mean(x^2) + eps) * w.   RoPE: rotate-half, base 10000, on q and k.
//   Attention: multi-query (1 KV head), scores / sqrt(head_dim), softmax in fp32, KV cache bf16.
//   FFN: GeGLU with the tanh form of GELU.   Embedding: the tied int4 output table, dequantised row.
#include "chadq_common.h"

namespace chadq {

__device__ __forceinline__ float block_sum(float v, float *scratch) {
    // 256 threads: wave sums, then 4 partials through LDS
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < (int)(blockDim.x >> 6); ++i) t += scratch[i];
    return t;
}

// x[d] = (u - 8) * scale of row `token` of the tied int4 table [V, d]
__global__ __launch_bounds__(256) void embed_i4g32_kernel(const int32_t *__restrict__ token, const uint8_t *__restrict__ wp,
                                                          const uint16_t *__restrict__ sc, float *__restrict__ x, int d, int V) {
    const int t = min(max(token[0], 0), V - 1);  // a token outside the table must not become an address
    const uint8_t *row = wp + (size_t)t * (d / 2);
    const uint16_t *srow = sc + (size_t)t * (d / 32);
    for (int k = threadIdx.x; k < d; k += blockDim.x) {
        const uint8_t b = row[k >> 1];
        const int u = (k & 1) ? (b >> 4) : (b & 15);
        x[k] = (float)(u - 8) * f16_bits_to_f32(srow[k >> 5]);
    }
}

// res += delta (if delta), y = bf16(rmsnorm(res) * w); one workgroup
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(float *__restrict__ res, const float *__restrict__ delta,
                                                          const float *__restrict__ w, uint16_t *__restrict__ y, int d,
                                                          float eps) {
    __shared__ float scratch[4];
    float ss = 0.f;
    for (int k = threadIdx.x; k < d; k += blockDim.x) {
        float v = res[k];
        if (delta) {
            v += delta[k];
            res[k] = v;
        }
        ss += v * v;
    }
    const float tot = block_sum(ss, scratch);
    const float r = rsqrtf(tot / (float)d + eps);
    for (int k = threadIdx.x; k < d; k += blockDim.x) y[k] = (uint16_t)f32_to_bf16_bits(res[k] * r * w[k]);
}

// qkv fp32 = [hq*dh | dh | dh].  Rotates q (all heads) and k at position *pos, writes k and v into the caches
// at row *pos (bf16) and the rotated q as fp32.  One thread per rotation pair / v element.
__global__ __launch_bounds__(256) void rope_kv_kernel(const float *__restrict__ qkv, const int32_t *__restrict__ pos,
                                                      float *__restrict__ q_out, uint16_t *__restrict__ kcache,
                                                      uint16_t *__restrict__ vcache, int hq, int dh, int max_ctx,
                                                      float base) {
    const int p = min(max(pos[0], 0), max_ctx - 1), half = dh / 2;  // clamped: never writes outside the cache
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    const int npair = (hq + 1) * half;
    if (i < npair) {
        const int head = i / half, j = i % half;
        const float inv = powf(base, -2.f * (float)j / (float)dh);
        float sn, cs;
        sincosf((float)p * inv, &sn, &cs);  // the accurate form: angles reach thousands of radians
        const float *src = qkv + (size_t)head * dh;  // head hq is k
        const float a = src[j], b = src[j + half];
        const float ra = a * cs - b * sn, rb = b * cs + a * sn;
        if (head < hq) {
            q_out[head * dh + j] = ra;
            q_out[head * dh + j + half] = rb;
        } else {
            kcache[(size_t)p * dh + j] = (uint16_t)f32_to_bf16_bits(ra);
            kcache[(size_t)p * dh + j + half] = (uint16_t)f32_to_bf16_bits(rb);
        }
    } else if (i < npair + dh) {
        const int j = i - npair;
        vcache[(size_t)p * dh + j] = (uint16_t)f32_to_bf16_bits(qkv[(size_t)(hq + 1) * dh + j]);
    }
}

// Multi-query decode attention, split over the context.  Workgroup b handles positions [b*CS, (b+1)*CS) of the
// shared K/V for all hq heads: part[b][h] = (max, sum, out[dh]) of its slice.  dh = 256, hq <= 8, CS = 64.
constexpr int ATT_CS = 64;
__global__ __launch_bounds__(256) void attn_mqa_partial_kernel(const float *__restrict__ q, const uint16_t *__restrict__ kc,
                                                               const uint16_t *__restrict__ vc, const int32_t *__restrict__ pos,
                                                               float *__restrict__ part, int hq, int dh, int max_ctx) {
    const int ctx = min(max(pos[0], 0), max_ctx - 1) + 1;  // positions 0..pos are valid (the current token was just written)
    const int p0 = blockIdx.x * ATT_CS;
    if (p0 >= ctx) return;
    const int np = (ctx - p0) < ATT_CS ? (ctx - p0) : ATT_CS;
    __shared__ float s_sc[8][ATT_CS];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const float scale = rsqrtf((float)dh);
    // scores: wave w handles heads w and w+4; lane l handles position p0+l
    for (int h = wave; h < hq; h += 4) {
        float s = -INFINITY;
        if (lane < np) {
            const uint16_t *kr = kc + (size_t)(p0 + lane) * dh;
            const float *qh = q + (size_t)h * dh;
            float acc = 0.f;
            for (int j = 0; j < dh; j += 8) {
                const u32x4 kv = *reinterpret_cast<const u32x4 *>(kr + j);
                const uint32_t kk[4] = {kv.x, kv.y, kv.z, kv.w};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    acc += qh[j + 2 * e] * bf16_bits_to_f32(kk[e] & 0xFFFFu);
                    acc += qh[j + 2 * e + 1] * bf16_bits_to_f32(kk[e] >> 16);
                }
            }
            s = acc * scale;
        }
        s_sc[h][lane] = s;
    }
    __syncthreads();
    // per head: max, exp, sum over the slice, then out[dh]: thread t handles column t of V (dh = 256 = blockDim)
    for (int h = 0; h < hq; ++h) {
        float mx = -INFINITY;
        for (int i = 0; i < np; ++i) mx = fmaxf(mx, s_sc[h][i]);
        float sum = 0.f, o = 0.f;
        for (int i = 0; i < np; ++i) {
            const float pr = __expf(s_sc[h][i] - mx);
            sum += pr;
            if (tid < dh) o += pr * bf16_bits_to_f32(vc[(size_t)(p0 + i) * dh + tid]);
        }
        float *dst = part + ((size_t)blockIdx.x * hq + h) * (dh + 2);
        if (tid == 0) {
            dst[0] = mx;
            dst[1] = sum;
        }
        if (tid < dh) dst[2 + tid] = o;
    }
}

// out[h] = bf16( sum_b exp(m_b - M) * o_b / sum_b exp(m_b - M) * s_b ); one workgroup per head
__global__ __launch_bounds__(256) void attn_mqa_combine_kernel(const float *__restrict__ part, const int32_t *__restrict__ pos,
                                                               uint16_t *__restrict__ out, int hq, int dh, int max_ctx) {
    const int ctx = min(max(pos[0], 0), max_ctx - 1) + 1, nb = (ctx + ATT_CS - 1) / ATT_CS, h = blockIdx.x, tid = threadIdx.x;
    float M = -INFINITY;
    for (int b = 0; b < nb; ++b) M = fmaxf(M, part[((size_t)b * hq + h) * (dh + 2)]);
    float den = 0.f, num = 0.f;
    for (int b = 0; b < nb; ++b) {
        const float *src = part + ((size_t)b * hq + h) * (dh + 2);
        const float f = __expf(src[0] - M);
        den += f * src[1];
        if (tid < dh) num += f * src[2 + tid];
    }
    if (tid < dh) out[(size_t)h * dh + tid] = (uint16_t)f32_to_bf16_bits(num / den);
}

// h = bf16( gelu_tanh(g) * u ), gu = [g(F) | u(F)] fp32
__global__ __launch_bounds__(256) void geglu_kernel(const float *__restrict__ gu, uint16_t *__restrict__ h, int F) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < F) {
        const float g = gu[i], u = gu[F + i];
        const float t = tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g));
        h[i] = (uint16_t)f32_to_bf16_bits(0.5f * g * (1.f + t) * u);
    }
}

// argmax over n fp32 values (lowest index wins ties): per-workgroup candidates, then one workgroup; the winner
// becomes the next token and the position advances, so that a replayed graph steps by itself.
__global__ __launch_bounds__(256) void argmax_partial_kernel(const float *__restrict__ v, int n, float *__restrict__ pv,
                                                             int32_t *__restrict__ pi) {
    __shared__ float sv[256];
    __shared__ int si[256];
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x)
        if (v[i] > best || (v[i] == best && i < bi)) {
            best = v[i];
            bi = i;
        }
    sv[threadIdx.x] = best;
    si[threadIdx.x] = bi;
    __syncthreads();
    for (int o = 128; o > 0; o >>= 1) {
        if ((int)threadIdx.x < o) {
            const float ov = sv[threadIdx.x + o];
            const int oi = si[threadIdx.x + o];
            if (ov > sv[threadIdx.x] || (ov == sv[threadIdx.x] && oi < si[threadIdx.x])) {
                sv[threadIdx.x] = ov;
                si[threadIdx.x] = oi;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        pv[blockIdx.x] = sv[0];
        pi[blockIdx.x] = si[0];
    }
}

__global__ __launch_bounds__(256) void argmax_final_kernel(const float *__restrict__ pv, const int32_t *__restrict__ pi, int nb,
                                                           int32_t *__restrict__ token, int32_t *__restrict__ pos,
                                                           int advance) {
    __shared__ float sv[256];
    __shared__ int si[256];
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < nb; i += blockDim.x)
        if (pv[i] > best || (pv[i] == best && pi[i] < bi)) {
            best = pv[i];
            bi = pi[i];
        }
    sv[threadIdx.x] = best;
    si[threadIdx.x] = bi;
    __syncthreads();
    for (int o = 128; o > 0; o >>= 1) {
        if ((int)threadIdx.x < o) {
            const float ov = sv[threadIdx.x + o];
            const int oi = si[threadIdx.x + o];
            if (ov > sv[threadIdx.x] || (ov == sv[threadIdx.x] && oi < si[threadIdx.x])) {
                sv[threadIdx.x] = ov;
                si[threadIdx.x] = oi;
            }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        token[0] = si[0];
        if (advance) pos[0] += 1;
    }
}

int embed_launch(const int32_t *token, const uint8_t *wp, const uint16_t *sc, float *x, int d, int V, hipStream_t st) {
    hipLaunchKernelGGL(embed_i4g32_kernel, dim3(1), dim3(256), 0, st, token, wp, sc, x, d, V);
    return hip_check(hipGetLastError(), "embed launch");
}

int add_rmsnorm_launch(float *res, const float *delta, const float *w, uint16_t *y, int d, float eps, hipStream_t st) {
    hipLaunchKernelGGL(add_rmsnorm_kernel, dim3(1), dim3(256), 0, st, res, delta, w, y, d, eps);
    return hip_check(hipGetLastError(), "add_rmsnorm launch");
}

int rope_kv_launch(const float *qkv, const int32_t *pos, float *q_out, uint16_t *kc, uint16_t *vc, int hq, int dh,
                   int max_ctx, float base, hipStream_t st) {
    const int n = (hq + 1) * (dh / 2) + dh;
    hipLaunchKernelGGL(rope_kv_kernel, dim3((n + 255) / 256), dim3(256), 0, st, qkv, pos, q_out, kc, vc, hq, dh, max_ctx, base);
    return hip_check(hipGetLastError(), "rope_kv launch");
}

int attn_mqa_launch(const float *q, const uint16_t *kc, const uint16_t *vc, const int32_t *pos, float *part, uint16_t *out,
                    int hq, int dh, int max_ctx, hipStream_t st) {
    const int nb = (max_ctx + ATT_CS - 1) / ATT_CS;
    hipLaunchKernelGGL(attn_mqa_partial_kernel, dim3(nb), dim3(256), 0, st, q, kc, vc, pos, part, hq, dh, max_ctx);
    hipLaunchKernelGGL(attn_mqa_combine_kernel, dim3(hq), dim3(256), 0, st, part, pos, out, hq, dh, max_ctx);
    return hip_check(hipGetLastError(), "attn_mqa launch");
}

int geglu_launch(const float *gu, uint16_t *h, int F, hipStream_t st) {
    hipLaunchKernelGGL(geglu_kernel, dim3((F + 255) / 256), dim3(256), 0, st, gu, h, F);
    return hip_check(hipGetLastError(), "geglu launch");
}

int argmax_launch(const float *v, int n, float *pv, int32_t *pi, int32_t *token, int32_t *pos, int advance, hipStream_t st) {
    const int nb = 256;
    hipLaunchKernelGGL(argmax_partial_kernel, dim3(nb), dim3(256), 0, st, v, n, pv, pi);
    hipLaunchKernelGGL(argmax_final_kernel, dim3(1), dim3(256), 0, st, pv, pi, nb, token, pos, advance);
    return hip_check(hipGetLastError(), "argmax launch");
}

}  // namespace chadq
