/*
 * Scalar C twin of chadq_oracle.py.  TEST INFRASTRUCTURE ONLY: it is the checker
 * for the HIP path, never the product; only tests/, __graft_entry__.smoke() and
 * bench.py's cpu_baseline leg may load it.
 *
 * The reference snapshot (happycube/chadslab) has no quantized matrix-product code,
 * so no function here follows a reference file:line; each one restates the closed
 * form of the benchmark configuration text with the plainest loops possible:
 *   int8 per-row:   y[m,n] = sum_k x[m,k] * (W[n,k] * s[n])
 *   int4 group-32:  y[m,n] = sum_k x[m,k] * ((u[n,k] - 8) * float(s16[n,k/32]))
 * Nibble order (this build's choice, parity unpinned): byte j of a row carries k=2j
 * in its low nibble and k=2j+1 in its high nibble.
 * It is written independently of the numpy twin (different loop structure, double
 * accumulation) so that the two check each other.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static float bf16_bits_to_f32(uint16_t b) {
    uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static uint16_t f32_to_bf16_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* NaN */
    uint32_t lsb = (u >> 16) & 1u;
    return (uint16_t)((u + 0x7fffu + lsb) >> 16);
}

/* IEEE binary16 -> float, all classes (zero, subnormal, normal, inf, nan). */
static float f16_bits_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    int exp = (h >> 10) & 0x1f;
    uint32_t man = h & 0x3ffu;
    float v;
    if (exp == 0) {
        v = ldexpf((float)man, -24);
    } else if (exp == 31) {
        uint32_t u = 0x7f800000u | (man << 13);
        memcpy(&v, &u, 4);
    } else {
        v = ldexpf((float)(man | 0x400u), exp - 25);
    }
    uint32_t u;
    memcpy(&u, &v, 4);
    u |= sign;
    memcpy(&v, &u, 4);
    return v;
}

void oracle_bf16_to_f32(const uint16_t *in, float *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = bf16_bits_to_f32(in[i]);
}

void oracle_f32_to_bf16(const float *in, uint16_t *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = f32_to_bf16_bits(in[i]);
}

void oracle_f16_to_f32(const uint16_t *in, float *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = f16_bits_to_f32(in[i]);
}

/* nbytes packed bytes -> 2*nbytes signed values in [-8,7] */
void oracle_unpack_i4(const uint8_t *wp, int8_t *q, int64_t nbytes) {
    for (int64_t i = 0; i < nbytes; ++i) {
        q[2 * i] = (int8_t)((int)(wp[i] & 0x0f) - 8);
        q[2 * i + 1] = (int8_t)((int)(wp[i] >> 4) - 8);
    }
}

void oracle_pack_i4(const int8_t *q, uint8_t *wp, int64_t nbytes) {
    for (int64_t i = 0; i < nbytes; ++i)
        wp[i] = (uint8_t)(((q[2 * i] + 8) & 0x0f) | (((q[2 * i + 1] + 8) & 0x0f) << 4));
}

/* y64[m,n] in double; x fp32 [M,K]; W int8 [N,K]; s fp32 [N] */
void oracle_gemm_i8row_f64(const float *x, const int8_t *w, const float *s, double *y, int M, int N, int K) {
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            double acc = 0.0;
            for (int k = 0; k < K; ++k) acc += (double)x[(int64_t)m * K + k] * (double)w[(int64_t)n * K + k];
            y[(int64_t)m * N + n] = acc * (double)s[n];
        }
}

/* y64[m,n] in double; x bf16 bits [M,K]; wp packed [N,K/2]; s16 fp16 bits [N,K/32] */
void oracle_gemm_i4g32_f64(const uint16_t *x, const uint8_t *wp, const uint16_t *s16, double *y, int M, int N,
                           int K) {
    int G = K / 32;
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            double acc = 0.0;
            for (int g = 0; g < G; ++g) {
                double part = 0.0;
                for (int kk = 0; kk < 32; ++kk) {
                    int k = g * 32 + kk;
                    uint8_t b = wp[(int64_t)n * (K / 2) + k / 2];
                    int u = (k & 1) ? (b >> 4) : (b & 0x0f);
                    part += (double)bf16_bits_to_f32(x[(int64_t)m * K + k]) * (double)(u - 8);
                }
                acc += part * (double)f16_bits_to_f32(s16[(int64_t)n * G + g]);
            }
            y[(int64_t)m * N + n] = acc;
        }
}

/* fp32 flavour of the same thing: what a scalar C runtime would run (used as a timed CPU baseline too). */
void oracle_gemm_i4g32_f32(const uint16_t *x, const uint8_t *wp, const uint16_t *s16, float *y, int M, int N,
                           int K) {
    int G = K / 32;
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            float acc = 0.0f;
            for (int g = 0; g < G; ++g) {
                float part = 0.0f;
                const uint8_t *row = wp + (int64_t)n * (K / 2) + g * 16;
                const uint16_t *xr = x + (int64_t)m * K + g * 32;
                for (int j = 0; j < 16; ++j) {
                    part += bf16_bits_to_f32(xr[2 * j]) * (float)((int)(row[j] & 0x0f) - 8);
                    part += bf16_bits_to_f32(xr[2 * j + 1]) * (float)((int)(row[j] >> 4) - 8);
                }
                acc += part * f16_bits_to_f32(s16[(int64_t)n * G + g]);
            }
            y[(int64_t)m * N + n] = acc;
        }
}

/* softmax over E experts, top-k by probability, lowest index wins ties, optional renormalisation. */
void oracle_moe_route(const float *logits, int32_t *idx, float *w, int T, int E, int top_k, int renorm) {
    for (int t = 0; t < T; ++t) {
        const float *z = logits + (int64_t)t * E;
        float p[256];
        float mx = z[0];
        for (int e = 1; e < E; ++e)
            if (z[e] > mx) mx = z[e];
        float sum = 0.0f;
        for (int e = 0; e < E; ++e) {
            p[e] = expf(z[e] - mx);
            sum += p[e];
        }
        for (int e = 0; e < E; ++e) p[e] /= sum;
        float wsum = 0.0f;
        for (int j = 0; j < top_k; ++j) {
            int best = -1;
            for (int e = 0; e < E; ++e) {
                int taken = 0;
                for (int i = 0; i < j; ++i)
                    if (idx[(int64_t)t * top_k + i] == e) taken = 1;
                if (taken) continue;
                if (best < 0 || z[e] > z[best]) best = e; /* order by logit: same set, no dependence on exp() rounding */
            }
            idx[(int64_t)t * top_k + j] = best;
            w[(int64_t)t * top_k + j] = p[best];
            wsum += p[best];
        }
        if (renorm)
            for (int j = 0; j < top_k; ++j) w[(int64_t)t * top_k + j] /= wsum;
    }
}

void oracle_silu(const float *in, float *out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = in[i] / (1.0f + expf(-in[i]));
}
