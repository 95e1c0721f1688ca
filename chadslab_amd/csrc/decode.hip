// The non-GEMV pieces of a Gemma-2B-shaped decode step (benchmark config 4), batch 1.  All of them are tiny
// next to the weight stream; they exist so that the whole step stays on the GPU and can be replayed from a
// HIP graph.  The position is read from device memory (`pos`), so one captured graph serves every step.
//
// Model conventions (the configuration text fixes shapes only; these are this build's plain choices):
//   RMSNorm: y = x / sqrt(mean(x^2) + eps) * w.   RoPE: rotate-half, base 10000, on q and k.
//   Attention: multi-query (1 KV head), scores / sqrt(head_dim), softmax in fp32, KV cache bf16.
//   FFN: GeGLU with the tanh form of GELU.   Embedding: the tied int4 output table, dequantised row.
#include <type_traits>

#include <climits>

#include "chadq_common.h"

namespace chadq {

// Sum / max over a workgroup of up to 256 threads; `scratch` holds one float per wave.  Both end with every
// thread holding the result and may be called back to back on the same scratch.
__device__ __forceinline__ float block_sum(float v, float *scratch) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < (int)(blockDim.x >> 6); ++i) t += scratch[i];
    return t;
}

__device__ __forceinline__ float block_max(float v, float *scratch) {
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = -INFINITY;
    for (int i = 0; i < (int)(blockDim.x >> 6); ++i) t = fmaxf(t, scratch[i]);
    return t;
}

// x[d] = (u - 8) * scale of row t of the tied int4 table [V, d], by one workgroup.  Eight weights per thread and round
// where the pointers allow it (one 4-byte load, one scale, two 16-byte stores), the plain loop otherwise: same values.
__device__ __forceinline__ void embed_row(int t, const uint8_t *__restrict__ wp, const uint16_t *__restrict__ sc,
                                          float *__restrict__ x, int d) {
    const uint8_t *row = wp + (size_t)t * (d / 2);
    const uint16_t *srow = sc + (size_t)t * (d / 32);
    if (((reinterpret_cast<uintptr_t>(row) & 3u) | (reinterpret_cast<uintptr_t>(x) & 15u)) == 0) {
        for (int k8 = threadIdx.x; k8 < (d >> 3); k8 += blockDim.x) {
            const uint32_t w = *reinterpret_cast<const uint32_t *>(row + 4 * k8);
            const float s = f16_bits_to_f32(srow[k8 >> 2]);
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = (float)((int)((w >> (4 * e)) & 15u) - 8) * s;
            *reinterpret_cast<f32x4 *>(x + 8 * k8) = f32x4{v[0], v[1], v[2], v[3]};
            *reinterpret_cast<f32x4 *>(x + 8 * k8 + 4) = f32x4{v[4], v[5], v[6], v[7]};
        }
        return;
    }
    for (int k = threadIdx.x; k < d; k += blockDim.x) {
        const uint8_t b = row[k >> 1];
        const int u = (k & 1) ? (b >> 4) : (b & 15);
        x[k] = (float)(u - 8) * f16_bits_to_f32(srow[k >> 5]);
    }
}

__global__ __launch_bounds__(256) void embed_i4g32_kernel(const int32_t *__restrict__ token, const uint8_t *__restrict__ wp,
                                                          const uint16_t *__restrict__ sc, float *__restrict__ x, int d, int V) {
    embed_row(min(max(token[0], 0), V - 1), wp, sc, x, d);  // a token outside the table must not become an address
}

// res += sum_j delta[j] (nd vectors of d floats, added in order), y = bf16(rmsnorm(res) * w); one workgroup.
// Any d, any nd: the plain loop form.
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(float *__restrict__ res, const float *__restrict__ delta, int nd,
                                                          const float *__restrict__ w, uint16_t *__restrict__ y, int d,
                                                          float eps) {
    __shared__ float scratch[4];
    float ss = 0.f;
    for (int k = threadIdx.x; k < d; k += blockDim.x) {
        float v = res[k];
        for (int j = 0; j < nd; ++j) v += delta[(size_t)j * d + k];
        if (nd > 0) res[k] = v;
        ss += v * v;
    }
    const float tot = block_sum(ss, scratch);
    const float r = rsqrtf(tot / (float)d + eps);
    for (int k = threadIdx.x; k < d; k += blockDim.x) y[k] = (uint16_t)f32_to_bf16_bits(res[k] * r * w[k]);
}

// The same for d % 4 == 0, d <= 1024 * NV: every load of the kernel is issued before anything waits (one memory
// round trip instead of three), the vector stays in registers between the two passes.
template <int NV, int ND>
__global__ __launch_bounds__(256) void add_rmsnorm_vec_kernel(float *__restrict__ res, const float *__restrict__ delta,
                                                              const float *__restrict__ w, uint16_t *__restrict__ y, int d,
                                                              float eps) {
    __shared__ float scratch[4];
    const int nv = d >> 2, tid = threadIdx.x;
    f32x4 r[NV], wv[NV], dl[ND > 0 ? ND : 1][NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int i = tid + 256 * j, ii = i < nv ? i : 0;  // clamped address, the data is discarded
        r[j] = reinterpret_cast<const f32x4 *>(res)[ii];
        wv[j] = reinterpret_cast<const f32x4 *>(w)[ii];
#pragma unroll
        for (int s = 0; s < ND; ++s) dl[s][j] = reinterpret_cast<const f32x4 *>(delta)[(size_t)s * nv + ii];
    }
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int i = tid + 256 * j;
#pragma unroll
        for (int s = 0; s < ND; ++s) r[j] += dl[s][j];
        if (i < nv) {
            if (ND > 0) reinterpret_cast<f32x4 *>(res)[i] = r[j];
            ss += r[j].x * r[j].x + r[j].y * r[j].y + r[j].z * r[j].z + r[j].w * r[j].w;
        }
    }
    const float tot = block_sum(ss, scratch);
    const float rinv = rsqrtf(tot / (float)d + eps);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int i = tid + 256 * j;
        if (i < nv) {
            const uint32_t lo = f32_to_bf16_bits(r[j].x * rinv * wv[j].x) | (f32_to_bf16_bits(r[j].y * rinv * wv[j].y) << 16);
            const uint32_t hi = f32_to_bf16_bits(r[j].z * rinv * wv[j].z) | (f32_to_bf16_bits(r[j].w * rinv * wv[j].w) << 16);
            reinterpret_cast<uint2 *>(y)[i] = make_uint2(lo, hi);
        }
    }
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
// shared K/V for all hq heads: part[b][h] = (max, sum, out[dh]) of its slice.  dh <= 256, hq <= 8, CS = 32.
// Every global load of the workgroup (its K rows, its V columns, q) is issued before the first wait: the
// kernel is one memory round trip plus a few hundred ALU operations per thread.
constexpr int ATT_CS = 32;
__global__ __launch_bounds__(256) void attn_mqa_partial_kernel(const float *__restrict__ q, const uint16_t *__restrict__ kc,
                                                               const uint16_t *__restrict__ vc, const int32_t *__restrict__ pos,
                                                               float *__restrict__ part, int hq, int dh, int max_ctx) {
    const int ctx = min(max(pos[0], 0), max_ctx - 1) + 1;  // positions 0..pos are valid (the current token was just written)
    const int p0 = blockIdx.x * ATT_CS;
    if (p0 >= ctx) return;
    __shared__ __attribute__((aligned(16))) float s_sc[8][ATT_CS];  // scores, then probabilities
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int half = lane >> 5, c = lane & 31, lpr = dh >> 3;  // 16-byte piece c of a K row; two rows per wave load

    // V: thread t owns column t of every row of the slice (rows beyond the context repeat the last valid one;
    // their probability is 0)
    const int col = tid < dh ? tid : dh - 1;
    uint16_t vv[ATT_CS];
#pragma unroll
    for (int i = 0; i < ATT_CS; ++i) {
        const int pi = (p0 + i < ctx) ? p0 + i : ctx - 1;
        vv[i] = vc[(size_t)pi * dh + col];
    }
    // K: wave w owns rows 8w..8w+7 of the slice
    const int cc = c < lpr ? c : 0;
    u32x4 kv[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int pl = wave * 8 + 2 * i + half;
        const int pi = (p0 + pl < ctx) ? p0 + pl : ctx - 1;
        kv[i] = *reinterpret_cast<const u32x4 *>(kc + (size_t)pi * dh + cc * 8);
    }
    // q: the lane's 8 columns of every head
    f32x4 qa[8], qb[8];
#pragma unroll
    for (int h = 0; h < 8; ++h) {
        const float *qh = q + (size_t)(h < hq ? h : 0) * dh + cc * 8;
        qa[h] = *reinterpret_cast<const f32x4 *>(qh);
        qb[h] = *reinterpret_cast<const f32x4 *>(qh + 4);
    }
    __builtin_amdgcn_sched_barrier(0);

    const bool live = c < lpr;
    const float scale = rsqrtf((float)dh);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int pl = wave * 8 + 2 * i + half;
        const uint32_t kk[4] = {kv[i].x, kv[i].y, kv[i].z, kv[i].w};
        float k8[8];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            k8[2 * e] = live ? bf16_bits_to_f32(kk[e] & 0xFFFFu) : 0.f;
            k8[2 * e + 1] = live ? bf16_bits_to_f32(kk[e] >> 16) : 0.f;
        }
#pragma unroll
        for (int h = 0; h < 8; ++h) {
            float acc = qa[h].x * k8[0] + qa[h].y * k8[1] + qa[h].z * k8[2] + qa[h].w * k8[3] + qb[h].x * k8[4] +
                        qb[h].y * k8[5] + qb[h].z * k8[6] + qb[h].w * k8[7];
            for (int o = 16; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);  // stays inside the 32-lane half
            if (c == 0) s_sc[h][pl] = (p0 + pl < ctx && h < hq) ? acc * scale : -INFINITY;
        }
    }
    __syncthreads();
    {
        // softmax of the slice: thread -> (head tid/32, position tid%32)
        const int h = tid >> 5, i = tid & 31;
        const float s = s_sc[h][i];
        float mx = s;
        for (int o = 16; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
        const float pr = (h < hq) ? __expf(s - mx) : 0.f;  // position p0 is always valid, so mx is finite for real heads
        float sum = pr;
        for (int o = 16; o > 0; o >>= 1) sum += __shfl_xor(sum, o, 64);
        s_sc[h][i] = pr;
        if (i == 0 && h < hq) {
            float *dst = part + ((size_t)blockIdx.x * hq + h) * (dh + 2);
            dst[0] = mx;
            dst[1] = sum;
        }
    }
    __syncthreads();
    float o[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < ATT_CS; i += 4) {
        const float v0 = bf16_bits_to_f32(vv[i]), v1 = bf16_bits_to_f32(vv[i + 1]), v2 = bf16_bits_to_f32(vv[i + 2]),
                    v3 = bf16_bits_to_f32(vv[i + 3]);
#pragma unroll
        for (int h = 0; h < 8; ++h) {
            const f32x4 p4 = *reinterpret_cast<const f32x4 *>(&s_sc[h][i]);
            o[h] += p4.x * v0 + p4.y * v1 + p4.z * v2 + p4.w * v3;
        }
    }
    if (tid < dh) {
#pragma unroll
        for (int h = 0; h < 8; ++h)
            if (h < hq) part[((size_t)blockIdx.x * hq + h) * (dh + 2) + 2 + tid] = o[h];
    }
}

// Max over the 64 lanes of a wavefront, returned to every lane (DPP moves; a lane a move does not reach keeps its own).
__device__ __forceinline__ float wave_max_all(float v) {
#define CHADQ_MAX_STEP(CTRL, MASK) \
    v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, MASK, 0xF, false)));
    CHADQ_MAX_STEP(0xB1, 0xF)   // quad_perm [1,0,3,2]
    CHADQ_MAX_STEP(0x4E, 0xF)   // quad_perm [2,3,0,1]
    CHADQ_MAX_STEP(0x141, 0xF)  // row_half_mirror
    CHADQ_MAX_STEP(0x140, 0xF)  // row_mirror
    CHADQ_MAX_STEP(0x142, 0xA)  // row_bcast15 into rows 1 and 3
    CHADQ_MAX_STEP(0x143, 0xC)  // row_bcast31 into rows 2 and 3
#undef CHADQ_MAX_STEP
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

__device__ __forceinline__ float lane_value(float v, int lane_index) {  // lane_index uniform
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane_index));
}

// out[h] = bf16( sum_b exp(m_b - M) * o_b / sum_b exp(m_b - M) * s_b ).  Workgroup (h, g): head h, columns
// 64g..64g+63; its four waves take the slices b = w, w+4, ...  Every wave works out M and the factors exp(m_b - M) for
// itself, slice b in lane b % 64 (reductions on DPP moves, factors handed out with v_readlane), so the workgroup
// meets only once, for the sum over the waves.  The loads of the first 64 slices do not depend on the position and
// are issued together with it.
__global__ __launch_bounds__(256) void attn_mqa_combine_kernel(const float *__restrict__ part, const int32_t *__restrict__ pos,
                                                               uint16_t *__restrict__ out, int hq, int dh, int max_ctx) {
    const int nbmax = (max_ctx + ATT_CS - 1) / ATT_CS;  // slices the workspace holds
    const int h = blockIdx.x, tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    __shared__ float s_num[4][64];
    const size_t stride = (size_t)hq * (dh + 2);
    const float *ph = part + (size_t)h * (dh + 2);
    const int colw = blockIdx.y * 64 + lane, colc = colw < dh ? colw : dh - 1;
    float pre[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int b = wave + 4 * i;
        pre[i] = ph[(size_t)(b < nbmax ? b : nbmax - 1) * stride + 2 + colc];
    }
    const int bl = lane < nbmax ? lane : nbmax - 1;
    const float m0 = ph[(size_t)bl * stride], l0 = ph[(size_t)bl * stride + 1];
    const int ctx = min(max(pos[0], 0), max_ctx - 1) + 1, nb = (ctx + ATT_CS - 1) / ATT_CS;

    float m = lane < nb ? m0 : -INFINITY;
    for (int b = lane + 64; b < nb; b += 64) m = fmaxf(m, ph[(size_t)b * stride]);
    const float M = wave_max_all(m);
    const float f0 = lane < nb ? __expf(m0 - M) : 0.f;
    float den = lane < nb ? f0 * l0 : 0.f;
    float num = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int b = wave + 4 * i;  // < 64
        if (b < nb) num += lane_value(f0, b) * pre[i];
    }
    for (int base = 64; base < nb; base += 64) {  // contexts beyond 2048 positions
        const int b = base + lane;
        const bool in = b < nb;
        const float mb = in ? ph[(size_t)b * stride] : -INFINITY, lb = in ? ph[(size_t)b * stride + 1] : 0.f;
        const float f = in ? __expf(mb - M) : 0.f;
        den += f * lb;
        for (int j = wave; j < 64 && base + j < nb; j += 4) num += lane_value(f, j) * ph[(size_t)(base + j) * stride + 2 + colc];
    }
    den = wave_sum_to_lane63(den);
    den = lane_value(den, 63);
    s_num[wave][lane] = num;
    __syncthreads();
    if (tid < 64 && colw < dh) {
        const float t = s_num[0][tid] + s_num[1][tid] + s_num[2][tid] + s_num[3][tid];
        out[(size_t)h * dh + colw] = (uint16_t)f32_to_bf16_bits(t / den);
    }
}

// ---- the same attention as one launch: RoPE, KV-cache write, split-context partials and their combination ----
// table[p][j] = (cos, sin)(p * base^(-2j/dh)), p < max_ctx, j < dh/2; computed once per model.
__global__ __launch_bounds__(256) void rope_table_kernel(float *__restrict__ table, int dh, int max_ctx, float base) {
    const int half = dh / 2;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)max_ctx * half) return;
    const int p = (int)(i / half), j = (int)(i % half);
    const float inv = powf(base, -2.f * (float)j / (float)dh);
    float sn, cs;
    sincosf((float)p * inv, &sn, &cs);
    table[2 * i] = cs;
    table[2 * i + 1] = sn;
}

// Eight fp32 values as two MFMA operands of eight bf16 each: `hi` holds the values cut off after 16 bits (exact), `lo`
// what is left, cut off the same way, so hi + lo carries 16 mantissa bits of every value - more than the bf16 K and V
// rows they are multiplied with.  Element e sits in half-word e.
__device__ __forceinline__ void split_bf16x8(const f32x4 a, const f32x4 b, bf16x8 &hi, bf16x8 &lo) {
    const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    uint32_t h[4], l[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const uint32_t u0 = __float_as_uint(v[2 * e]), u1 = __float_as_uint(v[2 * e + 1]);
        h[e] = __builtin_amdgcn_perm(u1, u0, 0x07060302u);  // the two high half-words
        const float r0 = v[2 * e] - __uint_as_float(u0 & 0xFFFF0000u), r1 = v[2 * e + 1] - __uint_as_float(u1 & 0xFFFF0000u);
        l[e] = __builtin_amdgcn_perm(__float_as_uint(r1), __float_as_uint(r0), 0x07060302u);
    }
    __builtin_memcpy(&hi, h, 16);
    __builtin_memcpy(&lo, l, 16);
}

// Workgroup b: positions [32b, 32b+32).  qkv fp32 = [hq*dh | dh | dh] straight from the projection.  Every
// workgroup rotates q itself (table lookup): thread (head, 8-column piece) rotates its piece once and the rotated q
// goes through LDS.  The workgroup that owns position pos also rotates k, writes row pos of both caches and puts the
// new rows into LDS instead of reading them back.  Partials as attn_mqa_partial_kernel.
//
// Both products run on the matrix cores (v_mfma_f32_16x16x32_bf16; as dot products and column sums in the vector
// units they took 1.5 us each of a kernel that lasted 5):
//   scores  D[position][head] = sum_d K[position][d] * q[head][d].  A = K rows: lane (i = lane % 16, g = lane / 16)
//           holds the 16 bytes K[16*blk + i][32*st + 8g .. +7], which is what it loads from the cache - no staging.
//           B = q: lane (head = lane % 16, g) holds q[head][32*st + 8g .. +7] as two bf16 operands (split_bf16x8); heads
//           8..15 are zeros.  Wave w takes the steps st = 2w, 2w+1 (64 of the 256 columns) for both blocks of 16
//           positions: 8 MFMAs; the four waves' sums meet in LDS, where thread (head, position) picks its score up.
//   output  D[head][column] = sum_p P[head][p] * V[p][column].  A = the probabilities (two bf16 operands again), B =
//           V[8g .. 8g+7][16*cb + lane % 16]: eight 2-byte reads down a column of the V slice in LDS (rows padded so that
//           the four lane groups use different banks).  Wave w takes the column blocks cb = 4w .. 4w+3: 8 MFMAs; lane
//           (column, g < 2) then holds heads 4g .. 4g+3 of its column and stores them.
// FULL: hq = 8 and dh = 256 (the host checks), where no operand needs a guard: the reads of a phase are then issued
// together and its stores sit behind a single condition.
template <bool FULL>
__global__ __launch_bounds__(256) void attn_mqa_fused_kernel(const float *__restrict__ qkv, const int32_t *__restrict__ pos,
                                                             const float *__restrict__ table, uint16_t *__restrict__ kc,
                                                             uint16_t *__restrict__ vc, float *__restrict__ ws,
                                                             int max_ctx, int hq_arg, int dh_arg, float *__restrict__ yz, int nz) {
    // (the first 14 dwords of arguments arrive in registers with the wave: everything the full instance needs for its
    // requests; yz and nz are fetched, and used only once those requests are out)
    const int hq = FULL ? 8 : hq_arg, dh = FULL ? 256 : dh_arg;  // constants in the full instance: no divisions by dh / 8
    const int p0 = blockIdx.x * ATT_CS;
    const int pos_raw = pos[0];  // asked for at once, waited for as late as possible
    // yz[0 .. nz): accumulators of the kernel that follows this one (the output projection adds two heads' products
    // into each); cleared here, by every workgroup whatever the context, so that they need no launch of their own
    auto clear_yz = [&]() {
        for (int i = blockIdx.x * 256 + threadIdx.x; i < nz; i += gridDim.x * 256) yz[i] = 0.f;
    };
    // The position comes from device memory, half a microsecond away.  The full instance does not wait for it before
    // asking for its K and V rows and q: rows are clamped to the cache instead of to the context (rows past the
    // context then hold whatever the cache holds: their scores are masked by selection, their V rows zeroed on the way
    // into LDS), and a workgroup past the context leaves once its requests are in LDS - which is why the host picks this
    // instance only for caches of up to 8192 rows (at most 8 MB of such reads per launch).
    int p = 0, ctx = 0;
    if (!FULL) {
        clear_yz();
        p = min(max(pos_raw, 0), max_ctx - 1), ctx = p + 1;
        if (p0 >= ctx) return;
    }
    const int lim = FULL ? max_ctx : ctx;  // rows below lim may be read
    float *part = ws;
    constexpr int VP = 264;  // half-words per row of the V slice in LDS
    __shared__ __attribute__((aligned(16))) float s_sc[8][ATT_CS];          // probabilities
    __shared__ __attribute__((aligned(16))) float s_q[8][256];              // rotated q
    __shared__ __attribute__((aligned(16))) uint16_t s_v[ATT_CS][VP];       // the slice of V
    __shared__ __attribute__((aligned(16))) uint16_t s_krow[256];           // the new (rotated) k row
    __shared__ __attribute__((aligned(16))) float s_part[4][64][9];         // the waves' partial scores (9: bank spread)
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = dh >> 1, lpr = dh >> 3;
    const int li = lane & 15, g = lane >> 4;

    // V: 16-byte pieces of the slice, piece ch = row * lpr + column piece, dealt round robin to the threads
    u32x4 vld[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int ch = tid + 256 * j, row = ch / lpr, vcc = ch % lpr;  // rows past the slice (short dh): loaded, not used
        const int pi = (p0 + row < lim) ? p0 + row : lim - 1;
        vld[j] = *reinterpret_cast<const u32x4 *>(vc + (size_t)pi * dh + vcc * 8);
    }
    // K: the A operands of this wave's MFMAs, kv[blk][s2] = K[16*blk + li][32*(2*wave + s2) + 8g .. +7]
    u32x4 kv[2][2];
#pragma unroll
    for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            const int d0 = 32 * (2 * wave + s2) + 8 * g, pl = 16 * blk + li;
            const int pi = (p0 + pl < lim) ? p0 + pl : lim - 1;
            kv[blk][s2] = *reinterpret_cast<const u32x4 *>(kc + (size_t)pi * dh + (d0 < dh ? d0 : 0));
        }
    // q: thread (head tid/32, piece tid%32) loads its 8 columns, the 8 columns they rotate with, and the angles
    const int qh = tid >> 5, qc = (tid & 31) < lpr ? (tid & 31) : 0;
    const bool qlive = qh < hq && (tid & 31) < lpr;
    const int colq = qc * 8, lo = colq < half;
    const int colp = lo ? colq + half : colq - half;  // partner columns
    const int jt = lo ? colq : colq - half;           // rotation index of element 0
    const float *qrow = qkv + (size_t)(qh < hq ? qh : 0) * dh;
    const f32x4 qa = *reinterpret_cast<const f32x4 *>(qrow + colq), qb = *reinterpret_cast<const f32x4 *>(qrow + colq + 4);
    const f32x4 pa = *reinterpret_cast<const f32x4 *>(qrow + colp), pb = *reinterpret_cast<const f32x4 *>(qrow + colp + 4);
    if (FULL) {
        // The requests above go out before the position is waited for.  A workgroup past the context leaves only behind
        // the first barrier: an exit here would make the compiler move those requests behind it, where they are needed.
        __builtin_amdgcn_sched_barrier(0);
        p = min(max(pos_raw, 0), max_ctx - 1), ctx = p + 1;
    }
    const bool own = p0 < ctx && (p - p0) < ATT_CS;  // this slice contains the new position
    const float *tp = table + ((size_t)p * half + jt) * 2;
    const f32x4 t0 = *reinterpret_cast<const f32x4 *>(tp), t1 = *reinterpret_cast<const f32x4 *>(tp + 4),
                t2 = *reinterpret_cast<const f32x4 *>(tp + 8), t3 = *reinterpret_cast<const f32x4 *>(tp + 12);
    // the owner's new K/V row
    float ka = 0.f, kb = 0.f, kcs = 1.f, ksn = 0.f, vnew = 0.f;
    if (own) {
        if (tid < half) {
            ka = qkv[(size_t)hq * dh + tid];
            kb = qkv[(size_t)hq * dh + tid + half];
            kcs = table[((size_t)p * half + tid) * 2];
            ksn = table[((size_t)p * half + tid) * 2 + 1];
        }
        if (tid < dh) vnew = qkv[(size_t)(hq + 1) * dh + tid];
    }
    __builtin_amdgcn_sched_barrier(0);
    if (FULL) clear_yz();

    // rotate q: low columns a*cos - b*sin, high columns b*cos + a*sin, (a, b) = (low, high) element of the pair
    {
        const float cs[8] = {t0.x, t0.z, t1.x, t1.z, t2.x, t2.z, t3.x, t3.z};
        const float sn[8] = {t0.y, t0.w, t1.y, t1.w, t2.y, t2.w, t3.y, t3.w};
        const float sg = lo ? -1.f : 1.f;
        const float own8[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        const float par8[8] = {pa.x, pa.y, pa.z, pa.w, pb.x, pb.y, pb.z, pb.w};
        float r[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) r[e] = qlive ? own8[e] * cs[e] + sg * par8[e] * sn[e] : 0.f;
        if ((tid & 31) < lpr) {  // heads past hq hold zeros
            *reinterpret_cast<f32x4 *>(&s_q[qh][colq]) = f32x4{r[0], r[1], r[2], r[3]};
            *reinterpret_cast<f32x4 *>(&s_q[qh][colq + 4]) = f32x4{r[4], r[5], r[6], r[7]};
        }
    }
    // the V slice into LDS; the owner's new row replaces the (not yet written) cache row
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int ch = tid + 256 * j, row = ch / lpr, vcc = ch % lpr;
        if (row < ATT_CS && !(own && p0 + row == p))
            *reinterpret_cast<u32x4 *>(&s_v[row][vcc * 8]) = (!FULL || p0 + row < ctx) ? vld[j] : u32x4{0, 0, 0, 0};
    }
    if (own) {
        if (tid < half) {
            const uint16_t ra = (uint16_t)f32_to_bf16_bits(ka * kcs - kb * ksn), rb = (uint16_t)f32_to_bf16_bits(kb * kcs + ka * ksn);
            s_krow[tid] = ra;
            s_krow[tid + half] = rb;
            kc[(size_t)p * dh + tid] = ra;
            kc[(size_t)p * dh + tid + half] = rb;
        }
        if (tid < dh) {
            const uint16_t vb16 = (uint16_t)f32_to_bf16_bits(vnew);
            vc[(size_t)p * dh + tid] = vb16;
            s_v[p - p0][tid] = vb16;
        }
    }
    __syncthreads();
    if (FULL && p0 >= ctx) return;  // uniform over the workgroup

    // scores: 2 blocks of positions x 2 steps x (hi, lo) = 8 MFMAs per wave
    {
        f32x4 acc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) {
            const int st = 2 * wave + s2, d0 = 32 * st + 8 * g;
            if (FULL || 32 * st < dh) {  // uniform over the wave
                const bool qok = li < 8 && (FULL || d0 < dh);  // heads 8..15 and columns past dh: zeros
                const int dq = (FULL || d0 < dh) ? d0 : 0;
                const f32x4 zero4 = f32x4{0.f, 0.f, 0.f, 0.f};
                f32x4 q0 = *reinterpret_cast<const f32x4 *>(&s_q[li & 7][dq]), q1 = *reinterpret_cast<const f32x4 *>(&s_q[li & 7][dq + 4]);
                q0 = qok ? q0 : zero4;  // selected, not branched around: the reads of both steps go out together
                q1 = qok ? q1 : zero4;
                bf16x8 bhi, blo;
                split_bf16x8(q0, q1, bhi, blo);
                const u32x4 krow = *reinterpret_cast<const u32x4 *>(s_krow + dq);  // meaningful in the owner only
#pragma unroll
                for (int blk = 0; blk < 2; ++blk) {
                    const u32x4 kw = (own && p0 + 16 * blk + li == p) ? krow : kv[blk][s2];
                    bf16x8 av;
                    __builtin_memcpy(&av, &kw, 16);
                    acc[blk] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bhi, acc[blk], 0, 0, 0);
                    acc[blk] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, blo, acc[blk], 0, 0, 0);
                }
            }
        }
        // lane (head = li, g) holds positions 16*blk + 4g + e, e = 0..3
#pragma unroll
        for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int e = 0; e < 4; ++e) s_part[wave][lane][blk * 4 + e] = acc[blk][e];
    }
    __syncthreads();
    {
        // thread -> (head tid/32, position tid%32): its score from the four waves' parts, then the softmax of the slice
        const int h = tid >> 5, i = tid & 31;
        const int src = 16 * ((i & 15) >> 2) + h, idx = (i >> 4) * 4 + (i & 3);
        const float dot = (s_part[0][src][idx] + s_part[1][src][idx]) + (s_part[2][src][idx] + s_part[3][src][idx]);
        const float s = (p0 + i < ctx && h < hq) ? dot * rsqrtf((float)dh) : -INFINITY;
        // over the 32 positions: rotations inside the 16-lane rows (DPP), then one exchange between the two rows
        float mx = s;
        mx = fmaxf(mx, dpp_f32<0x128, 0xF>(mx));  // row_ror:8
        mx = fmaxf(mx, dpp_f32<0x124, 0xF>(mx));  // row_ror:4
        mx = fmaxf(mx, dpp_f32<0x122, 0xF>(mx));  // row_ror:2
        mx = fmaxf(mx, dpp_f32<0x121, 0xF>(mx));  // row_ror:1
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        const float pr = (h < hq) ? __expf(s - mx) : 0.f;
        float sum = pr;
        sum += dpp_f32<0x128, 0xF>(sum);
        sum += dpp_f32<0x124, 0xF>(sum);
        sum += dpp_f32<0x122, 0xF>(sum);
        sum += dpp_f32<0x121, 0xF>(sum);
        sum += __shfl_xor(sum, 16, 64);
        s_sc[h][i] = pr;
        if (i == 0 && h < hq) {
            float *dst = part + ((size_t)blockIdx.x * hq + h) * (dh + 2);
            dst[0] = mx;
            dst[1] = sum;
        }
    }
    __syncthreads();
    // output: 4 column blocks x (hi, lo) = 8 MFMAs per wave
    {
        const f32x4 zero4 = f32x4{0.f, 0.f, 0.f, 0.f};
        f32x4 p0v = *reinterpret_cast<const f32x4 *>(&s_sc[li & 7][8 * g]), p1v = *reinterpret_cast<const f32x4 *>(&s_sc[li & 7][8 * g + 4]);
        p0v = li < 8 ? p0v : zero4;  // rows 8..15 of A are zeros
        p1v = li < 8 ? p1v : zero4;
        bf16x8 ahi, alo;
        split_bf16x8(p0v, p1v, ahi, alo);
        // all the wave's column reads first, then its MFMAs, then its stores behind one condition
        uint32_t bw[4][4];
#pragma unroll
        for (int c4 = 0; c4 < 4; ++c4) {
            const int cb = 4 * wave + c4, col = (FULL || 16 * cb < dh) ? 16 * cb + li : 0;  // past dh: any valid column
#pragma unroll
            for (int e = 0; e < 4; ++e)
                bw[c4][e] = (uint32_t)s_v[8 * g + 2 * e][col] | ((uint32_t)s_v[8 * g + 2 * e + 1][col] << 16);
        }
        f32x4 d[4];
#pragma unroll
        for (int c4 = 0; c4 < 4; ++c4) {
            bf16x8 bv;
            __builtin_memcpy(&bv, bw[c4], 16);
            d[c4] = f32x4{0.f, 0.f, 0.f, 0.f};
            d[c4] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ahi, bv, d[c4], 0, 0, 0);
            d[c4] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(alo, bv, d[c4], 0, 0, 0);
        }
        if (g < 2) {  // heads 4g .. 4g+3 of column 16*cb + li
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4) {
                const int cb = 4 * wave + c4, col = 16 * cb + li;
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (FULL || (16 * cb < dh && 4 * g + e < hq)) part[((size_t)blockIdx.x * hq + 4 * g + e) * (dh + 2) + 2 + col] = d[c4][e];
            }
        }
    }
}

// ---- the combination of the partials folded into the output projection that consumes the attention vector ----
// y_part[h / 2][n] += sum over the 256 k of head h of Wo[n][k] * att[k], Wo int4 group-32 [N, hq*256], att the bf16 attention
// vector attn_mqa_combine_kernel would have written.  A launch less per layer: the combination has no kernel of its own,
// every workgroup of the projection forms the 256 attention values it multiplies with for itself.
//
// What a workgroup costs is what it pulls through its compute unit before it can start: the partials of its head,
// 64 slices * 258 floats = 66 KB per 2048 positions.  Hence one head per workgroup (hq * N/64 workgroups: 256 for a
// 2048-row matrix) and not a pair.  The consumer adds the vectors it is given while it forms its own activation vector,
// and every vector more costs it time, so the two heads of a pair add into one vector by hardware float atomics.  Two
// addends on a cleared accumulator: a + b and b + a are the same float, the result does not depend on who arrives first.
// The attention kernel in front clears the accumulators (attn_mqa_fused_kernel's yz).  y must be ordinary device memory.
//
// Workgroup (h, row block): 16 waves, 64*NL weight rows.
//   1. Wave w takes the slices b = w + 16i of each batch of 64: lane q fetches columns 4q..4q+3 of those 4 slices (the
//      rows of the workspace are 8-byte aligned only, hence the loads of that alignment) and lane b the running maximum
//      and sum of slice b; every wave works out the factors exp(m_b - M) itself.  Batches beyond the first (contexts over
//      2048 positions) are folded in with the usual rescaling.  The workgroup's weight loads - one 8-byte load per lane
//      and 4 rows: lane (r, g2) holds half of a scale group of its row - are issued behind the first batch and land while
//      the combination runs.
//   2. The sixteen slice groups meet in LDS; thread c sums column c, divides, rounds to bf16 and stores it where the dot
//      products want it: 16-byte pieces of 8 k in the pair order of unpack8_magic.
//   3. dot products with v_dot2_f32_bf16 on 128+u, -136 * sum(x) per half group, the group's scale, a sum over the 16
//      lanes of the row.
typedef float f32x4_a8 __attribute__((ext_vector_type(4), aligned(8)));

template <int NL>
__global__ __launch_bounds__(1024) void attn_combine_oproj_kernel(const float *__restrict__ part, const int32_t *__restrict__ pos,
                                                                  const uint8_t *__restrict__ wp, const uint16_t *__restrict__ sc,
                                                                  float *__restrict__ y, int hq, int max_ctx, int N) {
    constexpr int dh = 256;
    const int K = hq * dh, KH = K >> 1, G = K >> 5;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = blockIdx.x, sg = wave;
    const int nbmax = (max_ctx + ATT_CS - 1) / ATT_CS;
    __shared__ __attribute__((aligned(16))) float s_num[16][dh];
    __shared__ __attribute__((aligned(16))) uint8_t s_x[dh * 2];
    __shared__ float s_den;

    const int pos0 = pos[0];  // asked for first: the only load the factors of the first batch wait for besides their own
    const size_t stride = (size_t)hq * (dh + 2);
    const float *ph = part + (size_t)h * (dh + 2);
    const int bl = lane < nbmax ? lane : nbmax - 1;
    const float m0 = ph[(size_t)bl * stride], l0 = ph[(size_t)bl * stride + 1];
    f32x4 pre[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int b = sg + 16 * i;
        pre[i] = *reinterpret_cast<const f32x4_a8 *>(ph + (size_t)(b < nbmax ? b : nbmax - 1) * stride + 2 + 4 * lane);
    }
    const int r = lane >> 4, g2 = lane & 15;
    const int n0 = (blockIdx.y * 16 + wave) * 4 * NL;
    u32x2 w[NL];
    uint16_t sw[NL];
#pragma unroll
    for (int l = 0; l < NL; ++l) {
        const int row = n0 + 4 * l + r, rowc = row < N ? row : N - 1;
        w[l] = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(wp + (size_t)rowc * KH + (size_t)(h * 16 + g2) * 8));
        sw[l] = sc[(size_t)rowc * G + h * 8 + (g2 >> 1)];
    }
    const int ctx = min(max(pos0, 0), max_ctx - 1) + 1, nb = (ctx + ATT_CS - 1) / ATT_CS;
    __builtin_amdgcn_sched_barrier(0);

    float M = wave_max_all(lane < nb ? m0 : -INFINITY);
    const float f0 = lane < nb ? __expf(m0 - M) : 0.f;
    float den = lane < nb ? f0 * l0 : 0.f;
    f32x4 num = {0.f, 0.f, 0.f, 0.f};
    const f32x4 zero4 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        // a slice past the context holds whatever the workspace held: selected away, not multiplied by zero (and not
        // skipped by a branch, which would move its load behind the branch)
        const int b = sg + 16 * i;
        num += lane_value(f0, b) * (b < nb ? pre[i] : zero4);
    }
    for (int base = 64; base < nb; base += 64) {
        const int b = base + lane;
        const bool in = b < nb;
        const float mb = in ? ph[(size_t)b * stride] : -INFINITY, lb = in ? ph[(size_t)b * stride + 1] : 0.f;
        f32x4 pv[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int bb = base + sg + 16 * i;  // uniform over the wave
            pv[i] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (bb < nb) pv[i] = *reinterpret_cast<const f32x4_a8 *>(ph + (size_t)bb * stride + 2 + 4 * lane);
        }
        const float Mn = fmaxf(M, wave_max_all(mb));
        const float rs = __expf(M - Mn), f = in ? __expf(mb - Mn) : 0.f;
        den = den * rs + f * lb;
        num *= rs;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (base + sg + 16 * i < nb) num += lane_value(f, sg + 16 * i) * pv[i];
        M = Mn;
    }
    den = wave_sum_to_lane63(den);
    *reinterpret_cast<f32x4 *>(&s_num[sg][4 * lane]) = num;
    if (sg == 0 && lane == 63) s_den = den;
    __syncthreads();
    if (tid < dh) {
        float t = s_num[0][tid];
#pragma unroll
        for (int s16 = 1; s16 < 16; ++s16) t += s_num[s16][tid];
        const int e = tid & 7;  // piece tid / 8 (8 k, 16 bytes); lane (r, g2) reads pieces 2*g2 and 2*g2 + 1
        *reinterpret_cast<uint16_t *>(s_x + (tid >> 3) * 16 + (e & 3) * 4 + (e >> 2) * 2) = (uint16_t)f32_to_bf16_bits(t / s_den);
    }
    __syncthreads();

    u32x4 xv[2];
    float sumx = 0.f;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
        xv[t] = *reinterpret_cast<const u32x4 *>(s_x + (2 * g2 + t) * 16);
        sumx = dot2_bf16(xv[t].x, 0x3F803F80u, sumx);
        sumx = dot2_bf16(xv[t].y, 0x3F803F80u, sumx);
        sumx = dot2_bf16(xv[t].z, 0x3F803F80u, sumx);
        sumx = dot2_bf16(xv[t].w, 0x3F803F80u, sumx);
    }
    const uint32_t mask_r = vgpr_const(0x000F000Fu), magic_r = vgpr_const(kBf16Magic);
#pragma unroll
    for (int l = 0; l < NL; ++l) {
        const uint32_t ww[2] = {w[l].x, w[l].y};
        float acc = 0.f;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            uint32_t pw[4];
            unpack8_magic_r(ww[t], mask_r, magic_r, pw);
            acc = dot2_bf16(pw[0], xv[t].x, acc);
            acc = dot2_bf16(pw[1], xv[t].y, acc);
            acc = dot2_bf16(pw[2], xv[t].z, acc);
            acc = dot2_bf16(pw[3], xv[t].w, acc);
        }
        float v = f16_bits_to_f32(sw[l]) * (acc - kMagicBias * sumx);
        v += dpp_f32<0x128, 0xF>(v);  // row_ror:8
        v += dpp_f32<0x124, 0xF>(v);  // row_ror:4
        v += dpp_f32<0x122, 0xF>(v);  // row_ror:2
        v += dpp_f32<0x121, 0xF>(v);  // row_ror:1: every lane of the 16-lane row holds the row's sum
        const int row = n0 + 4 * l + r;
        if (g2 == 0 && row < N) unsafeAtomicAdd(&y[(size_t)(h >> 1) * N + row], v);
    }
}

// h = bf16( gelu_tanh(g) * u ), gu = [g(F) | u(F)] fp32
__global__ __launch_bounds__(256) void geglu_kernel(const float *__restrict__ gu, uint16_t *__restrict__ h, int F) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < F) {
        h[i] = (uint16_t)f32_to_bf16_bits(gelu_tanh_dev(gu[i]) * gu[F + i]);
    }
}

// argmax over n fp32 values (lowest index wins ties, NaN is never the winner; token 0 if every value is NaN):
// per-workgroup candidates, then one workgroup; the winner becomes the next token and the position advances, so that
// a replayed graph steps by itself.  A thread keeps the best of its elements (loads four at a time), a wave finds its
// winner with DPP moves and a ballot, and the four waves meet once in LDS.
__device__ __forceinline__ void argmax_block(float best, int bi, float *out_v, int32_t *out_i) {
    __shared__ float s_v[4];
    __shared__ int32_t s_i[4];
    const int wave = threadIdx.x >> 6;
    const uint32_t gi = wave_winner<64>(bi != INT_MAX, best, bi);
    if (gi == 0xFFFFFFFFu) {
        if ((threadIdx.x & 63) == 0) {
            s_v[wave] = -INFINITY;
            s_i[wave] = INT_MAX;
        }
    } else if ((uint32_t)bi == gi) {  // one lane: indices are distinct
        s_v[wave] = best;
        s_i[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float bv = s_v[0];
        int bb = s_i[0];
#pragma unroll
        for (int w = 1; w < 4; ++w)
            if (s_i[w] != INT_MAX && (bb == INT_MAX || s_v[w] > bv || (s_v[w] == bv && s_i[w] < bb))) {
                bv = s_v[w];
                bb = s_i[w];
            }
        *out_v = bv;
        *out_i = bb;
    }
}

__global__ __launch_bounds__(256) void argmax_partial_kernel(const float *__restrict__ v, int n, float *__restrict__ pv,
                                                             int32_t *__restrict__ pi) {
    float best = -INFINITY;
    int bi = INT_MAX;
    const int stride = gridDim.x * blockDim.x;
    for (int i0 = blockIdx.x * blockDim.x + threadIdx.x; i0 < n; i0 += 4 * stride) {
        float x[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) x[j] = (i0 + j * stride < n) ? v[i0 + j * stride] : __builtin_nanf("");
#pragma unroll
        for (int j = 0; j < 4; ++j)  // increasing index: an equal value later never replaces an earlier one
            if (x[j] > best || (x[j] == best && bi == INT_MAX)) {
                best = x[j];
                bi = i0 + j * stride;
            }
    }
    argmax_block(best, bi, pv + blockIdx.x, pi + blockIdx.x);
}

// ex != nullptr: the winner's row of the tied int4 table [n, d] is also written to ex as embed_i4g32_kernel would write
// it - the residual vector the next decode step starts from, without a launch of its own.
__global__ __launch_bounds__(256) void argmax_final_kernel(const float *__restrict__ pv, const int32_t *__restrict__ pi, int nb, int n,
                                                           int32_t *__restrict__ token, int32_t *__restrict__ pos,
                                                           int advance, const uint8_t *__restrict__ ewp,
                                                           const uint16_t *__restrict__ esc, float *__restrict__ ex, int d) {
    __shared__ float fv;
    __shared__ int32_t fi;
    float best = -INFINITY;
    int bi = INT_MAX;
    for (int i0 = threadIdx.x; i0 < nb; i0 += 16 * 256) {  // 16 candidates in flight per thread: one workgroup reads them all
        float x[16];
        int xi[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int i = i0 + 256 * j;
            x[j] = pv[i < nb ? i : 0];
            xi[j] = i < nb ? pi[i] : INT_MAX;
        }
#pragma unroll
        for (int j = 0; j < 16; ++j)
            if (xi[j] != INT_MAX && (bi == INT_MAX || x[j] > best || (x[j] == best && xi[j] < bi))) {
                best = x[j];
                bi = xi[j];
            }
    }
    argmax_block(best, bi, &fv, &fi);
    if (threadIdx.x == 0) {
        token[0] = (fi == INT_MAX) ? 0 : min(max(fi, 0), n - 1);
        if (advance) pos[0] += 1;
    }
    if (ex) {
        __syncthreads();  // fi, written by the first thread
        embed_row((fi == INT_MAX) ? 0 : min(max(fi, 0), n - 1), ewp, esc, ex, d);
    }
}

int embed_launch(const int32_t *token, const uint8_t *wp, const uint16_t *sc, float *x, int d, int V, hipStream_t st) {
    hipLaunchKernelGGL(embed_i4g32_kernel, dim3(1), dim3(256), 0, st, token, wp, sc, x, d, V);
    return hip_check(hipGetLastError(), "embed launch");
}

template <int NV>
static void add_rmsnorm_vec_launch(float *res, const float *delta, int nd, const float *w, uint16_t *y, int d, float eps,
                                   hipStream_t st) {
    switch (nd) {
        case 0: hipLaunchKernelGGL((add_rmsnorm_vec_kernel<NV, 0>), dim3(1), dim3(256), 0, st, res, delta, w, y, d, eps); break;
        case 1: hipLaunchKernelGGL((add_rmsnorm_vec_kernel<NV, 1>), dim3(1), dim3(256), 0, st, res, delta, w, y, d, eps); break;
        case 2: hipLaunchKernelGGL((add_rmsnorm_vec_kernel<NV, 2>), dim3(1), dim3(256), 0, st, res, delta, w, y, d, eps); break;
        default: hipLaunchKernelGGL((add_rmsnorm_vec_kernel<NV, 4>), dim3(1), dim3(256), 0, st, res, delta, w, y, d, eps); break;
    }
}

int add_rmsnorm_launch(float *res, const float *delta, int nd, const float *w, uint16_t *y, int d, float eps, hipStream_t st) {
    const bool vec = (d % 4 == 0) && d <= 4096 && (nd == 0 || nd == 1 || nd == 2 || nd == 4) &&
                     ((reinterpret_cast<uintptr_t>(res) | reinterpret_cast<uintptr_t>(delta) | reinterpret_cast<uintptr_t>(w)) & 15u) == 0 &&
                     (reinterpret_cast<uintptr_t>(y) & 7u) == 0;
    if (!vec)
        hipLaunchKernelGGL(add_rmsnorm_kernel, dim3(1), dim3(256), 0, st, res, delta, nd, w, y, d, eps);
    else if (d <= 2048)
        add_rmsnorm_vec_launch<2>(res, delta, nd, w, y, d, eps, st);
    else
        add_rmsnorm_vec_launch<4>(res, delta, nd, w, y, d, eps, st);
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
    hipLaunchKernelGGL(attn_mqa_combine_kernel, dim3(hq, (dh + 63) / 64), dim3(256), 0, st, part, pos, out, hq, dh, max_ctx);
    return hip_check(hipGetLastError(), "attn_mqa launch");
}

int rope_table_launch(float *table, int dh, int max_ctx, float base, hipStream_t st) {
    const int64_t n = (int64_t)max_ctx * (dh / 2);
    hipLaunchKernelGGL(rope_table_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, table, dh, max_ctx, base);
    return hip_check(hipGetLastError(), "rope_table launch");
}

int attn_mqa_fused_launch(const float *qkv, const int32_t *pos, const float *table, uint16_t *kc, uint16_t *vc, float *ws,
                          uint16_t *out, int hq, int dh, int max_ctx, hipStream_t st) {
    const int nb = (max_ctx + ATT_CS - 1) / ATT_CS;
    if (hq == 8 && dh == 256 && max_ctx <= 8192)
        hipLaunchKernelGGL(attn_mqa_fused_kernel<true>, dim3(nb), dim3(256), 0, st, qkv, pos, table, kc, vc, ws, max_ctx, hq, dh, (float *)nullptr, 0);
    else
        hipLaunchKernelGGL(attn_mqa_fused_kernel<false>, dim3(nb), dim3(256), 0, st, qkv, pos, table, kc, vc, ws, max_ctx, hq, dh, (float *)nullptr, 0);
    hipLaunchKernelGGL(attn_mqa_combine_kernel, dim3(hq, (dh + 63) / 64), dim3(256), 0, st, ws, pos, out, hq, dh, max_ctx);
    return hip_check(hipGetLastError(), "attn_mqa_fused launch");
}

// The fused attention with its combination folded into the output projection: two launches for what were three
// (partials, combination, projection).  y receives hq/2 partial vectors of N floats.
bool attn_mqa_fused_oproj_ok(int hq, int dh) { return dh == 256 && hq >= 2 && hq <= 8 && hq % 2 == 0; }

int attn_mqa_fused_oproj_launch(const float *qkv, const int32_t *pos, const float *table, uint16_t *kc, uint16_t *vc, float *ws,
                                const uint8_t *wp, const uint16_t *sc, float *y, int hq, int dh, int max_ctx, int N, hipStream_t st) {
    const int nb = (max_ctx + ATT_CS - 1) / ATT_CS;
    if (hq == 8 && max_ctx <= 8192)  // dh = 256 here
        hipLaunchKernelGGL(attn_mqa_fused_kernel<true>, dim3(nb), dim3(256), 0, st, qkv, pos, table, kc, vc, ws, max_ctx, hq, dh, y, (hq / 2) * N);
    else
        hipLaunchKernelGGL(attn_mqa_fused_kernel<false>, dim3(nb), dim3(256), 0, st, qkv, pos, table, kc, vc, ws, max_ctx, hq, dh, y, (hq / 2) * N);
    // 64 rows per workgroup up to 4096 rows (hq * N/64 workgroups: 256 for a 2048-row matrix), 128 beyond
    if (N <= 4096)
        hipLaunchKernelGGL((attn_combine_oproj_kernel<1>), dim3(hq, (N + 63) / 64), dim3(1024), 0, st, ws, pos, wp, sc, y, hq, max_ctx, N);
    else
        hipLaunchKernelGGL((attn_combine_oproj_kernel<2>), dim3(hq, (N + 127) / 128), dim3(1024), 0, st, ws, pos, wp, sc, y, hq, max_ctx, N);
    return hip_check(hipGetLastError(), "attn_mqa_fused_oproj launch");
}

// ---- the fused attention without a caller-supplied workspace ---------------------------------------------------
// The split-context partials (32 positions per slice: running maximum, sum and dh weighted columns per head) go to a
// file-scope device array instead: 256 slices (a cache of up to 8192 rows) x 8 heads x (256 + 2) floats = 2,113,536
// bytes, held by every GPU the library runs on until the process ends.  In host code the array's name is only a
// stand-in for the symbol; its address on a device comes from hipGetSymbolAddress, asked once per device - by the first
// call of any entry point on that device, so never under graph capture - and kept.
// Nothing in the array has to start at zero: a call writes the slices 0 .. pos/32 before the combine kernel reads
// exactly those.  Calls that overlap on one GPU (two streams) would share the array and race.
constexpr int ATT_STATIC_MAX_CTX = 8192;
constexpr size_t ATT_STATIC_FLOATS = (size_t)(ATT_STATIC_MAX_CTX / ATT_CS) * 8 * (256 + 2);
static __device__ __align__(256) float scratch[ATT_STATIC_FLOATS];
static std::atomic<float *> g_scratch_ptr[64];  // per device; zero-initialised

int attn_mqa_fused_static_max_ctx() { return ATT_STATIC_MAX_CTX; }

// Called once per device, from the first entry-point call made on it (api.hip, check_device), with that device current.
int attn_mqa_fused_static_init(int dev) {
    if (dev < 0 || dev >= 64) return 0;  // such a device gets no scratch; the entry point refuses it
    if (g_scratch_ptr[dev].load(std::memory_order_acquire)) return 0;
    float *ptr = nullptr;
    CHADQ_HIP(hipGetSymbolAddress(reinterpret_cast<void **>(&ptr), HIP_SYMBOL(scratch)));
    CHADQ_REQUIRE(ptr != nullptr, CHADQ_ERR_HIP, "hipGetSymbolAddress returned a null address for the attention scratch");
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // two threads racing here obtain the same address
    return 0;
}

int attn_mqa_fused_static_launch(const float *qkv, const int32_t *pos, const float *table, uint16_t *kc, uint16_t *vc,
                                 uint16_t *out, int hq, int dh, int max_ctx, hipStream_t st) {
    int dev = 0;
    CHADQ_HIP(hipGetDevice(&dev));
    CHADQ_REQUIRE(dev >= 0 && dev < 64, CHADQ_ERR_DEVICE, "attention without workspace: device index %d is not below 64", dev);
    float *ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);  // set by the device's first entry-point call
    CHADQ_REQUIRE(ptr != nullptr, CHADQ_ERR_HIP, "attention without workspace: the scratch address of device %d was not resolved", dev);
    if ((size_t)((max_ctx + ATT_CS - 1) / ATT_CS) * hq * (dh + 2) > ATT_STATIC_FLOATS)
        return fail(CHADQ_ERR_WORKSPACE, "attention without workspace: hq=%d dh=%d max_ctx=%d needs more than the %zu-float scratch", hq, dh,
                    max_ctx, ATT_STATIC_FLOATS);
    return attn_mqa_fused_launch(qkv, pos, table, kc, vc, ptr, out, hq, dh, max_ctx, st);
}

int geglu_launch(const float *gu, uint16_t *h, int F, hipStream_t st) {
    hipLaunchKernelGGL(geglu_kernel, dim3((F + 255) / 256), dim3(256), 0, st, gu, h, F);
    return hip_check(hipGetLastError(), "geglu launch");
}

int argmax_launch(const float *v, int n, float *pv, int32_t *pi, int32_t *token, int32_t *pos, int advance, hipStream_t st) {
    const int nb = 256;
    hipLaunchKernelGGL(argmax_partial_kernel, dim3(nb), dim3(256), 0, st, v, n, pv, pi);
    hipLaunchKernelGGL(argmax_final_kernel, dim3(1), dim3(256), 0, st, pv, pi, nb, n, token, pos, advance, (const uint8_t *)nullptr,
                       (const uint16_t *)nullptr, (float *)nullptr, 0);
    return hip_check(hipGetLastError(), "argmax launch");
}

// The second stage alone, over nb candidates some other kernel left (or, partial = true, both stages over the n values v),
// with the winner's table row written to ex (ex = nullptr: not).
int argmax_embed_launch(const float *v, bool partial, float *pv, int32_t *pi, int nb, int n, int32_t *token, int32_t *pos, int advance,
                        const uint8_t *ewp, const uint16_t *esc, float *ex, int d, hipStream_t st) {
    if (partial) {
        nb = 256;
        hipLaunchKernelGGL(argmax_partial_kernel, dim3(nb), dim3(256), 0, st, v, n, pv, pi);
    }
    hipLaunchKernelGGL(argmax_final_kernel, dim3(1), dim3(256), 0, st, pv, pi, nb, n, token, pos, advance, ewp, esc, ex, d);
    return hip_check(hipGetLastError(), "argmax launch");
}

}  // namespace chadq
