// Decode GEMV on int4 group-32 weights:  y[m,n] = sum_g s[n,g] * sum_{k in g} x[m,k] * (u[n,k]-8).
//
// HBM-bound.  A wavefront owns whole output rows.  One 128-bit load per lane brings 32 nibbles = exactly
// one scale group, so a wave-wide load covers 2048 consecutive k of one row (1 KiB contiguous) and the
// matching scale load is 128 contiguous bytes.  All weight loads of a wave are issued before any
// arithmetic; the activations (a few KiB, shared by every row) are fetched and rearranged while those
// loads are in flight and then live in registers.
//
// Arithmetic per group: nibbles become bf16 128+u by OR-ing them into a magic constant (7 integer ops per
// 8 nibbles), v_dot2_f32_bf16 accumulates x*(128+u) in fp32 starting from -136*sum(x) (which turns 128+u
// into u-8), and one fp32 FMA applies the group scale.  Every product and the bias term are exact in
// fp32 for integer-valued x, so integer accumulation is bit-exact.  The 64 partial sums of a row are
// folded with DPP adds; no LDS is used.
#include "chadq_common.h"

namespace chadq {

// CH: 2048-wide k chunks per row held by one wave (K <= CH*2048).  R: rows per wave.  MB: activation rows.
template <int CH, int R, int MB>
__global__ __launch_bounds__(256) void gemv_i4g32_rows_kernel(const uint16_t *__restrict__ x,
                                                              const uint8_t *__restrict__ wp,
                                                              const uint16_t *__restrict__ sc,
                                                              float *__restrict__ y, int N, int K) {
    const int lane = threadIdx.x & 63;
    const int gw = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int row0 = gw * R;
    if (row0 >= N) return;
    const int KH = K >> 1, G = K >> 5;

    // 1. activation loads first.  Memory returns in order, so a wait for the activations must not sit
    //    behind the weight stream issued next.
    u32x4 xv[MB][CH][4];
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int k0 = c * 2048 + lane * 32;
            const u32x4 *xp = reinterpret_cast<const u32x4 *>(x + (size_t)m * K + (k0 < K ? k0 : 0));
#pragma unroll
            for (int i = 0; i < 4; ++i) xv[m][c][i] = xp[i];
        }

    // 2. every weight and scale load of this wave.  Loads are unconditional (a predicated load becomes a
    //    branch with its own wait and serialises the stream): out-of-range rows and k positions read a
    //    clamped, valid address and are neutralised through a zero activation / zero scale below.
    u32x4 w[R][CH];
    uint32_t s16[R][CH];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int row = (row0 + r < N) ? row0 + r : N - 1;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int k0 = c * 2048 + lane * 32;
            const int kc = (k0 < K) ? k0 : 0;
            w[r][c] = load_nt_b128(wp + (size_t)row * KH + (kc >> 1));
            const uint32_t sv = __builtin_nontemporal_load(sc + (size_t)row * G + (kc >> 5));
            s16[r][c] = (k0 < K) ? sv : 0u;
        }
    }
    __builtin_amdgcn_sched_barrier(0);  // every load above is issued before anything below may wait

    // activations of this lane's groups, paired to match the unpack order; bias = -136 * sum(x)
    uint32_t xs[MB][CH][16];
    float bias[MB][CH];
#pragma unroll
    for (int m = 0; m < MB; ++m) {
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const bool ok = (c * 2048 + lane * 32) < K;
            float sum = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                u32x4 v = xv[m][c][i];
                if (!ok) v = u32x4{0, 0, 0, 0};
                uint32_t a[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) sum = dot2_bf16(a[j], 0x3F803F80u, sum);  // (1.0, 1.0)
                pair_x8(a, &xs[m][c][i * 4]);
            }
            bias[m][c] = -kMagicBias * sum;
        }
    }

    // 3. rows in load order
    const uint32_t mask_r = vgpr_const(0x000F000Fu), magic_r = vgpr_const(kBf16Magic);
#pragma unroll
    for (int r = 0; r < R; ++r) {
        float acc[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[m] = 0.f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            uint32_t p[16];
            unpack8_magic_r(w[r][c].x, mask_r, magic_r, &p[0]);
            unpack8_magic_r(w[r][c].y, mask_r, magic_r, &p[4]);
            unpack8_magic_r(w[r][c].z, mask_r, magic_r, &p[8]);
            unpack8_magic_r(w[r][c].w, mask_r, magic_r, &p[12]);
            const float s = f16_bits_to_f32((uint16_t)s16[r][c]);
#pragma unroll
            for (int m = 0; m < MB; ++m) {
                float g = bias[m][c];
#pragma unroll
                for (int i = 0; i < 16; ++i) g = dot2_bf16(p[i], xs[m][c][i], g);
                acc[m] = __builtin_fmaf(s, g, acc[m]);
            }
        }
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const float t = wave_sum_to_lane63(acc[m]);
            if (lane == 63 && row0 + r < N) y[(size_t)m * N + row0 + r] = t;
        }
    }
}

// Any K % 32 == 0 and any M: one wave per row, chunks of 2048 k streamed in a loop, activations re-read
// from cache for every row.  Correct everywhere, fast nowhere; used for shapes the tuned kernels decline.
__global__ __launch_bounds__(256) void gemv_i4g32_generic_kernel(const uint16_t *__restrict__ x,
                                                                 const uint8_t *__restrict__ wp,
                                                                 const uint16_t *__restrict__ sc,
                                                                 float *__restrict__ y, int M, int N, int K) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= N) return;
    const int KH = K >> 1, G = K >> 5;
    for (int m = 0; m < M; ++m) {
        float acc = 0.f;
        for (int k0 = lane * 32; k0 < K; k0 += 2048) {
            const u32x4 wv = *reinterpret_cast<const u32x4 *>(wp + (size_t)row * KH + (k0 >> 1));
            const float s = f16_bits_to_f32(sc[(size_t)row * G + (k0 >> 5)]);
            const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
            const u32x4 *xp = reinterpret_cast<const u32x4 *>(x + (size_t)m * K + k0);
            float sum = 0.f, g = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const u32x4 v = xp[i];
                uint32_t a[4] = {v.x, v.y, v.z, v.w}, xq[4], p[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) sum = dot2_bf16(a[j], 0x3F803F80u, sum);
                pair_x8(a, xq);
                unpack8_magic(ww[i], p);
#pragma unroll
                for (int j = 0; j < 4; ++j) g = dot2_bf16(p[j], xq[j], g);
            }
            acc = __builtin_fmaf(s, g - kMagicBias * sum, acc);
        }
        const float t = wave_sum_to_lane63(acc);
        if (lane == 63) y[(size_t)m * N + row] = t;
    }
}

template <int CH, int R, int MB>
static void launch_rows(const uint16_t *x, const uint8_t *wp, const uint16_t *sc, float *y, int N, int K,
                        hipStream_t st) {
    const int waves = (N + R - 1) / R;
    hipLaunchKernelGGL((gemv_i4g32_rows_kernel<CH, R, MB>), dim3((waves + 3) / 4), dim3(256), 0, st, x, wp, sc, y, N, K);
}

int gemv_i4g32_dispatch(const uint16_t *x, const uint8_t *wp, const uint16_t *sc, float *y, int M, int N, int K,
                        hipStream_t st) {
    if (K <= 4096) {
        // rows per wave: enough waves to fill 256 CUs several times over, few enough to keep loads deep
        const bool big = N >= 8192;
        int m0 = 0;
        while (m0 < M) {
            const uint16_t *xm = x + (size_t)m0 * K;
            float *ym = y + (size_t)m0 * N;
            const int mb = (M - m0 >= 2) ? 2 : 1;
            if (K <= 2048) {
                if (mb == 2) big ? launch_rows<1, 8, 2>(xm, wp, sc, ym, N, K, st) : launch_rows<1, 2, 2>(xm, wp, sc, ym, N, K, st);
                else big ? launch_rows<1, 8, 1>(xm, wp, sc, ym, N, K, st) : launch_rows<1, 2, 1>(xm, wp, sc, ym, N, K, st);
            } else {
                if (mb == 2) big ? launch_rows<2, 4, 2>(xm, wp, sc, ym, N, K, st) : launch_rows<2, 1, 2>(xm, wp, sc, ym, N, K, st);
                else big ? launch_rows<2, 4, 1>(xm, wp, sc, ym, N, K, st) : launch_rows<2, 1, 1>(xm, wp, sc, ym, N, K, st);
            }
            m0 += mb;
        }
    } else {
        hipLaunchKernelGGL(gemv_i4g32_generic_kernel, dim3((N + 3) / 4), dim3(256), 0, st, x, wp, sc, y, M, N, K);
    }
    return hip_check(hipGetLastError(), "gemv_i4g32 launch");
}

}  // namespace chadq
