// Decode GEMV on int8 weights with one fp32 scale per output row:  y[m,n] = s[n] * sum_k x[m,k] * W[n,k].
//
// HBM-bound stream of W.  A wavefront owns whole rows; one 128-bit load per lane = 16 weights, a wave-wide
// load = 1024 consecutive k (1 KiB contiguous).  All loads of a wave are issued first; the fp32 activations
// come once per workgroup, through LDS, and a lane's k positions stay in registers.  A signed byte becomes a float in one
// instruction (v_cvt_f32_i32 with a sign-extending byte select), so every product is x[k] * float(W[n,k]) itself: an
// activation's error does not depend on its neighbours (flipping the bytes to unsigned for v_cvt_f32_ubyteN and taking
// 128 * sum(x) back out costs the same and does depend on them).  DPP adds fold the 64 partial sums; no LDS.
#include "chadq_common.h"

namespace chadq {

__device__ __forceinline__ float sbyte_to_f32(uint32_t v, int i) { return (float)(int)(int8_t)(v >> (8 * i)); }

template <int CH, int R, int MB, int WPB>
__global__ __launch_bounds__(64 * WPB) void gemv_i8row_rows_kernel(const float *__restrict__ x,
                                                              const int8_t *__restrict__ w8,
                                                              const float *__restrict__ sc, float *__restrict__ y,
                                                              int N, int K) {
    const int lane = threadIdx.x & 63;
    const int gw = blockIdx.x * WPB + (threadIdx.x >> 6);
    const int row0 = gw * R;  // waves past the last row run on clamped rows and store nothing (no return before the barrier)

    // Activation loads first (memory returns in order, so waiting for them must not sit behind the weights): the
    // workgroup fetches each activation once, CH 16-byte pieces per thread and row, and shares it through LDS -
    // a quarter of the requests of every wave fetching its own copy.  Piece q (4 floats) lives at slot
    // q ^ ((q >> 4) & 3), which makes the read-back below (lane l reads pieces 4l .. 4l+3) free of bank conflicts.
    __shared__ __attribute__((aligned(16))) float sx[MB][CH * 1024];
    constexpr int T = 64 * WPB, XP = (CH * 256 + T - 1) / T;  // threads, pieces per thread and row
    f32x4 xg[MB][XP];
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int c = 0; c < XP; ++c) {
            const int k0 = (c * T + (int)threadIdx.x) * 4;
            xg[m][c] = *reinterpret_cast<const f32x4 *>(x + (size_t)m * K + ((k0 < K) ? k0 : 0));
        }

    u32x4 w[R][CH];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        // unconditional loads from clamped addresses; out-of-range k meets a zero activation below
        const int row = (row0 + r < N) ? row0 + r : N - 1;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int k0 = c * 1024 + lane * 16;
            w[r][c] = load_nt_b128(w8 + (size_t)row * K + ((k0 < K) ? k0 : 0));
        }
    }
    __builtin_amdgcn_sched_barrier(0);  // every load above is issued before anything below may wait

#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int c = 0; c < XP; ++c) {
            const int q = c * T + (int)threadIdx.x;
            f32x4 v = xg[m][c];
            if (q * 4 >= K) v = f32x4{0.f, 0.f, 0.f, 0.f};
            if (q < CH * 256) *reinterpret_cast<f32x4 *>(&sx[m][(q ^ ((q >> 4) & 3)) * 4]) = v;
        }
    __syncthreads();
    float xs[MB][CH][16];
#pragma unroll
    for (int m = 0; m < MB; ++m) {
#pragma unroll
        for (int c = 0; c < CH; ++c) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int q = c * 256 + lane * 4 + i;
                const f32x4 v = *reinterpret_cast<const f32x4 *>(&sx[m][(q ^ ((q >> 4) & 3)) * 4]);
                xs[m][c][4 * i + 0] = v.x;
                xs[m][c][4 * i + 1] = v.y;
                xs[m][c][4 * i + 2] = v.z;
                xs[m][c][4 * i + 3] = v.w;
            }
        }
    }

#pragma unroll
    for (int r = 0; r < R; ++r) {
        float acc[MB];
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[m] = 0.f;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const uint32_t ww[4] = {w[r][c].x, w[r][c].y, w[r][c].z, w[r][c].w};
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float f = sbyte_to_f32(ww[j], i);
#pragma unroll
                    for (int m = 0; m < MB; ++m) acc[m] = __builtin_fmaf(xs[m][c][4 * j + i], f, acc[m]);
                }
        }
        const int row = row0 + r;
        const float s = (row < N) ? sc[row] : 0.f;
#pragma unroll
        for (int m = 0; m < MB; ++m) {
            const float t = wave_sum_to_lane63(acc[m]);
            if (lane == 63 && row < N) y[(size_t)m * N + row] = t * s;
        }
    }
}

// Any K % 16 == 0 and any M; one wave per row, 1024-wide chunks streamed in a loop.
__global__ __launch_bounds__(256) void gemv_i8row_generic_kernel(const float *__restrict__ x,
                                                                 const int8_t *__restrict__ w8,
                                                                 const float *__restrict__ sc,
                                                                 float *__restrict__ y, int M, int N, int K) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= N) return;
    const float s = sc[row];
    for (int m = 0; m < M; ++m) {
        float acc = 0.f;
        for (int k0 = lane * 16; k0 < K; k0 += 1024) {
            const u32x4 wv = *reinterpret_cast<const u32x4 *>(w8 + (size_t)row * K + k0);
            const uint32_t ww[4] = {wv.x, wv.y, wv.z, wv.w};
            const f32x4 *xp = reinterpret_cast<const f32x4 *>(x + (size_t)m * K + k0);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f32x4 v = xp[j];
                acc = __builtin_fmaf(v.x, sbyte_to_f32(ww[j], 0), acc);
                acc = __builtin_fmaf(v.y, sbyte_to_f32(ww[j], 1), acc);
                acc = __builtin_fmaf(v.z, sbyte_to_f32(ww[j], 2), acc);
                acc = __builtin_fmaf(v.w, sbyte_to_f32(ww[j], 3), acc);
            }
        }
        const float t = wave_sum_to_lane63(acc);
        if (lane == 63) y[(size_t)m * N + row] = t * s;
    }
}

template <int CH, int R, int MB, int WPB>
static void launch_rows8(const float *x, const int8_t *w8, const float *sc, float *y, int N, int K, hipStream_t st) {
    const int waves = (N + R - 1) / R;
    hipLaunchKernelGGL((gemv_i8row_rows_kernel<CH, R, MB, WPB>), dim3((waves + WPB - 1) / WPB), dim3(64 * WPB), 0, st, x, w8, sc, y,
                       N, K);
}

bool gemv_i8row_mfma_ok(int M, int K);
int gemv_i8row_mfma_launch(const float *, const int8_t *, const float *, float *, int, int, int, hipStream_t);

// fp32_only: the fp32 kernels for every K (chadq_gemv_i8row_fp32)
int gemv_i8row_dispatch(const float *x, const int8_t *w8, const float *sc, float *y, int M, int N, int K, bool fp32_only,
                        hipStream_t st) {
    // K a multiple of 128: the int8 matrix core, one pass over W for all M (gemv_i8row_mfma.hip); the fp32 kernels
    // below keep the other row lengths
    if (!fp32_only && N > 0 && gemv_i8row_mfma_ok(M, K)) return gemv_i8row_mfma_launch(x, w8, sc, y, M, N, K, st);
    // <1024-wide chunks per row, rows per wave, activation rows, waves per workgroup>, picked by measurement: eight
    // waves share one copy of the activations; matrices with many rows give a wave 2 or 4 rows
    if (K <= 2048) {
        const bool big = N >= 8192;
        for (int m0 = 0; m0 < M;) {
            const float *xm = x + (size_t)m0 * K;
            float *ym = y + (size_t)m0 * N;
            const int mb = (M - m0 >= 2) ? 2 : 1;
            if (K <= 1024) {
                if (mb == 2) big ? launch_rows8<1, 4, 2, 8>(xm, w8, sc, ym, N, K, st) : launch_rows8<1, 2, 2, 8>(xm, w8, sc, ym, N, K, st);
                else big ? launch_rows8<1, 4, 1, 8>(xm, w8, sc, ym, N, K, st) : launch_rows8<1, 2, 1, 8>(xm, w8, sc, ym, N, K, st);
            } else {
                if (mb == 2) big ? launch_rows8<2, 2, 2, 8>(xm, w8, sc, ym, N, K, st) : launch_rows8<2, 1, 2, 8>(xm, w8, sc, ym, N, K, st);
                else big ? launch_rows8<2, 2, 1, 8>(xm, w8, sc, ym, N, K, st) : launch_rows8<2, 1, 1, 8>(xm, w8, sc, ym, N, K, st);
            }
            m0 += mb;
        }
    } else if (K <= 8192) {  // rows of up to 4096 / 8192 k: the same kernel with 4 or 8 chunks per row, one activation row at a time
        for (int m0 = 0; m0 < M; ++m0) {
            const float *xm = x + (size_t)m0 * K;
            float *ym = y + (size_t)m0 * N;
            if (K <= 4096) N >= 4096 ? launch_rows8<4, 2, 1, 8>(xm, w8, sc, ym, N, K, st) : launch_rows8<4, 1, 1, 8>(xm, w8, sc, ym, N, K, st);
            else launch_rows8<8, 1, 1, 8>(xm, w8, sc, ym, N, K, st);
        }
    } else {
        hipLaunchKernelGGL(gemv_i8row_generic_kernel, dim3((N + 3) / 4), dim3(256), 0, st, x, w8, sc, y, M, N, K);
    }
    return hip_check(hipGetLastError(), "gemv_i8row launch");
}

}  // namespace chadq
