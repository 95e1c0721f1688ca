// Decode GEMV on int8 per-row weights on the int8 matrix core, any 1..16 activation rows in ONE pass over W (the
// per-row kernel in gemv_i8row.hip streams W once per pair of activation rows).
//
// v_mfma_i32_16x16x64_i8 takes the stored weight bytes as they are, so the K loop has no conversion work at all.
// The fp32 activations are what has to change shape: per activation row and per 2048 k, x is written in fixed point
// with a power-of-two scale, X = rint(x * 2^(20 - e)) with 2^e <= max|x| < 2^(e+1) (|X| <= 2^21), and X as three
// balanced base-256 digits, X = a0 * 2^16 + a1 * 2^8 + a2 with -128 <= a <= 127.  Each digit is one int8 operand
// row; the three int32 dot products are exact and meet again in fp32: y = s[n] * sum over blocks 2^(e-20) * (D0 *
// 2^16 + D1 * 2^8 + D2).  What is dropped is at most 2^-21 of the block's largest |x| per element, so a result is off by
// at most scale[n] * sum over blocks of 2^-21 * max_block|x| * sum_{k in block} |W[n,k]| (the result is held to a 1e-3
// relative tolerance; one outlier among the activations costs the small elements of its block their low bits, also
// in rows whose weight at the outlier is zero: chadq_gemv_i8row_fp32 is the form without this).  Integer-valued
// activations below 2^20 are represented exactly and the three digit sums are recombined exactly (in float64), so
// integer sums below 2^24 are exact as in the per-row kernel.  A block with a non-finite activation makes its rows'
// results NaN (the fp32 kernels follow IEEE arithmetic element by element).
//
// One MFMA, D[16x16] += A[16x64] * B[64x16]:
//   B = weights.  Column c is weight row n0 + c (16 rows per wave); lane (c, g = lane/16) supplies 16 k-slots.  A
//       wave fetches 128 k of its 16 rows with two loads of 8 rows x 128 B (lane (c, g) loads piece (c >> 3) + 2g of
//       row c & 7, then of row 8 + (c & 7)); two DPP half-row rotations per word hand every lane the 32 consecutive
//       bytes k = 32g .. 32g + 31 of ITS row c: the B operands of two MFMAs.
//   A = activations.  SETS <= 2 (M <= 4, M <= 8): operand row 4q + d of set s is digit d of activation row 4s + q
//       (row 4q + 3 is zero), so the three digit sums of a result sit in one lane's accumulator registers.  SETS = 3
//       (M <= 16): set d holds digit d of all 16 rows.
// Workgroup = 8 waves on 64 weight rows: wave (rw, kh) multiplies rows 16 rw .. 16 rw + 15 with the kh-th 1024 k of
// every 2048, so at K <= 2048 a wave's 16 loads - all of its weights - are in flight from the start and nothing
// about the activations can stall the stream.  The 512 threads turn 2048 k of all M activation rows into operand
// order in LDS (SETS x 32 KiB); the activation loads are issued before the weight loads because memory returns in
// order.  Longer rows repeat this per 2048 k with the ring refilled as it is consumed (every load unconditional:
// addresses past the end are clamped and their activations staged as zeros).  The two K halves meet in LDS at the end.
#include <type_traits>

#include "chadq_common.h"

namespace chadq {

typedef __attribute__((ext_vector_type(4))) int i32x4;

template <int SETS>
struct GemvI8Cfg {
    static constexpr int PAIRS = 8;                       // 128-k pair-steps per wave and round (1024 k)
    static constexpr int PAIR_BYTES = SETS * 2048;        // A operands of one pair-step: SETS x 2 MFMAs x 1 KiB
    static constexpr int BUF_BYTES = PAIRS * PAIR_BYTES;  // one round's operands: SETS x 16 KiB
    static constexpr int MROWS = SETS == 3 ? 16 : 4 * SETS;  // activation rows the staging covers
    static constexpr int PARTS = 512 / MROWS;             // staging threads per activation row
    static constexpr int XIT = 128 / PARTS;               // 16-k pieces a thread stages per 2048 k: 1 / 2 / 4
    static constexpr int RES = SETS == 3 ? 4 : SETS;      // results per lane
    static constexpr int AMAX_OFF = 2 * BUF_BYTES;        // [MROWS][8 waves] largest |x| bits
    static constexpr int FOLD_OFF = AMAX_OFF + 16 * 8 * 4;  // [4 row blocks][64 lanes] x 16 B from the upper K half
    static constexpr int LDS = FOLD_OFF + 4 * 64 * 16;
};

// lanes 8..15 of every row of 16 take src from the lane 8 below, lanes 0..7 keep old (BANKS = 0xC); or lanes 0..7 take
// src from the lane 8 above and lanes 8..15 keep old (BANKS = 0x3)
template <int BANKS>
__device__ __forceinline__ int half_row_merge(uint32_t old, uint32_t src) {
    return __builtin_amdgcn_update_dpp((int)old, (int)src, 0x128, 0xF, BANKS, false);
}

template <int SETS>
__global__ __launch_bounds__(512) void gemv_i8row_mfma_kernel(const float *__restrict__ x, const int8_t *w8,
                                                              const float *sc, float *__restrict__ y, int M, int N,
                                                              int K) {
    using C = GemvI8Cfg<SETS>;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    uint32_t *amax = reinterpret_cast<uint32_t *>(smem + C::AMAX_OFF);

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rw = wave & 3, kh = wave >> 2;
    const int c = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 64 + rw * 16;
    // the two loads of a pair-step: rows (c & 7) and 8 + (c & 7) of the wave's 16, piece (c >> 3) + 2g of 128 bytes;
    // rows past the end are clamped, computed and never stored
    const int rx = (n0 + (c & 7) < N) ? n0 + (c & 7) : N - 1, ry = (n0 + 8 + (c & 7) < N) ? n0 + 8 + (c & 7) : N - 1;
    const unsigned char *wbase = reinterpret_cast<const unsigned char *>(w8) + 16 * ((c >> 3) + 2 * g);
    const unsigned char *wpx = wbase + (size_t)rx * K, *wpy = wbase + (size_t)ry * K;
    const int pairs = K >> 7, supers = (K + 2047) >> 11;
    auto pair_off = [&](int sr, int t) {  // byte offset of pair-step t of this wave's round in 2048-block sr
        const int p = (sr * 2 + kh) * C::PAIRS + t;
        return (size_t)((p < pairs) ? p : pairs - 1) * 128;
    };

    // staging role of this thread: activation row sm (clamped for the loads), 16-k pieces so, so + PARTS, ... of 2048 k
    const int sm = threadIdx.x % C::MROWS, so = threadIdx.x / C::MROWS;
    const float *xrow = x + (size_t)((sm < M) ? sm : M - 1) * K;
    f32x4 xr[C::XIT][4];
    auto request_x = [&](int sr) {
#pragma unroll
        for (int it = 0; it < C::XIT; ++it) {
            int k = sr * 2048 + 16 * (so + it * C::PARTS);
            k = (k < K) ? k : K - 16;
#pragma unroll
            for (int q = 0; q < 4; ++q) xr[it][q] = *reinterpret_cast<const f32x4 *>(xrow + k + 4 * q);
        }
    };
    // registers -> fixed point with the block's scale -> three digits -> operand order; leaves the block's row scales
    // 2^(e-20) (NaN for a non-finite block) in bscale[] of every lane
    float bscale[C::RES];
    auto stage_x = [&](int sr) {
        float v[C::XIT][16];
        uint32_t big = 0;  // largest exponent field among this thread's values
#pragma unroll
        for (int it = 0; it < C::XIT; ++it) {
            const bool live = sr * 2048 + 16 * (so + it * C::PARTS) < K;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                v[it][4 * q + 0] = live ? xr[it][q].x : 0.f;
                v[it][4 * q + 1] = live ? xr[it][q].y : 0.f;
                v[it][4 * q + 2] = live ? xr[it][q].z : 0.f;
                v[it][4 * q + 3] = live ? xr[it][q].w : 0.f;
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const uint32_t b = __builtin_amdgcn_ubfe(__float_as_uint(v[it][e]), 23, 8);
                big = b > big ? b : big;
            }
        }
        // the row's largest exponent in this block: over the lanes of this wave that stage the row, then over the waves
#pragma unroll
        for (int off = C::MROWS; off < 64; off <<= 1) {
            const uint32_t o = (uint32_t)__shfl_xor((int)big, off);
            big = o > big ? o : big;
        }
        if (lane < C::MROWS) amax[sm * 8 + wave] = big;
        __syncthreads();
        auto row_exp = [&](int m) {  // exponent field of the row's largest |x| (255: non-finite)
            const u32x4 a = *reinterpret_cast<const u32x4 *>(amax + m * 8), b = *reinterpret_cast<const u32x4 *>(amax + m * 8 + 4);
            uint32_t t = a.x > a.y ? a.x : a.y, u = a.z > a.w ? a.z : a.w, p = b.x > b.y ? b.x : b.y, q = b.z > b.w ? b.z : b.w;
            t = t > u ? t : u;
            p = p > q ? p : q;
            return (int)(t > p ? t : p);
        };
#pragma unroll
        for (int r = 0; r < C::RES; ++r) {
            const int m = (SETS == 3) ? 4 * g + r : 4 * r + g;
            const int eb = row_exp(m);
            // 2^(e - 20) as a float built from its exponent field; tiny blocks are scaled as if max|x| were 2^-100
            const int ec = eb < 27 ? 27 : eb;
            bscale[r] = (eb == 255) ? __uint_as_float(0x7FC00000u) : __uint_as_float((uint32_t)(ec - 20) << 23);
        }
        const int ebm = row_exp(sm);
        const int ecm = ebm < 27 ? 27 : (ebm > 254 ? 254 : ebm);
        const float up = __uint_as_float((uint32_t)(274 - ecm) << 23);  // 2^(20 - e)
#pragma unroll
        for (int it = 0; it < C::XIT; ++it) {
            uint32_t d0[4], d1[4], d2[4];
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                // X = rint(x * 2^(20 - e)) sits in the mantissa of x * 2^(20 - e) + 1.5 * 2^23 as 0x400000 + X; the
                // low three bytes of (X + 0x808080) ^ 0x808080 are the balanced base-256 digits a2, a1, a0 of X
                uint32_t z[4];
#pragma unroll
                for (int b = 0; b < 4; ++b)
                    z[b] = (__float_as_uint(__builtin_fmaf(v[it][4 * w + b], up, 12582912.0f)) + 0x408080u) ^ 0x808080u;
                // 4 x 4 byte transpose (three rows of it): digit d of four consecutive k in one word
                const uint32_t l01 = __builtin_amdgcn_perm(z[1], z[0], 0x05010400u), h01 = __builtin_amdgcn_perm(z[1], z[0], 0x07030602u);
                const uint32_t l23 = __builtin_amdgcn_perm(z[3], z[2], 0x05010400u), h23 = __builtin_amdgcn_perm(z[3], z[2], 0x07030602u);
                d2[w] = __builtin_amdgcn_perm(l23, l01, 0x05040100u);
                d1[w] = __builtin_amdgcn_perm(l23, l01, 0x07060302u);
                d0[w] = __builtin_amdgcn_perm(h23, h01, 0x05040100u);
            }
            const int osr = so + it * C::PARTS;  // piece of the 2048-block: round osr >> 6, piece o of the round
            const int o = osr & 63, t8 = o >> 3, gg = (o >> 1) & 3, jj = o & 1;
            unsigned char *blk = smem + (osr >> 6) * C::BUF_BYTES + t8 * C::PAIR_BYTES + jj * 1024;
            if constexpr (SETS == 3) {
                *reinterpret_cast<u32x4 *>(blk + (gg * 16 + sm) * 16) = u32x4{d0[0], d0[1], d0[2], d0[3]};
                *reinterpret_cast<u32x4 *>(blk + 2048 + (gg * 16 + sm) * 16) = u32x4{d1[0], d1[1], d1[2], d1[3]};
                *reinterpret_cast<u32x4 *>(blk + 4096 + (gg * 16 + sm) * 16) = u32x4{d2[0], d2[1], d2[2], d2[3]};
            } else {
                // the four operand rows of activation row (set, q); XOR-ing the low slot bits with (pair-step, MFMA)
                // spreads a wave's 64 pieces over all banks
                const int f = jj + 2 * (t8 & 1), base = (gg * 16 + 4 * (sm & 3)) ^ f;
                blk += (sm >> 2) * 2048;
                *reinterpret_cast<u32x4 *>(blk + (base ^ 0) * 16) = u32x4{d0[0], d0[1], d0[2], d0[3]};
                *reinterpret_cast<u32x4 *>(blk + (base ^ 1) * 16) = u32x4{d1[0], d1[1], d1[2], d1[3]};
                *reinterpret_cast<u32x4 *>(blk + (base ^ 2) * 16) = u32x4{d2[0], d2[1], d2[2], d2[3]};
                *reinterpret_cast<u32x4 *>(blk + (base ^ 3) * 16) = u32x4{0u, 0u, 0u, 0u};
            }
        }
    };

    request_x(0);
    u32x4 ring[2 * C::PAIRS];
#pragma unroll
    for (int t = 0; t < C::PAIRS; ++t) {
        ring[2 * t] = load_nt_b128(wpx + pair_off(0, t));
        ring[2 * t + 1] = load_nt_b128(wpy + pair_off(0, t));
    }
    // the weight stream starts before the staging below waits for anything (w8 and sc are not declared restrict so
    // that these loads cannot be moved below this point)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    stage_x(0);
    if (supers > 1) request_x(1);
    __syncthreads();

    float yacc[C::RES];
#pragma unroll
    for (int r = 0; r < C::RES; ++r) yacc[r] = 0.f;
    const unsigned char *abuf = smem + kh * C::BUF_BYTES;
    auto multiply = [&](int sr, auto refill) {  // this wave's 1024 k of 2048-block sr; refill: request the next block's
        i32x4 acc[SETS][2];
#pragma unroll
        for (int s = 0; s < SETS; ++s) acc[s][0] = acc[s][1] = i32x4{0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < C::PAIRS; ++t) {
            // wait for this pair-step's weights, then put the request for the next 2048-block in the queue
            asm volatile("" : "+v"(ring[2 * t]), "+v"(ring[2 * t + 1]));
            const u32x4 wx = ring[2 * t], wy = ring[2 * t + 1];
            if constexpr (decltype(refill)::value) {
                ring[2 * t] = load_nt_b128(wpx + pair_off(sr + 1, t));
                ring[2 * t + 1] = load_nt_b128(wpy + pair_off(sr + 1, t));
            }
            __builtin_amdgcn_sched_barrier(0);
            // this lane's row, k = 32g .. 32g + 15 and 32g + 16 .. 32g + 31 of the pair-step
            const i32x4 b0 = {half_row_merge<0xC>(wx.x, wy.x), half_row_merge<0xC>(wx.y, wy.y), half_row_merge<0xC>(wx.z, wy.z),
                              half_row_merge<0xC>(wx.w, wy.w)};
            const i32x4 b1 = {half_row_merge<0x3>(wy.x, wx.x), half_row_merge<0x3>(wy.y, wx.y), half_row_merge<0x3>(wy.z, wx.z),
                              half_row_merge<0x3>(wy.w, wx.w)};
#pragma unroll
            for (int jj = 0; jj < 2; ++jj)
#pragma unroll
                for (int s = 0; s < SETS; ++s) {
                    const int slot = (SETS == 3) ? lane : (lane ^ (jj + 2 * (t & 1)));
                    const i32x4 av = *reinterpret_cast<const i32x4 *>(abuf + t * C::PAIR_BYTES + (s * 2 + jj) * 1024 + slot * 16);
                    acc[s][jj] = __builtin_amdgcn_mfma_i32_16x16x64_i8(av, jj ? b1 : b0, acc[s][jj], 0, 0, 0);
                }
        }
        // the block's digit sums -> fp32 with the block's scales.  D0 * 2^16 + D1 * 2^8 + D2 can need more than the 24
        // bits of a float before its terms cancel, so the three are combined in float64 (exact: below 2^53) and rounded
        // to fp32 once
        auto combine = [](int d0, int d1, int d2) {
            return (float)__builtin_fma((double)d0, 65536.0, __builtin_fma((double)d1, 256.0, (double)d2));
        };
        if constexpr (SETS == 3) {
            const i32x4 e0 = acc[0][0] + acc[0][1], e1 = acc[1][0] + acc[1][1], e2 = acc[2][0] + acc[2][1];
            const int q0[4] = {e0.x, e0.y, e0.z, e0.w}, q1[4] = {e1.x, e1.y, e1.z, e1.w}, q2[4] = {e2.x, e2.y, e2.z, e2.w};
#pragma unroll
            for (int r = 0; r < 4; ++r)
                yacc[r] = __builtin_fmaf(bscale[r], combine(q0[r], q1[r], q2[r]), yacc[r]);
        } else {
#pragma unroll
            for (int s = 0; s < SETS; ++s) {
                const i32x4 e = acc[s][0] + acc[s][1];
                yacc[s] = __builtin_fmaf(bscale[s], combine(e.x, e.y, e.z), yacc[s]);
            }
        }
    };
    for (int sr = 0; sr + 1 < supers; ++sr) {
        multiply(sr, std::true_type{});
        __syncthreads();  // every wave is done with this block's operands and row maxima
        stage_x(sr + 1);
        request_x(sr + 2 < supers ? sr + 2 : supers - 1);
        __syncthreads();
    }
    multiply(supers - 1, std::false_type{});

    // the upper K half hands its sums over
    f32x4 *fold = reinterpret_cast<f32x4 *>(smem + C::FOLD_OFF) + rw * 64 + lane;
    if (kh) {
        f32x4 o = {0.f, 0.f, 0.f, 0.f};
        o.x = yacc[0];
        if constexpr (C::RES > 1) o.y = yacc[1];
        if constexpr (C::RES > 2) {
            o.z = yacc[2];
            o.w = yacc[3];
        }
        *fold = o;
    }
    __syncthreads();
    if (kh) return;
    const f32x4 o = *fold;
    const float other[4] = {o.x, o.y, o.z, o.w};
    const int n = n0 + c;
    const float scale = (n < N) ? sc[n] : 0.f;
#pragma unroll
    for (int r = 0; r < C::RES; ++r) {
        const int m = (SETS == 3) ? 4 * g + r : 4 * r + g;
        if (m < M && n < N) y[(size_t)m * N + n] = (yacc[r] + other[r]) * scale;
    }
}

bool gemv_i8row_mfma_ok(int M, int K) { return M >= 1 && M <= 16 && K % 128 == 0; }

template <int SETS>
static int launch_i8_mfma(const float *x, const int8_t *w8, const float *sc, float *y, int M, int N, int K, hipStream_t st) {
    using C = GemvI8Cfg<SETS>;
    static std::atomic<bool> attr_set{false};  // setting it twice from two threads is harmless
    if (!attr_set.load(std::memory_order_acquire)) {
        CHADQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_i8row_mfma_kernel<SETS>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS));
        attr_set.store(true, std::memory_order_release);
    }
    hipLaunchKernelGGL(gemv_i8row_mfma_kernel<SETS>, dim3((N + 63) / 64), dim3(512), C::LDS, st, x, w8, sc, y, M, N, K);
    return hip_check(hipGetLastError(), "gemv_i8row_mfma launch");
}

// 1..16 activation rows, K a multiple of 128 (x and w8 16-byte aligned as for every int8 GEMV)
int gemv_i8row_mfma_launch(const float *x, const int8_t *w8, const float *sc, float *y, int M, int N, int K,
                           hipStream_t st) {
    if (M <= 4) return launch_i8_mfma<1>(x, w8, sc, y, M, N, K, st);
    if (M <= 8) return launch_i8_mfma<2>(x, w8, sc, y, M, N, K, st);
    return launch_i8_mfma<3>(x, w8, sc, y, M, N, K, st);
}

}  // namespace chadq
