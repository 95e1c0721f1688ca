// Prefill dequant-GEMM:  y[m,n] = bf16( sum_k x[m,k] * w[n,k] ),  x bf16 [M,K], fp32 accumulate on MFMA.
//   int4 group-32:  w = bf16_rne((u-8) * scale[n,k/32])          (dequantised to bf16 for the matrix core)
//   int8 per-row :  w = W[n,k] exactly in bf16, scale[n] applied to the fp32 accumulator afterwards
//
// Workgroup = 4 waves, output tile 128 x 64, and the four waves split K: wave w owns every fourth slice of
// K and accumulates a full 128 x 64 partial tile (8 accumulators of v_mfma_f32_32x32x16_bf16).  That choice
// makes both operands private to a wave:
//   * B (weights): lane (n = lane%32, kq = lane/32) loads 16 packed bytes of output row n, which is 32 k
//     (int4, exactly one scale group) or 16 k (int8), dequantises them in registers and feeds them to the
//     MFMA directly.  Weights never touch LDS.
//   * A (activations): the wave copies its own 128 x KW slice through a wave-private LDS buffer purely to
//     transpose from coalesced row-major loads (8 rows x 128 B per instruction) to MFMA fragments.  No other
//     wave reads it, so the main loop has no barriers.
// The MFMA k-slot of a lane is free to choose as long as A and B agree: slot group kq covers the kq-th
// 16-byte weight load, and step t of that load is its t-th 8-k word.
// The four partial tiles are summed through LDS at the end, rounded to bf16 (RNE) and stored coalesced.
#include "chadq_common.h"

namespace chadq {

typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;

__device__ __forceinline__ f16x2 as_f16x2(uint32_t v) {
    f16x2 r;
    __builtin_memcpy(&r, &v, 4);
    return r;
}

__device__ __forceinline__ uint32_t pack_bf16_rne(float a, float b) {
    f32x2 f = {a, b};
    bf16x2 h = __builtin_convertvector(f, bf16x2);
    uint32_t r;
    __builtin_memcpy(&r, &h, 4);
    return r;
}

struct FmtI4G32 {
    static constexpr int KL = 32;  // k per 16-byte weight load
    typedef uint16_t scale_t;
    // 8 nibbles of word `w` -> 8 bf16 of (u-8)*s, k order.  fp16 magic: 0x6400|u = 1024+u, and a nibble left
    // in bits 7:4 reads as 1024+16u; one fp32 FMA per element removes the offsets and applies the scale.
    __device__ static __forceinline__ bf16x8 dequant(uint32_t w, float s, float s16, float c0, float c1) {
        constexpr uint32_t magic = 0x64006400u;
        const f16x2 h0 = as_f16x2((w & 0x000F000Fu) | magic);  // u0, u4
        const f16x2 h1 = as_f16x2((w & 0x00F000F0u) | magic);  // 16*u1, 16*u5
        const uint32_t w8 = w >> 8;
        const f16x2 h2 = as_f16x2((w8 & 0x000F000Fu) | magic);  // u2, u6
        const f16x2 h3 = as_f16x2((w8 & 0x00F000F0u) | magic);  // 16*u3, 16*u7
        const float f0 = __builtin_fmaf((float)h0.x, s, c0), f4 = __builtin_fmaf((float)h0.y, s, c0);
        const float f1 = __builtin_fmaf((float)h1.x, s16, c1), f5 = __builtin_fmaf((float)h1.y, s16, c1);
        const float f2 = __builtin_fmaf((float)h2.x, s, c0), f6 = __builtin_fmaf((float)h2.y, s, c0);
        const float f3 = __builtin_fmaf((float)h3.x, s16, c1), f7 = __builtin_fmaf((float)h3.y, s16, c1);
        const u32x4 r = {pack_bf16_rne(f0, f1), pack_bf16_rne(f2, f3), pack_bf16_rne(f4, f5), pack_bf16_rne(f6, f7)};
        bf16x8 o;
        __builtin_memcpy(&o, &r, 16);
        return o;
    }
};

struct FmtI8Row {
    static constexpr int KL = 16;
    typedef float scale_t;
    // 8 signed bytes (two words) -> 8 bf16, exact.  b^0x80 = b+128 as unsigned; 0x6400|that = 1024+b+128.
    __device__ static __forceinline__ bf16x8 dequant(uint32_t wa, uint32_t wb) {
        const uint32_t a = wa ^ 0x80808080u, b = wb ^ 0x80808080u;
        const f16x2 h0 = as_f16x2(__builtin_amdgcn_perm(0x64646464u, a, 0x04010400u));
        const f16x2 h1 = as_f16x2(__builtin_amdgcn_perm(0x64646464u, a, 0x04030402u));
        const f16x2 h2 = as_f16x2(__builtin_amdgcn_perm(0x64646464u, b, 0x04010400u));
        const f16x2 h3 = as_f16x2(__builtin_amdgcn_perm(0x64646464u, b, 0x04030402u));
        constexpr float c = -1152.f;
        const u32x4 r = {pack_bf16_rne((float)h0.x + c, (float)h0.y + c), pack_bf16_rne((float)h1.x + c, (float)h1.y + c),
                         pack_bf16_rne((float)h2.x + c, (float)h2.y + c), pack_bf16_rne((float)h3.x + c, (float)h3.y + c)};
        bf16x8 o;
        __builtin_memcpy(&o, &r, 16);
        return o;
    }
};

constexpr int BM = 128, BN = 64, NWAVE = 4;

template <typename F>
struct Tile {
    static constexpr int KL = F::KL;
    static constexpr int KW = 2 * KL;               // k per wave per iteration (two 16-byte loads side by side)
    static constexpr int KIT = NWAVE * KW;          // k per workgroup iteration
    static constexpr int T = KL / 8;                // MFMA steps per 16-byte load
    static constexpr int ROWB = KW * 2 + 16;        // LDS row pitch in bytes (+16: conflict-free fragment reads)
    static constexpr int LPR = KW * 2 / 16;         // lanes per activation row in a staging load
    static constexpr int RPI = 64 / LPR;            // rows per staging instruction
    static constexpr int NI = BM / RPI;             // staging instructions per iteration
    static constexpr int STAGE_BYTES = BM * ROWB;   // per wave
    static constexpr int EPI_BYTES = NWAVE * BM * 32 * 4;
    static constexpr int LDS_BYTES = (NWAVE * STAGE_BYTES > EPI_BYTES) ? NWAVE * STAGE_BYTES : EPI_BYTES;
};

template <typename F>
__global__ __launch_bounds__(256) void gemm_q_bf16_kernel(const uint16_t *__restrict__ x, const void *__restrict__ wq,
                                                          const typename F::scale_t *__restrict__ sc,
                                                          uint16_t *__restrict__ y, int M, int N, int K) {
    typedef Tile<F> TL;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nl = lane & 31, kq = lane >> 5;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    uint8_t *stage = lds + wave * TL::STAGE_BYTES;
    const bool i4 = (TL::KL == 32);
    const size_t wrow_bytes = i4 ? (size_t)(K >> 1) : (size_t)K;
    const int G = K >> 5;

    f32x16 acc[4][2];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

    // weight rows of this lane (clamped so that loads stay in bounds; results for n >= N are never stored)
    int wr[2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
        const int n = n0 + nb * 32 + nl;
        wr[nb] = n < N ? n : N - 1;
    }
    // staging coordinates of this lane
    const int srow = lane / TL::LPR, scol = (lane % TL::LPR) * 8;  // row within an instruction, k offset (elements)

    u32x4 bq[2];
    float bs[2];
    u32x4 ar[TL::NI];

    auto issue_loads = [&](int it) {
        const int kb = it * TL::KIT + wave * TL::KW;
        const int kw = kb + kq * TL::KL;  // first k of this lane's weight load
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            if (kw < K) {
                const uint8_t *p = (const uint8_t *)wq + (size_t)wr[nb] * wrow_bytes + (i4 ? (kw >> 1) : kw);
                bq[nb] = *reinterpret_cast<const u32x4 *>(p);
                if (i4) bs[nb] = f16_bits_to_f32(((const uint16_t *)sc)[(size_t)wr[nb] * G + (kw >> 5)]);
            } else {
                bq[nb] = u32x4{0, 0, 0, 0};
                bs[nb] = 0.f;
            }
        }
#pragma unroll
        for (int i = 0; i < TL::NI; ++i) {
            int m = m0 + i * TL::RPI + srow;
            m = m < M ? m : M - 1;
            const int k = kb + scol;
            ar[i] = (k < K) ? *reinterpret_cast<const u32x4 *>(x + (size_t)m * K + k) : u32x4{0, 0, 0, 0};
        }
    };
    auto store_stage = [&]() {
#pragma unroll
        for (int i = 0; i < TL::NI; ++i)
            *reinterpret_cast<u32x4 *>(stage + (i * TL::RPI + srow) * TL::ROWB + scol * 2) = ar[i];
    };

    const int iters = (K + TL::KIT - 1) / TL::KIT;
    issue_loads(0);
    for (int it = 0; it < iters; ++it) {
        store_stage();
        const u32x4 cq[2] = {bq[0], bq[1]};
        const float cs[2] = {bs[0], bs[1]};
        const bool live = (it * TL::KIT + wave * TL::KW + kq * TL::KL) < K;
        if (it + 1 < iters) issue_loads(it + 1);
#pragma unroll
        for (int t = 0; t < TL::T; ++t) {
            bf16x8 bf[2];
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                if constexpr (TL::KL == 32) {
                    const float s = cs[nb];
                    const uint32_t wsel = t == 0 ? cq[nb].x : t == 1 ? cq[nb].y : t == 2 ? cq[nb].z : cq[nb].w;
                    bf[nb] = FmtI4G32::dequant(wsel, s, s * 0.0625f, -1032.f * s, -72.f * s);
                } else {
                    bf[nb] = t == 0 ? FmtI8Row::dequant(cq[nb].x, cq[nb].y) : FmtI8Row::dequant(cq[nb].z, cq[nb].w);
                    if (!live) {
                        const u32x4 z = {0, 0, 0, 0};
                        __builtin_memcpy(&bf[nb], &z, 16);
                    }
                }
            }
#pragma unroll
            for (int mb = 0; mb < 4; ++mb) {
                const bf16x8 af = *reinterpret_cast<const bf16x8 *>(stage + (mb * 32 + nl) * TL::ROWB + (kq * TL::KL + 8 * t) * 2);
#pragma unroll
                for (int nb = 0; nb < 2; ++nb)
                    acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bf[nb], acc[mb][nb], 0, 0, 0);
            }
        }
    }

    // cross-wave sum, one 128 x 32 half tile at a time: [wave][row][32] fp32 in LDS
    float rs[2] = {1.f, 1.f};
#pragma unroll
    for (int nb = 0; nb < 2; ++nb) {
        __syncthreads();
        float *red = reinterpret_cast<float *>(lds) + wave * (BM * 32);
#pragma unroll
        for (int mb = 0; mb < 4; ++mb)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = mb * 32 + 8 * (v >> 2) + 4 * kq + (v & 3);
                red[row * 32 + nl] = acc[mb][nb][v];
            }
        __syncthreads();
        // 128 x 32 outputs, 256 threads: thread handles 4 consecutive columns of 4 rows
        const int c4 = (tid & 7) * 4;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int row = (tid >> 3) + p * 32;
            f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int w2 = 0; w2 < NWAVE; ++w2)
                s += *reinterpret_cast<const f32x4 *>(reinterpret_cast<const float *>(lds) + w2 * (BM * 32) + row * 32 + c4);
            const int m = m0 + row, n = n0 + nb * 32 + c4;
            if (m < M) {
                if constexpr (TL::KL == 16) {
                    const float *scf = (const float *)sc;
                    s.x *= (n + 0 < N) ? scf[n + 0] : 0.f;
                    s.y *= (n + 1 < N) ? scf[n + 1] : 0.f;
                    s.z *= (n + 2 < N) ? scf[n + 2] : 0.f;
                    s.w *= (n + 3 < N) ? scf[n + 3] : 0.f;
                }
                uint16_t *yp = y + (size_t)m * N + n;
                if (n + 3 < N && ((N & 3) == 0)) {
                    u32x2 o = {pack_bf16_rne(s.x, s.y), pack_bf16_rne(s.z, s.w)};
                    *reinterpret_cast<u32x2 *>(yp) = o;
                } else {
                    const float sv[4] = {s.x, s.y, s.z, s.w};
                    for (int j = 0; j < 4; ++j)
                        if (n + j < N) yp[j] = (uint16_t)f32_to_bf16_bits(sv[j]);
                }
            }
        }
    }
    (void)rs;
}

template <typename F>
static int launch_gemm(const uint16_t *x, const void *wq, const typename F::scale_t *sc, uint16_t *y, int M, int N,
                       int K, hipStream_t st) {
    typedef Tile<F> TL;
    static bool attr_set = false;
    if (!attr_set) {
        CHADQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q_bf16_kernel<F>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, TL::LDS_BYTES));
        attr_set = true;
    }
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
    hipLaunchKernelGGL((gemm_q_bf16_kernel<F>), grid, dim3(256), TL::LDS_BYTES, st, x, wq, sc, y, M, N, K);
    return hip_check(hipGetLastError(), "gemm_q_bf16 launch");
}

int gemm_i4g32_bf16_dispatch(const uint16_t *x, const uint8_t *wp, const uint16_t *sc, uint16_t *y, int M, int N,
                             int K, hipStream_t st) {
    return launch_gemm<FmtI4G32>(x, wp, sc, y, M, N, K, st);
}

int gemm_i8row_bf16_dispatch(const uint16_t *x, const int8_t *w8, const float *sc, uint16_t *y, int M, int N, int K,
                             hipStream_t st) {
    return launch_gemm<FmtI8Row>(x, w8, sc, y, M, N, K, st);
}

}  // namespace chadq
