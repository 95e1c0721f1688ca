// Grouped "skinny" dequant-GEMM for the mixture-of-experts FFN: few activation rows (the tokens routed to one
// expert, tens to a hundred or so) against many int4 group-32 weight rows.  The prefill tile (128 x 64) is the
// wrong shape here: half of its rows are padding and every 64 weight rows re-read the whole activation panel.
// This kernel turns the tile around: one workgroup takes up to 128 tokens of one expert and 256 weight rows,
//   - the activation tile (32*MB rows x 64 k per iteration, MB = 1..4 from the expert's actual row count) goes
//     through LDS once per workgroup and is shared by the four waves (XOR-swizzled 16-byte pieces);
//   - each wave owns 64 weight rows: its lanes stream them straight from global memory (16 B = one group of 32
//     nibbles per load), dequantise in registers (fp16 magic number, one FMA per element, RNE to bf16) and feed
//     v_mfma_f32_32x32x16_bf16; every weight byte is fetched once per token tile;
//   - 272 B of operands per k for 2*64*256 flop per k (64 tokens): 2.1 x the arithmetic intensity of the
//     prefill tile, which is what the cache-to-CU bandwidth needs.
// MODE 1 (gate/up): the wave's two 32-row blocks are the same 32 features of the gate and of the up matrix, so
//   silu(gate) * up is formed in registers and written as bf16 - the fp32 gate/up matrices never exist.
// MODE 0 (down): fp32 partial outputs, optionally split over K (blockIdx.z) for more workgroups; the combine
//   kernel adds the parts.
// Needs K % 256 == 0 (and the K range per split a multiple of 256), 256 | N (MODE 0) or 128 | N (MODE 1).
#include "chadq_common.h"

namespace chadq {

constexpr int SK_MT = 128;  // tokens per workgroup tile
constexpr int SK_KI = 64;   // k per iteration

struct SkDequant {
    // 8 nibbles of word `w` -> 8 bf16 of (u-8)*s in k order; see FmtI4G32::dequant in the prefill kernel for the
    // magic-number scheme (0x6400|u reads 1024+u, a nibble left in bits 7:4 reads 1024+16u).
    __device__ static __forceinline__ bf16x8 run(uint32_t w, float s, float s16, float c0, float c1, uint32_t mlo,
                                                 uint32_t mhi, uint32_t magic) {
        const f16x2 h0 = as_f16x2(and_or(w, mlo, magic));
        const f16x2 h1 = as_f16x2(and_or(w, mhi, magic));
        const uint32_t w8 = w >> 8;
        const f16x2 h2 = as_f16x2(and_or(w8, mlo, magic));
        const f16x2 h3 = as_f16x2(and_or(w8, mhi, magic));
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

template <int MODE, int MB>
__device__ __forceinline__ void skinny_body(const uint16_t *__restrict__ x, const uint8_t *__restrict__ w0,
                                            const uint16_t *__restrict__ s0, const uint8_t *__restrict__ w1,
                                            const uint16_t *__restrict__ s1, void *__restrict__ yv, int m0, int rows,
                                            int n0, int N, int K, int kbeg, int kend, uint8_t *lds) {
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nl = lane & 31, kq = lane >> 5;
    constexpr int STAGE = MB * 32 * 128;  // bytes of one activation stage

    // weight rows of this lane
    const uint8_t *wrow[2];
    const uint16_t *srow[2];
    if (MODE == 1) {
        const int f = n0 + wave * 32 + nl;
        wrow[0] = w0 + (size_t)f * (K >> 1);
        wrow[1] = w1 + (size_t)f * (K >> 1);
        srow[0] = s0 + (size_t)f * (K >> 5);
        srow[1] = s1 + (size_t)f * (K >> 5);
    } else {
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            const int n = n0 + wave * 64 + nb * 32 + nl;
            wrow[nb] = w0 + (size_t)n * (K >> 1);
            srow[nb] = s0 + (size_t)n * (K >> 5);
        }
    }
    // activation pieces of this thread: piece p of rows r, r+32, ...; rows past the tile repeat its last row
    const int p = tid & 7, r = tid >> 3;
    const uint16_t *arow[MB];
    uint32_t awr[MB];
#pragma unroll
    for (int i = 0; i < MB; ++i) {
        const int rr = i * 32 + r, rc = rr < rows ? rr : rows - 1;
        arow[i] = x + (size_t)(m0 + rc) * K + p * 8;
        awr[i] = (uint32_t)(rr * 128 + ((p ^ (r & 7)) << 4));
    }
    // fragment read offsets: row mb*32+nl, piece kq*4+j lives in slot (kq*4+j) ^ (nl & 7)
    uint32_t ard[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) ard[j] = (uint32_t)(nl * 128 + (((kq * 4 + j) ^ (nl & 7)) << 4));

    f32x16 acc[MB][2];
#pragma unroll
    for (int a = 0; a < MB; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

    const uint32_t c_mlo = vgpr_const(0x000F000Fu), c_mhi = vgpr_const(0x00F000F0u), c_magic = vgpr_const(0x64006400u);
    u32x4 ra[2][MB];          // activation pieces in flight: ra[it & 1] = iteration it
    u32x4 rb[3][2];           // packed weights: rb[0] = this iteration, rb[1], rb[2] = the next two
    u32x4 rs_cur[2], rs_nxt[2];  // 8 group scales (256 k) per weight row block

    auto load_a = [&](int par, int k0) {
#pragma unroll
        for (int i = 0; i < MB; ++i) ra[par][i] = *reinterpret_cast<const u32x4 *>(arow[i] + k0);
    };
    auto load_b = [&](int slot, int k0) {
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) rb[slot][nb] = load_nt_b128(wrow[nb] + ((k0 + 32 * kq) >> 1));
    };
    auto load_s = [&](u32x4(&dst)[2], int k0) {
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) dst[nb] = *reinterpret_cast<const u32x4 *>(srow[nb] + (k0 >> 5));
    };
    auto store_a = [&](int par, int stage) {
#pragma unroll
        for (int i = 0; i < MB; ++i) *reinterpret_cast<u32x4 *>(lds + stage * STAGE + awr[i]) = ra[par][i];
    };

    const int nit = (kend - kbeg) / SK_KI;  // a multiple of 4
    load_s(rs_cur, kbeg);
    load_a(0, kbeg);
    load_b(0, kbeg);
    load_a(1, kbeg + SK_KI);
    load_b(1, kbeg + SK_KI);
    store_a(0, 0);
    __syncthreads();

    for (int it0 = 0; it0 < nit; it0 += 4) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int it = it0 + u, k0 = kbeg + it * SK_KI;
            const int s = u & 1;
            // prefetch two iterations ahead; past the end the loads repeat the first iteration (never used)
            const int k2 = (it + 2 < nit) ? k0 + 2 * SK_KI : kbeg;
            load_a(s, k2);  // ra[s] (iteration it) went to LDS one iteration ago
            load_b(2, k2);
            if (u == 0) load_s(rs_nxt, (it0 + 4 < nit) ? k0 + 4 * SK_KI : kbeg);

            // this iteration's group scale: group 2*u + kq of the 8 held
            float cs[2][4];
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                const uint32_t wsel = u == 0 ? rs_cur[nb].x : u == 1 ? rs_cur[nb].y : u == 2 ? rs_cur[nb].z : rs_cur[nb].w;
                const float sc = f16_bits_to_f32((wsel >> (16 * kq)) & 0xFFFFu);
                cs[nb][0] = sc;
                cs[nb][1] = sc * 0.0625f;
                cs[nb][2] = -1032.f * sc;
                cs[nb][3] = -72.f * sc;
            }
            const uint8_t *ab = lds + s * STAGE;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                bf16x8 bf[2];
#pragma unroll
                for (int nb = 0; nb < 2; ++nb) {
                    const u32x4 q = rb[0][nb];
                    const uint32_t wsel = j == 0 ? q.x : j == 1 ? q.y : j == 2 ? q.z : q.w;
                    bf[nb] = SkDequant::run(wsel, cs[nb][0], cs[nb][1], cs[nb][2], cs[nb][3], c_mlo, c_mhi, c_magic);
                }
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    const bf16x8 af = *reinterpret_cast<const bf16x8 *>(ab + mb * 4096 + ard[j]);
#pragma unroll
                    for (int nb = 0; nb < 2; ++nb)
                        acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, bf[nb], acc[mb][nb], 0, 0, 0);
                }
            }
            // the next iteration's activations go to the other stage (last read one iteration ago, barrier since)
            store_a(s ^ 1, s ^ 1);
            __syncthreads();
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) {
                rb[0][nb] = rb[1][nb];
                rb[1][nb] = rb[2][nb];
            }
            if (u == 3) {
                rs_cur[0] = rs_nxt[0];
                rs_cur[1] = rs_nxt[1];
            }
        }
    }

    // epilogue: lane (nl, kq) holds column nl of rows 8*(v/4) + 4*kq + v%4 of each 32 x 32 block
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = mb * 32 + 8 * (v >> 2) + 4 * kq + (v & 3);
            if (row < rows) {
                if (MODE == 1) {
                    const float g = acc[mb][0][v], up = acc[mb][1][v];
                    const float h = g / (1.f + __expf(-g)) * up;
                    reinterpret_cast<uint16_t *>(yv)[(size_t)(m0 + row) * N + n0 + wave * 32 + nl] = (uint16_t)f32_to_bf16_bits(h);
                } else {
#pragma unroll
                    for (int nb = 0; nb < 2; ++nb)
                        reinterpret_cast<float *>(yv)[(size_t)(m0 + row) * N + n0 + wave * 64 + nb * 32 + nl] = acc[mb][nb][v];
                }
            }
        }
}

// groups: [E] gate, [E] up, [E] down descriptors as the router writes them.
// grid: x = N tiles, y = expert * mtiles + token tile, z = K split (MODE 0 only).
template <int MODE>
__global__ __launch_bounds__(256, 2) void gemm_skinny_i4g32_kernel(const GemmGroup *__restrict__ groups, int E, int N, int K,
                                                                  int kspan, int mtiles, size_t ysplit_stride) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int g = blockIdx.y / mtiles, mt = blockIdx.y % mtiles;
    const GemmGroup ga = groups[MODE == 1 ? g : 2 * E + g];
    const int M = ga.M, m0 = mt * SK_MT;
    if (m0 >= M) return;
    const int rows = (M - m0) < SK_MT ? (M - m0) : SK_MT;
    const int kbeg = blockIdx.z * kspan, kend = (kbeg + kspan < K) ? kbeg + kspan : K;
    const uint8_t *w0 = reinterpret_cast<const uint8_t *>(ga.w), *w1 = nullptr;
    const uint16_t *s0 = reinterpret_cast<const uint16_t *>(ga.sc), *s1 = nullptr;
    void *y;
    int n0;
    if (MODE == 1) {
        const GemmGroup gu = groups[E + g], gd = groups[2 * E + g];
        w1 = reinterpret_cast<const uint8_t *>(gu.w);
        s1 = reinterpret_cast<const uint16_t *>(gu.sc);
        y = const_cast<uint16_t *>(gd.x);  // the down projection's input rows of this expert
        n0 = blockIdx.x * 128;
    } else {
        y = reinterpret_cast<float *>(ga.y) + (size_t)blockIdx.z * ysplit_stride;
        n0 = blockIdx.x * 256;
    }
    switch ((rows + 31) >> 5) {
        case 1: skinny_body<MODE, 1>(ga.x, w0, s0, w1, s1, y, m0, rows, n0, N, K, kbeg, kend, lds); break;
        case 2: skinny_body<MODE, 2>(ga.x, w0, s0, w1, s1, y, m0, rows, n0, N, K, kbeg, kend, lds); break;
        case 3: skinny_body<MODE, 3>(ga.x, w0, s0, w1, s1, y, m0, rows, n0, N, K, kbeg, kend, lds); break;
        default: skinny_body<MODE, 4>(ga.x, w0, s0, w1, s1, y, m0, rows, n0, N, K, kbeg, kend, lds); break;
    }
}

constexpr int SK_LDS = 2 * 4 * 32 * 128;  // two stages of up to 128 rows x 64 k bf16

bool gemm_skinny_ok(int H, int F) { return H % 256 == 0 && F % 256 == 0; }

// gate/up with the SiLU epilogue: h[P,F] bf16 (through the down descriptors' x pointers)
int gemm_skinny_gateup(const GemmGroup *groups, int E, int m_max, int F, int H, hipStream_t st) {
    const int mtiles = (m_max + SK_MT - 1) / SK_MT;
    hipLaunchKernelGGL((gemm_skinny_i4g32_kernel<1>), dim3(F / 128, E * mtiles, 1), dim3(256), SK_LDS, st, groups, E, F, H, H,
                       mtiles, (size_t)0);
    return hip_check(hipGetLastError(), "gemm_skinny gate/up launch");
}

// down: fp32 parts [ksplit][P,H]
int gemm_skinny_down(const GemmGroup *groups, int E, int m_max, int H, int F, int ksplit, size_t ysplit_stride, hipStream_t st) {
    const int mtiles = (m_max + SK_MT - 1) / SK_MT;
    hipLaunchKernelGGL((gemm_skinny_i4g32_kernel<0>), dim3(H / 256, E * mtiles, ksplit), dim3(256), SK_LDS, st, groups, E, H, F,
                       F / ksplit, mtiles, ysplit_stride);
    return hip_check(hipGetLastError(), "gemm_skinny down launch");
}

}  // namespace chadq
