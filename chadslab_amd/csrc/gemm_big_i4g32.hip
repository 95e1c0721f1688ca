// Prefill dequant-GEMM for many activation rows:  y[m,n] = bf16( sum_k x[m,k] * w[n,k] ),  x bf16 [M,K],
// w = bf16_rne((u-8) * scale[n,k/32]) (int4 group-32), fp32 accumulate on v_mfma_f32_32x32x16_bf16.
//
// Two facts about the chip shape this kernel (both measured on it).  A compute unit reads at most 64 B per clock from
// its LDS (ds_read_b128: 150 B/ns) while its four matrix cores consume 256 B of operands per clock at full rate, so a
// wave has to reuse every fragment it reads as often as its registers allow.  And the clock follows the power the
// arithmetic draws: a plain bf16 GEMM of the vendor library runs at 1.2 PFLOP/s on random data and 1.9 on zeros
// (4096^3), so every instruction next to the MFMAs costs twice, its issue slot and the clock.
//
// Output tile 256 x 256 per workgroup of 4 waves, K walked in steps of 64; a wave owns WMB x WNB blocks of 32 x 32
// (256 accumulator registers).  The kernel is written for both ways of dealing the tile to four waves:
//   1 x 4 (a wave owns all 256 rows of 64 columns; the one that is launched): every weight is dequantised exactly
//     once per workgroup, i.e. once per 256 activation rows, and a fragment set (8 A fragments) feeds 16 MFMAs:
//     0.5 KiB of LDS reads per MFMA.  4096^3: 146 us.
//   2 x 2 (128 x 128 each): 0.25 KiB of LDS reads per MFMA, but the two waves of a column half dequantise the same
//     weights (twice the dequantisation instructions).  4096^3: 155 us.
//   A (activations): global -> LDS by DMA (global_load_lds_dwordx4, 8 rows x 128 B per instruction), three stages,
//      16-byte pieces XOR-swizzled by row so that fragment reads are bank-conflict free; wave w moves rows 64w..64w+63.
//   B (weights): never in the LDS as bf16.  A wave DMAs the packed bytes of its own columns (32 B per row and step)
//      and their group scales (16 B = 8 groups per row, once per four steps) into slots of its own; lane (n, kq) reads
//      back 16 bytes = the 32 nibbles of one scale group and dequantises them in registers into the B operands of the
//      step's four MFMA slices (slot group kq of slice t holds k = 32 kq + 8 t ..+7; the A fragment reads use the same
//      assignment).
//   One barrier per step, in front of the step's last slice (see step_body).
// Needs K % 256 == 0 and 16-byte aligned scale rows; M and N are arbitrary (rows past the end repeat the last one
// and are never stored).
#include <type_traits>

#include "chadq_common.h"

namespace chadq {

namespace big {
constexpr int BM = 256, BN = 256, BK = 64;
constexpr int A_STAGE = BM * BK * 2;  // 32 KiB
constexpr int A_STAGES = 3;
constexpr int A_BYTES = A_STAGES * A_STAGE;

template <int WM, int WN>
struct Cfg {
    static_assert(WM * WN == 4, "four waves");
    static constexpr int WMB = 8 / WM, WNB = 8 / WN;   // 32 x 32 blocks per wave along M and N
    static constexpr int COLS = 32 * WNB;              // a wave's columns
    static constexpr int BP_SLOT = COLS * 32;          // its packed weights of one step
    static constexpr int SC_SLOT = COLS * 16;          // its scales of four steps
    static constexpr int BP_OFF = A_BYTES, BP_WAVE = 2 * BP_SLOT;
    static constexpr int SC_OFF = BP_OFF + 4 * BP_WAVE, SC_WAVE = 2 * SC_SLOT;
    static constexpr int LDS_BYTES = SC_OFF + 4 * SC_WAVE;
    // the epilogue passes 128 rows of a wave's columns through LDS at a time; the pad spreads rows over the banks
    static constexpr int EP_PITCH = COLS * 2 + 16;
    static_assert(4 * 128 * EP_PITCH <= LDS_BYTES, "the four result tiles fit the operand area");
};
}  // namespace big

// The bare barrier instruction (__syncthreads() would add a fence that waits for every outstanding request, which
// drains the prefetch); the empty asm statements keep the compiler from moving LDS accesses across it.
__device__ __forceinline__ void wg_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

template <int WM, int WN>
__global__ __launch_bounds__(256) void gemm_big_i4g32_kernel(const uint16_t *__restrict__ x, const uint8_t *__restrict__ wp,
                                                             const uint16_t *__restrict__ sc, uint16_t *__restrict__ y, int M,
                                                             int N, int K) {
    using namespace big;
    typedef Cfg<WM, WN> C;
    constexpr int WMB = C::WMB, WNB = C::WNB;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nl = lane & 31, kq = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;
    // workgroup i runs on XCD i % 8: deal the tiles so that one XCD walks consecutive n-tiles of the same m-panel
    const int tiles_n = (N + BN - 1) / BN, tiles = tiles_n * ((M + BM - 1) / BM);
    const int wg = blockIdx.x, per_xcd = (tiles + 7) / 8;
    const int tile = (wg % 8) * per_xcd + wg / 8;
    if (tile >= tiles) return;
    const int m0 = (tile / tiles_n) * BM, n0 = (tile % tiles_n) * BN;
    const int G = K >> 5, steps = K / BK;
    const int row0 = wm * (32 * WMB), col0 = wn * C::COLS;  // the wave's corner inside the tile

    // ---- request addresses
    // A: instruction q of wave w fills LDS rows 64w + 8q .. +7 (lane -> row lane/8, position lane%8, which holds piece
    // position ^ (row & 7)); byte offsets into x are 32-bit (the host checks M*K*2 < 2^32)
    uint32_t aoff[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        const int rr = wave * 64 + q * 8 + (lane >> 3);
        const int m = m0 + rr < M ? m0 + rr : M - 1;
        aoff[q] = (uint32_t)m * (uint32_t)K * 2u + 16u * (uint32_t)((lane & 7) ^ (rr & 7));
    }
    // packed weights of the wave's columns: instruction nb -> rows 32nb + lane/2, half lane%2 (16 B = one scale
    // group); lane l's 16 bytes land at LDS position l of the block
    const uint8_t *bsrc[WNB];
#pragma unroll
    for (int nb = 0; nb < WNB; ++nb) {
        const int nn = n0 + col0 + nb * 32 + (lane >> 1);
        bsrc[nb] = wp + (size_t)(nn < N ? nn : N - 1) * (size_t)(K >> 1) + (lane & 1) * 16;
    }
    // scales: instruction h -> rows 64h + lane, 8 groups (256 k) per request
    constexpr int SCI = C::COLS / 64;
    const uint16_t *ssrc[SCI];
#pragma unroll
    for (int h = 0; h < SCI; ++h) {
        const int nn = n0 + col0 + h * 64 + lane;
        ssrc[h] = sc + (size_t)(nn < N ? nn : N - 1) * G;
    }
    uint8_t *const a_lds = lds + wave * 64 * 128;  // + stage * A_STAGE + q * 1024
    uint8_t *const bp_lds = lds + C::BP_OFF + wave * C::BP_WAVE;
    uint8_t *const sc_lds = lds + C::SC_OFF + wave * C::SC_WAVE;

    auto issue_a = [&](int step, int q0, int nq) {  // instructions q0 .. q0+nq-1 of the step's eight
        const uint8_t *src = reinterpret_cast<const uint8_t *>(x) + (size_t)step * (BK * 2);
        uint8_t *dst = a_lds + (step % A_STAGES) * A_STAGE;
#pragma unroll
        for (int q = 0; q < 8; ++q)
            if (q >= q0 && q < q0 + nq) dma16_to_lds(src + aoff[q], dst + q * 1024);
    };
    auto issue_bp = [&](int step) {
        uint8_t *dst = bp_lds + (step & 1) * C::BP_SLOT;
#pragma unroll
        for (int nb = 0; nb < WNB; ++nb) dma16_to_lds(bsrc[nb] + (size_t)step * (BK / 2), dst + nb * 1024);
    };
    auto issue_sc = [&](int blk) {
#pragma unroll
        for (int h = 0; h < SCI; ++h) dma16_to_lds(ssrc[h] + blk * 8, sc_lds + (blk & 1) * C::SC_SLOT + h * 1024);
    };

    // ---- fragment read offsets: row nl of a 32-row block, piece 4kq + t at position (4kq + t) ^ (row & 7)
    uint32_t foff[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) foff[t] = (uint32_t)((row0 + nl) * 128 + (((4 * kq + t) ^ (nl & 7)) << 4));

    const uint32_t c_mlo = vgpr_const(0x000F000Fu), c_mhi = vgpr_const(0x00F000F0u), c_magic = vgpr_const(0x64006400u);

    f32x16 acc[WMB][WNB];
#pragma unroll
    for (int a = 0; a < WMB; ++a)
#pragma unroll
        for (int b = 0; b < WNB; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

    // the lane's packed weights and scales of a step: row 32nb + nl, group kq
    u32x4 bq[WNB];
    uint16_t sraw[WNB];
    float cs[WNB][4];
    auto deq_fetch = [&](int step) {  // LDS reads only; deq_prep turns the scales into the FMA constants
        const uint8_t *slot = bp_lds + (step & 1) * C::BP_SLOT;
        const uint8_t *ss = sc_lds + ((step >> 2) & 1) * C::SC_SLOT;
#pragma unroll
        for (int nb = 0; nb < WNB; ++nb) {
            bq[nb] = *reinterpret_cast<const u32x4 *>(slot + nb * 1024 + (2 * nl + kq) * 16);
            sraw[nb] = *reinterpret_cast<const uint16_t *>(ss + (nb * 32 + nl) * 16 + ((step & 3) * 2 + kq) * 2);
        }
    };
    auto deq_prep = [&]() {
#pragma unroll
        for (int nb = 0; nb < WNB; ++nb) {
            const float s = f16_bits_to_f32(sraw[nb]);
            cs[nb][0] = s;
            cs[nb][1] = s * 0.0625f;
            cs[nb][2] = -1032.f * s;
            cs[nb][3] = -72.f * s;
        }
    };
    bf16x8 bf[2][4][WNB];  // [set][slice t][n-block]
    auto deq_slice = [&](int set, int t) {
#pragma unroll
        for (int nb = 0; nb < WNB; ++nb) {
            const uint32_t w = t == 0 ? bq[nb].x : t == 1 ? bq[nb].y : t == 2 ? bq[nb].z : bq[nb].w;
            bf[set][t][nb] = dequant8_i4(w, cs[nb][0], cs[nb][1], cs[nb][2], cs[nb][3], c_mlo, c_mhi, c_magic);
        }
    };

    // ---- prologue: scales of the first four steps, packed weights of steps 0 and 1, activations of steps 0 and 1
    issue_sc(0);
    issue_bp(0);
    if (steps > 1) issue_bp(1);
    issue_a(0, 0, 8);
    if (steps > 1) issue_a(1, 0, 8);
    if (steps > 1) wait_vmcnt<8>();  // everything but A(1)
    else wait_vmcnt<0>();
    deq_fetch(0);
    deq_prep();
#pragma unroll
    for (int t = 0; t < 4; ++t) deq_slice(0, t);
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    wg_barrier();

    // Step i: MFMAs on A(i) and the weights dequantised during step i-1; meanwhile the packed weights of step i+2 and
    // then A(i+2) are requested (spread over the slices: a burst of requests stalls the wave at their issue) and the
    // weights of step i+1 are dequantised.  The workgroup meets once per step, in front of the step's LAST slice:
    // that slice's fragments are in registers by then, so its MFMAs cover the LDS round trip of the next step's
    // first fragments, which may only be read after the barrier.  Memory returns in order, so "no more outstanding
    // than the six requests of A(i+2) issued so far" means A(i+1) and the packed weights of step i+2 have landed.
    bf16x8 af[2][WMB];
    auto read_frags = [&](int buf, int step, int t) {
        const uint8_t *ab = lds + (step % A_STAGES) * A_STAGE;
#pragma unroll
        for (int mb = 0; mb < WMB; ++mb) af[buf][mb] = *reinterpret_cast<const bf16x8 *>(ab + mb * 4096 + foff[t]);
    };
    read_frags(0, 0, 0);
    auto step_body = [&](int i, auto set_c, auto more1_c, auto more2_c) {
        constexpr int set = decltype(set_c)::value;       // which set of dequantised weights this step consumes
        constexpr bool more1 = decltype(more1_c)::value;  // step i+1 exists
        constexpr bool more2 = decltype(more2_c)::value;  // step i+2 exists
        if (more1) deq_fetch(i + 1);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if (t < 3) {
                read_frags((t + 1) & 1, i, t + 1);  // requested before this slice's MFMAs
            } else if (more1) {
                if (more2) wait_vmcnt<6>();
                else wait_vmcnt<0>();
                __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this step's fragment reads are done
                wg_barrier();
                read_frags(0, i + 1, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int mb = 0; mb < WMB; ++mb)
#pragma unroll
                for (int nb = 0; nb < WNB; ++nb)
                    acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[t & 1][mb], bf[set][t][nb], acc[mb][nb], 0, 0, 0);
            if (t == 0) {  // the packed weights (and scales) go out before any of A(i+2)
                if (((i + 3) & 3) == 0 && i + 3 < steps) issue_sc((i + 3) >> 2);
                if (more2) issue_bp(i + 2);
                if (more1) deq_prep();
            } else if (more2) {
                issue_a(i + 2, t == 1 ? 0 : t == 2 ? 3 : 6, t == 3 ? 2 : 3);
            }
            if (more1) deq_slice(set ^ 1, t);
        }
    };
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    using T = std::true_type;
    using F = std::false_type;
    int i = 0;
    for (; i + 3 < steps; i += 2) {  // steady state: steps i+2 and i+3 exist
        step_body(i, S0{}, T{}, T{});
        step_body(i + 1, S1{}, T{}, T{});
    }
    // the last one to three steps (i is even here)
    const int left = steps - i;
    if (left == 3) {
        step_body(i, S0{}, T{}, T{});
        step_body(i + 1, S1{}, T{}, F{});
        step_body(i + 2, S0{}, F{}, F{});
    } else if (left == 2) {
        step_body(i, S0{}, T{}, F{});
        step_body(i + 1, S1{}, F{}, F{});
    } else {
        step_body(i, S0{}, F{}, F{});
    }

    // ---- epilogue.  The lane holds, for every (mb, nb), column nl of rows 8*(v/4) + 4*kq + v%4 of a 32 x 32 block.
    // Stored from there, every instruction would write 2 bytes per lane in two 64-byte runs.  Instead the results go
    // through a tile of the wave's own in LDS as bf16, 128 rows at a time, and leave as whole rows: neighbouring lanes
    // first swap one value of each row pair (one DPP move), so that a lane writes two adjacent columns of one row as a
    // 32-bit word; the tile is then read back 16 bytes per lane.
    wg_barrier();  // every wave is done reading the activation stages, which the tiles reuse
    constexpr int EP = C::EP_PITCH, HALVES = WMB / 4, LPR = C::COLS / 8;  // 16-byte pieces (lanes) per tile row
    uint8_t *const ep = lds + wave * (128 * EP);
    const bool odd = lane & 1;
    const bool y_vec = ((N & 7) == 0) && ((reinterpret_cast<uintptr_t>(y) & 15u) == 0);
#pragma unroll
    for (int hf = 0; hf < HALVES; ++hf) {
#pragma unroll
        for (int mq = 0; mq < 4; ++mq)
#pragma unroll
            for (int nb = 0; nb < WNB; ++nb)
#pragma unroll
                for (int v = 0; v < 16; v += 2) {
                    const float a0 = acc[hf * 4 + mq][nb][v], a1 = acc[hf * 4 + mq][nb][v + 1];  // rows r and r+1, column nl
                    const float send = odd ? a0 : a1;
                    const float recv = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(send), 0xB1, 0xF, 0xF, false));  // lane ^ 1
                    // even lane: row r, columns (nl, nl+1) = (own a0, neighbour's a0); odd lane: row r+1, columns (nl-1, nl)
                    const uint32_t word = odd ? pack_bf16_rne(recv, a1) : pack_bf16_rne(a0, recv);
                    const int row = mq * 32 + 8 * (v >> 2) + 4 * kq + (v & 3) + (odd ? 1 : 0);
                    const int col = nb * 32 + (nl & ~1);
                    *reinterpret_cast<uint32_t *>(ep + row * EP + col * 2) = word;
                }
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the wave's own tile is written (no other wave touches it)
#pragma unroll 4
        for (int p = 0; p < 128 * LPR / 64; ++p) {
            const int row = p * (64 / LPR) + lane / LPR, c8 = (lane % LPR) * 8;
            const u32x4 o = *reinterpret_cast<const u32x4 *>(ep + row * EP + c8 * 2);
            const int m = m0 + row0 + hf * 128 + row, n = n0 + col0 + c8;
            if (m < M) {
                uint16_t *yp = y + (size_t)m * N + n;
                if (y_vec && n + 8 <= N) {
                    *reinterpret_cast<u32x4 *>(yp) = o;
                } else {
                    const uint32_t w4[4] = {o.x, o.y, o.z, o.w};
                    for (int e = 0; e < 8; ++e)
                        if (n + e < N) yp[e] = (uint16_t)(w4[e >> 1] >> (16 * (e & 1)));
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): read out before the next half overwrites the tile
    }
}

bool gemm_big_i4g32_ok(const uint16_t *x, const uint8_t *wp, const uint16_t *sc, int M, int N, int K) {
    return K % 256 == 0 && aligned16(x) && aligned16(wp) && aligned16(sc) && (int64_t)M * K * 2 < ((int64_t)1 << 32);
}

template <int WM, int WN>
static int launch_big(const uint16_t *x, const uint8_t *wp, const uint16_t *sc, uint16_t *y, int M, int N, int K, hipStream_t st) {
    typedef big::Cfg<WM, WN> C;
    static std::atomic<bool> attr_set{false};
    if (!attr_set.load(std::memory_order_acquire)) {
        CHADQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_big_i4g32_kernel<WM, WN>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES));
        attr_set.store(true, std::memory_order_release);
    }
    const int tiles = ((N + big::BN - 1) / big::BN) * ((M + big::BM - 1) / big::BM);
    const int grid = ((tiles + 7) / 8) * 8;
    hipLaunchKernelGGL((gemm_big_i4g32_kernel<WM, WN>), dim3(grid), dim3(256), C::LDS_BYTES, st, x, wp, sc, y, M, N, K);
    return hip_check(hipGetLastError(), "gemm_big_i4g32 launch");
}

int gemm_big_i4g32_launch(const uint16_t *x, const uint8_t *wp, const uint16_t *sc, uint16_t *y, int M, int N, int K,
                          hipStream_t st) {
    return launch_big<1, 4>(x, wp, sc, y, M, N, K, st);
}

}  // namespace chadq
