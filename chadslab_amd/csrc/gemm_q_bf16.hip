// Prefill dequant-GEMM:  y[m,n] = bf16( sum_k x[m,k] * w[n,k] ),  x bf16 [M,K], fp32 accumulate on MFMA.
//   int4 group-32:  w = bf16_rne((u-8) * scale[n,k/32])          (dequantised to bf16 for the matrix core)
//   int8 per-row :  w = W[n,k] exactly in bf16, scale[n] applied to the fp32 accumulator afterwards
//
// Workgroup = 4 waves, output tile 128 x 64, and the four waves split K: wave w owns every fourth slice of
// K and accumulates a full 128 x 64 partial tile (8 accumulators of v_mfma_f32_32x32x16_bf16).  That choice
// makes both operands private to a wave:
//   * B (weights): lane (n = lane%32, kq = lane/32) owns 16 packed bytes of output row n per iteration, which
//     is 32 k (int4, exactly one scale group) or 16 k (int8).  They arrive by direct global->LDS load in a
//     wave-private slot (fetched so that the two pieces of a row come from neighbouring lanes: one 32-byte
//     request), the owning lane reads them back, dequantises them in registers (fp16 magic numbers, one fp32 FMA
//     per element, RNE to bf16) and feeds them to the MFMA.  No other wave ever needs them.
//   * A (activations): the wave moves its own 128 x KW slice into a wave-private, double-buffered LDS tile with
//     direct global->LDS loads (global_load_lds_dwordx4: 8 rows x 128 B per instruction, no VGPR round trip),
//     purely to turn row-major memory into MFMA fragments.  16-byte pieces are XOR-swizzled by row so that
//     fragment reads are bank-conflict free.  No other wave reads the tile, so the main loop has no barriers.
//     The tile lives in a ring of eight 32-row slots (two iterations); a slot is refilled for iteration i+2 as
//     soon as iteration i has consumed it, and the weights of i+1 are dequantised between i's MFMAs.
// The MFMA k-slot of a lane is free to choose as long as A and B agree: slot group kq covers the kq-th
// 16-byte weight load, and step t of that load is its t-th 8-k word.
// The four partial tiles are summed through LDS at the end, rounded to bf16 (RNE) and stored coalesced.
#include <type_traits>

#include "chadq_common.h"

#ifndef CHADQ_GEMM_ABLATE
#define CHADQ_GEMM_ABLATE 0  // measurement builds only: 1 = the dequantisation compiled out (packed words go to the matrix core as they are)
#endif

namespace chadq {

struct FmtI4G32 {
    static constexpr int KL = 32;  // k per 16-byte weight load
    typedef uint16_t scale_t;
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

constexpr int BM = 128, NWAVE = 4;

template <typename F, int NB>
struct Tile {
    static constexpr int BN = 32 * NB;              // output columns per workgroup: NB n-blocks of 32
    static constexpr int KL = F::KL;
    static constexpr int KW = 2 * KL;               // k per wave per iteration (two 16-byte loads side by side)
    static constexpr int KIT = NWAVE * KW;          // k per workgroup iteration
    static constexpr int T = KL / 8;                // MFMA steps per 16-byte load
    static constexpr int ROWB = KW * 2;             // LDS row bytes (128 for int4, 64 for int8)
    static constexpr int PPR = ROWB / 16;           // 16-byte pieces per row (8 or 4)
    static constexpr int RPL = 8 / PPR;             // rows per 128 bytes of LDS (1 or 2)
    static constexpr int RPI = 64 / PPR;            // rows per DMA instruction (8 or 16)
    static constexpr int DPM = 32 / RPI;            // DMA instructions per 32-row m-block (4 or 2)
    static constexpr int SLOT_BYTES = 32 * ROWB;    // one m-block of one iteration
    static constexpr int NSLOT = 8;                 // ring: two iterations of four m-blocks
    static constexpr int A_BYTES = NWAVE * NSLOT * SLOT_BYTES;
    // weights and scales of one iteration of one wave: NB x 1 KiB of weights (16 B per lane) + 1 KiB for the scales
    // (general form: 2 bytes in a 4-byte place per lane and n-block; unguarded int4 form: 16 bytes per weight row)
    static constexpr int BSLOT_BYTES = NB * 1024 + 1024;
    static constexpr int B_OFF = A_BYTES;
    static constexpr int STAGE_BYTES = A_BYTES + NWAVE * BSLOT_BYTES;
    static constexpr int EPI_BYTES = NWAVE * BM * 32 * 4;
    static constexpr int LDS_BYTES = STAGE_BYTES > EPI_BYTES ? STAGE_BYTES : EPI_BYTES;
};

// 16-byte piece `piece` of row `row` lives in slot piece ^ key(row): fragment reads of 8 consecutive rows
// then hit 8 different 16-byte bank groups.
template <typename TL>
__device__ __forceinline__ int swz(int row, int piece) { return piece ^ ((row / TL::RPL) % TL::PPR); }

// GUARD = false assumes K is a multiple of the workgroup's k step (no range checks in the loop).
// OUTF32: y is fp32 [M,N] instead of bf16.  groups != nullptr: grouped launch, blockIdx.y selects a descriptor
// (activations, weights, output and row count of one group; N and K are common) - this is how the MoE expert
// GEMMs run as one launch over experts whose row counts only the GPU knows.
template <typename F, int NB, bool GUARD, bool OUTF32>
__global__ __launch_bounds__(256) void gemm_q_bf16_kernel(const uint16_t *__restrict__ x, const void *__restrict__ wq,
                                                          const typename F::scale_t *__restrict__ sc,
                                                          uint16_t *__restrict__ y, int M, int N, int K,
                                                          const GemmGroup *__restrict__ groups) {
    typedef Tile<F, NB> TL;
    if (groups) {
        const GemmGroup g = groups[blockIdx.y];
        x = g.x;
        wq = g.w;
        sc = reinterpret_cast<const typename F::scale_t *>(g.sc);
        y = reinterpret_cast<uint16_t *>(g.y);
        M = g.M;
    }
    constexpr int BN = TL::BN;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: LDS and global bases stay in SGPRs
    const int nl = lane & 31, kq = lane >> 5;
    // Tile order.  Workgroup i runs on XCD i % 8 (each XCD has its own 4 MiB L2), so tiles are dealt out such
    // that one XCD walks consecutive n-tiles of the same m-panel: the 128-row activation panel then stays in
    // that XCD's L2 while the weights stream past, instead of every L2 seeing every panel.
    const int tiles_n = (N + BN - 1) / BN, tiles = tiles_n * ((M + BM - 1) / BM);
    const int wg = blockIdx.x, per_xcd = (tiles + 7) / 8;
    const int tile = (wg % 8) * per_xcd + wg / 8;
    if (tile >= tiles) return;
    const int m0 = (tile / tiles_n) * BM, n0 = (tile % tiles_n) * BN;
    uint8_t *ring = lds + wave * (TL::NSLOT * TL::SLOT_BYTES);
    constexpr bool i4 = (TL::KL == 32);
    const size_t wrow_bytes = i4 ? (size_t)(K >> 1) : (size_t)K;
    const int G = K >> 5;

    f32x16 acc[4][NB];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

    // Weight rows (clamped so that loads stay in bounds; results for n >= N are never stored).  The weight request of
    // n-block nb is issued with lane l fetching piece l % 2 of row l / 2, so that the two 16-byte pieces of a row come
    // from neighbouring lanes (one 32-byte request, not two of 16); lane (nl, kq) reads its operand back from LDS
    // position 2 * nl + kq.  Scales in the general form stay one 2-byte request per lane (nl, kq).
    const int wl_row = lane >> 1, wl_kq = lane & 1;
    const uint8_t *wbase[NB];
    const uint16_t *sbase[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int nw = n0 + nb * 32 + wl_row, n = n0 + nb * 32 + nl;
        wbase[nb] = (const uint8_t *)wq + (size_t)(nw < N ? nw : N - 1) * wrow_bytes;  // row starts; k offsets are added per load
        sbase[nb] = (const uint16_t *)sc + (size_t)(n < N ? n : N - 1) * G;
    }
    // Scales, unguarded form: one request per iteration fetches, for each of the tile's 32*NB weight rows (lane -> row),
    // the aligned 16 bytes = 8 groups = this iteration's 256 k of all four waves; a lane later picks its own group.
    // (Two requests of 2 bytes per lane, the general form, cost 9 % of the kernel's time: requests, not bytes, count.)
    constexpr bool SBLK = i4 && !GUARD && NB == 2;
    const uint16_t *srow_blk = nullptr;
    if (SBLK) {
        const int n = n0 + lane;
        srow_blk = (const uint16_t *)sc + (size_t)(n < N ? n : N - 1) * G;
    }
    // DMA: LDS position lane*16 inside each 1 KiB block is (row dr, slot dslot); the piece that belongs there is
    // dslot ^ key(row).  Per-lane byte offsets into x are 32-bit (the host checks M*K*2 < 2^32); the k advance
    // per iteration goes into the scalar base.
    const int dr = lane / TL::PPR, dslot = lane % TL::PPR;
    uint32_t doff[4 * TL::DPM], drow[4 * TL::DPM];
    int dpiece[4 * TL::DPM];
#pragma unroll
    for (int i = 0; i < 4 * TL::DPM; ++i) {
        const int row = i * TL::RPI + dr;
        const int m = m0 + row < M ? m0 + row : M - 1;
        dpiece[i] = swz<TL>(row, dslot);
        drow[i] = (uint32_t)m * (uint32_t)K * 2u;  // byte offset of the row start
        doff[i] = drow[i] + 16u * dpiece[i];
    }
    const uint8_t *xw = reinterpret_cast<const uint8_t *>(x) + (size_t)wave * TL::KW * 2;  // scalar

    auto issue_dma = [&](int it, int mb) {
        const uint8_t *src = xw + (size_t)it * TL::KIT * 2;
        uint8_t *dst = ring + ((it & 1) * 4 + mb) * TL::SLOT_BYTES;
        const int kb = it * TL::KIT + wave * TL::KW;
#pragma unroll
        for (int q = 0; q < TL::DPM; ++q) {
            const int i = mb * TL::DPM + q;
            const uint8_t *ptr = src + doff[i];  // = x + (m*K + kb + 8*piece) * 2, inside row m when kb+8*piece < K
            // columns past K: fetch the start of the row instead (they only ever meet zero weights)
            if (GUARD && kb + 8 * dpiece[i] >= K) ptr = reinterpret_cast<const uint8_t *>(x) + drow[i];
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)ptr,
                                             (__attribute__((address_space(3))) void *)(dst + q * 1024), 16, 0, 0);
        }
    };
    // Weights take the same road: a lane DMAs 16 packed bytes (and, for int4 in the general form, lane (nl, kq) its
    // group's scale) into a wave-private slot; lane (nl, kq) reads its operand back one iteration later.  With every
    // global access a DMA, the explicit counts below are the only waits on vector memory in the loop.
    uint8_t *bslot = lds + TL::B_OFF + wave * TL::BSLOT_BYTES;
    auto issue_b = [&](int it) {
        const int kw = it * TL::KIT + wave * TL::KW + kq * TL::KL;  // first k of the 16 bytes lane (nl, kq) will use
        const int kc = (!GUARD || kw < K) ? kw : 0;                   // past K: the row start, zeroed on use
        const int kww = it * TL::KIT + wave * TL::KW + wl_kq * TL::KL;  // first k of the 16 bytes this lane fetches
        const int kcw = (!GUARD || kww < K) ? kww : 0;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(wbase[nb] + (i4 ? kcw / 2 : kcw)),
                                             (__attribute__((address_space(3))) void *)(bslot + nb * 1024), 16, 0, 0);
            if (i4 && !SBLK)
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(sbase[nb] + (kc >> 5)),
                                                 (__attribute__((address_space(3))) void *)(bslot + NB * 1024 + nb * 256), 2, 0, 0);
        }
        if (SBLK) dma16_to_lds(srow_blk + it * (TL::KIT / 32), bslot + NB * 1024);
    };
    const uint32_t c_mlo = vgpr_const(0x000F000Fu), c_mhi = vgpr_const(0x00F000F0u), c_magic = vgpr_const(0x64006400u);
    bf16x8 bf[2][TL::T][NB];  // [set][step][n-block]: dequantised weights of one iteration
    u32x4 cq[NB];                // the lane's packed weights of the iteration being dequantised
    float cs[NB][4];             // int4: s, s/16, -1032 s, -72 s
    auto fetch_b = [&](int it) {  // LDS -> registers, once per iteration; frees the slot for the next request
        const bool live = !GUARD || ((it * TL::KIT + wave * TL::KW + kq * TL::KL) < K);
        const uint8_t *src = bslot;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            cq[nb] = *reinterpret_cast<const u32x4 *>(src + nb * 1024 + (2 * nl + kq) * 16);
            if constexpr (i4) {
                const uint16_t sb16 = SBLK ? *reinterpret_cast<const uint16_t *>(src + NB * 1024 + (nb * 32 + nl) * 16 + (2 * wave + kq) * 2)
                                           : *reinterpret_cast<const uint16_t *>(src + NB * 1024 + nb * 256 + lane * 4);
                const float s = live ? f16_bits_to_f32(sb16) : 0.f;
                cs[nb][0] = s;
                cs[nb][1] = s * 0.0625f;
                cs[nb][2] = -1032.f * s;
                cs[nb][3] = -72.f * s;
            } else if (!live) {
                cq[nb] = u32x4{0, 0, 0, 0};  // int8 zero is the value zero
            }
        }
    };
    auto dequant_step = [&](int set, int t) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const u32x4 q = cq[nb];
            if constexpr (CHADQ_GEMM_ABLATE == 1) {
                const u32x4 raw = {q.x + (uint32_t)t, q.y, q.z, q.w};
                __builtin_memcpy(&bf[set][t][nb], &raw, 16);
            } else if constexpr (i4) {
                const uint32_t wsel = t == 0 ? q.x : t == 1 ? q.y : t == 2 ? q.z : q.w;
                bf[set][t][nb] = dequant8_i4(wsel, cs[nb][0], cs[nb][1], cs[nb][2], cs[nb][3], c_mlo, c_mhi, c_magic);
            } else {
                bf[set][t][nb] = t == 0 ? FmtI8Row::dequant(q.x, q.y) : FmtI8Row::dequant(q.z, q.w);
            }
        }
    };

    const int iters = (K + TL::KIT - 1) / TL::KIT;
    constexpr int DPM = TL::DPM, NBL = SBLK ? NB + 1 : (i4 ? 2 : 1) * NB, LPI = 4 * DPM + NBL;  // VMEM instructions: m-block, weights, iteration
    // Request order (memory returns in order, so "X has landed" is "at most so many younger requests are out"):
    //   prologue   W(0) T(0,0..3) | W(1) T(1,0..3)          W = weights+scales of an iteration, T(i,mb) = m-block
    //   iteration i issues, after consuming m-block mb, the refill T(i+2,mb); W(i+2) goes out right after the
    //   first refill, once W(i+1) has been moved from its (single) LDS slot into registers:
    //              T(i+2,0) W(i+2) T(i+2,1) T(i+2,2) T(i+2,3)
    // Counts used below are the smallest number of requests that can be younger than the awaited one in any
    // of these layouts (a smaller count only waits a little longer, never too little).
    issue_b(0);
#pragma unroll
    for (int mb = 0; mb < 4; ++mb) issue_dma(0, mb);
    wait_vmcnt<4 * DPM>();  // W(0) is in; T(0,*) may still be out
    fetch_b(0);
    if (iters > 1) {
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the slot has been read before it is requested again
        issue_b(1);
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) issue_dma(1, mb);
    }
#pragma unroll
    for (int t = 0; t < TL::T; ++t) dequant_step(0, t);

    auto iteration = [&](int it, auto set_c, auto more1_c, auto more2_c) {
        constexpr int set = decltype(set_c)::value;
        constexpr bool more1 = decltype(more1_c)::value, more2 = decltype(more2_c)::value;  // it+1 / it+2 exist
        const uint8_t *abase = ring + set * 4 * TL::SLOT_BYTES;
        // The activation fragments of m-block mb+1 are read from LDS while the MFMAs of m-block mb run (a read
        // placed right in front of its MFMA costs an exposed LDS round trip, 16 of them per iteration).
        bf16x8 af[2][TL::T];
        auto read_frags = [&](int buf, int mb) {
            const uint8_t *ab = abase + mb * TL::SLOT_BYTES;
#pragma unroll
            for (int t = 0; t < TL::T; ++t)
                af[buf][t] = *reinterpret_cast<const bf16x8 *>(ab + nl * TL::ROWB + swz<TL>(nl, kq * TL::T + t) * 16);
        };
        // T(it, 0) has landed: younger are the rest of its group, the group of it+1 (nothing issued yet by `it`)
        if (more1) wait_vmcnt<3 * DPM + LPI>();
        else wait_vmcnt<3 * DPM>();
        read_frags(0, 0);
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) {
            if (mb < 3) {
                // T(it, mb+1) has landed.  Younger: T(it, mb+2..3), the group of it+1, and what `it` has issued so
                // far: the refills of m-blocks 0..mb-1 and, once the first of them is out, the weights of it+2.
                if (more2) {
                    if (mb == 0) wait_vmcnt<2 * DPM + LPI>();
                    else wait_vmcnt<2 * DPM + LPI + NBL>();
                } else if (more1) {
                    if (mb == 0) wait_vmcnt<2 * DPM + LPI>();
                    if (mb == 1) wait_vmcnt<1 * DPM + LPI>();
                    if (mb == 2) wait_vmcnt<LPI>();
                } else {
                    if (mb == 0) wait_vmcnt<2 * DPM>();
                    if (mb == 1) wait_vmcnt<1 * DPM>();
                    if (mb == 2) wait_vmcnt<0>();
                }
                read_frags((mb + 1) & 1, mb + 1);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < TL::T; ++t)
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
                    acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[mb & 1][t], bf[set][t][nb], acc[mb][nb], 0, 0, 0);
            if (more2) issue_dma(it + 2, mb);  // the slot just consumed
            // next iteration's weights become MFMA operands while this iteration's MFMAs run
            if (more1) {
                if (mb == 0) {
                    // W(it+1) has landed: younger are T(it+1,1..3) and, if issued, the refill above
                    if (more2) wait_vmcnt<4 * DPM>();
                    else wait_vmcnt<3 * DPM>();
                    fetch_b(it + 1);
                    if (more2) {
                        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): read out before it is requested again
                        issue_b(it + 2);
                    }
                }
                if (mb < TL::T) dequant_step(set ^ 1, mb);
            }
        }
    };
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    int it = 0;
    for (; it + 3 < iters; it += 2) {  // steady state: no conditions inside, so the scheduler sees one block
        iteration(it, S0{}, std::true_type{}, std::true_type{});
        iteration(it + 1, S1{}, std::true_type{}, std::true_type{});
    }
    // the last one to three iterations (it is even here)
    const int left = iters - it;
    if (left == 3) {
        iteration(it, S0{}, std::true_type{}, std::true_type{});
        iteration(it + 1, S1{}, std::true_type{}, std::false_type{});
        iteration(it + 2, S0{}, std::false_type{}, std::false_type{});
    } else if (left == 2) {
        iteration(it, S0{}, std::true_type{}, std::false_type{});
        iteration(it + 1, S1{}, std::false_type{}, std::false_type{});
    } else if (left == 1) {
        iteration(it, S0{}, std::false_type{}, std::false_type{});
    }

    // cross-wave sum, one 128 x 32 half tile at a time: [wave][row][32] fp32 in LDS
    const bool y_vec = ((N & 3) == 0) && ((reinterpret_cast<uintptr_t>(y) & 15u) == 0);
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
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
                if constexpr (!i4) {
                    const float *scf = (const float *)sc;
                    s.x *= (n + 0 < N) ? scf[n + 0] : 0.f;
                    s.y *= (n + 1 < N) ? scf[n + 1] : 0.f;
                    s.z *= (n + 2 < N) ? scf[n + 2] : 0.f;
                    s.w *= (n + 3 < N) ? scf[n + 3] : 0.f;
                }
                if constexpr (OUTF32) {
                    float *yp = reinterpret_cast<float *>(y) + (size_t)m * N + n;
                    if (n + 3 < N && y_vec) {
                        *reinterpret_cast<f32x4 *>(yp) = s;
                    } else {
                        const float sv[4] = {s.x, s.y, s.z, s.w};
                        for (int j = 0; j < 4; ++j)
                            if (n + j < N) yp[j] = sv[j];
                    }
                } else {
                    uint16_t *yp = y + (size_t)m * N + n;
                    if (n + 3 < N && y_vec) {
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
    }
}

template <typename F, int NB, bool GUARD, bool OUTF32>
static int launch_gemm_g(const uint16_t *x, const void *wq, const typename F::scale_t *sc, void *y, int M, int N,
                         int K, const GemmGroup *groups, int ngroups, hipStream_t st) {
    typedef Tile<F, NB> TL;
    static std::atomic<bool> attr_set{false};  // setting it twice from two threads is harmless
    if (!attr_set.load(std::memory_order_acquire)) {
        CHADQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_q_bf16_kernel<F, NB, GUARD, OUTF32>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, TL::LDS_BYTES));
        attr_set.store(true, std::memory_order_release);
    }
    const int tiles = ((N + TL::BN - 1) / TL::BN) * ((M + BM - 1) / BM);  // M = the largest group in a grouped launch
    const int grid = ((tiles + 7) / 8) * 8;  // a multiple of the 8 XCDs; surplus workgroups exit at once
    hipLaunchKernelGGL((gemm_q_bf16_kernel<F, NB, GUARD, OUTF32>), dim3(grid, groups ? ngroups : 1), dim3(256),
                       TL::LDS_BYTES, st, x, wq, sc, reinterpret_cast<uint16_t *>(y), M, N, K, groups);
    return hip_check(hipGetLastError(), "gemm_q_bf16 launch");
}

// NB = 2 (128 x 64 tiles).  The kernel is written for any NB; NB = 4 halves the traffic on the activation panel
// but needs 256 accumulator registers plus two sets of dequantised operands and spills, so it is not instantiated.
template <typename F, bool OUTF32>
static int launch_gemm(const uint16_t *x, const void *wq, const typename F::scale_t *sc, void *y, int M, int N, int K,
                       const GemmGroup *groups, int ngroups, hipStream_t st) {
    CHADQ_REQUIRE((int64_t)M * K * 2 < ((int64_t)1 << 32), CHADQ_ERR_SHAPE,
                  "gemm: activations of %d x %d exceed the 4 GiB the kernel's 32-bit offsets cover", M, K);
    // the unguarded int4 form fetches scale rows 16 bytes at a time: it needs 16-byte aligned scale rows, which only a
    // plain launch can check here (a grouped launch's pointers live in device memory)
    const bool scale_rows_ok = Tile<F, 2>::KL != 32 || (!groups && (reinterpret_cast<uintptr_t>(sc) & 15u) == 0);
    if (K % Tile<F, 2>::KIT != 0 || !scale_rows_ok)
        return launch_gemm_g<F, 2, true, OUTF32>(x, wq, sc, y, M, N, K, groups, ngroups, st);
    return launch_gemm_g<F, 2, false, OUTF32>(x, wq, sc, y, M, N, K, groups, ngroups, st);
}

bool gemm_big_i4g32_ok(const uint16_t *x, const uint8_t *wp, const uint16_t *sc, int M, int N, int K);
int gemm_big_i4g32_launch(const uint16_t *x, const uint8_t *wp, const uint16_t *sc, uint16_t *y, int M, int N, int K, hipStream_t st);

int gemm_i4g32_bf16_dispatch(const uint16_t *x, const uint8_t *wp, const uint16_t *sc, uint16_t *y, int M, int N,
                             int K, hipStream_t st) {
    // many rows: the 256 x 256 tile, which dequantises a weight once per 256 rows, as soon as its tiles cover most of
    // the chip (a tile alone on a compute unit takes about as long as all of them together: at 4096 columns the small
    // tile is still ahead at 2048 rows, 101 against 115 us)
    const int64_t big_tiles = (int64_t)((M + 255) / 256) * ((N + 255) / 256);
    if (big_tiles >= 176 && gemm_big_i4g32_ok(x, wp, sc, M, N, K)) return gemm_big_i4g32_launch(x, wp, sc, y, M, N, K, st);
    return launch_gemm<FmtI4G32, false>(x, wp, sc, y, M, N, K, nullptr, 0, st);
}

int gemm_i8row_bf16_dispatch(const uint16_t *x, const int8_t *w8, const float *sc, uint16_t *y, int M, int N, int K,
                             hipStream_t st) {
    return launch_gemm<FmtI8Row, false>(x, w8, sc, y, M, N, K, nullptr, 0, st);
}

// One launch over `ngroups` int4 group-32 products that share N and K; m_max bounds every group's row count.
int gemm_i4g32_grouped(const GemmGroup *groups, int ngroups, int m_max, int N, int K, bool out_f32, hipStream_t st) {
    if (out_f32) return launch_gemm<FmtI4G32, true>(nullptr, nullptr, nullptr, nullptr, m_max, N, K, groups, ngroups, st);
    return launch_gemm<FmtI4G32, false>(nullptr, nullptr, nullptr, nullptr, m_max, N, K, groups, ngroups, st);
}

}  // namespace chadq
