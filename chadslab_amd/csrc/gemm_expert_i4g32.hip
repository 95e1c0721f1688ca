// Grouped dequant-GEMM for the experts of the mixture-of-experts FFN on weights in TILE ORDER, and the preparation
// kernel that feeds it.  One workgroup = up to 96 tokens of one expert x 128*NB weight rows (4 waves x NB bands of
// 32 rows), as in gemm_skinny_i4g32.hip, but built for a loop that is bound by the matrix cores alone:
//
//   weights    come straight into registers: in tile order the 16 bytes a lane needs for one 64-k iteration of one band
//              are consecutive over the wave, so one load instruction fetches 1 KiB of contiguous memory and nothing
//              passes through LDS; four iterations are in flight per wave;
//   dequant    is fp16 arithmetic on pairs: (w & 0x000F000F) | 0x6400 reads 1024 + u, (w & 0x00F000F0) | 0x5400 reads
//              64 + u, and one v_pk_fma_f16 per pair with the constants -1024 s and -64 s (exact: powers of two) gives
//              fp16(u * s): 9 instructions per 8 weights where the bf16 form needs 17.  The zero point is not
//              subtracted here; see `correction`;
//   products   v_mfma_f32_32x32x16_f16.  The activations arrive as fp16, scaled per row by a power of two so that the
//              row's largest magnitude lies in [128, 256) (exact for bf16 inputs; the factor is undone in the
//              epilogue), each aligned run of 8 in the order 0,4,1,5,2,6,3,7 in which the dequantisation leaves the
//              weights.  expert_prep_kernel writes them, gathered into expert order;
//   correction sum_k x_k (u_k - 8) s_g = sum_k x_k u_k s_g - 8 s_g X_g with X_g the sum of the group's 32 activations:
//              a second product with one term per scale group.  The preparation also writes -8 X_g (fp16, as a high and
//              a low part), and once per 512 k one pair of MFMAs per accumulator block multiplies them with the
//              lane's scales of those 512 k, which are exactly the 8 values it already holds in registers: 1/16 more
//              matrix work instead of 4 more vector instructions per 8 weights.
//
// MODE 1 (gate/up): bands come in pairs (gate rows, up rows of the same 32 features); silu(gate) * up is formed in
//   registers and written as bf16.  MODE 0 (down): fp32 partial outputs, optionally split over K (blockIdx decoding as
//   in the skinny kernel); the combine kernel adds the parts.
// Needs K % 256 == 0, the K range of a split a multiple of 512, 64*NB | F (MODE 1), 128*NB | H (MODE 0), and scales
// below 64 in magnitude (1024 s must be finite in fp16).
#include "chadq_common.h"
#include "expert_prep.h"

namespace chadq {

typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;

constexpr int EX_MT = 96;              // tokens per workgroup tile
constexpr int EX_D = 3;                // iterations of 64 k requested ahead (activations and weights alike)
constexpr int EX_NS = EX_D + 1;        // activation stages / weight register sets
constexpr int EX_RING = EX_NS * (EX_MT / 32) * 4096;  // activation ring for the fullest tile: 48 KiB
constexpr int EX_LDS = EX_RING + 2 * EX_MT * 4;       // + the tile's row factors and row maxima

#ifndef CHADQ_EXPERT_ABLATE
#define CHADQ_EXPERT_ABLATE 0  // measurement builds only: 1 = memory traffic without arithmetic, 2 = arithmetic without weight loads
#endif

__device__ __forceinline__ uint32_t pk_fma_f16(uint32_t a, uint32_t b, uint32_t c) {
    uint32_t r;
    asm("v_pk_fma_f16 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ uint32_t pk_mul_f16(uint32_t a, uint32_t b) {
    uint32_t r;
    asm("v_pk_mul_f16 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}

struct ExConst {
    uint32_t mlo, mhi, magic_lo, magic_hi, m1024, m64;
};

// 8 nibbles of `w` (u0 lowest) -> 8 fp16 of u * s in the order u0,u4,u1,u5,u2,u6,u3,u7
__device__ __forceinline__ f16x8 dequant8_us(uint32_t w, uint32_t s_pk, uint32_t c_lo, uint32_t c_hi, const ExConst &c) {
    const uint32_t h0 = and_or(w, c.mlo, c.magic_lo);  // 1024 + (u0, u4)
    const uint32_t h1 = and_or(w, c.mhi, c.magic_hi);  // 64 + (u1, u5)
    const uint32_t w8 = w >> 8;
    const uint32_t h2 = and_or(w8, c.mlo, c.magic_lo);  // 1024 + (u2, u6)
    const uint32_t h3 = and_or(w8, c.mhi, c.magic_hi);  // 64 + (u3, u7)
    const u32x4 r = {pk_fma_f16(h0, s_pk, c_lo), pk_fma_f16(h1, s_pk, c_hi), pk_fma_f16(h2, s_pk, c_lo), pk_fma_f16(h3, s_pk, c_hi)};
    f16x8 o;
    __builtin_memcpy(&o, &r, 16);
    return o;
}

template <int MODE, int MB, int NB>
__device__ __forceinline__ void expert_body(const uint16_t *__restrict__ xa, const float *__restrict__ rs,
                                            const uint16_t *__restrict__ ghi, const uint16_t *__restrict__ glo, int G16,
                                            const int32_t *__restrict__ rowidx, uint32_t *__restrict__ rowmax,
                                            const uint8_t *__restrict__ w0, const uint8_t *__restrict__ s0,
                                            const uint8_t *__restrict__ w1, const uint8_t *__restrict__ s1, void *__restrict__ yv,
                                            int m0, int rows, int n0, int N, int K, int kbeg, int kend, uint8_t *lds) {
    constexpr int ASTAGE = MB * 4096;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nl = lane & 31, kq = lane >> 5;
    const int U = K >> 8;  // 256-k units per band

    // band nb of this wave -> first byte of the band's packed tiles / scale blocks, plus the lane's place in a 1-KiB
    // piece (16 B) / a 512-B scale block (8 B).  MODE 1: even bands are gate rows, odd bands the up rows of the same
    // 32 features.
    const uint8_t *wband[NB], *sband[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
        const int fb = (MODE == 1) ? (n0 >> 5) + wave * (NB / 2) + (nb >> 1) : (n0 >> 5) + wave * NB + nb;
        const uint8_t *wm = (MODE == 1 && (nb & 1)) ? w1 : w0, *sm = (MODE == 1 && (nb & 1)) ? s1 : s0;
        wband[nb] = wm + (size_t)fb * U * 4096 + lane * 16;
        sband[nb] = sm + (size_t)fb * U * 512 + lane * 8;
    }
    // activation pieces this lane requests: DMA instruction i of wave w fills LDS bytes (4i + w) * 1024 + 16 * lane of a
    // stage, i.e. row rr = (4i + w) * 8 + lane / 8, slot lane % 8, which holds piece slot ^ (rr & 7).  Rows past the
    // tile repeat its last row (their results are never stored).
    // The copy is the buffer form of the instruction (base in a resource descriptor, 32-bit byte offsets: the host
    // checks that the matrix stays below 2 GiB): the compiler then counts it like any other load, where the global form
    // makes it wait for every outstanding request whenever a loaded register is used.
    const __amdgpu_buffer_rsrc_t arsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(xa), 0, 0x7FFFFFFF, 0x00020000);
    uint32_t asrc[MB];
#pragma unroll
    for (int i = 0; i < MB; ++i) {
        const int rr = (4 * i + wave) * 8 + (lane >> 3), rc = rr < rows ? rr : rows - 1;
        const size_t srow = rowidx ? (size_t)rowidx[m0 + rc] : (size_t)(m0 + rc);  // gate/up: the token of the expert's row
        asrc[i] = (uint32_t)((srow * K + (((lane & 7) ^ (rr & 7)) << 3)) * 2);
        // A row past the tile is requested beyond the descriptor's range: the copy then delivers zeros.  Its products are
        // never stored either way, but the matrix cores run at the clock their power allows, and a multiplier fed zeros
        // draws less: a quarter of the rows of a typical routing are such padding.
        if (rr >= rows) asrc[i] = 0x80000000u;
    }
    // fragment read offsets: row mb*32 + nl, piece kq*4 + j lives in slot (kq*4 + j) ^ (nl & 7)
    uint32_t ard[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) ard[j] = (uint32_t)(nl * 128 + (((kq * 4 + j) ^ (nl & 7)) << 4));
    // the correction's activation-side operand: 8 values of row mb*32 + nl per 512 k, at element kq*8 of the block
    const uint16_t *chi[MB], *clo[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
        const int rr = mb * 32 + nl, rc = rr < rows ? rr : rows - 1;
        const size_t srow = rowidx ? (size_t)rowidx[m0 + rc] : (size_t)(m0 + rc);
        chi[mb] = ghi + srow * G16 + kq * 8;
        clo[mb] = glo + srow * G16 + kq * 8;
    }

    // the tile's row factors (and, MODE 1, its rows' running maxima) live in LDS behind the ring: the epilogue reads
    // them there instead of chasing row index -> factor through memory once per row
    float *l_rs = reinterpret_cast<float *>(lds + EX_RING);
    uint32_t *l_max = reinterpret_cast<uint32_t *>(lds + EX_RING + EX_MT * 4);
    if (tid < EX_MT) {
        const int rc = tid < rows ? tid : rows - 1;
        l_rs[tid] = rs[rowidx ? (size_t)rowidx[m0 + rc] : (size_t)(m0 + rc)];
        l_max[tid] = 0u;
    }

    f32x16 acc[MB][NB];
#pragma unroll
    for (int a = 0; a < MB; ++a)
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.f;

    const ExConst cst = {vgpr_const(0x000F000Fu), vgpr_const(0x00F000F0u), vgpr_const(0x64006400u), vgpr_const(0x54005400u),
                         vgpr_const(0xE400E400u), vgpr_const(0xD400D400u)};  // -1024, -64 as fp16 pairs
    const int nit = (kend - kbeg) >> 6;   // a multiple of 4
    const int it_abs0 = kbeg >> 6, un_abs0 = kbeg >> 8, nun = nit >> 2;

    u32x4 wq[EX_NS][NB];       // weight words of four iterations in flight
    u32x2 sqE[NB], sqO[NB], sqN[NB];  // the lane's scales of the even unit, the odd unit and the next even unit
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) sqN[nb] = u32x2{0u, 0u};
    u32x4 cah[MB], cal[MB];    // correction operands of the current 512 k

    auto issue_a = [&](int itn, int stage) {
        const int k = kbeg + ((itn < nit) ? itn : 0) * 64;  // past the end: repeat the first addresses (never read)
        uint8_t *adst = lds + stage * ASTAGE + wave * 1024;
#pragma unroll
        for (int i = 0; i < MB; ++i)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(arsrc, (__attribute__((address_space(3))) void *)(adst + i * 4096), 16, asrc[i], k * 2, 0, 0);
    };
    auto issue_w = [&](int itn, int set) {
        const size_t off = (size_t)(it_abs0 + ((itn < nit) ? itn : 0)) * 1024;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            if (CHADQ_EXPERT_ABLATE == 2) wq[set][nb] = u32x4{0x12345678u + (uint32_t)lane, 0x9abcdef0u, 0x0fedcba9u, 0x87654321u};
            else wq[set][nb] = load_nt_b128(wband[nb] + off);
        }
    };
    auto load_s = [&](int un, u32x2 (&dst)[NB]) {
        const size_t off = (size_t)(un_abs0 + ((un < nun) ? un : 0)) * 512;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) dst[nb] = *reinterpret_cast<const u32x2 *>(sband[nb] + off);
    };
    auto load_c = [&](int it0) {  // the 512 k that begin at iteration it0
        const int blk = (it_abs0 + it0) >> 3;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
            cah[mb] = *reinterpret_cast<const u32x4 *>(chi[mb] + blk * 16);
            cal[mb] = *reinterpret_cast<const u32x4 *>(clo[mb] + blk * 16);
        }
    };

    // one iteration (64 k): weights of register set `set`, activations of stage `stage`, t = iteration inside its unit
    auto compute = [&](int stage, int set, int t, const u32x2 (&sq)[NB]) {
        const uint8_t *ab = lds + stage * ASTAGE;
        uint32_t s_pk[NB], c_lo[NB], c_hi[NB];
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const uint32_t word = (t < 2) ? sq[nb].x : sq[nb].y;
            s_pk[nb] = __builtin_amdgcn_perm(word, word, (t & 1) ? 0x03020302u : 0x01000100u);
            c_lo[nb] = pk_mul_f16(s_pk[nb], cst.m1024);
            c_hi[nb] = pk_mul_f16(s_pk[nb], cst.m64);
        }
        f16x8 af[2][MB], bf[2][NB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) af[0][mb] = *reinterpret_cast<const f16x8 *>(ab + mb * 4096 + ard[0]);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) bf[0][nb] = dequant8_us(wq[set][nb].x, s_pk[nb], c_lo[nb], c_hi[nb], cst);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (j < 3) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                    af[(j + 1) & 1][mb] = *reinterpret_cast<const f16x8 *>(ab + mb * 4096 + ard[j + 1]);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (CHADQ_EXPERT_ABLATE != 1) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                    for (int nb = 0; nb < NB; ++nb)
                        acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[j & 1][mb], bf[j & 1][nb], acc[mb][nb], 0, 0, 0);
            }
            if (j < 3) {
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) {
                    const uint32_t wsel = j == 0 ? wq[set][nb].y : j == 1 ? wq[set][nb].z : wq[set][nb].w;
                    if (CHADQ_EXPERT_ABLATE != 1) bf[(j + 1) & 1][nb] = dequant8_us(wsel, s_pk[nb], c_lo[nb], c_hi[nb], cst);
                }
            }
            if (CHADQ_EXPERT_ABLATE == 1) {  // keep the loaded words and fragments alive without arithmetic on them
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) asm volatile("" ::"v"(af[j & 1][mb]));
#pragma unroll
                for (int nb = 0; nb < NB; ++nb) asm volatile("" ::"v"(wq[set][nb]));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // four iterations of one unit; `first` = index of the unit's first iteration
    auto unit = [&](int first, const u32x2 (&sq)[NB]) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int it = first + t;
            // the last weight word of iteration `it` was requested after the activations of iteration `it` (same
            // group of requests, memory returns in order): once it is here, so are they
            asm volatile("" : "+v"(wq[t][NB - 1]));
            // the bare barrier instruction: __syncthreads() would add a fence that waits for every outstanding request
            __builtin_amdgcn_s_barrier();  // everybody's part of A(it) has landed; everybody is done reading A(it-1)
            __builtin_amdgcn_sched_barrier(0);
            issue_a(it + EX_D, (t + EX_D) & 3);  // into the stage of A(it-1)
            __builtin_amdgcn_sched_barrier(0);
            issue_w(it + EX_D, (t + EX_D) & 3);  // into the registers of W(it-1)
            __builtin_amdgcn_sched_barrier(0);
            compute(t, t, t, sq);
        }
    };

    // prologue: the first EX_D iterations' requests, the first unit's scales
#pragma unroll
    for (int e = 0; e < EX_D; ++e) {
        issue_a(e, e);
        __builtin_amdgcn_sched_barrier(0);
        issue_w(e, e);
        __builtin_amdgcn_sched_barrier(0);
    }
    load_s(0, sqE);
    // A pass of the loop is 512 k = two units.  A K range of an odd number of units (K % 512 == 256) runs its last
    // pass with the second unit's scales forced to zero: its requests repeat the range's first addresses (finite
    // values), its products are zero, and the group sums past K are stored as zeros.
    for (int it0 = 0; it0 < nit; it0 += 8) {
        const uint32_t oddmask = (it0 + 4 < nit) ? 0xFFFFFFFFu : 0u;
        load_s((it0 >> 2) + 1, sqO);
        load_c(it0);
        __builtin_amdgcn_sched_barrier(0);
        unit(it0, sqE);
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) sqO[nb] = u32x2{sqO[nb].x & oddmask, sqO[nb].y & oddmask};
        load_s((it0 >> 2) + 2, sqN);
        __builtin_amdgcn_sched_barrier(0);
        unit(it0 + 4, sqO);
        if (CHADQ_EXPERT_ABLATE != 1) {
#pragma unroll
            for (int nb = 0; nb < NB; ++nb) {
                const u32x4 bw = {sqE[nb].x, sqE[nb].y, sqO[nb].x, sqO[nb].y};
                f16x8 bs;
                __builtin_memcpy(&bs, &bw, 16);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    f16x8 ah, al;
                    __builtin_memcpy(&ah, &cah[mb], 16);
                    __builtin_memcpy(&al, &cal[mb], 16);
                    acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bs, acc[mb][nb], 0, 0, 0);
                    acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, bs, acc[mb][nb], 0, 0, 0);
                }
            }
        }
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) sqE[nb] = sqN[nb];
    }
    wait_vmcnt<0>();  // the surplus requests of the last iterations must not outlive the workgroup's LDS

    // epilogue: lane (nl, kq) holds column nl of rows 8*(v/4) + 4*kq + v%4 of each 32 x 32 block; the row's power of
    // two comes back in.  MODE 1 also gathers, per row of h, the largest finite magnitude it stores (bf16 bits, which
    // order like the magnitudes): over its feature pairs, then over the 32 lanes that hold the row (DPP inside the
    // 16-lane rows, then lanes 16..31 / 48..63 take their neighbour row's result), then one atomic maximum per row
    // from lane 31 / 63.  expert_prep_h_kernel scales the row by it.
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = mb * 32 + 8 * (v >> 2) + 4 * kq + (v & 3);
            const bool live = row < rows;
            const float r = l_rs[row];
            if (MODE == 1) {
                uint32_t amax = 0;
#pragma unroll
                for (int p = 0; p < NB / 2; ++p) {
                    const float g = acc[mb][2 * p][v] * r, up = acc[mb][2 * p + 1][v] * r;
                    const float h = g / (1.f + __expf(-g)) * up;
                    const uint32_t hb = f32_to_bf16_bits(h), ab = hb & 0x7FFFu;
                    if (live) {
                        reinterpret_cast<uint16_t *>(yv)[(size_t)(m0 + row) * N + n0 + (wave * (NB / 2) + p) * 32 + nl] = (uint16_t)hb;
                        if (ab < 0x7F80u && ab > amax) amax = ab;
                    }
                }
#define CHADQ_MAX_STEP(CTRL, MASK)                                                                         \
    {                                                                                                      \
        const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)amax, CTRL, MASK, 0xF, false);    \
        amax = o > amax ? o : amax;                                                                        \
    }
                CHADQ_MAX_STEP(0xB1, 0xF)   // quad_perm [1,0,3,2]
                CHADQ_MAX_STEP(0x4E, 0xF)   // quad_perm [2,3,0,1]
                CHADQ_MAX_STEP(0x141, 0xF)  // row_half_mirror
                CHADQ_MAX_STEP(0x140, 0xF)  // row_mirror: every lane of a 16-lane row holds the row's maximum
                CHADQ_MAX_STEP(0x142, 0xA)  // row_bcast15 into rows 1 and 3
#undef CHADQ_MAX_STEP
                if (nl == 31 && live && amax) atomicMax(l_max + row, amax);  // LDS: the four waves hold different features of the row
            } else if (live) {
#pragma unroll
                for (int nb = 0; nb < NB; ++nb)
                    reinterpret_cast<float *>(yv)[(size_t)(m0 + row) * N + n0 + (wave * NB + nb) * 32 + nl] = acc[mb][nb][v] * r;
            }
        }
    if (MODE == 1) {
        __syncthreads();
        if (tid < rows && l_max[tid]) atomicMax(rowmax + m0 + tid, l_max[tid]);
    }
}

// The operands of one call, by value in the kernel arguments.
struct ExpertArgs {
    const GemmGroup *groups;  // [E] gate, [E] up, [E] down descriptors as the router writes them (M, w, sc, and y of down)
    const int32_t *tiles;     // token tiles that exist: expert | tile << 16, -1 past the last
    const uint16_t *xa;       // fp16 activations [., K]: MODE 1 one row per token (addressed through tok), MODE 0 in expert order
    const float *rs;          // [.] power of two each row of xa was divided by
    const uint16_t *ghi, *glo;  // [., G16] -8 * group sums of xa, high and low part
    const int32_t *tok;       // MODE 1: token of every row in expert order
    uint32_t *rowmax;         // MODE 1: [P] largest finite bf16 magnitude of every row of h (atomic maxima; zeroed by the router)
    void *y;                  // MODE 1: bf16 h [P, N]; MODE 0: fp32 parts [nz][P, N]
    int E, N, K, G16, kspan, nx, ny, nz;
    size_t ysplit_stride;
};

// grid: one dimension, decoded into n-tile, entry of the tile list and K split as in gemm_skinny_i4g32_kernel.
template <int MODE, int NB>
__global__ __launch_bounds__(256, NB == 2 ? 2 : 1) void gemm_expert_i4g32_kernel(ExpertArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    int bx, by, bz;
    if (MODE == 1) {
        bx = blockIdx.x % a.nx;
        by = blockIdx.x / a.nx;
        bz = 0;
        if (by >= a.ny) return;
    } else {
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
        const int pair = (slot / a.nx) * 8 + xcd;
        bx = slot % a.nx;
        if (pair >= a.ny * a.nz) return;
        by = pair / a.nz;
        bz = pair % a.nz;
    }
    const int tile = a.tiles[by];
    if (tile < 0) return;
    const int g = tile & 0xFFFF, mt = tile >> 16;
    const GemmGroup ga = a.groups[MODE == 1 ? g : 2 * a.E + g];
    const int M = ga.M, m0 = mt * EX_MT;
    if (m0 >= M) return;
    const int rows = (M - m0) < EX_MT ? (M - m0) : EX_MT;
    const int kbeg = bz * a.kspan, kend = (kbeg + a.kspan < a.K) ? kbeg + a.kspan : a.K;
    const uint8_t *w0 = reinterpret_cast<const uint8_t *>(ga.w), *w1 = nullptr;
    const uint8_t *s0 = reinterpret_cast<const uint8_t *>(ga.sc), *s1 = nullptr;
    const int first = a.groups[g].pad;  // the expert's first row in expert order (the router keeps it in the gate descriptor)
    void *y;
    int n0;
    if (MODE == 1) {
        const GemmGroup gu = a.groups[a.E + g];
        w1 = reinterpret_cast<const uint8_t *>(gu.w);
        s1 = reinterpret_cast<const uint8_t *>(gu.sc);
        y = a.y;
        n0 = bx * 64 * NB;
    } else {
        y = reinterpret_cast<float *>(a.y) + (size_t)bz * a.ysplit_stride;
        n0 = bx * 128 * NB;
    }
    const int mrow = first + m0;
    const int32_t *rowidx = (MODE == 1) ? a.tok : nullptr;
    switch ((rows + 31) >> 5) {
        case 1: expert_body<MODE, 1, NB>(a.xa, a.rs, a.ghi, a.glo, a.G16, rowidx, a.rowmax, w0, s0, w1, s1, y, mrow, rows, n0, a.N, a.K, kbeg, kend, lds); break;
        case 2: expert_body<MODE, 2, NB>(a.xa, a.rs, a.ghi, a.glo, a.G16, rowidx, a.rowmax, w0, s0, w1, s1, y, mrow, rows, n0, a.N, a.K, kbeg, kend, lds); break;
        default: expert_body<MODE, 3, NB>(a.xa, a.rs, a.ghi, a.glo, a.G16, rowidx, a.rowmax, w0, s0, w1, s1, y, mrow, rows, n0, a.N, a.K, kbeg, kend, lds); break;
    }
}

// h bf16 [P, K] -> its fp16 form, one thread per run of 8 (grid-stride): the scale of a row comes from rowmax[p], the
// bits of the row's largest finite bf16 magnitude, which the gate/up kernel's epilogue gathered with atomic maxima.
//   dst[p]  fp16, the row times 2^-e (prep_scale), every aligned run of 8 in the order 0,4,1,5,2,6,3,7;
//   rs[p]   2^e;
//   ghi/glo [p][G16]: -8 * (sum of the 32 fp16 values of each scale group), high part and remainder (prep_store_group).
__global__ __launch_bounds__(256) void expert_prep_h_kernel(const uint16_t *__restrict__ src, const uint32_t *__restrict__ rowmax,
                                                            int P, int K, uint16_t *__restrict__ dst, float *__restrict__ rs,
                                                            uint16_t *__restrict__ ghi, uint16_t *__restrict__ glo, int G16) {
    const int nblk = K >> 3;  // a multiple of 32: the four threads of a quad always work on one group of one row
    const int64_t total = (int64_t)P * nblk, stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i0 = (int64_t)blockIdx.x * blockDim.x; i0 < total; i0 += stride) {
        const int64_t i = i0 + threadIdx.x;
        float sum = 0.f;
        int p = 0, b = 0;
        if (i < total) {
            p = (int)(i / nblk);
            b = (int)(i % nblk);
            float mult, back;
            prep_scale(rowmax[p], mult, back);
            u32x4 o;
            sum = prep_run8(*reinterpret_cast<const u32x4 *>(src + (size_t)p * K + b * 8), mult, o);
            *reinterpret_cast<u32x4 *>(dst + (size_t)p * K + b * 8) = o;
            if (b == 0) rs[p] = back;
            if (b < 8) prep_clear_tail(K >> 5, b, ghi + (size_t)p * G16, glo + (size_t)p * G16);
        }
        sum += dpp_f32<0xB1, 0xF>(sum);
        sum += dpp_f32<0x4E, 0xF>(sum);
        if (i < total && (threadIdx.x & 3) == 0) prep_store_group(sum, b >> 2, ghi + (size_t)p * G16, glo + (size_t)p * G16);
    }
}

int expert_prep_h_launch(const uint16_t *h, const uint32_t *rowmax, int P, int K, uint16_t *dst, float *rs, uint16_t *ghi, uint16_t *glo,
                         hipStream_t st) {
    const int64_t total = (int64_t)P * (K >> 3);
    const int blocks = (int)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
    hipLaunchKernelGGL(expert_prep_h_kernel, dim3(blocks), dim3(256), 0, st, h, rowmax, P, K, dst, rs, ghi, glo, ((K >> 5) + 15) & ~15);
    return hip_check(hipGetLastError(), "expert_prep_h launch");
}

bool gemm_expert_ok(int H, int F) { return H % 256 == 0 && F % 256 == 0; }
int gemm_expert_tile_rows() { return EX_MT; }
// K splits of the down projection: four when every part is a multiple of 512 k, else one
int gemm_expert_down_splits(int F) { return (F % (512 * 4) == 0) ? 4 : 1; }

template <int MODE, int NB>
static int expert_launch(const ExpertArgs &a, hipStream_t st) {
    static std::atomic<bool> attr_set{false};  // setting it twice from two threads is harmless
    if (!attr_set.load(std::memory_order_acquire)) {
        CHADQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_expert_i4g32_kernel<MODE, NB>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, EX_LDS));
        attr_set.store(true, std::memory_order_release);
    }
    const int pairs8 = (a.ny * a.nz + 7) / 8 * 8;  // (list entry, split) pairs, dealt to the 8 XCDs
    hipLaunchKernelGGL((gemm_expert_i4g32_kernel<MODE, NB>), dim3(pairs8 * a.nx), dim3(256), EX_LDS, st, a);
    return hip_check(hipGetLastError(), "gemm_expert launch");
}

// gate/up with the SiLU epilogue: h[P,F] bf16 and the rows' maxima.  Activations: xa fp16 [T,H], one row per token, with rs,
// ghi, glo as prep_row_block writes them; tok = token of every row in expert order.  Two workgroups per compute unit
// (64 weight rows per wave) measured faster here, one (128 rows per wave) on the down projection.
int gemm_expert_gateup(const GemmGroup *groups, const int32_t *tiles, const int32_t *tok, int ntiles, int E, int F, int H,
                       const uint16_t *xa, const float *rs, const uint16_t *ghi, const uint16_t *glo, uint16_t *h, uint32_t *rowmax,
                       hipStream_t st) {
    ExpertArgs a = {groups, tiles, xa, rs, ghi, glo, tok, rowmax, h, E, F, H, ((H >> 5) + 15) & ~15, H, F / 128, ntiles, 1, 0};
    return expert_launch<1, 2>(a, st);
}

// down: fp32 parts [ksplit][P,H]; ha fp16 [P,F] in expert order with rs, ghi, glo from expert_prep_h_launch
int gemm_expert_down(const GemmGroup *groups, const int32_t *tiles, int ntiles, int E, int H, int F, const uint16_t *ha,
                     const float *rs, const uint16_t *ghi, const uint16_t *glo, float *yp, int ksplit, size_t ysplit_stride,
                     hipStream_t st) {
    ExpertArgs a = {groups, tiles, ha, rs, ghi, glo, nullptr, nullptr, yp, E, H, F, ((F >> 5) + 15) & ~15, F / ksplit, 0, ntiles, ksplit,
                    ysplit_stride};
    if (H % 512 == 0) {
        a.nx = H / 512;
        return expert_launch<0, 4>(a, st);
    }
    a.nx = H / 256;
    return expert_launch<0, 2>(a, st);
}

}  // namespace chadq
