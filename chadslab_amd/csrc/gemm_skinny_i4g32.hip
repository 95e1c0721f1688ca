// Grouped "skinny" dequant-GEMM for the mixture-of-experts FFN: few activation rows (the tokens routed to one
// expert, tens to a hundred or so) against many int4 group-32 weight rows.  The prefill tile (128 x 64) is the
// wrong shape here: half of its rows are padding and every 64 weight rows re-read the whole activation panel.
// This kernel turns the tile around: one workgroup takes up to 96 tokens of one expert and 256 weight rows,
//   - the activation tile (32*MB rows x 64 k per iteration, MB = 1..3 from the expert's actual row count) goes
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

constexpr int SK_MT = 96;   // tokens per workgroup tile
constexpr int SK_KI = 64;   // k per iteration

// Operand supply: everything comes global -> LDS by DMA, ahead of its use, so that memory latency is covered by
// bytes in flight rather than by registers or occupancy:
//   activation ring (shared by the workgroup): 3 stages of 32*SK_MB rows x 64 k, each wave fetches a quarter,
//     two iterations ahead;
//   weight ring (private to a wave): 2 slots of 128 k: 64 rows x 64 B of packed weights fetched as 4 DMA
//     instructions of 16 rows x 64 contiguous bytes (whole 64-byte sectors: fetching 32 B per row per iteration
//     made HBM traffic 2.5 x the weight bytes), plus 64 rows x 16 B of group scales; a slot serves two
//     iterations and is refilled right after its last use, one slot (two iterations) ahead.
// Every wave issues MB DMA instructions per iteration plus 5 on even ones; memory returns in order, so the waits
// below count how many younger requests may still be outstanding.  Past the end of K the requests repeat the
// first addresses so the counts stay uniform (their slots are never read).
constexpr int SK_MB = SK_MT / 32;
// Depth 2 keeps the rings at 76 KiB, two workgroups per CU.  Depth 4 (120 KiB, one workgroup per CU, twice the
// bytes in flight per workgroup) measured 3 % slower on the benchmark's expert shapes: with one wave per SIMD the
// LDS and barrier latencies of an iteration are no longer covered by a second workgroup.
constexpr int SK_DA = 2;                // activation stages requested ahead (even)
constexpr int SK_DB = SK_DA / 2;        // weight slots (two iterations each) requested ahead
constexpr int SK_NSA = SK_DA + 1, SK_NSB = SK_DB + 1;
constexpr int SK_ASTAGE = SK_MB * 32 * 128;
constexpr int SK_A_BYTES = SK_NSA * SK_ASTAGE;
constexpr int SK_BSLOT = 64 * 64 + 64 * 16;
constexpr int SK_B_WAVE = SK_NSB * SK_BSLOT;
constexpr int SK_LDS = SK_A_BYTES + 4 * SK_B_WAVE;
constexpr int SK_WGS_PER_CU = (2 * SK_LDS <= 160 * 1024) ? 2 : 1;

template <int MODE, int MB>
__device__ __forceinline__ void skinny_body(const uint16_t *__restrict__ x, const uint8_t *__restrict__ w0,
                                            const uint16_t *__restrict__ s0, const uint8_t *__restrict__ w1,
                                            const uint16_t *__restrict__ s1, void *__restrict__ yv,
                                            const int32_t *__restrict__ rowidx, int m0, int rows, int n0, int N, int K,
                                            int kbeg, int kend, uint8_t *lds) {
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nl = lane & 31, kq = lane >> 5;

    // wave-local weight row rho (0..63) -> matrix row: MODE 0: n0 + 64*wave + rho; MODE 1: rows 0..31 are gate
    // features n0 + 32*wave + rho, rows 32..63 the same features of the up matrix
    auto wptr = [&](int rho) -> const uint8_t * {
        if (MODE == 1) return (rho < 32 ? w0 : w1) + (size_t)(n0 + wave * 32 + (rho & 31)) * (K >> 1);
        return w0 + (size_t)(n0 + wave * 64 + rho) * (K >> 1);
    };
    auto sptr = [&](int rho) -> const uint16_t * {
        if (MODE == 1) return (rho < 32 ? s0 : s1) + (size_t)(n0 + wave * 32 + (rho & 31)) * (K >> 5);
        return s0 + (size_t)(n0 + wave * 64 + rho) * (K >> 5);
    };
    // weight fetch: DMA instruction i, lane l -> row 16i + l/4, LDS position l%4, which holds 16-byte piece
    // (l%4) ^ ((row >> 1) & 3) of the row's 64 bytes (bank-conflict-free read-back)
    const uint8_t *wsrc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int rho = 16 * i + (lane >> 2);
        wsrc[i] = wptr(rho) + (((lane & 3) ^ ((rho >> 1) & 3)) << 4);
    }
    // scale fetch: lane l -> row l, 8 groups (256 k)
    const uint16_t *ssrc = sptr(lane);
    // read-back: lane (nl, kq), block nb -> row nb*32 + nl; half h of the slot -> piece 2h + kq
    uint32_t brd[2][2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int rho = nb * 32 + nl;
            brd[nb][h] = (uint32_t)(rho * 64 + (((2 * h + kq) ^ ((rho >> 1) & 3)) << 4));
        }
    // activation pieces this lane requests: DMA instruction i of wave w fills LDS bytes (4i + w) * 1024 + 16 * lane
    // of a stage, i.e. row rr = (4i + w) * 8 + lane / 8, slot lane % 8, which holds piece slot ^ (rr & 7).  Rows
    // past the tile repeat its last row (their results are never stored).  With a row index (gate/up: the tokens
    // routed to the expert, in the expert's row order) row m of the tile is row rowidx[m] of x: the activations are
    // read where they lie, no gathered copy exists.
    const uint16_t *asrc[MB];
#pragma unroll
    for (int i = 0; i < MB; ++i) {
        const int rr = (4 * i + wave) * 8 + (lane >> 3), rc = rr < rows ? rr : rows - 1;
        const size_t srow = rowidx ? (size_t)rowidx[m0 + rc] : (size_t)(m0 + rc);
        asrc[i] = x + srow * K + (((lane & 7) ^ (rr & 7)) << 3);
    }
    // fragment read offsets: row mb*32 + nl, piece kq*4 + j lives in slot (kq*4 + j) ^ (nl & 7)
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
    uint8_t *bring = lds + SK_A_BYTES + wave * SK_B_WAVE;
    const int nit = (kend - kbeg) / SK_KI;  // even

    auto issue_a = [&](int itn, int stage) {
        const int k = (itn < nit) ? kbeg + itn * SK_KI : kbeg;
        uint8_t *adst = lds + stage * SK_ASTAGE + wave * 1024;
#pragma unroll
        for (int i = 0; i < MB; ++i) dma16_to_lds(asrc[i] + k, adst + i * 4096);
    };
    auto issue_b = [&](int m, int slot) {  // weights and scales of iterations 2m, 2m+1
        const int k = (2 * m < nit) ? kbeg + m * 2 * SK_KI : kbeg;
        uint8_t *bdst = bring + slot * SK_BSLOT;
#pragma unroll
        for (int i = 0; i < 4; ++i) dma16_to_lds(wsrc[i] + (size_t)(k >> 1), bdst + i * 1024);
        dma16_to_lds(ssrc + (size_t)((k & ~255) >> 5), bdst + 4096);
    };

    // one iteration (64 k): weights of half `h` of weight slot `bslot`, activations of stage `stage`
    auto compute = [&](int stage, int bslot, int h, int k) {
        const uint8_t *bs = bring + bslot * SK_BSLOT;
        const uint8_t *ab = lds + stage * SK_ASTAGE;
        const int gi = ((k & 255) >> 5) + kq;  // the lane's group among the 8 whose scales the slot holds
        u32x4 q[2];
        uint32_t sbits[2];
        bf16x8 af[2][MB];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            q[nb] = *reinterpret_cast<const u32x4 *>(bs + brd[nb][h]);
            sbits[nb] = *reinterpret_cast<const uint16_t *>(bs + 4096 + (nb * 32 + nl) * 16 + gi * 2);
        }
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) af[0][mb] = *reinterpret_cast<const bf16x8 *>(ab + mb * 4096 + ard[0]);
        __builtin_amdgcn_sched_barrier(0);
        float cs[2][4];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            const float sc = f16_bits_to_f32(sbits[nb]);
            cs[nb][0] = sc;
            cs[nb][1] = sc * 0.0625f;
            cs[nb][2] = -1032.f * sc;
            cs[nb][3] = -72.f * sc;
        }
        // LDS reads of a step are issued one step ahead of their use, and the dequantisation of step j+1 follows
        // the MFMAs of step j in program order, so that it runs on the VALU while the matrix core works.
        bf16x8 bf[2][2];
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
            bf[0][nb] = dequant8_i4(q[nb].x, cs[nb][0], cs[nb][1], cs[nb][2], cs[nb][3], c_mlo, c_mhi, c_magic);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (j < 3) {
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                    af[(j + 1) & 1][mb] = *reinterpret_cast<const bf16x8 *>(ab + mb * 4096 + ard[j + 1]);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                for (int nb = 0; nb < 2; ++nb)
                    acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[j & 1][mb], bf[j & 1][nb], acc[mb][nb], 0, 0, 0);
            if (j < 3) {
#pragma unroll
                for (int nb = 0; nb < 2; ++nb) {
                    const uint32_t wsel = j == 0 ? q[nb].y : j == 1 ? q[nb].z : q[nb].w;
                    bf[(j + 1) & 1][nb] = dequant8_i4(wsel, cs[nb][0], cs[nb][1], cs[nb][2], cs[nb][3], c_mlo, c_mhi, c_magic);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // Request groups: iteration e issues A(e + DA) and, when e is even, B(e/2 + DB) after it.  The prologue plays
    // e = -DA .. -1.  Waiting for the group of iteration it - DA leaves the DA - 1 younger groups outstanding:
    // they alternate odd (MB requests) and even (MB + 5), starting with the parity opposite to `it`.
    constexpr int W_EVEN = (SK_DA / 2) * MB + (SK_DA / 2 - 1) * (MB + 5);  // younger: odd, even, ..., odd
    constexpr int W_ODD = (SK_DA / 2) * (MB + 5) + (SK_DA / 2 - 1) * MB;   // younger: even, odd, ..., even
    int sa_fill = 0, sb_fill = 0;  // next stage / slot to fill
#pragma unroll
    for (int e = -SK_DA; e < 0; ++e) {
        issue_a(e + SK_DA, sa_fill);
        sa_fill = sa_fill + 1 == SK_NSA ? 0 : sa_fill + 1;
        if ((e & 1) == 0) {
            issue_b(e / 2 + SK_DB, sb_fill);
            sb_fill = sb_fill + 1 == SK_NSB ? 0 : sb_fill + 1;
        }
    }
    int sa = 0, sb = 0;  // stage of iteration it, slot of iterations it, it+1
    for (int it = 0; it < nit; it += 2) {
        const int m = it >> 1;
        wait_vmcnt<W_EVEN>();  // A(it) and B(m) have landed
        // the bare barrier instruction: __syncthreads() would add a fence that waits for every outstanding
        // request (vmcnt 0) and with it the whole prefetch
        __builtin_amdgcn_s_barrier();  // everybody's part of A(it) has landed; everybody is done reading A(it-1)
        __builtin_amdgcn_sched_barrier(0);
        issue_a(it + SK_DA, sa_fill);  // into the stage of A(it-1)
        sa_fill = sa_fill + 1 == SK_NSA ? 0 : sa_fill + 1;
        issue_b(m + SK_DB, sb_fill);   // into the slot of B(m-1), which this wave finished in iteration it-1
        sb_fill = sb_fill + 1 == SK_NSB ? 0 : sb_fill + 1;
        compute(sa, sb, 0, kbeg + it * SK_KI);
        sa = sa + 1 == SK_NSA ? 0 : sa + 1;
        wait_vmcnt<W_ODD>();   // A(it+1) has landed
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        issue_a(it + 1 + SK_DA, sa_fill);  // into the stage of A(it)
        sa_fill = sa_fill + 1 == SK_NSA ? 0 : sa_fill + 1;
        compute(sa, sb, 1, kbeg + (it + 1) * SK_KI);
        sa = sa + 1 == SK_NSA ? 0 : sa + 1;
        sb = sb + 1 == SK_NSB ? 0 : sb + 1;
    }
    wait_vmcnt<0>();  // the surplus requests of the last iterations must not outlive the workgroup's LDS

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

// groups: [E] gate, [E] up, [E] down descriptors as the router writes them; tiles: the token tiles that exist
// (expert | tile << 16, -1 past the last), also from the router, fullest first.  MODE 1 with tok != nullptr: the
// gate/up descriptors' x is the ungathered activation matrix and `pad` the expert's first row in tok, the token of
// every expert-sorted row.
// grid: one dimension, decoded in the kernel into n-tile, entry of the tile list and K split (MODE 0 only).
template <int MODE>
__global__ __launch_bounds__(256, SK_WGS_PER_CU) void gemm_skinny_i4g32_kernel(const GemmGroup *__restrict__ groups,
                                                                  const int32_t *__restrict__ tiles,
                                                                  const int32_t *__restrict__ tok, int E, int N, int K,
                                                                  int kspan, size_t ysplit_stride, int nx, int ny, int nz) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    // Workgroup -> (n-tile bx, list entry by, K split bz).  Workgroup i runs on XCD i % 8, each with its own L2.
    // Down projection: the nx n-tiles of one (entry, split) read the same activation rows, so they are dealt to ONE XCD
    // (spread over all of them, every XCD fetched the routed activations once: a quarter of the kernel's memory
    // traffic); pairs count splits fastest, so the entries that exist (the first of the list) come out evenly.
    // Gate/up: n-tiles fastest, which spreads every expert over all XCDs whatever the experts' sizes (its activation
    // tiles fit the L2s anyway).
    int bx, by, bz;
    if (MODE == 1) {
        bx = blockIdx.x % nx;
        by = blockIdx.x / nx;
        bz = 0;
        if (by >= ny) return;
    } else {
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
        const int pair = (slot / nx) * 8 + xcd;
        bx = slot % nx;
        if (pair >= ny * nz) return;
        by = pair / nz;
        bz = pair % nz;
    }
    const int tile = tiles[by];
    if (tile < 0) return;
    const int g = tile & 0xFFFF, mt = tile >> 16;
    const GemmGroup ga = groups[MODE == 1 ? g : 2 * E + g];
    const int M = ga.M, m0 = mt * SK_MT;
    if (m0 >= M) return;
    const int rows = (M - m0) < SK_MT ? (M - m0) : SK_MT;
    const int kbeg = bz * kspan, kend = (kbeg + kspan < K) ? kbeg + kspan : K;
    const uint8_t *w0 = reinterpret_cast<const uint8_t *>(ga.w), *w1 = nullptr;
    const uint16_t *s0 = reinterpret_cast<const uint16_t *>(ga.sc), *s1 = nullptr;
    void *y;
    int n0;
    if (MODE == 1) {
        const GemmGroup gu = groups[E + g], gd = groups[2 * E + g];
        w1 = reinterpret_cast<const uint8_t *>(gu.w);
        s1 = reinterpret_cast<const uint16_t *>(gu.sc);
        y = const_cast<uint16_t *>(gd.x);  // the down projection's input rows of this expert
        n0 = bx * 128;
    } else {
        y = reinterpret_cast<float *>(ga.y) + (size_t)bz * ysplit_stride;
        n0 = bx * 256;
    }
    const int32_t *rowidx = (MODE == 1 && tok) ? tok + ga.pad : nullptr;
    switch ((rows + 31) >> 5) {
        case 1: skinny_body<MODE, 1>(ga.x, w0, s0, w1, s1, y, rowidx, m0, rows, n0, N, K, kbeg, kend, lds); break;
        case 2: skinny_body<MODE, 2>(ga.x, w0, s0, w1, s1, y, rowidx, m0, rows, n0, N, K, kbeg, kend, lds); break;
        default: skinny_body<MODE, 3>(ga.x, w0, s0, w1, s1, y, rowidx, m0, rows, n0, N, K, kbeg, kend, lds); break;
    }
}

bool gemm_skinny_ok(int H, int F) { return H % 256 == 0 && F % 256 == 0; }

template <int MODE>
static int skinny_launch(const GemmGroup *groups, const int32_t *tiles, const int32_t *tok, int mtiles, int E, int ntiles, int N,
                         int K, int ksplit, size_t ystride, hipStream_t st) {
    static std::atomic<bool> attr_set{false};  // setting it twice from two threads is harmless
    if (!attr_set.load(std::memory_order_acquire)) {
        CHADQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemm_skinny_i4g32_kernel<MODE>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, SK_LDS));
        attr_set.store(true, std::memory_order_release);
    }
    const int pairs8 = (mtiles * ksplit + 7) / 8 * 8;  // (list entry, split) pairs, dealt to the 8 XCDs
    hipLaunchKernelGGL((gemm_skinny_i4g32_kernel<MODE>), dim3(pairs8 * ntiles), dim3(256), SK_LDS, st, groups, tiles, tok, E, N, K,
                       K / ksplit, ystride, ntiles, mtiles, ksplit);
    return hip_check(hipGetLastError(), "gemm_skinny launch");
}

int gemm_skinny_tile_rows() { return SK_MT; }

// gate/up with the SiLU epilogue: h[P,F] bf16 (through the down descriptors' x pointers).  tok != nullptr: the
// descriptors address the activations through the token of each row instead of a gathered copy.
int gemm_skinny_gateup(const GemmGroup *groups, const int32_t *tiles, const int32_t *tok, int ntiles, int E, int F, int H,
                       hipStream_t st) {
    return skinny_launch<1>(groups, tiles, tok, ntiles, E, F / 128, F, H, 1, 0, st);
}

// down: fp32 parts [ksplit][P,H]
int gemm_skinny_down(const GemmGroup *groups, const int32_t *tiles, int ntiles, int E, int H, int F, int ksplit, size_t ysplit_stride,
                     hipStream_t st) {
    return skinny_launch<0>(groups, tiles, nullptr, ntiles, E, H / 256, H, F, ksplit, ysplit_stride, st);
}

}  // namespace chadq
