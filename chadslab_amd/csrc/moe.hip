// Mixture-of-experts FFN on int4 group-32 expert weights (benchmark config 3):
//   p = softmax(logits[t,:]);  the top_k experts of token t by logit (lowest index wins ties), weights p
//   renormalised to sum 1 if asked;  y[t] = bf16( sum_j w[t,j] * down_e( bf16( silu(gate_e x_t) * (up_e x_t) ) ) ).
//
// Everything runs on the caller's stream without a host round trip: the router kernel also sorts the
// (token, slot) pairs by expert (stable: by pair index inside an expert) and writes the per-expert descriptors
// of the grouped GEMM launches and the list of token tiles that exist, so row counts never leave the GPU.
// Gate/up/down run on the skinny grouped kernel (gate and up fused with the SiLU gate and reading the activations
// through the sorted token list, down split over K) when H and F are multiples of 256, else on the prefill
// dequant-GEMM kernel in grouped mode on a gathered copy of the activations with a separate SiLU kernel; the small
// kernels here are the router, the gather, the SiLU gate and the weighted combine.
#include "chadq_common.h"
#include "expert_prep.h"

namespace chadq {

constexpr int MOE_MAX_E = 16;
constexpr int MOE_MAX_K = 8;

struct MoeExperts {  // by value in the kernel arguments
    const void *wg[MOE_MAX_E], *sg[MOE_MAX_E], *wu[MOE_MAX_E], *su[MOE_MAX_E], *wd[MOE_MAX_E], *sd[MOE_MAX_E];
};

struct MoeWs {  // workspace carved up on the host
    int32_t *idx;        // [T,top_k] expert of each pair
    float *w;            // [T,top_k] routing weight of each pair
    int32_t *pos;        // [P] row of the pair in expert-sorted order
    int32_t *tok;        // [P] token of the sorted row
    int32_t *cnt;        // [E] rows per expert, then [E] offsets
    GemmGroup *groups;   // [3*E] gate, up, down
    int32_t *tiles;      // token tiles of the expert GEMMs: expert | tile << 16, -1 past the last one
    uint16_t *xs;        // [P,H] gathered activations (bf16)
    float *g, *u;        // [P,F]
    uint16_t *h;         // [P,F] bf16
    float *yp;           // [MOE_KSPLIT][P,H] partial down projections
    // tile-order path: fp16 forms of the two activation matrices (expert_prep.h); xs doubles as the first, one row per token
    uint16_t *ha;        // [P,F] fp16 form of h
    float *rsx, *rsh;    // [T] / [P] power of two of each row of xs / ha
    uint16_t *gxh, *gxl; // [T, H/32 rounded up to 16] group sums of xs, high and low part
    uint16_t *ghh, *ghl; // [P, F/32 rounded up to 16] group sums of ha
    uint32_t *rowmax;    // [P] largest finite bf16 magnitude of each row of h
};

constexpr int MOE_KSPLIT = 4;

int gemm_i4g32_grouped(const GemmGroup *groups, int ngroups, int m_max, int N, int K, bool out_f32, hipStream_t st);
bool gemm_skinny_ok(int H, int F);
int gemm_skinny_tile_rows();
int gemm_skinny_gateup(const GemmGroup *groups, const int32_t *tiles, const int32_t *tok, int ntiles, int E, int F, int H,
                       hipStream_t st);
int gemm_skinny_down(const GemmGroup *groups, const int32_t *tiles, int ntiles, int E, int H, int F, int ksplit, size_t ysplit_stride,
                     hipStream_t st);
// weights in tile order (gemm_expert_i4g32.hip)
bool gemm_expert_ok(int H, int F);
int gemm_expert_tile_rows();
int gemm_expert_down_splits(int F);
int expert_prep_h_launch(const uint16_t *h, const uint32_t *rowmax, int P, int K, uint16_t *dst, float *rs, uint16_t *ghi, uint16_t *glo,
                         hipStream_t st);
int gemm_expert_gateup(const GemmGroup *groups, const int32_t *tiles, const int32_t *tok, int ntiles, int E, int F, int H,
                       const uint16_t *xa, const float *rs, const uint16_t *ghi, const uint16_t *glo, uint16_t *h, uint32_t *rowmax,
                       hipStream_t st);
int gemm_expert_down(const GemmGroup *groups, const int32_t *tiles, int ntiles, int E, int H, int F, const uint16_t *ha,
                     const float *rs, const uint16_t *ghi, const uint16_t *glo, float *yp, int ksplit, size_t ysplit_stride,
                     hipStream_t st);

// Workgroup 0.  Phase 1: softmax + top-k per token.  Phase 2: stable counting sort of the pairs by expert.
// Phase 3: descriptors.  idx/w may be the caller's arrays (chadq_moe_route) with everything else null.
// Workgroups 1..T (launched for the tile-order path only, prep_x != nullptr): workgroup t+1 turns row t of the
// activations into the fp16 operands of the tile-order expert GEMM (expert_prep.h) - work that does not depend on the
// routing and so shares its launch.
__global__ __launch_bounds__(1024) void moe_route_kernel(const float *__restrict__ logits, int32_t *__restrict__ idx,
                                                         float *__restrict__ w, int T, int E, int top_k, int renorm,
                                                         MoeWs ws, MoeExperts ex, int H, int F,
                                                         const uint16_t *__restrict__ x_src, int tile_rows, int ntiles_max,
                                                         const uint16_t *__restrict__ prep_x) {
    if (blockIdx.x > 0) {
        __shared__ uint32_t s_pmax[16];
        const int t = blockIdx.x - 1, g16 = ((H >> 5) + 15) & ~15;
        prep_row_block(prep_x + (size_t)t * H, H, ws.xs + (size_t)t * H, ws.rsx + t, ws.gxh + (size_t)t * g16, ws.gxl + (size_t)t * g16, s_pmax);
        return;
    }
    __shared__ int s_base[MOE_MAX_E];   // rows of expert e seen so far
    __shared__ int s_cnt[16][MOE_MAX_E];  // per-wave counts of every expert in the current chunk
    __shared__ int s_off[MOE_MAX_E + 1];
    __shared__ int s_tn[4 * MOE_MAX_E];  // token tiles per (fullness class, expert)
    // expert and rank of every pair stay in LDS between the phases when they fit (a global write followed by a read
    // from other threads costs a memory round trip per phase)
    constexpr int LP = 4096;
    __shared__ uint8_t s_e[LP];
    __shared__ uint16_t s_r[LP];
    const int tid = threadIdx.x, B = blockDim.x, lane = tid & 63, wave = tid >> 6, nw = B >> 6;
    const bool in_lds = (T * top_k <= LP) && ws.pos;
    if (tid < MOE_MAX_E) s_base[tid] = 0;
    // the expert's six pointers are asked for now (they sit in the kernel-argument buffer, indexed per lane) and used at
    // the very end
    const void *e_wg = nullptr, *e_sg = nullptr, *e_wu = nullptr, *e_su = nullptr, *e_wd = nullptr, *e_sd = nullptr;
    if (ws.pos && tid < E) {
        e_wg = ex.wg[tid];
        e_sg = ex.sg[tid];
        e_wu = ex.wu[tid];
        e_su = ex.su[tid];
        e_wd = ex.wd[tid];
        e_sd = ex.sd[tid];
    }

    for (int t = tid; t < T; t += B) {
        // the token's logits go to registers once (every load in flight together); places past E hold -inf and are
        // never candidates
        const float *z = logits + (size_t)t * E;
        float zr[MOE_MAX_E];
#pragma unroll
        for (int e = 0; e < MOE_MAX_E; ++e) zr[e] = (e < E) ? z[e] : -INFINITY;
        float mx = zr[0];
#pragma unroll
        for (int e = 1; e < MOE_MAX_E; ++e)
            if (e < E) mx = fmaxf(mx, zr[e]);
        float sum = 0.f;
#pragma unroll
        for (int e = 0; e < MOE_MAX_E; ++e)
            if (e < E) sum += __expf(zr[e] - mx);
        uint32_t taken = 0;
        int chosen[MOE_MAX_K];
        float pw[MOE_MAX_K], wsum = 0.f;
#pragma unroll
        for (int j = 0; j < MOE_MAX_K; ++j) {
            if (j < top_k) {
                int best = -1;
                float bv = 0.f;
#pragma unroll
                for (int e = 0; e < MOE_MAX_E; ++e)
                    if (e < E && !((taken >> e) & 1u) && (best < 0 || zr[e] > bv)) {  // strict >: the lowest index wins ties
                        best = e;
                        bv = zr[e];
                    }
                taken |= 1u << best;
                chosen[j] = best;
                pw[j] = __expf(bv - mx) / sum;
                wsum += pw[j];
            }
        }
#pragma unroll
        for (int j = 0; j < MOE_MAX_K; ++j)
            if (j < top_k) {
                idx[(size_t)t * top_k + j] = chosen[j];
                w[(size_t)t * top_k + j] = renorm ? pw[j] / wsum : pw[j];
                if (in_lds) s_e[t * top_k + j] = (uint8_t)chosen[j];
            }
    }
    if (!ws.pos) return;  // routing only
    if (prep_x)
        for (int p = tid; p < T * top_k; p += B) ws.rowmax[p] = 0u;  // the gate/up kernel takes atomic maxima on these
    __syncthreads();      // idx (global) written by this workgroup is visible to it after the barrier

    const int P = T * top_k;
    for (int c0 = 0; c0 < P; c0 += B) {
        const int p = c0 + tid;
        const int e_mine = p < P ? (in_lds ? (int)s_e[p] : idx[p]) : -1;
        // every wave counts all experts by itself (one ballot each, no barrier), the counts meet in LDS once per chunk
        int below = 0;
        for (int e = 0; e < E; ++e) {
            const unsigned long long m = __ballot(e_mine == e);
            if (e_mine == e) below = __popcll(m & ((1ull << lane) - 1ull));
            if (lane == 0) s_cnt[wave][e] = __popcll(m);
        }
        __syncthreads();
        int rank = 0;
        if (e_mine >= 0) {
            rank = s_base[e_mine] + below;
            for (int i = 0; i < wave; ++i) rank += s_cnt[i][e_mine];
        }
        __syncthreads();
        if (tid < E) {
            int total = 0;
            for (int i = 0; i < nw; ++i) total += s_cnt[i][tid];
            s_base[tid] += total;
        }
        __syncthreads();
        if (p < P) {  // rank inside its expert for now
            if (in_lds) s_r[p] = (uint16_t)rank;
            else ws.pos[p] = rank;
        }
    }
    if (tid < E) {  // first row of every expert: each of the E threads adds the counts before its own
        int o = 0;
#pragma unroll
        for (int e = 0; e < MOE_MAX_E; ++e)
            if (e < tid) o += s_base[e];
        s_off[tid] = o;
        ws.cnt[tid] = s_base[tid];
        ws.cnt[E + tid] = o;
        if (tid == E - 1) s_off[E] = o + s_base[tid];
    }
    __syncthreads();
    for (int p = tid; p < P; p += B) {
        const int row = in_lds ? s_off[s_e[p]] + (int)s_r[p] : s_off[idx[p]] + ws.pos[p];
        ws.pos[p] = row;
        ws.tok[row] = p / top_k;
    }
    if (tid < E) {
        const int e = tid, o = s_off[e], m = s_base[e];
        // x_src: the gate/up GEMM reads row tok[o + m] of the caller's activations; else rows o.. of the gathered copy
        const uint16_t *xe = x_src ? x_src : ws.xs + (size_t)o * H;
        ws.groups[e] = GemmGroup{xe, e_wg, e_sg, ws.g + (size_t)o * F, m, x_src ? o : 0};
        ws.groups[E + e] = GemmGroup{xe, e_wu, e_su, ws.u + (size_t)o * F, m, x_src ? o : 0};
        ws.groups[2 * E + e] = GemmGroup{ws.h + (size_t)o * F, e_wd, e_sd, ws.yp + (size_t)o * H, m, 0};
    }
    // The token tiles of the expert GEMMs (expert | tile << 16, then -1), the fullest first: they take longest, and no
    // workgroup is launched for a tile that does not exist except at the end of the grid.  Class c holds the tiles
    // with tile_rows - 32c - 31 .. tile_rows - 32c rows; thread (c, e) counts expert e's tiles of class c, finds its
    // place behind the classes and experts before it, and writes them.  Needs tile_rows <= 128.
    if (ws.tiles && tile_rows > 0) {
        const int ncls = (tile_rows + 31) >> 5;
        int mine = 0, nfull = 0, cls_rem = -1;
        if (tid < ncls * E) {
            const int c = tid / E, m = s_base[tid % E];
            nfull = m / tile_rows;
            const int rem = m % tile_rows;
            cls_rem = rem > 0 ? (tile_rows - rem) >> 5 : -1;
            mine = (c == 0 ? nfull : 0) + (cls_rem == c ? 1 : 0);
            s_tn[tid] = mine;
        }
        __syncthreads();
        int total = 0;
        for (int i = 0; i < ncls * E; ++i) total += s_tn[i];
        if (tid < ncls * E) {
            const int c = tid / E, e = tid % E;
            int at = 0;
            for (int i = 0; i < tid; ++i) at += s_tn[i];
            if (c == 0)
                for (int mt = 0; mt < nfull && at < ntiles_max; ++mt) ws.tiles[at++] = e | (mt << 16);
            if (cls_rem == c && at < ntiles_max) ws.tiles[at] = e | (nfull << 16);
        }
        for (int n = total + tid; n < ntiles_max; n += B) ws.tiles[n] = -1;
    }
}

// xs[row] = x[tok[row]]; one 16-byte piece per thread.  Only the path through the prefill kernel needs the copy: the
// skinny kernel reads the activations through tok.
__global__ __launch_bounds__(256) void moe_gather_kernel(const uint16_t *__restrict__ x, const int32_t *__restrict__ tok,
                                                         uint16_t *__restrict__ xs, int P, int H) {
    const int pieces = H / 8;
    const int64_t total = (int64_t)P * pieces, stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int row = (int)(i / pieces), c = (int)(i % pieces);
        reinterpret_cast<u32x4 *>(xs)[i] = reinterpret_cast<const u32x4 *>(x + (size_t)tok[row] * H)[c];
    }
}

// h = bf16( silu(g) * u ), 4 elements per thread
__global__ __launch_bounds__(256) void moe_act_kernel(const float *__restrict__ g, const float *__restrict__ u,
                                                      uint16_t *__restrict__ h, int64_t n4) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
        const f32x4 a = reinterpret_cast<const f32x4 *>(g)[i], b = reinterpret_cast<const f32x4 *>(u)[i];
        float r[4];
        const float av[4] = {a.x, a.y, a.z, a.w}, bv[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) r[j] = av[j] / (1.f + __expf(-av[j])) * bv[j];
        u32x2 o = {f32_to_bf16_bits(r[0]) | (f32_to_bf16_bits(r[1]) << 16), f32_to_bf16_bits(r[2]) | (f32_to_bf16_bits(r[3]) << 16)};
        reinterpret_cast<u32x2 *>(h)[i] = o;
    }
}

// y[t] = bf16( sum_j w[t,j] * sum_s yp[s][pos[t*top_k+j]] ), slots in order, K-split parts in order; 4 columns per thread
__global__ __launch_bounds__(256) void moe_combine_kernel(const float *__restrict__ yp, const int32_t *__restrict__ pos,
                                                          const float *__restrict__ w, uint16_t *__restrict__ y, int T,
                                                          int H, int top_k, int nsplit, size_t split_stride) {
    const int q = H / 4;
    const int64_t total = (int64_t)T * q, stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int t = (int)(i / q), c = (int)(i % q);
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        for (int j = 0; j < top_k; ++j) {
            f32x4 v = reinterpret_cast<const f32x4 *>(yp + (size_t)pos[t * top_k + j] * H)[c];
            for (int sp = 1; sp < nsplit; ++sp)
                v += reinterpret_cast<const f32x4 *>(yp + sp * split_stride + (size_t)pos[t * top_k + j] * H)[c];
            acc += v * w[t * top_k + j];
        }
        u32x2 o = {f32_to_bf16_bits(acc.x) | (f32_to_bf16_bits(acc.y) << 16), f32_to_bf16_bits(acc.z) | (f32_to_bf16_bits(acc.w) << 16)};
        reinterpret_cast<u32x2 *>(y)[i] = o;
    }
}

static size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

// carve-up of the workspace; base == nullptr just measures
static size_t moe_layout(uint8_t *base, int T, int H, int F, int E, int top_k, MoeWs *ws) {
    const size_t P = (size_t)T * top_k;
    size_t o = 0;
    auto take = [&](size_t bytes) {
        uint8_t *p = base ? base + o : nullptr;
        o += align_up(bytes);
        return p;
    };
    MoeWs w;
    w.idx = (int32_t *)take(P * 4);
    w.w = (float *)take(P * 4);
    w.pos = (int32_t *)take(P * 4);
    w.tok = (int32_t *)take(P * 4);
    w.cnt = (int32_t *)take((size_t)2 * E * 4);
    w.groups = (GemmGroup *)take((size_t)3 * E * sizeof(GemmGroup));
    w.tiles = (int32_t *)take(((size_t)E + P / 32 + 1) * 4);
    w.xs = (uint16_t *)take(P * H * 2);
    w.g = (float *)take(P * F * 4);
    w.u = (float *)take(P * F * 4);
    w.h = (uint16_t *)take(P * F * 2);
    w.yp = (float *)take(P * H * 4 * MOE_KSPLIT);
    const size_t g16h = (size_t)(((H >> 5) + 15) & ~15), g16f = (size_t)(((F >> 5) + 15) & ~15);
    w.ha = (uint16_t *)take(P * F * 2);
    w.rsx = (float *)take(P * 4);
    w.rsh = (float *)take(P * 4);
    w.gxh = (uint16_t *)take(P * g16h * 2);
    w.gxl = (uint16_t *)take(P * g16h * 2);
    w.ghh = (uint16_t *)take(P * g16f * 2);
    w.ghl = (uint16_t *)take(P * g16f * 2);
    w.rowmax = (uint32_t *)take(P * 4);
    if (ws) *ws = w;
    return o;
}

size_t moe_workspace_bytes(int T, int H, int F, int E, int top_k) { return moe_layout(nullptr, T, H, F, E, top_k, nullptr); }

int moe_route_launch(const float *logits, int32_t *idx, float *w, int T, int E, int top_k, int renorm, hipStream_t st) {
    MoeWs ws = {};
    MoeExperts ex = {};
    hipLaunchKernelGGL(moe_route_kernel, dim3(1), dim3(1024), 0, st, logits, idx, w, T, E, top_k, renorm, ws, ex, 0, 0, nullptr, 0, 0, nullptr);
    return hip_check(hipGetLastError(), "moe_route launch");
}

// tiled: the experts' weights and scales are in the tile order of chadq_repack_i4g32_tiles (the skinny kernel only)
bool moe_ffn_tiled_ok(int H, int F) { return gemm_expert_ok(H, F); }

int moe_ffn_i4g32_launch(const uint16_t *x, const float *logits, const chadq_moe_expert_i4g32 *experts, uint16_t *y,
                         int T, int H, int F, int E, int top_k, int renorm, void *workspace, bool tiled, hipStream_t st) {
    MoeWs ws;
    moe_layout(reinterpret_cast<uint8_t *>(workspace), T, H, F, E, top_k, &ws);
    MoeExperts ex = {};
    for (int e = 0; e < E; ++e) {
        ex.wg[e] = experts[e].wg;
        ex.sg[e] = experts[e].sg;
        ex.wu[e] = experts[e].wu;
        ex.su[e] = experts[e].su;
        ex.wd[e] = experts[e].wd;
        ex.sd[e] = experts[e].sd;
    }
    const int P = T * top_k;
    const int m_max = P < T ? P : T;  // an expert gets a token at most once
    const int tile_rows = tiled ? gemm_expert_tile_rows() : gemm_skinny_tile_rows();
    const int ntiles = E + P / tile_rows;  // sum over experts of ceil(rows / tile_rows) <= this
    int nsplit = 1;
    bool aligned = true;  // the expert kernels load scales 16 bytes at a time
    for (int e = 0; e < E; ++e)
        aligned = aligned && aligned16(experts[e].wg) && aligned16(experts[e].sg) && aligned16(experts[e].wu) &&
                  aligned16(experts[e].su) && aligned16(experts[e].wd) && aligned16(experts[e].sd);
    const bool skinny = aligned && (tiled ? gemm_expert_ok(H, F) : gemm_skinny_ok(H, F)) && tile_rows <= 128;
    if (tiled && !skinny) return fail(CHADQ_ERR_ALIGN, "moe_ffn (tiled): weights and scales must be 16-byte aligned, H and F multiples of 256");
    const int route_threads = P <= 256 ? 256 : P <= 512 ? 512 : 1024;
    int rc;
    if (skinny) {  // the router also lists the token tiles; gate/up read the activations through tok
        hipLaunchKernelGGL(moe_route_kernel, dim3(tiled ? 1 + T : 1), dim3(route_threads), 0, st, logits, ws.idx, ws.w, T, E, top_k, renorm,
                           ws, ex, H, F, x, tile_rows, ntiles, tiled ? x : nullptr);
        rc = hip_check(hipGetLastError(), "moe route launch");
    } else {
        hipLaunchKernelGGL(moe_route_kernel, dim3(1), dim3(route_threads), 0, st, logits, ws.idx, ws.w, T, E, top_k, renorm, ws, ex,
                           H, F, nullptr, 0, 0, nullptr);
        hipLaunchKernelGGL(moe_gather_kernel, dim3(512), dim3(256), 0, st, x, ws.tok, ws.xs, P, H);
        rc = hip_check(hipGetLastError(), "moe route/gather launch");
    }
    if (rc) return rc;
    if (tiled) {
        // (the router's launch also made the fp16 form of the activations) gate/up with the SiLU gate, h to fp16, down split over K
        rc = gemm_expert_gateup(ws.groups, ws.tiles, ws.tok, ntiles, E, F, H, ws.xs, ws.rsx, ws.gxh, ws.gxl, ws.h, ws.rowmax, st);
        if (rc) return rc;
        rc = expert_prep_h_launch(ws.h, ws.rowmax, P, F, ws.ha, ws.rsh, ws.ghh, ws.ghl, st);
        if (rc) return rc;
        nsplit = gemm_expert_down_splits(F);
        rc = gemm_expert_down(ws.groups, ws.tiles, ntiles, E, H, F, ws.ha, ws.rsh, ws.ghh, ws.ghl, ws.yp, nsplit, (size_t)P * H, st);
        if (rc) return rc;
    } else if (skinny) {
        rc = gemm_skinny_gateup(ws.groups, ws.tiles, ws.tok, ntiles, E, F, H, st);  // h = bf16(silu(gate) * up), [P,F]
        if (rc) return rc;
        nsplit = (F % (256 * MOE_KSPLIT) == 0) ? MOE_KSPLIT : 1;
        rc = gemm_skinny_down(ws.groups, ws.tiles, ntiles, E, H, F, nsplit, (size_t)P * H, st);  // fp32 parts [nsplit][P,H]
        if (rc) return rc;
    } else {
        rc = gemm_i4g32_grouped(ws.groups, 2 * E, m_max, F, H, true, st);  // gate and up: fp32 [P,F] each
        if (rc) return rc;
        hipLaunchKernelGGL(moe_act_kernel, dim3(2048), dim3(256), 0, st, ws.g, ws.u, ws.h, (int64_t)P * F / 4);
        rc = gemm_i4g32_grouped(ws.groups + 2 * E, E, m_max, H, F, true, st);  // down: fp32 [P,H]
        if (rc) return rc;
    }
    hipLaunchKernelGGL(moe_combine_kernel, dim3(1024), dim3(256), 0, st, ws.yp, ws.pos, ws.w, y, T, H, top_k, nsplit,
                       (size_t)P * H);
    return hip_check(hipGetLastError(), "moe act/combine launch");
}

}  // namespace chadq
