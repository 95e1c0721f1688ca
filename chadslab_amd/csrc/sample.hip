// Top-k sampling of the next token from n fp32 logits, on the GPU so that a captured decode step can end with it.
//
//   candidates: the k largest logits, larger first, lower index first among equals (NaN is never chosen)
//   p_j = exp((v_j - v_0) / temperature) over the candidates in that order
//   token = the first candidate whose running sum of p exceeds u * (sum of all p);  u in [0, 1) comes from device memory
//
// k = 1 is argmax.  Two launches.  Small k (below 16): in the first, each of 96 x 4 waves picks the k best of its own
// slice of the logits, held in registers (k rounds of "best of the lanes' cached bests"; only the lane that owned the
// winner rescans its elements; no workgroup barriers), and one wave merges the workgroup's four sorted lists; in the
// second, one wave merges the 96 sorted lists by their heads and draws.  Wave-wide max/min run on DPP moves, not on LDS
// permutes.  Larger k: the k best are found by a search for the k-th largest key (see "selection by threshold" below),
// whose cost does not grow with k.
#include <climits>

#include "chadq_common.h"

namespace chadq {

constexpr int TOPK_MAX = 64, TOPK_NB = 96;  // a lane holds up to 32 logits: the entry point limits n to 96 * 4 * 64 * 32
constexpr int TOPK_PICK_MIN = 16;           // k from which the selection by threshold is used (the rounds cost 5 + 1.25 k us, it 23-29)

// One wave moves the k first of the `cnt` values v[base ..] to ov/oi, in order.  Lane holds elements lane + 64 j, j < E,
// in registers (cnt <= 64 E); a taken or absent element is NaN, which is never a candidate.  Missing places are
// filled with (-inf, INT_MAX).
template <int E>
__device__ __forceinline__ void wave_select(const float *__restrict__ v, int base, int cnt, int k, float *ov, int32_t *oi) {
    const int lane = threadIdx.x & 63;
    float rv[E];
#pragma unroll
    for (int j = 0; j < E; ++j) rv[j] = (lane + 64 * j < cnt) ? v[base + lane + 64 * j] : __builtin_nanf("");
    float bv;
    int bj;
    auto rescan = [&]() {  // branch-free: the maximum (fmaxf skips NaN), then the first place that holds it
        bv = rv[0];
#pragma unroll
        for (int j = 1; j < E; ++j) bv = __builtin_fmaxf(bv, rv[j]);
        bj = -1;
#pragma unroll
        for (int j = E - 1; j >= 0; --j) bj = (rv[j] == bv) ? j : bj;  // all NaN: no place compares equal
    };
    rescan();
    int r = 0;
    for (; r < k; ++r) {
        const int bi = base + lane + 64 * bj;
        const uint32_t gi = wave_winner<64>(bj >= 0, bv, bi);
        if (gi == 0xFFFFFFFFu) break;  // uniform: nothing left
        if (bj >= 0 && (uint32_t)bi == gi) {
            ov[r] = bv;
            oi[r] = bi;
#pragma unroll
            for (int j = 0; j < E; ++j) rv[j] = (j == bj) ? __builtin_nanf("") : rv[j];
            rescan();
        }
    }
    for (int j = r + lane; j < k; j += 64) {
        ov[j] = -INFINITY;
        oi[j] = INT_MAX;
    }
}

// One wave merges nl <= LANES * LPL sorted lists of k pairs each (list l at lv[l*k..], li[l*k..], exhausted places hold
// index INT_MAX) into the k first overall, by the lists' heads, which the lanes keep in registers.  Lane owns lists
// lane, lane + LANES, ...
template <int LPL, int LANES>
__device__ __forceinline__ void wave_merge(const float *lv, const int32_t *li, int nl, int k, float *ov, int32_t *oi) {
    const int lane = threadIdx.x & 63;
    int hp[LPL], hi[LPL];
    float hv[LPL];
#pragma unroll
    for (int j = 0; j < LPL; ++j) {
        const int l = lane + LANES * j;
        const bool own = lane < LANES && l < nl;
        hp[j] = 0;
        hv[j] = own ? lv[l * k] : -INFINITY;
        hi[j] = own ? li[l * k] : INT_MAX;
    }
    int r = 0;
    for (; r < k; ++r) {
        float bv = -INFINITY;
        int bi = INT_MAX, bj = -1;
#pragma unroll
        for (int j = 0; j < LPL; ++j)
            if (hi[j] != INT_MAX && (bj < 0 || hv[j] > bv || (hv[j] == bv && hi[j] < bi))) {
                bv = hv[j];
                bi = hi[j];
                bj = j;
            }
        const uint32_t gi = wave_winner<LANES>(bj >= 0, bv, bi);
        if (gi == 0xFFFFFFFFu) break;
        if (bj >= 0 && (uint32_t)bi == gi) {
            ov[r] = bv;
            oi[r] = bi;
#pragma unroll
            for (int j = 0; j < LPL; ++j)
                if (j == bj) {
                    const int l = lane + LANES * j;
                    ++hp[j];
                    hv[j] = hp[j] < k ? lv[l * k + hp[j]] : -INFINITY;
                    hi[j] = hp[j] < k ? li[l * k + hp[j]] : INT_MAX;
                }
        }
    }
    for (int j = r + lane; j < k; j += 64) {
        ov[j] = -INFINITY;
        oi[j] = INT_MAX;
    }
}

template <int E>
__global__ __launch_bounds__(256) void topk_partial_kernel(const float *__restrict__ v, int n, int k, float *__restrict__ cv,
                                                           int32_t *__restrict__ ci) {
    __shared__ float wv[4 * TOPK_MAX];
    __shared__ int32_t wi[4 * TOPK_MAX];
    const int wave = threadIdx.x >> 6;
    const int per_wave = (n + 4 * (int)gridDim.x - 1) / (4 * (int)gridDim.x);  // <= 64 E, the launcher's choice of E
    const int base = (blockIdx.x * 4 + wave) * per_wave;
    const int cnt = max(0, min(per_wave, n - base));
    wave_select<E>(v, base, cnt, k, wv + wave * k, wi + wave * k);
    __syncthreads();
    if (wave == 0) wave_merge<1, 4>(wv, wi, 4, k, cv + (size_t)blockIdx.x * k, ci + (size_t)blockIdx.x * k);
}

__global__ __launch_bounds__(256) void topk_final_kernel(const float *__restrict__ cv, const int32_t *__restrict__ ci, int nl, int k,
                                                         float inv_temperature, const float *__restrict__ u, int n,
                                                         int32_t *__restrict__ token, int32_t *__restrict__ pos, int advance) {
    extern __shared__ float sv[];
    const int ncand = nl * k;
    int32_t *si = reinterpret_cast<int32_t *>(sv + ncand);
    __shared__ float ov[TOPK_MAX];
    __shared__ int32_t oi[TOPK_MAX];
    const int tid = threadIdx.x;
    for (int e = tid; e < ncand; e += 256) {
        sv[e] = cv[e];
        si[e] = ci[e];
    }
    __syncthreads();
    if (tid >= 64) return;
    wave_merge<(TOPK_NB + 63) / 64, 64>(sv, si, nl, k, ov, oi);
    const bool valid = tid < k && oi[tid] != INT_MAX;
    // a best logit of -inf would make every difference NaN: then only the first candidate counts
    float p = 0.f;
    if (valid) p = (ov[0] == -INFINITY) ? (tid == 0 ? 1.f : 0.f) : expf((ov[tid] - ov[0]) * inv_temperature);
    float c = p;
    for (int o = 1; o < 64; o <<= 1) {
        const float t = __shfl_up(c, o, 64);
        if (tid >= o) c += t;
    }
    const float total = __shfl(c, 63, 64);
    const float thr = u[0] * total;
    const unsigned long long hit = __ballot(valid && c > thr);
    const unsigned long long any = __ballot(valid);
    if (tid == 0) {
        int j = 0;
        if (hit) j = __ffsll((long long)hit) - 1;
        else if (any) j = 63 - __clzll((long long)any);  // rounding left the last sum at the threshold: the last candidate
        const int t = any ? oi[j] : 0;                   // no candidate at all (every logit NaN): token 0
        token[0] = min(max(t, 0), n - 1);
        if (advance) pos[0] += 1;
    }
}

// ---- selection by threshold (larger k) ----
// The k rounds above cost a wave-wide reduction each.  For larger k a wave instead finds the k-th largest key among its
// pairs by building it bit by bit (32 counts over the wave, each a compare and a population count per register), takes
// everything above it and, of the pairs that equal it, those with the lowest indices (a second bit-by-bit search, over
// the index, only when the boundary cuts through equal values).  The cost does not depend on k.

// key of a candidate: 0 for NaN and for "no pair" (the keys of numbers, -inf included, are above 0x007FFFFF)
__device__ __forceinline__ uint32_t cand_key(float v, int idx) { return (v != v || idx == INT_MAX) ? 0u : order_key(v); }

// One wave picks the k best of the pairs (v[j], idx[j]) its lanes hold (idx INT_MAX: no pair) and writes them to
// ov/oi[0 .. k) in no particular order; places for which no pair exists receive (-inf, INT_MAX).
template <int E>
__device__ __forceinline__ void wave_pick(const float (&v)[E], const int (&idx)[E], int k, float *ov, int32_t *oi) {
    const int lane = threadIdx.x & 63;
    uint32_t key[E];
#pragma unroll
    for (int j = 0; j < E; ++j) key[j] = cand_key(v[j], idx[j]);
    // a ballot and a scalar population count per register (per-lane counts summed over the wave by DPP moves took a
    // third longer: six dependent moves per count)
    auto count_ge = [&](uint32_t t) {
        int c = 0;
#pragma unroll
        for (int j = 0; j < E; ++j) c += __popcll(__ballot(key[j] >= t));
        return c;
    };
    uint32_t t = 0;  // the largest t with at least k keys >= t: the k-th largest key
    for (int bit = 31; bit >= 0; --bit) {
        const uint32_t cand = t | (1u << bit);
        if (count_ge(cand) >= k) t = cand;
    }
    if (t == 0) t = 1;  // fewer than k pairs: all of them are above 1, none equals it
    const int cgt = count_ge(t + 1);         // pairs above the boundary: all taken
    const int ceq = count_ge(t) - cgt;       // pairs on it
    const int r = min(k - cgt, ceq);         // how many of those are taken: the lowest indices
    uint32_t u = 0xFFFFFFFFu;                // taken: index <= u
    if (ceq > r) {
        u = 0;  // the smallest u with r boundary pairs of index <= u (indices are below 2^20 and distinct)
        for (int bit = 19; bit >= 0; --bit) {
            const uint32_t hi = u | ((1u << bit) - 1u);
            int c = 0;
#pragma unroll
            for (int j = 0; j < E; ++j) c += __popcll(__ballot(key[j] == t && (uint32_t)idx[j] <= hi));
            if (c < r) u |= 1u << bit;
        }
    }
    const unsigned long long below = (1ull << lane) - 1ull;
    int gbase = 0, ebase = cgt;
#pragma unroll
    for (int j = 0; j < E; ++j) {
        const bool g = key[j] > t, e = key[j] == t && (uint32_t)idx[j] <= u;
        const unsigned long long mg = __ballot(g), me = __ballot(e);
        if (g || e) {
            const int p = g ? gbase + __popcll(mg & below) : ebase + __popcll(me & below);
            ov[p] = v[j];
            oi[p] = idx[j];
        }
        gbase += __popcll(mg);
        ebase += __popcll(me);
    }
    for (int p = ebase + lane; p < k; p += 64) {
        ov[p] = -INFINITY;
        oi[p] = INT_MAX;
    }
}

// The pairs of `nlists` lists of k (LDS) -> the k best, by one wave: list l at lv/li + l * k.  nlists <= 4.
__device__ __forceinline__ void wave_pick_lists(const float *lv, const int32_t *li, int nlists, int k, float *ov, int32_t *oi) {
    const int lane = threadIdx.x & 63;
    float mv[4];
    int mi[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int e = lane + 64 * j;
        mv[j] = e < nlists * k ? lv[e] : 0.f;
        mi[j] = e < nlists * k ? li[e] : INT_MAX;
    }
    wave_pick<4>(mv, mi, k, ov, oi);
}

// Sixteen waves each pick the k best of their share (held in registers, E per lane), four waves the k best of four of
// those lists each, one wave the k best of the four that remain: three short searches instead of one long one (a
// search costs 32 passes over the wave's registers).  Returns true in the wave (wave 0) that holds the result in ov/oi.
constexpr int TOPK_PW = 16;  // waves per workgroup of the selection by threshold
template <int E>
__device__ __forceinline__ bool block_pick(const float (&v)[E], const int (&idx)[E], int k, float *ov, int32_t *oi) {
    __shared__ float l1v[TOPK_PW * TOPK_MAX], l2v[4 * TOPK_MAX];
    __shared__ int32_t l1i[TOPK_PW * TOPK_MAX], l2i[4 * TOPK_MAX];
    const int wave = threadIdx.x >> 6;
    wave_pick<E>(v, idx, k, l1v + wave * k, l1i + wave * k);
    __syncthreads();
    if (wave < 4) wave_pick_lists(l1v + 4 * wave * k, l1i + 4 * wave * k, 4, k, l2v + wave * k, l2i + wave * k);
    __syncthreads();
    if (wave != 0) return false;
    wave_pick_lists(l2v, l2i, 4, k, ov, oi);
    return true;
}

template <int E>
__global__ __launch_bounds__(64 * TOPK_PW) void topk_pick_partial_kernel(const float *__restrict__ logits, int n, int k,
                                                                         float *__restrict__ cv, int32_t *__restrict__ ci) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int nwaves = TOPK_PW * (int)gridDim.x;
    const int per_wave = (n + nwaves - 1) / nwaves;  // <= 64 E, the launcher's choice of E
    const int base = (blockIdx.x * TOPK_PW + wave) * per_wave;
    const int cnt = max(0, min(per_wave, n - base));
    float v[E];
    int idx[E];
#pragma unroll
    for (int j = 0; j < E; ++j) {
        const bool in = lane + 64 * j < cnt;
        v[j] = in ? logits[base + lane + 64 * j] : 0.f;
        idx[j] = in ? base + lane + 64 * j : INT_MAX;
    }
    block_pick<E>(v, idx, k, cv + (size_t)blockIdx.x * k, ci + (size_t)blockIdx.x * k);
}

// nl * k <= 96 * 64 candidates, up to 6 per lane of the sixteen waves; wave 0 ends up with the k best and orders them by
// counting, for every candidate, the candidates that come before it.
constexpr int TOPK_FE = (TOPK_NB * TOPK_MAX / TOPK_PW + 63) / 64;
__global__ __launch_bounds__(64 * TOPK_PW) void topk_pick_final_kernel(const float *__restrict__ cv, const int32_t *__restrict__ ci, int nl,
                                                                       int k, float inv_temperature, const float *__restrict__ u, int n,
                                                                       int32_t *__restrict__ token, int32_t *__restrict__ pos,
                                                                       int advance) {
    __shared__ float ov[TOPK_MAX];
    __shared__ int32_t oi[TOPK_MAX];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int ncand = nl * k, share = (ncand + TOPK_PW - 1) / TOPK_PW;
    float v[TOPK_FE];
    int idx[TOPK_FE];
#pragma unroll
    for (int j = 0; j < TOPK_FE; ++j) {
        const int e = lane + 64 * j, g = wave * share + e;
        const bool in = e < share && g < ncand;
        v[j] = in ? cv[g] : 0.f;
        idx[j] = in ? ci[g] : INT_MAX;
    }
    if (!block_pick<TOPK_FE>(v, idx, k, ov, oi)) return;  // unordered, in wave 0
    // order: the place of a candidate is the number of candidates before it (greater value; lower index among equal
    // values; lower lane among the empty places, which all look alike)
    const float myv = lane < k ? ov[lane] : -INFINITY;
    const int myi = lane < k ? oi[lane] : INT_MAX;
    const uint32_t myk = cand_key(myv, myi);
    int place = 0;
    for (int j = 0; j < k; ++j) {
        const uint32_t kj = (uint32_t)__builtin_amdgcn_readlane((int)myk, j);
        const int ij = __builtin_amdgcn_readlane(myi, j);
        place += (kj > myk || (kj == myk && (ij < myi || (ij == myi && j < lane)))) ? 1 : 0;
    }
    if (lane < k) {
        ov[place] = myv;
        oi[place] = myi;
    }
    // (one wave: LDS accesses of a wave execute in order, no barrier needed)
    const bool valid = tid < k && oi[tid] != INT_MAX;
    // a best logit of -inf would make every difference NaN: then only the first candidate counts
    float p = 0.f;
    if (valid) p = (ov[0] == -INFINITY) ? (tid == 0 ? 1.f : 0.f) : expf((ov[tid] - ov[0]) * inv_temperature);
    float c = p;
    for (int o = 1; o < 64; o <<= 1) {
        const float t = __shfl_up(c, o, 64);
        if (tid >= o) c += t;
    }
    const float total = __shfl(c, 63, 64);
    const float thr = u[0] * total;
    const unsigned long long hit = __ballot(valid && c > thr);
    const unsigned long long any = __ballot(valid);
    if (tid == 0) {
        int j = 0;
        if (hit) j = __ffsll((long long)hit) - 1;
        else if (any) j = 63 - __clzll((long long)any);  // rounding left the last sum at the threshold: the last candidate
        const int t = any ? oi[j] : 0;                   // no candidate at all (every logit NaN): token 0
        token[0] = min(max(t, 0), n - 1);
        if (advance) pos[0] += 1;
    }
}

int sample_topk_launch(const float *v, int n, int k, float temperature, const float *u, float *cv, int32_t *ci, int32_t *token,
                       int32_t *pos, int advance, hipStream_t st) {
    const int per_wave = (n + 4 * TOPK_NB - 1) / (4 * TOPK_NB);
    const float inv_t = 1.f / temperature;
    if (k >= TOPK_PICK_MIN) {  // cost independent of k
        const int pw = (n + TOPK_PW * TOPK_NB - 1) / (TOPK_PW * TOPK_NB);  // logits per wave: at most 512
        const dim3 grid(TOPK_NB), block(64 * TOPK_PW);
        if (pw <= 64) hipLaunchKernelGGL(topk_pick_partial_kernel<1>, grid, block, 0, st, v, n, k, cv, ci);
        else if (pw <= 128) hipLaunchKernelGGL(topk_pick_partial_kernel<2>, grid, block, 0, st, v, n, k, cv, ci);
        else if (pw <= 256) hipLaunchKernelGGL(topk_pick_partial_kernel<4>, grid, block, 0, st, v, n, k, cv, ci);
        else hipLaunchKernelGGL(topk_pick_partial_kernel<8>, grid, block, 0, st, v, n, k, cv, ci);
        hipLaunchKernelGGL(topk_pick_final_kernel, dim3(1), block, 0, st, cv, ci, TOPK_NB, k, inv_t, u, n, token, pos, advance);
        return hip_check(hipGetLastError(), "sample_topk launch");
    }
    if (per_wave <= 256) hipLaunchKernelGGL(topk_partial_kernel<4>, dim3(TOPK_NB), dim3(256), 0, st, v, n, k, cv, ci);
    else if (per_wave <= 512) hipLaunchKernelGGL(topk_partial_kernel<8>, dim3(TOPK_NB), dim3(256), 0, st, v, n, k, cv, ci);
    else if (per_wave <= 1024) hipLaunchKernelGGL(topk_partial_kernel<16>, dim3(TOPK_NB), dim3(256), 0, st, v, n, k, cv, ci);
    else hipLaunchKernelGGL(topk_partial_kernel<32>, dim3(TOPK_NB), dim3(256), 0, st, v, n, k, cv, ci);
    hipLaunchKernelGGL(topk_final_kernel, dim3(1), dim3(256), (size_t)TOPK_NB * k * 8, st, cv, ci, TOPK_NB, k, inv_t, u, n, token, pos,
                       advance);
    return hip_check(hipGetLastError(), "sample_topk launch");
}

}  // namespace chadq
