// Top-k sampling of the next token from n fp32 logits, on the GPU so that a captured decode step can end with it.
//
//   candidates: the k largest logits, larger first, lower index first among equals (NaN is never chosen)
//   p_j = exp((v_j - v_0) / temperature) over the candidates in that order
//   token = the first candidate whose running sum of p exceeds u * (sum of all p);  u in [0, 1) comes from device memory
//
// k = 1 is argmax.  Two launches.  In the first, each of 96 x 4 waves picks the k best of its own slice of the logits,
// held in registers (k rounds of "best of the lanes' cached bests"; only the lane that owned the winner rescans its
// elements; no workgroup barriers), and one wave merges the workgroup's four sorted lists.  In the second, one wave merges the 96
// sorted lists by their heads and draws.  Wave-wide max/min run on DPP moves, not on LDS permutes.
#include <climits>

#include "chadq_common.h"

namespace chadq {

constexpr int TOPK_MAX = 64, TOPK_NB = 96;  // a lane holds up to 32 logits: the entry point limits n to 96 * 4 * 64 * 32

// floats as unsigned keys of the same order; -0 and +0 get the same key
__device__ __forceinline__ uint32_t order_key(float v) {
    const uint32_t b = __float_as_uint(v + 0.f);
    return b ^ ((b >> 31) ? 0xFFFFFFFFu : 0x80000000u);
}

// max (or min) of an unsigned value over the first LANES lanes of the wave (64, or 4: one quad), returned to every lane:
// butterflies inside the 16-lane rows, then the two row broadcasts gather the total in lane 63.  Lanes a DPP move
// does not reach receive the operation's identity, so that the compiler can fold each move into its max / min.
template <bool IS_MAX, int LANES>
__device__ __forceinline__ uint32_t wave_reduce_u32(uint32_t v) {
    constexpr int IDENT = IS_MAX ? 0 : -1;
#define CHADQ_DPP_STEP(CTRL, MASK)                                                                                  \
    {                                                                                                               \
        const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(IDENT, (int)v, CTRL, MASK, 0xF, false);            \
        v = IS_MAX ? (o > v ? o : v) : (o < v ? o : v);                                                             \
    }
    CHADQ_DPP_STEP(0xB1, 0xF)  // quad_perm [1,0,3,2]
    CHADQ_DPP_STEP(0x4E, 0xF)  // quad_perm [2,3,0,1]
    if (LANES == 4) return (uint32_t)__builtin_amdgcn_readlane((int)v, 0);
    CHADQ_DPP_STEP(0x141, 0xF)  // row_half_mirror
    CHADQ_DPP_STEP(0x140, 0xF)  // row_mirror
    CHADQ_DPP_STEP(0x142, 0xA)  // row_bcast15 into rows 1 and 3
    CHADQ_DPP_STEP(0x143, 0xC)  // row_bcast31 into rows 2 and 3
#undef CHADQ_DPP_STEP
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}

// The winner among one (value, index) pair per lane (has = false: the lane has none): the largest value, the lowest
// index among equal values.  Returns the winner's index, or 0xFFFFFFFF if no lane has a pair.  One reduction finds the
// largest value; a second one, over the indices, runs only when several lanes hold it.
template <int LANES>
__device__ __forceinline__ uint32_t wave_winner(bool has, float v, int i) {
    const uint32_t key = has ? order_key(v) : 0u;  // below the key of -inf
    const uint32_t best = wave_reduce_u32<true, LANES>(key);
    const bool match = has && key == best;
    const unsigned long long m = __ballot(match);
    if (m == 0) return 0xFFFFFFFFu;
    if ((m & (m - 1)) == 0) return (uint32_t)__builtin_amdgcn_readlane(i, __ffsll((long long)m) - 1);
    return wave_reduce_u32<false, LANES>(match ? (uint32_t)i : 0xFFFFFFFFu);
}

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

int sample_topk_launch(const float *v, int n, int k, float temperature, const float *u, float *cv, int32_t *ci, int32_t *token,
                       int32_t *pos, int advance, hipStream_t st) {
    const int per_wave = (n + 4 * TOPK_NB - 1) / (4 * TOPK_NB);
    if (per_wave <= 256) hipLaunchKernelGGL(topk_partial_kernel<4>, dim3(TOPK_NB), dim3(256), 0, st, v, n, k, cv, ci);
    else if (per_wave <= 512) hipLaunchKernelGGL(topk_partial_kernel<8>, dim3(TOPK_NB), dim3(256), 0, st, v, n, k, cv, ci);
    else if (per_wave <= 1024) hipLaunchKernelGGL(topk_partial_kernel<16>, dim3(TOPK_NB), dim3(256), 0, st, v, n, k, cv, ci);
    else hipLaunchKernelGGL(topk_partial_kernel<32>, dim3(TOPK_NB), dim3(256), 0, st, v, n, k, cv, ci);
    hipLaunchKernelGGL(topk_final_kernel, dim3(1), dim3(256), (size_t)TOPK_NB * k * 8, st, cv, ci, TOPK_NB, k, 1.f / temperature, u, n, token,
                       pos, advance);
    return hip_check(hipGetLastError(), "sample_topk launch");
}

}  // namespace chadq
