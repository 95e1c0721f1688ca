// Device helpers that turn bf16 activation rows into the operands of the tile-order expert GEMM
// (gemm_expert_i4g32.hip): fp16 values scaled per row by a power of two, and -8 times the sum of every scale group.
#pragma once
#include "chadq_common.h"

namespace chadq {

// bits of the largest finite bf16 magnitude of a row -> (2^-e, 2^e) with e such that the magnitude times 2^-e lies in
// [128, 256): largest = 1.m * 2^(E-127) gives e = E - 134.  A zero (or tiny) row keeps E = 8, the smallest e whose
// 2^e is a normal float.
__device__ __forceinline__ void prep_scale(uint32_t amax_bits, float &mult, float &back) {
    int E = (int)(amax_bits >> 7);
    E = E < 8 ? 8 : E;
    mult = __uint_as_float((uint32_t)(261 - E) << 23);
    back = __uint_as_float((uint32_t)(E - 7) << 23);
}

// largest finite magnitude among the 8 bf16 values of `v` and `amax` (bf16 bit patterns order like the magnitudes)
__device__ __forceinline__ uint32_t prep_amax8(u32x4 v, uint32_t amax) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const uint32_t lo = w[e] & 0x7FFFu, hi = (w[e] >> 16) & 0x7FFFu;
        if (lo < 0x7F80u && lo > amax) amax = lo;
        if (hi < 0x7F80u && hi > amax) amax = hi;
    }
    return amax;
}

// 8 consecutive bf16 values -> 8 fp16 of value * mult in the order 0,4,1,5,2,6,3,7 (the order in which the expert
// kernel's dequantisation leaves the 8 weights of a word); returns the sum of the 8 fp16 values.  Exact for a bf16
// input whose scaled magnitude is a normal fp16; smaller ones lose their last bits, infinities and NaNs carry over.
__device__ __forceinline__ float prep_run8(u32x4 v, float mult, u32x4 &out) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    _Float16 h[8];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        h[2 * e] = (_Float16)(bf16_bits_to_f32(w[e] & 0xFFFFu) * mult);
        h[2 * e + 1] = (_Float16)(bf16_bits_to_f32(w[e] >> 16) * mult);
    }
    float sum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) sum += (float)h[e];
    const _Float16 o[8] = {h[0], h[4], h[1], h[5], h[2], h[6], h[3], h[7]};
    __builtin_memcpy(&out, o, 16);
    return sum;
}

// -8 * (sum of scale group g of a row) as an fp16 high part and remainder; the 16 groups of a 512-k block are kept in
// the order 0,2,..,14,1,3,..,15 (a lane of the expert kernel works on the even or on the odd groups).
__device__ __forceinline__ void prep_store_group(float sum, int g, uint16_t *ghi_row, uint16_t *glo_row) {
    const int gi = g & 15, at = (g & ~15) + (gi & 1) * 8 + (gi >> 1);
    const float c = -8.f * sum;
    const _Float16 hi = (_Float16)c, lo = (_Float16)(c - (float)hi);
    uint16_t hb, lb;
    __builtin_memcpy(&hb, &hi, 2);
    __builtin_memcpy(&lb, &lo, 2);
    ghi_row[at] = hb;
    glo_row[at] = lb;
}

// K % 512 == 256: groups 8..15 of the last block do not exist and must read as zero; thread j < 8 of somebody clears one
__device__ __forceinline__ void prep_clear_tail(int G, int j, uint16_t *ghi_row, uint16_t *glo_row) {
    if ((G & 15) && j < 8) {
        const int gi = 8 + j, at = (G & ~15) + (gi & 1) * 8 + (gi >> 1);
        ghi_row[at] = 0;
        glo_row[at] = 0;
    }
}

// One whole row by the calling workgroup (any size that is a multiple of 64, up to 1024 threads): two passes over the row.
__device__ __forceinline__ void prep_row_block(const uint16_t *__restrict__ row, int K, uint16_t *__restrict__ dst_row,
                                               float *__restrict__ back_out, uint16_t *__restrict__ ghi_row,
                                               uint16_t *__restrict__ glo_row, uint32_t *s_max /* 16 words of LDS */) {
    const int tid = threadIdx.x, B = blockDim.x, lane = tid & 63, wave = tid >> 6, nw = B >> 6;
    const int nblk = K >> 3;
    uint32_t amax = 0;
    for (int b = tid; b < nblk; b += B) amax = prep_amax8(*reinterpret_cast<const u32x4 *>(row + b * 8), amax);
    amax = wave_reduce_u32<true, 64>(amax);
    if (lane == 0) s_max[wave] = amax;
    __syncthreads();
    amax = 0;
    for (int i = 0; i < nw; ++i) amax = max(amax, s_max[i]);
    float mult, back;
    prep_scale(amax, mult, back);
    if (tid == 0) *back_out = back;
    for (int b0 = 0; b0 < nblk; b0 += B) {
        const int b = b0 + tid;  // nblk is a multiple of 32: whole quads are in or out together
        float sum = 0.f;
        if (b < nblk) {
            u32x4 o;
            sum = prep_run8(*reinterpret_cast<const u32x4 *>(row + b * 8), mult, o);
            *reinterpret_cast<u32x4 *>(dst_row + b * 8) = o;
        }
        sum += dpp_f32<0xB1, 0xF>(sum);  // the 4 runs of a group sit in 4 adjacent lanes
        sum += dpp_f32<0x4E, 0xF>(sum);
        if (b < nblk && (tid & 3) == 0) prep_store_group(sum, b >> 2, ghi_row, glo_row);
    }
    prep_clear_tail(K >> 5, tid, ghi_row, glo_row);
}

}  // namespace chadq
