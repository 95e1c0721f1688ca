// Unpack / pack / dequantise kernels.  Pure streaming: 16-byte loads and stores, grid-stride.
#include "chadq_common.h"

namespace chadq {

// 16 packed bytes -> 32 int8 in [-8,7].  Nibbles are split with two masks; interleaving low/high nibbles of
// consecutive bytes back into k order is a byte permute.
__global__ __launch_bounds__(256) void unpack_i4_kernel(const uint8_t *__restrict__ wp, int8_t *__restrict__ q,
                                                        int64_t nbytes) {
    const int64_t nvec = nbytes >> 4;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += stride) {
        const u32x4 v = reinterpret_cast<const u32x4 *>(wp)[i];
        const uint32_t in[4] = {v.x, v.y, v.z, v.w};
        uint32_t out[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            // u - 8 per byte without borrows crossing bytes: (u | 0x80) - 8 lies in [0x78,0x87]; flipping
            // bit 7 gives [0xF8..0x07] = u - 8 as int8.
            const uint32_t lo = in[j] & 0x0F0F0F0Fu;         // k = 0,2,4,6 of this word
            const uint32_t hi = (in[j] >> 4) & 0x0F0F0F0Fu;  // k = 1,3,5,7
            const uint32_t slo = ((lo | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
            const uint32_t shi = ((hi | 0x80808080u) - 0x08080808u) ^ 0x80808080u;
            out[2 * j] = __builtin_amdgcn_perm(shi, slo, 0x05010400u);      // lo.b0 hi.b0 lo.b1 hi.b1
            out[2 * j + 1] = __builtin_amdgcn_perm(shi, slo, 0x07030602u);  // lo.b2 hi.b2 lo.b3 hi.b3
        }
        u32x4 *o = reinterpret_cast<u32x4 *>(q) + 2 * i;
        o[0] = u32x4{out[0], out[1], out[2], out[3]};
        o[1] = u32x4{out[4], out[5], out[6], out[7]};
    }
    // tail bytes (nbytes % 16), one thread each
    const int64_t tail0 = nvec << 4;
    const int64_t t = tail0 + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t < nbytes) {
        const uint8_t b = wp[t];
        q[2 * t] = (int8_t)((int)(b & 0x0F) - 8);
        q[2 * t + 1] = (int8_t)((int)(b >> 4) - 8);
    }
}

// Byte-at-a-time form for pointers that are not 16-byte aligned.
__global__ __launch_bounds__(256) void unpack_i4_bytes_kernel(const uint8_t *__restrict__ wp,
                                                              int8_t *__restrict__ q, int64_t nbytes) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nbytes; i += stride) {
        const uint8_t b = wp[i];
        q[2 * i] = (int8_t)((int)(b & 0x0F) - 8);
        q[2 * i + 1] = (int8_t)((int)(b >> 4) - 8);
    }
}

__global__ __launch_bounds__(256) void pack_i4_kernel(const int8_t *__restrict__ q, uint8_t *__restrict__ wp,
                                                      int64_t nbytes) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nbytes; i += stride) {
        const int lo = (q[2 * i] + 8) & 0x0F, hi = (q[2 * i + 1] + 8) & 0x0F;
        wp[i] = (uint8_t)(lo | (hi << 4));
    }
}

// fp32 [N,K] = (u-8) * float(scale); one thread per 16 packed bytes (= one scale group).
__global__ __launch_bounds__(256) void dequant_i4g32_kernel(const uint8_t *__restrict__ wp,
                                                            const uint16_t *__restrict__ sc, float *__restrict__ w,
                                                            int64_t ngroups) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; g < ngroups; g += stride) {
        const u32x4 v = reinterpret_cast<const u32x4 *>(wp)[g];
        const float s = f16_bits_to_f32(sc[g]);
        const uint32_t in[4] = {v.x, v.y, v.z, v.w};
        f32x4 *o = reinterpret_cast<f32x4 *>(w + g * 32);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float f[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) f[i] = (float)((int)((in[j] >> (4 * i)) & 0xF) - 8) * s;
            o[2 * j] = f32x4{f[0], f[1], f[2], f[3]};
            o[2 * j + 1] = f32x4{f[4], f[5], f[6], f[7]};
        }
    }
}

__global__ __launch_bounds__(256) void dequant_i8row_kernel(const int8_t *__restrict__ w8,
                                                            const float *__restrict__ sc, float *__restrict__ w,
                                                            int N, int K) {
    const int64_t total = (int64_t)N * K;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride)
        w[i] = (float)w8[i] * sc[i / K];
}

static int grid_for(int64_t items) {
    int64_t b = (items + 255) / 256;
    if (b < 1) b = 1;
    if (b > 256 * 32) b = 256 * 32;
    return (int)b;
}

int unpack_i4_launch(const uint8_t *wp, int8_t *q, int64_t nbytes, hipStream_t st) {
    if (aligned16(wp) && aligned16(q)) {
        const int64_t nvec = nbytes >> 4;
        hipLaunchKernelGGL(unpack_i4_kernel, dim3(grid_for(nvec)), dim3(256), 0, st, wp, q, nbytes);
    } else {
        hipLaunchKernelGGL(unpack_i4_bytes_kernel, dim3(grid_for(nbytes)), dim3(256), 0, st, wp, q, nbytes);
    }
    return hip_check(hipGetLastError(), "unpack_i4 launch");
}

int pack_i4_launch(const int8_t *q, uint8_t *wp, int64_t nbytes, hipStream_t st) {
    hipLaunchKernelGGL(pack_i4_kernel, dim3(grid_for(nbytes)), dim3(256), 0, st, q, wp, nbytes);
    return hip_check(hipGetLastError(), "pack_i4 launch");
}

int dequant_i4g32_launch(const uint8_t *wp, const uint16_t *sc, float *w, int N, int K, hipStream_t st) {
    const int64_t ngroups = (int64_t)N * (K / 32);
    hipLaunchKernelGGL(dequant_i4g32_kernel, dim3(grid_for(ngroups)), dim3(256), 0, st, wp, sc, w, ngroups);
    return hip_check(hipGetLastError(), "dequant_i4g32 launch");
}

int dequant_i8row_launch(const int8_t *w8, const float *sc, float *w, int N, int K, hipStream_t st) {
    hipLaunchKernelGGL(dequant_i8row_kernel, dim3(grid_for((int64_t)N * K)), dim3(256), 0, st, w8, sc, w, N, K);
    return hip_check(hipGetLastError(), "dequant_i8row launch");
}

}  // namespace chadq
