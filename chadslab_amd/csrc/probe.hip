// A measuring aid, not part of the path: a read of `bytes` bytes with the decode GEMV's access shape and nothing else
// (every wave keeps four 1-KiB loads in flight, folds what it read across its lanes and stores one word), so that the
// benchmark can report what this machine delivers for a cold read of the same size next to the GEMV's own time.
#include "chadq_common.h"

namespace chadq {

constexpr int PROBE_WAVE_BYTES = 16384;  // per wave: 16 loads of 1 KiB, like a wave of the GEMV at K = 4096

__global__ __launch_bounds__(256) void probe_read_kernel(const uint8_t *__restrict__ src, size_t nwaves, uint32_t *__restrict__ out) {
    const size_t wave = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (wave >= nwaves) return;
    const uint8_t *p = src + wave * PROBE_WAVE_BYTES + lane * 16;
    u32x4 v[16];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = load_nt_b128(p + i * 1024);
    uint32_t acc = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        asm volatile("" : "+v"(v[i]));  // wait for exactly this load
        if (i + 4 < 16) v[i + 4] = load_nt_b128(p + (i + 4) * 1024);
        acc ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
    }
    for (int o = 1; o < 64; o <<= 1) acc ^= (uint32_t)__shfl_xor((int)acc, o, 64);
    if (lane == 0) out[wave] = acc;
}

int probe_read_launch(const uint8_t *src, size_t bytes, uint32_t *out, hipStream_t st) {
    const size_t nwaves = bytes / PROBE_WAVE_BYTES;
    if (nwaves == 0) return 0;
    hipLaunchKernelGGL(probe_read_kernel, dim3((unsigned)((nwaves + 3) / 4)), dim3(256), 0, st, src, nwaves, out);
    return hip_check(hipGetLastError(), "probe_read launch");
}

}  // namespace chadq
