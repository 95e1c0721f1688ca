// A measuring aid for bench.py, not part of libchadq: a read of `bytes` bytes with the decode GEMV's per-wave footprint
// and nothing else (every wave owns 16 KiB, keeps four 1-KiB loads in flight, folds what it read across its lanes and
// stores one word), so that the benchmark can report what this machine delivers for a cold read of the same size next
// to the GEMV's own time.  Built into bench_probe.so next to bench.py by __graft_entry__.build().
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

constexpr int PROBE_WAVE_BYTES = 16384;  // per wave: 16 loads of 1 KiB, like a wave of the GEMV at K = 4096

__global__ __launch_bounds__(256) void probe_read_kernel(const uint8_t *__restrict__ src, size_t nwaves, uint32_t *__restrict__ out) {
    const size_t wave = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (wave >= nwaves) return;
    const uint8_t *p = src + wave * PROBE_WAVE_BYTES + lane * 16;
    u32x4 v[16];
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p + i * 1024));
    uint32_t acc = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        asm volatile("" : "+v"(v[i]));  // wait for exactly this load
        if (i + 4 < 16) v[i + 4] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p + (i + 4) * 1024));
        acc ^= v[i].x ^ v[i].y ^ v[i].z ^ v[i].w;
    }
    for (int o = 1; o < 64; o <<= 1) acc ^= (uint32_t)__shfl_xor((int)acc, o, 64);
    if (lane == 0) out[wave] = acc;
}

// Reads the first bytes / 16384 * 16384 bytes of src (16-byte aligned device memory) and stores one word per 16 KiB to
// out.  Returns 0, or the HIP error code of the launch.
extern "C" int bench_probe_read(const void *src, int64_t bytes, uint32_t *out, void *stream) {
    if (!src || !out || bytes < 0 || (reinterpret_cast<uintptr_t>(src) & 15u)) return -1;
    const size_t nwaves = (size_t)bytes / PROBE_WAVE_BYTES;
    if (nwaves == 0) return 0;
    hipLaunchKernelGGL(probe_read_kernel, dim3((unsigned)((nwaves + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
                       reinterpret_cast<const uint8_t *>(src), nwaves, out);
    return (int)hipGetLastError();
}

// A kernel that does nothing (one workgroup of one wave): what a dependent launch costs in a replayed graph on this
// machine, the floor under every small kernel of the decode step.
__global__ void probe_empty_kernel() {}

extern "C" int bench_probe_empty(void *stream) {
    hipLaunchKernelGGL(probe_empty_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream);
    return (int)hipGetLastError();
}

// What the matrix cores sustain on operands that are not zero, registers only (no memory traffic at all): 512 workgroups
// of four waves, six accumulator chains per wave, 4 x 6 MFMAs of 32 x 32 x 16 per trip.  The clock follows the power
// the arithmetic draws, so this, not the nominal peak, is the ceiling of every matrix-core-bound kernel here.
typedef __attribute__((ext_vector_type(8))) _Float16 probe_f16x8;
typedef __attribute__((ext_vector_type(8))) __bf16 probe_bf16x8;
typedef __attribute__((ext_vector_type(16))) float probe_f32x16;

template <int KIND>
__global__ __launch_bounds__(256) void probe_mfma_kernel(float *__restrict__ out, int trips) {
    probe_f32x16 acc[6];
    for (int i = 0; i < 6; ++i)
        for (int v = 0; v < 16; ++v) acc[i][v] = 0.f;
    probe_f16x8 a, b;
    probe_bf16x8 ab, bb;
    for (int e = 0; e < 8; ++e) {
        a[e] = (_Float16)(0.37f * (float)((threadIdx.x * 7 + e) % 61) - 9.f);
        b[e] = (_Float16)(0.11f * (float)((threadIdx.x * 3 + e + 1) % 53) - 2.f);
        ab[e] = (__bf16)(float)a[e];
        bb[e] = (__bf16)(float)b[e];
    }
    for (int t = 0; t < trips; ++t) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int i = 0; i < 6; ++i) {
                if (KIND == 0) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
                else acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ab, bb, acc[i], 0, 0, 0);
            }
    }
    float s = 0.f;
    for (int i = 0; i < 6; ++i)
        for (int v = 0; v < 16; ++v) s += acc[i][v];
    out[blockIdx.x * 256 + threadIdx.x] = s;
}

// kind 0: fp16, 1: bf16.  out: 512 * 256 floats.  flop per launch = 512 * 4 * trips * 24 * 32768.
extern "C" int bench_probe_mfma(int kind, int trips, float *out, void *stream) {
    if (!out || trips < 1 || kind < 0 || kind > 1) return -1;
    if (kind == 0) hipLaunchKernelGGL(probe_mfma_kernel<0>, dim3(512), dim3(256), 0, (hipStream_t)stream, out, trips);
    else hipLaunchKernelGGL(probe_mfma_kernel<1>, dim3(512), dim3(256), 0, (hipStream_t)stream, out, trips);
    return (int)hipGetLastError();
}
