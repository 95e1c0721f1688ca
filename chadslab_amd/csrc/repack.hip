// Tile order for int4 group-32 weights, the form the mixture-of-experts kernel streams fastest.
//
// The row-major container has a row's packed bytes K/2 apart from the next row's, so a workgroup that needs 64 rows x
// 128 k fetches 64 separate 64-byte runs.  In tile order the same bytes are contiguous:
//   packed   tile (band b = n / 32, column tile t = k / 128) = 2048 bytes at ((b * K/128) + t) * 2048.  Inside the
//            tile row r = n % 32 has its 64 bytes at r * 64 as four 16-byte pieces (one scale group each), piece p
//            stored at position p ^ ((r >> 1) & 3) - the order the kernel keeps them in LDS, where that swizzle
//            spreads the fragment reads over the banks, so that its DMA is a linear copy.
//   scales   block (band b, column block c = k / 256) = 512 bytes at ((b * K/256) + c) * 512: row r's 8 fp16 scales at
//            r * 16.
// A band holds the same bytes as the 32 rows it replaces, so the arrays keep their sizes.  N % 32 == 0, K % 256 == 0.
// Both directions move 16 bytes per thread; the mapping is a bijection (checked bit for bit against the CPU
// restatement and by the round trip).
#include "chadq_common.h"

namespace chadq {

// piece index i over the packed array in ROW-MAJOR order: row n, 16-byte piece g (= scale group) of that row
__device__ __forceinline__ size_t tiled_packed_piece(size_t n, size_t g, int K) {
    const size_t b = n >> 5, r = n & 31, t = g >> 2, p = g & 3;
    return ((b * (size_t)(K >> 7) + t) * 2048 + r * 64 + ((p ^ ((r >> 1) & 3)) << 4)) >> 4;
}
// 16-byte piece c (8 groups = 256 k) of row n's scales
__device__ __forceinline__ size_t tiled_scale_piece(size_t n, size_t c, int K) {
    const size_t b = n >> 5, r = n & 31;
    return ((b * (size_t)(K >> 8) + c) * 512 + r * 16) >> 4;
}

template <bool TO_TILES>
__global__ __launch_bounds__(256) void repack_i4g32_tiles_kernel(const u32x4 *__restrict__ wp_in, const u32x4 *__restrict__ sc_in,
                                                                 u32x4 *__restrict__ wp_out, u32x4 *__restrict__ sc_out, int N, int K) {
    const size_t G = (size_t)(K >> 5), C = (size_t)(K >> 8);
    const size_t n_w = (size_t)N * G, n_s = (size_t)N * C;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_w + n_s; i += (size_t)gridDim.x * blockDim.x) {
        if (i < n_w) {
            const size_t n = i / G, g = i % G, j = tiled_packed_piece(n, g, K);
            if (TO_TILES) wp_out[j] = wp_in[i];
            else wp_out[i] = wp_in[j];
        } else {
            const size_t q = i - n_w, n = q / C, c = q % C, j = tiled_scale_piece(n, c, K);
            if (TO_TILES) sc_out[j] = sc_in[q];
            else sc_out[q] = sc_in[j];
        }
    }
}

int repack_i4g32_tiles_launch(const uint8_t *wp_in, const uint16_t *sc_in, uint8_t *wp_out, uint16_t *sc_out, int N, int K,
                              bool to_tiles, hipStream_t st) {
    if (N == 0 || K == 0) return 0;
    const size_t pieces = (size_t)N * (K >> 5) + (size_t)N * (K >> 8);
    const int blocks = (int)((pieces + 255) / 256 < 65536 ? (pieces + 255) / 256 : 65536);
    const u32x4 *wi = reinterpret_cast<const u32x4 *>(wp_in), *si = reinterpret_cast<const u32x4 *>(sc_in);
    u32x4 *wo = reinterpret_cast<u32x4 *>(wp_out), *so = reinterpret_cast<u32x4 *>(sc_out);
    if (to_tiles) hipLaunchKernelGGL((repack_i4g32_tiles_kernel<true>), dim3(blocks), dim3(256), 0, st, wi, si, wo, so, N, K);
    else hipLaunchKernelGGL((repack_i4g32_tiles_kernel<false>), dim3(blocks), dim3(256), 0, st, wi, si, wo, so, N, K);
    return hip_check(hipGetLastError(), "repack_i4g32_tiles launch");
}

}  // namespace chadq
