// Tile order for int4 group-32 weights, the form the mixture-of-experts kernel streams fastest.
//
// The row-major container has a row's packed bytes K/2 apart from the next row's, so a wave that needs one scale group
// (16 bytes) of each of 32 rows fetches 32 separate pieces.  In tile order the same bytes are contiguous in the order
// the expert kernel's lanes consume them, so that each of its load instructions reads 1 KiB of consecutive memory
// straight into registers:
//   packed   unit (band b = n / 32, column unit c = k / 256) = 4096 bytes at ((b * K/256) + c) * 4096.  Inside the unit
//            the 16-byte piece (= one scale group) of row r = n % 32 and group g = (k % 256) / 32 sits at
//            (g * 32 + r) * 16: group-major, the 32 rows of a group next to each other.
//   scales   block (band b, column unit c) = 512 bytes at ((b * K/256) + c) * 512: the scale of row r and group g at
//            ((g % 2) * 32 + r) * 8 + (g / 2) * 2, i.e. per row first the four even groups' scales, 256 bytes further
//            the four odd groups' (a lane of the kernel works on the even or on the odd groups of its row).
// A band holds the same bytes as the 32 rows it replaces, so the arrays keep their sizes.  N % 32 == 0, K % 256 == 0.
// Both directions move 16 bytes per thread; the mapping is a bijection (checked bit for bit against the CPU
// restatement and by the round trip).
#include "chadq_common.h"

namespace chadq {

// piece index i over the packed array in ROW-MAJOR order: row n, 16-byte piece g (= scale group) of that row
__device__ __forceinline__ size_t tiled_packed_piece(size_t n, size_t g, int K) {
    const size_t b = n >> 5, r = n & 31, c = g >> 3, g8 = g & 7;
    return ((b * (size_t)(K >> 8) + c) * 4096 + (g8 * 32 + r) * 16) >> 4;
}
// the eight scales of row n in column unit c (16 bytes in row-major order) live as two 8-byte halves: index of the
// even groups' half in units of 8 bytes; the odd groups' half is 32 further
__device__ __forceinline__ size_t tiled_scale_half(size_t n, size_t c, int K) {
    const size_t b = n >> 5, r = n & 31;
    return ((b * (size_t)(K >> 8) + c) * 512 + r * 8) >> 3;
}

template <bool TO_TILES>
__global__ __launch_bounds__(256) void repack_i4g32_tiles_kernel(const u32x4 *__restrict__ wp_in, const void *__restrict__ sc_in,
                                                                 u32x4 *__restrict__ wp_out, void *__restrict__ sc_out, int N, int K) {
    const size_t G = (size_t)(K >> 5), C = (size_t)(K >> 8);
    const size_t n_w = (size_t)N * G, n_s = (size_t)N * C;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_w + n_s; i += (size_t)gridDim.x * blockDim.x) {
        if (i < n_w) {
            const size_t n = i / G, g = i % G, j = tiled_packed_piece(n, g, K);
            if (TO_TILES) wp_out[j] = wp_in[i];
            else wp_out[i] = wp_in[j];
        } else {
            const size_t q = i - n_w, n = q / C, c = q % C, j = tiled_scale_half(n, c, K);
            if (TO_TILES) {  // s0..s7 -> (s0,s2,s4,s6), (s1,s3,s5,s7)
                const u32x4 v = reinterpret_cast<const u32x4 *>(sc_in)[q];
                const u32x2 ev = {__builtin_amdgcn_perm(v.y, v.x, 0x05040100u), __builtin_amdgcn_perm(v.w, v.z, 0x05040100u)};
                const u32x2 od = {__builtin_amdgcn_perm(v.y, v.x, 0x07060302u), __builtin_amdgcn_perm(v.w, v.z, 0x07060302u)};
                reinterpret_cast<u32x2 *>(sc_out)[j] = ev;
                reinterpret_cast<u32x2 *>(sc_out)[j + 32] = od;
            } else {
                const u32x2 ev = reinterpret_cast<const u32x2 *>(sc_in)[j], od = reinterpret_cast<const u32x2 *>(sc_in)[j + 32];
                const u32x4 v = {__builtin_amdgcn_perm(od.x, ev.x, 0x05040100u), __builtin_amdgcn_perm(od.x, ev.x, 0x07060302u),
                                 __builtin_amdgcn_perm(od.y, ev.y, 0x05040100u), __builtin_amdgcn_perm(od.y, ev.y, 0x07060302u)};
                reinterpret_cast<u32x4 *>(sc_out)[q] = v;
            }
        }
    }
}

int repack_i4g32_tiles_launch(const uint8_t *wp_in, const uint16_t *sc_in, uint8_t *wp_out, uint16_t *sc_out, int N, int K,
                              bool to_tiles, hipStream_t st) {
    if (N == 0 || K == 0) return 0;
    const size_t pieces = (size_t)N * (K >> 5) + (size_t)N * (K >> 8);
    const int blocks = (int)((pieces + 255) / 256 < 65536 ? (pieces + 255) / 256 : 65536);
    const u32x4 *wi = reinterpret_cast<const u32x4 *>(wp_in);
    const void *si = sc_in;
    u32x4 *wo = reinterpret_cast<u32x4 *>(wp_out);
    void *so = sc_out;
    if (to_tiles) hipLaunchKernelGGL((repack_i4g32_tiles_kernel<true>), dim3(blocks), dim3(256), 0, st, wi, si, wo, so, N, K);
    else hipLaunchKernelGGL((repack_i4g32_tiles_kernel<false>), dim3(blocks), dim3(256), 0, st, wi, si, wo, so, N, K);
    return hip_check(hipGetLastError(), "repack_i4g32_tiles launch");
}

}  // namespace chadq
