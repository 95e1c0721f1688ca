// Shared device helpers and the host-side error plumbing for libchadq (gfx950 only).
#pragma once
#include <atomic>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/chadq.h"

namespace chadq {

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int kWave = 64;
constexpr int kGroup = 32;                  // int4 scale group along K
constexpr uint32_t kBf16Magic = 0x43004300u;  // two bf16 128.0: OR a nibble into the low mantissa bits -> 128+u
constexpr float kMagicBias = 136.0f;          // 128 (magic) + 8 (zero point)

// ---- host side: status + thread-local message -------------------------------------------------
int fail(int code, const char *fmt, ...);
void clear_error();
// 0 if `call` succeeded, else records the HIP error and returns CHADQ_ERR_HIP.
int hip_check(hipError_t e, const char *what);
// checks that the current device is gfx950 (cached per device)
int check_device();

#define CHADQ_HIP(call)                                  \
    do {                                                 \
        int _rc = ::chadq::hip_check((call), #call);     \
        if (_rc != 0) return _rc;                        \
    } while (0)

#define CHADQ_REQUIRE(cond, code, ...)                       \
    do {                                                     \
        if (!(cond)) return ::chadq::fail((code), __VA_ARGS__); \
    } while (0)

// One member of a grouped GEMM launch (device memory): y[M,N] = x[M,K] * w[N,K]^T with int4 group-32 weights.
struct GemmGroup {
    const uint16_t *x;  // bf16 [M,K]
    const void *w;      // packed weights [N,K/2]
    const void *sc;     // fp16 scales [N,K/32]
    void *y;            // bf16 or fp32 [M,N]
    int M;
    int pad;
};

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// ---- device side ------------------------------------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t lo16) { return __uint_as_float(lo16 << 16); }

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
}

// fp32 -> bf16 bits, round to nearest even, NaN kept quiet.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x0040u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}

__device__ __forceinline__ bf16x2 as_bf16x2(uint32_t v) {
    bf16x2 r;
    __builtin_memcpy(&r, &v, 4);
    return r;
}

typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;

__device__ __forceinline__ f16x2 as_f16x2(uint32_t v) {
    f16x2 r;
    __builtin_memcpy(&r, &v, 4);
    return r;
}

__device__ __forceinline__ uint32_t pack_bf16_rne(float a, float b) {
    f32x2 f = {a, b};
    bf16x2 h = __builtin_convertvector(f, bf16x2);
    uint32_t r;
    __builtin_memcpy(&r, &h, 4);
    return r;
}

// s_waitcnt with only the vector-memory counter set (gfx9 encoding: vmcnt in bits 3:0 and 15:14)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0F70);
}

// 16 (or 2) bytes per lane from global memory straight into LDS at `lds_dst` + lane * 16 (lane * 4 for 2 bytes);
// lds_dst must be the same for the whole wave.  Completion is tracked by vmcnt; the compiler inserts no wait
// for later LDS reads of that data, so callers wait explicitly.
__device__ __forceinline__ void dma16_to_lds(const void *gsrc, void *lds_dst) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gsrc,
                                     (__attribute__((address_space(3))) void *)lds_dst, 16, 0, 0);
}
__device__ __forceinline__ void dma2_to_lds(const void *gsrc, void *lds_dst) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)gsrc,
                                     (__attribute__((address_space(3))) void *)lds_dst, 2, 0, 0);
}

// One 32-bit word of packed weights = 8 nibbles u0..u7 (u0 lowest).  Returns four registers of bf16
// pairs holding 128+u: p[i] = (128+u_i , 128+u_{i+4}), i = 0..3.  Exact: 128+u <= 143 fits bf16.
__device__ __forceinline__ void unpack8_magic(uint32_t w, uint32_t p[4]) {
    constexpr uint32_t m = 0x000F000Fu;
    p[0] = (w & m) | kBf16Magic;
    p[1] = ((w >> 4) & m) | kBf16Magic;
    p[2] = ((w >> 8) & m) | kBf16Magic;
    p[3] = ((w >> 12) & m) | kBf16Magic;
}

// (a & mask) | magic in one v_and_or_b32.  The compiler will not form it from C when both constants are
// literals (a VOP3 instruction cannot carry two), so the constants are passed in registers.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask_reg, uint32_t magic_reg) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(mask_reg), "v"(magic_reg));
    return r;
}

// Same as unpack8_magic in 7 instructions: mask_reg = 0x000F000F and magic_reg = kBf16Magic live in VGPRs.
__device__ __forceinline__ void unpack8_magic_r(uint32_t w, uint32_t mask_reg, uint32_t magic_reg, uint32_t p[4]) {
    p[0] = and_or(w, mask_reg, magic_reg);
    p[1] = and_or(w >> 4, mask_reg, magic_reg);
    p[2] = and_or(w >> 8, mask_reg, magic_reg);
    p[3] = and_or(w >> 12, mask_reg, magic_reg);
}

// 8 nibbles of word `w` (u0 lowest) -> 8 bf16 of (u-8)*s in k order, the int4 group-32 dequantisation the matrix-core
// kernels share.  fp16 magic: 0x6400|u reads 1024+u, and a nibble left in bits 7:4 reads 1024+16u; one fp32 FMA per
// element removes the offset and applies the scale, then RNE to bf16.  Callers pass s16 = s/16, c0 = -1032 s,
// c1 = -72 s, and mlo = 0x000F000F, mhi = 0x00F000F0, magic = 0x64006400 in registers so that each pair of nibbles
// costs one v_and_or_b32.
__device__ __forceinline__ bf16x8 dequant8_i4(uint32_t w, float s, float s16, float c0, float c1, uint32_t mlo, uint32_t mhi,
                                              uint32_t magic) {
    const f16x2 h0 = as_f16x2(and_or(w, mlo, magic));   // u0, u4
    const f16x2 h1 = as_f16x2(and_or(w, mhi, magic));   // 16*u1, 16*u5
    const uint32_t w8 = w >> 8;
    const f16x2 h2 = as_f16x2(and_or(w8, mlo, magic));  // u2, u6
    const f16x2 h3 = as_f16x2(and_or(w8, mhi, magic));  // 16*u3, 16*u7
    const float f0 = __builtin_fmaf((float)h0.x, s, c0), f4 = __builtin_fmaf((float)h0.y, s, c0);
    const float f1 = __builtin_fmaf((float)h1.x, s16, c1), f5 = __builtin_fmaf((float)h1.y, s16, c1);
    const float f2 = __builtin_fmaf((float)h2.x, s, c0), f6 = __builtin_fmaf((float)h2.y, s, c0);
    const float f3 = __builtin_fmaf((float)h3.x, s16, c1), f7 = __builtin_fmaf((float)h3.y, s16, c1);
    const u32x4 r = {pack_bf16_rne(f0, f1), pack_bf16_rne(f2, f3), pack_bf16_rne(f4, f5), pack_bf16_rne(f6, f7)};
    bf16x8 o;
    __builtin_memcpy(&o, &r, 16);
    return o;
}

// A constant the optimiser must keep in a vector register.
__device__ __forceinline__ uint32_t vgpr_const(uint32_t v) {
    uint32_t r;
    asm volatile("v_mov_b32 %0, %1" : "=v"(r) : "s"(v));
    return r;
}

// Eight consecutive bf16 activations in four registers a[0..3] = (x0,x1),(x2,x3),(x4,x5),(x6,x7) are
// rearranged to match unpack8_magic's pairing: o[i] = (x_i, x_{i+4}).
__device__ __forceinline__ void pair_x8(const uint32_t a[4], uint32_t o[4]) {
    o[0] = __builtin_amdgcn_perm(a[2], a[0], 0x05040100u);
    o[1] = __builtin_amdgcn_perm(a[2], a[0], 0x07060302u);
    o[2] = __builtin_amdgcn_perm(a[3], a[1], 0x05040100u);
    o[3] = __builtin_amdgcn_perm(a[3], a[1], 0x07060302u);
}

__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
    return __builtin_amdgcn_fdot2_f32_bf16(as_bf16x2(a), as_bf16x2(b), c, false);
}

// GELU, tanh form: 0.5 g (1 + tanh z), z = sqrt(2/pi) (g + 0.044715 g^3), which equals g / (1 + exp(-2z)).
// One exp and one reciprocal: cheap enough to be recomputed by every workgroup that stages an activation vector.
__device__ __forceinline__ float gelu_tanh_dev(float g) {
    const float z = 0.7978845608028654f * (g + 0.044715f * g * g * g);
    return g * __builtin_amdgcn_rcpf(1.f + __expf(-2.f * z));
}

// data-parallel-primitive move: value of `v` from the lane selected by CTRL, 0 where masked off
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xF, false));
}

// Sum over the 64 lanes of a wavefront; the total is valid in lane 63 only.
__device__ __forceinline__ float wave_sum_to_lane63(float v) {
    v += dpp_f32<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
    v += dpp_f32<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
    v += dpp_f32<0x141, 0xF>(v);  // row_half_mirror
    v += dpp_f32<0x140, 0xF>(v);  // row_mirror: every lane of a 16-lane row now holds the row sum
    v += dpp_f32<0x142, 0xA>(v);  // row_bcast15 into rows 1 and 3
    v += dpp_f32<0x143, 0xC>(v);  // row_bcast31 into rows 2 and 3
    return v;
}

__device__ __forceinline__ u32x4 load_nt_b128(const void *p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
}

// ---- wave-wide selection helpers (argmax, top-k) ----
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


}  // namespace chadq
