// Decode GEMV on int4 group-32 weights, matrix-core form, for 1 <= M <= 8 activation rows.
//
// The kernel is HBM-bound by design; the matrix core is used only because it makes the dot products free
// of vector-ALU work, which is what limits a plain dot-product kernel on this shape (about 12 VALU
// instructions per 8 nibbles are affordable at full HBM rate; unpack alone costs 7).
//
// One v_mfma_f32_16x16x32_bf16 step, D[16x16] += A[16x32] * B[32x16]:
//   B = weights.  Lane (n = lane%16, j = lane/16) loads 16 packed bytes of output row n0+n: the 32 nibbles
//       of scale group 4c+j.  A wave-wide load is 16 rows x 64 contiguous bytes.  The four 32-bit words of
//       the load are the B operands of four MFMA steps t = 0..3 (8 k each); lane group j supplies k-slots
//       8j..8j+7.  Nibbles become bf16 128+u by OR-ing into 0x4300 (exact).
//   A = activations, block diagonal.  Row i = 4j'+m of A is activation row m restricted to lane group j':
//       A[4j'+m][k-slot group j] = x[m][those 8 k] if j == j', else 0.  So D[4j+m][n] is the dot product of
//       activation row m with ONE scale group (4c+j) of weight row n, and the lane that holds D[4j..4j+3][n]
//       is lane (n, j) - the lane that loaded that group and its scale.  One fp32 FMA per activation row
//       applies the scale; nothing crosses lanes inside the K loop.
//   C = -136 * sum of the group's activations, which turns 128+u into u-8.  For integer-valued activations
//       every term is an exact fp32 integer, so integer accumulation stays bit-exact.
// Up to 4 activation rows ride in one pass; MP = 2 runs two passes over the same unpacked weights.
//
// Workgroup = RBW row blocks (16 rows each) x 4 K-slices, one wave each.  K is consumed in chunks of 4096
// (1024 k = 8 steps per wave).  Every wave issues, in this order, its activation loads, ONE load for its
// 16 x 32 tile of scales (parked in a wave-private LDS tile and read back 2 bytes at a time) and its eight
// weight loads, all before the first wait; memory returns in order, so what is needed first is asked for
// first.  The workgroup then stages the chunk's activations into LDS in A-operand order while the weights
// are still in flight.  Partial
// sums of the 4 lane groups and 4 K-slices meet in LDS at the end; results are written once, in a fixed
// order (deterministic).
#include "chadq_common.h"

namespace chadq {

constexpr int KC = 4096;             // k per chunk
constexpr int CSC = KC / 128;        // 128-k steps per chunk (32)
constexpr int XA_BYTES = CSC * 1024; // A operands of one pass for one chunk: [c][t][j][m] x 16 B
constexpr int NX_BYTES = (KC / 32) * 16;  // C operands: [group][m] fp32
constexpr int ZERO_BYTES = 1024;

template <int MP, int RBW>
struct GemvLds {
    static constexpr int PASS = XA_BYTES + NX_BYTES;
    static constexpr int ZERO_OFF = MP * PASS;
    static constexpr int SC_OFF = ZERO_OFF + ZERO_BYTES;  // per-wave scale tiles: 16 rows x (64 B + 16 pad)
    static constexpr int SC_WAVE = 16 * 80;
    static constexpr int OPER_BYTES = SC_OFF + RBW * 4 * SC_WAVE;
    static constexpr int RED_BYTES = RBW * 4 * 64 * MP * 16;  // reuses the operand area after the K loop
    static constexpr int TOTAL = OPER_BYTES > RED_BYTES ? OPER_BYTES : RED_BYTES;
};

// waves_per_eu(4): at most 128 VGPRs, which also makes the compiler pick the MFMA form that writes VGPRs
// MT = number of activation rows (compile time, so that no staging load hides behind a branch).
template <int MT, int RBW>
__global__ __launch_bounds__(256 * RBW) __attribute__((amdgpu_waves_per_eu(4))) void gemv_i4g32_mfma_kernel(const uint16_t *__restrict__ x,
                                                                    const uint8_t *__restrict__ wp,
                                                                    const uint16_t *__restrict__ sc,
                                                                    float *__restrict__ y, int N, int K) {
    constexpr int M = MT, MP = (MT + 3) / 4;
    typedef GemvLds<MP, RBW> L;
    constexpr int T = 256 * RBW;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rbl = wave >> 2, ks = wave & 3;
    const int nl = lane & 15, j = lane >> 4;
    const int n0 = (blockIdx.x * RBW + rbl) * 16;
    const int KH = K >> 1, G = K >> 5;
    const int row = (n0 + nl < N) ? n0 + nl : N - 1;
    const uint32_t wrow = (uint32_t)row * (uint32_t)KH;  // byte offset; the host checks N*K/2 < 2^31
    const uint32_t srow = (uint32_t)row * (uint32_t)G;
    const uint32_t mask_r = vgpr_const(0x000F000Fu), magic_r = vgpr_const(kBf16Magic);

    // the zero block that A lanes off the diagonal (and padding activation rows) read from
    for (int o = tid * 16; o < ZERO_BYTES; o += T * 16) *reinterpret_cast<u32x4 *>(lds + L::ZERO_OFF + o) = u32x4{0, 0, 0, 0};

    // A-operand address of this lane per pass: real data only where row 4j'+m meets k-slot group j'=j and
    // activation row 4p+m exists; every other lane reads zeros (stride 0 keeps it inside the zero block)
    uint32_t a_base[MP], a_step[MP];
#pragma unroll
    for (int p = 0; p < MP; ++p) {
        const bool act = (((lane & 15) >> 2) == j) && (4 * p + (lane & 3) < M);
        a_base[p] = act ? (uint32_t)(p * L::PASS + ks * 8192 + 64 * j + 16 * (lane & 3)) : (uint32_t)L::ZERO_OFF;
        a_step[p] = act ? 1024u : 0u;  // LDS bytes between this wave's consecutive 128-k steps
    }

    f32x4 acc[MP];
#pragma unroll
    for (int p = 0; p < MP; ++p) acc[p] = f32x4{0.f, 0.f, 0.f, 0.f};

    constexpr int XI = (4 * (KC / 8)) / T;  // activation pieces (16 B) per thread per pass when 4 rows are live
    for (int kc0 = 0; kc0 < K; kc0 += KC) {
        // 1. activation loads FIRST: memory returns in order, so the wait for these must not sit behind the
        //    weight stream.  Piece `it` = tid + T*r of pass p: row m = it / 512, i8 = it % 512 = 16c + 4j + t.
        u32x4 xr[MP][XI];
#pragma unroll
        for (int p = 0; p < MP; ++p)
#pragma unroll
            for (int r = 0; r < XI; ++r) {
                const int m = (T * r) / (KC / 8);  // same for the whole workgroup: T divides KC/8
                if (4 * p + m >= M) continue;      // compile-time after unrolling
                const int k = kc0 + 8 * ((tid + T * r) % (KC / 8));
                xr[p][r] = *reinterpret_cast<const u32x4 *>(x + (k < K ? (size_t)(4 * p + m) * K + k : 0));
            }

        // 2. the wave's scale tile: 16 rows x 32 groups (64 B per row) in one load; lane (n,j) takes groups
        //    8j..8j+7 of the wave's K-slice.  Needs G % 8 == 0 (16-byte aligned rows), checked on the host.
        const int gs = (kc0 >> 5) + 32 * ks + 8 * j;
        u32x4 sv = *reinterpret_cast<const u32x4 *>(sc + (srow + (uint32_t)(gs < G ? gs : 0)));
        if (gs >= G) sv = u32x4{0, 0, 0, 0};

        // 3. this wave's weight loads for the chunk: steps c = 8*ks + i, lane (n,j) takes group 4c+j
        u32x4 w[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int g = (kc0 >> 5) + 4 * (8 * ks + i) + j;
            w[i] = load_nt_b128(wp + (wrow + (uint32_t)(g < G ? g : 0) * 16u));
        }
        __builtin_amdgcn_sched_barrier(0);  // every load above is issued before anything below may wait

        // 4. stage the activations: 16-byte pieces (8 k) -> [c][t][j][m], paired for the unpack order, and
        //    the C operands -136 * (sum of the group's 32 activations)
        __syncthreads();  // previous chunk's operand reads (or the zero fill) are done
        uint8_t *sct = lds + L::SC_OFF + wave * L::SC_WAVE;  // wave-private: no barrier between write and reads
        *reinterpret_cast<u32x4 *>(sct + nl * 80 + j * 16) = sv;
#pragma unroll
        for (int p = 0; p < MP; ++p)
#pragma unroll
            for (int r = 0; r < XI; ++r) {
                const int m = (T * r) / (KC / 8);  // same for the whole workgroup: T divides KC/8
                if (4 * p + m >= M) continue;      // padding row (compile time): its A lanes read the zero block
                const int i8 = (tid + T * r) % (KC / 8);
                u32x4 v = xr[p][r];
                if (kc0 + 8 * i8 >= K) v = u32x4{0, 0, 0, 0};
                uint32_t a[4] = {v.x, v.y, v.z, v.w}, o[4];
                float sum = 0.f;
#pragma unroll
                for (int q = 0; q < 4; ++q) sum = dot2_bf16(a[q], 0x3F803F80u, sum);
                pair_x8(a, o);
                const int c = i8 >> 4, jj = (i8 >> 2) & 3, t = i8 & 3;
                *reinterpret_cast<u32x4 *>(lds + p * L::PASS + c * 1024 + t * 256 + jj * 64 + m * 16) =
                    u32x4{o[0], o[1], o[2], o[3]};
                sum += dpp_f32<0xB1, 0xF>(sum);  // the 4 pieces of a group sit in 4 adjacent lanes
                sum += dpp_f32<0x4E, 0xF>(sum);
                if (t == 0)
                    *reinterpret_cast<float *>(lds + p * L::PASS + XA_BYTES + (i8 >> 2) * 16 + m * 4) = -kMagicBias * sum;
            }
        __syncthreads();

        // 5. the chunk's 8 steps of this wave
        uint32_t a_addr[MP];
#pragma unroll
        for (int p = 0; p < MP; ++p) a_addr[p] = a_base[p];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int c = 8 * ks + i;
            uint32_t pw[16];
            unpack8_magic_r(w[i].x, mask_r, magic_r, &pw[0]);
            unpack8_magic_r(w[i].y, mask_r, magic_r, &pw[4]);
            unpack8_magic_r(w[i].z, mask_r, magic_r, &pw[8]);
            unpack8_magic_r(w[i].w, mask_r, magic_r, &pw[12]);
            const float s = f16_bits_to_f32(*reinterpret_cast<const uint16_t *>(sct + nl * 80 + (4 * i + j) * 2));
#pragma unroll
            for (int p = 0; p < MP; ++p) {
                f32x4 d = *reinterpret_cast<const f32x4 *>(lds + p * L::PASS + XA_BYTES + (4 * c + j) * 16);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const bf16x8 av = *reinterpret_cast<const bf16x8 *>(lds + a_addr[p] + t * 256);
                    const u32x4 bw = {pw[4 * t], pw[4 * t + 1], pw[4 * t + 2], pw[4 * t + 3]};
                    bf16x8 bv;
                    __builtin_memcpy(&bv, &bw, 16);
                    d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bv, d, 0, 0, 0);
                }
                acc[p] += d * s;
                a_addr[p] += a_step[p];
            }
        }
    }

    // 6. fold the 4 lane groups and the 4 K-slices: RED[wave][lane][pass] = 4 floats
    __syncthreads();  // every wave is done with the operand area, which the partial sums now reuse
    u32x4 *red = reinterpret_cast<u32x4 *>(lds);
#pragma unroll
    for (int p = 0; p < MP; ++p) {
        u32x4 v;
        __builtin_memcpy(&v, &acc[p], 16);
        red[(wave * 64 + lane) * MP + p] = v;
    }
    __syncthreads();
    if (tid < RBW * 16 * 4 * MP) {
        // tid -> (row block, pass, activation row m, weight row n); n fastest so that stores are contiguous
        const int n = tid & 15, m = (tid >> 4) & 3, p = (tid >> 6) % MP, rb = tid / (64 * MP);
        float t = 0.f;
#pragma unroll
        for (int k4 = 0; k4 < 4; ++k4)
#pragma unroll
            for (int q = 0; q < 4; ++q)
                t += reinterpret_cast<const float *>(red)[(((rb * 4 + k4) * 64 + n + 16 * q) * MP + p) * 4 + m];
        const int nn = (blockIdx.x * RBW + rb) * 16 + n, mm = 4 * p + m;
        if (nn < N && mm < M) y[(size_t)mm * N + nn] = t;
    }
}

int gemv_i4g32_dispatch(const uint16_t *, const uint8_t *, const uint16_t *, float *, int, int, int, hipStream_t);

template <int MT, int RBW>
static int launch_mfma(const uint16_t *x, const uint8_t *wp, const uint16_t *sc, float *y, int N, int K,
                       hipStream_t st) {
    typedef GemvLds<(MT + 3) / 4, RBW> L;
    static bool attr_set = false;
    if (!attr_set) {
        CHADQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_i4g32_mfma_kernel<MT, RBW>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, L::TOTAL));
        attr_set = true;
    }
    const int rbs = (N + 15) / 16;
    hipLaunchKernelGGL((gemv_i4g32_mfma_kernel<MT, RBW>), dim3((rbs + RBW - 1) / RBW), dim3(256 * RBW), L::TOTAL, st, x,
                       wp, sc, y, N, K);
    return hip_check(hipGetLastError(), "gemv_i4g32_mfma launch");
}

int gemv_i4g32_mfma_dispatch(const uint16_t *x, const uint8_t *wp, const uint16_t *sc, float *y, int M, int N, int K,
                             hipStream_t st) {
    // up to 8 activation rows per launch; more rows reuse the kernel on the next 8
    // the matrix-core kernel wants 16-byte aligned scale rows (K % 256 == 0) and 32-bit byte offsets
    if ((K & 255) != 0 || (int64_t)N * (K / 2) >= ((int64_t)1 << 31) || (reinterpret_cast<uintptr_t>(sc) & 15u) != 0)
        return gemv_i4g32_dispatch(x, wp, sc, y, M, N, K, st);
    for (int m0 = 0; m0 < M; m0 += 8) {
        const int mm = (M - m0) < 8 ? (M - m0) : 8;
        const uint16_t *xm = x + (size_t)m0 * K;
        float *ym = y + (size_t)m0 * N;
        int rc = 0;
        switch (mm) {
            case 1: rc = launch_mfma<1, 1>(xm, wp, sc, ym, N, K, st); break;
            case 2: rc = launch_mfma<2, 1>(xm, wp, sc, ym, N, K, st); break;
            case 3: rc = launch_mfma<3, 1>(xm, wp, sc, ym, N, K, st); break;
            case 4: rc = launch_mfma<4, 1>(xm, wp, sc, ym, N, K, st); break;
            case 5: rc = launch_mfma<5, 2>(xm, wp, sc, ym, N, K, st); break;
            case 6: rc = launch_mfma<6, 2>(xm, wp, sc, ym, N, K, st); break;
            case 7: rc = launch_mfma<7, 2>(xm, wp, sc, ym, N, K, st); break;
            default: rc = launch_mfma<8, 2>(xm, wp, sc, ym, N, K, st); break;
        }
        if (rc != 0) return rc;
    }
    return 0;
}

}  // namespace chadq
