// Decode GEMV on int4 group-32 weights, matrix-core form, for 1 <= M <= 8 activation rows per launch.
//
// The kernel is HBM-bound by design; the matrix core is used only because it makes the dot products free
// of vector-ALU work, which is what limits a plain dot-product kernel on this shape (about 12 VALU
// instructions per 8 nibbles are affordable at full HBM rate; unpacking alone costs 7).
//
// One v_mfma_f32_16x16x32_bf16 step, D[16x16] += A[16x32] * B[32x16]:
//   B = weights.  The 16 columns are P = 16/HP weight rows times HP "K-parts": column n = h*P + r.  Lane
//       (n, j = lane/16) loads 16 packed bytes of row r: the 32 nibbles of scale group (c*HP + h)*4 + j at
//       step c.  A wave-wide load therefore covers P rows x (HP * 64) contiguous bytes: 4 rows x 256 B for
//       HP = 4, 16 rows x 64 B for HP = 1.  The four 32-bit words of the load are the B operands of four
//       MFMA steps t = 0..3 (8 k each); lane group j supplies k-slots 8j..8j+7.  Nibbles become bf16 128+u
//       by OR-ing them into 0x4300 (exact).
//   A = activations, block diagonal.  Row i = 4j' + v, v = h'*MPASS + m (MPASS = 4/HP activation rows per
//       pass): A[i][k-slots of lane group j] = x[m][the 8 k of group (c*HP + h')*4 + j', word t] if j == j',
//       else 0.  D[4j + v][n] is then the dot product of activation row m with ONE scale group of weight
//       row r - meaningful where the column's K-part h equals h' - and the lane that holds D[4j..4j+3][n]
//       is lane (n, j), the lane that loaded exactly that group and owns its scale.  One fp32 FMA per D
//       register applies the scale; nothing crosses lanes inside the K loop.  Entries with h' != h are
//       computed and never used.
//   C = -136 * sum of the group's activations, which turns 128+u into u-8.  For integer-valued activations
//       every term is an exact fp32 integer, so integer accumulation stays bit-exact.
// HP trades activation rows per pass for contiguity of the weight stream: M = 1 runs HP = 4, M = 2 runs
// HP = 2, M = 3 and 4 run HP = 1.  Five to eight rows run gemv_i4g32_mfma_pair_kernel further down, which
// regroups the loaded words between lane groups so that eight rows fit one pass.
//
// Workgroup = 4*RBW waves; each group of 4 waves covers 16 weight rows.  K is consumed in chunks of 4096;
// a wave takes 8 steps of a chunk (8 x 16 B per lane in flight), so 4/HP waves split a chunk of one row
// block.  Every wave issues, in this order, its activation loads, ONE load for its tile of scales (parked
// in a wave-private LDS tile and read back 2 bytes at a time) and its first D weight loads, all before the
// first wait: memory returns in order, so what is needed first is asked for first.  Step i issues weight
// load i+D when its own data has arrived (prefetch distance D): a wave's requests are then spread over the
// whole stream and its last bytes meet one step of arithmetic instead of eight.  The workgroup stages the
// chunk's activations into LDS in A-operand order while the weights are still in flight.  Partial sums
// of lane groups, K-parts and K-slices meet in LDS at the end; results are written once, in a fixed order
// (deterministic).
#include "chadq_common.h"

namespace chadq {

constexpr int ZERO_BYTES = 1024;

// KC = k per chunk (4096, or 2048 for short rows)
template <int MT, int HP, int S, int RBW, int KC>
struct GemvCfg {
    static constexpr int P = 16 / HP;                    // weight rows per MFMA tile
    static constexpr int MPASS = 4 / HP;                 // activation rows per pass
    static constexpr int MP = (MT + MPASS - 1) / MPASS;  // passes
    static constexpr int STEPS = KC / (128 * HP);        // steps per chunk of one row block
    static constexpr int KS = STEPS / S;                 // waves that split a chunk of one row block (S steps each)
    static constexpr int UR = P * 4 / KS;                // weight rows covered by a group of 4 waves
    static_assert(KS >= 1 && KS <= 4 && KS * S == STEPS, "a chunk of one row block is split over 1, 2 or 4 waves");
    static constexpr int XA_BYTES = STEPS * 1024;        // A operands of one pass: [c][t][j][v] x 16 B
    static constexpr int NX_BYTES = STEPS * 64;          // C operands of one pass: [c][j][v] fp32
    static constexpr int PASS = XA_BYTES + NX_BYTES;
    static constexpr int ZERO_OFF = MP * PASS;
    static constexpr int SC_OFF = ZERO_OFF + ZERO_BYTES;
    static constexpr int SC_PPR = S * HP / 2;            // 16-byte pieces (8 groups) per scale tile row
    static constexpr int SC_PITCH = SC_PPR * 16 + 16;    // scale tile row: S*4*HP fp16 + pad
    static constexpr int SC_NL = (P * SC_PPR + 63) / 64; // 16-byte scale loads per lane: the tile has 8*S pieces
    static constexpr int SC_WAVE = P * SC_PITCH;
    static constexpr int OPER_BYTES = SC_OFF + RBW * 4 * SC_WAVE;
    static constexpr int RED_BYTES = RBW * 4 * 64 * MP * 16;  // reuses the operand area after the K loop
    static constexpr int TOTAL = OPER_BYTES > RED_BYTES ? OPER_BYTES : RED_BYTES;
    static constexpr int T = 256 * RBW;
    static constexpr int XI = (MPASS * (KC / 8) + T - 1) / T;  // 16-byte activation pieces per thread per pass
};

// waves_per_eu(4): at most 128 VGPRs, which also makes the compiler pick the MFMA form that writes VGPRs.
// XM: how the activation vector comes about (M = 1 for the modes other than 0).
//   0  given: x bf16 [M,K].
//   1  GeGLU folded in: x[k] = bf16( gelu_tanh(gu[k]) * gu[K + k] ) from gu fp32 [2K] (`x` points at gu) - a gated FFN's
//      activation formed inside its down projection.
//   2  residual add and RMSNorm folded in: r = pre.res + pre.delta[0] + .. + pre.delta[n-1] (fp32, in order),
//      x = bf16( r / sqrt(mean(r^2) + eps) * pre.w ); the first workgroup also writes r to pre.res_out (a different
//      buffer than pre.res: the other workgroups are still reading that one).  One chunk only (K <= KC).
struct GemvPre {
    const float *res, *delta, *w;
    float *res_out;
    int n;
    float eps;
};

// YM: what becomes of the sums.  0: y[m,n] fp32.  1 (M = 1): the rows come in pairs (2i, 2i+1) = (gate, up) of feature i
//     of a gated FFN and the kernel writes h[i] = bf16( gelu_tanh(gate) * up ) through `y` (as uint16_t): the GeGLU of
//     a decoder layer folded into the projection that produces its inputs.  The tile rows in use (pv) must be even.
//     2 (M = 1, one wave per row block): y as for 0, and every workgroup also leaves the largest of its sums and that row's
//     index in cand_v[blockIdx.x] / cand_i[blockIdx.x] (a1 / a2 of the kernel; lowest row among equal sums, NaN never a
//     candidate, (-inf, INT_MAX) if the workgroup has none): the first stage of an argmax over y, so that a greedy
//     decoder's pass over its 256000 logits needs no read of them.
template <int MT, int HP, int S, int RBW, int D, int KC, int XM = 0, int YM = 0, int D0 = D>
// Argument order: the first 14 dwords of a kernel's arguments arrive in registers with the wave, the rest has to be
// fetched (and waited for) by its first instructions.  Everything a wave needs for its first requests is therefore put
// first - a0 = x (modes 0, 1) or pre.res (mode 2), a1 = pre.delta, a2 = pre.w, pvn = pv | pre.n << 8 - and what is
// needed late (y, pre.res_out, pre.eps) last.
__global__ __launch_bounds__(256 * RBW) __attribute__((amdgpu_waves_per_eu(4))) void gemv_i4g32_mfma_kernel(
    const uint8_t *__restrict__ wp, const uint16_t *__restrict__ sc, const void *__restrict__ a0, const float *__restrict__ a1,
    const float *__restrict__ a2, int N, int K, int pvn, int kspan, float *__restrict__ y, float *__restrict__ res_out, float eps) {
    const uint16_t *__restrict__ x = reinterpret_cast<const uint16_t *>(a0);
    const int pv = pvn & 0xFF;
    const GemvPre pre{reinterpret_cast<const float *>(a0), a1, a2, res_out, pvn >> 8, eps};
    constexpr bool XG = (XM == 1), XN = (XM == 2);
    typedef GemvCfg<MT, HP, S, RBW, KC> C;
    constexpr int M = MT, MP = C::MP, MPASS = C::MPASS, P = C::P, KS = C::KS, T = C::T, XI = C::XI;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int unit = wave >> 2, wv = wave & 3;     // group of 4 waves (UR rows) inside the workgroup, wave inside it
    const int rbs = wv / KS, ks = wv % KS;         // row block inside the unit, K-slice
    const int nl = lane & 15, j = lane >> 4;
    const int h = nl / P, r = nl % P;              // K-part and row of this lane's MFMA column
    // A tile uses its first pv <= P rows (the host picks pv so that the workgroups fill whole rounds of the chip);
    // the lanes of the other rows repeat the tile's first row and their sums are dropped.
    const int n0 = ((blockIdx.x * RBW + unit) * (4 / KS) + rbs) * pv;
    const int KH = K >> 1, G = K >> 5;
    const int row = (r < pv && n0 + r < N) ? n0 + r : (n0 < N ? n0 : N - 1);
    const uint32_t wrow = (uint32_t)row * (uint32_t)KH;  // byte offset; the host checks N*K/2 < 2^31

    // scale tile of this wave: P rows x 32*HP groups; lane -> (row, 8-group piece) for the single load
    int srow_l[C::SC_NL], spiece[C::SC_NL], srow[C::SC_NL];  // piece lane + 64*l; pieces beyond P rows repeat a valid row
#pragma unroll
    for (int l = 0; l < C::SC_NL; ++l) {
        srow_l[l] = (lane + 64 * l) / C::SC_PPR;
        spiece[l] = (lane + 64 * l) % C::SC_PPR;
        srow[l] = (srow_l[l] < pv && n0 + srow_l[l] < N) ? n0 + srow_l[l] : (n0 < N ? n0 : N - 1);
    }

    // blockIdx.y selects a K range of kspan (a multiple of KC, or all of K) whose partial sums go to their own
    // [M,N] block of y: the split-K form for matrices with too few rows to fill the chip
    const int kbeg = blockIdx.y * kspan, kend = (kbeg + kspan < K) ? kbeg + kspan : K;
    y += (size_t)blockIdx.y * M * N;

    // ---- the requests of a chunk.  Every wave issues, in this order, its activation loads, ONE load for its tile of
    // scales and its first D weight loads, all before the first wait (memory returns in order, so what is needed first
    // is asked for first).  For the first chunk this is the first thing the kernel does: only the addresses above stand
    // between the wave's start and its requests, and everything else the kernel sets up (operand addresses, the zero
    // block, constants) is computed while they are on their way - the wave's first weights are asked for some 0.7 us
    // earlier than when that set-up came first (about 250 vector instructions on SIMDs shared by two waves).
    u32x4 xr[MP][XI];
    f32x4 gr[XG ? XI : 1][4];  // XG: 8 gate and 8 up values per piece
    f32x4 nr[XN ? 12 : 1];     // XN: residual (2), norm weight (2), up to four delta vectors (8)
    static_assert(!XN || (M == 1 && MP == 1 && KC / 8 <= T), "the norm-folding mode stages one piece per thread");
    const bool stager = !XN || tid < KC / 8;  // XN in a workgroup of more than KC/8 threads: the first KC/8 stage
    u32x4 sv[C::SC_NL];
    u32x4 w[S];
    int kc0 = kbeg;
    auto issue_w = [&](int i) {  // steps c = S*ks + i of the chunk at kc0; the lane takes group (c*HP + h)*4 + j
        const int g = (kc0 >> 5) + ((S * ks + i) * HP + h) * 4 + j;
        w[i] = load_nt_b128(wp + (wrow + (uint32_t)(g < G ? g : 0) * 16u));
    };
    auto request = [&]() {
        // 1. activation loads FIRST.  Piece `it` = tid + T*q of pass p: row m = it / 512, i8 = it % 512.
#pragma unroll
        for (int p = 0; p < MP; ++p)
#pragma unroll
            for (int q = 0; q < XI; ++q) {
                const int m = (T * q) / (KC / 8);  // same for the whole workgroup: T divides KC/8
                if (m >= MPASS || p * MPASS + m >= M) continue;  // compile time after unrolling
                const int k = kc0 + 8 * ((tid + T * q) % (KC / 8));
                if constexpr (XN) {
                    if (!stager) continue;  // whole waves
                    const int kk = k < K ? k : 0;
                    nr[0] = *reinterpret_cast<const f32x4 *>(pre.res + kk);
                    nr[1] = *reinterpret_cast<const f32x4 *>(pre.res + kk + 4);
                    nr[2] = *reinterpret_cast<const f32x4 *>(pre.w + kk);
                    nr[3] = *reinterpret_cast<const f32x4 *>(pre.w + kk + 4);
#pragma unroll
                    for (int jd = 0; jd < 4; ++jd) {  // pre.n is uniform: absent vectors cost no load
                        if (jd < pre.n) {
                            const float *dp = pre.delta + (size_t)jd * K + kk;
                            nr[4 + 2 * jd] = *reinterpret_cast<const f32x4 *>(dp);
                            nr[5 + 2 * jd] = *reinterpret_cast<const f32x4 *>(dp + 4);
                        } else {
                            nr[4 + 2 * jd] = f32x4{0.f, 0.f, 0.f, 0.f};
                            nr[5 + 2 * jd] = f32x4{0.f, 0.f, 0.f, 0.f};
                        }
                    }
                } else if constexpr (XG) {
                    const float *gp = reinterpret_cast<const float *>(x) + (k < K ? k : 0);
                    gr[q][0] = *reinterpret_cast<const f32x4 *>(gp);
                    gr[q][1] = *reinterpret_cast<const f32x4 *>(gp + 4);
                    gr[q][2] = *reinterpret_cast<const f32x4 *>(gp + K);
                    gr[q][3] = *reinterpret_cast<const f32x4 *>(gp + K + 4);
                } else {
                    xr[p][q] = *reinterpret_cast<const u32x4 *>(x + (k < K ? (size_t)(p * MPASS + m) * K + k : 0));
                }
            }
        // 2. the wave's scale tile in one load.  Needs G % 8 == 0 (16-byte aligned pieces), checked on the host.
#pragma unroll
        for (int l = 0; l < C::SC_NL; ++l) {
            const int gs = (kc0 >> 5) + ks * S * 4 * HP + spiece[l] * 8;
            sv[l] = *reinterpret_cast<const u32x4 *>(sc + ((size_t)srow[l] * G + (gs < G ? gs : 0)));
            if (gs >= G) sv[l] = u32x4{0, 0, 0, 0};
        }
        // 3. the wave's weight loads for the chunk.  Only the first D are issued now; step i issues load i+D once its
        //    own data has arrived, so a wave's requests are spread over the stream and its last data meets one step of
        //    work, not S.  (D0 < D: only D0 of them now, the others behind the staging barrier.  In the 16-wave
        //    workgroups of the norm-folding mode four waves fetch what the activation vector is formed from and twelve
        //    wait for them: every weight load those twelve put in front of the compute unit's queue delays all sixteen.)
#pragma unroll
        for (int i = 0; i < (D0 < S ? D0 : S); ++i) issue_w(i);
        __builtin_amdgcn_sched_barrier(0);  // every load above is issued before anything below may wait
    };
    request();

    const uint32_t mask_r = vgpr_const(0x000F000Fu), magic_r = vgpr_const(kBf16Magic);

    // the zero block that A lanes off the diagonal (and padding activation rows) read from
    for (int o = tid * 16; o < ZERO_BYTES; o += T * 16)
        *reinterpret_cast<u32x4 *>(lds + C::ZERO_OFF + o) = u32x4{0, 0, 0, 0};

    // A-operand address of this lane per pass: real data only on the diagonal (row 4j'+v meets k-slot
    // group j = j') and where activation row p*MPASS + v%MPASS exists; all other lanes read zeros (stride
    // 0 keeps them inside the zero block)
    uint32_t a_base[MP], a_step[MP];
#pragma unroll
    for (int p = 0; p < MP; ++p) {
        const int v = lane & 3;
        const bool act = (((lane & 15) >> 2) == j) && (p * MPASS + (v % MPASS) < M);
        a_base[p] = act ? (uint32_t)(p * C::PASS + ks * S * 1024 + 64 * j + 16 * v) : (uint32_t)C::ZERO_OFF;
        a_step[p] = act ? 1024u : 0u;
    }

    f32x4 acc[MP];
#pragma unroll
    for (int p = 0; p < MP; ++p) acc[p] = f32x4{0.f, 0.f, 0.f, 0.f};

    uint8_t *sct = lds + C::SC_OFF + wave * C::SC_WAVE;  // the wave's scale tile in LDS

    for (;;) {  // one pass per chunk of KC; the norm-folding mode has a single chunk by contract
        // 4. stage the activations: 16-byte pieces (8 k) -> [c][t][j][v], paired for the unpack order, and
        //    the C operands -136 * (sum of the group's 32 activations)
        float nv[8];
        __shared__ float s_ss[4 * RBW];
        if constexpr (XN) {
            const int k = kc0 + 8 * (tid % (KC / 8));
            float ss = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                float v = nr[e >> 2][e & 3];
#pragma unroll
                for (int jd = 0; jd < 4; ++jd)
                    if (jd < pre.n) v += nr[4 + 2 * jd + (e >> 2)][e & 3];
                nv[e] = (k < K && stager) ? v : 0.f;
                ss += nv[e] * nv[e];
            }
            if (blockIdx.x == 0 && blockIdx.y == 0 && k < K && stager) {
                *reinterpret_cast<f32x4 *>(pre.res_out + k) = f32x4{nv[0], nv[1], nv[2], nv[3]};
                *reinterpret_cast<f32x4 *>(pre.res_out + k + 4) = f32x4{nv[4], nv[5], nv[6], nv[7]};
            }
            ss = wave_sum_to_lane63(ss);
            if (lane == 63) s_ss[wave] = ss;
        }
        // the previous chunk's operand reads are done (first chunk: nothing written below is read before the next
        // barrier, the zero block included; the norm-folding mode needs the barrier for its sums of squares)
        if (XN || kc0 != kbeg) __syncthreads();
#pragma unroll
        for (int l = 0; l < C::SC_NL; ++l)  // wave-private tile
            if (srow_l[l] < P) *reinterpret_cast<u32x4 *>(sct + srow_l[l] * C::SC_PITCH + spiece[l] * 16) = sv[l];
#pragma unroll
        for (int p = 0; p < MP; ++p)
#pragma unroll
            for (int q = 0; q < XI; ++q) {
                const int m = (T * q) / (KC / 8);
                if (m >= MPASS || p * MPASS + m >= M) continue;  // padding row: its A lanes read the zero block
                if (XN && !stager) continue;                     // whole waves
                const int i8 = (tid + T * q) % (KC / 8);
                u32x4 v;
                if constexpr (XN) {
                    float tot = 0.f;
#pragma unroll
                    for (int wv2 = 0; wv2 < 4 * RBW; ++wv2) tot += s_ss[wv2];
                    const float rinv = rsqrtf(tot / (float)K + pre.eps);
                    uint32_t hb[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) hb[e] = f32_to_bf16_bits(nv[e] * rinv * nr[2 + (e >> 2)][e & 3]);
                    v = u32x4{hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16), hb[4] | (hb[5] << 16), hb[6] | (hb[7] << 16)};
                } else if constexpr (XG) {
                    const float g8[8] = {gr[q][0].x, gr[q][0].y, gr[q][0].z, gr[q][0].w, gr[q][1].x, gr[q][1].y, gr[q][1].z, gr[q][1].w};
                    const float u8[8] = {gr[q][2].x, gr[q][2].y, gr[q][2].z, gr[q][2].w, gr[q][3].x, gr[q][3].y, gr[q][3].z, gr[q][3].w};
                    uint32_t hb[8];
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        hb[e] = f32_to_bf16_bits(gelu_tanh_dev(g8[e]) * u8[e]);
                    }
                    v = u32x4{hb[0] | (hb[1] << 16), hb[2] | (hb[3] << 16), hb[4] | (hb[5] << 16), hb[6] | (hb[7] << 16)};
                } else {
                    v = xr[p][q];
                }
                if (kc0 + 8 * i8 >= K) v = u32x4{0, 0, 0, 0};
                uint32_t a[4] = {v.x, v.y, v.z, v.w}, o[4];
                float sum = 0.f;
#pragma unroll
                for (int e = 0; e < 4; ++e) sum = dot2_bf16(a[e], 0x3F803F80u, sum);
                pair_x8(a, o);
                // chunk-local group gl = (c*HP + h')*4 + j'
                const int gl = i8 >> 2, t = i8 & 3;
                const int c = gl / (4 * HP), hh = (gl >> 2) % HP, jj = gl & 3;
                const int vv = hh * MPASS + m;
                *reinterpret_cast<u32x4 *>(lds + p * C::PASS + c * 1024 + t * 256 + jj * 64 + vv * 16) =
                    u32x4{o[0], o[1], o[2], o[3]};
                sum += dpp_f32<0xB1, 0xF>(sum);  // the 4 pieces of a group sit in 4 adjacent lanes
                sum += dpp_f32<0x4E, 0xF>(sum);
                if (t == 0)
                    *reinterpret_cast<float *>(lds + p * C::PASS + C::XA_BYTES + (c * 4 + jj) * 16 + vv * 4) = -kMagicBias * sum;
            }
        __syncthreads();
        if (D0 < D) {
#pragma unroll
            for (int i = D0; i < (D < S ? D : S); ++i) issue_w(i);
        }

        // 5. the chunk's 8 steps of this wave
        uint32_t a_addr[MP];
#pragma unroll
        for (int p = 0; p < MP; ++p) a_addr[p] = a_base[p];
#pragma unroll
        for (int i = 0; i < S; ++i) {
            const int c = S * ks + i;
            uint32_t pw[16];
            if (D < S) {
                // wait for this step's weights, then put the next request in the queue before computing
                asm volatile("" : "+v"(w[i]));
                if (i + D < S) issue_w(i + D);
                __builtin_amdgcn_sched_barrier(0);
            }
            unpack8_magic_r(w[i].x, mask_r, magic_r, &pw[0]);
            unpack8_magic_r(w[i].y, mask_r, magic_r, &pw[4]);
            unpack8_magic_r(w[i].z, mask_r, magic_r, &pw[8]);
            unpack8_magic_r(w[i].w, mask_r, magic_r, &pw[12]);
            const float s = f16_bits_to_f32(
                *reinterpret_cast<const uint16_t *>(sct + r * C::SC_PITCH + ((i * HP + h) * 4 + j) * 2));
#pragma unroll
            for (int p = 0; p < MP; ++p) {
                f32x4 d = *reinterpret_cast<const f32x4 *>(lds + p * C::PASS + C::XA_BYTES + (4 * c + j) * 16);
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
        kc0 += KC;
        if (XN || kc0 >= kend) break;
        request();
    }

    // 6a. One activation row and one wave per row block (KS = 1): everything a row's sum consists of sits in this wave -
    //     lane (h*P + r, j) holds the part of K-part h and lane group j in register h*MPASS - so the wave folds it with
    //     rotations inside the 16-lane rows and two lane-group exchanges and stores its P sums itself.  No LDS, no
    //     workgroup barrier: a wave's last load is followed by a dozen instructions, not by the slowest wave of the
    //     workgroup (7.46 -> 7.36 us at 14336 x 4096, 634 -> 626 us on the 112 launches of a decode step).
    if constexpr (M == 1 && KS == 1 && HP >= 2) {
        float t = acc[0][0];
#pragma unroll
        for (int hh = 1; hh < HP; ++hh) t = (h == hh) ? acc[0][hh * MPASS] : t;
        if (P == 4) t += dpp_f32<0x124, 0xF>(t);  // row_ror:4
        t += dpp_f32<0x128, 0xF>(t);              // row_ror:8: every lane of a row holds the row's sum for its r = lane % P
        const u32x2 a16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(t), __float_as_uint(t), false, false);
        t = __uint_as_float(a16.x) + __uint_as_float(a16.y);  // rows 0+1 and 2+3
        const u32x2 a32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(t), __float_as_uint(t), false, false);
        t = __uint_as_float(a32.x) + __uint_as_float(a32.y);  // all four lane groups
        const int nn = n0 + lane;
        if constexpr (YM == 1) {
            const float up = dpp_f32<0xB1, 0xF>(t);  // quad_perm [1,0,3,2]: the up row of the pair sits in the next lane
            if (lane < P && !(lane & 1) && lane + 1 < pv && nn + 1 < N)
                reinterpret_cast<uint16_t *>(y)[nn >> 1] = (uint16_t)f32_to_bf16_bits(gelu_tanh_dev(t) * up);
        } else if constexpr (YM == 2) {
            const bool valid = lane < P && lane < pv && nn < N;
            if (valid) y[nn] = t;
            // the wave's candidate, then the workgroup's: the one place where this path meets the other waves
            __shared__ float s_cv[4 * RBW];
            __shared__ int32_t s_ci[4 * RBW];
            const uint32_t gi = wave_winner<64>(valid && t == t, t, nn);
            if (gi == 0xFFFFFFFFu) {
                if (lane == 0) {
                    s_cv[wave] = -INFINITY;
                    s_ci[wave] = INT_MAX;
                }
            } else if (valid && (uint32_t)nn == gi) {  // one lane: rows are distinct
                s_cv[wave] = t;
                s_ci[wave] = nn;
            }
            __syncthreads();
            if (tid == 0) {
                float bv = s_cv[0];
                int32_t bb = s_ci[0];
#pragma unroll
                for (int w2 = 1; w2 < 4 * RBW; ++w2)
                    if (s_ci[w2] != INT_MAX && (bb == INT_MAX || s_cv[w2] > bv || (s_cv[w2] == bv && s_ci[w2] < bb))) {
                        bv = s_cv[w2];
                        bb = s_ci[w2];
                    }
                const_cast<float *>(a1)[blockIdx.x] = bv;
                reinterpret_cast<int32_t *>(const_cast<float *>(a2))[blockIdx.x] = bb;
            }
        } else {
            if (lane < P && lane < pv && nn < N) y[nn] = t;
        }
        return;
    }
    static_assert(YM != 2 || (M == 1 && KS == 1 && HP >= 2), "argmax candidates: only the form whose waves fold their own sums writes them");
    // 6b. fold lane groups, K-parts and K-slices through LDS: RED[wave][lane][pass] = 4 floats
    __syncthreads();  // every wave is done with the operand area, which the partial sums now reuse
    u32x4 *red = reinterpret_cast<u32x4 *>(lds);
#pragma unroll
    for (int p = 0; p < MP; ++p) {
        u32x4 v;
        __builtin_memcpy(&v, &acc[p], 16);
        red[(wave * 64 + lane) * MP + p] = v;
    }
    __syncthreads();
    constexpr int UR = C::UR, OUT_PER_UNIT = UR * MPASS * MP;  // weight rows x activation rows (padded to MPASS*MP)
    if (tid < RBW * OUT_PER_UNIT) {
        // tid -> (unit, pass, activation row m, weight row n16 of the unit); n16 fastest: contiguous stores
        const int n16 = tid % UR, m = (tid / UR) % MPASS, p = (tid / (UR * MPASS)) % MP, un = tid / OUT_PER_UNIT;
        const int rb = n16 / P, rr = n16 % P;
        float t = 0.f;
#pragma unroll
        for (int k4 = 0; k4 < KS; ++k4)
#pragma unroll
            for (int hh = 0; hh < HP; ++hh)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int wsrc = un * 4 + rb * KS + k4, lsrc = 16 * q + hh * P + rr;
                    t += reinterpret_cast<const float *>(red)[((wsrc * 64 + lsrc) * MP + p) * 4 + hh * MPASS + m];
                }
        const int nn = ((blockIdx.x * RBW + un) * (4 / KS) + rb) * pv + rr, mm = p * MPASS + m;
        if constexpr (YM == 1) {
            static_assert(YM == 0 || (M == 1 && (C::P % 2) == 0), "gate/up pairs: one activation row, even tiles");
            // n16 runs fastest over the threads and tiles start at even rows: the up row of a pair sits in the next lane
            const float up = dpp_f32<0xB1, 0xF>(t);  // quad_perm [1,0,3,2]
            if (!(rr & 1) && rr + 1 < pv && nn + 1 < N && mm < M)  // mm: the padding rows of a two-row pass write nothing
                reinterpret_cast<uint16_t *>(y)[nn >> 1] = (uint16_t)f32_to_bf16_bits(gelu_tanh_dev(t) * up);
        } else {
            if (rr < pv && nn < N && mm < M) y[(size_t)mm * N + nn] = t;
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Eight rows of A per scale group: 5 to 8 activation rows in one pass over the unpacked weights.
//
// The kernel above gives every lane group j of an MFMA column its own scale group, which leaves four rows of A per
// group.  Here the two lane-group pairs (0,1) and (2,3) each work on one scale group, eight rows of A per group:
//   load     as above with one K-part: lane (r, j) fetches the 16 bytes of group 4c + j of weight row r.
//   exchange v_permlane16_swap on words (0,1) and on words (2,3): lane groups 0 and 1 then hold group 4c (pair 0) and
//            group 4c+1 (pair 1), lane groups 2 and 3 hold 4c+2 and 4c+3 - word `half` of each, lane group j & 1
//            supplying k 16*half + 8*(j&1) .. +7 of the group.  Two instructions per 16-byte load.
//   A        row i = 8*g + m (g = which of the pair's two groups, m = activation row); real data where the lane's
//            k-slot group j has j >> 1 == g, zeros elsewhere.
//   D        lane (r, j) holds activation rows 4*(j&1) .. +3 of weight row r against group 4c + p + 2*(j>>1): one
//            scale per lane and pair, four FMAs.
// Per 16-byte load: 4 MFMAs and 8 scale FMAs for up to eight rows (the form above would need 8 and 8): 9.4-9.6 us
// against 10.4-10.7 at 14336 x 4096 and 8 rows.  (The same regrouping with two K-parts of four rows each - loads of
// 8 weight rows x 128 contiguous bytes for 3 and 4 activation rows - was built, is correct, and measured slower than
// the form above there: 8.6 against 8.2 us.)
template <int S, int RBW, int KC>
struct GemvPairCfg {
    static constexpr int P = 16;
    static constexpr int MR = 8;
    static constexpr int STEPS = KC / 128;
    static constexpr int KS = STEPS / S;
    static constexpr int UR = P * 4 / KS;
    static_assert(KS >= 1 && KS <= 4 && KS * S == STEPS, "a chunk of one row block is split over 1, 2 or 4 waves");
    static constexpr int XA_BYTES = STEPS * 2048;  // A operands: [c][pair][half][g][j&1][v] x 16 B
    static constexpr int NX_BYTES = STEPS * 128;   // C operands: [c][pair][j][v%4] fp32
    static constexpr int ZERO_OFF = XA_BYTES + NX_BYTES;
    static constexpr int ZERO_SPAN = 2048;  // lanes off the diagonal add the same per-MFMA offsets (up to 1536) as the others
    static constexpr int SC_OFF = ZERO_OFF + ZERO_SPAN;
    static constexpr int SC_PPR = S / 2;
    static constexpr int SC_PITCH = SC_PPR * 16 + 16;
    static constexpr int SC_NL = (P * SC_PPR + 63) / 64;
    static constexpr int SC_WAVE = P * SC_PITCH;
    static constexpr int OPER_BYTES = SC_OFF + RBW * 4 * SC_WAVE;
    static constexpr int RED_BYTES = RBW * 4 * 64 * 16;
    static constexpr int TOTAL = OPER_BYTES > RED_BYTES ? OPER_BYTES : RED_BYTES;
    static constexpr int T = 256 * RBW;
    static constexpr int XI = (MR * (KC / 8) + T - 1) / T;  // 16-byte activation pieces per thread and chunk
    static_assert((MR * (KC / 8)) % T == 0, "whole rounds of pieces");
};

template <int MT, int S, int RBW, int D, int KC>
__global__ __launch_bounds__(256 * RBW) __attribute__((amdgpu_waves_per_eu(S == 16 ? 2 : 4))) void gemv_i4g32_mfma_pair_kernel(
    const uint16_t *__restrict__ x, const uint8_t *__restrict__ wp, const uint16_t *__restrict__ sc,
    float *__restrict__ y, int N, int K, int pv) {
    typedef GemvPairCfg<S, RBW, KC> C;
    constexpr int M = MT, P = C::P, MR = C::MR, KS = C::KS, T = C::T, XI = C::XI;
    static_assert(M >= 1 && M <= MR, "eight rows of A per scale group");
    // S = 16: one 8-wave workgroup per compute unit (its LDS), so a wave may use 256 registers
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int unit = wave >> 2, wv = wave & 3;
    const int rbs = wv / KS, ks = wv % KS;
    const int nl = lane & 15, j = lane >> 4, r = nl;
    const int n0 = ((blockIdx.x * RBW + unit) * (4 / KS) + rbs) * pv;
    const int KH = K >> 1, G = K >> 5;
    const int row = (r < pv && n0 + r < N) ? n0 + r : (n0 < N ? n0 : N - 1);
    const uint32_t wrow = (uint32_t)row * (uint32_t)KH;

    int srow_l[C::SC_NL], spiece[C::SC_NL], srow[C::SC_NL];
#pragma unroll
    for (int l = 0; l < C::SC_NL; ++l) {
        srow_l[l] = (lane + 64 * l) / C::SC_PPR;
        spiece[l] = (lane + 64 * l) % C::SC_PPR;
        srow[l] = (srow_l[l] < pv && n0 + srow_l[l] < N) ? n0 + srow_l[l] : (n0 < N ? n0 : N - 1);
    }

    // Piece it = tid + T*q of a chunk: word t = it % 4 of its scale group (the four pieces of a group in one quad of
    // lanes), activation row m = it / 4 % 8, then pair, g and step from the bits above.  A wave's store to LDS is four
    // runs of 256 contiguous bytes (conflict free), its load 8 rows x 128 contiguous bytes.
    auto piece = [&](int it, int &t, int &m, int &c, int &pr, int &g) {
        t = it & 3;
        m = (it >> 2) & 7;
        const int rest = it >> 5;
        pr = rest & 1;
        g = (rest >> 1) & 1;
        c = rest >> 2;
    };

    // the requests of a chunk, as in the kernel above: asked for before anything else is set up
    u32x4 xr[XI];
    u32x4 sv[C::SC_NL];
    u32x4 w[S];
    int kc0 = 0;
    auto issue_w = [&](int i) {
        const int gg = (kc0 >> 5) + (S * ks + i) * 4 + j;
        w[i] = load_nt_b128(wp + (wrow + (uint32_t)(gg < G ? gg : 0) * 16u));
    };
    auto request = [&]() {
        // 1. activation loads first
#pragma unroll
        for (int q = 0; q < XI; ++q) {
            int t, m, c, pr, g;
            piece(tid + T * q, t, m, c, pr, g);
            const int k = kc0 + 32 * (c * 4 + g * 2 + pr) + 8 * t;
            xr[q] = u32x4{0, 0, 0, 0};
            if (m < M && k < K) xr[q] = *reinterpret_cast<const u32x4 *>(x + (size_t)m * K + k);
        }
        // 2. the wave's scale tile
#pragma unroll
        for (int l = 0; l < C::SC_NL; ++l) {
            const int gs = (kc0 >> 5) + ks * S * 4 + spiece[l] * 8;
            sv[l] = *reinterpret_cast<const u32x4 *>(sc + ((size_t)srow[l] * G + (gs < G ? gs : 0)));
            if (gs >= G) sv[l] = u32x4{0, 0, 0, 0};
        }
        // 3. the first D weight loads
#pragma unroll
        for (int i = 0; i < (D < S ? D : S); ++i) issue_w(i);
        __builtin_amdgcn_sched_barrier(0);
    };
    request();

    const uint32_t mask_r = vgpr_const(0x000F000Fu), magic_r = vgpr_const(kBf16Magic);

    for (int o = tid * 16; o < C::ZERO_SPAN; o += T * 16) *reinterpret_cast<u32x4 *>(lds + C::ZERO_OFF + o) = u32x4{0, 0, 0, 0};

    // A operand: lane (i = lane & 15, j) is row 8g + m with g = i >> 3, m = i & 7
    const bool a_live = ((nl >> 3) == (j >> 1)) && ((nl & 7) < M);
    const uint32_t a_base = a_live ? (uint32_t)(ks * S * 2048 + (j >> 1) * 256 + (j & 1) * 128 + (nl & 7) * 16) : (uint32_t)C::ZERO_OFF;
    const uint32_t a_step = a_live ? 2048u : 0u;

    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};

    uint8_t *sct = lds + C::SC_OFF + wave * C::SC_WAVE;

    for (;;) {
        // 4. stage the activations
        __syncthreads();  // the previous chunk's operand reads (or the zero fill) are done
#pragma unroll
        for (int l = 0; l < C::SC_NL; ++l)
            if (srow_l[l] < P) *reinterpret_cast<u32x4 *>(sct + srow_l[l] * C::SC_PITCH + spiece[l] * 16) = sv[l];
#pragma unroll
        for (int q = 0; q < XI; ++q) {
            int t, m, c, pr, g;
            piece(tid + T * q, t, m, c, pr, g);
            uint32_t a[4] = {xr[q].x, xr[q].y, xr[q].z, xr[q].w}, o[4];
            float sum = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) sum = dot2_bf16(a[e], 0x3F803F80u, sum);
            pair_x8(a, o);
            if (m < M)
                *reinterpret_cast<u32x4 *>(lds + c * 2048 + (pr * 2 + (t >> 1)) * 512 + g * 256 + (t & 1) * 128 + m * 16) =
                    u32x4{o[0], o[1], o[2], o[3]};
            sum += dpp_f32<0xB1, 0xF>(sum);  // the four pieces of a group sit in four adjacent lanes
            sum += dpp_f32<0x4E, 0xF>(sum);
            if (t == 0 && m < M)
                *reinterpret_cast<float *>(lds + C::XA_BYTES + ((c * 2 + pr) * 4 + g * 2 + (m >> 2)) * 16 + (m & 3) * 4) =
                    -kMagicBias * sum;
        }
        __syncthreads();

        // 5. the chunk's S steps of this wave
        uint32_t a_addr = a_base;
#pragma unroll
        for (int i = 0; i < S; ++i) {
            const int c = S * ks + i;
            if (D < S) {
                asm volatile("" : "+v"(w[i]));
                if (i + D < S) issue_w(i + D);
                __builtin_amdgcn_sched_barrier(0);
            }
            const u32x2 lo = __builtin_amdgcn_permlane16_swap(w[i].x, w[i].y, false, false);
            const u32x2 hi = __builtin_amdgcn_permlane16_swap(w[i].z, w[i].w, false, false);
            uint32_t pw[16];  // [pair][half][4]
            unpack8_magic_r(lo.x, mask_r, magic_r, &pw[0]);
            unpack8_magic_r(hi.x, mask_r, magic_r, &pw[4]);
            unpack8_magic_r(lo.y, mask_r, magic_r, &pw[8]);
            unpack8_magic_r(hi.y, mask_r, magic_r, &pw[12]);
#pragma unroll
            for (int pr = 0; pr < 2; ++pr) {
                const float s = f16_bits_to_f32(
                    *reinterpret_cast<const uint16_t *>(sct + r * C::SC_PITCH + (i * 4 + pr + 2 * (j >> 1)) * 2));
                f32x4 d = *reinterpret_cast<const f32x4 *>(lds + C::XA_BYTES + ((2 * c + pr) * 4 + j) * 16);
#pragma unroll
                for (int hf = 0; hf < 2; ++hf) {
                    const bf16x8 av = *reinterpret_cast<const bf16x8 *>(lds + a_addr + (pr * 2 + hf) * 512);
                    const u32x4 bw = {pw[(pr * 2 + hf) * 4], pw[(pr * 2 + hf) * 4 + 1], pw[(pr * 2 + hf) * 4 + 2], pw[(pr * 2 + hf) * 4 + 3]};
                    bf16x8 bv;
                    __builtin_memcpy(&bv, &bw, 16);
                    d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bv, d, 0, 0, 0);
                }
                acc += d * s;
            }
            a_addr += a_step;
        }
        kc0 += KC;
        if (kc0 >= K) break;
        request();
    }

    // 6. fold the two scale-group halves and the K-slices
    __syncthreads();
    u32x4 *red = reinterpret_cast<u32x4 *>(lds);
    {
        u32x4 v;
        __builtin_memcpy(&v, &acc, 16);
        red[wave * 64 + lane] = v;
    }
    __syncthreads();
    constexpr int UR = C::UR, OUT_PER_UNIT = UR * MR;
    for (int o = tid; o < RBW * OUT_PER_UNIT; o += T) {
        const int n16 = o % UR, m = (o / UR) % MR, un = o / OUT_PER_UNIT;
        const int rb = n16 / P, rr = n16 % P;
        float t = 0.f;
#pragma unroll
        for (int k4 = 0; k4 < KS; ++k4)
#pragma unroll
            for (int g = 0; g < 2; ++g) {
                const int wsrc = un * 4 + rb * KS + k4, lsrc = 16 * (2 * g + (m >> 2)) + rr;
                t += reinterpret_cast<const float *>(red)[(wsrc * 64 + lsrc) * 4 + (m & 3)];
            }
        const int nn = ((blockIdx.x * RBW + un) * (4 / KS) + rb) * pv + rr;
        if (rr < pv && nn < N && m < M) y[(size_t)m * N + nn] = t;
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Sixteen rows of A per scale group: 9 to 16 activation rows in one pass over the weights.
//
// After v_permlane16_swap on words (0,1) and (2,3) as above, v_permlane32_swap between the two results moves the
// halves of a group together: register t of a lane then holds word j (= the lane's group of 16 lanes) of scale
// group 4c + t, so MFMA t works on ONE scale group with all four k-slot groups and all 16 rows of A are activation
// rows.  Per 16-byte load: 4 exchanges, 4 MFMAs, 16 scale FMAs.  M is a run-time argument (rows past M read zeros).
template <int S, int RBW, int KC>
struct GemvRows16Cfg {
    static constexpr int P = 16;
    static constexpr int STEPS = KC / 128;
    static constexpr int KS = STEPS / S;
    static constexpr int UR = P * 4 / KS;
    static_assert(KS >= 1 && KS <= 4 && KS * S == STEPS, "a chunk of one row block is split over 1, 2 or 4 waves");
    static constexpr int XA_BYTES = STEPS * 4096;  // A operands: [c][t][word j][row i] x 16 B
    static constexpr int NX_BYTES = STEPS * 256;   // C operands: [c][t][j][v] fp32
    static constexpr int ZERO_OFF = XA_BYTES + NX_BYTES;
    static constexpr int ZERO_SPAN = 4096;         // rows past M add the same per-MFMA offsets (up to 3072) as the others
    static constexpr int SC_OFF = ZERO_OFF + ZERO_SPAN;
    static constexpr int SC_PPR = S / 2;
    static constexpr int SC_PITCH = SC_PPR * 16 + 16;
    static constexpr int SC_NL = (P * SC_PPR + 63) / 64;
    static constexpr int SC_WAVE = P * SC_PITCH;
    static constexpr int OPER_BYTES = SC_OFF + RBW * 4 * SC_WAVE;
    static constexpr int RED_BYTES = RBW * 4 * 64 * 16;
    static constexpr int TOTAL = OPER_BYTES > RED_BYTES ? OPER_BYTES : RED_BYTES;
    static constexpr int T = 256 * RBW;
    static constexpr int XI = (16 * (KC / 8)) / T;  // 16-byte activation pieces per thread and chunk
    static_assert((16 * (KC / 8)) % T == 0, "whole rounds of pieces");
};

template <int S, int RBW, int D, int KC>
// (two waves per SIMD at most: a workgroup's operands take 68 KB or more of LDS, so a wave may use 256 registers)
__global__ __launch_bounds__(256 * RBW) __attribute__((amdgpu_waves_per_eu(2))) void gemv_i4g32_mfma_rows16_kernel(
    const uint16_t *__restrict__ x, const uint8_t *__restrict__ wp, const uint16_t *__restrict__ sc,
    float *__restrict__ y, int M, int N, int K, int pv) {
    typedef GemvRows16Cfg<S, RBW, KC> C;
    constexpr int P = C::P, KS = C::KS, T = C::T, XI = C::XI;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int unit = wave >> 2, wv = wave & 3;
    const int rbs = wv / KS, ks = wv % KS;
    const int r = lane & 15, j = lane >> 4;
    const int n0 = ((blockIdx.x * RBW + unit) * (4 / KS) + rbs) * pv;
    const int KH = K >> 1, G = K >> 5;
    const int row = (r < pv && n0 + r < N) ? n0 + r : (n0 < N ? n0 : N - 1);
    const uint32_t wrow = (uint32_t)row * (uint32_t)KH;

    int srow_l[C::SC_NL], spiece[C::SC_NL], srow[C::SC_NL];
#pragma unroll
    for (int l = 0; l < C::SC_NL; ++l) {
        srow_l[l] = (lane + 64 * l) / C::SC_PPR;
        spiece[l] = (lane + 64 * l) % C::SC_PPR;
        srow[l] = (srow_l[l] < pv && n0 + srow_l[l] < N) ? n0 + srow_l[l] : (n0 < N ? n0 : N - 1);
    }

    // the requests of a chunk, as in the kernels above: asked for before anything else is set up
    u32x4 xr[XI];
    u32x4 sv[C::SC_NL];
    u32x4 w[S];
    int kc0 = 0;
    auto issue_w = [&](int i) {
        const int gg = (kc0 >> 5) + (S * ks + i) * 4 + j;
        w[i] = load_nt_b128(wp + (wrow + (uint32_t)(gg < G ? gg : 0) * 16u));
    };
    auto request = [&]() {
        // 1. activation loads first.  Piece it = tid + T*q: word it % 4 of its scale group, activation row
        //    it / 4 % 16, chunk-local group it / 64: a wave stores 1 KiB of contiguous LDS.
#pragma unroll
        for (int q = 0; q < XI; ++q) {
            const int it = tid + T * q, m = (it >> 2) & 15, k = kc0 + 32 * (it >> 6) + 8 * (it & 3);
            xr[q] = u32x4{0, 0, 0, 0};
            if (m < M && k < K) xr[q] = *reinterpret_cast<const u32x4 *>(x + (size_t)m * K + k);
        }
        // 2. the wave's scale tile
#pragma unroll
        for (int l = 0; l < C::SC_NL; ++l) {
            const int gs = (kc0 >> 5) + ks * S * 4 + spiece[l] * 8;
            sv[l] = *reinterpret_cast<const u32x4 *>(sc + ((size_t)srow[l] * G + (gs < G ? gs : 0)));
            if (gs >= G) sv[l] = u32x4{0, 0, 0, 0};
        }
        // 3. the first D weight loads
#pragma unroll
        for (int i = 0; i < (D < S ? D : S); ++i) issue_w(i);
        __builtin_amdgcn_sched_barrier(0);
    };
    request();

    const uint32_t mask_r = vgpr_const(0x000F000Fu), magic_r = vgpr_const(kBf16Magic);

    for (int o = tid * 16; o < C::ZERO_SPAN; o += T * 16) *reinterpret_cast<u32x4 *>(lds + C::ZERO_OFF + o) = u32x4{0, 0, 0, 0};

    const bool a_live = r < M;  // A row i = lane & 15 is activation row i
    const uint32_t a_base = a_live ? (uint32_t)(ks * S * 4096 + j * 256 + r * 16) : (uint32_t)C::ZERO_OFF;
    const uint32_t a_step = a_live ? 4096u : 0u;

    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};

    uint8_t *sct = lds + C::SC_OFF + wave * C::SC_WAVE;

    for (;;) {
        // 4. stage the activations
        __syncthreads();  // the previous chunk's operand reads (or the zero fill) are done
#pragma unroll
        for (int l = 0; l < C::SC_NL; ++l)
            if (srow_l[l] < P) *reinterpret_cast<u32x4 *>(sct + srow_l[l] * C::SC_PITCH + spiece[l] * 16) = sv[l];
#pragma unroll
        for (int q = 0; q < XI; ++q) {
            const int it = tid + T * q, tw = it & 3, m = (it >> 2) & 15, gl = it >> 6;
            const int c = gl >> 2, t = gl & 3;
            uint32_t a[4] = {xr[q].x, xr[q].y, xr[q].z, xr[q].w}, o[4];
            float sum = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) sum = dot2_bf16(a[e], 0x3F803F80u, sum);
            pair_x8(a, o);
            if (m < M) *reinterpret_cast<u32x4 *>(lds + c * 4096 + t * 1024 + tw * 256 + m * 16) = u32x4{o[0], o[1], o[2], o[3]};
            sum += dpp_f32<0xB1, 0xF>(sum);  // the four pieces of a group sit in four adjacent lanes
            sum += dpp_f32<0x4E, 0xF>(sum);
            if (tw == 0)  // rows past M get a zero correction
                *reinterpret_cast<float *>(lds + C::XA_BYTES + ((c * 4 + t) * 4 + (m >> 2)) * 16 + (m & 3) * 4) =
                    m < M ? -kMagicBias * sum : 0.f;
        }
        __syncthreads();

        // 5. the chunk's S steps of this wave
        uint32_t a_addr = a_base;
#pragma unroll
        for (int i = 0; i < S; ++i) {
            const int c = S * ks + i;
            if (D < S) {
                asm volatile("" : "+v"(w[i]));
                if (i + D < S) issue_w(i + D);
                __builtin_amdgcn_sched_barrier(0);
            }
            const u32x2 lo = __builtin_amdgcn_permlane16_swap(w[i].x, w[i].y, false, false);
            const u32x2 hi = __builtin_amdgcn_permlane16_swap(w[i].z, w[i].w, false, false);
            const u32x2 g02 = __builtin_amdgcn_permlane32_swap(lo.x, hi.x, false, false);  // groups 4c and 4c+2
            const u32x2 g13 = __builtin_amdgcn_permlane32_swap(lo.y, hi.y, false, false);  // groups 4c+1 and 4c+3
            uint32_t pw[16];  // [t][4]
            unpack8_magic_r(g02.x, mask_r, magic_r, &pw[0]);
            unpack8_magic_r(g13.x, mask_r, magic_r, &pw[4]);
            unpack8_magic_r(g02.y, mask_r, magic_r, &pw[8]);
            unpack8_magic_r(g13.y, mask_r, magic_r, &pw[12]);
            const u32x2 s4 = *reinterpret_cast<const u32x2 *>(sct + r * C::SC_PITCH + i * 8);  // the step's four scales
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const uint32_t sw = t < 2 ? s4.x : s4.y;
                const float s = f16_bits_to_f32((uint16_t)((t & 1) ? (sw >> 16) : (sw & 0xFFFFu)));
                f32x4 d = *reinterpret_cast<const f32x4 *>(lds + C::XA_BYTES + ((4 * c + t) * 4 + j) * 16);
                const bf16x8 av = *reinterpret_cast<const bf16x8 *>(lds + a_addr + t * 1024);
                const u32x4 bw = {pw[t * 4], pw[t * 4 + 1], pw[t * 4 + 2], pw[t * 4 + 3]};
                bf16x8 bv;
                __builtin_memcpy(&bv, &bw, 16);
                d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(av, bv, d, 0, 0, 0);
                acc += d * s;
            }
            a_addr += a_step;
        }
        kc0 += KC;
        if (kc0 >= K) break;
        request();
    }

    // 6. fold the K-slices
    __syncthreads();
    u32x4 *red = reinterpret_cast<u32x4 *>(lds);
    {
        u32x4 v;
        __builtin_memcpy(&v, &acc, 16);
        red[wave * 64 + lane] = v;
    }
    __syncthreads();
    constexpr int UR = C::UR, OUT_PER_UNIT = UR * 16;
    for (int o = tid; o < RBW * OUT_PER_UNIT; o += T) {
        const int n16 = o % UR, m = (o / UR) % 16, un = o / OUT_PER_UNIT;
        const int rb = n16 / P, rr = n16 % P;
        float t = 0.f;
#pragma unroll
        for (int k4 = 0; k4 < KS; ++k4) {
            const int wsrc = un * 4 + rb * KS + k4, lsrc = 16 * (m >> 2) + rr;
            t += reinterpret_cast<const float *>(red)[(wsrc * 64 + lsrc) * 4 + (m & 3)];
        }
        const int nn = ((blockIdx.x * RBW + un) * (4 / KS) + rb) * pv + rr;
        if (rr < pv && nn < N && m < M) y[(size_t)m * N + nn] = t;
    }
}

int gemv_i4g32_dispatch(const uint16_t *, const uint8_t *, const uint16_t *, float *, int, int, int, hipStream_t);

// Rows of a P-row tile to use.  All workgroups of these grids are resident at once, so the launch lasts as long as
// the compute unit with the most workgroups: ceil(workgroups / CUs) of them.  Using a few rows less per tile can turn
// 1.75 workgroups per CU (two on most, one on the rest) into exactly 2 shorter ones.  The fill is
// N / (rounds * CUs * rows per workgroup); fewer rows are taken only for a gain of more than 5 %.
static int pick_tile_rows(int N, int P, int tiles_per_wg, int ksplit) {
    static std::atomic<int> n_cu{0};
    int cus = n_cu.load(std::memory_order_relaxed);
    if (cus == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return P;
        cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
        n_cu.store(cus, std::memory_order_relaxed);
    }
    int best = P;
    double fill_p = 0.0, best_fill = 0.0;
    for (int pv = P; pv >= P - P / 4; --pv) {
        const int64_t tiles = (N + pv - 1) / pv;
        const int64_t wgs = (tiles + tiles_per_wg - 1) / tiles_per_wg * ksplit;
        const int64_t rounds = (wgs + cus - 1) / cus;
        const double fill = (double)N * ksplit / ((double)rounds * cus * pv * tiles_per_wg);
        if (pv == P) fill_p = best_fill = fill;
        if (fill > best_fill && fill > 1.05 * fill_p) {
            best = pv;
            best_fill = fill;
        }
    }
    return best;
}

template <int MT, int HP, int S, int RBW, int D, int KC = 4096, int XM = 0, int YM = 0, int D0 = D>
static int launch_mfma(const uint16_t *x, const uint8_t *wp, const uint16_t *sc, float *y, int N, int K,
                       hipStream_t st, int ksplit = 1, GemvPre pre = GemvPre{}, int *workgroups = nullptr) {
    typedef GemvCfg<MT, HP, S, RBW, KC> C;
    static std::atomic<bool> attr_set{false};  // setting it twice from two threads is harmless
    if (!attr_set.load(std::memory_order_acquire)) {
        CHADQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_i4g32_mfma_kernel<MT, HP, S, RBW, D, KC, XM, YM, D0>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, C::TOTAL));
        attr_set.store(true, std::memory_order_release);
    }
    const int tiles_per_wg = 4 / C::KS * RBW;
    int pv = pick_tile_rows(N, C::P, tiles_per_wg, ksplit);
    if (YM == 1 && (pv & 1)) pv = C::P;  // pairs of rows must not straddle tiles
    const int tiles = (N + pv - 1) / pv;
    const void *a0 = (XM == 2) ? static_cast<const void *>(pre.res) : static_cast<const void *>(x);
    if (workgroups) *workgroups = (tiles + tiles_per_wg - 1) / tiles_per_wg;
    if (workgroups && !wp) return 0;  // asked for the grid only
    hipLaunchKernelGGL((gemv_i4g32_mfma_kernel<MT, HP, S, RBW, D, KC, XM, YM, D0>), dim3((tiles + tiles_per_wg - 1) / tiles_per_wg, ksplit),
                       dim3(256 * RBW), C::TOTAL, st, wp, sc, a0, pre.delta, pre.w, N, K, pv | (pre.n << 8), K / ksplit, y, pre.res_out,
                       pre.eps);
    return hip_check(hipGetLastError(), "gemv_i4g32_mfma launch");
}

template <int MT, int S, int RBW, int D, int KC = 4096>
static int launch_pair(const uint16_t *x, const uint8_t *wp, const uint16_t *sc, float *y, int N, int K, hipStream_t st) {
    typedef GemvPairCfg<S, RBW, KC> C;
    static std::atomic<bool> attr_set{false};
    if (!attr_set.load(std::memory_order_acquire)) {
        CHADQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_i4g32_mfma_pair_kernel<MT, S, RBW, D, KC>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, C::TOTAL));
        attr_set.store(true, std::memory_order_release);
    }
    const int tiles_per_wg = 4 / C::KS * RBW;
    const int pv = pick_tile_rows(N, C::P, tiles_per_wg, 1);
    const int tiles = (N + pv - 1) / pv;
    hipLaunchKernelGGL((gemv_i4g32_mfma_pair_kernel<MT, S, RBW, D, KC>), dim3((tiles + tiles_per_wg - 1) / tiles_per_wg), dim3(256 * RBW),
                       C::TOTAL, st, x, wp, sc, y, N, K, pv);
    return hip_check(hipGetLastError(), "gemv_i4g32_mfma_pair launch");
}

template <int S, int RBW, int D, int KC = 2048>
static int launch_rows16(const uint16_t *x, const uint8_t *wp, const uint16_t *sc, float *y, int M, int N, int K, hipStream_t st) {
    typedef GemvRows16Cfg<S, RBW, KC> C;
    static std::atomic<bool> attr_set{false};
    if (!attr_set.load(std::memory_order_acquire)) {
        CHADQ_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&gemv_i4g32_mfma_rows16_kernel<S, RBW, D, KC>),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, C::TOTAL));
        attr_set.store(true, std::memory_order_release);
    }
    const int tiles_per_wg = 4 / C::KS * RBW;
    const int pv = pick_tile_rows(N, C::P, tiles_per_wg, 1);
    const int tiles = (N + pv - 1) / pv;
    hipLaunchKernelGGL((gemv_i4g32_mfma_rows16_kernel<S, RBW, D, KC>), dim3((tiles + tiles_per_wg - 1) / tiles_per_wg), dim3(256 * RBW),
                       C::TOTAL, st, x, wp, sc, y, M, N, K, pv);
    return hip_check(hipGetLastError(), "gemv_i4g32_mfma_rows16 launch");
}

int gemv_i4g32_mfma_dispatch(const uint16_t *x, const uint8_t *wp, const uint16_t *sc, float *y, int M, int N, int K,
                             hipStream_t st) {
    // the matrix-core kernel wants 16-byte aligned scale rows (K % 256 == 0) and 32-bit byte offsets
    if ((K & 255) != 0 || (int64_t)N * (K / 2) >= ((int64_t)1 << 31) || (reinterpret_cast<uintptr_t>(sc) & 15u) != 0)
        return gemv_i4g32_dispatch(x, wp, sc, y, M, N, K, st);
    // 9 to 16 activation rows: the 16-row form reads the weights once
    if (M > 8 && M <= 16)
        return N >= 8192 ? launch_rows16<8, 2, 4>(x, wp, sc, y, M, N, K, st) : launch_rows16<4, 1, 4>(x, wp, sc, y, M, N, K, st);
    // up to 8 activation rows per launch (more than 16 rows: the kernels run on 8 rows at a time)
    for (int m0 = 0; m0 < M; m0 += 8) {
        const int mm = (M - m0) < 8 ? (M - m0) : 8;
        const uint16_t *xm = x + (size_t)m0 * K;
        float *ym = y + (size_t)m0 * N;
        int rc = 0;
        // <rows, K-parts, steps per wave, 4-wave groups per workgroup, prefetch distance>, picked by measurement
        // Matrices with many rows run with 32 (M <= 4) or 64-row workgroups whose waves walk 16 steps of a chunk:
        // half as many workgroups stage the activations and each wave's stream is twice as long.  Short matrices
        // keep 16-row workgroups so that the grid still covers the chip.
        const bool tall = N >= 8192;
        switch (mm) {
            case 1:
                if (K <= 2048)  // rows of at most 2048 k: 2048-wide chunks (no loads past the row)
                    rc = tall ? launch_mfma<1, 2, 8, 1, 4, 2048>(xm, wp, sc, ym, N, K, st)
                              : launch_mfma<1, 4, 4, 1, 4, 2048>(xm, wp, sc, ym, N, K, st);
                else
                    rc = tall ? launch_mfma<1, 2, 16, 1, 4>(xm, wp, sc, ym, N, K, st) : launch_mfma<1, 4, 8, 1, 3>(xm, wp, sc, ym, N, K, st);
                break;
            case 2:
                rc = tall ? launch_mfma<2, 2, 16, 1, 3>(xm, wp, sc, ym, N, K, st) : launch_mfma<2, 2, 8, 1, 2>(xm, wp, sc, ym, N, K, st);
                break;
            case 3:
                rc = tall ? launch_mfma<3, 1, 16, 1, 4>(xm, wp, sc, ym, N, K, st) : launch_mfma<3, 1, 8, 1, 8>(xm, wp, sc, ym, N, K, st);
                break;
            case 4:
                rc = tall ? launch_mfma<4, 1, 16, 1, 4>(xm, wp, sc, ym, N, K, st) : launch_mfma<4, 1, 8, 1, 8>(xm, wp, sc, ym, N, K, st);
                break;
            case 5:
                rc = tall ? launch_pair<5, 16, 2, 4>(xm, wp, sc, ym, N, K, st) : launch_pair<5, 8, 2, 3>(xm, wp, sc, ym, N, K, st);
                break;
            case 6:
                rc = tall ? launch_pair<6, 16, 2, 4>(xm, wp, sc, ym, N, K, st) : launch_pair<6, 8, 2, 3>(xm, wp, sc, ym, N, K, st);
                break;
            case 7:
                rc = tall ? launch_pair<7, 16, 2, 4>(xm, wp, sc, ym, N, K, st) : launch_pair<7, 8, 2, 3>(xm, wp, sc, ym, N, K, st);
                break;
            default:
                rc = tall ? launch_pair<8, 16, 2, 4>(xm, wp, sc, ym, N, K, st) : launch_pair<8, 8, 2, 3>(xm, wp, sc, ym, N, K, st);
                break;
        }
        if (rc != 0) return rc;
    }
    return 0;
}

// y = W x (M = 1) with the per-workgroup argmax candidates of y written beside it (YM = 2 above).  Only the shape of a
// decoder's output table is covered: many rows, K <= 2048.  *n_cand receives the number of candidates (workgroups);
// wp = nullptr asks for that number only.
bool gemv_i4g32_argmax_ok(const uint16_t *sc, int N, int K) {
    return N >= 8192 && K <= 2048 && (K & 255) == 0 && (int64_t)N * (K / 2) < ((int64_t)1 << 31) &&
           (reinterpret_cast<uintptr_t>(sc) & 15u) == 0;
}

int gemv_i4g32_argmax_launch(const uint16_t *x, const uint8_t *wp, const uint16_t *sc, float *y, int N, int K, float *cand_v,
                             int32_t *cand_i, int *n_cand, hipStream_t st) {
    const GemvPre pre{nullptr, cand_v, reinterpret_cast<const float *>(cand_i), nullptr, 0, 0.f};
    return launch_mfma<1, 2, 8, 1, 4, 2048, 0, 2>(x, wp, sc, y, N, K, st, 1, pre, n_cand);
}

// Split-K form, M = 1: part s of y_parts [ksplit, N] holds the sum over k in [s*K/ksplit, (s+1)*K/ksplit).
// K / ksplit must be a multiple of the 4096-wide chunk.
int gemv_i4g32_splitk_launch(const uint16_t *x, const uint8_t *wp, const uint16_t *sc, float *y_parts, int N, int K,
                             int ksplit, hipStream_t st) {
    return launch_mfma<1, 4, 8, 1, 4>(x, wp, sc, y_parts, N, K, st, ksplit);
}

// The same with x[k] = bf16( gelu_tanh(gu[k]) * gu[K + k] ) formed inside the kernel.
int gemv_i4g32_splitk_geglu_launch(const float *gu, const uint8_t *wp, const uint16_t *sc, float *y_parts, int N, int K,
                                   int ksplit, hipStream_t st) {
    // 8-wave workgroups: a compute unit forms its K range of the gated activation once instead of twice
    return launch_mfma<1, 4, 8, 2, 3, 4096, 1>(reinterpret_cast<const uint16_t *>(gu), wp, sc, y_parts, N, K, st, ksplit);
}

// y = W x with x = bf16(rmsnorm(res + sum of n delta vectors) * w) formed inside the kernel; res_out receives the sum.
// K <= 2048 and a multiple of 256.
int gemv_i4g32_addnorm_launch(const float *res, const float *delta, int n, const float *w, float eps, float *res_out,
                              const uint8_t *wp, const uint16_t *sc, float *y, int N, int K, hipStream_t st) {
    const GemvPre pre{res, delta, w, res_out, n, eps};
    // many rows: workgroups of 16 waves, so that a compute unit forms the activation vector once, not four times; two
    // weight loads per wave before the vector is formed and a prefetch distance of three behind it measured best
    if (N >= 8192) return launch_mfma<1, 2, 8, 4, 3, 2048, 2, 0, 2>(nullptr, wp, sc, y, N, K, st, 1, pre);
    return launch_mfma<1, 4, 4, 1, 4, 2048, 2>(nullptr, wp, sc, y, N, K, st, 1, pre);
}

// The same with the rows of W taken as (gate, up) pairs: h[i] = bf16( gelu_tanh(y[2i]) * y[2i+1] ), N/2 values.
int gemv_i4g32_addnorm_geglu_launch(const float *res, const float *delta, int n, const float *w, float eps, float *res_out,
                                    const uint8_t *wp, const uint16_t *sc, uint16_t *h, int N, int K, hipStream_t st) {
    const GemvPre pre{res, delta, w, res_out, n, eps};
    float *y = reinterpret_cast<float *>(h);
    if (N >= 8192) return launch_mfma<1, 2, 8, 4, 3, 2048, 2, 1, 2>(nullptr, wp, sc, y, N, K, st, 1, pre);
    return launch_mfma<1, 4, 4, 1, 4, 2048, 2, 1>(nullptr, wp, sc, y, N, K, st, 1, pre);
}

}  // namespace chadq
