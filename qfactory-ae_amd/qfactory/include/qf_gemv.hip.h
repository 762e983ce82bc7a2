// Dequant-fused low-bit GEMV for gfx950, small-M regime (HBM-bound).
//
//   C[m][n] = fp16( sum_k A[m][k] * (q[n][k] - Z[n][k/GS]) * s[n][k/GS] )        (grouped)
//   C[m][n] = fp16( sum_k A[m][k] * q[n][k] )                                    (QPARAM == false)
//
// Replaces kernel_gptq / gptq_gemv_impl (qfactory/include/gptq_gemv.h:14-205) and kernel_gemv /
// gemv_impl (qfactory/include/gemv.h:12-135) of the reference; consumes the same packed tensors.
//
// Mapping (one "team" = WK waves sweeps rows of the packed weight matrix):
//   * a lane owns IT fixed 'chunks' of the K axis (VB bytes of packed weight each, chunk index
//     tt + 64*WK*it) so that every wave-wide weight load is 64*VB contiguous bytes of one row;
//   * the activations of those chunks are loaded once and stay in registers for all the rows the
//     team visits (A-stationary), the weights stream through with U rows in flight per stage and
//     the next stage prefetched while the current one is consumed;
//   * fields are decoded to fp16 pairs holding 1024 + 2^o*q and fed to v_dot2_f32_f16 with fp32
//     accumulators; the 1024 offsets, the 2^-o factors, the zero-point and the scale are applied
//     once per chunk in fp32:  s * (sum a*q - Z * sum a);
//   * the U*MT partial sums of a stage are summed across the wave with a halving butterfly, across
//     the WK waves through LDS, and every output element is written exactly once.
#pragma once

#include <cstdio>
#include "qf_common.hip.h"

// 1: a kernel that adds to its output (QF_OUT_ACCUMULATE) requests the output elements a thread will write when the
// block starts; 0: right in front of the store.
#ifndef QF_GEMV_EARLY_OUT
#define QF_GEMV_EARLY_OUT 1
#endif

namespace qf {

template <int NBITS_, int GS_, bool SYM_, bool QPARAM_, int N_, int K_, int MT_, int WK_, int WN_,
          int U_, int STEPS_, int VB_, bool NT_B_>
struct GemvCfg {
    static constexpr int NBITS = NBITS_;      // weight field width: 2, 3, 4 or 8
    static constexpr int GS = GS_;            // group size along K (ignored when !QPARAM)
    static constexpr bool SYM = SYM_;         // implicit zero-point 2^(b-1), no zero tensor read
    static constexpr bool QPARAM = QPARAM_;   // false: no scale / zero at all (group_size == -1 path)
    static constexpr int N = N_, K = K_;
    static constexpr int MT = MT_;            // activation rows handled per block (grid.y tiles M)
    static constexpr int WK = WK_;            // waves along K per team
    static constexpr int WN = WN_;            // teams per block
    static constexpr int U = U_;              // weight rows in flight per team and stage
    static constexpr int STEPS = STEPS_;      // stages per block
    static constexpr int VB = VB_;            // bytes of packed weight per lane and load: 16, 8 or 4
    static constexpr bool NT_B = NT_B_;       // stream the weights with non-temporal loads

    static constexpr int PB = plane_bits(NBITS);        // field width of the main plane (3-bit: 2 + 1-bit plane)
    static constexpr int NW = VB / 4;                   // 32-bit words of the main plane per chunk
    static constexpr int NWH = NBITS == 3 ? NW / 2 : 0; // 32-bit words of the 1-bit plane per chunk
    static constexpr int HI_OFF = K / 4;                // byte offset of the 1-bit plane in a 3-bit row
    static constexpr int EPC = VB * 8 / PB;             // elements per chunk
    static constexpr int NCH = K / EPC;                 // chunks per row
    static constexpr int T = 64 * WK;                   // threads per team
    static constexpr int IT = (NCH + T - 1) / T;        // chunks per lane and row
    static constexpr int THREADS = 64 * WK * WN;
    static constexpr int RPT = U * STEPS;               // rows per team
    static constexpr int RPB = RPT * WN;                // rows per block
    static constexpr int V = U * MT;                    // partial sums per stage
    static constexpr int RB = K * NBITS / 8;            // packed weight row bytes
    static constexpr int G = QPARAM ? K / (GS > 0 ? GS : 1) : 0;   // groups per row
    static constexpr int ZFB = zero_field_bits(NBITS);  // stored width of one zero-point
    static constexpr int ZRB = G * ZFB / 8;             // packed zero row bytes
    static constexpr int GRID_X = (N + RPB - 1) / RPB;
};

// Timing experiments (results are wrong when non-zero): bit 0 replaces the decode + dot products by
// an xor of the loaded words, bit 1 skips the activation loads, bit 2 reads the scales / zero-points of row 0 for
// every row, bit 3 drops the cross-lane sums, the LDS exchange and the stores.
// A translation unit that sets it must also define QF_ALLOW_TIMING_EXPERIMENTS; the code generator never does.
#ifndef QF_GEMV_EXPERIMENT
#define QF_GEMV_EXPERIMENT 0
#endif
#if QF_GEMV_EXPERIMENT != 0 && !defined(QF_ALLOW_TIMING_EXPERIMENTS)
#error "QF_GEMV_EXPERIMENT gives wrong results: timing builds only (define QF_ALLOW_TIMING_EXPERIMENTS)"
#endif

// Decode strategy (the reference's search dimension, qfactory/core/qfunc.py:85-91; utils.h:46-62 against :193-213).
// 0, "deferred": integer dot products per chunk, then s * (sum a*q - Z * sum a) once per chunk in fp32.
// 1, "eager": every field pair becomes the fp16 weight first -- (x - (1024 + 2^o Z)) * s with packed fp16 adds and
// multiplies, i.e. 2^o * fp16_rn((q - Z) * s) -- and the dot product runs on those; the 2^-o of a class is applied
// to its fp32 sum.  Two more packed instructions per pair; no per-chunk activation sums.
#ifndef QF_GEMV_EAGER
#define QF_GEMV_EAGER 0
#endif

#ifndef QF_GEMV_A_FIRST
#define QF_GEMV_A_FIRST 1
#endif

// 1: the weight matrix is a fused gate+up projection (rows 0 .. N/2-1 gate, rows N/2 .. N-1 up) and the
// kernel writes the (M, N/2) SwiGLU activation out[m][i] = fp16(silu(gate[m][i])) * up[m][i] instead of
// the (M, N) projection: a team's rows alternate between a gate row and its up row, and the pair meets in
// the block's final sum.  Same roundings as the projection followed by qf_silu_mul of libqfactory_hip.so
// (both results rounded to fp16 first; silu(x) = x * rcp(1 + exp2(-x * log2(e)))), which it replaces for
// few rows.  The reference has no such fusion; its end-to-end runs leave the step to vLLM's SiluAndMul.
#ifndef QF_GEMV_GATE_UP_SILU
#define QF_GEMV_GATE_UP_SILU 0
#endif

// 1: the kernel's activations are not read but made: residual add and RMSNorm of the decoder layer run in front of
// the dot products,  h = fp16(x + delta),  a = fp16(fp16(h * rsqrt(mean(h^2) + eps)) * gamma)  -- the roundings of
// qf_add_rmsnorm in libqfactory_hip.so, which this replaces for few rows.  Every team holds a whole activation row
// in its lanes (that is the kernel's mapping), so the sum of squares is one butterfly and one exchange through LDS,
// done by every block for itself while its first weights are in flight; the first team of block (0, y) also
// writes h to x_out, the next residual stream (a buffer of its own: other blocks still read x and delta).
// fp16 only.  Not in the reference, whose end-to-end runs leave the norm to vLLM's fused_add_rms_norm.
#ifndef QF_GEMV_NORM_PROLOGUE
#define QF_GEMV_NORM_PROLOGUE 0
#endif

// 1: the scales and zero-points of the block's rows go through LDS (the reference's SMEM_QUANT choice,
// qfactory/include/gptq_gemv.h:62-82): the rows of a block are contiguous in both tensors, so the block fetches
// them with coalesced loads issued ahead of everything else, and a lane reads its group's pair from LDS instead
// of issuing two narrow global loads behind every 16 bytes of weights.
#ifndef QF_GEMV_SMEM_QUANT
#define QF_GEMV_SMEM_QUANT 0
#endif

// 1: scales and zero-points are applied after the first steps of the cross-lane sum instead of per lane.  The
// lanes that share a group (GS / elements-per-chunk consecutive lanes, four at 4 bits and groups of 128) first
// add their integer-domain chunk sums with the butterfly's own first halving steps; a lane then owns one row
// (of the stage's U) and one group, loads that one scale and zero-point, applies  s * (T - Z * sum a)  and the
// butterfly goes on.  Per stage and chunk a lane issues U >> PRE scale loads instead of U (PRE = 2 at best), and
// the scale arithmetic shrinks alike.  Deferred decode only; not with the scales through LDS.
#ifndef QF_GEMV_QUANT_DEDUP
#define QF_GEMV_QUANT_DEDUP 0
#endif

// Lower bound on resident waves per SIMD the register allocator must leave room for (0: no bound).
#ifndef QF_GEMV_WAVES_PER_EU
#define QF_GEMV_WAVES_PER_EU 0
#endif
#if QF_GEMV_WAVES_PER_EU > 0
#define QF_GEMV_OCCUPANCY __attribute__((amdgpu_waves_per_eu(QF_GEMV_WAVES_PER_EU)))
#else
#define QF_GEMV_OCCUPANCY
#endif

template <class C>
__global__ __launch_bounds__(C::THREADS) QF_GEMV_OCCUPANCY void gemv_kernel(
    const uint16_t* __restrict__ A, const uint8_t* __restrict__ W, uint16_t* __restrict__ Cout,
    const uint16_t* __restrict__ S, const uint8_t* __restrict__ Zp, int m_total, NormArgs norm) {
    using D = Decode<C::NBITS>;
    constexpr int NW = C::NW, EPC = C::EPC, NCH = C::NCH, T = C::T, IT = C::IT;
    constexpr int MT = C::MT, U = C::U, STEPS = C::STEPS, V = C::V, WK = C::WK;
    constexpr int PAIRS = D::PAIRS, NCLS = D::NCLS;
    constexpr int AR = NW * PAIRS;                     // 32-bit activation registers per chunk
    constexpr int P8 = 8 / C::ZFB;                     // zero-point fields per byte
    constexpr uint32_t ZMASK = (1u << C::ZFB) - 1u;
    constexpr int NWH = C::NWH;
    constexpr bool SILU = QF_GEMV_GATE_UP_SILU != 0;
    constexpr bool NORM = QF_GEMV_NORM_PROLOGUE != 0;
    constexpr bool EAGER = QF_GEMV_EAGER != 0 && C::QPARAM;
    constexpr bool SMEMQ = QF_GEMV_SMEM_QUANT != 0 && C::QPARAM;
    constexpr int LPG = C::QPARAM ? C::GS / EPC : 1;                              // lanes per group
    constexpr int PRE = !(QF_GEMV_QUANT_DEDUP && C::QPARAM && !EAGER && !SMEMQ) ? 0
                        : ((LPG % 4 == 0 && U % 4 == 0) ? 2 : ((LPG % 2 == 0 && U % 2 == 0) ? 1 : 0));
    constexpr int UP = U >> PRE, VP = V >> PRE;                                   // rows / partial sums a lane keeps after PRE halving steps
    constexpr int SQ_WORDS = SMEMQ ? (C::RPB * C::G * 2 + 3) / 4 : 1;           // 32-bit words of the block's scales
    constexpr int ZQ_WORDS = SMEMQ && !C::SYM ? (C::RPB * C::ZRB + 3) / 4 : 1;  // and of its zero-points

    __shared__ uint32_t sq_s[SQ_WORDS], sq_z[ZQ_WORDS];
    __shared__ float red[C::WN][WK][STEPS * V];
    __shared__ float norm_ss[NORM ? C::WN : 1][NORM ? WK : 1][MT];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    // wave-uniform indices in scalar registers: row pointers are then scalar bases advanced with
    // scalar adds, and every load is base + one 32-bit lane offset (no 64-bit vector arithmetic)
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wk = wave % WK;
    const int team = wave / WK;
    const int tt = wk * 64 + lane;
    const int m0 = blockIdx.y * MT;
    const int row_base = blockIdx.x * C::RPB + team * C::RPT;

    // ---- scales / zero-points of the block's RPB rows: requested before anything else (SMEM_QUANT) ----
    constexpr int SQ_PER = (SQ_WORDS + C::THREADS - 1) / C::THREADS, ZQ_PER = (ZQ_WORDS + C::THREADS - 1) / C::THREADS;
    uint32_t sq_reg[SQ_PER], zq_reg[ZQ_PER];
    if constexpr (SMEMQ) {
        // rows past N (last block) clamp to the end of the tensor: loaded, never used
        const size_t s_words = ((size_t)C::N * C::G * 2) / 4, z_words = ((size_t)C::N * C::ZRB) / 4;
        const uint32_t* sg = reinterpret_cast<const uint32_t*>(S) + ((size_t)blockIdx.x * C::RPB * C::G * 2) / 4;
        const uint32_t* zg = reinterpret_cast<const uint32_t*>(Zp) + ((size_t)blockIdx.x * C::RPB * C::ZRB) / 4;
        const size_t s_first = ((size_t)blockIdx.x * C::RPB * C::G * 2) / 4, z_first = ((size_t)blockIdx.x * C::RPB * C::ZRB) / 4;
#pragma unroll
        for (int i = 0; i < SQ_PER; i++) {
            const int wd = tid + i * C::THREADS;
            sq_reg[i] = sg[min((size_t)wd, s_words - 1 - s_first)];
        }
        if constexpr (!C::SYM) {
#pragma unroll
            for (int i = 0; i < ZQ_PER; i++) {
                const int wd = tid + i * C::THREADS;
                zq_reg[i] = zg[min((size_t)wd, z_words - 1 - z_first)];
            }
        }
    }

    // ---- per-lane chunk bookkeeping ----
    int coff[IT];            // byte offset of the chunk inside a packed weight row
    int goff[IT];            // group index of the chunk
    bool cvalid[IT];
#pragma unroll
    for (int it = 0; it < IT; it++) {
        const int c = tt + T * it;
        cvalid[it] = c < NCH;
        const int cc = cvalid[it] ? c : 0;
        coff[it] = cc * C::VB;
        goff[it] = C::QPARAM ? (cc * EPC) / (C::GS > 0 ? C::GS : 1) : 0;
    }

    // ---- streaming stages ----
    struct Stage {
        uint32_t w[U][IT][NW];
        uint32_t h[U][IT][NWH > 0 ? NWH : 1];
        scale_holder_t s[UP][IT];
        zero_holder_t z[UP][IT];
    };
    // after PRE halving steps a lane keeps rows j + u_lane, j < UP, of a stage (the halving sends the upper half of
    // the values to the lanes whose distance bit is set)
    int u_lane = 0;
    if constexpr (PRE >= 1) u_lane += (lane & kLaneOrder(0)) ? U / 2 : 0;
    if constexpr (PRE >= 2) u_lane += (lane & kLaneOrder(1)) ? U / 4 : 0;

    auto load_stage = [&](Stage& st, int step) {
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int lrow = min(row_base + step * U + u, C::N - 1);
            // gate+up: even positions of the sweep are gate rows, odd ones the up rows of the same output
            const int row = SILU ? (lrow >> 1) + (lrow & 1) * (C::N / 2) : lrow;
            const uint8_t* wrow = W + (size_t)row * C::RB;
            const uint8_t* srow = reinterpret_cast<const uint8_t*>(S) + (size_t)row * C::G * 2;
            const uint8_t* zrow = Zp + (size_t)row * C::ZRB;
#pragma unroll
            for (int it = 0; it < IT; it++) {
                load_words<NW, C::NT_B>(wrow + (uint32_t)coff[it], st.w[u][it]);
                if constexpr (NWH > 0) load_words<NWH, C::NT_B>(wrow + (uint32_t)(C::HI_OFF + coff[it] / 2), st.h[u][it]);
                if constexpr (C::QPARAM && !SMEMQ && PRE == 0) {
                    const uint8_t* sr = (QF_GEMV_EXPERIMENT & 4) ? reinterpret_cast<const uint8_t*>(S) : srow;   // timing: always row 0 (cache hits)
                    const uint8_t* zr = (QF_GEMV_EXPERIMENT & 4) ? Zp : zrow;
                    st.s[u][it] = *reinterpret_cast<const uint16_t*>(sr + (uint32_t)(goff[it] * 2));
                    if constexpr (!C::SYM) st.z[u][it] = zr[(uint32_t)(goff[it] / P8)];
                }
            }
        }
        if constexpr (PRE > 0) {
            // one scale and one zero-point per row this lane will own after the first halving steps
#pragma unroll
            for (int j = 0; j < UP; j++) {
                const int lrow = min(row_base + step * U + j + u_lane, C::N - 1);            // per lane
                const int row = SILU ? (lrow >> 1) + (lrow & 1) * (C::N / 2) : lrow;
#pragma unroll
                for (int it = 0; it < IT; it++) {
                    st.s[j][it] = *reinterpret_cast<const uint16_t*>(
                        reinterpret_cast<const uint8_t*>(S) + (uint32_t)(row * (C::G * 2) + goff[it] * 2));
                    if constexpr (!C::SYM) st.z[j][it] = Zp[(uint32_t)(row * C::ZRB + goff[it] / P8)];
                }
            }
        }
    };

    // Load order (QF_GEMV_A_FIRST, default 1).  Loads complete in issue order, so whatever is issued
    // behind the first stage of weights is only seen once those have arrived from HBM.  With the
    // activation loads issued first (they come from L2, a few hundred ns) their per-chunk sums are
    // computed while the weights are still in flight; issued second, that work waits for the weights.
    Stage st0, st1;
    uint32_t a[MT][IT][AR];
    float c1[MT][IT];        // sum over classes of 1024 * 2^-o * (sum of a in that class)
    float sa[MT][IT];        // sum of a over the chunk
    if constexpr (!QF_GEMV_A_FIRST) load_stage(st0, 0);
    // ---- the stationary activations ----
#pragma unroll
    for (int it = 0; it < IT; it++) {
#pragma unroll
        for (int m = 0; m < MT; m++) {
            const int mm = min(m0 + m, m_total - 1);
            const uint16_t* ap = A + (size_t)mm * C::K + (size_t)(coff[it] / C::VB) * EPC;
#pragma unroll
            for (int r = 0; r < AR; r += (AR >= 4 ? 4 : AR)) {
                constexpr int LW = AR >= 4 ? 4 : AR;
                uint32_t tmp[LW];
                if (QF_GEMV_EXPERIMENT & 2) { for (int j = 0; j < LW; j++) tmp[j] = 0x3C003C00u; }
                else load_words<LW, false>(ap + 2 * r, tmp);
#pragma unroll
                for (int j = 0; j < LW; j++) a[m][it][r + j] = tmp[j];
            }
        }
    }
    if constexpr (QF_GEMV_A_FIRST) load_stage(st0, 0);
#if QF_OUT_ACCUMULATE && QF_GEMV_EARLY_OUT
    // Adding to the output: the elements this thread will write at the end (the cross-wave sum below deals them by
    // thread index) are requested now, behind the activations and the first weight stage, instead of in front of the
    // store, where a one-shot block would wait out their round trip with nothing else to do.
    constexpr int OUTS = (STEPS * V + T - 1) / T;
    uint16_t old_out[OUTS];
    if constexpr (!(WK == 1 && !SILU)) {
#pragma unroll
        for (int i = 0; i < OUTS; i++) {
            const int j = min(tt + i * T, STEPS * V - 1);
            const int step = j / V, v = j % V;
            const int row = min(row_base + step * U + v / MT, C::N - 1), m = min(m0 + v % MT, m_total - 1);
            old_out[i] = Cout[(size_t)m * C::N + row];
        }
    }
#endif
    if constexpr (NORM) {
        static_assert(!QF_IN_BF16, "the norm prologue is fp16 only");
        // ---- residual add, sum of squares, normalisation: a[][][] becomes the normalised row ----
        uint32_t gam[IT][AR];
#pragma unroll
        for (int it = 0; it < IT; it++) {
            const uint16_t* gp = norm.gamma + (size_t)(coff[it] / C::VB) * EPC;
#pragma unroll
            for (int r = 0; r < AR; r += (AR >= 4 ? 4 : AR)) {
                constexpr int LW = AR >= 4 ? 4 : AR;
                uint32_t tmp[LW];
                load_words<LW, false>(gp + 2 * r, tmp);
#pragma unroll
                for (int j = 0; j < LW; j++) gam[it][r + j] = tmp[j];
            }
        }
        float ss[MT];
        const bool writer = norm.x_out != nullptr && blockIdx.x == 0 && team == 0;
#pragma unroll
        for (int m = 0; m < MT; m++) {
            ss[m] = 0.0f;
            const int mm = min(m0 + m, m_total - 1);
#pragma unroll
            for (int it = 0; it < IT; it++) {
                const size_t eoff = (size_t)mm * C::K + (size_t)(coff[it] / C::VB) * EPC;
                if (norm.delta != nullptr) {
#pragma unroll
                    for (int r = 0; r < AR; r += (AR >= 4 ? 4 : AR)) {
                        constexpr int LW = AR >= 4 ? 4 : AR;
                        uint32_t tmp[LW];
                        load_words<LW, false>(norm.delta + eoff + 2 * r, tmp);
#pragma unroll
                        for (int j = 0; j < LW; j++)
                            a[m][it][r + j] = __builtin_bit_cast(uint32_t, as_f16x2(a[m][it][r + j]) + as_f16x2(tmp[j]));
                    }
                }
                if (writer && cvalid[it] && m0 + m < m_total) {
#pragma unroll
                    for (int r = 0; r < AR; r++) reinterpret_cast<uint32_t*>(norm.x_out + eoff)[r] = a[m][it][r];
                }
#pragma unroll
                for (int r = 0; r < AR; r++) {
                    if (!cvalid[it]) a[m][it][r] = 0u;
                    ss[m] = __builtin_amdgcn_fdot2(as_f16x2(a[m][it][r]), as_f16x2(a[m][it][r]), ss[m], false);
                }
            }
            ss[m] += lane_xor<1>(ss[m]);
            ss[m] += lane_xor<2>(ss[m]);
            ss[m] += lane_xor<4>(ss[m]);
            ss[m] += lane_xor<8>(ss[m]);
            ss[m] += lane_xor<16>(ss[m]);
            ss[m] += lane_xor<32>(ss[m]);
            if (lane == 0) norm_ss[team][wk][m] = ss[m];
        }
        __syncthreads();
#pragma unroll
        for (int m = 0; m < MT; m++) {
            float total = 0.0f;
#pragma unroll
            for (int w2 = 0; w2 < WK; w2++) total += norm_ss[team][w2][m];
            const float rn = rsqrtf(total / (float)C::K + norm.eps);
#pragma unroll
            for (int it = 0; it < IT; it++)
#pragma unroll
                for (int r = 0; r < AR; r++) {
                    const f16x2 h = as_f16x2(a[m][it][r]);
                    f16x2 n;
                    n.x = (_Float16)((float)h.x * rn);
                    n.y = (_Float16)((float)h.y * rn);
                    a[m][it][r] = __builtin_bit_cast(uint32_t, n * as_f16x2(gam[it][r]));
                }
        }
    }
    if constexpr (SMEMQ) {
#pragma unroll
        for (int i = 0; i < SQ_PER; i++)
            if (tid + i * C::THREADS < SQ_WORDS) sq_s[tid + i * C::THREADS] = sq_reg[i];
        if constexpr (!C::SYM) {
#pragma unroll
            for (int i = 0; i < ZQ_PER; i++)
                if (tid + i * C::THREADS < ZQ_WORDS) sq_z[tid + i * C::THREADS] = zq_reg[i];
        }
        __syncthreads();
    }
    // ---- and their per-chunk sums ----
#pragma unroll
    for (int it = 0; it < IT; it++) {
#pragma unroll
        for (int m = 0; m < MT; m++) {
            float cls_sum[NCLS];
#pragma unroll
            for (int c2 = 0; c2 < NCLS; c2++) cls_sum[c2] = 0.0f;
#pragma unroll
            for (int r = 0; r < AR; r++) {
                const uint32_t val = cvalid[it] ? act_pair(a[m][it][r]) : 0u;   // once per block: the activations stay in registers
                a[m][it][r] = val;
                // sum of the pair in one instruction: dot2 with (1, 1)
                cls_sum[D::cls(r % PAIRS)] = __builtin_amdgcn_fdot2(
                    as_f16x2(val), as_f16x2(0x3C003C00u), cls_sum[D::cls(r % PAIRS)], false);
            }
            float c1v = 0.0f, sav = 0.0f;
#pragma unroll
            for (int c2 = 0; c2 < NCLS; c2++) {
                c1v += 1024.0f * D::inv_scale(c2) * cls_sum[c2];
                sav += cls_sum[c2];
            }
            c1[m][it] = c1v;
            sa[m][it] = sav;
        }
    }

    // sum of the activations over a group's share of lanes (the lanes PRE halving steps bring together)
    float saq[MT][IT];
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int it = 0; it < IT; it++) {
            float v = sa[m][it];
            if constexpr (PRE >= 1) v += lane_xor<kLaneOrder(0)>(v);
            if constexpr (PRE >= 2) v += lane_xor<kLaneOrder(1)>(v);
            saq[m][it] = v;
        }

    auto compute_stage = [&](const Stage& st, int step) {
        float part[V];
        float tq[PRE > 0 ? IT : 1][V];        // PRE > 0: integer-domain chunk sums, scaled after the first halving steps
#pragma unroll
        for (int v = 0; v < V; v++) part[v] = 0.0f;
#pragma unroll
        for (int u = 0; u < U; u++) {
#pragma unroll
            for (int it = 0; it < IT; it++) {
                float acc[MT][NCLS];
#pragma unroll
                for (int m = 0; m < MT; m++)
#pragma unroll
                    for (int c2 = 0; c2 < NCLS; c2++) acc[m][c2] = 0.0f;
                uint32_t sbits = 0x3C00u, zint = 0u;               // scale (fp16 bits) and zero-point of this chunk's group
                if constexpr (C::QPARAM && PRE == 0) {
                    const int brow = team * C::RPT + step * U + u;            // row inside the block
                    if constexpr (SMEMQ) sbits = reinterpret_cast<const uint16_t*>(sq_s)[brow * C::G + goff[it]];
                    else sbits = (uint16_t)st.s[u][it];
                    if constexpr (C::SYM) {
                        zint = 1u << (C::NBITS - 1);
                    } else {
                        const uint32_t zbyte = SMEMQ ? reinterpret_cast<const uint8_t*>(sq_z)[brow * C::ZRB + goff[it] / P8] : st.z[u][it];
                        zint = (zbyte >> ((goff[it] % P8) * C::ZFB)) & ZMASK;
                    }
                }
                // eager: per class the fp16 pair -(1024 + 2^o Z) (exact: below 2048) and the scale pair
                f16x2 off[NCLS];
                const f16x2 s2 = as_f16x2(sbits * 0x00010001u);
                if constexpr (EAGER) {
#pragma unroll
                    for (int c2 = 0; c2 < NCLS; c2++) off[c2] = as_f16x2((0xE400u + (zint << D::shift(c2))) * 0x00010001u);
                }
                if constexpr ((QF_GEMV_EXPERIMENT & 1) != 0) {
                    uint32_t t = 0;
                    for (int j = 0; j < NW; j++) t ^= st.w[u][it][j];
                    acc[0][0] += (float)(t & 1u);
                } else
#pragma unroll
                for (int j = 0; j < NW; j++) {
                    uint32_t x[PAIRS];
                    if constexpr (C::NBITS == 3) {
                        if (j % 2 == 0) D::template word<0>(st.w[u][it][j], st.h[u][it][j / 2], x);
                        else D::template word<1>(st.w[u][it][j], st.h[u][it][j / 2], x);
                    } else {
                        D::word(st.w[u][it][j], x);
                    }
#pragma unroll
                    for (int p = 0; p < PAIRS; p++) {
                        f16x2 wv = as_f16x2(x[p]);
                        if constexpr (EAGER) wv = (wv + off[D::cls(p)]) * s2;     // 2^o * fp16((q - Z) * s)
#pragma unroll
                        for (int m = 0; m < MT; m++)
                            acc[m][D::cls(p)] = __builtin_amdgcn_fdot2(
                                as_f16x2(a[m][it][j * PAIRS + p]), wv, acc[m][D::cls(p)], false);
                    }
                }
                const float sc = f16_bits_to_f32((uint16_t)sbits), zf = (float)zint;
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    float t = acc[m][0];
#pragma unroll
                    for (int c2 = 1; c2 < NCLS; c2++) t = __builtin_fmaf(acc[m][c2], D::inv_scale(c2), t);
                    if constexpr (EAGER) {
                        part[u * MT + m] += t;                   // the weights were dequantised before the dot product
                    } else {
                        t -= c1[m][it];                          // = sum a*q over the chunk
                        if constexpr (PRE > 0) {
                            tq[it][u * MT + m] = t;
                        } else if constexpr (C::QPARAM) {
                            t = __builtin_fmaf(-zf, sa[m][it], t);   // sum a*(q - Z)
                            part[u * MT + m] = __builtin_fmaf(sc, t, part[u * MT + m]);
                        } else {
                            part[u * MT + m] += t;
                        }
                    }
                }
            }
        }
        if constexpr (PRE > 0) {
            // the lanes of a group add their chunk sums (the butterfly's first PRE halving steps); the lane then
            // owns rows j + u_lane of the stage and applies its own row's scale and zero-point
#pragma unroll
            for (int it = 0; it < IT; it++) {
                halve_step<kLaneOrder(0), V, V>(tq[it], lane);
                if constexpr (PRE >= 2) halve_step<kLaneOrder(1), V / 2, V>(tq[it], lane);
#pragma unroll
                for (int i = 0; i < VP; i++) {
                    const int j = i / MT, m = i % MT;
                    const float sc = f16_bits_to_f32((uint16_t)st.s[j][it]);
                    float zf = (float)(1 << (C::NBITS - 1));
                    if constexpr (!C::SYM) zf = (float)((st.z[j][it] >> ((goff[it] % P8) * C::ZFB)) & ZMASK);
                    part[i] = __builtin_fmaf(sc, __builtin_fmaf(-zf, saq[m][it], tq[it][i]), part[i]);
                }
            }
            reduce_from<VP, PRE, V>(part, lane);
        } else if constexpr ((QF_GEMV_EXPERIMENT & 8) != 0) {          // timing: no cross-lane sums, no LDS, no stores
            float t = 0.f;
            for (int v = 0; v < V; v++) t += part[v];
            if (t == 12345.678f) Cout[lane] = 1;
            return;
        }
        if constexpr (PRE == 0) wave_reduce_many<V>(part, lane);
        if (reduce_owner<V>(lane)) {
            const int v = reduce_index<V>(lane);
            if constexpr (WK == 1 && !SILU) { // one wave owns the rows: store straight from the lane
                const int u = v / MT, m = v % MT;
                const int row = row_base + step * U + u;
                if (row < C::N && m0 + m < m_total)
                    store_out(Cout + (size_t)(m0 + m) * C::N + row, part[0]);
            } else {
                red[team][wk][step * V + v] = part[0];
            }
        }
    };

    QF_SCHED_FENCE();
#pragma unroll
    for (int step = 0; step < STEPS; step += 2) {
        if (step + 1 < STEPS) {
            load_stage(st1, step + 1);
            QF_SCHED_FENCE();  // the prefetch is issued before any compute of this step
        }
        compute_stage(st0, step);
        if (step + 1 < STEPS) {
            if (step + 2 < STEPS) {
                load_stage(st0, step + 2);
                QF_SCHED_FENCE();
            }
            compute_stage(st1, step + 1);
        }
    }

    if constexpr (WK == 1 && !SILU) return;
    if constexpr ((QF_GEMV_EXPERIMENT & 8) != 0) return;
    __syncthreads();

    if constexpr (SILU) {
        // ---- cross-wave sums of a gate row and its up row, one store of their SwiGLU product ----
        for (int j = tt; j < STEPS * V / 2; j += T) {
            const int step = j / (V / 2), r = j % (V / 2);
            const int u2 = r / MT, m = r % MT;
            float gate = 0.0f, up = 0.0f;
#pragma unroll
            for (int w2 = 0; w2 < WK; w2++) {
                gate += red[team][w2][step * V + (2 * u2) * MT + m];
                up += red[team][w2][step * V + (2 * u2 + 1) * MT + m];
            }
            const int lrow = row_base + step * U + 2 * u2;
            if (lrow < C::N && m0 + m < m_total) Cout[(size_t)(m0 + m) * (C::N / 2) + (lrow >> 1)] = silu_mul_f16(gate, up);
        }
        return;
    }

    // ---- cross-wave sum and the single store of every output element ----
    for (int j = tt; j < STEPS * V; j += T) {
        float total = 0.0f;
#pragma unroll
        for (int w2 = 0; w2 < WK; w2++) total += red[team][w2][j];
        const int step = j / V, v = j % V;
        const int u = v / MT, m = v % MT;
        const int row = row_base + step * U + u;
#if QF_OUT_ACCUMULATE && QF_GEMV_EARLY_OUT
        if (row < C::N && m0 + m < m_total) {
            // out = fp16(out + fp16(projection)) on the value requested at the top
            const _Float16 sum = __builtin_bit_cast(_Float16, old_out[(j - tt) / T]) + (_Float16)total;
            Cout[(size_t)(m0 + m) * C::N + row] = __builtin_bit_cast(uint16_t, sum);
        }
#else
        if (row < C::N && m0 + m < m_total) store_out(Cout + (size_t)(m0 + m) * C::N + row, total);
#endif
    }
}

// Host launcher: static validity checks (return 1 and say why on stderr), then the launch.
template <class C>
int gemv_launch(const void* A, const void* W, void* Cout, const void* S, const void* Zp, int m,
                hipStream_t stream, NormArgs norm = NormArgs{}) {
    const char* why = nullptr;
    if (C::NBITS != 2 && C::NBITS != 3 && C::NBITS != 4 && C::NBITS != 8) why = "NBITS must be 2, 3, 4 or 8";
    else if (C::VB != 4 && C::VB != 8 && C::VB != 16) why = "VB must be 4, 8 or 16";
    else if (C::NBITS == 3 && C::VB < 8) why = "3-bit rows need VB >= 8 (a whole word of the 1-bit plane per chunk)";
    else if ((C::K * C::PB) % (8 * C::VB) != 0) why = "a packed row (main plane) must be a multiple of VB bytes";
    else if (C::QPARAM && (C::GS <= 0 || C::K % C::GS != 0)) why = "GS must divide K";
    else if (C::QPARAM && C::GS % C::EPC != 0) why = "a VB-byte chunk must lie inside one group";
    else if (C::QPARAM && !C::SYM && (C::G % (8 / C::ZFB)) != 0) why = "K/GS must fill whole zero-point bytes";
    else if ((C::V & (C::V - 1)) != 0 || C::V > 64) why = "U*MT must be a power of two <= 64";
    else if (C::THREADS > 1024) why = "block too large";
    else if (QF_GEMV_GATE_UP_SILU && (C::N % 2 != 0 || C::U % 2 != 0)) why = "gate+up rows come in pairs: N and U must be even";
    else if (QF_GEMV_GATE_UP_SILU && (QF_IN_BF16 || QF_OUT_BF16)) why = "the SwiGLU epilogue is fp16 only";
    else if (QF_GEMV_SMEM_QUANT && QF_GEMV_GATE_UP_SILU) why = "scales through LDS need a block's rows contiguous: not with the gate+up row order";
    else if (QF_GEMV_SMEM_QUANT && C::QPARAM && ((C::N * C::G * 2) % 4 != 0 || (!C::SYM && (C::N * C::ZRB) % 4 != 0 )|| (C::RPB * C::G * 2) % 4 != 0 || (!C::SYM && (C::RPB * C::ZRB) % 4 != 0)))
        why = "scales through LDS: a block's scales and zero-points must be whole 32-bit words";
    else if (QF_GEMV_SMEM_QUANT && C::QPARAM && (size_t)C::RPB * C::G * 2 + (size_t)C::RPB * C::ZRB + sizeof(float) * C::WN * C::WK * C::STEPS * C::V > 64 * 1024) why = "scales through LDS exceed LDS";
    else if (C::WN * C::WK * C::STEPS * C::V * 4 > 64 * 1024) why = "reduction scratch exceeds LDS";
    else if (QF_GEMV_NORM_PROLOGUE && (QF_IN_BF16 || QF_OUT_BF16)) why = "the norm prologue is fp16 only";
    else if (QF_OUT_ACCUMULATE && (QF_OUT_BF16 || QF_GEMV_GATE_UP_SILU)) why = "adding to the output is fp16 only and not combined with the SwiGLU epilogue";
    else if (QF_GEMV_NORM_PROLOGUE && norm.gamma == nullptr) why = "an object with the norm prologue is called through launch_norm (RMSNorm weight missing)";
    else if (!QF_GEMV_NORM_PROLOGUE && norm.gamma != nullptr) why = "this object was compiled without the norm prologue";
    else if (QF_GEMV_NORM_PROLOGUE && (norm.x_out == A || (norm.x_out != nullptr && norm.x_out == norm.delta))) why = "x_out must be a buffer of its own: other blocks still read x and delta";
    if (why) {
        fprintf(stderr, "qfactory gemv: invalid configuration: %s (NBITS=%d GS=%d N=%d K=%d MT=%d WK=%d WN=%d U=%d STEPS=%d VB=%d)\n",
                why, C::NBITS, C::GS, C::N, C::K, C::MT, C::WK, C::WN, C::U, C::STEPS, C::VB);
        return 1;
    }
    if (m <= 0) return 0;
    dim3 grid(C::GRID_X, (m + C::MT - 1) / C::MT);
    hipLaunchKernelGGL(gemv_kernel<C>, grid, dim3(C::THREADS), 0, stream, (const uint16_t*)A, (const uint8_t*)W,
                       (uint16_t*)Cout, (const uint16_t*)S, (const uint8_t*)Zp, m, norm);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        fprintf(stderr, "qfactory gemv: launch failed: %s\n", hipGetErrorString(err));
        return 2;
    }
    return 0;
}

}  // namespace qf
