// Dequant-fused low-bit GEMM for large M on the gfx950 matrix cores (v_mfma_f32_32x32x16_f16).
//
//   C[m][n] = fp16( sum_k A[m][k] * DQ[n][k] ),   DQ[n][k] = fp16_rn((q[n][k] - Z[n][k/GS]) * s[n][k/GS])
//
// Same packed operands and semantics as the reference's kernel_gptq in eager-decode mode
// (qfactory/include/gptq_gemv.h:14-154, utils.h:46-81).  The reference has no matrix-core path
// (its M is a register-array size, gptq_gemv.h:34); this tiling is this project's own.
//
//   * Block tile BM x BN, K-iterations of BK; WM x WN waves, each owning a (BM/WM) x (BN/WN)
//     register tile of 32x32 MFMA accumulators.
//   * Packed weights travel global -> registers -> LDS in "supers" of 128 bytes per row (eight
//     lanes share a row: fully coalesced), one super every 1024/NBITS/BK iterations, loaded about
//     two supers ahead of use; the scales and zero-points of the super ride along.
//   * Weights are dequantised ONCE per block, from the packed LDS copy into the fp16 LDS tile: a
//     thread takes 16 packed bytes of one row (128/NBITS fields inside one group), decodes them
//     with the in-place-mask trick, brings them to the exact q - Z with one packed fp16 add/fma
//     and scales with one packed fp16 multiply (bit-identical to the reference's dequantised
//     weight).  Activations are staged in LDS as they are, through a register ring.
//   * Both operands are read from LDS in MFMA fragment order with ds_read_b128 (rows padded by
//     16 bytes: conflict-free).  Weights are MFMA source A (rows = n), activations source B
//     (columns = m): a lane ends with groups of four consecutive n of one m -> 8-byte stores.
//   * LDS is double-buffered, one barrier per K-iteration; the dequantisation of tile i+1 is
//     interleaved with the MFMAs of tile i.
//   * KS > 1 splits K over blocks (grid.z).  Every block writes its fp32 partial tile to a
//     workspace, then takes a ticket; the last block to arrive adds the other partials to its
//     registers and writes the fp16 result.  Nobody spins.
#pragma once

#include <cstdio>
#include "qf_dequant.hip.h"

// Timing experiments (results are wrong when non-zero): bit 0 skips the dequant arithmetic, bit 1 the
// activation loads, bit 2 the MFMAs, bit 3 the LDS fragment reads, bit 4 the per-iteration barrier,
// bit 5 the weight/scale/zero loads, bit 6 the split-K reduction (every split stores its own partial).
#ifndef QF_GEMM_EXPERIMENT
#define QF_GEMM_EXPERIMENT 0
#endif

namespace qf {

template <int NBITS_, int GS_, bool SYM_, int N_, int K_, int BM_, int BN_, int BK_, int WM_, int WN_, int KS_, int PA_, bool NT_B_>
struct GemmCfg {
    static constexpr int NBITS = NBITS_, GS = GS_, N = N_, K = K_;
    static constexpr bool SYM = SYM_, NT_B = NT_B_;
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_, KS = KS_;
    static constexpr int PA = PA_;                             // activation tiles in flight (register ring)
    static constexpr int T = 64 * WM * WN;
    static constexpr int TM = BM / WM, TN = BN / WN;          // wave tile
    static constexpr int MT32 = TM / 32, NT32 = TN / 32;
    static constexpr int KPER = K / KS;                        // K range of one split
    static constexpr int ITERS = KPER / BK;
    static constexpr int EPL = 128 / NBITS;                    // fields in one 16-byte unit
    static constexpr int UPRW = BK / EPL;                      // weight units per row and iteration
    static constexpr int WUNITS = BN * UPRW;
    static constexpr int UW = WUNITS / T;                      // weight units per thread (exact)
    static constexpr int AUNITS = BM * (BK / 8);
    static constexpr int UA = AUNITS / T;                      // activation units per thread (exact)
    static constexpr int PITCH = BK + 8;                       // LDS row pitch in halves
    static constexpr int RB = K * NBITS / 8;
    static constexpr int G = K / GS;
    static constexpr int ZRB = G * NBITS / 8;
    static constexpr int GRID_X = (N + BN - 1) / BN;
    // packed weights travel global -> registers -> LDS in "supers" of 128 bytes per row (fully
    // coalesced: 8 lanes per row), SUP K-iterations each; scales / zero-points ride along
    static constexpr int SUPK = 128 * 8 / NBITS;               // elements of K per super
    static constexpr int SUP = SUPK / BK;                      // iterations per super
    static constexpr int NSUP = (KPER + SUPK - 1) / SUPK;
    static constexpr int UPS = BN * 8 / T;                     // packed 16-byte units per thread and super
    static constexpr int NGS = SUPK / GS > 0 ? SUPK / GS : 1;  // groups per row and super
    static constexpr int US = (BN * NGS + T - 1) / T;          // scale (and zero) loads per thread and super
    static constexpr int WP_PITCH = 128 + 16;
    static constexpr size_t LDS_TILES = (size_t)2 * (BM + BN) * PITCH * 2;
    static constexpr size_t LDS_PACKED = (size_t)2 * BN * WP_PITCH;
    static constexpr size_t LDS_SCALES = (size_t)2 * BN * NGS * 2;
    static constexpr size_t LDS_ZEROS = (size_t)2 * BN * NGS;
    static constexpr size_t LDS_BYTES = LDS_TILES + LDS_PACKED + LDS_SCALES + ((LDS_ZEROS + 15) / 16) * 16;
    static constexpr int ACC_PER_THREAD = MT32 * NT32 * 16;
};

template <class C>
__global__ __launch_bounds__(C::T) void gemm_kernel(
    const uint16_t* __restrict__ A, const uint8_t* __restrict__ W, uint16_t* __restrict__ Cout,
    const uint16_t* __restrict__ S, const uint8_t* __restrict__ Zp, int m_total,
    float* __restrict__ ws, unsigned int* __restrict__ counters) {
    constexpr int BM = C::BM, BN = C::BN, BK = C::BK, WN = C::WN;
    constexpr int MT32 = C::MT32, NT32 = C::NT32, PITCH = C::PITCH;
    constexpr int EPL = C::EPL, UPRW = C::UPRW, UW = C::UW, UA = C::UA;
    constexpr int P8 = 8 / C::NBITS;
    constexpr uint32_t ZMASK = (1u << C::NBITS) - 1u;
    constexpr int KSTEPS = BK / 16;
    constexpr int WSTEPS = EPL / 8;                            // 8-field words per weight unit

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint16_t* As = reinterpret_cast<uint16_t*>(smem);                          // [2][BM][PITCH]
    uint16_t* Ws = As + (size_t)2 * BM * PITCH;                                 // [2][BN][PITCH]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wn = wave % WN, wm = wave / WN;
    const int li = lane & 31, kb = lane >> 5;

    const int n_blk = blockIdx.x * BN;
    const int m_blk = blockIdx.y * BM;
    const int k_blk = blockIdx.z * C::KPER;

    uint8_t* Wp = smem + C::LDS_TILES;                                          // [2][BN][WP_PITCH] packed
    uint16_t* Ss = reinterpret_cast<uint16_t*>(Wp + C::LDS_PACKED);             // [2][BN][NGS]
    uint8_t* Zs = reinterpret_cast<uint8_t*>(Ss) + C::LDS_SCALES;               // [2][BN][NGS] zero-point values

    constexpr int SUP = C::SUP, UPS = C::UPS, NGS = C::NGS, US = C::US, WPP = C::WP_PITCH;

    // ---- activations: UA 16-byte units per thread and iteration, register ring of depth PA ----
    struct AStage { u32x4 a[UA]; };
    auto load_a = [&](AStage& st, int it) {
        const int k0 = k_blk + it * BK;
#pragma unroll
        for (int p = 0; p < UA; p++) {
            const int u = tid + p * C::T;
            const int row = u / (BK / 8), col = (u % (BK / 8)) * 8;
            const int m = min(m_blk + row, m_total - 1);
            if (!(QF_GEMM_EXPERIMENT & 2)) st.a[p] = *reinterpret_cast<const u32x4*>(A + (size_t)m * C::K + k0 + col);
        }
    };
    auto store_a = [&](const AStage& st, int buf) {
#pragma unroll
        for (int p = 0; p < UA; p++) {
            const int u = tid + p * C::T;
            const int row = u / (BK / 8), col = (u % (BK / 8)) * 8;
            *reinterpret_cast<u32x4*>(As + ((size_t)buf * BM + row) * PITCH + col) = st.a[p];
        }
    };

    // ---- packed weights, scales and zero-points of one super: coalesced loads into registers ... ----
    struct PStage { u32x4 w[UPS]; uint32_t s[US]; uint32_t z[US]; };
    auto load_super = [&](PStage& st, int sup) {
        const int k0 = k_blk + sup * C::SUPK;
#pragma unroll
        for (int p = 0; p < UPS; p++) {
            const int u = tid + p * C::T;
            const int n = min(n_blk + u / 8, C::N - 1);
            // the last super of a K range may be shorter than 128 bytes: clamp inside the row
            const int byte = min(k0 * C::NBITS / 8 + (u % 8) * 16, C::RB - 16);
            const uint8_t* wp = W + (size_t)n * C::RB + byte;
            if (!(QF_GEMM_EXPERIMENT & 32)) st.w[p] = C::NT_B ? __builtin_nontemporal_load((const u32x4*)wp) : *(const u32x4*)wp;
        }
#pragma unroll
        for (int p = 0; p < US; p++) {
            const int u = min(tid + p * C::T, BN * NGS - 1);
            const int n = min(n_blk + u / NGS, C::N - 1);
            const int g = min(k0 / C::GS + u % NGS, C::G - 1);
            if (!(QF_GEMM_EXPERIMENT & 32)) {
                st.s[p] = S[(size_t)n * C::G + g];
                if constexpr (!C::SYM) st.z[p] = (uint32_t)(Zp[(size_t)n * C::ZRB + g / P8] >> ((g % P8) * C::NBITS)) & ZMASK;
            }
        }
    };
    // ... and from registers into LDS buffer `sbuf`
    auto store_super = [&](const PStage& st, int sbuf, int sup) {
        const int k0 = k_blk + sup * C::SUPK;
#pragma unroll
        for (int p = 0; p < UPS; p++) {
            const int u = tid + p * C::T;
            // when the load was clamped to the row end, the data sits at the matching offset
            const int want = k0 * C::NBITS / 8 + (u % 8) * 16;
            const int got = min(want, C::RB - 16);
            const int off = (u % 8) * 16 - (want - got);
            if (off >= 0) *reinterpret_cast<u32x4*>(Wp + ((size_t)sbuf * BN + u / 8) * WPP + off) = st.w[p];
        }
#pragma unroll
        for (int p = 0; p < US; p++) {
            const int u = min(tid + p * C::T, BN * NGS - 1);
            Ss[(size_t)sbuf * BN * NGS + u] = (uint16_t)st.s[p];
            if constexpr (!C::SYM) Zs[(size_t)sbuf * BN * NGS + u] = (uint8_t)st.z[p];
        }
    };
    // dequantise word `t` (8 fields) of this thread's weight units of tile `it` (iteration q of
    // the super held in LDS buffer `sbuf`) and store fp16 to the tile buffer `buf`
    auto dequant_store = [&](int buf, int sbuf, int it, int q, int t) {
        const int k0 = k_blk + it * BK;
        const int g0 = (k_blk + (it / SUP) * C::SUPK) / C::GS;
#pragma unroll
        for (int p = 0; p < UW; p++) {
            const int u = tid + p * C::T;
            const int row = u / UPRW, col = u % UPRW;
            const int gi = min((k0 + col * EPL) / C::GS, C::G - 1) - g0;
            const uint32_t sbits = Ss[((size_t)sbuf * BN + row) * NGS + gi];
            const uint32_t zero = C::SYM ? (1u << (C::NBITS - 1)) : (uint32_t)Zs[((size_t)sbuf * BN + row) * NGS + gi];
            const QConst qc = make_qconst<C::NBITS>((uint16_t)sbits, zero);
            const u32x4 wv = *reinterpret_cast<const u32x4*>(Wp + ((size_t)sbuf * BN + row) * WPP + (q * UPRW + col) * 16);
            const uint32_t w4[4] = {wv.x, wv.y, wv.z, wv.w};
            f16x8 v;
            if (QF_GEMM_EXPERIMENT & 1) v = __builtin_bit_cast(f16x8, wv);
            else v = DequantStep<C::NBITS>::run(w4, t, qc);
            *reinterpret_cast<f16x8*>(Ws + ((size_t)buf * BN + row) * PITCH + col * EPL + t * 8) = v;
        }
    };

    f32x16 acc[NT32][MT32];
#pragma unroll
    for (int j = 0; j < NT32; j++)
#pragma unroll
        for (int i = 0; i < MT32; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[j][i][v] = 0.0f;

    const uint16_t* a_frag_base = As + ((size_t)wm * C::TM + li) * PITCH + kb * 8;
    const uint16_t* w_frag_base = Ws + ((size_t)wn * C::TN + li) * PITCH + kb * 8;

    // One K-iteration `it` (s = it % (2*SUP) is a compile-time constant at every call site):
    //   * MFMAs on tile buffer it%2;
    //   * tile it+1 is prepared in the other tile buffer: activations from the register ring (loaded
    //     PA-1 iterations ago), weights dequantised from the packed super in LDS;
    //   * q == 0:      the loads of super P+2 go into the register slot super P has vacated;
    //   * q == SUP-2:  super P+1 (loaded about 2*SUP-2 iterations ago) moves from registers to LDS.
    AStage ringA[C::PA];
    PStage ringP[2];
    auto iteration = [&](int it, int s) {
        const int buf = it & 1;
        const int q = s % SUP, pslot = s / SUP;
        const int P = it / SUP;
        load_a(ringA[s % C::PA], min(it + C::PA, C::ITERS - 1));
        if (q == 0) load_super(ringP[pslot], min(P + 2, C::NSUP - 1));
        const AStage& na = ringA[(s + 1) % C::PA];
        const int nq = (s + 1) % SUP, nsbuf = ((s + 1) / SUP) & 1;      // super position of tile it+1
#pragma unroll
        for (int ks = 0; ks < KSTEPS; ks++) {
            f16x8 wf[NT32], af[MT32];
#pragma unroll
            for (int j = 0; j < NT32; j++) {
                if ((QF_GEMM_EXPERIMENT & 8) && (ks > 0 || it > 0)) wf[j] = __builtin_bit_cast(f16x8, na.a[0]);
                else wf[j] = *reinterpret_cast<const f16x8*>(w_frag_base + ((size_t)buf * BN + j * 32) * PITCH + ks * 16);
            }
#pragma unroll
            for (int i = 0; i < MT32; i++) {
                if ((QF_GEMM_EXPERIMENT & 8) && (ks > 0 || it > 0)) af[i] = __builtin_bit_cast(f16x8, na.a[0]);
                else af[i] = *reinterpret_cast<const f16x8*>(a_frag_base + ((size_t)buf * BM + i * 32) * PITCH + ks * 16);
            }
#pragma unroll
            for (int j = 0; j < NT32; j++)
#pragma unroll
                for (int i = 0; i < MT32; i++) {
                    if (QF_GEMM_EXPERIMENT & 4) acc[j][i][0] += (float)wf[j][0] * (float)af[i][0];
                    else acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[j], af[i], acc[j][i], 0, 0, 0);
                }
            // staging work for the next tile is spread over the k-steps so that it runs in the
            // shadow of the MFMAs just issued (on the last iteration it restages the clamped last
            // tile into the idle buffer: wasted work, but the loop body has no data-dependent branch)
#pragma unroll
            for (int t = ks * WSTEPS / KSTEPS; t < (ks + 1) * WSTEPS / KSTEPS; t++)
                dequant_store(buf ^ 1, nsbuf, min(it + 1, C::ITERS - 1), nq, t);
            if (ks == KSTEPS - 1) store_a(na, buf ^ 1);
        }
        if (q == SUP - 2) store_super(ringP[pslot ^ 1], (pslot ^ 1), min(P + 1, C::NSUP - 1));
        if (!(QF_GEMM_EXPERIMENT & 16)) __syncthreads();
    };

    // ---- prologue: supers 0 and 1 and activation tiles 0 .. PA-1 in flight; super 0 and tile 0 into LDS ----
    load_super(ringP[0], 0);
    load_super(ringP[1], min(1, C::NSUP - 1));
#pragma unroll
    for (int p = 0; p < C::PA; p++) load_a(ringA[p], min(p, C::ITERS - 1));
    store_super(ringP[0], 0, 0);
    store_a(ringA[0], 0);
    __syncthreads();
#pragma unroll
    for (int t = 0; t < WSTEPS; t++) dequant_store(0, 0, 0, 0, t);
    __syncthreads();

#pragma unroll 1
    for (int it0 = 0; it0 < C::ITERS; it0 += 2 * SUP) {
#pragma unroll
        for (int s = 0; s < 2 * SUP; s++)
            if (it0 + s < C::ITERS) iteration(it0 + s, s);
    }

    // ---- split-K: park the partial tile, take a ticket, the last arriver sums ----
    if constexpr (C::KS > 1 && !(QF_GEMM_EXPERIMENT & 64)) {
        const int tile_id = blockIdx.y * gridDim.x + blockIdx.x;
        float* my = ws + ((size_t)tile_id * C::KS + blockIdx.z) * ((size_t)C::T * C::ACC_PER_THREAD);
#pragma unroll
        for (int j = 0; j < NT32; j++)
#pragma unroll
            for (int i = 0; i < MT32; i++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const f32x4 v = f32x4{acc[j][i][4 * q], acc[j][i][4 * q + 1], acc[j][i][4 * q + 2], acc[j][i][4 * q + 3]};
                    *reinterpret_cast<f32x4*>(my + ((size_t)((j * MT32 + i) * 4 + q) * C::T + tid) * 4) = v;
                }
        if (!(QF_GEMM_EXPERIMENT & 128)) __threadfence();
        __syncthreads();
        __shared__ unsigned int ticket_s;
        if (tid == 0) ticket_s = __hip_atomic_fetch_add(&counters[tile_id], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (ticket_s != C::KS - 1) return;
        if (!(QF_GEMM_EXPERIMENT & 128)) __threadfence();
#pragma unroll 1
        for (int z = 0; z < C::KS; z++) {
            if (z == (int)blockIdx.z) continue;
            const float* other = ws + ((size_t)tile_id * C::KS + z) * ((size_t)C::T * C::ACC_PER_THREAD);
#pragma unroll
            for (int j = 0; j < NT32; j++)
#pragma unroll
                for (int i = 0; i < MT32; i++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const f32x4 v = *reinterpret_cast<const f32x4*>(other + ((size_t)((j * MT32 + i) * 4 + q) * C::T + tid) * 4);
#pragma unroll
                        for (int e = 0; e < 4; e++) acc[j][i][4 * q + e] += v[e];
                    }
        }
        if (tid == 0) counters[tile_id] = 0;               // ready for the next launch
    }

    // ---- store: accumulator register v of a 32x32 tile is (n = 8*(v/4) + 4*(lane/32) + v%4, m = lane%32) ----
#pragma unroll
    for (int i = 0; i < MT32; i++) {
        const int m = m_blk + wm * C::TM + i * 32 + li;
        if (m >= m_total) continue;
#pragma unroll
        for (int j = 0; j < NT32; j++) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int n = n_blk + wn * C::TN + j * 32 + 8 * q + 4 * kb;
                uint16_t h[4];
#pragma unroll
                for (int e = 0; e < 4; e++) h[e] = f32_to_f16_bits(acc[j][i][4 * q + e]);
                uint16_t* dst = Cout + (size_t)m * C::N + n;
                if constexpr (C::N % 4 == 0) {
                    if (n < C::N) *reinterpret_cast<u32x2*>(dst) = u32x2{(uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16)};
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (n + e < C::N) dst[e] = h[e];
                }
            }
        }
    }
}

// Split-K scratch: fp32 partial tiles and per-tile tickets.  Owned by the object, grown on demand,
// never freed before the process ends; tickets are zeroed once at allocation and reset by the
// kernel itself.  Calls that overlap on different streams would share it and must not do so.
struct GemmWorkspace {
    float* partials = nullptr;
    unsigned int* counters = nullptr;
    size_t partial_bytes = 0;
    size_t n_counters = 0;
};

template <class C>
int gemm_launch(const void* A, const void* W, void* Cout, const void* S, const void* Zp, int m, hipStream_t stream) {
    const char* why = nullptr;
    if (C::NBITS != 2 && C::NBITS != 4 && C::NBITS != 8) why = "NBITS must be 2, 4 or 8 for this kernel";
    else if (C::BM % (32 * C::WM) != 0 || C::BN % (32 * C::WN) != 0) why = "wave tiles must be multiples of 32";
    else if (C::BK % 16 != 0 || C::BK % C::EPL != 0) why = "BK must be a multiple of 16 and of 128/NBITS";
    else if (C::K % (C::KS * C::BK) != 0) why = "K must be a multiple of KS*BK";
    else if (C::GS <= 0 || C::K % C::GS != 0) why = "GS must divide K";
    else if (C::GS % C::EPL != 0) why = "a 16-byte unit of fields must lie inside one group";
    else if (!C::SYM && (C::G % (8 / C::NBITS)) != 0) why = "K/GS must fill whole zero-point bytes";
    else if (C::T > 1024) why = "block too large";
    else if (C::SUPK % C::BK != 0 || C::SUP < 2) why = "BK must divide 1024/NBITS at least twice";
    else if (C::PA < 2 || (2 * C::SUP) % C::PA != 0) why = "PA must be >= 2 and divide 2*SUP";
    else if ((C::BN * 8) % C::T != 0) why = "packed supers must split evenly over the threads";
    else if (C::GS < C::SUPK && C::SUPK % C::GS != 0) why = "GS must divide 1024/NBITS or be a multiple of it";
    else if (C::GS > C::SUPK && C::GS % C::SUPK != 0) why = "GS must divide 1024/NBITS or be a multiple of it";
    else if (C::KS > 1 && C::KPER % (C::GS < C::SUPK ? C::GS : C::SUPK) != 0) why = "a K split must start on a group / 128-byte boundary";
    else if (C::RB % 16 != 0 || C::RB < 128) why = "a packed row must be a multiple of 16 bytes and at least 128";
    else if (C::WUNITS % C::T != 0 || C::AUNITS % C::T != 0) why = "tiles must split evenly over the threads";
    else if (C::LDS_BYTES > 160 * 1024) why = "tiles exceed the 160 KB of LDS";
    else if (C::ACC_PER_THREAD > 256) why = "accumulator tile exceeds the register file";
    if (why) {
        fprintf(stderr, "qfactory gemm: invalid configuration: %s (NBITS=%d GS=%d N=%d K=%d BM=%d BN=%d BK=%d WM=%d WN=%d KS=%d PA=%d)\n",
                why, C::NBITS, C::GS, C::N, C::K, C::BM, C::BN, C::BK, C::WM, C::WN, C::KS, C::PA);
        return 1;
    }
    if (m <= 0) return 0;
    static bool attr_set = false;
    if (!attr_set && C::LDS_BYTES > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<C>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)C::LDS_BYTES);
        if (e != hipSuccess) {
            fprintf(stderr, "qfactory gemm: cannot reserve %zu bytes of LDS: %s\n", C::LDS_BYTES, hipGetErrorString(e));
            return 2;
        }
        attr_set = true;
    }
    const int grid_y = (m + C::BM - 1) / C::BM;
    static GemmWorkspace wsp;
    if constexpr (C::KS > 1) {
        const size_t tiles = (size_t)C::GRID_X * grid_y;
        const size_t need = tiles * C::KS * C::T * C::ACC_PER_THREAD * sizeof(float);
        if (need > wsp.partial_bytes || tiles > wsp.n_counters) {
            // grow: the old buffers stay allocated (work in flight may still use them)
            float* p = nullptr;
            unsigned int* c = nullptr;
            if (hipMalloc(&p, need) != hipSuccess || hipMalloc(&c, tiles * sizeof(unsigned int)) != hipSuccess ||
                hipMemsetAsync(c, 0, tiles * sizeof(unsigned int), stream) != hipSuccess) {
                fprintf(stderr, "qfactory gemm: cannot allocate %zu bytes of split-K workspace\n", need);
                return 2;
            }
            wsp.partials = p; wsp.counters = c; wsp.partial_bytes = need; wsp.n_counters = tiles;
        }
    }
    dim3 grid(C::GRID_X, grid_y, C::KS);
    hipLaunchKernelGGL(gemm_kernel<C>, grid, dim3(C::T), C::LDS_BYTES, stream, (const uint16_t*)A, (const uint8_t*)W,
                       (uint16_t*)Cout, (const uint16_t*)S, (const uint8_t*)Zp, m, wsp.partials, wsp.counters);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        fprintf(stderr, "qfactory gemm: launch failed: %s\n", hipGetErrorString(err));
        return 2;
    }
    return 0;
}

}  // namespace qf
