// Dequant-fused low-bit GEMM for a few activation rows (M <= 16) on the gfx950 matrix cores, HBM-bound:
// the activations live in LDS, shared by the whole block, and the packed weights stream past them.
//
//   C[m][n] = fp16( sum_g s[n][g] * sum_{k in g} A[m][k] * (q[n][k] - Z[n][g]) )
//
// Same operands as the reference's kernel_gptq (qfactory/include/gptq_gemv.h:14-154) in its deferred-decode
// form (utils.h:193-213); the reference keeps M activation rows in registers per thread and has no
// matrix-core path (gptq_gemv.h:34).  The packed weights are read exactly once, from the reference layout.
//
//   * Persistent blocks, one per CU: block b owns the 16-row weight tiles b, b + grid, ...
//   * A "panel" of the activations -- all (up to 16) rows, KP columns -- is loaded into LDS once and serves
//     every tile of the block: 16 x 4096 fp16 are 128 KB.  Longer K runs panel after panel; the partial 16 x 16
//     tiles then wait in LDS between panels.  No wave keeps activations in registers, so sixteen waves with
//     several tiles of weight loads in flight each fit a CU.
//   * The WV waves of a block split the K range of a panel between them in chunks of 64 packed bytes per row
//     (512/NBITS elements): a wave-wide load takes 16 rows x 64 bytes (four lanes per row), reaches MFMA
//     fragment order by a lane permutation through the LDS crossbar (ds_bpermute, no LDS memory), and every
//     lane dequantises the 128/NBITS fields of its own fragment: masked in place (1024 + 2^o q), brought to
//     the exact integer q - Z with one packed fp16 add or fma, summed per group on the matrix core
//     (v_mfma_f32_16x16x32_f16, activations source A = rows m, weights source B = columns n) and scaled once
//     per chunk in fp32.  Groups narrower than a chunk are scaled per element in fp16 first (eager).
//   * The loads of D tiles are in flight per wave (a ring of register stages, statically indexed; the waits
//     are the compiler's own vmcnt bookkeeping).
//   * Per tile the WV partial 16 x 16 tiles meet in LDS (two alternating sets of slots, one barrier per tile)
//     and every output element is written once, in a fixed order of summation: results are deterministic.
//     No global workspace, no atomics.
#pragma once

#include <cstdio>
#include "qf_dequant.hip.h"

// Timing experiments (results are wrong when non-zero): bit 0 skips the scale / zero-point loads, bit 1 the
// activation fragment reads from LDS, bit 2 the lane permutation of the packed words, bit 3 the dequantisation and
// the MFMAs, bit 4 the cross-wave sum and the stores (the barrier stays), bit 5 the weight loads.
#ifndef QF_PANEL_EXPERIMENT
#define QF_PANEL_EXPERIMENT 0
#endif
#if QF_PANEL_EXPERIMENT != 0 && !defined(QF_ALLOW_TIMING_EXPERIMENTS)
#error "QF_PANEL_EXPERIMENT gives wrong results: timing builds only (define QF_ALLOW_TIMING_EXPERIMENTS)"
#endif

// 1: scales and zero-points through LDS where the geometry allows (see PanelCfg::QSTAGE); 0: every lane loads its own.
#ifndef QF_PANEL_QSTAGE
#define QF_PANEL_QSTAGE 1
#endif

namespace qf {

template <int V> struct PanelTag { static constexpr int value = V; };
template <int I, int N, class F>
__device__ __forceinline__ void panel_static_for(F&& f) {
    if constexpr (I < N) {
        f(PanelTag<I>{});
        panel_static_for<I + 1, N>(f);
    }
}

// Wait for this wave's LDS operations (not for its global loads, which stay in flight), then meet the other
// waves of the block.
__device__ __forceinline__ void panel_lds_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xC07F);          // vmcnt 63 (no wait), expcnt 7 (no wait), lgkmcnt 0
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

template <int NBITS_, int GS_, bool SYM_, int N_, int K_, int WV_, int D_, int KP_, int PB_, bool NT_B_>
struct PanelCfg {
    static constexpr int NBITS = NBITS_, GS = GS_, N = N_, K = K_;
    static constexpr bool SYM = SYM_, NT_B = NT_B_;
    static constexpr int WV = WV_;                 // waves per block, splitting the K range of a panel
    static constexpr int D = D_;                   // tiles whose loads are in flight per wave
    static constexpr int KP = KP_;                 // activation columns per panel
    static constexpr int PB = PB_;                 // upper bound on blocks
    static constexpr int EPL = 128 / NBITS;        // fields per lane and 16 packed bytes
    static constexpr int KSTEPS = EPL / 8;         // MFMA k-steps per chunk
    static constexpr int CHUNK = 4 * EPL;          // elements of K in 64 packed bytes of a row
    static constexpr int NCH = K / CHUNK;          // chunks per row
    static constexpr int PCH = KP / CHUNK;         // chunks per panel
    static constexpr int NPANEL = (NCH + PCH - 1) / PCH;
    static constexpr int CPW = (PCH + WV - 1) / WV;            // chunks per wave, tile and panel
    static constexpr int THREADS = 64 * WV;
    static constexpr int NT = (N + 15) / 16;       // 16-row weight tiles
    static constexpr int GRID_X = NT < PB ? NT : PB;
    static constexpr int SLOTS = (NT + GRID_X - 1) / GRID_X;   // tiles per block
    static constexpr int NSTAGE = NPANEL * SLOTS;  // (panel, tile) pairs a block works through, in this order
    static constexpr int RB = K * NBITS / 8;
    static constexpr int G = K / GS;
    static constexpr int ZRB = G * NBITS / 8;
    static constexpr bool EAGER = (GS % CHUNK) != 0;           // a chunk spans several groups: scale per element
    // One activation row of a panel in LDS.  No padding: the 16-byte unit u of row m sits at position u ^ m, so the
    // sixteen lanes that read the same unit of sixteen different rows hit sixteen different bank groups.
    static constexpr int A_PITCH = KP * 2;
    // Scales and zero-points of a (panel, tile) pair: 16 rows x the panel's groups.  When they are whole 32-bit words
    // per row the block fetches them with one coalesced word per thread, a stage ahead, and lanes read them from LDS
    // (QSTAGE); a lane loading its own row's values -- sixteen rows per wave-wide load, nothing to coalesce --
    // measured several times slower per load.
    static constexpr int PG = KP / GS;             // groups per panel (QSTAGE needs whole groups)
    static constexpr int SW = PG / 2;              // 32-bit words of scales per row and panel
    static constexpr int ZB = PG * NBITS / 8;      // bytes of zero-points per row and panel
    static constexpr int QT = 16 * (SW + (SYM ? 0 : ZB));      // threads that fetch one item each: a scale word or a zero byte
    static constexpr int QWORDS = 16 * SW + (16 * ZB + 3) / 4; // LDS words of one quantisation buffer
    static constexpr bool QSTAGE = QF_PANEL_QSTAGE && KP % GS == 0 && PG % 2 == 0 && G % 2 == 0 && (PG * NBITS) % 8 == 0 &&
                                   QT <= 64 * WV && D >= 2;
    static constexpr size_t LDS_A = (size_t)16 * A_PITCH;
    static constexpr size_t LDS_CT = NPANEL > 1 ? (size_t)SLOTS * 1024 : 0;    // partial tiles between panels
    static constexpr size_t LDS_Q = QSTAGE ? (size_t)2 * QWORDS * 4 : 0;       // two alternating quantisation buffers
    // Partial-tile slots of the WV waves: two alternating sets (one barrier per tile) when LDS has the room, else one
    // set and a second barrier per tile (16 rows x 4096 columns of activations fill 128 of the 160 KB).
    static constexpr int SETS = (LDS_A + LDS_CT + LDS_Q + (size_t)2 * WV * 1024 <= 160 * 1024) ? 2 : 1;
    static constexpr size_t LDS_RED = (size_t)SETS * WV * 1024;
    static constexpr size_t LDS_BYTES = LDS_A + LDS_RED + LDS_CT + LDS_Q;
};

template <class C>
__global__ __launch_bounds__(C::THREADS) void panel_kernel(
    const uint16_t* __restrict__ A, const uint8_t* __restrict__ W, uint16_t* __restrict__ Cout,
    const uint16_t* __restrict__ S, const uint8_t* __restrict__ Zp, int m_total) {
    constexpr int WV = C::WV, D = C::D, CPW = C::CPW, PCH = C::PCH, NPANEL = C::NPANEL, SLOTS = C::SLOTS;
    constexpr int EPL = C::EPL, KSTEPS = C::KSTEPS, CHUNK = C::CHUNK, NSTAGE = C::NSTAGE;
    constexpr uint32_t ZMASK = (1u << C::NBITS) - 1u;
    constexpr int P8 = 8 / C::NBITS;                               // zero-points per byte

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* panel = smem;                                          // [16][A_PITCH]
    f32x4* red = reinterpret_cast<f32x4*>(smem + C::LDS_A);         // [SETS][WV][64]
    float* ctile = reinterpret_cast<float*>(smem + C::LDS_A + C::LDS_RED);   // [SLOTS][256]
    uint32_t* qbuf = reinterpret_cast<uint32_t*>(smem + C::LDS_A + C::LDS_RED + C::LDS_CT);   // [2][QWORDS]: scales [16][SW], zeros [16][ZW]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);       // wave-uniform: addresses are scalar base + lane offset
    const int r = lane & 15, kb = lane >> 4;
    const int team = blockIdx.x;
    const int m0 = blockIdx.y * 16;

    // ---- one stage: the loads of this wave for one (panel, tile) pair: CPW chunks of 16 rows x 64 bytes, and the
    //      scale / zero-point of this lane's row (r) for the group of each chunk ----
    struct Stage { u32x4 w[CPW]; uint32_t s[CPW]; uint32_t z[CPW]; uint32_t qd; };
    constexpr bool QSTAGE = C::QSTAGE;
    constexpr int SW = C::SW, ZB = C::ZB, QWORDS = C::QWORDS;
    // chunk i of the wave in panel p: its index in the row, clamped into the row (a clamped chunk is loaded, not used)
    auto chunk_of = [&](int p, int i) { return min(p * PCH + wv * CPW + i, C::NCH - 1); };
    auto chunk_live = [&](int p, int i) { return (wv * CPW + i < PCH) && (p * PCH + wv * CPW + i < C::NCH); };
    auto load_stage = [&](Stage& st, int p, int slot) {
        const int tile = min(team + slot * C::GRID_X, C::NT - 1);                    // block-uniform
        const int last = C::N - 1 - tile * 16;                                       // rows past N re-read the last one
        const uint8_t* wrow = W + (size_t)tile * 16 * C::RB;
        const uint32_t woff = (uint32_t)min(lane >> 2, last) * C::RB + (lane & 3) * 16;
        const uint32_t qrow = (uint32_t)(tile * 16 + min(r, last));
        if constexpr (QSTAGE) {
            // word `tid` of the pair's quantisation block, requested ahead of the weights of the same stage: the
            // wait for it, a stage before its use, then leaves those in flight
            st.qd = 0;
            if (tid < C::QT && !(QF_PANEL_EXPERIMENT & 1)) {
                if (tid < 16 * SW) {
                    // a word of two scales; groups past the end of the row (a partial last panel) repeat the first pair
                    const int row = min(tid / SW, last);
                    const int col = (p * C::PG + 2 * (tid % SW) + 1 < C::G) ? tid % SW : 0;
                    st.qd = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint8_t*>(S) +
                                                               ((size_t)(tile * 16 + row) * C::G + p * C::PG) * 2 + col * 4);
                } else {
                    // a byte of zero-points (rows of zero-points need not be word-aligned)
                    const int t2 = tid - 16 * SW;
                    const int row = min(t2 / ZB, last);
                    const int col = ((p * C::PG * C::NBITS) / 8 + t2 % ZB < C::ZRB) ? t2 % ZB : 0;
                    st.qd = Zp[(size_t)(tile * 16 + row) * C::ZRB + (p * C::PG * C::NBITS) / 8 + col];
                }
            }
        }
#pragma unroll
        for (int i = 0; i < CPW; i++) {
            const int ch = chunk_of(p, i);
            const uint8_t* src = wrow + (size_t)ch * 64 + woff;
            if (QF_PANEL_EXPERIMENT & 32) st.w[i] = u32x4{(uint32_t)lane, 1u, 2u, 3u};
            else st.w[i] = C::NT_B ? __builtin_nontemporal_load((const u32x4*)src) : *(const u32x4*)src;
            if (QF_PANEL_EXPERIMENT & 1) { st.s[i] = 0x2000u + i; st.z[i] = 0x77u; continue; }
            if constexpr (QSTAGE) continue;
            const int g = C::EAGER ? (ch * CHUNK + kb * EPL) / C::GS : (ch * CHUNK) / C::GS;
            st.s[i] = *reinterpret_cast<const uint16_t*>(reinterpret_cast<const uint8_t*>(S) + ((size_t)qrow * C::G + g) * 2);
            st.z[i] = 0;
            if constexpr (!C::SYM) st.z[i] = Zp[(size_t)qrow * C::ZRB + g / P8];
        }
    };
    const int frag_src = (4 * r + kb) << 2;                        // ds_bpermute address of the lane holding (row r, piece kb)
    auto to_fragment = [&](const u32x4& v) {
        u32x4 o;
        o.x = (uint32_t)__builtin_amdgcn_ds_bpermute(frag_src, (int)v.x);
        o.y = (uint32_t)__builtin_amdgcn_ds_bpermute(frag_src, (int)v.y);
        o.z = (uint32_t)__builtin_amdgcn_ds_bpermute(frag_src, (int)v.z);
        o.w = (uint32_t)__builtin_amdgcn_ds_bpermute(frag_src, (int)v.w);
        return o;
    };

    // ---- the activation panel p: every thread moves 16-byte units, coalesced, into LDS.  Rows past m_total
    //      repeat the last row (their outputs are never stored). ----
    constexpr int UPR = C::KP / 8;                                 // 16-byte units per panel row
    constexpr int UNITS = 16 * UPR;
    constexpr int UPT = (UNITS + C::THREADS - 1) / C::THREADS;     // units per thread
    auto fill_panel = [&](int p) {
        constexpr int HALF = (UPT + 1) / 2;                        // in two halves: half the registers
#pragma unroll
        for (int h = 0; h < 2; h++) {
            u32x4 v[HALF];
#pragma unroll
            for (int j = 0; j < HALF; j++) {
                const int u = tid + (h * HALF + j) * C::THREADS;
                const int row = min(u / UPR, 15), cu = u % UPR;
                const int mm = min(m0 + row, m_total - 1);
                const int k = min(p * C::KP + cu * 8, C::K - 8);   // columns past K (a partial last panel): repeated, never used
                v[j] = act_unit(*reinterpret_cast<const u32x4*>(A + (size_t)mm * C::K + k));
            }
#pragma unroll
            for (int j = 0; j < HALF; j++) {
                const int u = tid + (h * HALF + j) * C::THREADS;
                if (h * HALF + j < UPT && u < UNITS)
                    *reinterpret_cast<u32x4*>(panel + (u / UPR) * C::A_PITCH + ((u % UPR) ^ (u / UPR)) * 16) = v[j];
            }
        }
    };

    int a_step[KSTEPS];                                            // byte offset of k-step t inside a lane's KSTEPS units
#pragma unroll
    for (int t = 0; t < KSTEPS; t++) a_step[t] = (t ^ (r & (KSTEPS - 1))) * 16;

    // ---- the work of one stage: partial 16 x 16 tile of this wave over its chunks of panel p ----
    auto compute = [&](const Stage& st, int p, int q) {
        f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i = 0; i < CPW; i++) {
            if (!chunk_live(p, i)) continue;                                     // wave-uniform
            const int ch = p * PCH + wv * CPW + i;
            const int g = C::EAGER ? (ch * CHUNK + kb * EPL) / C::GS : (ch * CHUNK) / C::GS;
            uint32_t sbits = st.s[i];
            uint32_t zero = 1u << (C::NBITS - 1);
            if constexpr (QSTAGE && !(QF_PANEL_EXPERIMENT & 1)) {
                const int gl = g - p * C::PG;                                    // group inside the panel
                const uint32_t* qb = qbuf + (q & 1) * QWORDS;
                sbits = reinterpret_cast<const uint16_t*>(qb)[r * (2 * SW) + gl];
                if constexpr (!C::SYM) zero = (reinterpret_cast<const uint8_t*>(qb + 16 * SW)[r * ZB + gl / P8] >> ((g % P8) * C::NBITS)) & ZMASK;
            } else if constexpr (!C::SYM) {
                zero = (st.z[i] >> ((g % P8) * C::NBITS)) & ZMASK;
            }
            const ZConst zc = make_zconst<C::NBITS>(zero);
            const u32x4 wv4 = (QF_PANEL_EXPERIMENT & 4) ? st.w[i] : to_fragment(st.w[i]);
            if (QF_PANEL_EXPERIMENT & 8) { acc[0] += (float)(wv4.x ^ wv4.y ^ wv4.z ^ wv4.w); continue; }
            const uint32_t w4[4] = {wv4.x, wv4.y, wv4.z, wv4.w};
            // k-step t of this lane reads unit base + t of row r, stored at (base + t) ^ r = (base ^ r_hi) + (t ^ r_lo)
            const uint8_t* arow = panel + r * C::A_PITCH + ((((wv * CPW + i) * CHUNK + kb * EPL) / 8) ^ (r & ~(KSTEPS - 1))) * 16;
            if constexpr (C::EAGER) {
                const _Float16 sh = __builtin_bit_cast(_Float16, (uint16_t)sbits);
                const f16x8 s8 = f16x8{sh, sh, sh, sh, sh, sh, sh, sh};
#pragma unroll
                for (int t = 0; t < KSTEPS; t++) {
                    const f16x8 wf = IntStep<C::NBITS>::run(w4, t, zc) * s8;
                    const f16x8 af = (QF_PANEL_EXPERIMENT & 2) ? __builtin_bit_cast(f16x8, u32x4{(uint32_t)t, 1u, 2u, 3u}) : *reinterpret_cast<const f16x8*>(arow + a_step[t]);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af, wf, acc, 0, 0, 0);
                }
            } else {
                f32x4 gsum = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < KSTEPS; t++) {
                    const f16x8 wf = IntStep<C::NBITS>::run(w4, t, zc);
                    const f16x8 af = (QF_PANEL_EXPERIMENT & 2) ? __builtin_bit_cast(f16x8, u32x4{(uint32_t)t, 1u, 2u, 3u}) : *reinterpret_cast<const f16x8*>(arow + a_step[t]);
                    gsum = __builtin_amdgcn_mfma_f32_16x16x32_f16(af, wf, gsum, 0, 0, 0);
                }
                const float sc = f16_bits_to_f32((uint16_t)sbits);
#pragma unroll
                for (int e = 0; e < 4; e++) acc[e] = __builtin_fmaf(sc, gsum[e], acc[e]);
            }
        }
        return acc;
    };

    // ---- the WV partial tiles of (panel p, tile slot) meet in LDS; threads 0 .. 255 own one output each
    //      (m = o / 16, n = o % 16): a partial tile sits in LDS as [lane = n + 16 * (m / 4)][e = m % 4] ----
    auto finish = [&](const f32x4& acc, int p, int slot, int q) {
        f32x4* set = red + (size_t)(C::SETS == 2 ? (q & 1) : 0) * (WV * 64);
        set[wv * 64 + lane] = acc;
        panel_lds_barrier();
        if (tid < 256 && !(QF_PANEL_EXPERIMENT & 16)) {
            const int m = tid >> 4, n = tid & 15;
            const float* src = reinterpret_cast<const float*>(set) + (n + 16 * (m >> 2)) * 4 + (m & 3);
            float total = 0.f;
#pragma unroll
            for (int w2 = 0; w2 < WV; w2++) total += src[w2 * 256];
            if constexpr (NPANEL > 1) {
                if (p > 0) total += ctile[slot * 256 + tid];
                if (p < NPANEL - 1) ctile[slot * 256 + tid] = total;
            }
            const int tile = team + slot * C::GRID_X;
            const int col = tile * 16 + n;
            if (p == NPANEL - 1 && tile < C::NT && col < C::N && m0 + m < m_total)
                Cout[(size_t)(m0 + m) * C::N + col] = f32_to_out_bits(total);
        }
        if constexpr (C::SETS == 1) panel_lds_barrier();            // the one set is free again
    };

    // the quantisation words of stage q go to LDS buffer q % 2 (last read two stages ago, with two barriers since)
    auto publish_quant = [&](const Stage& st, int q) {
        uint32_t* qb = qbuf + (q & 1) * QWORDS;
        if (tid < 16 * SW) qb[tid] = st.qd;
        else if (tid < C::QT) reinterpret_cast<uint8_t*>(qb + 16 * SW)[tid - 16 * SW] = (uint8_t)st.qd;
    };

    // ---- main: stages q = p * SLOTS + slot in order; the loads of stages q + 1 .. q + D - 1 are in flight while q is computed ----
    Stage ring[D];
    panel_static_for<0, (D - 1 < NSTAGE ? D - 1 : NSTAGE)>([&](auto q_tag) {
        constexpr int q = decltype(q_tag)::value;
        load_stage(ring[q % D], q / SLOTS, q % SLOTS);
    });
    panel_static_for<0, NSTAGE>([&](auto q_tag) {
        constexpr int q = decltype(q_tag)::value;
        constexpr int p = q / SLOTS, slot = q % SLOTS;
        if constexpr (slot == 0) {
            if constexpr (p > 0) panel_lds_barrier();               // every wave has finished reading the previous panel
            fill_panel(p);
            if constexpr (QSTAGE && q == 0) publish_quant(ring[0], 0);
            panel_lds_barrier();
        }
        if constexpr (q + D - 1 < NSTAGE) load_stage(ring[(q + D - 1) % D], (q + D - 1) / SLOTS, (q + D - 1) % SLOTS);
        const f32x4 acc = compute(ring[q % D], p, q);
        if constexpr (QSTAGE && q + 1 < NSTAGE) publish_quant(ring[(q + 1) % D], q + 1);    // visible after the barrier in finish
        finish(acc, p, slot, q);
    });
}

template <class C>
int panel_launch(const void* A, const void* W, void* Cout, const void* S, const void* Zp, int m, hipStream_t stream) {
    const char* why = nullptr;
    if (C::NBITS != 2 && C::NBITS != 4 && C::NBITS != 8) why = "NBITS must be 2, 4 or 8";
    else if (C::WV < 4 || C::WV > 16) why = "4 .. 16 waves per block";
    else if (C::D < 1 || C::D > 8) why = "1 .. 8 tiles in flight";
    else if (C::K % C::CHUNK != 0) why = "K must be a multiple of 512/NBITS";
    else if (C::KP % C::CHUNK != 0 || C::KP % 128 != 0) why = "a panel must be whole chunks of 512/NBITS columns and a multiple of 128";
    else if (C::GS <= 0 || C::K % C::GS != 0) why = "GS must divide K";
    else if (C::GS % C::EPL != 0) why = "a lane's 16 bytes of fields must lie inside one group";
    else if (!C::EAGER && C::GS % C::CHUNK != 0) why = "GS must be a multiple of 512/NBITS or divide it";
    else if (C::EAGER && C::CHUNK % C::GS != 0) why = "GS must be a multiple of 512/NBITS or divide it";
    else if (!C::SYM && (C::G % (8 / C::NBITS)) != 0) why = "K/GS must fill whole zero-point bytes";
    else if (C::NSTAGE > 40) why = "too many (panel, tile) pairs per block for the unrolled schedule";
    else if (C::LDS_BYTES > 160 * 1024) why = "activation panel and partial tiles exceed the 160 KB of LDS";
    else if ((size_t)C::N * C::RB >= ((size_t)1 << 32)) why = "packed weight tensor above 4 GiB";
    if (why) {
        fprintf(stderr, "qfactory panel: invalid configuration: %s (NBITS=%d GS=%d N=%d K=%d WV=%d D=%d KP=%d PB=%d)\n",
                why, C::NBITS, C::GS, C::N, C::K, C::WV, C::D, C::KP, C::PB);
        return 1;
    }
    if (m <= 0) return 0;
    static bool attr_set = false;
    if (!attr_set && C::LDS_BYTES > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&panel_kernel<C>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)C::LDS_BYTES);
        if (e != hipSuccess) {
            fprintf(stderr, "qfactory panel: cannot reserve %zu bytes of LDS: %s\n", C::LDS_BYTES, hipGetErrorString(e));
            return 2;
        }
        attr_set = true;
    }
    dim3 grid(C::GRID_X, (m + 15) / 16);
    hipLaunchKernelGGL(panel_kernel<C>, grid, dim3(C::THREADS), C::LDS_BYTES, stream, (const uint16_t*)A, (const uint8_t*)W,
                       (uint16_t*)Cout, (const uint16_t*)S, (const uint8_t*)Zp, m);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        fprintf(stderr, "qfactory panel: launch failed: %s\n", hipGetErrorString(err));
        return 2;
    }
    return 0;
}

}  // namespace qf
