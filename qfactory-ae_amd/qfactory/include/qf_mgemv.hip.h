// Dequant-fused low-bit "skinny GEMM" on the gfx950 matrix cores for 2 <= M <= 32, HBM-bound.
//
//   C[m][n] = fp16( sum_g s[n][g] * sum_{k in g} A[m][k] * (q[n][k] - Z[n][g]) )
//
// Same operands as the reference's kernel_gptq (qfactory/include/gptq_gemv.h:14-154) in its
// deferred-decode form (utils.h:193-213): the integer part is summed first, the scale is applied
// once per group -- here in fp32 and on the matrix cores.  Organised like qf::gemv_kernel: the
// packed weights are read exactly once, straight from the reference layout.
//
//   * Persistent blocks: at most PB blocks, each sweeping SLOTS 16-row weight tiles, so the
//     activations are fetched once per block and not once per tile.
//   * A team of WK waves splits K; wave wk owns CH consecutive "chunks" (a chunk is the 4*128/NBITS
//     elements that one 16-byte load per lane covers for 16 weight rows).  The activations of a
//     wave's chunks stay in VGPRs in MFMA fragment order (A-stationary): no LDS staging and no
//     barrier in the main loop.
//   * Per tile: CH 16-byte loads per lane (next tile prefetched); fields are masked in place
//     (1024 + 2^o*q) and brought to the exact integer q - Z with one packed fp16 add or fma;
//     v_mfma_f32_16x16x32_f16 with the activations as source A (rows m) and the weights as source
//     B (columns n), so a lane holds one n and needs one scale: acc += s * group_sum in fp32.
//   * Each wave parks its partial 16x16 tiles in its own LDS slots; one barrier at the end of the
//     block, then the partials of the WK waves are summed and every output is written once.
//   * Long rows (KS > 1): K is also split over KS blocks (a power of two), each holding the activations of its own
//     K/KS only.  Their fp32 sums meet pairwise in a scratch buffer in device memory, one atomic exchange per element
//     and level of a binary tree over the blocks; the result does not depend on who arrives when (see the kernel).
#pragma once

#include <atomic>
#include <cstdio>
#include <mutex>
#include "qf_dequant.hip.h"

// Tiles a block finishes between two reductions through LDS (a multiple of the ring depth PF).
#ifndef QF_MGEMV_SB
#define QF_MGEMV_SB 4
#endif

// 1: the weight matrix is a fused gate+up projection (rows 0 .. N/2-1 gate, the rest up) and the kernel writes
// the (M, N/2) SwiGLU activation fp16(silu(gate)) * up instead of the (M, N) projection: a block's tiles
// alternate between a gate tile and the up tile of the same outputs, and the two meet in the batch's final sum
// (same bits as the projection followed by qf_silu_mul of libqfactory_hip.so).  Not in the reference.
#ifndef QF_MGEMV_GATE_UP_SILU
#define QF_MGEMV_GATE_UP_SILU 0
#endif

// 1: the activations are made, not read: residual add and RMSNorm of the decoder layer run while a block brings
// its activation slices into registers (the roundings of qf_add_rmsnorm in libqfactory_hip.so, which this replaces
// up to 32 rows; same contract as QF_GEMV_NORM_PROLOGUE in qf_gemv.hip.h).  A wave adds the squares of its own K-slice
// per row, the WK waves meet once through LDS; the persistent block does this once for all the tiles it sweeps.
// Block (0, y) also writes x + delta to x_out.  fp16 only.  Not in the reference.
#ifndef QF_MGEMV_NORM_PROLOGUE
#define QF_MGEMV_NORM_PROLOGUE 0
#endif

// 1: a slot past a block's last real tile (it holds the clamped last tile) is computed like any other and never stored;
// 0: its arithmetic is skipped, which puts every tile's arithmetic into a conditional block (see there).
#ifndef QF_MGEMV_COMPUTE_CLAMPED
#define QF_MGEMV_COMPUTE_CLAMPED 1
#endif
// Non-zero: the order in which the first PF weight tiles and the activations are requested is fixed by scheduling
// barriers (1, 2, 3: the orders listed where the loads are issued; measured on sixteen shapes at 4 and 16 rows, 3 is the
// best or level everywhere, 1 - 3.5 % in front of the compiler's own order); 0 leaves the order to the compiler.
#ifndef QF_MGEMV_PIN_FIRST_LOADS
#define QF_MGEMV_PIN_FIRST_LOADS 3
#endif

// Timing experiments (results are wrong when non-zero): bit 0 skips the activation loads, bit 1 the
// dequantisation and MFMAs, bit 2 the cross-wave reduction and the stores (with K split over blocks: the partial sums
// and the meeting of the blocks), bit 3 the weight loads; bit 4 keeps the
// loads and their prefetch order but replaces the hand-off through LDS, the decode and the MFMAs by an XOR of what
// was loaded; bit 5 skips the scale and zero-point loads.
#ifndef QF_MGEMV_EXPERIMENT
#define QF_MGEMV_EXPERIMENT 0
#endif
#if QF_MGEMV_EXPERIMENT != 0 && !defined(QF_ALLOW_TIMING_EXPERIMENTS)
#error "QF_MGEMV_EXPERIMENT gives wrong results: timing builds only (define QF_ALLOW_TIMING_EXPERIMENTS)"
#endif

// Decode strategy (the reference's search dimension, qfactory/core/qfunc.py:85-91).  0: "deferred" wherever a chunk
// lies inside one group (integer sums on the matrix core, one fp32 scale per chunk), "eager" elsewhere.
// 1: "eager" everywhere -- every field becomes fp16_rn((q - Z) * s) before the contraction.
#ifndef QF_MGEMV_EAGER
#define QF_MGEMV_EAGER 0
#endif

namespace qf {

template <int V> struct MgTag { static constexpr int value = V; };
template <class T> struct mg_is_tag { static constexpr bool value = false; };
template <int V> struct mg_is_tag<MgTag<V>> { static constexpr bool value = true; };
template <int I, int N, class F>
__device__ __forceinline__ void mg_static_for(F&& f) {
    if constexpr (I < N) {
        f(MgTag<I>{});
        mg_static_for<I + 1, N>(f);
    }
}

// Scratch memory of a launch that splits K over blocks: per unit and batch of tiles, KS - 1 slots per output element
// in which pairs of blocks exchange their sums, and one nobody reads.  The slots must be zero when a launch starts;
// every launch leaves them zero.  Launches that share one buffer must not overlap in time.
struct MGemvScratch {
    float* partial = nullptr;
};

template <int NBITS_, int GS_, bool SYM_, int N_, int K_, int MT16_, int WK_, int CH_, int PB_, int PF_, bool NT_B_, int KS_ = 1>
struct MGemvCfg {
    static constexpr int NBITS = NBITS_, GS = GS_, N = N_, K = K_;
    static constexpr bool SYM = SYM_, NT_B = NT_B_;
    static constexpr int MT16 = MT16_;             // 16-row activation tiles held per wave
    static constexpr int WK = WK_;                 // waves along K per team
    static constexpr int CH = CH_;                 // chunks per wave
    static constexpr int PB = PB_;                 // upper bound on blocks along N
    static constexpr int PBITS = plane_bits(NBITS);   // 3-bit rows: a 2-bit main plane followed by a 1-bit plane
    static constexpr int ZFB = zero_field_bits(NBITS); // stored width of one zero-point
    static constexpr bool HI = NBITS == 3;
    static constexpr int EPL = 128 / PBITS;        // fields per lane and 16-byte load of the main plane
    static constexpr int KSTEPS = EPL / 8;         // MFMA k-steps per chunk
    static constexpr int CHUNK = 4 * EPL;          // elements of K per chunk
    static constexpr int NCHUNK = K / CHUNK;
    static constexpr int KS = KS_;                 // blocks splitting K (1: a block covers all of K)
    static constexpr int NCHUNK_B = (NCHUNK + KS - 1) / KS;              // chunks of one block
    static constexpr int THREADS = 64 * WK;
    static constexpr int BM = 16 * MT16;
    static constexpr int NT = (N + 15) / 16;       // 16-row weight tiles
    static constexpr bool SILU = QF_MGEMV_GATE_UP_SILU != 0;
    static constexpr int NPAIR = NT / 2;           // gate+up: pairs of a gate tile and its up tile
    static constexpr int NUNIT = SILU ? NPAIR : NT;                        // what the blocks deal among themselves
    static constexpr int GRID_X = NUNIT < PB ? NUNIT : PB;
    static constexpr int SLOTS = (NUNIT + GRID_X - 1) / GRID_X * (SILU ? 2 : 1);   // tiles per block
    static constexpr int PF = PF_;                 // weight tiles in flight per wave (ring of stages): 2 or 4
    // tiles per batch (partials are reduced and stored per batch): no more than the block has
    static constexpr int SB = SLOTS < QF_MGEMV_SB ? (SLOTS + PF - 1) / PF * PF : QF_MGEMV_SB;
    static constexpr int NBATCH = (SLOTS + SB - 1) / SB;
    static constexpr int RB = K * NBITS / 8;
    static constexpr int G = K / GS;
    static constexpr int ZRB = G * ZFB / 8;
    static constexpr int HI_OFF = K / 4;           // byte offset of the 1-bit plane in a 3-bit row
    static constexpr bool DEFERRED = (GS % CHUNK == 0) && !QF_MGEMV_EAGER;   // a chunk lies inside one group
    static constexpr int LPR = CH * 4;             // lanes covering one row's K-slice (CH*64 bytes)
    static constexpr int RPI = 64 / LPR;           // rows per coalesced weight load
    // groups and zero-point bytes of one row inside a wave's K-slice
    // (upper bounds when a slice may start inside a group / inside a byte; indices are clamped to the row)
    static constexpr int GWN = (GS <= CHUNK) ? CH * CHUNK / GS : (CH * CHUNK) / GS + 2;
    static constexpr int ZB = (GWN * ZFB + 7) / 8 + 1;
    // 1-bit plane of a tile: CH*32 bytes per row, loaded 16 bytes per lane
    static constexpr int LPRH = CH * 2;            // lanes per row
    static constexpr int RPIH = 64 / LPRH;         // rows per load (may exceed 16: the extra lanes idle)
    static constexpr int NHI = HI ? (16 + RPIH - 1) / RPIH : 0;
    static constexpr int PITCH_W = CH * 64 + 16;
    static constexpr int PITCH_H = CH * 32 + 16;
    static constexpr int WBUF_W = 16 * PITCH_W + (HI ? 16 * PITCH_H : 0);
    static constexpr int WBUF_A = 16 * (CHUNK * 2 + 16);
    static constexpr int WBUF = WBUF_W > WBUF_A ? WBUF_W : WBUF_A;    // per-wave transposition buffer
    static constexpr size_t LDS_BYTES = (size_t)WK * SB * MT16 * 1024 + (size_t)WK * WBUF;
    // split K: fp32 sums of one block and batch, and what one row block (grid.y) of a launch needs
    static constexpr int PART = SB * MT16 * 256;
    static constexpr size_t SCRATCH_FLOATS = KS > 1 ? (size_t)GRID_X * NBATCH * KS * PART : 0;
    static constexpr size_t SCRATCH_BYTES = (SCRATCH_FLOATS * 4 + 255) / 256 * 256;
};

template <class C>
__global__ __launch_bounds__(C::THREADS) void mgemv_kernel(
    const uint16_t* __restrict__ A, const uint8_t* __restrict__ W, uint16_t* __restrict__ Cout,
    const uint16_t* __restrict__ S, const uint8_t* __restrict__ Zp, int m_total, NormArgs norm, MGemvScratch scratch) {
    constexpr int MT16 = C::MT16, WK = C::WK, CH = C::CH, SLOTS = C::SLOTS, PF = C::PF, SB = C::SB, KS = C::KS;
    constexpr bool NORM = QF_MGEMV_NORM_PROLOGUE != 0;
    constexpr int EPL = C::EPL, KSTEPS = C::KSTEPS, CHUNK = C::CHUNK;
    constexpr int P8 = 8 / C::ZFB;                      // zero-point fields per byte
    constexpr uint32_t ZMASK = (1u << C::ZFB) - 1u;
    constexpr int NHI = C::NHI;
    constexpr bool DEFERRED = C::DEFERRED;
    constexpr int LPR = C::LPR, RPI = C::RPI;            // lanes per row and rows per coalesced weight load
    constexpr int GWN = C::GWN, ZB = C::ZB;              // scales / zero bytes per row in a wave's K-slice
    constexpr int NSI = (16 * GWN + 63) / 64;            // load instructions for the scales of one tile
    constexpr int NZI = (16 * ZB + 63) / 64;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    f32x4* red = reinterpret_cast<f32x4*>(smem);                                    // [WK][SB][MT16][64]
    uint8_t* wbuf = smem + (size_t)WK * SB * MT16 * 1024 + (size_t)(threadIdx.x >> 6) * C::WBUF;   // private to the wave

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wk = tid >> 6;
    const int r = lane & 15, kb = lane >> 4;
    const int m0 = blockIdx.y * C::BM;
    const int team_id = blockIdx.x;
    constexpr int TEAM_STRIDE = C::GRID_X;
    // weight tile of the block's slot: plain, teams deal the tiles round-robin; gate+up, they deal pairs, and
    // slots 2i and 2i + 1 are the gate tile and the up tile of pair i
    auto unit_of = [&](int slot) { return team_id + (C::SILU ? slot >> 1 : slot) * TEAM_STRIDE; };
    auto tile_ok = [&](int slot) { return unit_of(slot) < C::NUNIT; };
    auto tile_clamped = [&](int slot) {
        return min(unit_of(slot), C::NUNIT - 1) + (C::SILU ? (slot & 1) * C::NPAIR : 0);
    };

    // chunks [lo, lo + CH) are read by this wave; it owns [own_from, own_from + CH) (a clamped last
    // wave re-reads chunks of its neighbours with zeroed activations: every address stays in bounds)
    // With K split over KS blocks, block z covers chunks [z NCHUNK_B, own_end).
    const int own_from = (KS > 1 ? (int)blockIdx.z * C::NCHUNK_B : 0) + wk * CH;
    const int own_end = KS > 1 ? min(((int)blockIdx.z + 1) * C::NCHUNK_B, C::NCHUNK) : C::NCHUNK;
    const int lo = max(min(own_from, C::NCHUNK - CH), 0);
    const int gw_lo = (lo * CHUNK) / C::GS;              // first group of the wave's K-slice

    // ---- coalesced loads: LPR consecutive lanes cover one row's K-slice (CH*64 bytes) ----
    struct WStage {
        u32x4 w[CH];                 // load i: row i*RPI + lane/LPR, bytes (lane%LPR)*16 of the slice
        u32x4 h[NHI ? NHI : 1];      // 1-bit plane, load i: row i*RPIH + lane/LPRH, bytes (lane%LPRH)*16
        uint32_t s[NSI];             // lane -> (row, group) = (idx / GWN, idx % GWN), idx = lane + 64*j
        uint32_t z[NZI];             // lane -> (row, byte)  = (idx / ZB,  idx % ZB)
    };
    auto load_tile_words = [&](WStage& st, int tile) {
        if (QF_MGEMV_EXPERIMENT & 8) return;
        const int n_base = tile * 16;
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const int n = min(n_base + i * RPI + lane / LPR, C::N - 1);
            const uint8_t* wp = W + (size_t)n * C::RB + (size_t)lo * 64 + (lane % LPR) * 16;
            st.w[i] = C::NT_B ? __builtin_nontemporal_load((const u32x4*)wp) : *(const u32x4*)wp;
        }
#pragma unroll
        for (int i = 0; i < NHI; i++) {
            const int n = min(n_base + min(i * C::RPIH + lane / C::LPRH, 15), C::N - 1);
            const uint8_t* hp = W + (size_t)n * C::RB + C::HI_OFF + (size_t)lo * 32 + (lane % C::LPRH) * 16;
            st.h[i] = C::NT_B ? __builtin_nontemporal_load((const u32x4*)hp) : *(const u32x4*)hp;
        }
    };
    auto load_tile_quant = [&](WStage& st, int tile) {
        if (QF_MGEMV_EXPERIMENT & 8) return;
        const int n_base = tile * 16;
        if (QF_MGEMV_EXPERIMENT & 32) {
#pragma unroll
            for (int j = 0; j < NSI; j++) st.s[j] = 0x2000u;
#pragma unroll
            for (int j = 0; j < NZI; j++) st.z[j] = 0x77u;
            return;
        }
#pragma unroll
        for (int j = 0; j < NSI; j++) {
            const int idx = lane + 64 * j;
            const int n = min(n_base + min(idx / GWN, 15), C::N - 1);
            st.s[j] = S[(size_t)n * C::G + min(gw_lo + idx % GWN, C::G - 1)];
        }
        if constexpr (!C::SYM) {
#pragma unroll
            for (int j = 0; j < NZI; j++) {
                const int idx = lane + 64 * j;
                const int n = min(n_base + min(idx / ZB, 15), C::N - 1);
                st.z[j] = Zp[(size_t)n * C::ZRB + min((gw_lo * C::ZFB) / 8 + idx % ZB, C::ZRB - 1)];
            }
        }
    };

    auto load_tile = [&](WStage& st, int tile) {
        load_tile_words(st, tile);
        load_tile_quant(st, tile);
    };

    // ring of PF stages: tiles slot .. slot+PF-1 of this team are in flight.  The first PF are requested with the
    // activations, in an order that is kept by scheduling barriers (QF_MGEMV_PIN_FIRST_LOADS): left to itself the
    // compiler issues the first tiles' scale and zero-point loads behind the whole activation phase (they are needed
    // last), and the first MFMA then waits for a second trip to memory that starts only when the activations are in.
    // Loads return in order, so what is requested in front of the activations also delays their hand-over through LDS.
    //   1: packed words, activations, scales and zero-points (the activations' hand-over runs under the latter's latency)
    //   2: whole tiles, then the activations            3: activations, then whole tiles
    WStage ring[PF];
#pragma unroll
    for (int p = 0; p < PF; p++)
        if (p < SLOTS) {
            if (QF_MGEMV_PIN_FIRST_LOADS == 1) load_tile_words(ring[p], tile_clamped(p));
            else if (QF_MGEMV_PIN_FIRST_LOADS != 3) load_tile(ring[p], tile_clamped(p));
        }
#if QF_MGEMV_PIN_FIRST_LOADS
    __builtin_amdgcn_sched_barrier(0);
#endif

    // ---- resident activations, brought into MFMA fragment order through the wave's LDS buffer:
    //      fragment (mt, c, t) = A[m0 + 16*mt + r][(lo+c)*CHUNK + kb*EPL + 8t .. +8] ----
    f16x8 af[MT16][CH][KSTEPS];
    {
        constexpr int ROWB = CHUNK * 2;                  // bytes of one chunk of one activation row
        constexpr int PITCH_A = ROWB + 16;
        constexpr int LPRA = ROWB / 16;                  // lanes per row
        constexpr int RPIA = 64 / LPRA;                  // rows per load (LPRA <= 64)
        // every global load of the slice goes out first (they are independent; issued one by one
        // behind the LDS round trips below they would each expose a full L2 latency), then the
        // chunks pass through the wave's LDS buffer one after another
        constexpr int LPC = 16 / RPIA;                   // loads per chunk
        u32x4 raw[MT16][CH][LPC];
#pragma unroll
        for (int mt = 0; mt < MT16; mt++)
#pragma unroll
            for (int c = 0; c < CH; c++)
#pragma unroll
                for (int i = 0; i < LPC; i++) {
                    const int row = i * RPIA + lane / LPRA;
                    const int m = m0 + 16 * mt + row;
                    const uint16_t* ap = A + (size_t)min(m, m_total - 1) * C::K + (size_t)(lo + c) * CHUNK + (lane % LPRA) * 8;
                    if (QF_MGEMV_EXPERIMENT & 1) raw[mt][c][i] = u32x4{(uint32_t)lane, 1u, 2u, 3u};
                    else raw[mt][c][i] = *reinterpret_cast<const u32x4*>(ap);
                }
#if QF_MGEMV_PIN_FIRST_LOADS
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int p = 0; p < PF; p++)
            if (p < SLOTS) {
                if (QF_MGEMV_PIN_FIRST_LOADS == 1) load_tile_quant(ring[p], tile_clamped(p));
                else if (QF_MGEMV_PIN_FIRST_LOADS == 3) load_tile(ring[p], tile_clamped(p));
            }
        __builtin_amdgcn_sched_barrier(0);
#endif
        if constexpr (NORM) {
            static_assert(!QF_IN_BF16, "the norm prologue is fp16 only");
            // raw[][][] holds the wave's slices of x in load order: lane -> (row i*RPIA + lane/LPRA, 8 elements at
            // (lane%LPRA)*8 of chunk c).  Add delta, keep the sum for x_out, add up the squares per row, normalise.
            u32x4 gam[CH];
#pragma unroll
            for (int c = 0; c < CH; c++)
                gam[c] = *reinterpret_cast<const u32x4*>(norm.gamma + (size_t)(lo + c) * CHUNK + (lane % LPRA) * 8);
            float ss[MT16][LPC];
            float* nrm = reinterpret_cast<float*>(smem);             // [WK][BM]: before the partial tiles need the space
            const bool writer = norm.x_out != nullptr && blockIdx.x == 0;
#pragma unroll
            for (int mt = 0; mt < MT16; mt++)
#pragma unroll
                for (int i = 0; i < LPC; i++) {
                    const int row = i * RPIA + lane / LPRA;
                    const int m = m0 + 16 * mt + row;
                    float acc2 = 0.0f;
#pragma unroll
                    for (int c = 0; c < CH; c++) {
                        const bool own = (lo + c >= own_from) && (lo + c < min(own_from + CH, own_end));
                        const size_t eoff = (size_t)min(m, m_total - 1) * C::K + (size_t)(lo + c) * CHUNK + (lane % LPRA) * 8;
                        u32x4 v = raw[mt][c][i];
                        if (norm.delta != nullptr) {
                            const u32x4 d = *reinterpret_cast<const u32x4*>(norm.delta + eoff);
                            v.x = __builtin_bit_cast(uint32_t, as_f16x2(v.x) + as_f16x2(d.x));
                            v.y = __builtin_bit_cast(uint32_t, as_f16x2(v.y) + as_f16x2(d.y));
                            v.z = __builtin_bit_cast(uint32_t, as_f16x2(v.z) + as_f16x2(d.z));
                            v.w = __builtin_bit_cast(uint32_t, as_f16x2(v.w) + as_f16x2(d.w));
                        }
                        const bool live = own && m < m_total;
                        if (writer && live) *reinterpret_cast<u32x4*>(norm.x_out + eoff) = v;
                        if (!live) v = u32x4{0, 0, 0, 0};
                        raw[mt][c][i] = v;
                        acc2 = __builtin_amdgcn_fdot2(as_f16x2(v.x), as_f16x2(v.x), acc2, false);
                        acc2 = __builtin_amdgcn_fdot2(as_f16x2(v.y), as_f16x2(v.y), acc2, false);
                        acc2 = __builtin_amdgcn_fdot2(as_f16x2(v.z), as_f16x2(v.z), acc2, false);
                        acc2 = __builtin_amdgcn_fdot2(as_f16x2(v.w), as_f16x2(v.w), acc2, false);
                    }
                    // the LPRA lanes of a row sit side by side
                    if constexpr (LPRA > 1) acc2 += lane_xor<1>(acc2);
                    if constexpr (LPRA > 2) acc2 += lane_xor<2>(acc2);
                    if constexpr (LPRA > 4) acc2 += lane_xor<4>(acc2);
                    if constexpr (LPRA > 8) acc2 += lane_xor<8>(acc2);
                    if constexpr (LPRA > 16) acc2 += lane_xor<16>(acc2);
                    if constexpr (LPRA > 32) acc2 += lane_xor<32>(acc2);
                    ss[mt][i] = acc2;
                    if (lane % LPRA == 0) nrm[wk * C::BM + 16 * mt + row] = acc2;
                }
            __syncthreads();
#pragma unroll
            for (int mt = 0; mt < MT16; mt++)
#pragma unroll
                for (int i = 0; i < LPC; i++) {
                    const int row = i * RPIA + lane / LPRA;
                    float total = 0.0f;
#pragma unroll
                    for (int w2 = 0; w2 < WK; w2++) total += nrm[w2 * C::BM + 16 * mt + row];
                    ss[mt][i] = rsqrtf(total / (float)C::K + norm.eps);
                }
            __syncthreads();                                         // the sums are read: the space may be written again
#pragma unroll
            for (int mt = 0; mt < MT16; mt++)
#pragma unroll
                for (int c = 0; c < CH; c++)
#pragma unroll
                    for (int i = 0; i < LPC; i++) {
                        const float rn = ss[mt][i];
                        auto scale2 = [&](uint32_t hw, uint32_t gw) {
                            const f16x2 h = as_f16x2(hw);
                            f16x2 n;
                            n.x = (_Float16)((float)h.x * rn);
                            n.y = (_Float16)((float)h.y * rn);
                            return __builtin_bit_cast(uint32_t, n * as_f16x2(gw));
                        };
                        u32x4 v = raw[mt][c][i];
                        v.x = scale2(v.x, gam[c].x);
                        v.y = scale2(v.y, gam[c].y);
                        v.z = scale2(v.z, gam[c].z);
                        v.w = scale2(v.w, gam[c].w);
                        raw[mt][c][i] = v;
                    }
        }
#pragma unroll
        for (int mt = 0; mt < MT16; mt++) {
#pragma unroll
            for (int c = 0; c < CH; c++) {
                const bool own = (lo + c >= own_from) && (lo + c < min(own_from + CH, own_end));
#pragma unroll
                for (int i = 0; i < LPC; i++) {
                    const int row = i * RPIA + lane / LPRA;
                    const int m = m0 + 16 * mt + row;
                    u32x4 v = act_unit(raw[mt][c][i]);
                    if (!(own && m < m_total)) v = u32x4{0, 0, 0, 0};
                    *reinterpret_cast<u32x4*>(wbuf + row * PITCH_A + (lane % LPRA) * 16) = v;
                }
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int t = 0; t < KSTEPS; t++)
                    af[mt][c][t] = *reinterpret_cast<const f16x8*>(wbuf + r * PITCH_A + kb * EPL * 2 + t * 16);
                __builtin_amdgcn_wave_barrier();
            }
        }
    }

    const float* redf = reinterpret_cast<const float*>(smem);
    static_assert(SB % PF == 0, "ring index must be static inside a batch");
    constexpr int PITCH_W = C::PITCH_W, PITCH_H = C::PITCH_H;
    uint8_t* hbuf = wbuf + 16 * PITCH_W;                 // 1-bit plane of the tile being handed over
    // One batch of SB tiles.  With few batches (the usual case) the batch index is a compile-time
    // constant, so "is there a tile PF ahead to load" is decided at compile time: a load inside a
    // run-time branch reaches its users through a copy at the join, and that copy waits for every
    // load in flight -- measured as a full drain (vmcnt(0)) at the end of every tile, i.e. weight
    // loads and compute did not overlap at all.
    // ---- K split over blocks: how the KS blocks of a unit add up their sums.
    // The blocks form a binary tree over blockIdx.z.  For every output element a pair of blocks shares one 32-bit slot
    // of the scratch buffer, empty (zero) between launches: each swaps its sum in with a device-scope atomic exchange.
    // Whoever gets "empty" back was first and is done with the element; the other gets the partner's sum back, adds
    // its own (one fp32 addition, the same in either order), empties the slot for the next launch and carries the
    // result up one level, where the pair of pairs shares the next slot -- until the block that is second at the top
    // stores the output.  So the sum of an element is (..(p0 + p1) + (p2 + p3)..): fixed by the tree, independent of
    // who arrives when, and the meeting is log2(KS) dependent trips to memory with no barrier, no counter and no
    // wait for acknowledged stores (the counted-arrival form it replaces took three trips and two block barriers
    // at KS = 2).  A sum is never -0 (accumulators start at +0), so +0 travels as the bit pattern of -0 and zero can
    // mean "empty".  Lanes that have nothing to swap at a level (they were first below, or lie past the batch's last
    // element) sit the swap out: a swap into a spare word instead -- tried, to keep the swaps out of branches -- makes
    // idle lanes of several blocks queue on the same addresses (2 - 28 times the kernel's time).
    constexpr int THREADS = 64 * WK;
    constexpr int EPB = KS > 1 ? (C::PART + THREADS - 1) / THREADS : 1;         // sums per thread and batch
    constexpr int NQ = KS > 1 && C::NBATCH <= 8 ? C::NBATCH : 1;                // batches whose meeting waits for the last batch
    constexpr int LV = KS <= 1 ? 0 : KS == 2 ? 1 : KS == 4 ? 2 : KS == 8 ? 3 : 4;
    float pair_mine[NQ][EPB];
    uint32_t pair_got[NQ][EPB];
    const size_t split_unit = (size_t)blockIdx.y * C::GRID_X + team_id;
    // node of the tree this block's sum enters at `level` (KS - 1 nodes; index KS - 1 is the slot nobody reads)
    auto node_of = [&](int level) { return KS - (KS >> level) + ((int)blockIdx.z >> (level + 1)); };
    auto node_slot = [&](int batch, int node, int o) {
        return reinterpret_cast<uint32_t*>(scratch.partial) + ((split_unit * C::NBATCH + batch) * KS + node) * C::PART + o;
    };
    auto swap_in = [&](uint32_t* slot, float v) {
        uint32_t bits = __builtin_bit_cast(uint32_t, v);
        bits = bits == 0u ? 0x80000000u : bits;
        return __hip_atomic_exchange(slot, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    // the meeting of the batches first_batch .. first_batch + NQ - 1, whose level-0 swaps are on their way
    auto meet = [&](int first_batch) {
        if (QF_MGEMV_EXPERIMENT & 4) return;
        bool alive[NQ][EPB];
#pragma unroll
        for (int qq = 0; qq < NQ; qq++)
#pragma unroll
            for (int e = 0; e < EPB; e++) alive[qq][e] = tid + e * THREADS < C::PART;
        mg_static_for<0, LV>([&](auto lv_tag) {
            constexpr int L = decltype(lv_tag)::value;
#pragma unroll
            for (int qq = 0; qq < NQ; qq++)
#pragma unroll
                for (int e = 0; e < EPB; e++) {
                    const int o = min(tid + e * THREADS, C::PART - 1);
                    const uint32_t got = pair_got[qq][e];
                    const bool second = alive[qq][e] && got != 0u;
                    const float other = __builtin_bit_cast(float, got == 0x80000000u ? 0u : got);
                    pair_mine[qq][e] = second ? other + pair_mine[qq][e] : pair_mine[qq][e];
                    alive[qq][e] = second;
                    pair_got[qq][e] = 0u;
                    if (second) {
                        // the slot is empty again for the next launch; the sum goes up one level
                        __hip_atomic_store(node_slot(first_batch + qq, node_of(L), o), 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        if constexpr (L + 1 < LV) pair_got[qq][e] = swap_in(node_slot(first_batch + qq, node_of(L + 1), o), pair_mine[qq][e]);
                    }
                }
        });
#pragma unroll
        for (int qq = 0; qq < NQ; qq++)
#pragma unroll
            for (int e = 0; e < EPB; e++) {
                const int o = tid + e * THREADS;
                const int p = o >> 8, ml = (o >> 4) & 15, nl = o & 15;
                const int sb = p / MT16, mt = p % MT16;
                const int slot = (first_batch + qq) * SB + sb;
                const int tile = unit_of(slot);
                const int m = m0 + 16 * mt + ml;
                const int n = tile * 16 + nl;
                if (alive[qq][e] && slot < SLOTS && tile < C::NT && m < m_total && n < C::N) store_out(Cout + (size_t)m * C::N + n, pair_mine[qq][e]);
            }
    };

    auto do_batch = [&](auto batch_v) {
        using BT = decltype(batch_v);
        constexpr bool STATIC_BATCH = mg_is_tag<BT>::value;
        int batch;
        if constexpr (STATIC_BATCH) batch = BT::value; else batch = batch_v;
        mg_static_for<0, SB>([&](auto sb_tag) {
            constexpr int sb = decltype(sb_tag)::value;
            const int slot = batch * SB + sb;
            WStage& cur = ring[sb % PF];
            f32x4 acc[MT16];
#pragma unroll
            for (int mt = 0; mt < MT16; mt++) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
            // Hand-off and refill of a slot the block really has run outside the run-time test for a
            // ragged last tile (its stage holds the clamped last tile: valid memory, results unused),
            // so that with a static batch index no load sits inside a run-time branch.
            bool have_slot = true;
            if constexpr (STATIC_BATCH) { if constexpr (BT::value * SB + sb >= SLOTS) have_slot = false; }
            else have_slot = slot < SLOTS;
            u32x4 wfrag[CH];
            u32x2 hfrag[C::HI ? CH : 1];
            uint32_t qs[NSI], qz[NZI];
            if (have_slot && (QF_MGEMV_EXPERIMENT & 16)) {
                uint32_t x = 0;
#pragma unroll
                for (int i = 0; i < CH; i++) x ^= cur.w[i].x ^ cur.w[i].y ^ cur.w[i].z ^ cur.w[i].w;
#pragma unroll
                for (int j = 0; j < NSI; j++) x ^= cur.s[j];
#pragma unroll
                for (int j = 0; j < NZI; j++) x ^= cur.z[j];
                acc[0][0] += __builtin_bit_cast(float, x & 0x3FFFFFFFu);
                if constexpr (STATIC_BATCH) {
                    if constexpr (BT::value * SB + sb + PF < SLOTS) load_tile(cur, tile_clamped(slot + PF));
                } else {
                    if (slot + PF < SLOTS) load_tile(cur, tile_clamped(slot + PF));
                }
            }
            if (have_slot && !(QF_MGEMV_EXPERIMENT & (2 | 16))) {
                // coalesced registers -> LDS -> fragment registers: lane (r, kb) takes the 16 bytes
                // of row r at chunk c, k-block kb
#pragma unroll
                for (int i = 0; i < CH; i++)
                    *reinterpret_cast<u32x4*>(wbuf + (i * RPI + lane / LPR) * PITCH_W + (lane % LPR) * 16) = cur.w[i];
#pragma unroll
                for (int i = 0; i < NHI; i++) {
                    const int row = i * C::RPIH + lane / C::LPRH;
                    if (row < 16) *reinterpret_cast<u32x4*>(hbuf + row * PITCH_H + (lane % C::LPRH) * 16) = cur.h[i];
                }
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int c = 0; c < CH; c++) {
                    wfrag[c] = *reinterpret_cast<const u32x4*>(wbuf + r * PITCH_W + c * 64 + kb * 16);
                    if constexpr (C::HI) hfrag[c] = *reinterpret_cast<const u32x2*>(hbuf + r * PITCH_H + c * 32 + kb * 8);
                }
                __builtin_amdgcn_wave_barrier();
                // the stage's packed words are in LDS and its scales / zero-points in `qs` / `qz`:
                // it takes the loads of the tile PF ahead right away, one whole tile of
                // dequantisation and MFMAs before they are needed
#pragma unroll
                for (int j = 0; j < NSI; j++) qs[j] = cur.s[j];
#pragma unroll
                for (int j = 0; j < NZI; j++) qz[j] = C::SYM ? 0u : cur.z[j];
                if constexpr (STATIC_BATCH) {
                    if constexpr (BT::value * SB + sb + PF < SLOTS) load_tile(cur, tile_clamped(slot + PF));
                } else {
                    if (slot + PF < SLOTS) load_tile(cur, tile_clamped(slot + PF));
                }
#if QF_MGEMV_PIN_FIRST_LOADS
                __builtin_amdgcn_sched_barrier(0);      // the refill stays in front of this tile's arithmetic
#endif
            }
            // A slot past the block's last real tile holds the clamped last tile (valid memory); it is computed like any
            // other and its sums are never stored.  Skipping it would put the arithmetic into a conditional block, and
            // the compiler then moves the first tile's scale and zero-point loads -- used nowhere else -- down into
            // that block, behind the activation phase: a second trip to memory in front of the first MFMA.
            if (have_slot && (QF_MGEMV_COMPUTE_CLAMPED || tile_ok(slot)) && !(QF_MGEMV_EXPERIMENT & (2 | 16))) {
#pragma unroll
                for (int c = 0; c < CH; c++) {
                    const int g = ((lo + c) * CHUNK + kb * EPL) / C::GS;     // group of this lane's fields
                    // scale and zero-point of (row r, group g) sit in lane/register (idx % 64, idx / 64)
                    const int sidx = r * GWN + (g - gw_lo);
                    uint32_t sraw = 0;
#pragma unroll
                    for (int j = 0; j < NSI; j++) {
                        const uint32_t v = (uint32_t)__builtin_amdgcn_ds_bpermute((sidx & 63) << 2, (int)qs[j]);
                        sraw = (NSI == 1 || (sidx >> 6) == j) ? v : sraw;
                    }
                    uint32_t zero = 1u << (C::NBITS - 1);
                    if constexpr (!C::SYM) {
                        const int zbyte = (g * C::ZFB) / 8 - (gw_lo * C::ZFB) / 8;
                        const int zidx = r * ZB + zbyte;
                        uint32_t zraw = 0;
#pragma unroll
                        for (int j = 0; j < NZI; j++) {
                            const uint32_t v = (uint32_t)__builtin_amdgcn_ds_bpermute((zidx & 63) << 2, (int)qz[j]);
                            zraw = (NZI == 1 || (zidx >> 6) == j) ? v : zraw;
                        }
                        zero = (zraw >> ((g % P8) * C::ZFB)) & ZMASK;
                    }
                    const ZConst zc = make_zconst<C::NBITS>(zero);
                    const uint32_t w4[4] = {wfrag[c].x, wfrag[c].y, wfrag[c].z, wfrag[c].w};
                    // fields 8t .. 8t+7 of the lane's EPL as exact integers q - Z (fp16)
                    auto fields = [&](auto t_tag) {
                        constexpr int t = decltype(t_tag)::value;
                        if constexpr (C::HI) {
                            // 32 fields = two words of the 2-bit plane + one word of the 1-bit plane
                            const uint32_t w2[4] = {w4[2 * (t / 4)], w4[2 * (t / 4) + 1], 0u, 0u};
                            return IntStep3::run<t % 4>(w2, t < 4 ? hfrag[c].x : hfrag[c].y, zc);
                        } else {
                            return IntStep<C::NBITS>::run(w4, t, zc);
                        }
                    };
                    if constexpr (DEFERRED) {
                        // the whole chunk lies in one group: integer sum on the matrix core, one fp32 scale
                        f32x4 gsum[MT16];
                        mg_static_for<0, KSTEPS>([&](auto t_tag) {
                            constexpr int t = decltype(t_tag)::value;
                            const f16x8 wf = fields(t_tag);
#pragma unroll
                            for (int mt = 0; mt < MT16; mt++)
                                gsum[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                                    af[mt][c][t], wf, t == 0 ? f32x4{0.f, 0.f, 0.f, 0.f} : gsum[mt], 0, 0, 0);
                        });
                        const float sc = f16_bits_to_f32((uint16_t)sraw);
#pragma unroll
                        for (int mt = 0; mt < MT16; mt++)
#pragma unroll
                            for (int e = 0; e < 4; e++) acc[mt][e] = __builtin_fmaf(sc, gsum[mt][e], acc[mt][e]);
                    } else {
                        // a chunk spans several groups (the four lanes of a row may sit in different
                        // ones): scale every element before the contraction
                        const _Float16 sh = __builtin_bit_cast(_Float16, (uint16_t)sraw);
                        const f16x8 s8 = f16x8{sh, sh, sh, sh, sh, sh, sh, sh};
                        mg_static_for<0, KSTEPS>([&](auto t_tag) {
                            constexpr int t = decltype(t_tag)::value;
                            const f16x8 wf = fields(t_tag) * s8;
#pragma unroll
                            for (int mt = 0; mt < MT16; mt++)
                                acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[mt][c][t], wf, acc[mt], 0, 0, 0);
                        });
                    }
                }
            }
#pragma unroll
            for (int mt = 0; mt < MT16; mt++)
                red[(((size_t)wk * SB + sb) * MT16 + mt) * 64 + lane] = acc[mt];
        });

        __syncthreads();

        // ---- sum the WK partial tiles of this batch and store.  A partial tile sits in LDS as
        //      [lane = n + 16*(m/4)][e = m%4].  Every thread of the block takes single outputs
        //      (m = o/16, n = o%16 inside a tile): sixteen neighbouring lanes read sixteen different
        //      banks and store 32 contiguous bytes, and the WK-deep sums are spread over all waves
        //      instead of one wave per tile. ----
        if constexpr (C::SILU) {
            // a gate tile (even slot) and its up tile (odd slot): both sums, one store of their SwiGLU product
            constexpr int OUTPUTS_P = SB / 2 * MT16 * 256;
            for (int o = tid; o < OUTPUTS_P; o += 64 * WK) {
                const int p = o >> 8, ml = (o >> 4) & 15, nl = o & 15;
                const int sp = p / MT16, mt = p % MT16;
                const int slot = batch * SB + 2 * sp;
                if (slot >= SLOTS || !tile_ok(slot)) continue;
                const float* base = redf + (((size_t)(2 * sp) * MT16 + mt) * 64 + nl + 16 * (ml >> 2)) * 4 + (ml & 3);
                float gate = 0.f, up = 0.f;
#pragma unroll
                for (int k2 = 0; k2 < WK; k2++) {
                    gate += base[(size_t)k2 * SB * MT16 * 256];
                    up += base[(size_t)k2 * SB * MT16 * 256 + MT16 * 256];
                }
                const int m = m0 + 16 * mt + ml;
                const int n = unit_of(slot) * 16 + nl;
                if (m < m_total) Cout[(size_t)m * (C::N / 2) + n] = silu_mul_f16(gate, up);
            }
        }
        if constexpr (KS > 1) {
            // ---- K split over blocks: every sum of this batch is swapped into the slot it shares with the partner
            //      block's sum (see the meeting below); the swaps' results are looked at behind the last batch ----
            static_assert(!C::SILU && !NORM, "a block that sees part of K cannot normalise the rows or pair the gate with the up tile");
            int q = 0;
            if constexpr (STATIC_BATCH && NQ > 1) q = BT::value;
#pragma unroll
            for (int e = 0; e < EPB; e++) {
                const int o = min(tid + e * THREADS, C::PART - 1);
                const int p = o >> 8, ml = (o >> 4) & 15, nl = o & 15;
                const float* base = redf + ((size_t)p * 64 + nl + 16 * (ml >> 2)) * 4 + (ml & 3);
                float total = 0.f;
#pragma unroll
                for (int k2 = 0; k2 < WK; k2++) total += base[(size_t)k2 * SB * MT16 * 256];
                pair_mine[q][e] = total;
                pair_got[q][e] = 0u;
                if (!(QF_MGEMV_EXPERIMENT & 4) && tid + e * THREADS < C::PART) pair_got[q][e] = swap_in(node_slot(batch, node_of(0), o), total);
            }
            if constexpr (NQ == 1) meet(batch);                // many batches: each one's meeting right away
        }
        constexpr int OUTPUTS = (C::SILU || KS > 1) ? 0 : SB * MT16 * 256;
        for (int o = tid; o < OUTPUTS && !(QF_MGEMV_EXPERIMENT & 4); o += 64 * WK) {
            const int p = o >> 8, ml = (o >> 4) & 15, nl = o & 15;
            const int sb = p / MT16, mt = p % MT16;
            const int slot = batch * SB + sb;
            const int tile = unit_of(slot);
            if (slot >= SLOTS || tile >= C::NT) continue;
            const float* base = redf + (((size_t)sb * MT16 + mt) * 64 + nl + 16 * (ml >> 2)) * 4 + (ml & 3);
            float total = 0.f;
#pragma unroll
            for (int k2 = 0; k2 < WK; k2++) total += base[(size_t)k2 * SB * MT16 * 256];
            const int m = m0 + 16 * mt + ml;
            const int n = tile * 16 + nl;
            if (m < m_total && n < C::N) store_out(Cout + (size_t)m * C::N + n, total);
        }
        if (batch + 1 < C::NBATCH) __syncthreads();           // LDS slots are reused by the next batch
    };
    if constexpr (C::NBATCH <= 8) {
        mg_static_for<0, C::NBATCH>(do_batch);
    } else {
#pragma unroll 1
        for (int batch = 0; batch < C::NBATCH; batch++) do_batch(batch);
    }

    if constexpr (KS > 1 && NQ > 1) meet(0);
}

// Row blocks (grid.y) a split-K object's scratch buffer is sized for.
constexpr int kMGemvScratchRowBlocks = 1;

// A buffer of kMGemvScratchRowBlocks * SCRATCH_BYTES bytes, 256-byte aligned and zero, as the kernel's slots.
template <class C>
MGemvScratch mgemv_scratch_at(void* base) {
    MGemvScratch s;
    s.partial = static_cast<float*>(base);
    return s;
}

// Largest scratch buffer a specialisation keeps as a static device array for its entry point that allocates nothing
// (the generated translation unit declares the array: every GPU the object runs on holds it until the process ends).
constexpr size_t kMGemvStaticScratchMax = 8u << 20;
template <class C>
constexpr size_t mgemv_static_scratch_bytes() {
    constexpr size_t need = C::SCRATCH_BYTES * kMGemvScratchRowBlocks;
    return need <= kMGemvStaticScratchMax ? need : 256;           // an object past the limit keeps a token array and refuses the call
}

// The scratch buffer of this specialisation on the current device, allocated and cleared at the first call there and
// kept until the process ends (null with a message if that fails).  The first call must not happen under stream
// capture; afterwards the function only looks the pointer up.
template <class C>
MGemvScratch mgemv_scratch() {
    static std::mutex lock;
    static void* per_device[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
        fprintf(stderr, "qfactory mgemv: cannot tell the current device\n");
        return MGemvScratch{};
    }
    std::lock_guard<std::mutex> guard(lock);
    if (per_device[dev] == nullptr) {
        void* p = nullptr;
        const size_t bytes = C::SCRATCH_BYTES * kMGemvScratchRowBlocks;
        hipError_t e = hipMalloc(&p, bytes);
        if (e == hipSuccess) e = hipMemset(p, 0, bytes);
        // the counters are zero before any launch can read them, on whatever stream it is enqueued (a stream created
        // non-blocking does not wait for the null stream's memset by itself)
        if (e == hipSuccess) e = hipDeviceSynchronize();
        if (e != hipSuccess) {
            fprintf(stderr, "qfactory mgemv: cannot set up %zu bytes of scratch memory: %s\n", bytes, hipGetErrorString(e));
            return MGemvScratch{};
        }
        per_device[dev] = p;
    }
    return mgemv_scratch_at<C>(per_device[dev]);
}

template <class C>
int mgemv_launch(const void* A, const void* W, void* Cout, const void* S, const void* Zp, int m, hipStream_t stream,
                 NormArgs norm = NormArgs{}, const MGemvScratch* given = nullptr) {
    const char* why = nullptr;
    if (C::NBITS != 2 && C::NBITS != 3 && C::NBITS != 4 && C::NBITS != 8) why = "NBITS must be 2, 3, 4 or 8 for this kernel";
    else if (C::K % C::CHUNK != 0) why = "K must be a multiple of 4*128 / (bits of the main plane)";
    else if (C::GS <= 0 || C::K % C::GS != 0) why = "GS must divide K";
    else if (C::GS % C::EPL != 0) why = "a lane's 16 bytes of fields must lie inside one group";
    else if (!C::SYM && (C::G % (8 / C::ZFB)) != 0) why = "K/GS must fill whole zero-point bytes";
    else if (C::CH > C::NCHUNK) why = "more chunks per wave than the row has";
    else if (C::KS == 1 && C::WK * C::CH < C::NCHUNK) why = "WK*CH must cover K";
    else if (C::KS == 1 && (C::WK - 1) * C::CH >= C::NCHUNK) why = "a wave would own no chunk";
    else if (C::THREADS > 1024) why = "block too large";
    else if (C::CH != 1 && C::CH != 2 && C::CH != 4 && C::CH != 8 && C::CH != 16) why = "CH must be 1, 2, 4, 8 or 16";
    else if (C::GS % C::CHUNK != 0 && C::CHUNK % C::GS != 0) why = "GS must divide the chunk or be a multiple of it";
    else if (C::PF != 1 && C::PF != 2 && C::PF != 4) why = "PF must be 1, 2 or 4";
    else if (C::LDS_BYTES > 160 * 1024) why = "partial tiles exceed the 160 KB of LDS";
    else if (C::SILU && (C::N % 32 != 0 || C::SB % 2 != 0)) why = "gate+up: N/2 must be whole 16-row tiles and a batch whole pairs";
    else if (C::SILU && (QF_IN_BF16 || QF_OUT_BF16)) why = "the SwiGLU epilogue is fp16 only";
    else if (QF_MGEMV_NORM_PROLOGUE && (QF_IN_BF16 || QF_OUT_BF16)) why = "the norm prologue is fp16 only";
    else if (QF_OUT_ACCUMULATE && (QF_OUT_BF16 || QF_MGEMV_GATE_UP_SILU)) why = "adding to the output is fp16 only and not combined with the SwiGLU epilogue";
    else if (QF_MGEMV_NORM_PROLOGUE && norm.gamma == nullptr) why = "an object with the norm prologue is called through launch_norm (RMSNorm weight missing)";
    else if (!QF_MGEMV_NORM_PROLOGUE && norm.gamma != nullptr) why = "this object was compiled without the norm prologue";
    else if (C::KS != 1 && C::KS != 2 && C::KS != 4 && C::KS != 8 && C::KS != 16) why = "KS must be 1, 2, 4, 8 or 16";
    else if (C::KS > 1 && (QF_MGEMV_NORM_PROLOGUE || QF_MGEMV_GATE_UP_SILU)) why = "K split over blocks: neither the norm prologue nor the SwiGLU epilogue";
    else if (C::KS > 1 && C::WK * C::CH < C::NCHUNK_B) why = "WK*CH must cover a block's share of K";
    else if (C::KS > 1 && (C::KS - 1) * C::NCHUNK_B >= C::NCHUNK) why = "a block would own no chunk";
    else if (QF_MGEMV_NORM_PROLOGUE && (norm.x_out == A || (norm.x_out != nullptr && norm.x_out == norm.delta))) why = "x_out must be a buffer of its own: other blocks still read x and delta";
    else if (QF_MGEMV_NORM_PROLOGUE && (size_t)C::WK * C::BM * 4 > (size_t)C::WK * C::SB * C::MT16 * 1024) why = "norm sums exceed the reduction space";
    if (why) {
        fprintf(stderr, "qfactory mgemv: invalid configuration: %s (NBITS=%d GS=%d N=%d K=%d MT16=%d WK=%d CH=%d PB=%d PF=%d KS=%d)\n",
                why, C::NBITS, C::GS, C::N, C::K, C::MT16, C::WK, C::CH, C::PB, C::PF, C::KS);
        return 1;
    }
    if (m <= 0) return 0;
    static std::atomic<bool> attr_set{false};        // launch is re-entrant: the attribute call is idempotent, the flag only saves repeats
    if (C::LDS_BYTES > 64 * 1024 && !attr_set.load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&mgemv_kernel<C>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)C::LDS_BYTES);
        if (e != hipSuccess) {
            fprintf(stderr, "qfactory mgemv: cannot reserve %zu bytes of LDS: %s\n", C::LDS_BYTES, hipGetErrorString(e));
            return 2;
        }
        attr_set.store(true, std::memory_order_release);
    }
    dim3 grid(C::GRID_X, (m + C::BM - 1) / C::BM, C::KS);
    MGemvScratch scratch;
    if constexpr (C::KS > 1) {
        if ((int)grid.y > kMGemvScratchRowBlocks) {
            fprintf(stderr, "qfactory mgemv: an object that splits K over blocks takes at most %d rows per launch (got %d)\n",
                    kMGemvScratchRowBlocks * C::BM, m);
            return 1;
        }
        scratch = given != nullptr ? *given : mgemv_scratch<C>();
        if (scratch.partial == nullptr) return 2;
    }
    hipLaunchKernelGGL(mgemv_kernel<C>, grid, dim3(C::THREADS), C::LDS_BYTES, stream, (const uint16_t*)A,
                       (const uint8_t*)W, (uint16_t*)Cout, (const uint16_t*)S, (const uint8_t*)Zp, m, norm, scratch);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        fprintf(stderr, "qfactory mgemv: launch failed: %s\n", hipGetErrorString(err));
        return 2;
    }
    return 0;
}

}  // namespace qf
