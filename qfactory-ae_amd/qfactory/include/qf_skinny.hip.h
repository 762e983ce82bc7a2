// Dequant-fused low-bit "skinny GEMM" on the gfx950 matrix cores for 3 <= M <= 16, HBM-bound
// (two 16-row tiles per block, M <= 32, are accepted but need more registers than two waves per
// SIMD have: measured 2 - 4 times slower than the GEMM kernel, which serves those row counts).
//
//   C[m][n] = fp16( sum_g s[n][g] * sum_{k in g} A[m][k] * (q[n][k] - Z[n][g]) )
//
// Same operands as the reference's kernel_gptq (qfactory/include/gptq_gemv.h:14-154) in its
// deferred-decode form (utils.h:193-213): the integer part is summed first, the scale is applied
// once per group -- here in fp32 and on the matrix cores.  The packed weights are read exactly
// once, straight from the reference layout:
//
//   * Persistent blocks: at most PB blocks; block b sweeps the 16-row weight tiles b, b + grid,
//     ..., SB of them ("a batch") at a time.
//   * The WK waves of a block split K: a row's packed bytes are cut into steps of 128 bytes
//     (1024/NBITS elements) and wave w owns the SPW consecutive steps w*SPW .. of every row.
//   * v_mfma_f32_16x16x32_f16 contracts over 4 k-blocks x 8 elements; which 32 elements of K those
//     are is free as long as both operands agree: lane (r, kb) takes the 16 packed bytes kb of a
//     64-byte chunk of weight row r -- 128/NBITS consecutive fields, eight per k-step -- and the
//     activations of exactly those columns of row r.
//   * Global loads are coalesced (four lanes per 64 contiguous bytes; a load in fragment order,
//     where neighbouring lanes read different rows, measured four times slower).  A weight chunk
//     (16 rows x 64 bytes = one load) reaches fragment order by a lane permutation through the LDS
//     crossbar (ds_bpermute, no LDS memory); an activation step goes through a small LDS buffer
//     private to the wave.
//   * A stage is one step of one batch: the activations of the step (shared by the batch's
//     tiles) and 2 x 16 packed bytes per tile; the scales and zero-points of a tile for all the
//     wave's steps ride with the first.  D stages are in flight in registers; the waits are the
//     compiler's own vmcnt bookkeeping.  Activation staging, weight streaming and dequantisation
//     of different steps overlap; there is no block barrier inside a batch.
//   * Fields are masked in place (1024 + 2^o*q) and brought to the exact integer q - Z with one
//     packed fp16 add or fma; the activations are MFMA source A (rows m), the weights source B
//     (columns n), so a lane ends with one n and needs one scale: acc += s * group_sum in fp32.
//   * Per batch each wave parks its partial 16x16 tiles in LDS (two sets of slots, used
//     alternately: one barrier per batch), the partials of the WK waves are summed and every
//     output is written once.  No global workspace, no atomics: results are deterministic.
#pragma once

#include <atomic>
#include <cstdio>
#include "qf_dequant.hip.h"

// Timing experiments (results are wrong when non-zero): bit 0 skips the activation loads, bit 1 the
// dequantisation and MFMAs, bit 2 the cross-wave reduction and the stores, bit 3 the weight loads.
#ifndef QF_SKINNY_EXPERIMENT
#define QF_SKINNY_EXPERIMENT 0
#endif
#if QF_SKINNY_EXPERIMENT != 0 && !defined(QF_ALLOW_TIMING_EXPERIMENTS)
#error "QF_SKINNY_EXPERIMENT gives wrong results: timing builds only (define QF_ALLOW_TIMING_EXPERIMENTS)"
#endif

// Decode strategy (the reference's search dimension, qfactory/core/qfunc.py:85-91).  0: "deferred" wherever the group
// geometry allows (integer sums on the matrix core, one fp32 scale per group), 1: "eager" everywhere (scale mode 2
// below: every field becomes fp16_rn((q - Z) * s) before the contraction).
#ifndef QF_SKINNY_EAGER
#define QF_SKINNY_EAGER 0
#endif

namespace qf {

constexpr int skinny_gcd(int a, int b) { return b == 0 ? a : skinny_gcd(b, a % b); }

template <int V> struct SkinnyTag { static constexpr int value = V; };
template <int I, int N, class F>
__device__ __forceinline__ void skinny_static_for(F&& f) {
    if constexpr (I < N) {
        f(SkinnyTag<I>{});
        skinny_static_for<I + 1, N>(f);
    }
}

// Wait for this wave's LDS operations (not for its global loads, which stay in flight), then meet
// the other waves of the block.
__device__ __forceinline__ void skinny_lds_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xC07F);          // vmcnt 63 (no wait), expcnt 7 (no wait), lgkmcnt 0
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

template <int NBITS_, int GS_, bool SYM_, int N_, int K_, int MT16_, int WK_, int SB_, int D_, bool AST_, int PB_, bool NT_B_>
struct SkinnyCfg {
    static constexpr int NBITS = NBITS_, GS = GS_, N = N_, K = K_;
    static constexpr bool SYM = SYM_, NT_B = NT_B_;
    static constexpr int MT16 = MT16_;             // 16-row activation tiles per block
    static constexpr int WK = WK_;                 // waves of a block, splitting K
    static constexpr int SB = SB_;                 // weight tiles per batch
    static constexpr int D = D_;                   // stages in flight per wave
    static constexpr bool AST = AST_;              // activation fragments of the wave's steps stay in registers across batches
    static constexpr int PB = PB_;                 // upper bound on blocks along N
    static constexpr int EPL = 128 / NBITS;        // fields per lane and 16 packed bytes
    static constexpr int KSTEPS = EPL / 8;         // MFMA k-steps per chunk
    static constexpr int CHUNK = 4 * EPL;          // elements of K in 64 packed bytes of a row
    static constexpr int STEPK = 2 * CHUNK;        // ... in a step of 128 packed bytes
    static constexpr int NSTEP = K / STEPK;
    static constexpr int SPW = (NSTEP + WK - 1) / WK;                       // steps per wave
    static constexpr int THREADS = 64 * WK;
    static constexpr int BM = 16 * MT16;
    static constexpr int NT = (N + 15) / 16;       // 16-row weight tiles
    static constexpr int GRID_X = NT < PB ? NT : PB;
    static constexpr int SLOTS = (NT + GRID_X - 1) / GRID_X;               // tiles per block
    static constexpr int NBATCH = (SLOTS + SB - 1) / SB;
    static constexpr int P = SPW / skinny_gcd(SPW, D) * D;                  // unrolled period: stage slots and steps both static
    static constexpr int BPP = P / SPW;            // batches per period
    static constexpr int RB = K * NBITS / 8;
    static constexpr int G = K / GS;
    static constexpr int ZRB = G * NBITS / 8;
    // 0: a step lies inside one group; 1: one group per chunk; 2: groups narrower than a chunk
    // (a lane's 128/NBITS fields still share one): the weights are scaled before the contraction
    static constexpr int SMODE = QF_SKINNY_EAGER ? 2 : (GS >= STEPK ? 0 : (GS == CHUNK ? 1 : 2));
    // scales of one row for the wave's SPW steps: SMODE 1 keeps a dword (two groups) per step and
    // fetches VS steps per load; the other modes fetch a half-word per step (and chunk)
    static constexpr int VS = SMODE != 1 ? 1 : ((SPW % 4 == 0 && NSTEP % 4 == 0) ? 4 : ((SPW % 2 == 0 && NSTEP % 2 == 0) ? 2 : 1));
    static constexpr int NQ = SMODE == 2 ? 2 * SPW : SPW;                   // scale / zero registers per tile and batch
    // activation step in LDS (private to the wave): 16 rows of STEPK halves, padded by 16 bytes
    static constexpr int A_ROWB = STEPK * 2;
    static constexpr int A_PITCH = A_ROWB + 16;
    static constexpr int A_LPR = A_ROWB / 16;      // lanes per row of a coalesced load
    static constexpr int A_RPI = 64 / A_LPR;       // rows per load
    static constexpr int NA = 16 / A_RPI;          // loads per 16 rows and step
    static constexpr size_t LDS_RED = (size_t)2 * WK * SB * MT16 * 1024;
    static constexpr size_t LDS_ABUF = (size_t)MT16 * 16 * A_PITCH;
    static constexpr size_t LDS_BYTES = LDS_RED + (size_t)WK * LDS_ABUF;
};

template <class C>
__global__ __launch_bounds__(C::THREADS) void skinny_kernel(
    const uint16_t* __restrict__ A, const uint8_t* __restrict__ W, uint16_t* __restrict__ Cout,
    const uint16_t* __restrict__ S, const uint8_t* __restrict__ Zp, int m_total) {
    constexpr int MT16 = C::MT16, WK = C::WK, SB = C::SB, D = C::D, SPW = C::SPW;
    constexpr int EPL = C::EPL, KSTEPS = C::KSTEPS, CHUNK = C::CHUNK, STEPK = C::STEPK;
    constexpr int SMODE = C::SMODE, NQ = C::NQ, VS = C::VS, NA = C::NA;
    constexpr uint32_t ZMASK = (1u << C::NBITS) - 1u;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wk = __builtin_amdgcn_readfirstlane(tid >> 6);     // wave-uniform: addresses are scalar base + lane offset
    const int r = lane & 15, kb = lane >> 4;
    const int m0 = blockIdx.y * C::BM;
    const int team = blockIdx.x;
    const int st0 = wk * SPW;                                      // first step of this wave
    uint8_t* abuf = smem + C::LDS_RED + (size_t)wk * C::LDS_ABUF;

    // ---- activations of one step: coalesced loads (A_LPR lanes per row), the wave's LDS buffer,
    //      then fragments (mt, c, t) = A[m0 + 16*mt + r][step*STEPK + c*CHUNK + kb*EPL + 8t .. +7] ----
    struct ARaw { u32x4 v[MT16][NA]; };
    struct AFrag { f16x8 f[MT16][2][KSTEPS]; };
    const int a_row = lane / C::A_LPR, a_col = lane % C::A_LPR;
    const uint32_t a_lane = ((uint32_t)(m0 + a_row) * C::K) * 2u + a_col * 16;    // this lane's first unit of a step
    auto load_a = [&](ARaw& raw, int s) {
        const int step = min(st0 + s, C::NSTEP - 1);               // a wave's steps past the end of K re-read the last one
        const uint8_t* base = reinterpret_cast<const uint8_t*>(A) + (size_t)step * C::A_ROWB;
#pragma unroll
        for (int mt = 0; mt < MT16; mt++)
#pragma unroll
            for (int i = 0; i < NA; i++) {
                const int dm = 16 * mt + i * C::A_RPI;             // rows below the lane's first
                u32x4 v = u32x4{0u, 0u, 0u, 0u};                   // rows past m_total contribute zeros and issue no load
                if (QF_SKINNY_EXPERIMENT & 1) v = u32x4{(uint32_t)lane, 1u, 2u, 3u};
                else if (m0 + dm + a_row < m_total) v = *reinterpret_cast<const u32x4*>(base + (size_t)dm * C::K * 2 + a_lane);
                raw.v[mt][i] = v;
            }
    };
    auto transpose_a = [&](AFrag& fr, const ARaw& raw) {
#pragma unroll
        for (int mt = 0; mt < MT16; mt++)
#pragma unroll
            for (int i = 0; i < NA; i++)
                *reinterpret_cast<u32x4*>(abuf + (mt * 16 + i * C::A_RPI + a_row) * C::A_PITCH + a_col * 16) = act_unit(raw.v[mt][i]);
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int mt = 0; mt < MT16; mt++)
#pragma unroll
            for (int c = 0; c < 2; c++)
#pragma unroll
                for (int t = 0; t < KSTEPS; t++)
                    fr.f[mt][c][t] = *reinterpret_cast<const f16x8*>(abuf + (mt * 16 + r) * C::A_PITCH + (c * CHUNK + kb * EPL + 8 * t) * 2);
        __builtin_amdgcn_wave_barrier();
    };

    // ---- scales and zero-points of one tile for all the wave's steps (loaded with step 0 of a
    //      batch); register i belongs to the wave's step i (steps past the end of K re-read the last) ----
    struct Quant { uint32_t s[NQ]; uint32_t z[NQ]; };
    auto load_quant = [&](Quant& q, int tile, uint32_t row) {
        const uint8_t* srow = reinterpret_cast<const uint8_t*>(S) + ((size_t)tile * 16 + row) * (C::G * 2);
        const uint8_t* zrow = Zp + ((size_t)tile * 16 + row) * C::ZRB;
        if constexpr (SMODE == 1) {
            // groups 2*step and 2*step + 1: one aligned dword of scales per step, VS steps per load
#pragma unroll
            for (int i = 0; i < SPW / VS; i++) {
                const int step = min(st0 + VS * i, C::NSTEP - VS);
                const uint8_t* sp = srow + step * 4;
                if constexpr (VS == 4) {
                    const u32x4 v = *reinterpret_cast<const u32x4*>(sp);
                    q.s[4 * i] = v.x; q.s[4 * i + 1] = v.y; q.s[4 * i + 2] = v.z; q.s[4 * i + 3] = v.w;
                } else if constexpr (VS == 2) {
                    const u32x2 v = *reinterpret_cast<const u32x2*>(sp);
                    q.s[2 * i] = v.x; q.s[2 * i + 1] = v.y;
                } else {
                    q.s[i] = *reinterpret_cast<const uint32_t*>(sp);
                }
            }
#pragma unroll
            for (int i = 0; i < SPW; i++) {
                q.z[i] = 0;
                if constexpr (!C::SYM) {
                    const int g = 2 * min(st0 + i, C::NSTEP - 1);
                    if constexpr (C::NBITS == 8) q.z[i] = *reinterpret_cast<const uint16_t*>(zrow + g);
                    else q.z[i] = zrow[(g * C::NBITS) / 8];
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < NQ; i++) {
                const int step = min(st0 + (SMODE == 2 ? i / 2 : i), C::NSTEP - 1);
                const int g = SMODE == 2 ? (step * STEPK + (i % 2) * CHUNK + kb * EPL) / C::GS : step * STEPK / C::GS;
                q.s[i] = *reinterpret_cast<const uint16_t*>(srow + g * 2);
                q.z[i] = 0;
                if constexpr (!C::SYM) q.z[i] = zrow[(g * C::NBITS) / 8];
            }
        }
    };
    // scale bits and zero-point of chunk c of the wave's step s (s is a constant at every call site)
    auto quant_of = [&](const Quant& q, int s, int c, uint32_t& sbits, uint32_t& zero) {
        const int step = st0 + s;
        if constexpr (SMODE == 0) {
            const int g = step * STEPK / C::GS;
            sbits = q.s[s];
            zero = (q.z[s] >> ((g * C::NBITS) % 8)) & ZMASK;
        } else if constexpr (SMODE == 1) {
            const int g = 2 * step + c;
            sbits = c ? q.s[s] >> 16 : q.s[s] & 0xFFFFu;
            if constexpr (C::NBITS == 8) zero = (q.z[s] >> (8 * c)) & ZMASK;
            else zero = (q.z[s] >> ((g * C::NBITS) % 8)) & ZMASK;
        } else {
            const int g = (step * STEPK + c * CHUNK + kb * EPL) / C::GS;
            sbits = q.s[2 * s + c];
            zero = (q.z[2 * s + c] >> ((g * C::NBITS) % 8)) & ZMASK;
        }
        if constexpr (C::SYM) zero = 1u << (C::NBITS - 1);
    };

    // ---- one stage: a step of the batch's SB tiles.  Weight loads are coalesced -- lane l takes the
    //      16 bytes l%4 of chunk c of row l/4 -- and reach fragment order (lane (r, kb) <- lane 4r + kb)
    //      through the LDS crossbar (ds_bpermute: no LDS memory) ----
    struct Stage {
        ARaw a;                      // unused when the activation fragments are resident (AST)
        u32x4 w[SB][2];
        Quant q[SB];                 // loaded only in a stage of the wave's first step
    };
    auto load_stage = [&](Stage& st, int batch, int s) {
        const int step = min(st0 + s, C::NSTEP - 1);
        if constexpr (!C::AST) load_a(st.a, s);
#pragma unroll
        for (int sb = 0; sb < SB; sb++) {
            const int tile = min(team + (batch * SB + sb) * C::GRID_X, C::NT - 1);   // block-uniform
            const int last = C::N - 1 - tile * 16;                                    // rows past N re-read the last one
            const uint8_t* wrow = W + (size_t)tile * 16 * C::RB + (size_t)step * 128;
            const uint32_t woff = (uint32_t)min(lane >> 2, last) * C::RB + (lane & 3) * 16;
#pragma unroll
            for (int c = 0; c < 2; c++) {
                if (QF_SKINNY_EXPERIMENT & 8) { st.w[sb][c] = u32x4{(uint32_t)lane, 2u, 3u, 4u}; continue; }
                const uint8_t* src = wrow + woff + c * 64;
                st.w[sb][c] = C::NT_B ? __builtin_nontemporal_load((const u32x4*)src) : *(const u32x4*)src;
            }
            if (s == 0) load_quant(st.q[sb], tile, (uint32_t)min(r, last));
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

    f32x4 acc[SB][MT16];
#pragma unroll
    for (int sb = 0; sb < SB; sb++)
#pragma unroll
        for (int mt = 0; mt < MT16; mt++) acc[sb][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    Quant quant[SB];                                               // of the batch being computed

    auto compute = [&](const Stage& st, const AFrag& a, int s) {
        if (QF_SKINNY_EXPERIMENT & 2) return;
        if (st0 + s >= C::NSTEP) return;                           // wave-uniform: this wave has fewer steps
#pragma unroll
        for (int sb = 0; sb < SB; sb++) {
            f32x4 gsum[MT16];
#pragma unroll
            for (int c = 0; c < 2; c++) {
                uint32_t sbits, zero;
                quant_of(quant[sb], s, c, sbits, zero);
                const ZConst zc = make_zconst<C::NBITS>(zero);
                const u32x4 wv = to_fragment(st.w[sb][c]);
                const uint32_t w4[4] = {wv.x, wv.y, wv.z, wv.w};
                if constexpr (SMODE == 2) {
                    // the four k-blocks of an MFMA sit in different groups: scale every element first
                    const _Float16 sh = __builtin_bit_cast(_Float16, (uint16_t)sbits);
                    const f16x8 s8 = f16x8{sh, sh, sh, sh, sh, sh, sh, sh};
#pragma unroll
                    for (int t = 0; t < KSTEPS; t++) {
                        const f16x8 wf = IntStep<C::NBITS>::run(w4, t, zc) * s8;
#pragma unroll
                        for (int mt = 0; mt < MT16; mt++)
                            acc[sb][mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a.f[mt][c][t], wf, acc[sb][mt], 0, 0, 0);
                    }
                } else {
                    // integer sum of a group on the matrix core, then one fp32 scale; with a group per
                    // step (SMODE 0) both chunks go into the same sum
                    const bool fresh = SMODE == 1 || c == 0;
#pragma unroll
                    for (int t = 0; t < KSTEPS; t++) {
                        const f16x8 wf = IntStep<C::NBITS>::run(w4, t, zc);
#pragma unroll
                        for (int mt = 0; mt < MT16; mt++)
                            gsum[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                                a.f[mt][c][t], wf, (fresh && t == 0) ? f32x4{0.f, 0.f, 0.f, 0.f} : gsum[mt], 0, 0, 0);
                    }
                    if (SMODE == 1 || c == 1) {
                        const float sc = f16_bits_to_f32((uint16_t)sbits);
#pragma unroll
                        for (int mt = 0; mt < MT16; mt++)
#pragma unroll
                            for (int e = 0; e < 4; e++) acc[sb][mt][e] = __builtin_fmaf(sc, gsum[mt][e], acc[sb][mt][e]);
                    }
                }
            }
        }
    };

    // ---- end of a batch: the WK partial tiles meet in LDS and every output is stored once.  A
    //      partial tile sits in LDS as [lane = n + 16*(m/4)][e = m%4]; every thread of the block takes
    //      single outputs (m = o/16, n = o%16 inside a tile), so sixteen neighbouring lanes read sixteen
    //      banks and store 32 contiguous bytes and the WK-deep sums are spread over all waves.  The two sets of slots
    //      alternate, so a fast wave parking batch b+1 never touches what a slow one still reads. ----
    auto finish_batch = [&](int batch) {
        f32x4* red = reinterpret_cast<f32x4*>(smem) + (size_t)(batch & 1) * (WK * SB * MT16 * 64);   // [WK][SB][MT16][64]
#pragma unroll
        for (int sb = 0; sb < SB; sb++)
#pragma unroll
            for (int mt = 0; mt < MT16; mt++) {
                red[(((size_t)wk * SB + sb) * MT16 + mt) * 64 + lane] = acc[sb][mt];
                acc[sb][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
        skinny_lds_barrier();
        const float* redf = reinterpret_cast<const float*>(red);
        constexpr int OUTPUTS = SB * MT16 * 256;
        for (int o = (int)threadIdx.x; o < OUTPUTS && !(QF_SKINNY_EXPERIMENT & 4); o += 64 * WK) {
            const int p = o >> 8, ml = (o >> 4) & 15, nl = o & 15;
            const int sb = p / MT16, mt = p % MT16;
            const int slot = batch * SB + sb;
            const int tile = team + slot * C::GRID_X;
            if (slot >= C::SLOTS || tile >= C::NT) continue;
            const float* base = redf + (((size_t)sb * MT16 + mt) * 64 + nl + 16 * (ml >> 2)) * 4 + (ml & 3);
            float total = 0.f;
#pragma unroll
            for (int k2 = 0; k2 < WK; k2++) total += base[(size_t)k2 * SB * MT16 * 256];
            const int m = m0 + 16 * mt + ml;
            const int n = tile * 16 + nl;
            if (m < m_total && n < C::N) store_out(Cout + (size_t)m * C::N + n, total);
        }
    };

    // ---- pipeline over the flattened (batch, step) sequence: stage f lives in ring slot f % D ----
    Stage ring[D];
    AFrag resident[C::AST ? SPW : 1];
    skinny_static_for<0, D>([&](auto tag) {
        constexpr int j = decltype(tag)::value;
        if (j / SPW < C::NBATCH) load_stage(ring[j], j / SPW, j % SPW);
    });
    if constexpr (C::AST) {
        ARaw raw[SPW];
#pragma unroll
        for (int s = 0; s < SPW; s++) load_a(raw[s], s);
#pragma unroll
        for (int s = 0; s < SPW; s++) transpose_a(resident[s], raw[s]);
    }

#pragma unroll 1
    for (int b0 = 0; b0 < C::NBATCH; b0 += C::BPP) {
        skinny_static_for<0, C::P>([&](auto tag) {
            constexpr int j = decltype(tag)::value;
            constexpr int s = j % SPW, slot = j % D;
            const int batch = b0 + j / SPW;
            if (batch < C::NBATCH) {
                if constexpr (s == 0) {
#pragma unroll
                    for (int sb = 0; sb < SB; sb++) quant[sb] = ring[slot].q[sb];
                }
                if constexpr (C::AST) {
                    compute(ring[slot], resident[C::AST ? s : 0], s);
                } else {
                    AFrag fr;
                    transpose_a(fr, ring[slot].a);
                    compute(ring[slot], fr, s);
                }
                // the slot takes the stage D ahead in the sequence
                constexpr int j2 = j + D;
                const int batch2 = b0 + j2 / SPW;
                if (batch2 < C::NBATCH) load_stage(ring[slot], batch2, j2 % SPW);
                if constexpr (s == SPW - 1) finish_batch(batch);
            }
        });
    }
}

template <class C>
int skinny_launch(const void* A, const void* W, void* Cout, const void* S, const void* Zp, int m, hipStream_t stream) {
    const char* why = nullptr;
    if (C::NBITS != 2 && C::NBITS != 4 && C::NBITS != 8) why = "NBITS must be 2, 4 or 8 for this kernel";
    else if (C::K % C::STEPK != 0 || C::NSTEP < 1) why = "K must be a multiple of 1024/NBITS";
    else if (C::GS <= 0 || C::K % C::GS != 0) why = "GS must divide K";
    else if (C::GS % C::EPL != 0) why = "a lane's 16 bytes of fields must lie inside one group";
    else if (C::GS >= C::STEPK ? C::GS % C::STEPK != 0 : C::CHUNK % C::GS != 0) why = "GS must divide 512/NBITS or be a multiple of 1024/NBITS";
    else if (!C::SYM && (C::G % (8 / C::NBITS)) != 0) why = "K/GS must fill whole zero-point bytes";
    else if (C::MT16 < 1 || C::MT16 > 2) why = "MT16 must be 1 or 2";
    else if (C::WK < 1 || C::THREADS > 1024) why = "1 .. 16 waves per block";
    else if ((C::WK - 1) * C::SPW >= C::NSTEP) why = "a wave would own no step";
    else if (C::SB < 1 || C::SB > 8) why = "SB must be 1 .. 8";
    else if (C::D < 1 || C::D > 4) why = "D must be 1 .. 4";
    else if (C::P > 32) why = "unrolled period too long (choose D dividing the steps per wave)";
    else if (C::LDS_BYTES > 160 * 1024) why = "partial tiles exceed the 160 KB of LDS";
    else if (QF_OUT_ACCUMULATE && QF_OUT_BF16) why = "adding to the output is fp16 only";
    if (why) {
        fprintf(stderr, "qfactory skinny: invalid configuration: %s (NBITS=%d GS=%d N=%d K=%d MT16=%d WK=%d SB=%d D=%d AST=%d PB=%d)\n",
                why, C::NBITS, C::GS, C::N, C::K, C::MT16, C::WK, C::SB, C::D, (int)C::AST, C::PB);
        return 1;
    }
    if (m <= 0) return 0;
    static std::atomic<bool> attr_set{false};        // launch is re-entrant: the attribute call is idempotent, the flag only saves repeats
    if (C::LDS_BYTES > 64 * 1024 && !attr_set.load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&skinny_kernel<C>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)C::LDS_BYTES);
        if (e != hipSuccess) {
            fprintf(stderr, "qfactory skinny: cannot reserve %zu bytes of LDS: %s\n", C::LDS_BYTES, hipGetErrorString(e));
            return 2;
        }
        attr_set.store(true, std::memory_order_release);
    }
    dim3 grid(C::GRID_X, (m + C::BM - 1) / C::BM);
    hipLaunchKernelGGL(skinny_kernel<C>, grid, dim3(C::THREADS), C::LDS_BYTES, stream, (const uint16_t*)A,
                       (const uint8_t*)W, (uint16_t*)Cout, (const uint16_t*)S, (const uint8_t*)Zp, m);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        fprintf(stderr, "qfactory skinny: launch failed: %s\n", hipGetErrorString(err));
        return 2;
    }
    return 0;
}

}  // namespace qf
