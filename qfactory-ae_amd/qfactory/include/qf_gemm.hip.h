// Dequant-fused low-bit GEMM for large M on the gfx950 matrix cores (v_mfma_f32_32x32x16_f16).
//
//   C[m][n] = fp16( sum_k A[m][k] * DQ[n][k] ),   DQ[n][k] = fp16_rn((q[n][k] - Z[n][k/GS]) * s[n][k/GS])
//
// Same packed operands and semantics as the reference's kernel_gptq in eager-decode mode
// (qfactory/include/gptq_gemv.h:14-154, utils.h:46-81).  The reference has no matrix-core path
// (its M is a register-array size, gptq_gemv.h:34); this tiling is this project's own.
//
//   * A block is WK groups of WN waves.  The waves of a group sit side by side along N (a wave
//     owns NT32 x 32 rows of the weight matrix) and share the block's BM activation rows; the
//     groups split K between them (group g takes the 128-byte "supers" g, g + WK, ... of every
//     row) and their accumulators meet once, through LDS, at the end.  Two groups put two waves
//     on every SIMD, so one wave's dequantisation runs under the other's MFMAs.
//   * Weights never exist as an fp16 tile in memory: a lane dequantises exactly the fields of its
//     own MFMA fragment, in registers (in-place mask -> 1024 + 2^o*q, one packed fp16 add/fma to
//     the exact q - Z, one packed fp16 multiply by the scale: bit-identical to the reference's
//     dequantised weight).  The contraction order inside an MFMA is free as long as both operands
//     agree: lane (row, kb) takes the 32 consecutive k of half kb of a 64-wide K-iteration, k-step
//     ks its eight fields 8*ks .. 8*ks+7, and the activation fragment is read to match.
//   * Packed weights travel global -> registers -> LDS in supers of 128 bytes per row (eight lanes
//     share a row: fully coalesced), one to two supers ahead of use, into a buffer private to the wave
//     (no block barrier on that path); a lane then picks its 4*NBITS bytes per K-iteration with
//     one LDS read.  The scales and zero-points of a super are loaded with it and stay in registers.
//   * Activations go from global memory straight into LDS (global_load_lds_dwordx4: no register
//     in between, no ds_write), PA tiles of BM x 64 in LDS per group.  The only wait is an explicit
//     s_waitcnt vmcnt(n) in front of the one block barrier per K-iteration, n being the number of
//     younger loads of the wave, which stay in flight (measured 6-12 % faster at M = 128 .. 256
//     than a register ring with ds_write, whose waits the compiler places itself).  Tiles are read
//     in fragment order with ds_read_b128 (XOR-swizzled columns: conflict-free) one whole
//     iteration before their MFMAs, so that no wave waits on LDS right behind a barrier (measured:
//     the barrier-then-read stall was half of the kernel).
//     Weights are MFMA source A (rows = n), activations source B (columns = m): a lane ends with
//     groups of four consecutive n of one m -> 8-byte stores.
#pragma once

#include <atomic>
#include <cstdio>
#include "qf_dequant.hip.h"

// Timing experiments (results are wrong when non-zero): bit 0 skips the dequantisation arithmetic,
// bit 1 the activation fragment reads, bit 2 the MFMAs, bit 3 the activation tile requests, bit 4 the block
// barrier of the K loop, bit 5 the global weight / scale / zero loads, bit 6 the wait for the activation tiles.
#ifndef QF_GEMM_EXPERIMENT
#define QF_GEMM_EXPERIMENT 0
#endif
#if QF_GEMM_EXPERIMENT != 0 && !defined(QF_ALLOW_TIMING_EXPERIMENTS)
#error "QF_GEMM_EXPERIMENT gives wrong results: timing builds only (define QF_ALLOW_TIMING_EXPERIMENTS)"
#endif

// 1: the wait in front of the K loop's barrier drains every vector-memory load of the wave (vmcnt(0)) instead of
// letting the counted younger loads stay in flight.  The counted wait is only right if the compiled code issues
// exactly the loads `loads_since` counts, in order; the JIT checks that on the generated ISA of every object and
// falls back to this conservative form when the check fails.
#ifndef QF_GEMM_FULL_DRAIN
#define QF_GEMM_FULL_DRAIN 0
#endif
#if QF_GEMM_FULL_DRAIN
#define QF_GEMM_WAIT_DESC " waits=drain"
#else
#define QF_GEMM_WAIT_DESC " waits=counted"
#endif

// When are the packed words of a super requested?  0: all of them in the last iteration of the super three before
// it, into the register slot that has just gone to LDS.  n > 0: in n instalments (16-byte unit p in instalment
// p % n), in the first n iterations of the super two before it.  Every wave of a block requesting a whole super in
// the same iteration, next to that iteration's LDS hand-over and scale loads, was measured (clock stamps per
// iteration) as ~1000 clocks every SUP iterations in which the waves queue behind each other's load instructions
// and no MFMA runs; two instalments take 3 - 13 % off the 4-bit launches.  Supers of fewer than four iterations
// (8 bits) keep the early whole-super request: they need its longer lead (12.4 against 14.2 us on 2048 x 2048 at M = 100).
#ifndef QF_GEMM_SPREAD
#define QF_GEMM_SPREAD 2
#endif

// 1: block -> tile map that keeps the slabs of one column of tiles together on one XCD (see the
// kernel), 0: plain blockIdx order.  The generator switches it on for launches of two to eight slabs (fewer bytes
// past L2 and 4 - 6 % faster there); with one slab there is nothing to share, with many the blocks of an XCD
// share no activation slab any more and the launch fetches four times the bytes.
#ifndef QF_GEMM_XCD_MAP
#define QF_GEMM_XCD_MAP 0
#endif

// 1: the weight matrix is a fused gate+up projection (rows 0 .. N/2-1 gate, rows N/2 .. N-1 up) and the kernel
// writes the (M, N/2) SwiGLU activation out[m][i] = fp16(silu(gate[m][i])) * up[m][i] instead of the (M, N)
// projection.  A wave's TN weight rows alternate between a gate row and its up row (local row r is packed row
// first/2 + r/2 + (r % 2) * N/2), so a lane's four consecutive accumulators of one m are two (gate, up) pairs and
// the epilogue needs nothing from another lane.  Same roundings as the projection followed by qf_silu_mul of
// libqfactory_hip.so (silu_mul_f16 in qf_common.hip.h).  The reference has no such fusion.
#ifndef QF_GEMM_GATE_UP_SILU
#define QF_GEMM_GATE_UP_SILU 0
#endif

// The activation tiles go from global memory to LDS without passing through registers, so this kernel
// cannot convert them on the way: it reads fp16 activations only (its output may be bf16).
static_assert(!QF_IN_BF16, "the GEMM kernel takes fp16 activations: convert bf16 rows before the launch");

namespace qf {

template <int NBITS_, int GS_, bool SYM_, int N_, int K_, int BM_, int NT32_, int WN_, int WK_, int PA_, bool NT_B_>
struct GemmCfg {
    static constexpr int NBITS = NBITS_, GS = GS_, N = N_, K = K_;
    static constexpr bool SYM = SYM_, NT_B = NT_B_;
    static constexpr int BM = BM_;                             // activation rows per block
    static constexpr int NT32 = NT32_;                         // 32-row weight tiles per wave
    static constexpr int WN = WN_;                             // waves along N per group
    static constexpr int WK = WK_;                             // groups along K
    static constexpr int PA = PA_;                             // activation tiles in flight towards LDS
    static constexpr int BK = 64;                              // K-iteration
    static constexpr int TN = 32 * NT32;                       // weight rows per wave
    static constexpr int BN = TN * WN;
    static constexpr int TG = 64 * WN;                         // threads per group
    static constexpr int T = TG * WK;
    static constexpr int MT32 = BM / 32;
    static constexpr int PB = plane_bits(NBITS);               // 3-bit rows: a 2-bit plane plus a 1-bit plane
    static constexpr int ZFB = zero_field_bits(NBITS);         // stored width of one zero-point
    static constexpr bool HI = NBITS == 3;
    static constexpr int SUPK = 1024 / PB;                     // elements of K in 128 bytes of the main plane
    static constexpr int SUP = SUPK / BK;                      // K-iterations per super
    static constexpr int SPREAD = (SUP < 4 || QF_GEMM_SPREAD < 1) ? 0 : (QF_GEMM_SPREAD < SUP ? QF_GEMM_SPREAD : SUP);   // instalments of a super's loads (0: one early request)
    // K need not be a whole number of supers: the last one may hold only TAIL_IT of its SUP iterations.  Its
    // 128-byte window (and those of the 1-bit plane, the scales and the zero-points) is then moved back to end
    // at the end of the row -- every load stays inside the row -- and iteration q of it reads position
    // q + TAIL_SHIFT of the window; the iterations past K are skipped.
    static constexpr int NSUP = (K + SUPK - 1) / SUPK;
    static constexpr int TAIL_IT = (K % SUPK) / BK;            // 0: K is a whole number of supers
    static constexpr bool TAIL = TAIL_IT != 0;
    static constexpr int TAIL_SHIFT = TAIL ? SUP - TAIL_IT : 0;
    static constexpr int SUP_PER_GROUP = (NSUP + WK - 1) / WK;
    static constexpr int ITERS = SUP_PER_GROUP * SUP;          // K-iterations of every group
    static constexpr int UPS = TN * 8 / 64;                    // 16-byte units per lane and super
    static constexpr int AB = BM * (BK / 8) / 64;              // 1 KB blocks (64 16-byte units, 8 rows) of an activation tile
    static constexpr int UA = (AB + WN - 1) / WN;              // activation units per thread and iteration
    static constexpr int LW = PB;                              // main-plane words per lane, tile and iteration
    static constexpr int NGS = SUPK / GS > 0 ? SUPK / GS : 1;  // groups per row and super
    static constexpr int SREGS = (NGS + 1) / 2;                // registers of fp16 scales per tile and super
    static constexpr int ZBITS = NGS * ZFB;                    // zero-point bits per tile and super
    static constexpr int WPP = 128 + 16;                       // packed super row pitch in bytes
    static constexpr int RB = K * NBITS / 8;
    static constexpr int G = K / GS;
    static constexpr int ZRB = G * ZFB / 8;
    static constexpr int HI_OFF = K / 4;                       // byte offset of the 1-bit plane in a 3-bit row
    static constexpr int HPP = 64 + 16;                        // 1-bit-plane super row pitch in bytes
    static constexpr int UPH = TN * 4 / 64;                    // its 16-byte units per lane and super
    static constexpr int GRID_X = (N + BN - 1) / BN;
    // PREFETCH_A: fetch the activation fragments of tile it+1 during iteration it (a second register
    // set of 16 * MT32 registers); tall tiles read each fragment just before its MFMAs instead
    static constexpr bool PREFETCH_A = BM / 32 <= 4;
    // activation tiles in LDS per group: tile t lives in buffer t % PA.  With fragment prefetch a
    // tile is requested at the end of an iteration, PA tiles ahead, into the buffer whose tile went
    // to registers an iteration ago; without, at the start of an iteration, PA - 1 tiles ahead, into
    // the buffer every wave finished reading before the barrier that has just been passed.
    static constexpr int NBUF = PA;
    static constexpr int ROWB = BK * 2;                        // bytes of one activation tile row in LDS
    static constexpr size_t LDS_A = (size_t)WK * NBUF * BM * ROWB;
    // vector-memory loads of one super per wave (packed words, 1-bit plane, scales, zero-points)
    static constexpr int SUPER_LOADS = UPS + (HI ? UPH : 0) + NT32 * (SYM ? 1 : 2);
    static constexpr size_t LDS_W = (size_t)WK * WN * TN * (WPP + (HI ? HPP : 0));
    static constexpr size_t LDS_RED = WK > 1 ? (size_t)(WK - 1) * BM * BN * 4 : 0;
    static constexpr size_t LDS_FRONT = LDS_A > LDS_RED ? LDS_A : LDS_RED;
    static constexpr size_t LDS_BYTES = LDS_FRONT + LDS_W;
    static constexpr int ACC_PER_THREAD = MT32 * NT32 * 16;
};

template <int V> struct IntTag { static constexpr int value = V; };
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(IntTag<I>{});
        static_for<I + 1, N>(f);
    }
}

// s_waitcnt immediate of gfx9: vmcnt in bits 3:0 and 15:14, expcnt (not waited for) in 6:4, lgkmcnt in 11:8
constexpr int waitcnt_imm(int vmcnt, int lgkmcnt) {
    const int vm = vmcnt > 63 ? 63 : vmcnt;
    return (vm & 0xF) | ((vm >> 4) << 14) | (0x7 << 4) | ((lgkmcnt & 0xF) << 8);
}

// Wait until at most ALLOWED of this wave's vector-memory loads (in issue order) and none of its
// LDS operations are outstanding, then meet the block's other waves.  A bare s_barrier: the
// fence of __syncthreads() would wait for every outstanding load.
template <int ALLOWED, bool BARRIER = true>
__device__ __forceinline__ void wait_loads_and_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(ALLOWED, 0));
    if constexpr (BARRIER) __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// 16 bytes per lane from global memory straight into LDS (no register in between): lane l's
// bytes land at lds + 16*l, `lds` being the same for the whole wave; counted by vmcnt like a load.
__device__ __forceinline__ void load_to_lds_16(const void* global, void* lds) {
    __builtin_amdgcn_global_load_lds(global, (__attribute__((address_space(3))) void*)lds, 16, 0, 0);
}

// Vector-memory loads of one super that a wave issues in iteration q of a super: its instalment of packed words
// (and of the 1-bit plane), and in the last iteration the scales and zero-points.
template <class C>
constexpr int super_loads_at(int q) {
    if (C::SPREAD == 0) return q == C::SUP - 1 ? C::SUPER_LOADS : 0;
    int n = 0;
    for (int p = 0; p < C::UPS; p++) n += (p % C::SPREAD == q) ? 1 : 0;
    if (C::HI)
        for (int p = 0; p < C::UPH; p++) n += (p % C::SPREAD == q) ? 1 : 0;
    if (q == C::SUP - 1) n += C::NT32 * (C::SYM ? 1 : 2);
    return n;
}
// Vector-memory loads a wave issues in the `back` iterations that end with iteration s (s counted
// modulo the super): UA activation loads each, plus that iteration's share of a super.
template <class C>
constexpr int loads_since(int s, int back) {
    int n = 0;
    for (int d = 0; d < back; d++)
        n += C::UA + super_loads_at<C>(((s - d) % C::SUP + C::SUP) % C::SUP);
    return n;
}

template <class C>
__global__ __launch_bounds__(C::T) void gemm_kernel(
    const uint16_t* __restrict__ A, const uint8_t* __restrict__ W, uint16_t* __restrict__ Cout,
    const uint16_t* __restrict__ S, const uint8_t* __restrict__ Zp, int m_total) {
    constexpr int BM = C::BM, BK = C::BK, WN = C::WN, WK = C::WK, TN = C::TN;
    constexpr int MT32 = C::MT32, NT32 = C::NT32, WPP = C::WPP;
    constexpr int SUP = C::SUP, UPS = C::UPS, UA = C::UA, LW = C::LW, NGS = C::NGS, SREGS = C::SREGS;
    constexpr uint32_t ZMASK = (1u << C::ZFB) - 1u;
    constexpr bool SILU = QF_GEMM_GATE_UP_SILU != 0;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    // wave-uniform indices live in scalar registers: every global address below is then a scalar
    // base (advanced with scalar adds) plus a 32-bit per-lane offset computed once
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave % WN, grp = wave / WN;
    const int li = lane & 31, kb = lane >> 5;

    // activation tiles live at the start of LDS (the final cross-group sum reuses that space)
    uint8_t* as_b = smem + (size_t)grp * C::NBUF * BM * C::ROWB;                           // [NBUF][BM][ROWB]
    uint8_t* wp = smem + C::LDS_FRONT + (size_t)wave * TN * (WPP + (C::HI ? C::HPP : 0));  // [TN][WPP] (+ [TN][HPP])
    uint8_t* hp = wp + TN * WPP;

    // Block -> tile map.  The hardware deals workgroups round-robin to the 8 XCDs (linear id % 8),
    // each with its own L2, in linear-id order.  The BM-row slabs of one column of tiles read the
    // same weight rows: they get ids 8 apart (same XCD, dispatched together), so the weights come
    // from HBM once and the other slabs hit in that XCD's L2.  With the plain (x, y) order the
    // slabs of a column are gridDim.x ids apart: once there are more tiles than CUs they run at
    // different times and every slab fetches the weights from memory again (measured with
    // FETCH_SIZE: 552 MB instead of 240 MB on the 57344 x 8192 layer at M = 256).
    const int linear = blockIdx.x + gridDim.x * blockIdx.y;
    int col = blockIdx.x, slab = blockIdx.y;
    if (QF_GEMM_XCD_MAP && C::GRID_X >= 8) {
        const int per_group = 8 * gridDim.y;                    // tiles of 8 columns
        const int full = C::GRID_X / 8 * per_group;             // ids of the whole groups of 8 columns
        if (linear < full) {
            const int grp8 = linear / per_group, rem = linear % per_group;
            col = grp8 * 8 + rem % 8;
            slab = rem / 8;
        } else {                                                // the last, narrower group: plain order inside it
            constexpr int LAST = C::GRID_X % 8 ? C::GRID_X % 8 : 8;
            const int rem = linear - full;
            col = C::GRID_X / 8 * 8 + rem % LAST;
            slab = rem / LAST;
        }
    }
    const int n_blk = col * C::BN;
    const int m_blk = slab * BM;
    const int n_wave = n_blk + wn * TN;

    // K offset of the group's iteration `it`: supers are dealt round-robin to the groups; a group
    // past the last super re-reads the last one and drops the products
    auto k_of = [&](int it) {
        const int sup = min((it / SUP) * WK + grp, C::NSUP - 1);
        const int k = sup * C::SUPK + (it % SUP) * BK;
        return C::TAIL ? min(k, C::K - BK) : k;                 // skipped iterations of a partial last super re-read the last tile
    };
    // does local super P of this group map to the partial last super (groups past the end re-read it)?
    auto is_tail = [&](int sup_local) { return C::TAIL && sup_local * WK + grp >= C::NSUP - 1; };

    // ---- activations: UA 16-byte units per lane and iteration, global memory -> LDS ----
    // Instruction p of wave wn fills the 1 KB of 16-byte slots (p*WN + wn)*64 .. +63 of the tile
    // (the hardware writes the 64 lanes' 16 bytes back to back); where WN does not divide the tile's
    // AB blocks, the instructions past the last block fetch the last block once more -- same bytes to
    // the same place -- so that every wave issues the same number of loads (the waits count them);
    // slot 8*row + (c ^ (row/2 % 8))
    // holds columns 8c .. 8c+7 of a row: an XOR swizzle instead of row padding.  A 16-byte fragment
    // read is served 16 lanes (= 16 rows, one column slot) at a time; rows 2a and 2a+1 start 32
    // banks apart and the eight values of a move the slot to eight different 4-bank groups: no
    // conflicts.
    uint32_t a_off[UA];                                        // byte offset of this lane's units inside the slab
#pragma unroll
    for (int p = 0; p < UA; p++) {
        const int u = min(p * WN + wn, C::AB - 1) * 64 + lane;
        const int row = u / 8, c8 = (u % 8) ^ ((row >> 1) & 7);
        a_off[p] = ((uint32_t)min(row, m_total - 1 - m_blk) * C::K + c8 * 8) * 2u;   // rows past the end re-read the last one
    }
    const uint8_t* a_slab = reinterpret_cast<const uint8_t*>(A + (size_t)m_blk * C::K);
    // tile `it` of the group into LDS buffer `buf`, asynchronously
    auto load_a = [&](int buf, int it) {
        if (QF_GEMM_EXPERIMENT & 8) return;
        const uint8_t* base = a_slab + (size_t)k_of(it) * 2;
        uint8_t* dst = as_b + (size_t)buf * BM * C::ROWB;
#pragma unroll
        for (int p = 0; p < UA; p++) load_to_lds_16(base + a_off[p], dst + (size_t)min(p * WN + wn, C::AB - 1) * 1024);
    };

    // ---- one super of this wave's TN weight rows: packed fields, scales, zero-points ----
    struct Quant { uint32_t s[NT32][SREGS]; uint32_t z[NT32]; };
    struct WStage { u32x4 w[UPS]; u32x4 h[C::HI ? C::UPH : 1]; };
    uint32_t w_off[UPS], h_off[C::HI ? C::UPH : 1], s_off[NT32], z_off[NT32];   // per-lane byte offsets from the wave's first row
    // first packed row of the wave and the packed row of its local row r, relative to it.  Plain: rows n_wave + r,
    // clamped to the last row (a wave wholly past the last row re-reads it).  Gate+up (N a multiple of TN, so a
    // wave is inside or wholly outside): local rows 2i, 2i+1 are gate row first/2 + i and its up row N/2 further on.
    const int n_base = SILU ? min(n_wave, C::N - TN) / 2 : min(n_wave, C::N - 1);
    auto rel_row = [&](int r) { return SILU ? (r >> 1) + (r & 1) * (C::N / 2) : min(r, C::N - 1 - n_base); };
#pragma unroll
    for (int p = 0; p < UPS; p++) {
        const int u = lane + 64 * p;
        w_off[p] = (uint32_t)rel_row(u / 8) * C::RB + (u % 8) * 16;
    }
    if constexpr (C::HI) {
#pragma unroll
        for (int p = 0; p < C::UPH; p++) {
            const int u = lane + 64 * p;                        // four lanes share a row: 64 bytes per super
            h_off[p] = (uint32_t)rel_row(u / 4) * C::RB + C::HI_OFF + (u % 4) * 16;
        }
    }
#pragma unroll
    for (int j = 0; j < NT32; j++) {
        const uint32_t row = (uint32_t)rel_row(j * 32 + li);
        s_off[j] = row * C::G * 2u;
        z_off[j] = row * C::ZRB;
    }
    const uint8_t* w_rows = W + (size_t)n_base * C::RB;
    const uint8_t* s_rows = reinterpret_cast<const uint8_t*>(S + (size_t)n_base * C::G);
    const uint8_t* z_rows = Zp + (size_t)n_base * C::ZRB;
    // instalment `part` of the super (part < 0: all of it)
    auto load_super = [&](WStage& st, int sup_local, int part) {
        if (QF_GEMM_EXPERIMENT & 32) return;
        const int sup = min(sup_local * WK + grp, C::NSUP - 1);
        // byte offset of the super's window in the main plane (half of it in the 1-bit plane); wave-uniform, and
        // opaque: requests past the end clamp to the same window and must not be merged (see the end of the K loop)
        uint32_t woff = __builtin_amdgcn_readfirstlane(is_tail(sup_local) ? (uint32_t)(C::K * C::PB / 8 - 128) : (uint32_t)sup * 128u);
        asm volatile("" : "+s"(woff));
        const uint8_t* wb = w_rows + woff;
#pragma unroll
        for (int p = 0; p < UPS; p++) {
            if (part >= 0 && p % (C::SPREAD ? C::SPREAD : 1) != part) continue;
            const uint8_t* src = wb + w_off[p];
            st.w[p] = C::NT_B ? __builtin_nontemporal_load((const u32x4*)src) : *(const u32x4*)src;
        }
        if constexpr (C::HI) {
            const uint8_t* hb = w_rows + woff / 2;
#pragma unroll
            for (int p = 0; p < C::UPH; p++) {
                if (part >= 0 && p % (C::SPREAD ? C::SPREAD : 1) != part) continue;
                const uint8_t* src = hb + h_off[p];
                st.h[p] = C::NT_B ? __builtin_nontemporal_load((const u32x4*)src) : *(const u32x4*)src;
            }
        }
    };
    auto load_quant = [&](Quant& qu, int sup_local) {
        if (QF_GEMM_EXPERIMENT & 32) return;
        const int sup = min(sup_local * WK + grp, C::NSUP - 1);
        // first group of the super's window (a partial last super: the window ends at the last group); opaque, as in load_super
        int g0 = __builtin_amdgcn_readfirstlane(is_tail(sup_local) ? (C::K - C::SUPK) / C::GS : sup * C::SUPK / C::GS);
        asm volatile("" : "+s"(g0));
        const uint8_t* sb = s_rows + (size_t)g0 * 2;
        const uint8_t* zb = z_rows + (g0 * C::ZFB) / 8;
#pragma unroll
        for (int j = 0; j < NT32; j++) {
            const uint8_t* sp = sb + s_off[j];
            if constexpr (NGS == 1) {
                qu.s[j][0] = *reinterpret_cast<const uint16_t*>(sp);
            } else if constexpr (NGS == 2) {
                qu.s[j][0] = *reinterpret_cast<const uint32_t*>(sp);
            } else if constexpr (NGS == 4) {
                const u32x2 v = *reinterpret_cast<const u32x2*>(sp);
                qu.s[j][0] = v.x; qu.s[j][1] = v.y;
            } else {
                const u32x4 v = *reinterpret_cast<const u32x4*>(sp);
                qu.s[j][0] = v.x; qu.s[j][1] = v.y; qu.s[j][2] = v.z; qu.s[j][3] = v.w;
            }
            qu.z[j] = 0;
            if constexpr (!C::SYM) {
                const uint8_t* zp = zb + z_off[j];
                if constexpr (C::ZBITS >= 32) qu.z[j] = *reinterpret_cast<const uint32_t*>(zp);
                else if constexpr (C::ZBITS == 16) qu.z[j] = *reinterpret_cast<const uint16_t*>(zp);
                else if constexpr (C::ZBITS == 8) qu.z[j] = *zp;
                else qu.z[j] = (uint32_t)*zp >> ((g0 * C::ZFB) % 8);         // fewer than 8 bits: inside one byte
            }
        }
    };
    auto store_super = [&](const WStage& st) {
#pragma unroll
        for (int p = 0; p < UPS; p++) {
            const int u = lane + 64 * p;
            *reinterpret_cast<u32x4*>(wp + (u / 8) * WPP + (u % 8) * 16) = st.w[p];
        }
        if constexpr (C::HI) {
#pragma unroll
            for (int p = 0; p < C::UPH; p++) {
                const int u = lane + 64 * p;
                *reinterpret_cast<u32x4*>(hp + (u / 4) * C::HPP + (u % 4) * 16) = st.h[p];
            }
        }
    };
    // this lane's packed fields of iteration q of the super in LDS: 32 fields = 4*NBITS bytes per tile
    struct Packed { uint32_t w[NT32][LW >= 4 ? LW : 4]; uint32_t h[NT32]; };
    auto read_packed = [&](Packed& pk, int q) {
#pragma unroll
        for (int j = 0; j < NT32; j++) {
            const uint8_t* src = wp + (j * 32 + li) * WPP + (q * BK + 32 * kb) * C::PB / 8;
            if constexpr (C::HI) pk.h[j] = *reinterpret_cast<const uint32_t*>(hp + (j * 32 + li) * C::HPP + (q * BK + 32 * kb) / 8);
            if constexpr (LW == 2) {
                const u32x2 v = *reinterpret_cast<const u32x2*>(src);
                pk.w[j][0] = v.x; pk.w[j][1] = v.y; pk.w[j][2] = 0; pk.w[j][3] = 0;
            } else {
#pragma unroll
                for (int h = 0; h < LW / 4; h++) {
                    const u32x4 v = *reinterpret_cast<const u32x4*>(src + 16 * h);
                    pk.w[j][4 * h] = v.x; pk.w[j][4 * h + 1] = v.y; pk.w[j][4 * h + 2] = v.z; pk.w[j][4 * h + 3] = v.w;
                }
            }
        }
    };
    // dequantisation constants of tile j in iteration q of the current super; the group of this
    // lane's 32 fields is a compile-time index unless a group is only 32 wide
    auto qconst_raw = [&](const Quant& qu, int j, int q, uint32_t& sbits, uint32_t& zero) {
        if constexpr (C::GS >= C::SUPK) {
            sbits = qu.s[j][0] & 0xFFFFu;
            zero = qu.z[j] & ZMASK;
        } else if constexpr (C::GS >= BK) {
            const int gi = q * BK / C::GS;
            sbits = (qu.s[j][gi / 2] >> (16 * (gi % 2))) & 0xFFFFu;
            zero = (qu.z[j] >> (gi * C::ZFB)) & ZMASK;
        } else {                                               // GS == 32: group 2q + kb
            sbits = kb ? (qu.s[j][q] >> 16) : (qu.s[j][q] & 0xFFFFu);
            zero = (qu.z[j] >> ((2 * q + kb) * C::ZFB)) & ZMASK;
        }
        if constexpr (C::SYM) zero = 1u << (C::NBITS - 1);
    };
    // q is a compile-time constant at every call site; in a partial last super (`tail`, wave-uniform) the
    // window position is q + TAIL_SHIFT: both candidates are extracted and one is selected
    auto qconst_of = [&](const Quant& qu, int j, int q, bool tail) {
        uint32_t sbits, zero;
        qconst_raw(qu, j, q, sbits, zero);
        if constexpr (C::TAIL) {
            uint32_t sbits_t, zero_t;
            qconst_raw(qu, j, min(q + C::TAIL_SHIFT, SUP - 1), sbits_t, zero_t);
            sbits = tail ? sbits_t : sbits;
            zero = tail ? zero_t : zero;
        }
        return make_qconst<C::NBITS>((uint16_t)sbits, zero);
    };

    f32x16 acc[NT32][MT32];
#pragma unroll
    for (int j = 0; j < NT32; j++)
#pragma unroll
        for (int i = 0; i < MT32; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[j][i][v] = 0.0f;

    // activation fragments of one tile: k-step ks of 32-row block i is row li, columns 32*kb + 8*ks .. + 7
    uint32_t a_frag_off[4];                                    // swizzled byte offset of k-step ks
#pragma unroll
    for (int ks = 0; ks < 4; ks++) a_frag_off[ks] = (uint32_t)li * C::ROWB + (((4 * kb + ks) ^ ((li >> 1) & 7)) * 16);
    auto frag_of = [&](int buf, int i, int ks) {
        return *reinterpret_cast<const f16x8*>(as_b + ((size_t)buf * BM + i * 32) * C::ROWB + a_frag_off[ks]);
    };
    struct AFrags { f16x8 f[MT32][4]; };
    auto read_frags = [&](AFrags& fr, int buf) {
#pragma unroll
        for (int i = 0; i < MT32; i++)
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                if (QF_GEMM_EXPERIMENT & 2) fr.f[i][ks] = __builtin_bit_cast(f16x8, u32x4{(uint32_t)buf, 1u, 2u, 3u});
                else fr.f[i][ks] = frag_of(buf, i, ks);
            }
    };

    WStage ringW[2];            // packed words of the two supers after the one in LDS
    Quant ringQ[2];             // scales and zero-points: slot P % 2 serves super P for its whole duration
    Packed cur, nxt;
    AFrags fcur, fnxt;

    // One K-iteration; s = it % (2*SUP) is a compile-time constant at every call site; b0, b1 and
    // b2 are the LDS buffers of tiles it, it+1 and it+PA-1 (tile t lives in buffer t % PA; tile
    // it+PA shares b0).
    //   * the fragments of tile it+1 (complete in LDS since the last barrier) are fetched now and
    //     used in the next iteration: no wave waits on LDS right after a barrier;
    //   * the MFMAs of tile it run on registers filled one iteration ago, interleaved with the
    //     dequantisation of their weight fragments;
    //   * tile it+PA is requested into the buffer whose tile every wave has finished reading
    //     before the last barrier; past the end of K the last tile is requested again, so that
    //     the count of loads in flight stays what the waits below assume.
    auto iteration = [&](int it, auto s_tag, int b0, int b1, int b2) __attribute__((always_inline)) {
        constexpr int s = decltype(s_tag)::value;
        const int q = s % SUP, pslot = (s / SUP) & 1;
        const int P = it / SUP;                                 // super index inside the group
        if constexpr (C::PREFETCH_A) read_frags(fnxt, b1);
        else load_a(b2, min(it + C::PA - 1, C::ITERS - 1));
        // every read of the current super has been issued one iteration ago: the next super
        // (loaded two supers back) takes its place in LDS
        if (q == SUP - 1) store_super(ringW[pslot ^ 1]);
        const bool tail = is_tail(P);
        {
            const int qn = (q + 1) % SUP;                       // the next iteration and the super it belongs to
            const bool tail_n = is_tail(q == SUP - 1 ? P + 1 : P);
            read_packed(nxt, C::TAIL && tail_n ? min(qn + C::TAIL_SHIFT, SUP - 1) : qn);
        }
        const bool live = (WK == 1 || (P * WK + grp < C::NSUP)) && !(C::TAIL && tail && q >= C::TAIL_IT);
        if (live) {
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                f16x8 wf[NT32], af[MT32];
#pragma unroll
                for (int i = 0; i < MT32; i++) {
                    if constexpr (C::PREFETCH_A) af[i] = fcur.f[i][ks];
                    else if (QF_GEMM_EXPERIMENT & 2) af[i] = __builtin_bit_cast(f16x8, u32x4{(uint32_t)b0, 1u, 2u, 3u});
                    else af[i] = frag_of(b0, i, ks);
                }
#pragma unroll
                for (int j = 0; j < NT32; j++) {
                    const QConst qc = qconst_of(ringQ[pslot], j, q, tail);
                    if constexpr ((QF_GEMM_EXPERIMENT & 1) != 0) {
                        wf[j] = __builtin_bit_cast(f16x8, u32x4{cur.w[j][0], cur.w[j][1], cur.w[j][2], cur.w[j][3] + (uint32_t)ks});
                    } else if constexpr (C::NBITS == 3) {
                        const uint32_t w4[4] = {cur.w[j][0], cur.w[j][1], 0u, 0u};
                        wf[j] = ks == 0 ? DequantStep3::run<0>(w4, cur.h[j], qc) : ks == 1 ? DequantStep3::run<1>(w4, cur.h[j], qc)
                              : ks == 2 ? DequantStep3::run<2>(w4, cur.h[j], qc) : DequantStep3::run<3>(w4, cur.h[j], qc);
                    } else if constexpr (C::NBITS == 8) {
                        const int h = 4 * (ks / 2);
                        const uint32_t w4[4] = {cur.w[j][h], cur.w[j][h + 1], cur.w[j][h + 2], cur.w[j][h + 3]};
                        wf[j] = DequantStep<8>::run(w4, ks % 2, qc);
                    } else {
                        const uint32_t w4[4] = {cur.w[j][0], cur.w[j][1], cur.w[j][2], cur.w[j][3]};
                        wf[j] = DequantStep<C::NBITS>::run(w4, ks, qc);
                    }
                }
#pragma unroll
                for (int j = 0; j < NT32; j++)
#pragma unroll
                    for (int i = 0; i < MT32; i++)
                        if (QF_GEMM_EXPERIMENT & 4) acc[j][i][ks] += (float)wf[j][0] * (float)af[i][0];
                        else acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[j], af[i], acc[j][i], 0, 0, 0);
            }
        }
        if constexpr (C::PREFETCH_A) load_a(b0, min(it + C::PA, C::ITERS - 1));
        cur = nxt;
        if constexpr (C::PREFETCH_A) fcur = fnxt;
        // The register slot whose super went to LDS when this super began (slot pslot) takes the super two after
        // this one, an instalment per iteration; the quantisation slot of the super that ends here goes to the
        // one after next (no register is copied: a copy of a loaded value at the loop's back-edge would wait
        // for every load in flight).
        if constexpr (C::SPREAD > 0) {
            if (q < C::SPREAD) load_super(ringW[pslot], P + 2, q);
        } else {
            if (q == SUP - 1) load_super(ringW[pslot ^ 1], P + 3, -1);          // the slot that went to LDS in this iteration
        }
        if (q == SUP - 1) load_quant(ringQ[pslot], P + 2);
        // Publish the tile the next iteration reads (tile it+2 with fragment prefetch, else it+1).
        // Either way its request is PA - 2 whole iterations old, and every vector-memory load the
        // wave has issued in those iterations (activation tiles and whole supers) may stay in
        // flight.  Loads return in order; what the requesting iteration itself issued next to the
        // request is not counted, wherever the compiler placed it.
        wait_loads_and_barrier<QF_GEMM_FULL_DRAIN ? 0 : ((QF_GEMM_EXPERIMENT & (8 | 64)) ? 63 : loads_since<C>(s, C::PA - 2)), !(QF_GEMM_EXPERIMENT & 16)>();
    };

    // ---- prologue: supers 0, 1 (with the early request: then 2) and activation tiles 0 .. PA-1 requested, all complete at the barrier ----
    load_super(ringW[0], 0, -1);
    load_quant(ringQ[0], 0);
    load_super(ringW[1], 1, -1);
    load_quant(ringQ[1], 1);
#pragma unroll
    for (int p = 0; p < (C::PREFETCH_A ? C::PA : C::PA - 1); p++) load_a(p, min(p, C::ITERS - 1));
    store_super(ringW[0]);
    if constexpr (C::SPREAD == 0) load_super(ringW[0], 2, -1);
    read_packed(cur, is_tail(0) ? C::TAIL_SHIFT : 0);
    wait_loads_and_barrier<0>();
    if constexpr (C::PREFETCH_A) read_frags(fcur, 0);

    // The K loop runs whole passes of 2*SUP iterations (the period of the register rings); what is left over is
    // a straight-line tail behind it.  No iteration is skipped by a branch inside the loop, so every path through
    // the loop issues the same loads -- which is what the wait counts assume and what the JIT re-counts on the ISA.
    constexpr int PASS = 2 * SUP, FULL_PASSES = C::ITERS / PASS, REST = C::ITERS % PASS;
    int b0 = 0, b1 = 1, b2 = C::PA - 1;
    auto step = [&](int it, auto s_tag) __attribute__((always_inline)) {
        iteration(it, s_tag, b0, b1, b2);
        b0 = b1;
        b1 = b1 == C::NBUF - 1 ? 0 : b1 + 1;
        b2 = b2 == C::NBUF - 1 ? 0 : b2 + 1;
    };
#pragma unroll 1
    for (int pass = 0; pass < FULL_PASSES; pass++)
        static_for<0, PASS>([&](auto s_tag) { step(pass * PASS + decltype(s_tag)::value, s_tag); });
    static_for<0, REST>([&](auto s_tag) { step(FULL_PASSES * PASS + decltype(s_tag)::value, s_tag); });
    // The wait counts above assume that every iteration really issues the loads `loads_since` counts.  What
    // the last iterations load for supers past the end is never used, and a compiler that can see that (a
    // K loop of a single trip) drops those loads or merges them (they all clamp to the last super): fewer
    // loads in flight than counted, and the wait lets an activation tile that is about to be read stay in
    // flight.  The super index is opaque to the compiler where the loads are issued, and naming the ring
    // registers here keeps every load alive, at no cost (no instruction is emitted; the drain below waits
    // for them anyway).
#pragma unroll
    for (int r = 0; r < 2; r++) {
#pragma unroll
        for (int p = 0; p < UPS; p++) asm volatile("" ::"v"(ringW[r].w[p]));
        if constexpr (C::HI) {
#pragma unroll
            for (int p = 0; p < C::UPH; p++) asm volatile("" ::"v"(ringW[r].h[p]));
        }
#pragma unroll
        for (int j = 0; j < NT32; j++) {
#pragma unroll
            for (int i = 0; i < SREGS; i++) asm volatile("" ::"v"(ringQ[r].s[j][i]));
            asm volatile("" ::"v"(ringQ[r].z[j]));
        }
    }
    // the repeated activation requests of the last iterations still target LDS: drain them before
    // the space is reused below or the wave ends
    wait_loads_and_barrier<0>();

    // ---- the groups' partial sums meet in LDS (the activation tiles are no longer needed) ----
    if constexpr (WK > 1) {
        float* red = reinterpret_cast<float*>(smem);
        constexpr int PER_GROUP = C::BM * C::BN;                // floats of one group's partial tile
        constexpr int PER_WAVE = NT32 * MT32 * 16 * 64;
        if (grp > 0) {
            float* mine = red + (size_t)(grp - 1) * PER_GROUP + (size_t)wn * PER_WAVE + lane;
#pragma unroll
            for (int j = 0; j < NT32; j++)
#pragma unroll
                for (int i = 0; i < MT32; i++)
#pragma unroll
                    for (int v = 0; v < 16; v++) mine[((j * MT32 + i) * 16 + v) * 64] = acc[j][i][v];
        }
        __syncthreads();
        if (grp > 0) return;
#pragma unroll
        for (int g = 1; g < WK; g++) {
            const float* other = red + (size_t)(g - 1) * PER_GROUP + (size_t)wn * PER_WAVE + lane;
#pragma unroll
            for (int j = 0; j < NT32; j++)
#pragma unroll
                for (int i = 0; i < MT32; i++)
#pragma unroll
                    for (int v = 0; v < 16; v++) acc[j][i][v] += other[((j * MT32 + i) * 16 + v) * 64];
        }
    }

    // ---- store: accumulator register v of a 32x32 tile is (n = 8*(v/4) + 4*(lane/32) + v%4, m = lane%32) ----
#pragma unroll
    for (int i = 0; i < MT32; i++) {
        const int m = m_blk + i * 32 + li;
        if (m >= m_total) continue;
#pragma unroll
        for (int j = 0; j < NT32; j++) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int n = n_wave + j * 32 + 8 * q + 4 * kb;
                if constexpr (SILU) {
                    // columns n, n+1 and n+2, n+3 are (gate, up) of outputs n/2 and n/2 + 1
                    if (n < C::N) {
                        const uint32_t lo = silu_mul_f16(acc[j][i][4 * q], acc[j][i][4 * q + 1]);
                        const uint32_t hi = silu_mul_f16(acc[j][i][4 * q + 2], acc[j][i][4 * q + 3]);
                        *reinterpret_cast<uint32_t*>(Cout + (size_t)m * (C::N / 2) + (n >> 1)) = lo | (hi << 16);
                    }
                    continue;
                }
                uint16_t h[4];
#pragma unroll
                for (int e = 0; e < 4; e++) h[e] = f32_to_out_bits(acc[j][i][4 * q + e]);
                uint16_t* dst = Cout + (size_t)m * C::N + n;
                if constexpr (C::N % 4 == 0) {
                    if (n < C::N) {
                        if constexpr (QF_OUT_ACCUMULATE != 0) {
                            // out = fp16(out + fp16(projection)): the lane reads the four elements it is about to write
                            const u32x2 old = *reinterpret_cast<const u32x2*>(dst);
                            const uint16_t o[4] = {(uint16_t)old.x, (uint16_t)(old.x >> 16), (uint16_t)old.y, (uint16_t)(old.y >> 16)};
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                h[e] = __builtin_bit_cast(uint16_t, (_Float16)(__builtin_bit_cast(_Float16, o[e]) + __builtin_bit_cast(_Float16, h[e])));
                        }
                        *reinterpret_cast<u32x2*>(dst) = u32x2{(uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16)};
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (n + e < C::N) store_out(dst + e, acc[j][i][4 * q + e]);
                }
            }
        }
    }
}

template <class C>
int gemm_launch(const void* A, const void* W, void* Cout, const void* S, const void* Zp, int m, hipStream_t stream) {
    const char* why = nullptr;
    if (C::NBITS != 2 && C::NBITS != 3 && C::NBITS != 4 && C::NBITS != 8) why = "NBITS must be 2, 3, 4 or 8";
    else if (C::BM % 32 != 0 || C::BM <= 0 || C::NT32 < 1 || C::WN < 1 || C::WK < 1) why = "BM must be a multiple of 32; NT32, WN, WK positive";
    else if (C::T > 1024) why = "block too large";
    else if (C::K % C::BK != 0 || C::K < C::SUPK) why = "K must be a multiple of 64 and hold at least 128 packed bytes of the main plane";
    else if ((C::K % C::SUPK) * C::PB / 8 % (C::HI ? 32 : 16) != 0) why = "a partial last 128-byte window must be whole 16-byte units in every plane";
    else if (C::GS <= 0 || C::K % C::GS != 0) why = "GS must divide K";
    else if (C::GS % 32 != 0) why = "a lane's 32 fields must lie inside one group (GS multiple of 32)";
    else if (C::GS < C::SUPK && C::SUPK % C::GS != 0) why = "GS must divide 1024/NBITS or be a multiple of it";
    else if (C::GS > C::SUPK && C::GS % C::SUPK != 0) why = "GS must divide 1024/NBITS or be a multiple of it";
    else if (C::NGS > 8 || C::ZBITS > 32) why = "too many groups per 128 packed bytes";
    else if (!C::SYM && (C::G % (8 / C::ZFB)) != 0) why = "K/GS must fill whole zero-point bytes";
    else if (C::PA < 3 || C::PA > 12) why = "PA (activation tiles in flight) must be 3 .. 12";
    else if (C::LDS_BYTES > 160 * 1024) why = "tiles exceed the 160 KB of LDS";
    else if (C::ACC_PER_THREAD > 256) why = "accumulator tile exceeds the register file";
    else if (QF_GEMM_GATE_UP_SILU && (C::N % 2 != 0 || C::N % C::TN != 0)) why = "gate+up rows come in pairs inside a wave: N must be a multiple of 32 * NT32";
    else if (QF_GEMM_GATE_UP_SILU && QF_OUT_BF16) why = "the SwiGLU epilogue is fp16 only";
    else if (QF_OUT_ACCUMULATE && (QF_OUT_BF16 || QF_GEMM_GATE_UP_SILU)) why = "adding to the output is fp16 only and not combined with the SwiGLU epilogue";
    else if (QF_GEMM_GATE_UP_SILU && ((size_t)C::N / 2 + C::TN) * C::RB >= ((size_t)1 << 32)) why = "gate+up: half the packed weight does not fit a 32-bit row offset";
    if (why) {
        fprintf(stderr, "qfactory gemm: invalid configuration: %s (NBITS=%d GS=%d N=%d K=%d BM=%d NT32=%d WN=%d WK=%d PA=%d)\n",
                why, C::NBITS, C::GS, C::N, C::K, C::BM, C::NT32, C::WN, C::WK, C::PA);
        return 1;
    }
    if (m <= 0) return 0;
    static std::atomic<bool> attr_set{false};        // launch is re-entrant: the attribute call is idempotent, the flag only saves repeats
    if (C::LDS_BYTES > 64 * 1024 && !attr_set.load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_kernel<C>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)C::LDS_BYTES);
        if (e != hipSuccess) {
            fprintf(stderr, "qfactory gemm: cannot reserve %zu bytes of LDS: %s\n", C::LDS_BYTES, hipGetErrorString(e));
            return 2;
        }
        attr_set.store(true, std::memory_order_release);
    }
    dim3 grid(C::GRID_X, (m + C::BM - 1) / C::BM);
    hipLaunchKernelGGL(gemm_kernel<C>, grid, dim3(C::T), C::LDS_BYTES, stream, (const uint16_t*)A, (const uint8_t*)W,
                       (uint16_t*)Cout, (const uint16_t*)S, (const uint8_t*)Zp, m);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        fprintf(stderr, "qfactory gemm: launch failed: %s\n", hipGetErrorString(err));
        return 2;
    }
    return 0;
}

}  // namespace qf
