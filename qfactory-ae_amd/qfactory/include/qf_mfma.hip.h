// Dequant-fused low-bit GEMM on the gfx950 matrix cores (v_mfma_f32_16x16x32_f16), for M above
// the register-resident GEMV's range.
//
//   C[m][n] = fp16( sum_k A[m][k] * DQ[n][k] ),   DQ[n][k] = fp16_rn((q[n][k] - Z[n][k/GS]) * s[n][k/GS])
//
// Same packed operands and semantics as the reference's kernel_gptq in eager-decode mode
// (qfactory/include/gptq_gemv.h:14-154, utils.h:46-81); the reference has no matrix-core path
// (its M is a register-array size, gptq_gemv.h:34), so the tiling below is this project's own.
//
// Roles: the packed weights are MFMA source A (rows i = n), the activations source B (columns
// j = m), so a lane ends up with four consecutive n of one m -- an 8-byte store into row-major C.
//
// Per wave and K-iteration (BK = 4 * 128/NBITS elements):
//   * weights: one 16-byte global load per lane and n-tile straight into fragment layout -- lane
//     (r = lane%16, kb = lane/16) takes the 128/NBITS consecutive fields of row n_tile+r starting
//     at element kb*128/NBITS; word t of those 16 bytes is k-step t.  The contraction index of an
//     MFMA may be permuted freely as long as both operands agree, so no shuffling is needed: the
//     activations are fetched in the matching order;
//   * fields are decoded with the in-place-mask trick (1024 + 2^o*q), brought to the exact integer
//     q - Z with one packed fp16 add or fma, and multiplied by the scale with one packed fp16
//     multiply: bit-identical to the reference's dequantised weight;
//   * activations: the block stages a BM x BK fp16 tile per K-slice in LDS (double-buffered, one
//     barrier per iteration); a lane reads its 8 consecutive k of one row with one ds_read_b128;
//   * WK > 1 splits K over waves of the same block; partial tiles are summed through LDS.
#pragma once

#include <atomic>
#include <cstdio>
#include "qf_dequant.hip.h"

namespace qf {

template <int NBITS_, int GS_, bool SYM_, int N_, int K_, int AT_, int BT_, int WM_, int WN_, int WK_, bool NT_B_>
struct MfmaCfg {
    static constexpr int NBITS = NBITS_, GS = GS_, N = N_, K = K_;
    static constexpr bool SYM = SYM_, NT_B = NT_B_;
    static constexpr int AT = AT_;                 // 16-row activation tiles per wave
    static constexpr int BT = BT_;                 // 16-row weight tiles per wave
    static constexpr int WM = WM_, WN = WN_, WK = WK_;
    static constexpr int BM = WM * AT * 16;        // activation rows per block
    static constexpr int BN = WN * BT * 16;        // weight rows (output columns) per block
    static constexpr int THREADS = 64 * WM * WN * WK;
    static constexpr int TPK = 64 * WM * WN;       // threads sharing one K-slice
    static constexpr int EPL = 128 / NBITS;        // fields per lane and 16-byte load
    static constexpr int KSTEPS = EPL / 8;         // MFMA k-steps per load
    static constexpr int BK = 4 * EPL;             // elements of K per iteration
    static constexpr int IT_TOTAL = K / BK;
    static constexpr int IPW = (IT_TOTAL + WK - 1) / WK;    // iterations per K-slice
    static constexpr int RB = K * NBITS / 8;
    static constexpr int G = K / GS;
    static constexpr int ZRB = G * NBITS / 8;
    static constexpr int PITCH = BK + 8;           // LDS row pitch in halves: BK*2 + 16 bytes
    static constexpr int UNITS = BM * BK / 8;      // 16-byte units in one activation tile
    static constexpr int UPT = (UNITS + TPK - 1) / TPK;
    static constexpr int GRID_X = (N + BN - 1) / BN;
    static constexpr size_t LDS_BYTES = (size_t)2 * WK * BM * PITCH * 2 +
                                        (WK > 1 ? (size_t)(WK - 1) * WM * WN * AT * BT * 256 * 4 : 0);
};

template <class C>
__global__ __launch_bounds__(C::THREADS) void mfma_kernel(
    const uint16_t* __restrict__ A, const uint8_t* __restrict__ W, uint16_t* __restrict__ Cout,
    const uint16_t* __restrict__ S, const uint8_t* __restrict__ Zp, int m_total) {
    constexpr int AT = C::AT, BT = C::BT, WM = C::WM, WN = C::WN, WK = C::WK;
    constexpr int EPL = C::EPL, KSTEPS = C::KSTEPS, BK = C::BK, PITCH = C::PITCH, UPT = C::UPT;
    constexpr int P8 = 8 / C::NBITS;
    constexpr uint32_t ZMASK = (1u << C::NBITS) - 1u;
    constexpr int UNITS_PER_ROW = BK / 8;

    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint16_t* As = reinterpret_cast<uint16_t*>(smem);                       // [2][WK][BM][PITCH]
    float* red = reinterpret_cast<float*>(smem + (size_t)2 * WK * C::BM * PITCH * 2);

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wn = wave % WN;
    const int wm = (wave / WN) % WM;
    const int wk = wave / (WN * WM);
    const int r = lane & 15, kb = lane >> 4;
    const int tpk = tid - wk * C::TPK;                   // thread index inside the K-slice

    const int mb = blockIdx.y * C::BM;                   // first activation row of the block
    const int n0 = blockIdx.x * C::BN + wn * BT * 16;    // first weight row of the wave
    const int it_begin = wk * C::IPW;

    // ---- per-lane constant addresses ----
    const uint8_t* wrow[BT];
    const uint16_t* srow[BT];
    const uint8_t* zrow[BT];
#pragma unroll
    for (int j = 0; j < BT; j++) {
        const int n = min(n0 + j * 16 + r, C::N - 1);
        wrow[j] = W + (size_t)n * C::RB + kb * 16;
        srow[j] = S + (size_t)n * C::G;
        zrow[j] = Zp + (size_t)n * C::ZRB;
    }

    struct WStage {
        uint32_t w[BT][4];
        scale_holder_t s[BT];
        zero_holder_t z[BT];
    };
    auto load_w = [&](WStage& st, int it) {
        const int itc = min(it, C::IT_TOTAL - 1);
        const int g = (itc * BK + kb * EPL) / C::GS;
#pragma unroll
        for (int j = 0; j < BT; j++) {
            load_words<4, C::NT_B>(wrow[j] + (size_t)itc * (BK * C::NBITS / 8), st.w[j]);
            st.s[j] = srow[j][g];
            if constexpr (!C::SYM) st.z[j] = zrow[j][g / P8];
        }
    };

    // activation tile: unit u of the slice = 16 bytes at (row u / UNITS_PER_ROW, 8 * (u % UNITS_PER_ROW))
    auto load_a = [&](u32x4 (&regs)[UPT], int it) {
        const int itc = min(it, C::IT_TOTAL - 1);
#pragma unroll
        for (int p = 0; p < UPT; p++) {
            const int u = tpk + p * C::TPK;
            const int row = u / UNITS_PER_ROW, col = (u % UNITS_PER_ROW) * 8;
            const int m = min(mb + row, m_total - 1);
            if (u < C::UNITS)
                regs[p] = *reinterpret_cast<const u32x4*>(A + (size_t)m * C::K + (size_t)itc * BK + col);
        }
    };
    auto store_a = [&](const u32x4 (&regs)[UPT], int buf) {
        uint16_t* base = As + ((size_t)(buf * WK + wk) * C::BM) * PITCH;
#pragma unroll
        for (int p = 0; p < UPT; p++) {
            const int u = tpk + p * C::TPK;
            const int row = u / UNITS_PER_ROW, col = (u % UNITS_PER_ROW) * 8;
            if (u < C::UNITS) *reinterpret_cast<u32x4*>(base + (size_t)row * PITCH + col) = act_unit(regs[p]);
        }
    };

    f32x4 acc[AT][BT];
#pragma unroll
    for (int i = 0; i < AT; i++)
#pragma unroll
        for (int j = 0; j < BT; j++) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    // ---- prologue: first weights in flight, first activation tile into LDS ----
    WStage wcur, wnext;
    u32x4 areg[UPT];
    load_w(wcur, it_begin);
    load_a(areg, it_begin);
    store_a(areg, 0);
    __syncthreads();

#pragma unroll 1
    for (int ii = 0; ii < C::IPW; ii++) {
        const int it = it_begin + ii;
        const int buf = ii & 1;
        const bool more = ii + 1 < C::IPW;
        if (more) {
            load_w(wnext, it + 1);
            load_a(areg, it + 1);
        }
        if (it < C::IT_TOTAL) {                           // wave-uniform
            QConst qc[BT];
            const int g = (it * BK + kb * EPL) / C::GS;
#pragma unroll
            for (int j = 0; j < BT; j++) {
                const uint32_t zero = C::SYM ? (1u << (C::NBITS - 1))
                                             : ((uint32_t)(wcur.z[j] >> ((g % P8) * C::NBITS)) & ZMASK);
                qc[j] = make_qconst<C::NBITS>((uint16_t)wcur.s[j], zero);
            }
            const uint16_t* abase = As + ((size_t)(buf * WK + wk) * C::BM + wm * AT * 16 + r) * PITCH + kb * EPL;
#pragma unroll
            for (int t = 0; t < KSTEPS; t++) {
                f16x8 af[AT];
#pragma unroll
                for (int i = 0; i < AT; i++)
                    af[i] = *reinterpret_cast<const f16x8*>(abase + (size_t)i * 16 * PITCH + t * 8);
#pragma unroll
                for (int j = 0; j < BT; j++) {
                    const f16x8 wf = DequantStep<C::NBITS>::run(wcur.w[j], t, qc[j]);
#pragma unroll
                    for (int i = 0; i < AT; i++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf, af[i], acc[i][j], 0, 0, 0);
                }
            }
        }
        if (more) {
            store_a(areg, buf ^ 1);
            wcur = wnext;
        }
        __syncthreads();
    }

    // ---- K-slices of one tile are summed through LDS ----
    if constexpr (WK > 1) {
        const int slot = (wm * WN + wn) * AT * BT;
        if (wk > 0) {
#pragma unroll
            for (int i = 0; i < AT; i++)
#pragma unroll
                for (int j = 0; j < BT; j++)
                    *reinterpret_cast<f32x4*>(red + ((size_t)((wk - 1) * WM * WN * AT * BT + slot + i * BT + j) * 64 + lane) * 4) = acc[i][j];
        }
        __syncthreads();
        if (wk > 0) return;
#pragma unroll
        for (int k2 = 0; k2 < WK - 1; k2++)
#pragma unroll
            for (int i = 0; i < AT; i++)
#pragma unroll
                for (int j = 0; j < BT; j++)
                    acc[i][j] += *reinterpret_cast<const f32x4*>(red + ((size_t)(k2 * WM * WN * AT * BT + slot + i * BT + j) * 64 + lane) * 4);
    }

    // ---- store: lane holds C[m][n .. n+3], m = tile row lane%16, n = 4*(lane/16) ----
#pragma unroll
    for (int i = 0; i < AT; i++) {
        const int m = mb + (wm * AT + i) * 16 + r;
        if (m >= m_total) continue;
#pragma unroll
        for (int j = 0; j < BT; j++) {
            const int n = n0 + j * 16 + kb * 4;
            uint16_t h[4];
#pragma unroll
            for (int e = 0; e < 4; e++) h[e] = f32_to_out_bits(acc[i][j][e]);
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

template <class C>
int mfma_launch(const void* A, const void* W, void* Cout, const void* S, const void* Zp, int m, hipStream_t stream) {
    const char* why = nullptr;
    if (C::NBITS != 2 && C::NBITS != 4 && C::NBITS != 8) why = "NBITS must be 2, 4 or 8 for this kernel";
    else if (C::K % C::BK != 0) why = "K must be a multiple of 4*128/NBITS";
    else if (C::GS <= 0 || C::K % C::GS != 0) why = "GS must divide K";
    else if (C::GS % C::EPL != 0) why = "a lane's 16 bytes of fields must lie inside one group";
    else if (!C::SYM && (C::G % (8 / C::NBITS)) != 0) why = "K/GS must fill whole zero-point bytes";
    else if (C::THREADS > 1024) why = "block too large";
    else if (C::LDS_BYTES > 160 * 1024) why = "tiles exceed the 160 KB of LDS";
    else if (C::WK > C::IT_TOTAL) why = "more K-slices than K-iterations";
    if (why) {
        fprintf(stderr, "qfactory mfma: invalid configuration: %s (NBITS=%d GS=%d N=%d K=%d AT=%d BT=%d WM=%d WN=%d WK=%d)\n",
                why, C::NBITS, C::GS, C::N, C::K, C::AT, C::BT, C::WM, C::WN, C::WK);
        return 1;
    }
    if (m <= 0) return 0;
    static std::atomic<bool> attr_set{false};        // launch is re-entrant: the attribute call is idempotent, the flag only saves repeats
    if (C::LDS_BYTES > 64 * 1024 && !attr_set.load(std::memory_order_acquire)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&mfma_kernel<C>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)C::LDS_BYTES);
        if (e != hipSuccess) {
            fprintf(stderr, "qfactory mfma: cannot reserve %zu bytes of LDS: %s\n", C::LDS_BYTES, hipGetErrorString(e));
            return 2;
        }
        attr_set.store(true, std::memory_order_release);
    }
    dim3 grid(C::GRID_X, (m + C::BM - 1) / C::BM);
    hipLaunchKernelGGL(mfma_kernel<C>, grid, dim3(C::THREADS), C::LDS_BYTES, stream, (const uint16_t*)A,
                       (const uint8_t*)W, (uint16_t*)Cout, (const uint16_t*)S, (const uint8_t*)Zp, m);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        fprintf(stderr, "qfactory mfma: launch failed: %s\n", hipGetErrorString(err));
        return 2;
    }
    return 0;
}

}  // namespace qf
