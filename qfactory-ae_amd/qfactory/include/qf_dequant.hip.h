// Register-level dequantisation of one MFMA k-step (8 fields of one lane) for 2/4/8-bit weights.
//
// IntStep   : packed word(s) -> eight exact fp16 integers q - Z
// DequantStep: the same, times the scale: fp16_rn((q - Z) * s), bit-identical to the reference's
//              eager decode (qfactory/include/utils.h:46-62: magic-number int->fp16, add of
//              -(1024 + Z), multiply by the scale -- one rounding).
#pragma once

#include "qf_common.hip.h"

namespace qf {

// ---- masked fields of one k-step (8 fields of one lane) -> exact fp16 integers q - Z ----
struct ZConst {
    f16x2 off[4];   // per class: -(1024 * 2^-o + Z), both halves
};

template <int NBITS>
__device__ __forceinline__ ZConst make_zconst(uint32_t zero) {
    // -(B + Z) for B = 1024 * 2^-o is representable and its bit pattern is linear in Z:
    // 0xE400 + Z, 0xDC00 + 4Z, 0xD400 + 16Z, 0xCC00 + 64Z for o = 0, 2, 4, 6
    ZConst c;
    using D = Decode<NBITS>;
#pragma unroll
    for (int k = 0; k < 4; k++) {
        const int cls = k < D::NCLS ? k : 0;
        const int o = (NBITS == 4) ? 4 * cls : ((NBITS == 2 || NBITS == 3) ? 2 * cls : 0);
        const uint32_t base = 0xE400u - 0x0400u * (uint32_t)o;          // exponent drops by one per factor 2
        const uint32_t h = base + (zero << o);
        c.off[k] = as_f16x2(h * 0x00010001u);
    }
    return c;
}

template <int NBITS> struct IntStep;

template <> struct IntStep<4> {
    __device__ __forceinline__ static f16x8 run(const uint32_t (&w)[4], int t, const ZConst& c) {
        uint32_t x[4];
        Decode<4>::word(w[t], x);
        const f16x2 sixteenth = f16x2{(_Float16)0.0625f, (_Float16)0.0625f};
        const f16x2 v0 = as_f16x2(x[0]) + c.off[0];
        const f16x2 v1 = __builtin_elementwise_fma(as_f16x2(x[1]), sixteenth, c.off[1]);
        const f16x2 v2 = as_f16x2(x[2]) + c.off[0];
        const f16x2 v3 = __builtin_elementwise_fma(as_f16x2(x[3]), sixteenth, c.off[1]);
        return f16x8{v0.x, v0.y, v1.x, v1.y, v2.x, v2.y, v3.x, v3.y};
    }
};

template <> struct IntStep<2> {
    __device__ __forceinline__ static f16x8 run(const uint32_t (&w)[4], int t, const ZConst& c) {
        const uint32_t word = (t & 1) ? (w[t >> 1] >> 8) : w[t >> 1];
        f16x2 v[4];
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const uint32_t x = (word & (0x00030003u << (2 * p))) | kMagic;
            const float inv = Decode<2>::inv_scale(p);
            v[p] = __builtin_elementwise_fma(as_f16x2(x), f16x2{(_Float16)inv, (_Float16)inv}, c.off[p]);
        }
        return f16x8{v[0].x, v[0].y, v[1].x, v[1].y, v[2].x, v[2].y, v[3].x, v[3].y};
    }
};

template <> struct IntStep<8> {
    __device__ __forceinline__ static f16x8 run(const uint32_t (&w)[4], int t, const ZConst& c) {
        uint32_t x[2], y[2];
        Decode<8>::word(w[2 * t], x);
        Decode<8>::word(w[2 * t + 1], y);
        const f16x2 v0 = as_f16x2(x[0]) + c.off[0];
        const f16x2 v1 = as_f16x2(x[1]) + c.off[0];
        const f16x2 v2 = as_f16x2(y[0]) + c.off[0];
        const f16x2 v3 = as_f16x2(y[1]) + c.off[0];
        return f16x8{v0.x, v0.y, v1.x, v1.y, v2.x, v2.y, v3.x, v3.y};
    }
};


// 3-bit: eight fields of k-step t of a lane's 32 come from 2-bit-plane word w[t / 2] (its low or
// high bytes) merged with the 1-bit-plane word `h` of the same 32 fields (see Decode<3>).
struct IntStep3 {
    template <int T>
    __device__ __forceinline__ static f16x8 run(const uint32_t (&w)[4], uint32_t h, const ZConst& c) {
        constexpr int R = T / 2;                      // which of the two 2-bit words
        constexpr bool UPPER = (T & 1) != 0;          // its high bytes
        const uint32_t wd = UPPER ? (w[R] >> 8) : w[R];
        const uint32_t he = UPPER ? (h >> (8 + R)) : (h >> R);
        const uint32_t ho = UPPER ? (h >> (4 + R)) : (h << (4 - R));
        const uint32_t mg = magic_register();
        f16x2 v[4];
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const uint32_t hs = (p % 2 == 0) ? he : ho;
            const uint32_t x = (wd & (0x00030003u << (2 * p))) | (hs & (0x00040004u << (2 * p))) | mg;
            const float inv = Decode<2>::inv_scale(p);
            v[p] = __builtin_elementwise_fma(as_f16x2(x), f16x2{(_Float16)inv, (_Float16)inv}, c.off[p]);
        }
        return f16x8{v[0].x, v[0].y, v[1].x, v[1].y, v[2].x, v[2].y, v[3].x, v[3].y};
    }
};

struct DequantStep3 {
    template <int T>
    __device__ __forceinline__ static f16x8 run(const uint32_t (&w)[4], uint32_t h, const struct QConst& c);
};

// scale splat + the offsets of make_zconst
struct QConst {
    f16x2 s2;
    ZConst z;
};

template <int NBITS>
__device__ __forceinline__ QConst make_qconst(uint16_t s_bits, uint32_t zero) {
    QConst c;
    c.s2 = as_f16x2((uint32_t)s_bits * 0x00010001u);
    c.z = make_zconst<NBITS>(zero);
    return c;
}

template <int NBITS> struct DequantStep {
    __device__ __forceinline__ static f16x8 run(const uint32_t (&w)[4], int t, const QConst& c) {
        const f16x8 s8 = f16x8{c.s2.x, c.s2.y, c.s2.x, c.s2.y, c.s2.x, c.s2.y, c.s2.x, c.s2.y};
        return IntStep<NBITS>::run(w, t, c.z) * s8;
    }
};

template <int T>
__device__ __forceinline__ f16x8 DequantStep3::run(const uint32_t (&w)[4], uint32_t h, const QConst& c) {
    const f16x8 s8 = f16x8{c.s2.x, c.s2.y, c.s2.x, c.s2.y, c.s2.x, c.s2.y, c.s2.x, c.s2.y};
    return IntStep3::run<T>(w, h, c.z) * s8;
}

}  // namespace qf
