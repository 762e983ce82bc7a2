// Shared device helpers for the gfx950 quantized-linear kernels: vector loads, the
// magic-number int->fp16 decode for 2/4/8-bit fields, and wave64 cross-lane exchange.
//
// Weight layout consumed here is the reference's packed layout (qfactory/convert.py:49-68):
// row n holds its K fields K-contiguously; inside every 32-bit word the even-indexed
// elements sit in bits 0..15 and the odd-indexed ones in bits 16..31, so that
// (word >> b*i) & (MASK | MASK << 16) is the pair (element 2i, element 2i+1)
// (qfactory/include/utils.h:11-25 decodes in the same order).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

// Scheduling fence between "issue the loads" and "consume earlier loads" regions.  0: none,
// 1: full scheduling barrier.
#ifndef QF_SCHED_FENCE_MODE
#define QF_SCHED_FENCE_MODE 0
#endif
#if QF_SCHED_FENCE_MODE == 1
#define QF_SCHED_FENCE() __builtin_amdgcn_sched_barrier(0)
#else
#define QF_SCHED_FENCE() ((void)0)
#endif

// Register holders of prefetched scale / zero-point loads.  1: 32-bit (the zero-extended load
// result stays untouched until its use), 0: 16- and 8-bit members (the compiler may pack them,
// which touches a load result right after its issue).
#ifndef QF_WIDE_HOLDERS
#define QF_WIDE_HOLDERS 1
#endif

namespace qf {

#if QF_WIDE_HOLDERS
typedef uint32_t scale_holder_t;
typedef uint32_t zero_holder_t;
#else
typedef uint16_t scale_holder_t;
typedef uint8_t zero_holder_t;
#endif

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t kMagic = 0x64006400u;  // the fp16 pair (1024, 1024): 1024 + q is exact for q < 1024

__device__ __forceinline__ f16x2 as_f16x2(uint32_t v) { return __builtin_bit_cast(f16x2, v); }
__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
__device__ __forceinline__ uint16_t f32_to_f16_bits(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }

// ---- element type of the activations and of the output ----
// The reference computes on fp16 activations only (qfactory/core/matmul.py:36, :133-136).  A
// translation unit compiled with QF_IN_BF16 reads bf16 activations, one with QF_OUT_BF16 writes a
// bf16 output (fp32 accumulator rounded to nearest even, once).  Inside, every kernel keeps
// computing on fp16 pairs against fp16 dequantised weights: a bf16 value has 8 significant bits
// and is exact in fp16 wherever fp16 is normal (2^-14 <= |a| <= 65504); larger magnitudes saturate
// to +-65504 and smaller ones are truncated to fp16's subnormal grid (the conversion rounds toward
// zero), infinities and NaN pass through.
#ifndef QF_IN_BF16
#define QF_IN_BF16 0
#endif
#ifndef QF_OUT_BF16
#define QF_OUT_BF16 0
#endif

// two activations as loaded (32 bits) -> the fp16 pair the kernels compute with
__device__ __forceinline__ uint32_t act_pair(uint32_t v) {
#if QF_IN_BF16
    const float lo = __builtin_bit_cast(float, v << 16);
    const float hi = __builtin_bit_cast(float, v & 0xFFFF0000u);
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
#else
    return v;
#endif
}
__device__ __forceinline__ u32x4 act_unit(u32x4 v) {
    return u32x4{act_pair(v.x), act_pair(v.y), act_pair(v.z), act_pair(v.w)};
}
// fp32 result -> the 16 bits stored in the output
__device__ __forceinline__ uint16_t f32_to_out_bits(float f) {
#if QF_OUT_BF16
    return __builtin_bit_cast(uint16_t, (__bf16)f);
#else
    return f32_to_f16_bits(f);
#endif
}

// 1: the kernel adds its result to what the output already holds -- out = fp16(out + fp16(result)), the two roundings
// of a projection followed by a residual add -- instead of overwriting it: the o and down projections of a decoder
// layer writing straight into the residual stream.  Every element is still touched by exactly one lane (read, then
// written).  fp16 only.  Not in the reference.
#ifndef QF_OUT_ACCUMULATE
#define QF_OUT_ACCUMULATE 0
#endif
__device__ __forceinline__ void store_out(uint16_t* p, float f) {
#if QF_OUT_ACCUMULATE
    const _Float16 add = (_Float16)f;
    const _Float16 old = __builtin_bit_cast(_Float16, *p);
    *p = __builtin_bit_cast(uint16_t, (_Float16)(old + add));
#else
    *p = f32_to_out_bits(f);
#endif
}

// SwiGLU on two fp32 sums of a fused gate+up projection: both are rounded to fp16 as the projection's output
// would be, then fp16(silu(gate)) * up with silu(x) = x * rcp(1 + exp2(-x * log2(e))) on the hardware's exp2 and
// reciprocal -- the expression of qf_silu_mul in libqfactory_hip.so, so that a kernel's fused epilogue and the
// projection followed by that call give the same bits.
__device__ __forceinline__ uint16_t silu_mul_f16(float gate_sum, float up_sum) {
    const _Float16 g = (_Float16)gate_sum, u = (_Float16)up_sum;
    const float x = (float)g;
    const float s = x * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
    return __builtin_bit_cast(uint16_t, (_Float16)((_Float16)s * u));
}

// ---- global loads of NW 32-bit words (NW in {1,2,4}); NT = streaming (non-temporal) ----
template <int NW, bool NT>
__device__ __forceinline__ void load_words(const void* p, uint32_t (&dst)[NW]) {
    static_assert(NW == 1 || NW == 2 || NW == 4, "vector width must be 4, 8 or 16 bytes");
    if constexpr (NW == 4) {
        u32x4 v = NT ? __builtin_nontemporal_load((const u32x4*)p) : *(const u32x4*)p;
        dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w;
    } else if constexpr (NW == 2) {
        u32x2 v = NT ? __builtin_nontemporal_load((const u32x2*)p) : *(const u32x2*)p;
        dst[0] = v.x; dst[1] = v.y;
    } else {
        dst[0] = NT ? __builtin_nontemporal_load((const uint32_t*)p) : *(const uint32_t*)p;
    }
}

// ---- field decode: one packed word -> PAIRS fp16 pairs holding 1024 + SCALE(class) * q ----
//
// Instead of shifting every field down to bit 0, fields are masked in place: a field at bit
// offset o inside its half-word decodes to 1024 + 2^o * q, still exact in fp16.  Pairs with the
// same o form a "class"; a dot product keeps one fp32 accumulator per class and folds the 2^-o
// factors and the 1024 offsets in once per chunk (see gemv kernel).  Only the upper byte of each
// half-word needs one shift per word.
template <int NBITS> struct Decode;

// (w & mask) | magic in ONE instruction.  gfx9 VOP3 encodings take no literal operands and read at
// most one SGPR, so the compiler, which sees two literals, emits v_and + v_or; with the mask in an
// SGPR and the magic pair in a VGPR the fused v_and_or_b32 is encodable.  Measured on MI355X at
// M = 1: 14 % fewer vector instructions, but the asm statements cost the GEMV kernel 30 more
// registers and one resident wave per SIMD; only K = 11008 gains (7.2 -> 6.7 us), the K = 4096
// shapes lose 0.3 - 1.6 us.  Off by default (plain C: v_and + v_or).
#ifndef QF_FUSED_AND_OR
#define QF_FUSED_AND_OR 0
#endif
template <uint32_t MASK>
__device__ __forceinline__ uint32_t and_or(uint32_t w, uint32_t magic_vgpr) {
#if QF_FUSED_AND_OR == 2
    // no instruction is spelled out: the mask is made opaque in a scalar register (the magic pair in a vector
    // register, magic_register()), so the compiler cannot fold either into a literal and selects v_and_or_b32
    // itself, and stays free to schedule it
    uint32_t m = MASK;
    asm("" : "+s"(m));
    return (w & m) | magic_vgpr;
#elif QF_FUSED_AND_OR
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(w), "s"(MASK), "v"(magic_vgpr));
    return r;
#else
    return (w & MASK) | magic_vgpr;
#endif
}
// The magic pair in a VGPR the compiler cannot fold back into a literal.
__device__ __forceinline__ uint32_t magic_register() {
    uint32_t m = kMagic;
#if QF_FUSED_AND_OR
    asm("" : "+v"(m));          // not volatile: identical copies merge, one register per kernel
#endif
    return m;
}

template <> struct Decode<4> {
    static constexpr int PAIRS = 4;   // pairs per 32-bit word
    static constexpr int NCLS = 2;    // field offsets 0 and 4
    __host__ __device__ static constexpr int cls(int pair) { return pair & 1; }
    __host__ __device__ static constexpr float inv_scale(int c) { return c == 0 ? 1.0f : 0.0625f; }
    __host__ __device__ static constexpr int shift(int c) { return 4 * c; }     // bit offset o of a class: inv_scale = 2^-o
    __device__ __forceinline__ static void word(uint32_t w, uint32_t (&x)[PAIRS]) {
        const uint32_t w8 = w >> 8;
        const uint32_t mg = magic_register();
        x[0] = and_or<0x000F000Fu>(w, mg);
        x[1] = and_or<0x00F000F0u>(w, mg);
        x[2] = and_or<0x000F000Fu>(w8, mg);
        x[3] = and_or<0x00F000F0u>(w8, mg);
    }
};

template <> struct Decode<2> {
    static constexpr int PAIRS = 8;
    static constexpr int NCLS = 4;    // field offsets 0, 2, 4, 6
    __host__ __device__ static constexpr int cls(int pair) { return pair & 3; }
    __host__ __device__ static constexpr float inv_scale(int c) {
        return c == 0 ? 1.0f : c == 1 ? 0.25f : c == 2 ? 0.0625f : 0.015625f;
    }
    __host__ __device__ static constexpr int shift(int c) { return 2 * c; }
    __device__ __forceinline__ static void word(uint32_t w, uint32_t (&x)[PAIRS]) {
        const uint32_t w8 = w >> 8;
        const uint32_t mg = magic_register();
        x[0] = and_or<0x00030003u>(w, mg);
        x[1] = and_or<0x000C000Cu>(w, mg);
        x[2] = and_or<0x00300030u>(w, mg);
        x[3] = and_or<0x00C000C0u>(w, mg);
        x[4] = and_or<0x00030003u>(w8, mg);
        x[5] = and_or<0x000C000Cu>(w8, mg);
        x[6] = and_or<0x00300030u>(w8, mg);
        x[7] = and_or<0x00C000C0u>(w8, mg);
    }
};

// 3-bit rows are a 2-bit plane followed by a 1-bit plane (this project's layout; the reference has
// no 3-bit).  Word `w` of the 2-bit plane holds 16 elements; word `h` of the 1-bit plane holds the
// high bits of 32 elements, i.e. of 2-bit words 2J (r = 0) and 2J + 1 (r = 1).  The plane's bit
// order is such that four shifts of `h` line every high bit up directly above its 2-bit field;
// one AND-OR per pair then yields 1024 + 2^o * (lo + 4 * hi), decoded exactly like a 2-bit pair.
template <> struct Decode<3> {
    static constexpr int PAIRS = 8;
    static constexpr int NCLS = 4;
    __host__ __device__ static constexpr int cls(int pair) { return pair & 3; }
    __host__ __device__ static constexpr float inv_scale(int c) { return Decode<2>::inv_scale(c); }
    __host__ __device__ static constexpr int shift(int c) { return 2 * c; }
    template <int R>
    __device__ __forceinline__ static void word(uint32_t w, uint32_t h, uint32_t (&x)[PAIRS]) {
        const uint32_t w8 = w >> 8;
        const uint32_t he0 = h >> R, he1 = h >> (8 + R);           // pairs 0, 2 of the low / high byte
        const uint32_t ho0 = h << (4 - R), ho1 = h >> (4 + R);     // pairs 1, 3 of the low / high byte
        const uint32_t mg = magic_register();
        x[0] = and_or<0x00040004u>(he0, and_or<0x00030003u>(w, mg));
        x[1] = and_or<0x00100010u>(ho0, and_or<0x000C000Cu>(w, mg));
        x[2] = and_or<0x00400040u>(he0, and_or<0x00300030u>(w, mg));
        x[3] = and_or<0x01000100u>(ho0, and_or<0x00C000C0u>(w, mg));
        x[4] = and_or<0x00040004u>(he1, and_or<0x00030003u>(w8, mg));
        x[5] = and_or<0x00100010u>(ho1, and_or<0x000C000Cu>(w8, mg));
        x[6] = and_or<0x00400040u>(he1, and_or<0x00300030u>(w8, mg));
        x[7] = and_or<0x01000100u>(ho1, and_or<0x00C000C0u>(w8, mg));
    }
};

// Bits per field of the main weight plane and of a stored zero-point (3-bit: 2-bit main plane plus
// a 1-bit plane; zero-points one per nibble).
__host__ __device__ constexpr int plane_bits(int nbits) { return nbits == 3 ? 2 : nbits; }
__host__ __device__ constexpr int zero_field_bits(int nbits) { return nbits == 3 ? 4 : nbits; }

template <> struct Decode<8> {
    static constexpr int PAIRS = 2;
    static constexpr int NCLS = 1;
    __host__ __device__ static constexpr int cls(int) { return 0; }
    __host__ __device__ static constexpr float inv_scale(int) { return 1.0f; }
    __host__ __device__ static constexpr int shift(int) { return 0; }
    __device__ __forceinline__ static void word(uint32_t w, uint32_t (&x)[PAIRS]) {
        // 8-bit fields are stored in natural byte order (PERMUTE_ORDER[8] is the identity):
        // byte-permute (b0, 0x64, b1, 0x64) and (b2, 0x64, b3, 0x64) in one instruction each.
        x[0] = __builtin_amdgcn_perm(0x64646464u, w, 0x04010400u);
        x[1] = __builtin_amdgcn_perm(0x64646464u, w, 0x04030402u);
    }
};

// Operands of the residual-add + RMSNorm prologue of the kernels for few rows (ignored by kernels compiled
// without it):  h = fp16(x + delta),  a = fp16(fp16(h * rsqrt(mean(h^2) + eps)) * gamma).
struct NormArgs {
    const uint16_t* delta = nullptr;   // (M, K) fp16 added to the activation rows first, or null
    const uint16_t* gamma = nullptr;   // (K) fp16 RMSNorm weight
    uint16_t* x_out = nullptr;         // (M, K) fp16: receives x + delta, or null
    float eps = 0.0f;
};

// ---- wave64 lane exchange: value held by lane (l ^ D) ----
template <int D>
__device__ __forceinline__ float lane_xor(float v) {
    const int iv = __builtin_bit_cast(int, v);
    int r;
    if constexpr (D == 1) {
        r = __builtin_amdgcn_update_dpp(0, iv, 0xB1, 0xF, 0xF, true);      // quad_perm [1,0,3,2]
    } else if constexpr (D == 2) {
        r = __builtin_amdgcn_update_dpp(0, iv, 0x4E, 0xF, 0xF, true);      // quad_perm [2,3,0,1]
    } else if constexpr (D == 4) {
        r = __builtin_amdgcn_ds_swizzle(iv, 0x101F);                       // bit mode, xor 4
    } else if constexpr (D == 8) {
        r = __builtin_amdgcn_update_dpp(0, iv, 0x128, 0xF, 0xF, true);     // row_ror:8 == xor 8 in a row of 16
    } else if constexpr (D == 16) {
        r = __builtin_amdgcn_ds_swizzle(iv, 0x401F);                       // bit mode, xor 16
    } else {
        static_assert(D == 32, "lane distance must be a power of two below 64");
        r = __builtin_amdgcn_ds_bpermute(((int)__lane_id() ^ 32) << 2, iv);
    }
    return __builtin_bit_cast(float, r);
}

// One "halving" butterfly step at lane distance D over the first VC entries of v: lanes with bit D
// clear keep the first half, lanes with bit D set keep the second half, each adding what its
// partner sent.  Afterwards the first VC/2 entries are live.
template <int D, int VC, int V>
__device__ __forceinline__ void halve_step(float (&v)[V], int lane) {
    constexpr int H = VC / 2;
    const bool up = (lane & D) != 0;
#pragma unroll
    for (int i = 0; i < H; i++) {
        const float keep = up ? v[i + H] : v[i];
        const float send = up ? v[i] : v[i + H];
        v[i] = keep + lane_xor<D>(send);
    }
}

// Order in which lane-distance bits are consumed by wave_reduce_many: DPP-only distances first
// (they carry the most values), the LDS-crossbar ones last.
__host__ __device__ constexpr int kLaneOrder(int t) {
    return t == 0 ? 1 : t == 1 ? 2 : t == 2 ? 8 : t == 3 ? 4 : t == 4 ? 16 : 32;
}

template <int VC, int T, int V>
__device__ __forceinline__ void reduce_from(float (&v)[V], int lane) {
    if constexpr (T < 6) {
        constexpr int D = kLaneOrder(T);
        if constexpr (VC > 1) {
            halve_step<D, VC, V>(v, lane);
            reduce_from<VC / 2, T + 1, V>(v, lane);
        } else {
            v[0] += lane_xor<D>(v[0]);
            reduce_from<1, T + 1, V>(v, lane);
        }
    }
}

// Sum V (power of two, <= 64) per-lane values across the 64 lanes of a wave.  On return v[0] of
// lane l holds the wave-wide total of the input value with index reduce_index<V>(l); lanes for
// which reduce_owner<V>(l) is true hold the V distinct totals.
template <int V>
__device__ __forceinline__ void wave_reduce_many(float (&v)[V], int lane) {
    static_assert(V >= 1 && V <= 64 && (V & (V - 1)) == 0, "V must be a power of two <= 64");
    reduce_from<V, 0, V>(v, lane);
}

template <int V>
__device__ __forceinline__ int reduce_index(int lane) {
    int idx = 0, span = V;
#pragma unroll
    for (int t = 0; t < 6; t++) {
        if (span > 1) {
            span >>= 1;
            if (lane & kLaneOrder(t)) idx += span;
        }
    }
    return idx;
}

template <int V>
__device__ __forceinline__ bool reduce_owner(int lane) {
    int used = 0, span = V;
#pragma unroll
    for (int t = 0; t < 6; t++) {
        if (span > 1) { span >>= 1; used |= kLaneOrder(t); }
    }
    return (lane & ~used & 63) == 0;
}

}  // namespace qf
