// libqfactory_hip.so, second translation unit: the steps of one decode token (one new position per
// sequence) that sit between the quantized linears of a Llama-style layer -- residual add + RMSNorm,
// rotary embedding + KV-cache append, attention of the new position over the cache, SiLU(gate) * up.
// Each is one launch; entry points and contracts are declared in include/qfactory_hip.h.
//
// All four are HBM/latency-bound fp16 kernels with fp32 arithmetic inside: 16-byte accesses, one block
// per row / per (sequence, head), reductions through wave shuffles and LDS.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <stdint.h>

#include "qfactory_hip.h"

namespace {

typedef _Float16 f16;
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

int fail(const char* fn, const char* why) {
    fprintf(stderr, "%s: %s\n", fn, why);
    return 1;
}

int launched(const char* fn) {
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        fprintf(stderr, "%s: launch failed: %s\n", fn, hipGetErrorString(err));
        return 2;
    }
    return 0;
}

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / 64;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Sum over the LPK (4, 8, 16 or 32) neighbouring lanes that share a key row, in every one of them: lane-exchange steps
// inside a row of sixteen lanes are data-parallel moves (no trip through the LDS crossbar), only the step across
// two rows of sixteen is a shuffle.
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

template <int LPK>
__device__ __forceinline__ float group_sum(float v) {
    static_assert(LPK == 4 || LPK == 8 || LPK == 16 || LPK == 32, "lanes per key row");
    v += dpp_move<0xB1>(v);                                    // quad_perm [1,0,3,2]: lane ^ 1
    v += dpp_move<0x4E>(v);                                    // quad_perm [2,3,0,1]: lane ^ 2
    if constexpr (LPK >= 8) v += dpp_move<0x141>(v);           // row_half_mirror: the other quad of the eight
    if constexpr (LPK >= 16) v += dpp_move<0x140>(v);          // row_mirror: the other eight of the sixteen
    if constexpr (LPK >= 32) v += __shfl_xor(v, 16, 64);
    return v;
}

// Sum (MAX = false) or maximum (MAX = true) over a block of WAVES waves; `slots` holds WAVES floats and
// may be reused right after the call returns.
template <bool MAX, int WAVES>
__device__ __forceinline__ float block_reduce(float v, float* slots) {
    v = MAX ? wave_max(v) : wave_sum(v);
    if ((threadIdx.x & 63) == 0) slots[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = slots[0];
#pragma unroll
    for (int w = 1; w < WAVES; w++) r = MAX ? fmaxf(r, slots[w]) : r + slots[w];
    __syncthreads();
    return r;
}

// ---------------------------------------------------------------------------------------------
// x += delta (optional);  out = fp16( fp16(x * rsqrt(mean(x^2) + eps)) * weight ).  One block per row;
// a thread keeps its (at most kNormVec) 8-element vectors in registers between the two passes.
// ---------------------------------------------------------------------------------------------
constexpr int kNormVec = 8;

__global__ __launch_bounds__(kThreads) void add_rmsnorm_kernel(f16* __restrict__ x, const f16* __restrict__ delta,
                                                               const f16* __restrict__ weight, f16* __restrict__ out,
                                                               int hidden, float eps) {
    __shared__ float slots[kWaves];
    const size_t row = (size_t)blockIdx.x * hidden;
    f16x8 v[kNormVec], w[kNormVec];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kNormVec; i++) {
        const int c = (threadIdx.x + i * kThreads) * 8;
        if (c < hidden) {
            w[i] = *reinterpret_cast<const f16x8*>(weight + c);       // requested with x: not a second round trip after the reduction
            v[i] = *reinterpret_cast<const f16x8*>(x + row + c);
            if (delta) {
                v[i] = v[i] + *reinterpret_cast<const f16x8*>(delta + row + c);      // fp16 add, as the residual stream is fp16
                *reinterpret_cast<f16x8*>(x + row + c) = v[i];
            }
#pragma unroll
            for (int e = 0; e < 8; e++) ss += (float)v[i][e] * (float)v[i][e];
        }
    }
    const float r = rsqrtf(block_reduce<false, kWaves>(ss, slots) / (float)hidden + eps);
#pragma unroll
    for (int i = 0; i < kNormVec; i++) {
        const int c = (threadIdx.x + i * kThreads) * 8;
        if (c < hidden) {
            f16x8 o;
#pragma unroll
            for (int e = 0; e < 8; e++) o[e] = (f16)((float)v[i][e] * r) * w[i][e];
            *reinterpret_cast<f16x8*>(out + row + c) = o;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Rotary embedding of q and k of the new position (pairs (2i, 2i+1), angle table row pos) and append
// of k, v to the cache.  qkv row b is [3][H][hd]; caches are (B, H, max_len, hd).  One thread per pair.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void rope_kv_store_kernel(const f16* __restrict__ qkv, const int64_t* __restrict__ pos_ptr,
                                                                 const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                                 f16* __restrict__ q_out, f16* __restrict__ k_cache,
                                                                 f16* __restrict__ v_cache, int batch, int heads, int hd, int max_len) {
#pragma clang fp contract(off)                                // two products and a sum, each rounded, like the ops this replaces
    const int64_t pos = pos_ptr[0];
    if (pos < 0 || pos >= max_len) return;                    // nothing is written for a position outside the cache
    const int half = hd / 2;
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= (int64_t)batch * heads * half) return;
    const int i = (int)(idx % half);
    const int h = (int)((idx / half) % heads);
    const int b = (int)(idx / ((int64_t)half * heads));
    const float c = cos_t[pos * half + i], s = sin_t[pos * half + i];
    const f16* row = qkv + (size_t)b * 3 * heads * hd;
    const size_t in_off = (size_t)h * hd + 2 * i;
    const size_t cache_off = (((size_t)b * heads + h) * max_len + (size_t)pos) * hd + 2 * i;
    const float q0 = (float)row[in_off], q1 = (float)row[in_off + 1];
    const float k0 = (float)row[(size_t)heads * hd + in_off], k1 = (float)row[(size_t)heads * hd + in_off + 1];
    f16* qo = q_out + ((size_t)b * heads + h) * hd + 2 * i;
    qo[0] = (f16)(q0 * c - q1 * s);
    qo[1] = (f16)(q0 * s + q1 * c);
    k_cache[cache_off] = (f16)(k0 * c - k1 * s);
    k_cache[cache_off + 1] = (f16)(k0 * s + k1 * c);
    v_cache[cache_off] = row[(size_t)2 * heads * hd + in_off];
    v_cache[cache_off + 1] = row[(size_t)2 * heads * hd + in_off + 1];
}

// ---------------------------------------------------------------------------------------------
// Attention of one query per (sequence, head) over cache positions 0 .. pos, one block of 16 or 4 waves per
// (head, sequence).  LPK = hd/8 lanes share a key or value row (16 bytes each), so a block covers
// 1024/LPK or 256/LPK positions per pass.  One pass over the cache: every group of LPK lanes walks its share of
// the positions with a running maximum (key and value row requested together), the groups of a wave are merged
// by lane shuffles, the waves through LDS.
//
// FUSED: q, k, v of the new position come straight from the QKV projection (row b = [3][H][hd]); q and k are
// rotated here (pairs (2i, 2i+1), angles of table row pos, rounded to fp16 as a separate rotation kernel would
// store them), k and v are appended to the cache, and the new position is served from LDS rather than
// re-read from memory the block has just written.
// ---------------------------------------------------------------------------------------------
// 8 waves per block and the first 8 positions of every group requested up front, at every batch size.  Measured with 32
// heads of 128 at 130 / 191 / 250 cache positions, cold caches: 5.4 / 5.6 / 6.0 us at batch 1, 10.4 / 12.4 / 14.9 at
// batch 16, 28.9 / 37.1 / 47.3 at batch 64 (there the kernel reads 200 MB of cache per launch and is HBM-bound).
// Against it: 16 waves walking the cache two positions at a time 5.6 / 6.2 / 6.8 and 11.5 / 14.2 / 16.7 at batch 1 and 16;
// 4 waves per block and one pass with a running maximum (the variant that served 1024 pairs and more) 8.7 / 10.8 /
// 13.7 at batch 4, 11.8 / 14.9 / 18.0 at batch 16, 30.8 / 41.9 / 52.8 at batch 64, and 5 - 7 % behind at 500 and 900
// positions too.  Every wave repeats the rotation of q and the merge steps, so more waves cost vector issue; a launch
// costs 4.0 us before it touches the cache (the position, then the new token's q / k / v, then the stores: three
// dependent round trips behind a 1.7 us launch).
constexpr int kAttnThreads = 512;
constexpr int kAttnPrefetch = 8;          // positions per group requested up front (256 at 128-wide heads)

__device__ __forceinline__ f16x8 rotate8(const f16x8 x, const float* __restrict__ c, const float* __restrict__ s) {
#pragma clang fp contract(off)                                // same roundings as rope_kv_store_kernel
    f16x8 r;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float x0 = (float)x[2 * i], x1 = (float)x[2 * i + 1];
        r[2 * i] = (f16)(x0 * c[i] - x1 * s[i]);
        r[2 * i + 1] = (f16)(x0 * s[i] + x1 * c[i]);
    }
    return r;
}

// ---------------------------------------------------------------------------------------------
// The same rotation and cache write for `tokens` positions per sequence (prefill): qkv row b * tokens + t is
// [3][H][hd] of token t of sequence b, pos[t] its position (shared by the sequences).  q goes out in the same row
// order, (batch, tokens, heads, hd) -- an attention that takes (batch, heads, tokens, hd) gets the transposed view and
// returns its output in row order too --, k and v to cache row pos[t].  One thread per eight elements; a token whose position is outside the cache writes nothing.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void rope_kv_store_rows_kernel(const f16* __restrict__ qkv, const int64_t* __restrict__ pos_ptr,
                                                                      const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                                      f16* __restrict__ q_out, f16* __restrict__ k_cache,
                                                                      f16* __restrict__ v_cache, int batch, int tokens, int heads, int hd,
                                                                      int max_len) {
    const int per_head = hd / 8;
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= (int64_t)batch * tokens * heads * per_head) return;
    const int j = (int)(idx % per_head);
    const int h = (int)((idx / per_head) % heads);
    const int64_t bt = idx / ((int64_t)per_head * heads);
    const int t = (int)(bt % tokens), b = (int)(bt / tokens);
    const int64_t pos = pos_ptr[t];
    if (pos < 0 || pos >= max_len) return;
    float c[4], s[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        c[i] = cos_t[pos * (hd / 2) + j * 4 + i];
        s[i] = sin_t[pos * (hd / 2) + j * 4 + i];
    }
    const f16* row = qkv + (size_t)bt * 3 * heads * hd + (size_t)h * hd + j * 8;
    const f16x8 q = rotate8(*reinterpret_cast<const f16x8*>(row), c, s);
    const f16x8 k = rotate8(*reinterpret_cast<const f16x8*>(row + (size_t)heads * hd), c, s);
    const f16x8 v = *reinterpret_cast<const f16x8*>(row + (size_t)2 * heads * hd);
    *reinterpret_cast<f16x8*>(q_out + ((size_t)bt * heads + h) * hd + j * 8) = q;
    const size_t cache_off = (((size_t)b * heads + h) * max_len + (size_t)pos) * hd + j * 8;
    *reinterpret_cast<f16x8*>(k_cache + cache_off) = k;
    *reinterpret_cast<f16x8*>(v_cache + cache_off) = v;
}

// PRE: how many of a group's first positions are requested before anything else -- before the position itself is
// known (rows are clamped to the cache; what lies past the sequence is fetched and never used) and before q has
// been rotated -- so that the cache rows, the position and the new token's q / k / v travel together instead of one
// after the other.  For the few-blocks variant only: with many blocks the rows past a short sequence would cost
// real bandwidth.
template <int LPK, bool FUSED, int THREADS, int PRE>
__global__ __launch_bounds__(THREADS) void decode_attention_kernel(const f16* __restrict__ q_or_qkv, f16* __restrict__ k_cache,
                                                                        f16* __restrict__ v_cache, const int64_t* __restrict__ pos_ptr,
                                                                        const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                                        f16* __restrict__ out, int heads, int max_len, float scale) {
    constexpr int HD = LPK * 8;
    constexpr int GROUPS = THREADS / LPK;
    constexpr int WAVES = THREADS / 64;
    __shared__ float part[WAVES * HD], part_m[WAVES], part_l[WAVES];
    __shared__ __attribute__((aligned(16))) f16 new_k[HD], new_v[HD];
    const int h = blockIdx.x, b = blockIdx.y;
    const int g = threadIdx.x / LPK, j = threadIdx.x % LPK;
    const size_t head = ((size_t)b * heads + h);
    f16* kc = k_cache + head * max_len * HD;
    f16* vc = v_cache + head * max_len * HD;
    const int64_t pos = pos_ptr[0];
    if (pos < 0 || (FUSED && pos >= max_len)) return;          // uniform over the block; nothing is written
    const int n = (int)(pos < max_len ? pos + 1 : max_len);    // keys 0 .. n-1

    // Everything the block needs from memory is requested here, in one go, before anything is computed: the new
    // token's q / k / v and angles first (they come from L2 and are needed first), then the group's first PRE
    // cache positions (rows past the sequence are clamped to its last row: one row per wave, never used).
    f16x8 qraw, kraw, vraw;
    float c[4], s[4];
    if constexpr (FUSED) {
        const f16* row = q_or_qkv + (size_t)b * 3 * heads * HD + (size_t)h * HD + j * 8;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            c[i] = cos_t[pos * (HD / 2) + j * 4 + i];
            s[i] = sin_t[pos * (HD / 2) + j * 4 + i];
        }
        qraw = *reinterpret_cast<const f16x8*>(row);
        if (g == 0) {
            kraw = *reinterpret_cast<const f16x8*>(row + (size_t)heads * HD);
            vraw = *reinterpret_cast<const f16x8*>(row + (size_t)2 * heads * HD);
        }
    } else {
        qraw = *reinterpret_cast<const f16x8*>(q_or_qkv + head * HD + j * 8);
    }
    f16x8 kpre[PRE > 0 ? PRE : 1], vpre[PRE > 0 ? PRE : 1];
#pragma unroll
    for (int i = 0; i < PRE; i++) {
        // a position past the sequence, and the new position itself (which the block is about to write and serves
        // from LDS), fetch row 0 instead: a row that is being read anyway, and never the line that is being written
        const int p = (g + i * GROUPS < (FUSED ? n - 1 : n)) ? g + i * GROUPS : 0;
        kpre[i] = *reinterpret_cast<const f16x8*>(kc + (size_t)p * HD + j * 8);
        vpre[i] = *reinterpret_cast<const f16x8*>(vc + (size_t)p * HD + j * 8);
    }
    f16x8 qv = qraw;
    if constexpr (FUSED) {
        qv = rotate8(qraw, c, s);
        if (g == 0) {
            const f16x8 kr = rotate8(kraw, c, s);
            *reinterpret_cast<f16x8*>(kc + (size_t)pos * HD + j * 8) = kr;
            *reinterpret_cast<f16x8*>(vc + (size_t)pos * HD + j * 8) = vraw;
            *reinterpret_cast<f16x8*>(new_k + j * 8) = kr;
            *reinterpret_cast<f16x8*>(new_v + j * 8) = vraw;
        }
        __syncthreads();
    }
    float qf[8];
#pragma unroll
    for (int e = 0; e < 8; e++) qf[e] = (float)qv[e] * scale;

    // one pass over the cache with a running maximum: key and value row of a position are requested together
    float m = -INFINITY, l = 0.f;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    auto visit = [&](const f16x8 kv, const f16x8 vv) {
        float d = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) d += qf[e] * (float)kv[e];
        d = group_sum<LPK>(d);                                                  // stays inside the group: all its lanes are here
        const float m_new = fmaxf(m, d);
        const float keep = __expf(m - m_new), w = __expf(d - m_new);           // m = -inf the first time: keep = 0
        l = l * keep + w;
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] = acc[e] * keep + w * (float)vv[e];
        m = m_new;
    };
    if constexpr (PRE > 0) {
        // the positions requested at the top, all at once: their scores are independent of each other, so the dot
        // products and the lane exchanges of the PRE positions overlap, and one maximum serves them all (no
        // rescaling chain from position to position)
        float d[PRE];
        f16x8 vsel[PRE];
#pragma unroll
        for (int i = 0; i < PRE; i++) {
            const bool fresh = FUSED && g + i * GROUPS == (int)pos;             // the block has just written this row: serve it from LDS
            const f16x8 kv = fresh ? *reinterpret_cast<const f16x8*>(new_k + j * 8) : kpre[i];
            vsel[i] = fresh ? *reinterpret_cast<const f16x8*>(new_v + j * 8) : vpre[i];
            d[i] = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) d[i] += qf[e] * (float)kv[e];
        }
#pragma unroll
        for (int i = 0; i < PRE; i++) d[i] = group_sum<LPK>(d[i]);
#pragma unroll
        for (int i = 0; i < PRE; i++) {
            if (g + i * GROUPS >= n) d[i] = -INFINITY;                          // past the sequence (row 0 was fetched instead)
            m = fmaxf(m, d[i]);
        }
        if (m != -INFINITY) {
#pragma unroll
            for (int i = 0; i < PRE; i++) {
                const float w = __expf(d[i] - m);                               // 0 for a position past the sequence
                l += w;
#pragma unroll
                for (int e = 0; e < 8; e++) acc[e] += w * (float)vsel[i][e];
            }
        }
    }
#pragma unroll 2
    for (int p = g + PRE * GROUPS; p < n; p += GROUPS) {
        const bool fresh = FUSED && p == (int)pos;
        visit(fresh ? *reinterpret_cast<const f16x8*>(new_k + j * 8) : *reinterpret_cast<const f16x8*>(kc + (size_t)p * HD + j * 8),
              fresh ? *reinterpret_cast<const f16x8*>(new_v + j * 8) : *reinterpret_cast<const f16x8*>(vc + (size_t)p * HD + j * 8));
    }
    // merge the 64/LPK groups of a wave (lanes that differ in the bits above log2(LPK)) ...
#pragma unroll
    for (int o = LPK; o < 64; o <<= 1) {
        const float m_o = __shfl_xor(m, o, 64), l_o = __shfl_xor(l, o, 64);
        const float top = fmaxf(m, m_o);
        const float a = (m == -INFINITY) ? 0.f : __expf(m - top), b = (m_o == -INFINITY) ? 0.f : __expf(m_o - top);
        l = l * a + l_o * b;
#pragma unroll
        for (int e = 0; e < 8; e++) acc[e] = acc[e] * a + __shfl_xor(acc[e], o, 64) * b;
        m = top;
    }
    // ... and the waves through LDS
    if ((threadIdx.x & 63) < LPK) {
#pragma unroll
        for (int e = 0; e < 8; e++) part[(threadIdx.x >> 6) * HD + j * 8 + e] = acc[e];
        if (j == 0) {
            part_m[threadIdx.x >> 6] = m;
            part_l[threadIdx.x >> 6] = l;
        }
    }
    __syncthreads();
    for (int d = threadIdx.x; d < HD; d += THREADS) {
        float top = -INFINITY;
#pragma unroll
        for (int w = 0; w < WAVES; w++) top = fmaxf(top, part_m[w]);
        float num = 0.f, den = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; w++) {
            const float f = (part_m[w] == -INFINITY) ? 0.f : __expf(part_m[w] - top);
            num += part[w * HD + d] * f;
            den += part_l[w] * f;
        }
        out[head * HD + d] = (f16)(num / den);
    }
}

// ---------------------------------------------------------------------------------------------
// out[m][i] = fp16(silu(gate[m][i])) * up[m][i], gate = gate_up[:, :mlp], up = gate_up[:, mlp:].
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void silu_mul_kernel(const f16* __restrict__ gate_up, f16* __restrict__ out,
                                                            int64_t rows, int mlp) {
    const int per_row = mlp / 8;
    const int64_t idx = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (idx >= rows * per_row) return;
    const int64_t m = idx / per_row;
    const int c = (int)(idx % per_row) * 8;
    const f16x8 gv = *reinterpret_cast<const f16x8*>(gate_up + m * 2 * mlp + c);
    const f16x8 uv = *reinterpret_cast<const f16x8*>(gate_up + m * 2 * mlp + mlp + c);
    f16x8 o;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        // the hardware's exp2 and reciprocal (one ulp each in fp32): the same expression as the GEMV kernel's
        // fused form of this step (qf_gemv.hip.h, QF_GEMV_SILU_MUL), so that the two give the same bits
        const float x = (float)gv[e];
        const float s = x * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(x * -1.4426950408889634f));
        o[e] = (f16)s * uv[e];
    }
    *reinterpret_cast<f16x8*>(out + m * mlp + c) = o;
}

// ---------------------------------------------------------------------------------------------
// Greedy choice of the next token and what the next decode step starts from, one block per sequence:
// tok[b] = the smallest index of the largest logit of row b (NaN is never chosen), x_next[b] = embed[tok[b]] (if
// embed is given), and *pos += 1 (block 0, if pos is given).
// ---------------------------------------------------------------------------------------------
constexpr int kPickThreads = 1024;

__global__ __launch_bounds__(kPickThreads) void greedy_next_kernel(const f16* __restrict__ logits, int64_t* __restrict__ tok,
                                                                  int64_t* __restrict__ pos, const f16* __restrict__ embed,
                                                                  f16* __restrict__ x_next, int vocab, int hidden) {
    __shared__ float best_v[kPickThreads / 64];
    __shared__ int best_i[kPickThreads / 64];
    __shared__ int chosen;
    const int b = blockIdx.x, tid = threadIdx.x;
    const f16* row = logits + (int64_t)b * vocab;
    float v = -__builtin_inff();
    int at = 0x7fffffff;
    for (int c = tid * 8; c < vocab; c += kPickThreads * 8) {            // ascending indices per thread: '>' keeps the first
        const f16x8 l = *reinterpret_cast<const f16x8*>(row + c);
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float f = (float)l[e];
            if (f > v || (f == v && c + e < at)) { v = f; at = c + e; }
        }
    }
    auto better = [](float fv, int fi, float gv, int gi) { return fv > gv || (fv == gv && fi < gi); };
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) {
        const float ov = __shfl_xor(v, d);
        const int oi = __shfl_xor(at, d);
        if (better(ov, oi, v, at)) { v = ov; at = oi; }
    }
    if ((tid & 63) == 0) { best_v[tid >> 6] = v; best_i[tid >> 6] = at; }
    __syncthreads();
    if (tid == 0) {
        float fv = best_v[0];
        int fi = best_i[0];
        for (int w = 1; w < kPickThreads / 64; w++)
            if (better(best_v[w], best_i[w], fv, fi)) { fv = best_v[w]; fi = best_i[w]; }
        if (fi >= vocab) fi = 0;                                           // a row without a finite or infinite maximum (all NaN)
        chosen = fi;
        tok[b] = fi;
        if (b == 0 && pos != nullptr) *pos += 1;
    }
    __syncthreads();
    if (embed != nullptr) {
        const f16* src = embed + (int64_t)chosen * hidden;
        for (int c = tid * 8; c < hidden; c += kPickThreads * 8)
            *reinterpret_cast<f16x8*>(x_next + (int64_t)b * hidden + c) = *reinterpret_cast<const f16x8*>(src + c);
    }
}

template <int LPK, bool FUSED>
int launch_attention(const char* fn, const f16* q_or_qkv, f16* k, f16* v, const int64_t* pos, const float* cos_t, const float* sin_t,
                     f16* out, int batch, int heads, int max_len, hipStream_t stream) {
    constexpr int HD = LPK * 8;
    const float scale = 1.0f / sqrtf((float)HD);
    hipLaunchKernelGGL((decode_attention_kernel<LPK, FUSED, kAttnThreads, kAttnPrefetch>), dim3(heads, batch), dim3(kAttnThreads), 0,
                       stream, q_or_qkv, k, v, pos, cos_t, sin_t, out, heads, max_len, scale);
    return launched(fn);
}

template <bool FUSED>
int dispatch_attention(const char* fn, const uint16_t* q_or_qkv, uint16_t* k_cache, uint16_t* v_cache, const int64_t* pos,
                       const float* cos_t, const float* sin_t, uint16_t* out, int64_t batch, int64_t heads, int64_t head_dim,
                       int64_t max_len, void* stream) {
    if (batch <= 0 || heads <= 0 || max_len <= 0 || batch > 65535 || heads > 0x7fffffff || max_len > 0x7fffffff)
        return fail(fn, "batch in 1..65535, heads and max_len positive");
    const f16* qp = (const f16*)q_or_qkv;
    f16 *kp = (f16*)k_cache, *vp = (f16*)v_cache, *op = (f16*)out;
    hipStream_t s = (hipStream_t)stream;
    const int B = (int)batch, H = (int)heads, L = (int)max_len;
    switch (head_dim) {
        case 32: return launch_attention<4, FUSED>(fn, qp, kp, vp, pos, cos_t, sin_t, op, B, H, L, s);
        case 64: return launch_attention<8, FUSED>(fn, qp, kp, vp, pos, cos_t, sin_t, op, B, H, L, s);
        case 128: return launch_attention<16, FUSED>(fn, qp, kp, vp, pos, cos_t, sin_t, op, B, H, L, s);
        case 256: return launch_attention<32, FUSED>(fn, qp, kp, vp, pos, cos_t, sin_t, op, B, H, L, s);
        default: return fail(fn, "head_dim must be 32, 64, 128 or 256");
    }
}

}  // namespace

extern "C" int qf_add_rmsnorm(uint16_t* x, const uint16_t* delta, const uint16_t* weight, uint16_t* out, int64_t rows,
                              int64_t hidden, float eps, void* stream) {
    if (!x || !weight || !out) return fail("qf_add_rmsnorm", "null pointer");
    if (rows <= 0 || hidden <= 0 || hidden % 8 != 0) return fail("qf_add_rmsnorm", "rows positive, hidden a positive multiple of 8");
    if (hidden > kThreads * 8 * kNormVec) return fail("qf_add_rmsnorm", "hidden above 16384");
    if (rows > 0x7fffffff) return fail("qf_add_rmsnorm", "too many rows");
    hipLaunchKernelGGL(add_rmsnorm_kernel, dim3((unsigned)rows), dim3(kThreads), 0, (hipStream_t)stream, (f16*)x, (const f16*)delta,
                       (const f16*)weight, (f16*)out, (int)hidden, eps);
    return launched("qf_add_rmsnorm");
}

extern "C" int qf_rope_kv_store(const uint16_t* qkv, const int64_t* pos, const float* cos_table, const float* sin_table,
                                uint16_t* q_out, uint16_t* k_cache, uint16_t* v_cache, int64_t batch, int64_t heads,
                                int64_t head_dim, int64_t max_len, void* stream) {
    if (!qkv || !pos || !cos_table || !sin_table || !q_out || !k_cache || !v_cache) return fail("qf_rope_kv_store", "null pointer");
    if (batch <= 0 || heads <= 0 || head_dim <= 0 || head_dim % 2 != 0 || max_len <= 0)
        return fail("qf_rope_kv_store", "batch, heads, max_len positive and head_dim even");
    const int64_t pairs = batch * heads * (head_dim / 2);
    if (pairs > (int64_t)0x7fffffff * kThreads || batch * heads * max_len * head_dim < 0) return fail("qf_rope_kv_store", "problem too large");
    hipLaunchKernelGGL(rope_kv_store_kernel, dim3((unsigned)((pairs + kThreads - 1) / kThreads)), dim3(kThreads), 0, (hipStream_t)stream,
                       (const f16*)qkv, pos, cos_table, sin_table, (f16*)q_out, (f16*)k_cache, (f16*)v_cache, (int)batch,
                       (int)heads, (int)head_dim, (int)max_len);
    return launched("qf_rope_kv_store");
}

extern "C" int qf_rope_kv_store_rows(const uint16_t* qkv, const int64_t* pos, const float* cos_table, const float* sin_table,
                                     uint16_t* q_out, uint16_t* k_cache, uint16_t* v_cache, int64_t batch, int64_t tokens,
                                     int64_t heads, int64_t head_dim, int64_t max_len, void* stream) {
    if (!qkv || !pos || !cos_table || !sin_table || !q_out || !k_cache || !v_cache) return fail("qf_rope_kv_store_rows", "null pointer");
    if (batch <= 0 || tokens <= 0 || heads <= 0 || head_dim <= 0 || head_dim % 8 != 0 || max_len <= 0)
        return fail("qf_rope_kv_store_rows", "batch, tokens, heads, max_len positive and head_dim a multiple of 8");
    if (tokens > 0x7fffffff || heads > 0x7fffffff || head_dim > 0x7fffffff || max_len > 0x7fffffff || batch > 0x7fffffff)
        return fail("qf_rope_kv_store_rows", "dimension too large");
    const int64_t units = batch * tokens * heads * (head_dim / 8);
    if (units > (int64_t)0x7fffffff * kThreads) return fail("qf_rope_kv_store_rows", "problem too large");
    hipLaunchKernelGGL(rope_kv_store_rows_kernel, dim3((unsigned)((units + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                       (hipStream_t)stream, (const f16*)qkv, pos, cos_table, sin_table, (f16*)q_out, (f16*)k_cache, (f16*)v_cache,
                       (int)batch, (int)tokens, (int)heads, (int)head_dim, (int)max_len);
    return launched("qf_rope_kv_store_rows");
}

extern "C" int qf_decode_attention(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache, const int64_t* pos,
                                   uint16_t* out, int64_t batch, int64_t heads, int64_t head_dim, int64_t max_len, void* stream) {
    if (!q || !k_cache || !v_cache || !pos || !out) return fail("qf_decode_attention", "null pointer");
    // the caches are only read on this path
    return dispatch_attention<false>("qf_decode_attention", q, const_cast<uint16_t*>(k_cache), const_cast<uint16_t*>(v_cache), pos,
                                     nullptr, nullptr, out, batch, heads, head_dim, max_len, stream);
}

extern "C" int qf_rope_decode_attention(const uint16_t* qkv, const int64_t* pos, const float* cos_table, const float* sin_table,
                                        uint16_t* k_cache, uint16_t* v_cache, uint16_t* out, int64_t batch, int64_t heads,
                                        int64_t head_dim, int64_t max_len, void* stream) {
    if (!qkv || !pos || !cos_table || !sin_table || !k_cache || !v_cache || !out) return fail("qf_rope_decode_attention", "null pointer");
    return dispatch_attention<true>("qf_rope_decode_attention", qkv, k_cache, v_cache, pos, cos_table, sin_table, out, batch, heads,
                                    head_dim, max_len, stream);
}

extern "C" int qf_silu_mul(const uint16_t* gate_up, uint16_t* out, int64_t rows, int64_t mlp, void* stream) {
    if (!gate_up || !out) return fail("qf_silu_mul", "null pointer");
    if (rows <= 0 || mlp <= 0 || mlp % 8 != 0) return fail("qf_silu_mul", "rows positive, mlp a positive multiple of 8");
    const int64_t work = rows * (mlp / 8);
    if (mlp > 0x7fffffff || work > (int64_t)0x7fffffff * kThreads) return fail("qf_silu_mul", "problem too large");
    hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)((work + kThreads - 1) / kThreads)), dim3(kThreads), 0, (hipStream_t)stream,
                       (const f16*)gate_up, (f16*)out, rows, (int)mlp);
    return launched("qf_silu_mul");
}

extern "C" int qf_greedy_next(const uint16_t* logits, int64_t* tok, int64_t* pos, const uint16_t* embed, uint16_t* x_next,
                              int64_t batch, int64_t vocab, int64_t hidden, void* stream) {
    if (!logits || !tok) return fail("qf_greedy_next", "null pointer");
    if ((embed == nullptr) != (x_next == nullptr)) return fail("qf_greedy_next", "embed and x_next come together");
    if (batch <= 0 || batch > 0x7fffffff || vocab <= 0 || vocab > 0x7fffff00 || vocab % 8 != 0)
        return fail("qf_greedy_next", "batch positive, vocab a positive multiple of 8");
    if (embed && (hidden <= 0 || hidden > 0x7fffffff || hidden % 8 != 0)) return fail("qf_greedy_next", "hidden a positive multiple of 8");
    hipLaunchKernelGGL(greedy_next_kernel, dim3((unsigned)batch), dim3(kPickThreads), 0, (hipStream_t)stream, (const f16*)logits, tok,
                       pos, (const f16*)embed, (f16*)x_next, (int)vocab, (int)hidden);
    return launched("qf_greedy_next");
}
