// libqfactory_hip.so: device-side repacking and memory-system calibration kernels for gfx950.
// Entry points and their contracts are declared in include/qfactory_hip.h.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <stdint.h>

#include "qfactory_hip.h"

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

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

// ---------------------------------------------------------------------------------------------
// Weight repack.  One thread builds one 32-bit output word of one output row.  Threads of a
// block are arranged 32 (rows n) x 8 (words): the reads of weight[k][n] are contiguous over n
// (128 B per k), the 4-byte writes of a row are contiguous over the 8 words.
// Position j of a word holds element (j < P/2 ? 2j : 2(j - P/2) + 1) of its P = 32/b elements
// (identity for 8-bit): evens in the low half-word, odds in the high half-word.  The 1-bit plane
// of the 3-bit layout has its own order (hi_plane_pos): every high bit sits where one shift of
// the word drops it directly above the element's field in the 2-bit plane.
// ---------------------------------------------------------------------------------------------
__host__ __device__ constexpr int hi_plane_pos(int e) {
    const int r = e / 16, ep = e % 16, i = ep / 2, h = ep % 2, p = i % 4, upper = i / 4;
    return ((p % 2 == 0) ? 2 * p + 2 : 2 * p - 2) + 8 * upper + r + 16 * h;
}

template <int B>   // field width of the plane being written: 1, 2, 4 or 8
__device__ __forceinline__ uint32_t build_word(const int32_t* __restrict__ weight, int64_t N, int64_t n,
                                               int64_t k0, int shift, uint32_t mask) {
    constexpr int P = 32 / B;
    uint32_t word = 0;
#pragma unroll
    for (int j = 0; j < P; j++) {
        // hi_plane_pos is its own inverse: bit j holds element hi_plane_pos(j)
        const int src = (B == 8) ? j : (B == 1) ? hi_plane_pos(j) : (j < P / 2 ? 2 * j : 2 * (j - P / 2) + 1);
        const uint32_t v = ((uint32_t)weight[(k0 + src) * N + n] >> shift) & mask;
        word |= v << (j * B);
    }
    return word;
}

template <int B>
__global__ __launch_bounds__(256) void pack_plane_kernel(const int32_t* __restrict__ weight, uint32_t* __restrict__ out,
                                                         int64_t K, int64_t N, int64_t row_words, int64_t word_offset,
                                                         int shift, uint32_t mask) {
    constexpr int P = 32 / B;
    const int64_t n = (int64_t)blockIdx.x * 32 + (threadIdx.x & 31);
    const int64_t wi = (int64_t)blockIdx.y * 8 + (threadIdx.x >> 5);
    if (n >= N || wi >= K / P) return;
    out[n * row_words + word_offset + wi] = build_word<B>(weight, N, n, wi * P, shift, mask);
}

template <int B>
void launch_plane(const int32_t* weight, int8_t* out, int64_t K, int64_t N, int64_t row_words, int64_t word_offset,
                  int shift, uint32_t mask, hipStream_t stream) {
    constexpr int P = 32 / B;
    dim3 grid((unsigned)((N + 31) / 32), (unsigned)((K / P + 7) / 8));
    hipLaunchKernelGGL(pack_plane_kernel<B>, grid, dim3(256), 0, stream, weight, (uint32_t*)out, K, N, row_words,
                       word_offset, shift, mask);
}

__global__ __launch_bounds__(256) void pack_zero_kernel(const int32_t* __restrict__ zero, uint8_t* __restrict__ out,
                                                        int64_t G, int64_t N, int nbits, int fb) {
    const int p8 = 8 / fb;
    const int64_t row_bytes = G / p8;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;      // over N * row_bytes, n fastest
    if (idx >= N * row_bytes) return;
    const int64_t n = idx % N, byte = idx / N;
    const int32_t maxv = (1 << nbits) - 1;
    uint32_t v = 0;
    for (int i = 0; i < p8; i++) {
        int32_t z = zero[(byte * p8 + i) * N + n] + 1;
        z = z > maxv ? maxv : z;
        v |= (uint32_t)z << (i * fb);
    }
    out[n * row_bytes + byte] = (uint8_t)v;
}

__global__ __launch_bounds__(256) void transpose_u16_kernel(const uint16_t* __restrict__ in, uint16_t* __restrict__ out,
                                                            int64_t G, int64_t N) {
    __shared__ uint16_t tile[32][33];
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;           // 32 x 8
    const int64_t n0 = (int64_t)blockIdx.x * 32, g0 = (int64_t)blockIdx.y * 32;
    for (int r = ty; r < 32; r += 8)
        if (g0 + r < G && n0 + tx < N) tile[r][tx] = in[(g0 + r) * N + n0 + tx];
    __syncthreads();
    for (int r = ty; r < 32; r += 8)
        if (n0 + r < N && g0 + tx < G) out[(n0 + r) * G + g0 + tx] = tile[tx][r];
}

// ---------------------------------------------------------------------------------------------
// Calibration kernels
// ---------------------------------------------------------------------------------------------
constexpr int kStreamThreads = 256;
constexpr int kStreamUnroll = 4;

// Every thread requests kStreamUnroll 16-byte units, all before it touches any, and folds them into one word.  The
// word is stored only if it equals a fixed constant, which random data practically never does: the loads cannot
// be dropped and the block ends with its last byte -- no cross-lane sum, no barrier, no store.  (A version that
// wrote one checksum word per block through a wave shuffle and LDS measured 6 % slower at 47 MB: the read ceiling
// is what this kernel is for.)
__global__ __launch_bounds__(kStreamThreads) void stream_read_kernel(const u32x4* __restrict__ src, size_t n16,
                                                                     uint32_t* __restrict__ sink) {
    const size_t per_block = (size_t)kStreamThreads * kStreamUnroll;
    size_t base = (size_t)blockIdx.x * per_block + threadIdx.x;
    uint32_t acc = 0;
    u32x4 v[kStreamUnroll];
#pragma unroll
    for (int u = 0; u < kStreamUnroll; u++) {
        const size_t i = base + (size_t)u * kStreamThreads;
        v[u] = __builtin_nontemporal_load(src + (i < n16 ? i : n16 - 1));
    }
#pragma unroll
    for (int u = 0; u < kStreamUnroll; u++) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    if (acc == 0x9E3779B9u) sink[blockIdx.x & 4095] = acc;
}

__global__ __launch_bounds__(kStreamThreads) void stream_copy_kernel(u32x4* __restrict__ dst, const u32x4* __restrict__ src,
                                                                     size_t n16) {
    const size_t per_block = (size_t)kStreamThreads * kStreamUnroll;
    size_t base = (size_t)blockIdx.x * per_block + threadIdx.x;
    u32x4 v[kStreamUnroll];
#pragma unroll
    for (int u = 0; u < kStreamUnroll; u++) {
        const size_t i = base + (size_t)u * kStreamThreads;
        if (i < n16) v[u] = __builtin_nontemporal_load(src + i);
    }
#pragma unroll
    for (int u = 0; u < kStreamUnroll; u++) {
        const size_t i = base + (size_t)u * kStreamThreads;
        if (i < n16) __builtin_nontemporal_store(v[u], dst + i);
    }
}

// bf16 -> fp16, eight elements per thread: exact wherever fp16 is normal, magnitudes above 65504 saturate
// (the conversion rounds toward zero), infinities and NaN pass through -- the conversion the quantized-linear
// kernels apply to bf16 activations they read themselves.
__device__ __forceinline__ uint32_t bf16_pair_to_f16_pair(uint32_t v) {
    const float lo = __builtin_bit_cast(float, v << 16);
    const float hi = __builtin_bit_cast(float, v & 0xFFFF0000u);
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
}

__global__ __launch_bounds__(256) void bf16_to_f16_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                          int64_t n) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
    if (i + 8 <= n) {
        const u32x4 v = *reinterpret_cast<const u32x4*>(src + i);
        *reinterpret_cast<u32x4*>(dst + i) = u32x4{bf16_pair_to_f16_pair(v.x), bf16_pair_to_f16_pair(v.y),
                                                   bf16_pair_to_f16_pair(v.z), bf16_pair_to_f16_pair(v.w)};
    } else {
        for (int64_t j = i; j < n; j++) dst[j] = (uint16_t)bf16_pair_to_f16_pair(src[j]);
    }
}

}  // namespace

extern "C" int qf_version(void) { return 102; }

extern "C" int qf_bf16_to_f16(const uint16_t* src, uint16_t* dst, int64_t n, void* stream_) {
    if (!src || !dst) return fail("qf_bf16_to_f16", "null pointer");
    if (n <= 0) return fail("qf_bf16_to_f16", "n must be positive");
    if (((uintptr_t)src | (uintptr_t)dst) % 16 != 0) return fail("qf_bf16_to_f16", "src and dst must be 16-byte aligned");
    hipLaunchKernelGGL(bf16_to_f16_kernel, dim3((unsigned)((n + 2047) / 2048)), dim3(256), 0, (hipStream_t)stream_, src, dst, n);
    return launched("qf_bf16_to_f16");
}

extern "C" int qf_pack_weight(const int32_t* weight, int8_t* out, int64_t K, int64_t N, int nbits, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (!weight || !out) return fail("qf_pack_weight", "null pointer");
    if (K <= 0 || N <= 0 || K % 32 != 0) return fail("qf_pack_weight", "K must be a positive multiple of 32, N positive");
    const uint32_t mask = (1u << nbits) - 1u;
    const int64_t row_words = K * nbits / 32;
    switch (nbits) {
        case 8: launch_plane<8>(weight, out, K, N, row_words, 0, 0, mask, stream); break;
        case 4: launch_plane<4>(weight, out, K, N, row_words, 0, 0, mask, stream); break;
        case 2: launch_plane<2>(weight, out, K, N, row_words, 0, 0, mask, stream); break;
        case 3:   // low two bits in the 2-bit layout, then the high bit as a 1-bit plane
            launch_plane<2>(weight, out, K, N, row_words, 0, 0, 3u, stream);
            launch_plane<1>(weight, out, K, N, row_words, K / 16, 2, 1u, stream);
            break;
        default: return fail("qf_pack_weight", "nbits must be 2, 3, 4 or 8");
    }
    return launched("qf_pack_weight");
}

extern "C" int qf_pack_zero(const int32_t* zero, int8_t* out, int64_t G, int64_t N, int nbits, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (!zero || !out) return fail("qf_pack_zero", "null pointer");
    if (nbits != 2 && nbits != 3 && nbits != 4 && nbits != 8) return fail("qf_pack_zero", "nbits must be 2, 3, 4 or 8");
    const int fb = nbits == 3 ? 4 : nbits;
    if (G <= 0 || N <= 0 || G % (8 / fb) != 0) return fail("qf_pack_zero", "G must fill whole bytes of zero-points");
    const int64_t total = N * (G / (8 / fb));
    hipLaunchKernelGGL(pack_zero_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, zero, (uint8_t*)out, G,
                       N, nbits, fb);
    return launched("qf_pack_zero");
}

extern "C" int qf_transpose_scale(const uint16_t* scale, uint16_t* out, int64_t G, int64_t N, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (!scale || !out) return fail("qf_transpose_scale", "null pointer");
    if (G <= 0 || N <= 0) return fail("qf_transpose_scale", "G and N must be positive");
    dim3 grid((unsigned)((N + 31) / 32), (unsigned)((G + 31) / 32));
    hipLaunchKernelGGL(transpose_u16_kernel, grid, dim3(256), 0, stream, scale, out, G, N);
    return launched("qf_transpose_scale");
}

__global__ void empty_kernel(uint32_t* sink) {
    if (sink == nullptr && threadIdx.x == 0xFFFFu) sink[0] = 1;     // never true: the kernel does nothing
}

extern "C" int qf_empty_launch(int64_t blocks, int64_t threads, void* stream_) {
    if (blocks <= 0 || blocks > 0x7fffffff || threads <= 0 || threads > 1024) return fail("qf_empty_launch", "blocks positive, threads in 1..1024");
    hipLaunchKernelGGL(empty_kernel, dim3((unsigned)blocks), dim3((unsigned)threads), 0, (hipStream_t)stream_, (uint32_t*)nullptr);
    return launched("qf_empty_launch");
}

extern "C" int qf_stream_read(const void* src, size_t bytes, uint32_t* sink, void* stream_) {
    if (!src || !sink) return fail("qf_stream_read", "null pointer");
    if (bytes == 0 || bytes % 16 != 0) return fail("qf_stream_read", "bytes must be a positive multiple of 16");
    const size_t n16 = bytes / 16, per_block = (size_t)kStreamThreads * kStreamUnroll;
    hipLaunchKernelGGL(stream_read_kernel, dim3((unsigned)((n16 + per_block - 1) / per_block)), dim3(kStreamThreads), 0,
                       (hipStream_t)stream_, (const u32x4*)src, n16, sink);
    return launched("qf_stream_read");
}

extern "C" int qf_stream_copy(void* dst, const void* src, size_t bytes, void* stream_) {
    if (!dst || !src) return fail("qf_stream_copy", "null pointer");
    if (bytes == 0 || bytes % 16 != 0) return fail("qf_stream_copy", "bytes must be a positive multiple of 16");
    const size_t n16 = bytes / 16, per_block = (size_t)kStreamThreads * kStreamUnroll;
    hipLaunchKernelGGL(stream_copy_kernel, dim3((unsigned)((n16 + per_block - 1) / per_block)), dim3(kStreamThreads), 0,
                       (hipStream_t)stream_, (u32x4*)dst, (const u32x4*)src, n16);
    return launched("qf_stream_copy");
}
