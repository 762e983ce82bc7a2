/*
 * C ABI of libqfactory_hip.so, the ahead-of-time part of the MI355X quantized-linear path:
 * device-side repacking (the load-time half of the path) and the memory-system calibration
 * kernels the benchmark uses to put its roofline numbers on a measured footing.
 *
 * All pointers are device addresses owned by the caller; `stream` is a hipStream_t; calls only
 * enqueue work.  Every function returns 0 on success, 1 on invalid arguments (reason on stderr),
 * 2 if the HIP launch failed.
 */
#ifndef QFACTORY_HIP_H
#define QFACTORY_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Library / interface version: major * 100 + minor. */
int qf_version(void);

/*
 * Repack GPTQ-orientation integer weights on the device.
 *   weight (K, N) int32 row-major, values in [0, 2^nbits)  ->  out (N, K*nbits/8) int8.
 * nbits in {2, 3, 4, 8}; K must be a multiple of 32.  Bit-identical to the reference's
 * _transform_weight_basic (qfactory/convert.py:55-68), which this replaces for device tensors;
 * nbits == 3 produces this project's two-plane layout (no reference counterpart).
 */
int qf_pack_weight(const int32_t* weight, int8_t* out, int64_t K, int64_t N, int nbits, void* stream);

/*
 * Repack zero-points on the device.
 *   zero (G, N) int32 in [0, 2^nbits)  ->  out (N, G*fb/8) int8 holding min(zero + 1, 2^nbits - 1),
 * fb = nbits (4 for nbits == 3), group g in field g % (8/fb) of byte g / (8/fb).
 * Replaces _transform_zero (qfactory/convert.py:74-81).
 */
int qf_pack_zero(const int32_t* zero, int8_t* out, int64_t G, int64_t N, int nbits, void* stream);

/*
 * scale (G, N) fp16 -> out (N, G) fp16.  Replaces _transform_scale (qfactory/convert.py:70-72).
 */
int qf_transpose_scale(const uint16_t* scale, uint16_t* out, int64_t G, int64_t N, void* stream);

/*
 * src (n) bf16 -> dst (n) fp16, both 16-byte aligned.  Exact wherever fp16 is normal; magnitudes above
 * 65504 saturate to +-65504, infinities and NaN pass through.  No reference counterpart: the reference
 * takes fp16 activations only (qfactory/core/matmul.py:36, :133-136).  The matrix-core GEMM kernel moves
 * its activation tiles from global memory to LDS without touching registers and cannot convert them on
 * the way; QMatmul's closure converts bf16 rows with this call first (the other kernels convert in
 * registers as they load).
 */
int qf_bf16_to_f16(const uint16_t* src, uint16_t* dst, int64_t n, void* stream);

/*
 * Calibration kernels (no reference counterpart; the reference times with triton's do_bench only,
 * qfactory/profile.py:5-10).  qf_stream_read reads `bytes` (multiple of 16) with 128-bit loads and
 * writes to `sink` (>= 4096 uint32) only where a thread's folded words equal a fixed constant (practically
 * never: the stores exist so that the loads cannot be dropped); qf_stream_copy copies `bytes`
 * (multiple of 16) from src to dst.  They give the achievable HBM rate for a given footprint and a
 * known-traffic dispatch against which hardware counters can be scaled.
 */
int qf_stream_read(const void* src, size_t bytes, uint32_t* sink, void* stream);
int qf_stream_copy(void* dst, const void* src, size_t bytes, void* stream);
/* A kernel that does nothing, `blocks` x `threads` (<= 1024): the launch floor of a given grid. */
int qf_empty_launch(int64_t blocks, int64_t threads, void* stream);

/*
 * Steps of one decode token between the quantized linears of a Llama-style layer, one launch each.
 * The reference has no kernels of its own for them: its end-to-end runs (reproduce/fig11/
 * run_all_qfactory.sh:22-40, through third_party/vllm-qfactory.patch) leave them to vLLM's RMSNorm,
 * rotary-embedding, paged-attention and SiluAndMul ops; the decode loop that stands in for those runs
 * here (decode_llama.py) calls these instead of ~45 small framework kernels per layer.
 * fp16 tensors are passed as uint16_t*; arithmetic inside is fp32.
 *
 * qf_add_rmsnorm: x (rows, hidden) += delta (same shape; NULL: no add), in place, fp16 addition;
 *   out = fp16(fp16(x * rsqrt(mean(x^2) + eps)) * weight).  hidden a multiple of 8, at most 16384.
 * qf_rope_kv_store: qkv (batch, 3, heads, head_dim) of the new position *pos (device int64):
 *   q_out (batch, heads, head_dim) = rotate(q), k_cache[b][h][*pos] = rotate(k), v_cache[b][h][*pos] = v;
 *   caches are (batch, heads, max_len, head_dim); rotation of pairs (2i, 2i+1) by the angles in row
 *   *pos of cos_table / sin_table (max_len, head_dim/2) fp32.  Writes nothing if *pos is outside
 *   [0, max_len).
 * qf_rope_kv_store_rows: the same for `tokens` positions per sequence (prefill): qkv (batch * tokens, 3, heads,
 *   head_dim), row b * tokens + t being token t of sequence b at position pos[t] (tokens device int64 values shared
 *   by the sequences); q_out (batch, tokens, heads, head_dim) = rotate(q), k_cache[b][h][pos[t]] = rotate(k),
 *   v_cache[b][h][pos[t]] = v.  head_dim a multiple of 8; a token whose position is outside [0, max_len) writes nothing.
 * qf_decode_attention: out (batch, heads*head_dim) = softmax(q k^T / sqrt(head_dim)) v over cache
 *   positions 0 .. *pos.  head_dim in {32, 64, 128, 256}.
 * qf_rope_decode_attention: the two above in one launch, straight from the QKV projection: rotates q and k
 *   of position *pos, appends k and v to the caches and writes the attention output; nothing is written
 *   if *pos is outside [0, max_len).  Results equal qf_rope_kv_store followed by qf_decode_attention.
 * qf_silu_mul: out (rows, mlp) = fp16(silu(gate_up[:, :mlp])) * gate_up[:, mlp:]; mlp a multiple of 8.
 * qf_greedy_next: the end of a greedy decode step in one launch: tok[b] = the smallest index of the largest of
 *   logits[b][0 .. vocab) (NaN is never chosen; vocab a multiple of 8), *pos += 1 if pos is given, and, if embed
 *   (vocab, hidden) is given, x_next[b] = embed[tok[b]] -- the residual stream the next step starts from (hidden a
 *   multiple of 8).  No counterpart in the reference, whose end-to-end runs leave sampling to vLLM.
 */
int qf_add_rmsnorm(uint16_t* x, const uint16_t* delta, const uint16_t* weight, uint16_t* out, int64_t rows,
                   int64_t hidden, float eps, void* stream);
int qf_rope_kv_store(const uint16_t* qkv, const int64_t* pos, const float* cos_table, const float* sin_table,
                     uint16_t* q_out, uint16_t* k_cache, uint16_t* v_cache, int64_t batch, int64_t heads,
                     int64_t head_dim, int64_t max_len, void* stream);
int qf_rope_kv_store_rows(const uint16_t* qkv, const int64_t* pos, const float* cos_table, const float* sin_table,
                          uint16_t* q_out, uint16_t* k_cache, uint16_t* v_cache, int64_t batch, int64_t tokens,
                          int64_t heads, int64_t head_dim, int64_t max_len, void* stream);
int qf_decode_attention(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache, const int64_t* pos,
                        uint16_t* out, int64_t batch, int64_t heads, int64_t head_dim, int64_t max_len, void* stream);
int qf_rope_decode_attention(const uint16_t* qkv, const int64_t* pos, const float* cos_table, const float* sin_table,
                             uint16_t* k_cache, uint16_t* v_cache, uint16_t* out, int64_t batch, int64_t heads,
                             int64_t head_dim, int64_t max_len, void* stream);
int qf_silu_mul(const uint16_t* gate_up, uint16_t* out, int64_t rows, int64_t mlp, void* stream);
int qf_greedy_next(const uint16_t* logits, int64_t* tok, int64_t* pos, const uint16_t* embed, uint16_t* x_next,
                   int64_t batch, int64_t vocab, int64_t hidden, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* QFACTORY_HIP_H */
