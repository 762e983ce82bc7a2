/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's quantized-linear path.
 *
 * This file is the parity checker for the HIP kernels and for the packer.  It is
 * plain scalar C, written to be obviously right rather than fast.  Nothing that
 * ships (the qfactory package, the JIT'd kernels, the AOT library) may link,
 * load or call it; only tests/, the smoke check and the cpu_baseline leg of the
 * bench do, and only as the checker.
 *
 * What each function follows in the reference (paths relative to the reference root):
 *   qfo_pack_weight      qfactory/convert.py:49-68   (PERMUTE_ORDER + _transform_weight_basic)
 *   qfo_pack_zero        qfactory/convert.py:74-81   (_transform_zero: +1, clamp, pack along groups)
 *   qfo_transpose_scale  qfactory/convert.py:70-72   (_transform_scale)
 *   qfo_unpack_weight    qfactory/include/utils.h:11-25 (decode order: pair i of a word is
 *                        ((w >> b*i) & MASK, (w >> (b*i+16)) & MASK)); 8-bit: utils.h:29-34
 *   qfo_unpack_zero      qfactory/include/gptq_gemv.h:65-82 (fetch_scale_zero: byte g/P8, field g%P8;
 *                        SYM -> 1 << (b-1))
 *   qfo_dequant          qfactory/include/utils.h:46-81 (eager decode: fp16_rn((q - Z) * s), one rounding)
 *   qfo_qlinear          tests/acc_gptq.py:31-38,52 (dequantise, then activation @ dequant_w) with the
 *                        accumulation the acceptance bar names (fp32 or wider; here double, rounded
 *                        once to fp16 at the end)
 *   qfo_gemv_plain       tests/acc_gemv.py:12-14   (activation @ weight.to(fp16), no scale / zero)
 *
 * 3-bit has no counterpart in the reference (PERMUTE_ORDER has keys 8/4/2 only,
 * convert.py:49-53).  The layout restated here is this project's own:
 * per row, a 2-bit plane (low two bits, packed exactly like the reference's
 * 2-bit layout) of K/4 bytes followed by a 1-bit plane (high bit) of K/8 bytes.
 * A 32-bit word of the 1-bit plane serves the two 2-bit words of the same 32
 * elements; element e sits at the bit that, after one shift of the whole word,
 * lands directly above that element's 2-bit field (hi_plane_pos below), so a
 * kernel merges the planes with one AND-OR per element pair.
 * Zero-points for 3-bit are stored one per nibble (two groups per byte).
 * PARITY UNPINNED by the reference for NBITS == 3: only round trips, the
 * dequant+matmul identity and the special cases in tests/ pin it.
 *
 * Pinned by tests/test_oracle.py: hand-worked known-answer vectors for every
 * packer, decode-order round trips, and closed-form special cases of the
 * forward (integer GEMV, one-hot activations, constant weights).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>

/* ---------- fp16 <-> fp32, IEEE round-to-nearest-even, written out by hand ---------- */

static float h2f(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: value = man * 2^-24 */
            float v = (float)man * (1.0f / 16777216.0f);
            memcpy(&bits, &v, 4);
            bits |= sign;
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* Round a double to the nearest fp16 (ties to even), overflow to inf. */
static uint16_t d2h(double d) {
    uint16_t sign = 0;
    if (d != d) return 0x7E00u;
    if (d < 0 || (d == 0 && 1.0 / d < 0)) { sign = 0x8000u; d = -d; }
    if (d == 0) return sign;
    if (d >= 65520.0) return sign | 0x7C00u;           /* >= max + half ulp rounds to inf */
    int e;
    double m = frexp(d, &e);                            /* d = m * 2^e, m in [0.5,1) */
    int exp = e - 1;                                    /* d = (2m) * 2^exp, 2m in [1,2) */
    if (exp < -14) {                                    /* subnormal: quantum 2^-24 */
        double q = nearbyint(ldexp(d, 24));             /* default rounding mode = ties-to-even */
        return sign | (uint16_t)q;                      /* q may be 1024 -> smallest normal, bit pattern still right */
    }
    double q = nearbyint(ldexp(d, 10 - exp));           /* in [1024, 2048] */
    uint32_t qi = (uint32_t)q;
    if (qi == 2048u) { qi = 1024u; exp += 1; }
    if (exp > 15) return sign | 0x7C00u;
    return sign | (uint16_t)(((uint32_t)(exp + 15) << 10) | (qi - 1024u));
}

uint16_t qfo_f32_to_f16(float f) { return d2h((double)f); }
float qfo_f16_to_f32(uint16_t h) { return h2f(h); }

/* ---------- packers (convert.py) ---------- */

static int perm_index(int nbits, int j) {
    /* convert.py:49-53: position j of a 32-bit word holds element PERM[j];
       8-bit identity, else evens first then odds. */
    int p32 = 32 / nbits;
    if (nbits == 8) return j;
    return (j < p32 / 2) ? 2 * j : 2 * (j - p32 / 2) + 1;
}

/* Bit of a 1-bit-plane word that holds the high bit of element e (0..31) of its 32 elements.
   r: which of the two 2-bit words, i: pair inside it, h: half-word (even / odd element),
   p: pair inside its byte, upper: which byte of the half-word. */
static int hi_plane_pos(int e) {
    int r = e / 16, ep = e % 16, i = ep / 2, h = ep % 2, p = i % 4, upper = i / 4;
    int base = (p % 2 == 0) ? 2 * p + 2 : 2 * p - 2;
    return base + 8 * upper + r + 16 * h;
}

/* bytes per packed weight row */
int64_t qfo_row_bytes(int64_t K, int nbits) { return K * nbits / 8; }

/* weight: (K,N) int32 row-major in [0,2^b) -> out: (N, K*b/8) int8 row-major */
int qfo_pack_weight(int64_t K, int64_t N, int nbits, const int32_t *weight, int8_t *out) {
    if (nbits == 3) {
        if (K % 32) return 1;
        int64_t rb = K * 3 / 8, lo_bytes = K / 4;
        for (int64_t n = 0; n < N; n++) {
            uint8_t *row = (uint8_t *)out + n * rb;
            for (int64_t i = 0; i < K / 16; i++) {       /* 2-bit plane, 16 elements per word */
                uint32_t u = 0;
                for (int j = 0; j < 16; j++)
                    u |= ((uint32_t)weight[(i * 16 + perm_index(2, j)) * N + n] & 3u) << (2 * j);
                for (int t = 0; t < 4; t++) row[i * 4 + t] = (uint8_t)(u >> (8 * t));
            }
            for (int64_t i = 0; i < K / 32; i++) {       /* 1-bit plane, 32 elements per word */
                uint32_t u = 0;
                for (int e = 0; e < 32; e++)
                    u |= (((uint32_t)weight[(i * 32 + e) * N + n] >> 2) & 1u) << hi_plane_pos(e);
                for (int t = 0; t < 4; t++) row[lo_bytes + i * 4 + t] = (uint8_t)(u >> (8 * t));
            }
        }
        return 0;
    }
    if (nbits != 2 && nbits != 4 && nbits != 8) return 1;
    int p32 = 32 / nbits;
    if (K % p32) return 1;
    int64_t rb = K * nbits / 8;
    for (int64_t n = 0; n < N; n++) {
        for (int64_t i = 0; i < K / p32; i++) {
            uint32_t u = 0;                                /* convert.py:58-62 */
            for (int j = 0; j < p32; j++)
                u |= (uint32_t)weight[(i * p32 + perm_index(nbits, j)) * N + n] << (j * nbits);
            for (int t = 0; t < 4; t++)                    /* convert.py:64-67: little-endian bytes, transposed */
                ((uint8_t *)out)[n * rb + i * 4 + t] = (uint8_t)(u >> (8 * t));
        }
    }
    return 0;
}

/* storage bits of one zero-point field: equals nbits except 3-bit, stored per nibble */
static int zero_field_bits(int nbits) { return nbits == 3 ? 4 : nbits; }

int64_t qfo_zero_row_bytes(int64_t G, int nbits) { return G * zero_field_bits(nbits) / 8; }

/* zero: (G,N) int32 in [0,2^b) -> out: (N, G*fb/8) int8; stores min(z+1, 2^b-1)  (convert.py:76-80) */
int qfo_pack_zero(int64_t G, int64_t N, int nbits, const int32_t *zero, int8_t *out) {
    int fb = zero_field_bits(nbits);
    int p8 = 8 / fb;
    if (G % p8) return 1;
    int32_t maxv = (1 << nbits) - 1;
    int64_t rb = G / p8;
    memset(out, 0, (size_t)(N * rb));
    for (int64_t g = 0; g < G; g++)
        for (int64_t n = 0; n < N; n++) {
            int32_t zp = zero[g * N + n] + 1;
            if (zp > maxv) zp = maxv;
            ((uint8_t *)out)[n * rb + g / p8] |= (uint8_t)(zp << ((g % p8) * fb));
        }
    return 0;
}

/* scale: (G,N) fp16 -> (N,G) fp16 (convert.py:70-72) */
void qfo_transpose_scale(int64_t G, int64_t N, const uint16_t *scale, uint16_t *out) {
    for (int64_t g = 0; g < G; g++)
        for (int64_t n = 0; n < N; n++) out[n * G + g] = scale[g * N + n];
}

/* ---------- decode side (utils.h / gptq_gemv.h) ---------- */

/* packed (N, K*b/8) -> q (N,K) int32 in natural k order, following the kernel's decode order */
int qfo_unpack_weight(int64_t K, int64_t N, int nbits, const int8_t *w, int32_t *q) {
    int64_t rb = K * nbits / 8;
    if (nbits == 3) {
        int64_t lo_bytes = K / 4;
        for (int64_t n = 0; n < N; n++) {
            const uint8_t *row = (const uint8_t *)w + n * rb;
            for (int64_t i = 0; i < K / 16; i++) {
                uint32_t u;
                memcpy(&u, row + i * 4, 4);
                for (int p = 0; p < 8; p++) {
                    q[n * K + i * 16 + 2 * p] = (int32_t)((u >> (2 * p)) & 3u);
                    q[n * K + i * 16 + 2 * p + 1] = (int32_t)((u >> (2 * p + 16)) & 3u);
                }
            }
            for (int64_t i = 0; i < K / 32; i++) {
                uint32_t u;
                memcpy(&u, row + lo_bytes + i * 4, 4);
                for (int e = 0; e < 32; e++)
                    q[n * K + i * 32 + e] |= (int32_t)(((u >> hi_plane_pos(e)) & 1u) << 2);
            }
        }
        return 0;
    }
    if (nbits == 8) {                                       /* utils.h:29-34: plain bytes, unsigned */
        for (int64_t i = 0; i < N * K; i++) q[i] = (int32_t)((const uint8_t *)w)[i];
        return 0;
    }
    if (nbits != 2 && nbits != 4) return 1;
    int p32 = 32 / nbits;
    uint32_t mask = (1u << nbits) - 1u;
    for (int64_t n = 0; n < N; n++)
        for (int64_t i = 0; i < K / p32; i++) {
            uint32_t u;
            memcpy(&u, (const uint8_t *)w + n * rb + i * 4, 4);
            for (int p = 0; p < p32 / 2; p++) {            /* utils.h:19-23 */
                q[n * K + i * p32 + 2 * p] = (int32_t)((u >> (nbits * p)) & mask);
                q[n * K + i * p32 + 2 * p + 1] = (int32_t)((u >> (nbits * p + 16)) & mask);
            }
        }
    return 0;
}

/* packed zeros (N, G*fb/8) -> Z (N,G) int32; z == NULL means symmetric: Z = 2^(b-1) (gptq_gemv.h:72-80) */
void qfo_unpack_zero(int64_t G, int64_t N, int nbits, const int8_t *z, int32_t *Z) {
    int fb = zero_field_bits(nbits);
    int p8 = 8 / fb;
    uint32_t mask = (1u << fb) - 1u;
    int64_t rb = G / p8;
    for (int64_t n = 0; n < N; n++)
        for (int64_t g = 0; g < G; g++)
            Z[n * G + g] = z ? (int32_t)((((const uint8_t *)z)[n * rb + g / p8] >> ((g % p8) * fb)) & mask)
                             : (1 << (nbits - 1));
}

/* dq (N,K) fp16 bits = fp16_rn((q - Z) * s)   (utils.h:53-60: exact difference, one rounding of the product) */
int qfo_dequant(int64_t K, int64_t N, int nbits, int64_t GS, const int8_t *w, const uint16_t *s,
                const int8_t *z, uint16_t *dq) {
    if (K % GS) return 1;
    int64_t G = K / GS;
    int32_t *q = (int32_t *)calloc((size_t)(N * K), 4);
    int32_t *Z = (int32_t *)malloc((size_t)(N * G) * 4);
    if (!q || !Z) { free(q); free(Z); return 2; }
    int rc = qfo_unpack_weight(K, N, nbits, w, q);
    if (!rc) {
        qfo_unpack_zero(G, N, nbits, z, Z);
        for (int64_t n = 0; n < N; n++)
            for (int64_t k = 0; k < K; k++) {
                double prod = (double)(q[n * K + k] - Z[n * G + k / GS]) * (double)h2f(s[n * G + k / GS]);
                dq[n * K + k] = d2h(prod);
            }
    }
    free(q); free(Z);
    return rc;
}

/* out (M,N) fp16 = fp16_rn( sum_k A[m][k] * dq[n][k] ), sum carried in double */
int qfo_qlinear(int64_t M, int64_t N, int64_t K, int nbits, int64_t GS, const uint16_t *A,
                const int8_t *w, const uint16_t *s, const int8_t *z, uint16_t *out) {
    uint16_t *dq = (uint16_t *)malloc((size_t)(N * K) * 2);
    float *dqf = (float *)malloc((size_t)K * 4);
    float *af = (float *)malloc((size_t)(M * K) * 4);
    if (!dq || !dqf || !af) { free(dq); free(dqf); free(af); return 2; }
    int rc = qfo_dequant(K, N, nbits, GS, w, s, z, dq);
    if (!rc) {
        for (int64_t i = 0; i < M * K; i++) af[i] = h2f(A[i]);
        for (int64_t n = 0; n < N; n++) {
            for (int64_t k = 0; k < K; k++) dqf[k] = h2f(dq[n * K + k]);
            for (int64_t m = 0; m < M; m++) {
                double acc = 0.0;
                for (int64_t k = 0; k < K; k++) acc += (double)af[m * K + k] * (double)dqf[k];
                out[m * N + n] = d2h(acc);
            }
        }
    }
    free(dq); free(dqf); free(af);
    return rc;
}

/* GS = -1 path: out (M,N) fp16 = fp16_rn( sum_k A[m][k] * q[n][k] ), raw unsigned q (acc_gemv.py:12-14) */
int qfo_gemv_plain(int64_t M, int64_t N, int64_t K, int nbits, const uint16_t *A, const int8_t *w,
                   uint16_t *out) {
    int32_t *q = (int32_t *)calloc((size_t)(N * K), 4);
    if (!q) return 2;
    int rc = qfo_unpack_weight(K, N, nbits, w, q);
    if (!rc)
        for (int64_t m = 0; m < M; m++)
            for (int64_t n = 0; n < N; n++) {
                double acc = 0.0;
                for (int64_t k = 0; k < K; k++) acc += (double)h2f(A[m * K + k]) * (double)q[n * K + k];
                out[m * N + n] = d2h(acc);
            }
    free(q);
    return rc;
}
