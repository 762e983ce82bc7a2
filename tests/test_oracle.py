"""Pins the CPU oracle (oracle/qf_oracle.c) before anything is compared against it.

Checks are chosen so that a plausible mistake fails one of them: hand-worked known-answer vectors
for every packer (a wrong permutation, shift or byte order changes them), the decode order of the
kernel side inverting the packer (two different reference files), numpy's fp16 conversion as an
independent rounding routine, and closed-form special cases of the forward.
"""
import numpy as np
import pytest
import torch


# ---------------------------------------------------------------- packers: known answers

def test_pack_weight_kat_4bit(oracle):
    # W[k] = k, K = 8: stored nibble order is elements 0,2,4,6,1,3,5,7 -> word 0x75316420
    w = oracle.pack_weight(np.arange(8, dtype=np.int32).reshape(8, 1), 4)
    assert w.tolist() == [[0x20, 0x64, 0x31, 0x75]]


def test_pack_weight_kat_2bit(oracle):
    # W[k] = k % 4, K = 16: evens (0,2,0,2,...) fill the low half-word, odds (1,3,1,3,...) the high one
    w = oracle.pack_weight((np.arange(16, dtype=np.int32) % 4).reshape(16, 1), 2)
    assert w.view(np.uint8).tolist() == [[0x88, 0x88, 0xDD, 0xDD]]
    assert w.tolist() == [[-120, -120, -35, -35]]


def test_pack_weight_kat_8bit(oracle):
    w = oracle.pack_weight(np.array([[1], [2], [3], [200]], dtype=np.int32), 8)
    assert w.tolist() == [[1, 2, 3, -56]]        # identity order, bytes >= 128 wrap negative


def test_pack_weight_kat_two_words_two_columns(oracle):
    # K = 16 (two words), N = 2: column 0 counts up, column 1 counts down; checks the transpose and
    # that the second word follows the first inside a row.
    W = np.stack([np.arange(16), 15 - np.arange(16)], axis=1).astype(np.int32)
    w = oracle.pack_weight(W, 4).view(np.uint8)
    assert w[0].tolist() == [0x20, 0x64, 0x31, 0x75, 0xA8, 0xEC, 0xB9, 0xFD]
    assert w[1].tolist() == [0xDF, 0x9B, 0xCE, 0x8A, 0x57, 0x13, 0x46, 0x02]


def test_pack_weight_kat_3bit(oracle):
    # 3-bit layout of this project: 2-bit plane (low bits) then 1-bit plane (high bit).
    # W[k] = k % 8 for K = 32: low bits k%4 -> two words 0xDDDD8888.  High bit set for k%8 >= 4, i.e.
    # pairs i = 2,3,6,7 of both 2-bit words: (p, upper) = (2,0),(3,0),(2,1),(3,1) -> bits 6,4,14,12 for
    # the first word and one higher for the second, in both half-words -> 0xF0F0F0F0.
    W = (np.arange(32, dtype=np.int32) % 8).reshape(32, 1)
    w = oracle.pack_weight(W, 3).view(np.uint8)
    assert w.shape == (1, 12)
    assert w[0].tolist() == [0x88, 0x88, 0xDD, 0xDD, 0x88, 0x88, 0xDD, 0xDD, 0xF0, 0xF0, 0xF0, 0xF0]


def test_3bit_planes_merge_with_one_shift_per_class(oracle):
    """The property the 1-bit plane's bit order exists for: after one shift of the whole plane
    word, every high bit sits directly above its element's 2-bit field, so
    (lo & 3<<o) | (hi_shifted & 4<<o) is the 3-bit value at offset o of each half-word."""
    rng = np.random.default_rng(11)
    K = 96
    W = rng.integers(0, 8, size=(K, 1), dtype=np.int32)
    row = oracle.pack_weight(W, 3).view(np.uint8)[0]
    lo = row[: K // 4].copy().view("<u4").astype(np.uint64)
    hi = row[K // 4:].copy().view("<u4").astype(np.uint64)
    M32 = 0xFFFFFFFF
    for j in range(K // 16):
        w, H = int(lo[j]), int(hi[j // 2])
        Hr = H >> (j % 2)
        for upper in (0, 1):
            wd = (w >> 8) if upper else w
            for p in range(4):
                if p % 2 == 0:
                    hsel = (Hr >> 8) if upper else Hr
                else:
                    hsel = (Hr >> 4) if upper else (Hr << 4) & M32
                x = (wd & (0x00030003 << (2 * p))) | (hsel & (0x00040004 << (2 * p)))
                i = p + 4 * upper
                assert (x >> (2 * p)) & 7 == W[16 * j + 2 * i, 0]
                assert (x >> (2 * p + 16)) & 7 == W[16 * j + 2 * i + 1, 0]


def test_pack_zero_kats(oracle):
    # stores min(z + 1, 2^b - 1); group g goes to field g % (8/b) of byte g // (8/b)
    z = oracle.pack_zero(np.array([[0], [14], [15], [7]], dtype=np.int32), 4)
    assert z.view(np.uint8).tolist() == [[0xF1, 0x8F]] and z.tolist() == [[-15, -113]]
    z = oracle.pack_zero(np.array([[0], [1], [2], [3]], dtype=np.int32), 2)
    assert z.view(np.uint8).tolist() == [[0xF9]]
    z = oracle.pack_zero(np.array([[254], [255]], dtype=np.int32), 8)
    assert z.tolist() == [[-1, -1]]
    z = oracle.pack_zero(np.array([[0], [6], [7], [3]], dtype=np.int32), 3)      # nibble per value, clamp at 7
    assert z.view(np.uint8).tolist() == [[0x71, 0x47]]


def test_transpose_scale(oracle):
    s = np.arange(12, dtype=np.float16).reshape(3, 4)
    assert np.array_equal(oracle.transpose_scale(s), s.T)


# ---------------------------------------------------------------- decode side inverts the packers

@pytest.mark.parametrize("nbits", [2, 3, 4, 8])
@pytest.mark.parametrize("K,N", [(32, 1), (64, 5), (256, 7)])
def test_decode_order_inverts_packer(oracle, nbits, K, N):
    rng = np.random.default_rng(nbits * 1000 + K + N)
    W = rng.integers(0, 2 ** nbits, size=(K, N), dtype=np.int32)
    packed = oracle.pack_weight(W, nbits)
    assert packed.shape == (N, K * nbits // 8) and packed.dtype == np.int8
    assert np.array_equal(oracle.unpack_weight(packed, K, nbits), W.T)


def test_decode_pairs_by_hand_4bit(oracle):
    # independent of the oracle's unpacker: decode one word with the pair rule of the kernels,
    # pair i = ((w >> 4i) & 15, (w >> (4i + 16)) & 15)
    W = np.array([3, 9, 14, 0, 7, 7, 1, 12], dtype=np.int32).reshape(8, 1)
    word = int(oracle.pack_weight(W, 4).view(np.uint32)[0, 0])
    got = []
    for i in range(4):
        got += [(word >> (4 * i)) & 15, (word >> (4 * i + 16)) & 15]
    assert got == W[:, 0].tolist()


@pytest.mark.parametrize("nbits", [2, 3, 4, 8])
def test_zero_round_trip_and_clamp(oracle, nbits):
    rng = np.random.default_rng(7 + nbits)
    G, N = 8, 6
    z = rng.integers(0, 2 ** nbits, size=(G, N), dtype=np.int32)
    z[0, 0], z[1, 0] = 2 ** nbits - 1, 0
    Z = oracle.unpack_zero(oracle.pack_zero(z, nbits), N, G, nbits)
    assert np.array_equal(Z, np.minimum(z + 1, 2 ** nbits - 1).T)
    # the reference's own test oracle (tests/acc_gptq.py:36) dequantises with the UNCLAMPED z + 1;
    # it differs from what the packed tensors hold exactly where z == 2^b - 1
    assert Z[0, 0] == 2 ** nbits - 1 != z[0, 0] + 1


@pytest.mark.parametrize("nbits", [2, 3, 4, 8])
def test_symmetric_zero_is_half_range(oracle, nbits):
    assert np.all(oracle.unpack_zero(None, 3, 4, nbits) == 2 ** (nbits - 1))


# ---------------------------------------------------------------- fp16 rounding

def test_fp16_conversion_matches_numpy(oracle):
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.normal(size=2000).astype(np.float32) * 10.0 ** rng.integers(-8, 5, size=2000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 6.1e-5, 6.097e-5,
                  1.0009765625, 1.00048828125, 1.00146484375, -3.0e-3], dtype=np.float32)])
    lib = oracle.lib()
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([lib.qfo_f32_to_f16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)
    back = np.array([lib.qfo_f16_to_f32(int(h)) for h in range(0, 0x7C00, 7)], dtype=np.float32)
    assert np.array_equal(back, np.arange(0, 0x7C00, 7, dtype=np.uint16).view(np.float16).astype(np.float32))


# ---------------------------------------------------------------- dequant and forward

def _random_problem(rng, M, N, K, nbits, GS, sym=False):
    W = rng.integers(0, 2 ** nbits, size=(K, N), dtype=np.int32)
    scale = rng.uniform(0.001, 0.02, size=(K // GS, N)).astype(np.float16)
    zero = None if sym else rng.integers(0, 2 ** nbits, size=(K // GS, N), dtype=np.int32)
    A = rng.normal(size=(M, K)).astype(np.float16)
    return A, W, scale, zero


@pytest.mark.parametrize("nbits", [2, 3, 4, 8])
@pytest.mark.parametrize("sym", [False, True])
def test_dequant_elementwise(oracle, nbits, sym):
    # fp16_rn((q - Z) * s): recomputed element by element with numpy scalars from the UNPACKED
    # inputs (not from the oracle's unpackers)
    rng = np.random.default_rng(11 * nbits + sym)
    K, N, GS = 128, 5, 32
    A, W, scale, zero = _random_problem(rng, 1, N, K, nbits, GS, sym)
    w, s = oracle.pack_weight(W, nbits), oracle.transpose_scale(scale)
    z = None if sym else oracle.pack_zero(zero, nbits)
    dq = oracle.dequant(w, s, z, K, nbits, GS)
    for n in range(N):
        for k in range(K):
            Z = 2 ** (nbits - 1) if sym else min(int(zero[k // GS, n]) + 1, 2 ** nbits - 1)
            want = np.float16(np.float32(int(W[k, n]) - Z) * np.float32(scale[k // GS, n]))
            assert dq[n, k] == want, (n, k)
    assert np.array_equal(dq, oracle.dequant_np(w, s, z, K, nbits, GS))


@pytest.mark.parametrize("nbits", [2, 4, 8])
def test_forward_one_hot_selects_dequantised_column(oracle, nbits):
    rng = np.random.default_rng(5)
    M, K, N, GS = 3, 128, 9, 32
    _, W, scale, zero = _random_problem(rng, M, N, K, nbits, GS)
    w, s, z = oracle.pack_weight(W, nbits), oracle.transpose_scale(scale), oracle.pack_zero(zero, nbits)
    A = np.zeros((M, K), dtype=np.float16)
    ks = [0, 77, 127]
    for m, k in enumerate(ks):
        A[m, k] = 1.0
    out = oracle.qlinear(A, w, s, z, nbits, GS)
    dq = oracle.dequant(w, s, z, K, nbits, GS)
    for m, k in enumerate(ks):
        assert np.array_equal(out[m], dq[:, k])


def test_forward_constant_weights_closed_form(oracle):
    # q == c everywhere, one scale and zero per row -> out[m][n] = fp16(d_n * sum(A[m])), d_n = fp16((c - Z_n) s_n)
    nbits, K, N, GS, c = 4, 256, 4, 128, 11
    rng = np.random.default_rng(9)
    W = np.full((K, N), c, dtype=np.int32)
    scale = np.repeat(rng.uniform(0.001, 0.02, size=(1, N)).astype(np.float16), K // GS, axis=0)
    zero = np.repeat(rng.integers(0, 15, size=(1, N), dtype=np.int32), K // GS, axis=0)
    A = rng.integers(-4, 5, size=(2, K)).astype(np.float16)      # integers: the sum is exact
    out = oracle.qlinear(A, oracle.pack_weight(W, nbits), oracle.transpose_scale(scale),
                         oracle.pack_zero(zero, nbits), nbits, GS)
    for n in range(N):
        d = np.float16(np.float32(c - (zero[0, n] + 1)) * np.float32(scale[0, n]))
        for m in range(2):
            assert out[m, n] == np.float16(float(d) * float(A[m].astype(np.float64).sum()))


@pytest.mark.parametrize("nbits", [2, 3, 4, 8])
def test_plain_gemv_is_integer_matmul(oracle, nbits):
    # no scales / zeros: with small integer activations every product and sum is exact
    rng = np.random.default_rng(3 + nbits)
    M, K, N = 4, 96, 10
    W = rng.integers(0, 2 ** nbits, size=(K, N), dtype=np.int32)
    A = rng.integers(-3, 4, size=(M, K)).astype(np.float16)
    out = oracle.gemv_plain(A, oracle.pack_weight(W, nbits), nbits)
    want = (A.astype(np.int64) @ W.astype(np.int64)).astype(np.float16)
    assert np.array_equal(out, want)
    assert np.array_equal(oracle.gemv_plain_np(A, oracle.pack_weight(W, nbits), nbits), want)


@pytest.mark.parametrize("nbits,sym", [(4, False), (4, True), (2, False), (8, False), (3, False)])
def test_forward_matches_float64_matmul_of_dequant(oracle, nbits, sym):
    rng = np.random.default_rng(21 + nbits)
    M, K, N, GS = 5, 512, 33, 128
    A, W, scale, zero = _random_problem(rng, M, N, K, nbits, GS, sym)
    w, s = oracle.pack_weight(W, nbits), oracle.transpose_scale(scale)
    z = None if sym else oracle.pack_zero(zero, nbits)
    out = oracle.qlinear(A, w, s, z, nbits, GS)
    dq = oracle.dequant(w, s, z, K, nbits, GS)
    want = (A.astype(np.float64) @ dq.astype(np.float64).T)
    # same numbers, summed in a different order by BLAS: allow one fp16 ulp
    assert np.max(np.abs(out.astype(np.float64) - want) / np.maximum(np.abs(want), 1e-3)) < 2 ** -10
    m = oracle.error_metrics(oracle.qlinear_np(A, w, s, z, nbits, GS), out)
    assert m["max_rel"] < 2 ** -10


def test_torch_cpu_port_agrees_with_oracle(oracle):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(2)
    for nbits, sym in [(4, False), (2, False), (8, True)]:
        M, K, N, GS = 2, 512, 17, 128
        A, W, scale, zero = _random_problem(rng, M, N, K, nbits, GS, sym)
        w, s = oracle.pack_weight(W, nbits), oracle.transpose_scale(scale)
        z = None if sym else oracle.pack_zero(zero, nbits)
        got = oracle.torch_cpu_forward(torch.from_numpy(A), torch.from_numpy(w), torch.from_numpy(s),
                                       None if z is None else torch.from_numpy(z), nbits, GS).numpy()
        m = oracle.error_metrics(got, oracle.qlinear(A, w, s, z, nbits, GS))
        assert m["max_rel"] < 2e-3 and m["nrms"] < 5e-4


# ---- bf16 activations / output (no reference counterpart; the oracle's conversions against torch's CPU casts) ----

def _all_bf16_bits():
    return np.arange(65536, dtype=np.uint32).astype(np.uint16)


def test_bf16_widening_equals_torch_on_every_bit_pattern(oracle):
    bits = _all_bf16_bits()
    t = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16)
    assert np.array_equal(oracle.bf16_bits_to_f32(bits).view(np.uint32), t.float().numpy().view(np.uint32))


def test_bf16_rounding_equals_torch(oracle):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(200000, generator=g) * torch.exp(torch.randn(200000, generator=g) * 8)
    x = torch.cat([x, torch.tensor([0.0, -0.0, float("inf"), -float("inf"), 3.3895314e38, 3.4e38, 1e-40,
                                    1.00390625, 1.01171875])])          # the last two are ties: to even
    ref = x.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16_bits(x.numpy()), ref)
    assert oracle.f32_to_bf16_bits(np.array([np.nan], dtype=np.float32))[0] == 0x7FC0


def test_bf16_to_fp16_is_exact_where_fp16_is_normal_and_saturates_above(oracle):
    bits = _all_bf16_bits()
    f = oracle.bf16_bits_to_f32(bits)
    h = oracle.bf16_bits_to_f16_sat(bits)
    t = torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16).to(torch.float16).numpy()
    mag = np.abs(f)
    normal = (mag >= 2.0 ** -14) & (mag <= 65504)
    assert np.array_equal(h[normal].view(np.uint16), t[normal].view(np.uint16))       # torch's cast, exact there
    big = np.isfinite(f) & (mag > 65504)
    assert np.array_equal(h[big], np.sign(f[big]).astype(np.float16) * np.float16(65504))
    assert np.isposinf(h[bits == 0x7F80]) and np.isneginf(h[bits == 0xFF80]) and np.isnan(h[bits == 0x7FC0])
    small = (mag < 2.0 ** -14) & (mag > 0)
    err = np.abs(h[small].astype(np.float64)) - mag[small].astype(np.float64)
    assert np.all(err <= 0) and np.all(err > -(2.0 ** -24))                           # toward zero, on the 2^-24 grid


def test_bf16_forward_one_hot_selects_dequantised_column(oracle):
    """A = one-hot row: the output is the dequantised weight column rounded to bf16."""
    rng = np.random.default_rng(3)
    N, K, nbits, GS = 24, 256, 4, 64
    weight = rng.integers(0, 16, (K, N), dtype=np.int32)
    scale = (rng.random((K // GS, N)) * 0.019 + 0.001).astype(np.float16)
    zero = rng.integers(0, 16, (K // GS, N), dtype=np.int32)
    w, s, z = oracle.pack_weight(weight, nbits), oracle.transpose_scale(scale), oracle.pack_zero(zero, nbits)
    dq = oracle.dequant(w, s, z, K, nbits, GS)
    A = np.zeros((3, K), dtype=np.uint16)
    for m, k in enumerate((0, 77, 255)):
        A[m, k] = 0x3F80                                                              # 1.0
    out = oracle.qlinear_bf16_np(A, w, s, z, nbits, GS)
    for m, k in enumerate((0, 77, 255)):
        assert np.array_equal(out[m], oracle.f32_to_bf16_bits(dq[:, k].astype(np.float32)))
