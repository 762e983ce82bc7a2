"""TEST INFRASTRUCTURE ONLY: loader for the C oracle (qf_oracle.c) plus a torch-CPU port of the
reference's dequantise-then-matmul test path.

Nothing in the shipped package may import this module.  Callers: tests/, the smoke check, and the
cpu_baseline leg of bench.py -- always as the checker or the reported CPU baseline, never as the
thing being measured or shipped.

Reference lines restated (relative to the reference root):
  * packers            qfactory/convert.py:49-81
  * decode order       qfactory/include/utils.h:11-81, qfactory/include/gptq_gemv.h:65-82
  * test oracle        tests/acc_gptq.py:31-38,52 ; tests/acc_gemv.py:12-14
The C file's header lists which function follows which lines and what pins it.
NBITS == 3 has no counterpart in the reference: PARITY UNPINNED for that width.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SRC = os.path.join(_HERE, "qf_oracle.c")
_BUILD = os.path.join(_HERE, "_build")
_SO = os.path.join(_BUILD, "libqf_oracle.so")

_lib = None


def build(force: bool = False) -> str:
    """Compile qf_oracle.c with gcc into oracle/_build/libqf_oracle.so."""
    os.makedirs(_BUILD, exist_ok=True)
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(_SRC):
        tmp = f"{_SO}.{os.getpid()}.tmp"
        subprocess.check_call(["gcc", "-O2", "-std=c11", "-shared", "-fPIC", "-ffp-contract=off",
                               "-o", tmp, _SRC, "-lm"])
        os.replace(tmp, _SO)
    return _SO


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
        _lib.qfo_f32_to_f16.restype = ctypes.c_uint16
        _lib.qfo_f32_to_f16.argtypes = [ctypes.c_float]
        _lib.qfo_f16_to_f32.restype = ctypes.c_float
        _lib.qfo_f16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.qfo_row_bytes.restype = ctypes.c_int64
        _lib.qfo_zero_row_bytes.restype = ctypes.c_int64
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _i64(x):
    return ctypes.c_int64(int(x))


def zero_field_bits(nbits):
    return 4 if nbits == 3 else nbits


def pack_weight(weight, nbits):
    """(K,N) int32 -> (N, K*b/8) int8."""
    weight = np.ascontiguousarray(weight, dtype=np.int32)
    K, N = weight.shape
    out = np.empty((N, K * nbits // 8), dtype=np.int8)
    rc = lib().qfo_pack_weight(_i64(K), _i64(N), nbits, _p(weight), _p(out))
    if rc:
        raise ValueError(f"qfo_pack_weight rc={rc}")
    return out


def pack_zero(zero, nbits):
    """(G,N) int32 -> (N, G*fb/8) int8 holding min(z+1, 2^b-1)."""
    zero = np.ascontiguousarray(zero, dtype=np.int32)
    G, N = zero.shape
    out = np.empty((N, G * zero_field_bits(nbits) // 8), dtype=np.int8)
    rc = lib().qfo_pack_zero(_i64(G), _i64(N), nbits, _p(zero), _p(out))
    if rc:
        raise ValueError(f"qfo_pack_zero rc={rc}")
    return out


def transpose_scale(scale):
    scale = np.ascontiguousarray(scale, dtype=np.float16)
    G, N = scale.shape
    out = np.empty((N, G), dtype=np.float16)
    lib().qfo_transpose_scale(_i64(G), _i64(N), _p(scale), _p(out))
    return out


def unpack_weight(w, K, nbits):
    """(N, K*b/8) int8 -> (N,K) int32 in natural k order."""
    w = np.ascontiguousarray(w, dtype=np.int8)
    N = w.shape[0]
    assert w.shape[1] == K * nbits // 8
    q = np.zeros((N, K), dtype=np.int32)
    rc = lib().qfo_unpack_weight(_i64(K), _i64(N), nbits, _p(w), _p(q))
    if rc:
        raise ValueError(f"qfo_unpack_weight rc={rc}")
    return q


def unpack_zero(z, N, G, nbits):
    """(N, G*fb/8) int8 or None (symmetric) -> (N,G) int32."""
    if z is not None:
        z = np.ascontiguousarray(z, dtype=np.int8)
        assert z.shape == (N, G * zero_field_bits(nbits) // 8)
    Z = np.empty((N, G), dtype=np.int32)
    lib().qfo_unpack_zero(_i64(G), _i64(N), nbits, _p(z), _p(Z))
    return Z


def dequant(w, s, z, K, nbits, GS):
    """-> (N,K) fp16 = fp16_rn((q - Z) * s)."""
    w = np.ascontiguousarray(w, dtype=np.int8)
    s = np.ascontiguousarray(s, dtype=np.float16)
    N = w.shape[0]
    if z is not None:
        z = np.ascontiguousarray(z, dtype=np.int8)
    dq = np.empty((N, K), dtype=np.float16)
    rc = lib().qfo_dequant(_i64(K), _i64(N), nbits, _i64(GS), _p(w), _p(s), _p(z), _p(dq))
    if rc:
        raise ValueError(f"qfo_dequant rc={rc}")
    return dq


def qlinear(A, w, s, z, nbits, GS):
    """A (M,K) fp16; packed w/s/z -> (M,N) fp16, double accumulation, one final rounding."""
    A = np.ascontiguousarray(A, dtype=np.float16)
    w = np.ascontiguousarray(w, dtype=np.int8)
    s = np.ascontiguousarray(s, dtype=np.float16)
    if z is not None:
        z = np.ascontiguousarray(z, dtype=np.int8)
    M, K = A.shape
    N = w.shape[0]
    out = np.empty((M, N), dtype=np.float16)
    rc = lib().qfo_qlinear(_i64(M), _i64(N), _i64(K), nbits, _i64(GS), _p(A), _p(w), _p(s), _p(z), _p(out))
    if rc:
        raise ValueError(f"qfo_qlinear rc={rc}")
    return out


def gemv_plain(A, w, nbits):
    """GS = -1 path: A (M,K) fp16, packed w -> (M,N) fp16 = A @ q^T with raw unsigned q."""
    A = np.ascontiguousarray(A, dtype=np.float16)
    w = np.ascontiguousarray(w, dtype=np.int8)
    M, K = A.shape
    N = w.shape[0]
    out = np.empty((M, N), dtype=np.float16)
    rc = lib().qfo_gemv_plain(_i64(M), _i64(N), _i64(K), nbits, _p(A), _p(w), _p(out))
    if rc:
        raise ValueError(f"qfo_gemv_plain rc={rc}")
    return out


# ----------------------------------------------------------------------------------------------
# numpy forward for sizes where the scalar C loops take too long: same dequant (from the C
# oracle, or vectorised below), matmul in float64 via BLAS, one rounding to fp16.
# ----------------------------------------------------------------------------------------------

def dequant_np(w, s, z, K, nbits, GS):
    """Vectorised dequant: fp16_rn((q - Z) * s); the product is exact in fp32 (<= 9 + 11 bits)."""
    N = w.shape[0]
    q = unpack_weight(w, K, nbits)
    Z = unpack_zero(z, N, K // GS, nbits)
    prod = (q - np.repeat(Z, GS, axis=1)).astype(np.float32) * np.repeat(
        np.asarray(s, dtype=np.float16).astype(np.float32), GS, axis=1)
    return prod.astype(np.float16)


def qlinear_np(A, w, s, z, nbits, GS):
    K = A.shape[1]
    dq = dequant_np(w, s, z, K, nbits, GS)
    return (np.asarray(A, dtype=np.float16).astype(np.float64) @ dq.astype(np.float64).T).astype(np.float16)


def gemv_plain_np(A, w, nbits):
    K = A.shape[1]
    q = unpack_weight(w, K, nbits)
    with np.errstate(over="ignore"):     # sums past the fp16 range round to infinity, as the fp16 output of the kernel does
        return (np.asarray(A, dtype=np.float16).astype(np.float64) @ q.astype(np.float64).T).astype(np.float16)


# ----------------------------------------------------------------------------------------------
# bf16 activations and output.  The reference has no such path (it asserts fp16, qfactory/core/
# matmul.py:36 and :133-136): this restates the project's own definition -- the activation converted
# to fp16 (exact wherever fp16 is normal, saturating at +-65504, truncated toward zero on fp16's
# subnormal grid below 2^-14), the fp16 dequantised weight of dequant_np, the sum carried exactly, one
# rounding to bf16 (nearest even).  bf16 tensors travel as uint16 bit patterns.  The two conversions are
# pinned against torch's CPU casts in tests/test_oracle.py; the forward itself is PARITY UNPINNED by the
# reference.
# ----------------------------------------------------------------------------------------------

def bf16_bits_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(x):
    """Round to nearest even; NaN becomes the quiet NaN 0x7FC0."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    rounded = ((u + (0x7FFF + ((u >> 16) & 1))) >> 16).astype(np.uint16)
    return np.where(np.isnan(x), np.uint16(0x7FC0), rounded)


def bf16_bits_to_f16_sat(bits):
    """bf16 -> fp16 rounding toward zero: finite magnitudes above 65504 become +-65504."""
    with np.errstate(invalid="ignore"):
        x = bf16_bits_to_f32(bits).astype(np.float64)
    mag = np.abs(x)
    with np.errstate(invalid="ignore", over="ignore"):
        # truncate to the fp16 grid: spacing 2^(e-10) for normal values, 2^-24 below 2^-14
        e = np.floor(np.log2(np.where((mag > 0) & np.isfinite(mag), mag, 1.0)))
        ulp = np.exp2(np.maximum(e, -14.0) - 10.0)
        trunc = np.floor(mag / ulp) * ulp
    trunc = np.where(np.isfinite(mag), np.minimum(trunc, 65504.0), mag)
    return np.copysign(trunc, x).astype(np.float16)


def qlinear_bf16_np(A_bits, w, s, z, nbits, GS, rounded=True):
    """A (M,K) bf16 bit patterns, packed w/s/z -> (M,N) bf16 bit patterns (or the float64 sums before the
    final rounding)."""
    K = A_bits.shape[1]
    dq = dequant_np(w, s, z, K, nbits, GS)
    acc = bf16_bits_to_f16_sat(A_bits).astype(np.float64) @ dq.astype(np.float64).T
    if not rounded:
        return acc
    with np.errstate(over="ignore"):
        return f32_to_bf16_bits(acc.astype(np.float32))


def gemv_plain_bf16_np(A_bits, w, nbits, rounded=True):
    K = A_bits.shape[1]
    q = unpack_weight(w, K, nbits)
    acc = bf16_bits_to_f16_sat(A_bits).astype(np.float64) @ q.astype(np.float64).T
    if not rounded:
        return acc
    with np.errstate(over="ignore"):
        return f32_to_bf16_bits(acc.astype(np.float32))


# ----------------------------------------------------------------------------------------------
# Error metrics of the acceptance bar (max relative error 1e-2, normalised RMS error 1e-3).
# The relative error of an element is taken against max(|ref|, rms(ref)) so that outputs that
# happen to fall near zero do not dominate; the reference itself only defines MSE < 0.1
# (tests/acc_gptq.py:61-62).
# ----------------------------------------------------------------------------------------------

def error_metrics(out, ref):
    out = np.asarray(out, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    rms = float(np.sqrt(np.mean(ref ** 2)))
    denom = np.maximum(np.abs(ref), rms) if rms > 0 else np.ones_like(ref)
    diff = np.abs(out - ref)
    nrms = float(np.sqrt(np.mean(diff ** 2)) / rms) if rms > 0 else float(np.sqrt(np.mean(diff ** 2)))
    return {"max_rel": float(np.max(diff / denom)), "nrms": nrms, "mse": float(np.mean(diff ** 2))}


# ----------------------------------------------------------------------------------------------
# torch-CPU port of the reference's test path, used as the reported CPU baseline: unpack the
# packed tensors, dequantise to fp16, matmul with fp32 accumulation on all host threads.
# ----------------------------------------------------------------------------------------------

def torch_cpu_dequant(w, s, z, nbits, GS):
    """Packed CPU tensors -> (N,K) fp16 tensor fp16((q - Z) * s) (tests/acc_gptq.py:31-38 over the packed layout)."""
    import torch
    N = w.shape[0]
    K = w.shape[1] * 8 // nbits
    assert nbits in (2, 4, 8)
    p32 = 32 // nbits
    words = w.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF      # (N, K/p32)
    mask = (1 << nbits) - 1
    half = p32 // 2
    lo = torch.stack([(words >> (nbits * p)) & mask for p in range(half)], dim=-1)
    hi = torch.stack([(words >> (nbits * p + 16)) & mask for p in range(half)], dim=-1)
    if nbits == 8:   # bytes are already in natural order
        q = (w.contiguous().view(torch.uint8)).to(torch.int32)
    else:
        q = torch.stack([lo, hi], dim=-1).reshape(N, K).to(torch.int32)
    G = K // GS
    if z is None:
        Z = torch.full((N, G), 1 << (nbits - 1), dtype=torch.int32)
    else:
        p8 = 8 // nbits
        zb = z.contiguous().view(torch.uint8).to(torch.int32)
        Z = torch.stack([(zb >> (nbits * i)) & mask for i in range(p8)], dim=-1).reshape(N, G)
    return ((q - Z.repeat_interleave(GS, dim=1)).to(torch.float32)
            * s.to(torch.float32).repeat_interleave(GS, dim=1)).to(torch.float16)


def torch_cpu_forward(A, w, s, z, nbits, GS):
    """A (M,K) fp16 CPU tensor; w/s/z packed CPU tensors -> (M,N) fp16 tensor (tests/acc_gptq.py:52 with fp32
    accumulation)."""
    import torch
    assert A.shape[1] == w.shape[1] * 8 // nbits
    dq = torch_cpu_dequant(w, s, z, nbits, GS)
    return (A.to(torch.float32) @ dq.to(torch.float32).T).to(torch.float16)
