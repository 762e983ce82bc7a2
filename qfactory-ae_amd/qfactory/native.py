"""ctypes binding of libqfactory_hip.so, the ahead-of-time HIP library (device-side repacking, the
stream read / copy calibration kernels and the per-token steps between the linears of a decoder layer).  Its C ABI is declared in include/qfactory_hip.h.

The library is built in-tree with hipcc (``build()``; no GPU needed) and loaded lazily.  There is
no substitute path: calling an entry point without the built library raises.
"""
import ctypes
import os
import subprocess
import threading

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
# sources and C-ABI headers: copies inside the package in a built distribution (setup.py), else the checkout's
# csrc/ beside the package and include/ at the repository root
CSRC_DIR = os.path.join(PKG_DIR, "csrc") if os.path.isdir(os.path.join(PKG_DIR, "csrc")) else os.path.join(os.path.dirname(PKG_DIR), "csrc")
REPO_INCLUDE = (os.path.join(PKG_DIR, "abi") if os.path.isdir(os.path.join(PKG_DIR, "abi"))
                else os.path.join(os.path.dirname(os.path.dirname(PKG_DIR)), "include"))
SOURCES = [os.path.join(CSRC_DIR, "qfactory_hip.hip"), os.path.join(CSRC_DIR, "qfactory_decode.hip")]
LIBRARY = os.path.join(CSRC_DIR, "libqfactory_hip.so")

HIPCC_FLAGS = ["--offload-arch=gfx950", "-std=c++20", "-shared", "-fPIC", "-O3",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]

# name -> (restype, argtypes); mirrors include/qfactory_hip.h
_P, _I64, _INT, _SZ, _F = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t, ctypes.c_float
SIGNATURES = {
    "qf_version": (_INT, []),
    "qf_pack_weight": (_INT, [_P, _P, _I64, _I64, _INT, _P]),
    "qf_pack_zero": (_INT, [_P, _P, _I64, _I64, _INT, _P]),
    "qf_transpose_scale": (_INT, [_P, _P, _I64, _I64, _P]),
    "qf_bf16_to_f16": (_INT, [_P, _P, _I64, _P]),
    "qf_stream_read": (_INT, [_P, _SZ, _P, _P]),
    "qf_stream_copy": (_INT, [_P, _P, _SZ, _P]),
    "qf_empty_launch": (_INT, [_I64, _I64, _P]),
    "qf_add_rmsnorm": (_INT, [_P, _P, _P, _P, _I64, _I64, _F, _P]),
    "qf_rope_kv_store": (_INT, [_P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _P]),
    "qf_rope_kv_store_rows": (_INT, [_P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _P]),
    "qf_decode_attention": (_INT, [_P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _P]),
    "qf_rope_decode_attention": (_INT, [_P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _P]),
    "qf_silu_mul": (_INT, [_P, _P, _I64, _I64, _P]),
    "qf_greedy_next": (_INT, [_P, _P, _P, _P, _P, _I64, _I64, _I64, _P]),
}

_lock = threading.Lock()
_lib = None


def build(force=False):
    """Compile csrc/*.hip for gfx950 into csrc/libqfactory_hip.so."""
    hipcc = os.environ.get("QFACTORY_HIPCC", "/opt/rocm/bin/hipcc")
    if not force and os.path.exists(LIBRARY) and os.path.getmtime(LIBRARY) >= max(os.path.getmtime(p) for p in SOURCES):
        return LIBRARY
    tmp = f"{LIBRARY}.tmp.{os.getpid()}"
    cmd = [hipcc, "-x", "hip", *SOURCES, "-o", tmp, *HIPCC_FLAGS, f"-I{REPO_INCLUDE}"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on {SOURCES}:\n{proc.stderr}")
    os.replace(tmp, LIBRARY)
    return LIBRARY


def load():
    """The loaded library with argument types set; raises if it has not been built."""
    global _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIBRARY):
                raise RuntimeError(f"{LIBRARY} is missing: build it with qfactory.native.build() "
                                   "(hipcc, no GPU needed); there is no CPU substitute for the device packers")
            lib = ctypes.CDLL(LIBRARY)
            for name, (res, args) in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype, fn.argtypes = res, args
            _lib = lib
    return _lib


def _stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def _check(rc, what):
    if rc != 0:
        raise RuntimeError(f"{what} failed with return code {rc}")


def pack_weight(weight, nbits):
    """(K, N) int32 device tensor -> (N, K*nbits/8) int8, bit-identical to convert._transform_weight_basic."""
    import torch
    assert weight.is_cuda and weight.dtype == torch.int32 and weight.is_contiguous() and weight.dim() == 2
    K, N = weight.shape
    out = torch.empty(N, K * nbits // 8, dtype=torch.int8, device=weight.device)
    _check(load().qf_pack_weight(weight.data_ptr(), out.data_ptr(), K, N, nbits, _stream()), "qf_pack_weight")
    return out


def pack_zero(zero, nbits):
    """(G, N) int32 device tensor -> (N, G*fb/8) int8 holding min(zero + 1, 2^nbits - 1)."""
    import torch
    assert zero.is_cuda and zero.dtype == torch.int32 and zero.is_contiguous() and zero.dim() == 2
    G, N = zero.shape
    fb = 4 if nbits == 3 else nbits
    out = torch.empty(N, G * fb // 8, dtype=torch.int8, device=zero.device)
    _check(load().qf_pack_zero(zero.data_ptr(), out.data_ptr(), G, N, nbits, _stream()), "qf_pack_zero")
    return out


def transpose_scale(scale):
    """(G, N) fp16 device tensor -> (N, G) fp16 contiguous."""
    import torch
    assert scale.is_cuda and scale.dtype == torch.float16 and scale.is_contiguous() and scale.dim() == 2
    G, N = scale.shape
    out = torch.empty(N, G, dtype=torch.float16, device=scale.device)
    _check(load().qf_transpose_scale(scale.data_ptr(), out.data_ptr(), G, N, _stream()), "qf_transpose_scale")
    return out


def bf16_to_f16(src, out=None):
    """bf16 device tensor -> fp16 tensor of the same shape (saturating; see include/qfactory_hip.h)."""
    import torch
    assert src.is_cuda and src.dtype == torch.bfloat16 and src.is_contiguous()
    if out is None:
        out = torch.empty(src.shape, dtype=torch.float16, device=src.device)
    assert out.is_cuda and out.dtype == torch.float16 and out.is_contiguous() and out.numel() == src.numel()
    if src.numel():
        _check(load().qf_bf16_to_f16(src.data_ptr(), out.data_ptr(), src.numel(), _stream()), "qf_bf16_to_f16")
    return out


def stream_read(src, sink):
    assert sink.numel() * sink.element_size() >= 4096 * 4, "qf_stream_read writes one word per block, index modulo 4096: the sink holds 4096 words"
    _check(load().qf_stream_read(src.data_ptr(), src.numel() * src.element_size(), sink.data_ptr(), _stream()), "qf_stream_read")


def empty_launch(blocks, threads):
    """A kernel that does nothing: what a launch of that grid costs."""
    _check(load().qf_empty_launch(blocks, threads, _stream()), "qf_empty_launch")


def stream_copy(dst, src):
    assert dst.numel() * dst.element_size() == src.numel() * src.element_size()
    _check(load().qf_stream_copy(dst.data_ptr(), src.data_ptr(), src.numel() * src.element_size(), _stream()), "qf_stream_copy")


def _f16(t):
    import torch
    assert t.is_cuda and t.dtype == torch.float16 and t.is_contiguous()
    return t.data_ptr()


ADD_RMSNORM_MAX_HIDDEN = 16384          # qf_add_rmsnorm holds a row in one block's registers


def add_rmsnorm(x, delta, weight, out, eps):
    """x (rows, hidden) fp16 += delta (or None) in place; out = RMSNorm(x) * weight."""
    rows, hidden = x.shape
    assert hidden <= ADD_RMSNORM_MAX_HIDDEN, f"qf_add_rmsnorm takes rows of up to {ADD_RMSNORM_MAX_HIDDEN} elements"
    assert out.shape == x.shape and weight.shape == (hidden,) and (delta is None or delta.shape == x.shape)
    _check(load().qf_add_rmsnorm(_f16(x), None if delta is None else _f16(delta), _f16(weight), _f16(out), rows, hidden,
                                 float(eps), _stream()), "qf_add_rmsnorm")
    return out


def rope_kv_store(qkv, pos, cos, sin, q_out, k_cache, v_cache):
    """qkv (B, 3*H*hd) of the position pos (one-element int64 device tensor): rotated q to q_out (B, H*hd),
    rotated k and v appended to the caches (B, H, max_len, hd)."""
    import torch
    B, H, max_len, hd = k_cache.shape
    assert qkv.shape == (B, 3 * H * hd) and q_out.shape == (B, H * hd) and v_cache.shape == k_cache.shape
    assert pos.is_cuda and pos.dtype == torch.int64 and pos.numel() == 1
    assert cos.dtype == torch.float32 and cos.is_contiguous() and cos.shape == (max_len, hd // 2) and sin.shape == cos.shape
    assert sin.dtype == torch.float32 and sin.is_contiguous()
    _check(load().qf_rope_kv_store(_f16(qkv), pos.data_ptr(), cos.data_ptr(), sin.data_ptr(), _f16(q_out), _f16(k_cache),
                                   _f16(v_cache), B, H, hd, max_len, _stream()), "qf_rope_kv_store")
    return q_out


def rope_kv_store_rows(qkv, pos, cos, sin, q_out, k_cache, v_cache):
    """qkv (B * T, 3*H*hd), row b * T + t being token t of sequence b at position pos[t] (pos: T int64 device values):
    rotated q to q_out (B, T, H, hd), rotated k and v to rows pos[t] of the caches (B, H, max_len, hd)."""
    import torch
    B, H, max_len, hd = k_cache.shape
    T = pos.numel()
    assert qkv.shape == (B * T, 3 * H * hd) and q_out.shape == (B, T, H, hd) and v_cache.shape == k_cache.shape
    assert qkv.is_contiguous() and q_out.is_contiguous() and k_cache.is_contiguous() and v_cache.is_contiguous()
    assert pos.is_cuda and pos.dtype == torch.int64 and pos.is_contiguous()
    assert cos.dtype == torch.float32 and cos.is_contiguous() and cos.shape == (max_len, hd // 2) and sin.shape == cos.shape
    assert sin.dtype == torch.float32 and sin.is_contiguous()
    _check(load().qf_rope_kv_store_rows(_f16(qkv), pos.data_ptr(), cos.data_ptr(), sin.data_ptr(), _f16(q_out), _f16(k_cache),
                                        _f16(v_cache), B, T, H, hd, max_len, _stream()), "qf_rope_kv_store_rows")
    return q_out


def decode_attention(q, k_cache, v_cache, pos, out):
    """q (B, H*hd), caches (B, H, max_len, hd), pos one-element int64 device tensor -> out (B, H*hd)."""
    import torch
    B, H, max_len, hd = k_cache.shape
    assert q.shape == (B, H * hd) and out.shape == q.shape and v_cache.shape == k_cache.shape
    assert pos.is_cuda and pos.dtype == torch.int64 and pos.numel() == 1
    _check(load().qf_decode_attention(_f16(q), _f16(k_cache), _f16(v_cache), pos.data_ptr(), _f16(out), B, H, hd, max_len,
                                      _stream()), "qf_decode_attention")
    return out


def rope_decode_attention(qkv, pos, cos, sin, k_cache, v_cache, out):
    """rope_kv_store and decode_attention in one launch: qkv (B, 3*H*hd) of position pos -> out (B, H*hd);
    rotated k and v are appended to the caches (B, H, max_len, hd)."""
    import torch
    B, H, max_len, hd = k_cache.shape
    assert qkv.shape == (B, 3 * H * hd) and out.shape == (B, H * hd) and v_cache.shape == k_cache.shape
    assert pos.is_cuda and pos.dtype == torch.int64 and pos.numel() == 1
    assert cos.dtype == torch.float32 and cos.is_contiguous() and cos.shape == (max_len, hd // 2)
    assert sin.dtype == torch.float32 and sin.is_contiguous() and sin.shape == cos.shape
    _check(load().qf_rope_decode_attention(_f16(qkv), pos.data_ptr(), cos.data_ptr(), sin.data_ptr(), _f16(k_cache),
                                           _f16(v_cache), _f16(out), B, H, hd, max_len, _stream()), "qf_rope_decode_attention")
    return out


def silu_mul(gate_up, out):
    """gate_up (rows, 2*mlp) -> out (rows, mlp) = silu(gate) * up."""
    rows, two_mlp = gate_up.shape
    assert out.shape == (rows, two_mlp // 2)
    _check(load().qf_silu_mul(_f16(gate_up), _f16(out), rows, two_mlp // 2, _stream()), "qf_silu_mul")
    return out


def greedy_next(logits, tok, pos=None, embed=None, x_next=None):
    """The end of a greedy decode step in one launch: ``tok`` (batch, 1) int64 <- argmax of ``logits`` (batch, vocab)
    fp16 (the first of equal maxima), ``pos`` (one int64) += 1, and ``x_next`` (batch, hidden) <- ``embed[tok]``, the
    residual stream of the next step."""
    import torch
    batch, vocab = logits.shape
    assert logits.dtype == torch.float16 and logits.is_contiguous() and logits.is_cuda
    assert tok.dtype == torch.int64 and tok.numel() == batch and tok.is_contiguous() and tok.device == logits.device
    assert pos is None or (pos.dtype == torch.int64 and pos.numel() == 1 and pos.device == logits.device)
    hidden = 0
    if embed is not None:
        hidden = embed.shape[1]
        assert embed.shape[0] == vocab and embed.dtype == torch.float16 and embed.is_contiguous() and embed.device == logits.device
        assert x_next is not None and x_next.shape == (batch, hidden) and x_next.dtype == torch.float16 and x_next.is_contiguous()
    else:
        assert x_next is None
    _check(load().qf_greedy_next(_f16(logits), tok.data_ptr(), None if pos is None else pos.data_ptr(),
                                 None if embed is None else _f16(embed), None if x_next is None else _f16(x_next),
                                 batch, vocab, hidden, _stream()), "qf_greedy_next")
    return tok
