"""Weight / scale / zero repacking for the quantized linear layer.

Drop-in for the reference's ``qfactory/convert.py`` (``convert_params`` at convert.py:84-97): the
same entry point, argument dictionaries, validation and -- bit for bit -- the same packed tensors
for 2/4/8-bit weights.  The reference builds the layout with Python loops over K (convert.py:58-66,
77-79); here every step is a whole-tensor integer operation (CPU tensors) or one HIP kernel of
libqfactory_hip.so (device tensors), so the routine stays usable on 70B-sized layers.

Layout produced (reference file:line in brackets):

* weight ``(K, N) int32`` in ``[0, 2^b)`` -> ``(N, K*b/8) int8``.  Per output row the K fields are
  stored K-contiguously as little-endian 32-bit words; position ``j`` of a word holds element
  ``PERMUTE_ORDER[b][j]`` of its ``32/b`` elements, i.e. even-indexed elements fill bits 0..15 and
  odd-indexed ones bits 16..31 [convert.py:49-68].
* scale ``(K/GS, N) fp16`` -> ``(N, K/GS) fp16`` [convert.py:70-72].
* zero ``(K/GS, N) int32`` in ``[0, 2^b)`` -> ``(N, K/GS*b/8) int8`` holding ``min(zero + 1, 2^b - 1)``
  packed along the group axis, group ``g`` in field ``g % (8/b)`` of byte ``g // (8/b)``
  [convert.py:74-81].

Extension with no counterpart in the reference: ``NBITS == 3``.  A row is a 2-bit plane (the low two
bits of every element, in exactly the 2-bit layout above, K/4 bytes) followed by a 1-bit plane (the
high bits, K/8 bytes): 3*K/8 bytes per row, both planes loadable with aligned vector loads.  One
32-bit word of the 1-bit plane serves the two 2-bit words of the same 32 elements; its bit order
(``_hi_plane_order``) puts every high bit where one shift of the whole word drops it directly above
the element's 2-bit field, so the kernels merge the planes with one AND-OR per element pair.
3-bit zero-points are stored one per nibble.
"""
import torch


def _check_weight(K, N, weight, nbits):
    assert weight.shape == (K, N)
    assert weight.dtype == torch.int32
    assert weight.min() >= 0
    assert weight.max() < 2 ** nbits


def _check_scale(K, N, GS, scale):
    assert scale.shape == (K // GS, N)
    assert scale.dtype == torch.float16


def _check_zero(K, N, GS, zero, nbits):
    assert zero.shape == (K // GS, N)
    assert zero.dtype == torch.int32
    assert zero.min() >= 0
    assert zero.max() < 2 ** nbits


def _check_gptq_gemv(args, params):
    if len(params) != 3:
        raise ValueError("gptq_gemv requires 3 parameters")
    weight, scale, zero = params
    K, N, NBITS, GS = args["K"], args["N"], args["NBITS"], args["GS"]
    _check_weight(K, N, weight, NBITS)
    _check_scale(K, N, GS, scale)
    if zero is not None:
        _check_zero(K, N, GS, zero, NBITS)
    return K, N, NBITS, GS, weight, scale, zero


def _check_gemv(args, params):
    if len(params) != 1:
        raise ValueError("gemv requires 1 parameters")
    weight = params[0]
    K, N, NBITS = args["K"], args["N"], args["NBITS"]
    _check_weight(K, N, weight, NBITS)
    return K, N, NBITS, weight


def _evens_then_odds(n):
    return list(range(0, n, 2)) + list(range(1, n, 2))


def _hi_plane_order():
    """Element held by each bit of a 1-bit-plane word.  Element e = 16*r + 2*i + h (r: which 2-bit
    word, i: pair, h: even/odd element = low/high half-word), with p = i % 4 the pair inside its byte
    and upper = i // 4 the byte, sits at bit (2p+2 if p even else 2p-2) + 8*upper + r + 16*h."""
    pos = []
    for e in range(32):
        r, ep = divmod(e, 16)
        i, h = divmod(ep, 2)
        p, upper = i % 4, i // 4
        pos.append((2 * p + 2 if p % 2 == 0 else 2 * p - 2) + 8 * upper + r + 16 * h)
    return [pos.index(j) for j in range(32)]


# Position j of a packed 32-bit word holds element PERMUTE_ORDER[b][j] (convert.py:49-53).  The
# 1-bit entry is only used for the high-bit plane of the 3-bit layout.
PERMUTE_ORDER = {
    8: [0, 1, 2, 3],
    4: _evens_then_odds(8),
    2: _evens_then_odds(16),
    1: _hi_plane_order(),
}


def weight_row_bytes(K, nbits):
    """Bytes of one packed weight row."""
    return K * nbits // 8


def zero_field_bits(nbits):
    """Storage width of one packed zero-point (3-bit values occupy a nibble)."""
    return 4 if nbits == 3 else nbits


def zero_row_bytes(G, nbits):
    return G * zero_field_bits(nbits) // 8


def _pack_fields(fields_nk, nbits):
    """(N, K) int fields of width nbits -> (N, K*nbits/8) int8 in the word layout above."""
    N, K = fields_nk.shape
    p32 = 32 // nbits
    assert K % p32 == 0, f"K ({K}) must be a multiple of {p32} for {nbits}-bit fields"
    order = torch.tensor(PERMUTE_ORDER[nbits], device=fields_nk.device)
    shifts = torch.arange(p32, device=fields_nk.device, dtype=torch.int64) * nbits
    grouped = fields_nk.reshape(N, K // p32, p32).index_select(2, order).to(torch.int64)
    words = (grouped << shifts).sum(dim=2)                 # fields do not overlap: sum == bitwise or
    words = torch.where(words >= 2 ** 31, words - 2 ** 32, words).to(torch.int32)
    return words.contiguous().view(torch.int8)             # little-endian bytes of every word


def _on_device(t):
    """Device tensors whose K fills whole 32-element words take the HIP packers of
    libqfactory_hip.so (one pass over the tensor); everything else the whole-tensor torch ops below,
    on whatever device the tensor lives.  Both produce identical bytes."""
    return t.is_cuda


def _transform_weight_basic(K, N, weight, nbits):
    if _on_device(weight) and K % 32 == 0:
        from . import native
        return native.pack_weight(weight.contiguous(), nbits)
    wt = weight.T
    if nbits == 3:
        lo = _pack_fields(wt & 3, 2)
        hi = _pack_fields((wt >> 2) & 1, 1)
        return torch.cat([lo, hi], dim=1).contiguous()
    return _pack_fields(wt, nbits)


def _transform_scale(K, N, GS, scale):
    if _on_device(scale):
        from . import native
        return native.transpose_scale(scale.contiguous())
    return scale.T.contiguous()


def _transform_zero(K, N, GS, zero, nbits):
    fb = zero_field_bits(nbits)
    pack_factor = 8 // fb
    G = zero.shape[0]
    assert G % pack_factor == 0, f"K/GS ({G}) must fill whole bytes of {pack_factor} zero-points"
    if _on_device(zero):
        from . import native
        return native.pack_zero(zero.contiguous(), nbits)
    zp = (zero + 1).clamp(max=(2 ** nbits - 1)).T.to(torch.int64)           # (N, G)
    shifts = torch.arange(pack_factor, device=zero.device, dtype=torch.int64) * fb
    packed = (zp.reshape(zp.shape[0], G // pack_factor, pack_factor) << shifts).sum(dim=2)
    return packed.to(torch.uint8).view(torch.int8).contiguous()


def convert_params(args, params):
    """Repack GPTQ-style tensors.  ``args``: ``{K, N, NBITS[, GS]}``.

    Without ``GS``: ``params = (weight,)`` -> ``w``.  With ``GS``: ``params = (weight, scale, zero)``
    -> ``(w, s, z)``, ``z`` is ``None`` when ``zero`` is ``None`` (symmetric).  Outputs live on the
    device of the inputs.
    """
    if "GS" not in args:
        K, N, NBITS, weight = _check_gemv(args, params)
        return _transform_weight_basic(K, N, weight, NBITS)
    K, N, NBITS, GS, weight, scale, zero = _check_gptq_gemv(args, params)
    w = _transform_weight_basic(K, N, weight, NBITS)
    s = _transform_scale(K, N, GS, scale)
    z = _transform_zero(K, N, GS, zero, NBITS) if zero is not None else None
    return w, s, z


# --------------------------------------------------------------------------------------------
# Inverse transforms (not in the reference): used by tooling that needs the integer fields back,
# e.g. re-tiling for a different kernel family or checkpoint inspection.
# --------------------------------------------------------------------------------------------

def _unpack_fields(packed, K, nbits):
    N = packed.shape[0]
    p32 = 32 // nbits
    words = packed.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    shifts = torch.arange(p32, device=packed.device, dtype=torch.int64) * nbits
    fields = (words.unsqueeze(-1) >> shifts) & ((1 << nbits) - 1)            # (N, K/p32, p32) in stored order
    order = torch.tensor(PERMUTE_ORDER[nbits], device=packed.device)
    out = torch.empty_like(fields)
    out.index_copy_(2, order, fields)
    return out.reshape(N, K).to(torch.int32)


def unpack_weight(w, K, nbits):
    """(N, K*b/8) int8 -> (N, K) int32 fields in natural k order."""
    if nbits == 3:
        lo = _unpack_fields(w[:, : K // 4], K, 2)
        hi = _unpack_fields(w[:, K // 4:], K, 1)
        return lo | (hi << 2)
    return _unpack_fields(w, K, nbits)


def unpack_zero(z, G, nbits):
    """(N, G*fb/8) int8 -> (N, G) int32 stored zero-points (i.e. already ``min(zero+1, 2^b-1)``)."""
    fb = zero_field_bits(nbits)
    p8 = 8 // fb
    zb = z.contiguous().view(torch.uint8).to(torch.int32)
    shifts = torch.arange(p8, device=z.device, dtype=torch.int32) * fb
    return ((zb.unsqueeze(-1) >> shifts) & ((1 << fb) - 1)).reshape(z.shape[0], G)
