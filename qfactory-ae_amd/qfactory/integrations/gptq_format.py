"""AutoGPTQ checkpoint tensors -> the integer tensors ``convert_params`` takes.

The step before the hot path: a GPTQ checkpoint stores, per linear layer,

* ``qweight (K / pf, N) int32`` -- pf = 32 / bits consecutive K elements per word, element j of a
  word in bits [j*bits, (j+1)*bits);
* ``qzeros (G, N / pf) int32``  -- pf consecutive N elements per word, same bit order; the stored
  value is the zero-point minus one (the "+1" the packed layout of this library re-applies,
  reference: qfactory/convert.py:76);
* ``scales (G, N) fp16`` and ``g_idx (K,) int32`` with the group of every input channel.

The reference's vLLM hook registers these tensors (third_party/vllm-qfactory.patch:123-186) but never
converts them (its ``process_weights_after_loading`` builds an empty layer, :188-203); this module is
that missing conversion.  Supported: bits in {2, 4, 8}; ``g_idx`` must be the trivial k // group_size
(activation reordering would need a permuted activation and is rejected).
"""
import torch


def _unpack_rows(packed, bits):
    """(R, C) int32 with 32/bits fields per word along dim 0 -> (R * 32/bits, C) int32."""
    pf = 32 // bits
    shifts = (torch.arange(pf, device=packed.device, dtype=torch.int32) * bits).view(1, pf, 1)
    fields = (packed.unsqueeze(1) >> shifts) & ((1 << bits) - 1)
    return fields.reshape(packed.shape[0] * pf, packed.shape[1]).contiguous()


def unpack_qweight(qweight, bits):
    """(K / pf, N) int32 -> (K, N) int32 in [0, 2^bits)."""
    assert bits in (2, 4, 8), "GPTQ word packing is implemented for 2, 4 and 8 bits"
    assert qweight.dtype == torch.int32 and qweight.dim() == 2
    return _unpack_rows(qweight, bits)


def unpack_qzeros(qzeros, bits):
    """(G, N / pf) int32 -> (G, N) int32 stored zero-points (checkpoint convention: zero - 1)."""
    assert bits in (2, 4, 8) and qzeros.dtype == torch.int32 and qzeros.dim() == 2
    return _unpack_rows(qzeros.T.contiguous(), bits).T.contiguous()


def pack_qweight(weight, bits):
    """Inverse of unpack_qweight (for writing test checkpoints)."""
    pf = 32 // bits
    K, N = weight.shape
    shifts = (torch.arange(pf, device=weight.device, dtype=torch.int64) * bits).view(1, pf, 1)
    words = (weight.to(torch.int64).reshape(K // pf, pf, N) << shifts).sum(dim=1)
    return torch.where(words >= 2 ** 31, words - 2 ** 32, words).to(torch.int32)


def pack_qzeros(zeros, bits):
    return pack_qweight(zeros.T.contiguous(), bits).T.contiguous()


def check_trivial_g_idx(g_idx, group_size):
    if g_idx is None or g_idx.numel() == 0:
        return
    expect = torch.arange(g_idx.numel(), device=g_idx.device, dtype=g_idx.dtype) // group_size
    if not torch.equal(g_idx, expect):
        raise NotImplementedError("GPTQ activation reordering (non-trivial g_idx) is not supported")


def gptq_to_qlinear_inputs(qweight, qzeros, scales, bits, group_size, g_idx=None):
    """Checkpoint tensors -> ``(weight (K,N) int32, scale (G,N) fp16, zero (G,N) int32)`` as
    ``QLinear.init`` / ``convert_params`` expect them (zero in the checkpoint's minus-one convention,
    which is exactly what ``convert_params`` re-increments)."""
    check_trivial_g_idx(g_idx, group_size)
    weight = unpack_qweight(qweight, bits)
    zero = unpack_qzeros(qzeros, bits)
    K, N = weight.shape
    assert scales.shape == (K // group_size, N) and zero.shape == scales.shape
    return weight, scales.to(torch.float16).contiguous(), zero
