"""Latency harness: a quantized linear against the dense fp16 GEMM of the same shape.

Counterpart of the reference's ``qfactory/testing.py:24-41`` (``LatencyTest``,
``QFactoryLatencyTest``, ``CuBLASLatencyTest``); its BitBLAS and Marlin comparisons are CUDA-only
baselines with no MI355X build and have no counterpart here.  The dense baseline is
``torch.matmul`` in fp16, which PyTorch-ROCm serves with hipBLASLt / rocBLAS; the reference's class
name is kept as an alias so that its benchmark scripts read the same.
"""
import torch

from .profile import benchmark
from .qlinear import QLinear


class LatencyTest:
    def __init__(self, func):
        self.func = func

    def latency(self):
        """Seconds per call, device-side, cold caches."""
        return benchmark(self.func)


class QFactoryLatencyTest(LatencyTest):
    def __init__(self, M, N, K, NBITS, GS, sym, compile_flags={}, base_impl=False):
        activation = torch.empty(M, K, dtype=torch.float16, device='cuda')
        qlinear = QLinear.empty(M, K, N, NBITS, GS, sym, compile_flags=compile_flags, base_impl=base_impl)
        self.qlinear = qlinear
        super().__init__(func=lambda: qlinear(activation))


class DenseLatencyTest(LatencyTest):
    def __init__(self, M, N, K):
        activation = torch.randn(M, K, dtype=torch.float16, device='cuda')
        weight = torch.randn(K, N, dtype=torch.float16, device='cuda')
        super().__init__(lambda: torch.matmul(activation, weight))


CuBLASLatencyTest = DenseLatencyTest


def speedup_over_dense(M, N, K, NBITS=4, GS=128, sym=False, compile_flags={}):
    """(quantized seconds, dense seconds, dense / quantized) for one shape."""
    tq = QFactoryLatencyTest(M, N, K, NBITS, GS, sym, compile_flags=compile_flags).latency()
    td = DenseLatencyTest(M, N, K).latency()
    return tq, td, td / tq
