"""Quantized matmul operators: build the QFunc(s), compile, optionally time the candidates, and
return the closure that ``QLinear.forward`` calls.

Interface of the reference's ``qfactory/core/matmul.py`` (QMatmul :14-153, Matmul :155-270): same
constructor arguments, same ``compile_profile(enable_transform, enable_schedule, enable_lower)``,
same ``$QFACTORY_CONFIG`` lookup keyed ``"{nbits}-{m}-{n}-{k}-{group_size}"``, and closures with the
same argument lists and checks.  Differences that matter to callers:

* the closure launches for the *actual* number of activation rows (the reference silently computes
  only the rows it was compiled for, matmul.py:128);
* supported widths are 2/3/4/8 bits; M may be anything >= 1 (large M runs on the matrix cores);
* ``dtype_a`` may be ``torch.bfloat16`` (the reference asserts fp16, matmul.py:36): activations and output
  are then bf16, scales stay fp16.  The kernels compute on fp16 pairs either way; bf16 activations are
  converted as they are loaded, or, for the GEMM kernel, by one ``qf_bf16_to_f16`` launch before it.
"""
import ctypes
import json
import logging
import os
from concurrent.futures import ThreadPoolExecutor, as_completed
from itertools import chain

import torch

from . import tiling
from .qtile import QTile, SymQTile, AsymQTile
from .qfunc import QMatmulQFunc, MatmulQFunc, apply_config
from ..convert import weight_row_bytes, zero_row_bytes
from ..jit import jit
from .. import fastpath

logger = logging.getLogger(__name__)


_get_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _raw_stream(tensor):
    """Handle of the current HIP stream of the tensor's device.  The C-level query costs a fraction of a
    microsecond; ``torch.cuda.current_stream()`` builds a Python Stream object and takes ~4 us, a third of
    the whole enqueue of a small launch."""
    if _get_raw_stream is not None:
        return _get_raw_stream(tensor.device.index)
    return torch.cuda.current_stream(tensor.device).cuda_stream


def require_gpu():
    if not torch.cuda.is_available():
        raise RuntimeError("qfactory kernels need a HIP device (torch.cuda.is_available() is False); "
                           "there is no CPU fallback")


def _load_predefined(shape_key):
    path = os.getenv("QFACTORY_CONFIG")
    if path is None or not os.path.exists(path):
        return None
    with open(path) as f:
        config = json.load(f)
    return config.get(shape_key)


def _compile_all(qfuncs):
    runtimes = [None] * len(qfuncs)
    workers = min(len(qfuncs), int(os.environ.get("QFACTORY_JIT_WORKERS", os.cpu_count() or 4)))
    with ThreadPoolExecutor(max_workers=max(1, workers)) as executor:
        futures = {executor.submit(jit.compile, q): i for i, q in enumerate(qfuncs)}
        for future in as_completed(futures):
            runtimes[futures[future]] = future.result()
    return runtimes


def _pick_best(runtimes, qfuncs, dummy_inputs, what):
    """Time every candidate that accepts its configuration; keep the fastest."""
    if len(runtimes) == 1:
        return runtimes[0], qfuncs[0]
    from ..profile import benchmark
    best = (None, None, None)
    for runtime, qfunc in zip(runtimes, qfuncs):
        if runtime.run(*dummy_inputs) != 0:
            continue
        t = benchmark(lambda: runtime.run(*dummy_inputs))
        logger.debug(f"[Profile] Kernel: {t * 1e6:.2f} us  {runtime.description}")
        if best[0] is None or t < best[2]:
            best = (runtime, qfunc, t)
    assert best[0] is not None, "No valid runtime found"
    logger.info(f"[Profile] Best latency for {what}: {best[2] * 1e6:.2f} us  ({best[0].description})")
    return best[0], best[1]


class QMatmul:
    def __init__(self, m: int, n: int, k: int, nbits: int, sym: bool, dtype_a, dtype_b,
                 group_size: int = -1, layout: str = "nt", base_impl: bool = False,
                 output_epilogue: str = "none", input_prologue: str = "none"):
        self.m, self.n, self.k = m, n, k
        # "add_rmsnorm" (beyond the reference): the closure takes the residual stream, the previous block's output and
        # the RMSNorm weight instead of ready activations -- closure(activation, delta, gamma, x_out, eps, weight,
        # output, scale, zero=None); rows of the dot2 GEMV kernel only (M < 3), fp16 only
        self.input_prologue = input_prologue
        assert input_prologue in ("none", "add_rmsnorm")
        # "silu_mul" (beyond the reference): the weight is a fused gate+up projection and the closure's output is
        # the (M, N/2) SwiGLU activation fp16(silu(gate)) * up; M <= 32 only (dot2 GEMV and A-stationary kernels), fp16 only
        self.output_epilogue = output_epilogue
        # "accumulate" (beyond the reference): the closure adds the projection to what ``output`` holds,
        # output = fp16(output + fp16(projection)); M <= 32 (dot2 GEMV, A-stationary and streaming kernels), fp16 only
        assert output_epilogue in ("none", "silu_mul", "accumulate")
        self.nbits, self.sym = nbits, sym
        self.dtype_a, self.dtype_b = dtype_a, dtype_b
        self.group_size = k if group_size == -1 else group_size
        self.layout = layout
        self.base_impl = base_impl
        assert self.k % self.group_size == 0, f"Group size {self.group_size} must divide k {self.k}"
        assert self.layout == "nt", f"Layout {layout} is not supported"
        assert dtype_a in (torch.float16, torch.bfloat16), f"Data type {dtype_a} is not supported"
        assert dtype_b == torch.int8, f"Data type {dtype_b} is not supported"
        assert nbits in (2, 3, 4, 8), f"{nbits}-bit weights are not supported"

    # packed operand shapes
    @property
    def weight_shape(self):
        return (self.n, weight_row_bytes(self.k, self.nbits))

    @property
    def scale_shape(self):
        return (self.n, self.k // self.group_size)

    @property
    def zero_shape(self):
        return (self.n, zero_row_bytes(self.k // self.group_size, self.nbits))

    def init_qfuncs(self):
        tile_b = SymQTile if self.sym else AsymQTile
        self.qfuncs = [QMatmulQFunc(
            QTile((self.m, self.k), self.dtype_a, 16),
            tile_b((self.n, self.k), self.dtype_b, self.nbits, (1, self.group_size)),
            "nt", self.base_impl, ksplit=self.input_prologue == "none" and self.output_epilogue != "silu_mul")]
        self.qfuncs[0].output_epilogue = self.output_epilogue
        self.qfuncs[0].input_prologue = self.input_prologue
        q = self.qfuncs[0]
        if self.input_prologue != "none" and q.regime == "gemv" and tiling.gemv_chunks_per_lane(self.k, self.nbits, q.tiling_configs) == 1:
            # every block normalises the row before its first dot product (loads from L2, a sum across the team, a
            # barrier): four stages per block spread that over four times the rows.  Measured at M = 1, cold
            # weights, against qf_add_rmsnorm + the plain kernel: 12288 x 4096 8.6 -> 7.4 us (one team per block),
            # 22016 x 4096 with the SwiGLU epilogue 11.9 -> 11.0 (two teams); with the plain kernel's one-stage
            # tiling the fused form is slower than the two launches (9.6 and 16.5 us)
            q.tiling_configs = tiling.gemv_tiling(self.m, self.n, self.k, self.nbits, self.group_size, u=4, steps=4,
                                                  wn=2 if self.n >= 16384 else 1)

    def get_dummy_inputs(self):
        require_gpu()
        activation = torch.zeros((self.m, self.k), dtype=dict(self.qfuncs[0].arg_name_type())["activation"], device="cuda")
        weight = torch.zeros(self.weight_shape, dtype=self.dtype_b, device="cuda")
        output = torch.empty((self.m, self.n // 2 if self.output_epilogue == "silu_mul" else self.n), dtype=self.dtype_a, device="cuda")
        scale = torch.zeros(self.scale_shape, dtype=torch.float16, device="cuda")
        zero = torch.zeros(self.zero_shape, dtype=self.dtype_b, device="cuda")
        return activation, weight, output, scale, zero, torch.cuda.current_stream()

    def compile_profile(self, enable_transform: bool = False, enable_schedule: bool = False,
                        enable_lower: bool = False):
        self.init_qfuncs()
        if self.input_prologue != "none":
            # the candidates are timed through `launch`, which these objects answer with 1: no search, the default tiling
            enable_transform = enable_schedule = enable_lower = False
        shape = f"{self.nbits}-{self.m}-{self.n}-{self.k}-{self.group_size}"
        predefined = _load_predefined(shape)
        if predefined is not None:
            logger.info(f"[Profile] Using predefined config for {shape}")
            self.qfuncs = [apply_config(self.qfuncs[0], predefined)]
        else:
            if enable_transform:
                self.qfuncs = list(chain.from_iterable(q.transform() for q in self.qfuncs))
            if enable_schedule:
                self.qfuncs = list(chain.from_iterable(q.schedule() for q in self.qfuncs))
            if enable_lower:
                self.qfuncs = list(chain.from_iterable(q.lower() for q in self.qfuncs))

        self.runtimes = _compile_all(self.qfuncs)
        dummy = self.get_dummy_inputs() if len(self.runtimes) > 1 else None
        self.best_runtime, self.best_qfunc = _pick_best(self.runtimes, self.qfuncs, dummy, shape)
        return self._wrap(self.best_runtime, self.best_qfunc)

    def _wrap(self, runtime, qfunc=None):
        n, k = self.n, self.k
        w_shape, s_shape, z_shape = self.weight_shape, self.scale_shape, self.zero_shape
        dtype_a = self.dtype_a
        n_out = n // 2 if self.output_epilogue == "silu_mul" else n         # columns of the output
        # bf16 rows into a kernel that reads fp16 only (the GEMM kernel): one conversion launch first
        convert_first = dtype_a == torch.bfloat16 and not (qfunc is not None and qfunc.converts_activations)
        if convert_first:
            from .. import native
        zero_empty = None
        if self.sym:
            require_gpu()
            zero_empty = torch.empty(z_shape, dtype=torch.int8, device="cuda")

        def check_packed(weight, scale, zero):
            assert weight.shape == w_shape
            assert scale.shape == s_shape
            assert zero.shape == z_shape
            assert weight.dtype == torch.int8
            assert scale.dtype == torch.float16
            assert zero.dtype == torch.int8
            assert weight.is_contiguous()
            assert scale.is_contiguous()
            assert zero.is_contiguous()
            assert weight.is_cuda and scale.is_cuda and zero.is_cuda

        def inner(activation, weight, output, scale, zero):
            # tensor shape / dtype / contiguity checks (reference: matmul.py:124-144)
            assert activation.shape[1] == k
            assert output.shape[1] == n_out
            assert activation.shape[0] == output.shape[0]
            assert activation.dtype == dtype_a
            assert output.dtype == dtype_a
            assert activation.is_contiguous()
            assert output.is_contiguous()
            assert activation.is_cuda and output.is_cuda
            check_packed(weight, scale, zero)
            if convert_first:
                activation = native.bf16_to_f16(activation)
            return runtime.run_raw(
                activation.shape[0],
                (activation.data_ptr(), weight.data_ptr(), output.data_ptr(), scale.data_ptr(), zero.data_ptr()),
                _raw_stream(activation))

        def inner_sym(activation, weight, output, scale):
            return inner(activation, weight, output, scale, zero_empty)

        def inner_norm(activation, delta, gamma, x_out, eps, weight, output, scale, zero=None):
            """Objects with the residual-add + RMSNorm prologue: ``activation`` is the residual stream, ``delta`` what
            is added to it first (or None), ``x_out`` receives the sum (or None)."""
            if zero is None:
                zero = zero_empty
            assert activation.shape[1] == k and output.shape[1] == n_out and activation.shape[0] == output.shape[0]
            assert activation.dtype == torch.float16 and output.dtype == torch.float16
            assert activation.is_contiguous() and output.is_contiguous() and activation.is_cuda and output.is_cuda
            assert gamma.shape == (k,) and gamma.dtype == torch.float16 and gamma.is_contiguous() and gamma.is_cuda
            for other in (delta, x_out):
                if other is not None:
                    assert other.shape == activation.shape and other.dtype == torch.float16
                    assert other.is_contiguous() and other.is_cuda
            if x_out is not None:
                assert x_out.data_ptr() != activation.data_ptr(), "x_out must not alias the residual stream it is computed from"
                assert delta is None or x_out.data_ptr() != delta.data_ptr(), "x_out must not alias delta"
            check_packed(weight, scale, zero)
            rc = ctypes.c_int(0)
            runtime._launch_norm(activation.shape[0], activation.data_ptr(), delta.data_ptr() if delta is not None else None,
                                 gamma.data_ptr(), x_out.data_ptr() if x_out is not None else None, float(eps),
                                 weight.data_ptr(), output.data_ptr(), scale.data_ptr(), zero.data_ptr(),
                                 _raw_stream(activation), ctypes.byref(rc))
            return rc.value

        if self.input_prologue == "add_rmsnorm":
            assert runtime._launch_norm is not None, "the compiled object does not export launch_norm"
            inner_norm.runtime = runtime
            return inner_norm

        def bind(weight, scale, zero=None):
            """The packed tensors of a layer never change between calls: validate them once and return
            ``launch(activation, output) -> rc`` that checks only what changes per call (the activation and the
            output) and passes raw addresses.  The bound tensors must stay alive and in place; rebinding is
            the caller's business when it replaces them."""
            if zero is None:
                zero = zero_empty
            check_packed(weight, scale, zero)
            device_index = weight.device.index
            fn = runtime._launch_m if runtime._launch_m is not None else runtime.lib.launch
            rc, rc_ref = runtime._rc, runtime._rc_ref
            wp, sp, zp = weight.data_ptr(), scale.data_ptr(), zero.data_ptr()
            get_stream = _get_raw_stream

            # With the native extension both forms of the call are one C++ call each: launch(activation, output)
            # -> rc into the caller's tensor, launch.alloc(activation) -> a new output tensor.  Either hands an
            # activation (or output) it was not bound for back to the checks of `inner`, which name the problem.
            bound = None
            if not convert_first and get_stream is not None and runtime._launch_m is not None:
                bound = fastpath.bound_launch(runtime._launch_m, weight, scale, zero, True, n_out, k, dtype_a, device_index)
            if bound is not None:
                into = bound.into

                def launch(activation, output):
                    rc = into(activation, output, get_stream(device_index))
                    return inner(activation, weight, output, scale, zero) if rc is None else rc

                launch.alloc = lambda activation: bound(activation, get_stream(device_index))
                return launch

            def launch(activation, output):
                m = activation.shape[0]
                if (activation.dim() != 2 or activation.shape[1] != k or output.shape != (m, n_out)
                        or activation.dtype != dtype_a or output.dtype != dtype_a
                        or not activation.is_contiguous() or not output.is_contiguous()
                        or activation.device.index != device_index or output.device.index != device_index):
                    return inner(activation, weight, output, scale, zero)       # the full checks name the problem
                if convert_first:
                    activation = native.bf16_to_f16(activation)
                stream = get_stream(device_index) if get_stream is not None else _raw_stream(activation)
                fn(m, activation.data_ptr(), wp, output.data_ptr(), sp, zp, stream, rc_ref)
                return rc.value

            launch.alloc = None
            return launch

        func = inner_sym if self.sym else inner
        func.runtime = runtime
        func.bind = bind
        return func


class Matmul:
    """group_size == -1: no scales, no zero-points, raw unsigned fields (reference matmul.py:155-270)."""

    def __init__(self, n: int, k: int, nbits: int, dtype_a, dtype_b, layout: str = "nt"):
        self.n, self.k = n, k
        self.nbits = nbits
        self.dtype_a, self.dtype_b = dtype_a, dtype_b
        self.layout = layout
        assert self.layout == "nt", f"Layout {layout} is not supported"
        assert dtype_a in (torch.float16, torch.bfloat16), f"Data type {dtype_a} is not supported"
        assert dtype_b == torch.int8, f"Data type {dtype_b} is not supported"
        assert nbits in (2, 3, 4, 8), f"{nbits}-bit weights are not supported"

    @property
    def weight_shape(self):
        return (self.n, weight_row_bytes(self.k, self.nbits))

    def init_qfuncs(self):
        self.qfuncs = [MatmulQFunc(
            QTile((0, self.k), self.dtype_a, 16),
            QTile((self.n, self.k), self.dtype_b, self.nbits),
            "nt")]

    def get_dummy_inputs(self):
        require_gpu()
        m = 1
        activation = torch.zeros((m, self.k), dtype=self.dtype_a, device="cuda")
        weight = torch.zeros(self.weight_shape, dtype=self.dtype_b, device="cuda")
        output = torch.empty((m, self.n), dtype=self.dtype_a, device="cuda")
        return m, activation, weight, output, torch.cuda.current_stream()

    def compile_profile(self, enable_transform: bool = False, enable_schedule: bool = False,
                        enable_lower: bool = False):
        self.init_qfuncs()
        shape = f"{self.nbits}-{1}-{self.n}-{self.k}-{-1}"
        predefined = _load_predefined(shape)
        if predefined is not None:
            logger.info(f"[Profile] Using predefined config for {shape}")
            self.qfuncs = [apply_config(self.qfuncs[0], predefined)]
        else:
            if enable_schedule:
                self.qfuncs = list(chain.from_iterable(q.schedule() for q in self.qfuncs))
            if enable_lower:
                self.qfuncs = list(chain.from_iterable(q.lower() for q in self.qfuncs))

        self.runtimes = _compile_all(self.qfuncs)
        dummy = self.get_dummy_inputs() if len(self.runtimes) > 1 else None
        self.best_runtime, self.best_qfunc = _pick_best(self.runtimes, self.qfuncs, dummy, shape)
        return self._wrap(self.best_runtime)

    def _wrap(self, runtime):
        n, k, w_shape = self.n, self.k, self.weight_shape
        dtype_a = self.dtype_a

        def inner(activation, weight, output):
            m = activation.shape[0]
            assert activation.shape == (m, k)
            assert weight.shape == w_shape
            assert output.shape == (m, n)
            assert activation.dtype == dtype_a
            assert weight.dtype == torch.int8
            assert output.dtype == dtype_a
            assert activation.is_contiguous()
            assert weight.is_contiguous()
            assert output.is_contiguous()
            assert activation.is_cuda and weight.is_cuda and output.is_cuda
            return runtime.run_raw(m, (activation.data_ptr(), weight.data_ptr(), output.data_ptr()),
                                   _raw_stream(activation))

        def bind(weight):
            """Validate the layer's packed weight once; ``launch(activation, output) -> rc`` then checks only the
            two tensors that change per call (see ``QMatmul``'s closure)."""
            assert weight.shape == w_shape and weight.dtype == torch.int8 and weight.is_contiguous() and weight.is_cuda
            device_index = weight.device.index
            fn, rc, rc_ref = runtime.lib.launch, runtime._rc, runtime._rc_ref
            wp = weight.data_ptr()
            get_stream = _get_raw_stream

            bound = None
            if get_stream is not None:
                bound = fastpath.bound_launch(fn, weight, None, None, False, n, k, dtype_a, device_index)
            if bound is not None:
                into = bound.into

                def launch(activation, output):
                    rc_native = into(activation, output, get_stream(device_index))
                    return inner(activation, weight, output) if rc_native is None else rc_native

                launch.alloc = lambda activation: bound(activation, get_stream(device_index))
                return launch

            def launch(activation, output):
                m = activation.shape[0]
                if (activation.dim() != 2 or activation.shape[1] != k or output.shape != (m, n)
                        or activation.dtype != dtype_a or output.dtype != dtype_a
                        or not activation.is_contiguous() or not output.is_contiguous()
                        or activation.device.index != device_index or output.device.index != device_index):
                    return inner(activation, weight, output)
                stream = get_stream(device_index) if get_stream is not None else _raw_stream(activation)
                fn(m, activation.data_ptr(), wp, output.data_ptr(), stream, rc_ref)
                return rc.value

            launch.alloc = None
            return launch

        inner.runtime = runtime
        inner.bind = bind
        return inner
