"""``nn.Module`` front end of the quantized linear layer.

Drop-in for the reference's ``qfactory/qlinear.py``: ``QLinear.init(...)`` / ``QLinear.empty(...)``
return a ``GPTQLinear`` (grouped scales, optional zero-points) or a ``GEMVLinear``
(``group_size == -1``: raw integer weights) whose ``forward(x)`` maps ``(M, K) fp16`` to ``(M, N) fp16``
on ``x``'s device.  Attributes ``.w .s .z .func`` keep the reference's meaning (packed tensors and
the compiled closure for the constructor's ``batch_size``).

Beyond the reference: ``forward`` accepts any number of rows.  The specialisation compiled at
construction is tuned for ``batch_size``; other row counts get their own specialisation (per M
bucket) on first use, because the best kernel family changes with M (register-resident GEMV for a
few rows, matrix-core GEMM for many).  ``forward`` also accepts bf16 activations (the reference asserts
fp16, qfactory/core/matmul.py:133-136) and then returns bf16; those specialisations are compiled on first
use as well.  Scales stay fp16.
"""
import torch

from .convert import convert_params, weight_row_bytes, zero_row_bytes
from .core import QMatmul, Matmul
from .core import tiling


def _m_bucket(m):
    """Row count a specialisation is compiled for when ``m`` rows arrive."""
    if m < tiling.MGEMV_MIN_M:
        return m
    if m <= 16:
        return 16
    bucket = 32
    # 512 .. 4096: prefill-sized tiles.  Several rounds of blocks pay for 256 x 256 tiles where one round of the
    # same layer does not (4096 x 11008: 128 x 128 tiles at 1024 rows, 256 x 256 from 4096 rows on, 884 -> 699 us at 8192 rows)
    while bucket < m and bucket < 4096:
        bucket *= 2
    return bucket


class GPTQLinear(torch.nn.Module):
    def __init__(self, in_features, out_features, n_bits, weight, group_size, scale, zero, bias,
                 compile_flags, skip_convert, batch_size, base_impl=False):
        super().__init__()

        if bias:
            raise NotImplementedError("Bias is not supported")

        if skip_convert:
            w, s, z = weight, scale, zero
        else:
            w, s, z = convert_params({
                "K": in_features,
                "N": out_features,
                "NBITS": n_bits,
                "GS": group_size,
            }, (weight, scale, zero))

        n_groups = in_features // group_size
        assert in_features % (group_size * 2) == 0
        assert w.dtype == torch.int8
        assert s.dtype == torch.float16
        assert len(w.shape) == 2
        assert w.shape[0] * w.shape[1] == out_features * weight_row_bytes(in_features, n_bits)
        assert s.shape == (out_features, n_groups)
        if z is not None:
            assert z.dtype == torch.int8
            assert z.shape == (out_features, zero_row_bytes(n_groups, n_bits))

        self.in_features, self.out_features = in_features, out_features
        self.n_bits, self.group_size = n_bits, group_size
        self.w, self.s, self.z = w, s, z
        self.compile_flags = dict(compile_flags)
        self.base_impl = base_impl
        self.batch_size = batch_size

        self._funcs = {}
        self._launchers = {}            # (row-count bucket, dtype) -> launch(activation, output) bound to this layer's packed tensors
        self._last = (None, None, None)  # (rows, dtype, launcher) of the previous call: decode repeats one row count
        # the specialisation of the hint's row-count bucket: the one forward() looks up for that many rows
        self.func = self._compile(_m_bucket(batch_size), self.compile_flags)
        self._funcs[(_m_bucket(batch_size), torch.float16)] = self.func

    def __setattr__(self, name, value):
        if name in ("w", "s", "z") and getattr(self, "_launchers", None):
            self._launchers.clear()     # bound launchers hold the addresses of the tensors they were made for
            super().__setattr__("_last", (None, None, None))
        super().__setattr__(name, value)

    def _compile(self, m, compile_flags, dtype=torch.float16, epilogue="none", prologue="none"):
        matmul = QMatmul(m, self.out_features, self.in_features, self.n_bits, self.z is None,
                         dtype, torch.int8, self.group_size, base_impl=self.base_impl, output_epilogue=epilogue,
                         input_prologue=prologue)
        func = matmul.compile_profile(**compile_flags)
        # One launch now: the first call of a specialisation loads its code object and may raise its
        # LDS limit (hipFuncSetAttribute), neither of which should happen inside a HIP-graph capture.
        if self.w.is_cuda:
            x = torch.zeros(m, self.in_features, dtype=dtype, device=self.w.device)
            out = torch.zeros(m, self.out_features // (2 if epilogue == "silu_mul" else 1), dtype=dtype, device=self.w.device)
            if prologue == "add_rmsnorm":
                rc = func(x, None, torch.ones(self.in_features, dtype=dtype, device=self.w.device), None, 1e-6,
                          self.w, out, self.s, self.z)
            else:
                rc = func(x, self.w, out, self.s, self.z) if self.z is not None else func(x, self.w, out, self.s)
            if rc != 0:
                raise RuntimeError(f"quantized linear launch failed with return code {rc}")
        return func

    def func_for(self, m, dtype=torch.float16):
        key = (_m_bucket(m), dtype)
        func = self._funcs.get(key)
        if func is None:
            func = self._funcs[key] = self._compile(key[0], self.compile_flags, dtype)
        return func

    def _launcher(self, m, dtype):
        """``launch(x, out)`` for ``m`` rows of ``dtype``: the bucket's closure with this layer's packed tensors
        validated once and bound (the reference re-checks all five tensors on every call, matmul.py:124-144; the
        three that belong to the layer cannot change between calls)."""
        key = (_m_bucket(m), dtype)      # one launcher per bucket: it takes the row count at call time
        launch = self._launchers.get(key)
        if launch is None:
            launch = self._launchers[key] = self.func_for(m, dtype).bind(self.w, self.s, self.z)
        self._last = (m, dtype, launch)
        return launch

    def forward(self, x: torch.Tensor, out: torch.Tensor = None):
        """``(M, K)`` -> ``(M, N)`` in ``x``'s dtype on ``x``'s device.  ``out`` (beyond the reference, which always
        allocates, qlinear.py:53): a preallocated contiguous ``(M, N)`` tensor to write into, e.g. under HIP-graph
        capture or in a loop that reuses its buffers."""
        m, dtype = x.shape[0], x.dtype
        launch = None
        if m > 0:
            last = self._last
            launch = last[2] if (last[0] == m and last[1] is dtype) else self._launcher(m, dtype)
        if out is None:
            if launch is not None and launch.alloc is not None:
                out = launch.alloc(x)                      # allocation and launch in one native call
                if out is not None:
                    return out
            out = torch.empty((m, self.out_features), dtype=dtype, device=x.device)
        if m == 0:
            assert out.shape == (0, self.out_features)
            return out                                     # no rows: nothing to launch
        rc = launch(x, out)
        if rc != 0:
            raise RuntimeError(f"quantized linear launch failed with return code {rc}")
        return out


    def fuses_silu_mul(self, m, dtype=torch.float16):
        """Does ``forward_silu_mul`` on ``m`` rows run as one launch?  Where the dot2 GEMV kernel serves and its
        rows come in pairs, or the A-stationary kernel and gate and up are whole 16-row tiles, or the GEMM kernel
        and every wave holds whole (gate, up) pairs of its own (N a multiple of the wave's weight rows)."""
        bucket = _m_bucket(m)
        if dtype != torch.float16 or self.out_features % 2:
            return False
        # (the kernel as it is built for an epilogue that pairs columns: long rows are not split over blocks)
        regime = tiling.regime_for(bucket, self.in_features, self.n_bits, self.group_size, self.out_features, ksplit=False)
        if regime == "mgemv":
            return self.out_features % 32 == 0
        if regime == "gemm":
            t = tiling.gemm_tiling(bucket, self.out_features, self.in_features, self.n_bits, self.group_size)
            return self.out_features % (32 * t["NT32"]) == 0
        if regime != "gemv":
            return False
        return tiling.gemv_tiling(bucket, self.out_features, self.in_features, self.n_bits, self.group_size)["U"] % 2 == 0

    def fuses_accumulate(self, m, dtype=torch.float16):
        """Does ``forward_accumulate`` on ``m`` rows run as one launch?  fp16, every kernel but the generic fallback."""
        regime = tiling.regime_for(_m_bucket(m), self.in_features, self.n_bits, self.group_size, self.out_features)
        return dtype == torch.float16 and regime in ("gemv", "mgemv", "skinny", "gemm")

    def forward_accumulate(self, x: torch.Tensor, out: torch.Tensor):
        """``out += self(x)`` in place: ``out = fp16(out + fp16(projection))``, the two roundings of the projection
        followed by a residual add -- the o and down projections of a decoder layer writing into the residual stream.
        One launch (the kernel's final sum reads the output element it is about to write) wherever
        ``fuses_accumulate`` says so; otherwise ``forward`` and an in-place add, which give the same bits.  Not in
        the reference."""
        m = x.shape[0]
        assert out.shape == (m, self.out_features) and out.dtype == x.dtype and out.is_contiguous()
        if m == 0:
            return out
        if not self.fuses_accumulate(m, x.dtype):
            return out.add_(self.forward(x))
        key = (_m_bucket(m), x.dtype, "accumulate")
        func = self._funcs.get(key)
        if func is None:
            func = self._funcs[key] = self._compile(key[0], self.compile_flags, x.dtype, "accumulate")
        rc = func(x, self.w, out, self.s, self.z) if self.z is not None else func(x, self.w, out, self.s)
        if rc != 0:
            raise RuntimeError(f"quantized linear launch failed with return code {rc}")
        return out

    def fuses_add_rmsnorm(self, m, dtype=torch.float16, silu_mul=False):
        """Does ``forward_add_rmsnorm`` on ``m`` rows run as one launch?  Where the dot2 GEMV kernel or the A-stationary
        kernel serves (up to 32 rows, fp16)."""
        if dtype != torch.float16 or (silu_mul and not self.fuses_silu_mul(m, dtype)):
            return False
        return tiling.regime_for(_m_bucket(m), self.in_features, self.n_bits, self.group_size, self.out_features,
                                 ksplit=False) in ("gemv", "mgemv")

    def forward_add_rmsnorm(self, x: torch.Tensor, delta, gamma: torch.Tensor, eps: float, x_out=None, silu_mul=False):
        """The step of a decoder layer that ends in this projection: ``h = x + delta`` (fp16 add; ``delta`` may be
        None), ``a = fp16(fp16(h * rsqrt(mean(h^2) + eps)) * gamma)``, then ``self(a)`` -- or, with ``silu_mul``,
        ``self.forward_silu_mul(a)``.  ``x_out`` (required with ``delta``; a buffer of its own) receives ``h``, the
        next residual stream.  One launch where the dot2 GEMV kernel (M < 3) or the A-stationary kernel (up to 32 rows)
        serves: every block normalises the rows for itself while its first weights are in flight.  Otherwise ``qf_add_rmsnorm`` followed by the projection,
        which is also what the one launch is checked against: its sum of squares is added in another order, so a
        normalised element may differ by one fp16 ulp.  Not in the reference, whose end-to-end runs leave residual
        add and norm to vLLM's ``fused_add_rms_norm``."""
        from . import native
        m = x.shape[0]
        assert delta is None or x_out is not None, "with delta, the sum needs a buffer to go to"
        # the same operand contract at every row count, whichever path serves it
        if x_out is not None:
            assert x_out.data_ptr() != x.data_ptr(), "x_out must not alias the residual stream it is computed from"
            assert delta is None or x_out.data_ptr() != delta.data_ptr(), "x_out must not alias delta"
        if m == 0 or not self.fuses_add_rmsnorm(m, x.dtype, silu_mul):
            h = x
            if delta is not None:
                h = torch.add(x, delta, out=x_out)
            elif x_out is not None:
                x_out.copy_(x)
            a = torch.empty_like(x)
            if m > 0 and x.dtype == torch.float16 and x.shape[1] <= native.ADD_RMSNORM_MAX_HIDDEN:
                native.add_rmsnorm(h, None, gamma, a, eps)
            elif m > 0:
                # rows longer than qf_add_rmsnorm takes, or bf16: the same expression (and roundings) in torch ops
                h32 = h.to(torch.float32)
                normed = (h32 * torch.rsqrt(h32.pow(2).mean(dim=1, keepdim=True) + eps)).to(x.dtype)
                torch.mul(normed, gamma, out=a)
            return self.forward_silu_mul(a) if silu_mul else self.forward(a)
        key = (_m_bucket(m), x.dtype, "add_rmsnorm+silu_mul" if silu_mul else "add_rmsnorm")
        func = self._funcs.get(key)
        if func is None:
            func = self._funcs[key] = self._compile(key[0], self.compile_flags, x.dtype,
                                                    "silu_mul" if silu_mul else "none", "add_rmsnorm")
        output = torch.empty(m, self.out_features // (2 if silu_mul else 1), dtype=x.dtype, device=x.device)
        rc = func(x, delta, gamma, x_out, eps, self.w, output, self.s, self.z)
        if rc != 0:
            raise RuntimeError(f"quantized linear launch failed with return code {rc}")
        if delta is None and x_out is not None:
            x_out.copy_(x)
        return output

    def forward_silu_mul(self, x: torch.Tensor):
        """For a fused gate+up projection (rows 0 .. N/2-1 gate, the rest up): the SwiGLU activation
        ``silu(gate) * up`` of shape (M, N/2), i.e. ``silu_mul(self(x))``.  The product is formed in the kernel's
        epilogue (one launch) wherever ``fuses_silu_mul`` says so; otherwise by ``forward`` followed by
        ``qf_silu_mul``.  Both give the same bits.  Not in the reference, whose end-to-end runs leave the step to vLLM's ``SiluAndMul``."""
        m, half = x.shape[0], self.out_features // 2
        output = torch.empty(m, half, dtype=x.dtype, device=x.device)
        if m == 0:
            return output
        if not self.fuses_silu_mul(m, x.dtype):
            y = self.forward(x)
            if x.dtype != torch.float16:
                # qf_silu_mul is an fp16 kernel: other activation types take the same expression in torch ops
                return torch.mul(torch.nn.functional.silu(y[:, :half]), y[:, half:], out=output)
            from . import native
            return native.silu_mul(y, output)
        key = (_m_bucket(m), x.dtype, "silu_mul")
        func = self._funcs.get(key)
        if func is None:
            func = self._funcs[key] = self._compile(key[0], self.compile_flags, x.dtype, "silu_mul")
        rc = func(x, self.w, output, self.s, self.z) if self.z is not None else func(x, self.w, output, self.s)
        if rc != 0:
            raise RuntimeError(f"quantized linear launch failed with return code {rc}")
        return output


class GEMVLinear(torch.nn.Module):
    def __init__(self, in_features, out_features, n_bits, weight, bias, compile_flags, skip_convert):
        super().__init__()

        if bias:
            raise NotImplementedError("Bias is not supported")

        if skip_convert:
            w = weight
        else:
            w = convert_params({
                "K": in_features,
                "N": out_features,
                "NBITS": n_bits,
            }, (weight,))

        assert w.dtype == torch.int8
        assert len(w.shape) == 2
        assert w.shape[0] * w.shape[1] == out_features * weight_row_bytes(in_features, n_bits)

        self.in_features, self.out_features, self.n_bits = in_features, out_features, n_bits
        self.w = w

        self.compile_flags = dict(compile_flags)
        self._launchers = {}
        matmul = Matmul(out_features, in_features, n_bits, torch.float16, torch.int8)
        self.func = matmul.compile_profile(**compile_flags)
        self._funcs = {torch.float16: self.func}

    def __setattr__(self, name, value):
        if name == "w" and getattr(self, "_launchers", None):
            self._launchers.clear()
        super().__setattr__(name, value)

    def func_for(self, dtype):
        func = self._funcs.get(dtype)
        if func is None:
            matmul = Matmul(self.out_features, self.in_features, self.n_bits, dtype, torch.int8)
            func = self._funcs[dtype] = matmul.compile_profile(**self.compile_flags)
        return func

    def forward(self, x: torch.Tensor, out: torch.Tensor = None):
        m, dtype = x.shape[0], x.dtype
        launch = self._launchers.get(dtype)
        if launch is None:
            launch = self._launchers[dtype] = self.func_for(dtype).bind(self.w)
        if out is None:
            if launch.alloc is not None:
                out = launch.alloc(x)                      # allocation and launch in one native call
                if out is not None:
                    return out
            out = torch.empty((m, self.out_features), dtype=dtype, device=x.device)
        if m == 0:
            assert out.shape == (0, self.out_features)
            return out
        rc = launch(x, out)
        if rc != 0:
            raise RuntimeError(f"quantized linear launch failed with return code {rc}")
        return out


class QLinear():
    @staticmethod
    def init(batch_size, in_features, out_features, n_bits, weight, group_size=-1, scale=None,
             zero=None, bias=False, compile_flags={}):
        if group_size == -1:
            return GEMVLinear(in_features, out_features, n_bits, weight, bias, compile_flags,
                              skip_convert=False)
        return GPTQLinear(in_features, out_features, n_bits, weight, group_size, scale, zero, bias,
                          compile_flags, skip_convert=False, batch_size=batch_size)

    @staticmethod
    def empty(M, K, N, NBITS, GS, sym, compile_flags, base_impl=False):
        w = torch.empty(N, weight_row_bytes(K, NBITS), dtype=torch.int8, device='cuda')
        if GS == -1:
            return GEMVLinear(K, N, NBITS, w, False, compile_flags, skip_convert=True)
        s = torch.empty(N, K // GS, dtype=torch.float16, device='cuda')
        z = torch.empty(N, zero_row_bytes(K // GS, NBITS), dtype=torch.int8, device='cuda')
        return GPTQLinear(K, N, NBITS, w, GS, s, None if sym else z, False, compile_flags,
                          skip_convert=True, batch_size=M, base_impl=base_impl)
