"""QFuncs: a quantized matmul described over QTiles, its search space, and the HIP translation unit
it emits.

Mirrors the reference's ``qfactory/core/qfunc.py`` at the interface level -- ``QMatmulQFunc`` /
``MatmulQFunc`` with ``arg_name_type() / transform() / schedule() / lower() / emit()`` and the
attributes a tuned-config JSON may set verbatim (``parallel_strategy``, ``tiling_configs``,
``decode_strategy``, ``l2cache_a``, ``l2cache_b``, ``smem_quant``; qfunc.py:27-41, matmul.py:76-77)
-- but what is emitted is a specialisation of the gfx950 templates in ``qfactory/include`` for one
(bits, group size, N, K, M-tile), compiled by hipcc.

The emitted object exports the reference's entry point (qfunc.py:139-152 / 233-238)

    extern "C" void launch(<pointers...>, void* stream, int& return_code)

plus ``launch_m`` (same, with the number of activation rows as a leading ``int``) and
``qf_describe`` (a string naming the specialisation).
"""
import copy
from typing import List

import torch

from . import tiling

Python2CppTypes = {  # python-side type -> (type in the C signature, type used inside)
    int: ("int", "int"),
    torch.float16: ("void*", "uint16_t*"),
    torch.bfloat16: ("void*", "uint16_t*"),
    torch.int8: ("void*", "uint8_t*"),
    torch.cuda.streams.Stream: ("void*", "hipStream_t"),
}


# Attributes of a QFunc that a tuned-config JSON ($QFACTORY_CONFIG) may set: the reference's file sets attributes
# verbatim (qfactory/core/matmul.py:76-77); here anything outside this list is an error, so a config file can choose
# among valid specialisations but cannot inject preprocessor definitions or other state.
CONFIG_ATTRIBUTES = ("regime", "parallel_strategy", "tiling_configs", "decode_strategy",
                     "l2cache_a", "l2cache_b", "smem_quant")

# Preprocessor knobs of the kernel headers that change how a kernel is scheduled, never what it computes; the only
# names `QFunc.defines` may hold.  (The headers' QF_*_EXPERIMENT timing knobs give wrong results and refuse to
# compile unless the translation unit itself asks for them; the generator cannot.)
TUNING_DEFINES = ("QF_FUSED_AND_OR", "QF_SCHED_FENCE_MODE", "QF_WIDE_HOLDERS", "QF_GEMV_A_FIRST",
                  "QF_GEMV_QUANT_DEDUP", "QF_GEMV_WAVES_PER_EU", "QF_GEMV_EARLY_OUT", "QF_MGEMV_SB", "QF_MGEMV_PIN_FIRST_LOADS",
                  "QF_MGEMV_COMPUTE_CLAMPED", "QF_GEMM_FULL_DRAIN", "QF_GEMM_XCD_MAP")


def apply_config(qfunc, entry):
    """Set the attributes of a tuned-config entry on ``qfunc``; unknown names raise."""
    for key, value in entry.items():
        if key not in CONFIG_ATTRIBUTES:
            raise ValueError(f"config attribute {key!r} is not one of {CONFIG_ATTRIBUTES}")
        if key == "regime" and value != qfunc.regime:
            raise ValueError(f"config entry is for the {value!r} kernel family, the problem runs on {qfunc.regime!r}")
        setattr(qfunc, key, value)
    return qfunc


class QFunc:
    regime = "gemv"

    def arg_name_type(self):
        raise NotImplementedError

    def emit(self) -> str:
        raise NotImplementedError

    def clone(self, **attrs):
        other = copy.deepcopy(self)
        for key, value in attrs.items():
            setattr(other, key, value)
        return other

    # -- shared emit helpers --------------------------------------------------------------
    def _signature(self, name, leading_m):
        lines = [f'extern "C" void {name} (']
        if leading_m:
            lines.append("\tint m,")
        for arg, t in self.arg_name_type():
            if t is int:
                continue
            lines.append(f"\t{Python2CppTypes[t][0]} _{arg},")
        lines.append("\tint& __return_code")
        lines.append(") {")
        return "\n".join(lines) + "\n"


def _problem_of(qtile_a, qtile_b):
    m, k = qtile_a.shape
    n, kb = qtile_b.shape
    assert k == kb, f"Shape mismatch: {k} != {kb}"
    return m, n, k


class QMatmulQFunc(QFunc):
    """activation (M,K) fp16  x  quantized weight (N,K), per-group scale (and zero)  ->  (M,N) fp16.

    Beyond the reference (fp16 only, matmul.py:36): a bf16 activation tile gives a bf16 output; scales
    stay fp16, the packed tensors are the same."""

    def __init__(self, qtile_a, qtile_b, layout, base_impl=False, ksplit=True):
        self.qtile_a, self.qtile_b, self.layout = qtile_a, qtile_b, layout
        # may long rows be split over several blocks that meet through device memory?  Not with the norm prologue or
        # the SwiGLU epilogue: a block that sees part of K can neither normalise a row nor pair gate with up
        self.ksplit = ksplit
        assert qtile_a.quant_method == "none", "Quantization method not supported for A"
        assert qtile_b.quant_method in ("sym", "asym"), "Quantization method of B must be 'sym' or 'asym'"
        assert layout == "nt", f"Layout {layout} is not supported"
        m, n, k = _problem_of(qtile_a, qtile_b)
        gs = qtile_b.quant_granularity[1]

        # Template-based code generation: which kernel family and how it is tiled
        self.regime = tiling.regime_for(m, k, qtile_b.nbits, gs, n, ksplit=ksplit)
        self.parallel_strategy = "row"          # teams sweep rows, K split over lanes and waves
        self.tiling_configs = self.default_tiling(self.regime)
        # Computation transformation (reference: qfunc.py:85-91): "deferred" applies scale and zero once per
        # chunk / group in fp32 after the integer dot product; "eager" dequantises every element to fp16 first.
        self._gs = gs
        self.decode_strategy = self.decode_strategies()[0]
        # Load-path scheduling
        self.l2cache_a = True                   # activations: normal (cached) loads
        self.l2cache_b = False                  # weights: streaming (non-temporal) loads
        self.smem_quant = False                 # scales / zero-points of a block's rows through LDS (dot2 GEMV kernel);
        #                                         measured slower at M = 1 (a barrier in a one-shot block), 3 % faster at M = 2
        self.base_impl = base_impl
        # "silu_mul": the weight is a fused gate+up projection and the kernel writes the (M, N/2) SwiGLU activation
        # fp16(silu(gate)) * up instead of the (M, N) projection (the kernels for M <= 32; not in the reference).
        # "accumulate": the kernel adds its projection to what the output holds, out = fp16(out + fp16(projection))
        # (the kernels for M <= 32, fp16; a projection that writes into the residual stream; not in the reference)
        self.output_epilogue = "none"
        # "add_rmsnorm": the kernel makes its activations itself -- residual add and RMSNorm of a decoder layer run in
        # front of the dot products -- and the object exports launch_norm (dot2 GEMV kernel, fp16; not in the reference)
        self.input_prologue = "none"
        assert qtile_a.dtype in (torch.float16, torch.bfloat16), f"Data type {qtile_a.dtype} is not supported for A"

    @property
    def act_dtype(self):
        return self.qtile_a.dtype

    @property
    def converts_activations(self):
        """Does the kernel read bf16 activations itself?  The GEMM kernel cannot (its activation tiles go
        from global memory to LDS untouched): its caller converts the rows to fp16 first."""
        return self.act_dtype == torch.bfloat16 and self.regime != "gemm"

    # -- description ------------------------------------------------------------------------
    @property
    def problem(self):
        m, n, k = _problem_of(self.qtile_a, self.qtile_b)
        return {"M": m, "N": n, "K": k, "NBITS": self.qtile_b.nbits, "GS": self._gs,
                "SYM": self.qtile_b.quant_method == "sym"}

    def default_tiling(self, regime):
        p = {"M": self.qtile_a.shape[0], "N": self.qtile_b.shape[0], "K": self.qtile_b.shape[1]}
        nbits, gs = self.qtile_b.nbits, self.qtile_b.quant_granularity[1]
        if regime == "gemv":
            return tiling.gemv_tiling(p["M"], p["N"], p["K"], nbits, gs)
        if regime == "mgemv":
            split = tiling.mgemv_ksplit_tiling(p["M"], p["N"], p["K"], nbits, gs) if self.ksplit else None
            return split or tiling.mgemv_tiling(p["M"], p["N"], p["K"], nbits, gs)
        if regime == "skinny":
            return tiling.skinny_tiling(p["M"], p["N"], p["K"], nbits, gs)
        if regime == "gemm":
            return tiling.gemm_tiling(p["M"], p["N"], p["K"], nbits, gs)
        return tiling.mfma_tiling(p["M"], p["N"], p["K"], nbits, gs)

    def arg_name_type(self):
        return [
            ("activation", self.act_dtype if self.converts_activations else torch.float16),
            ("weight", torch.int8), ("output", self.act_dtype),
            ("scale", torch.float16), ("zero", torch.int8),
            ("stream", torch.cuda.streams.Stream),
        ]

    # -- search space -------------------------------------------------------------------------
    def decode_strategies(self):
        """Decode strategies this problem's kernel family implements, its default first.

        * dot2 GEMV: deferred (default) and eager in packed fp16.
        * A-stationary and streaming matrix-core kernels: deferred where a chunk of 512/b fields lies inside one
          group (the group sum is formed on the matrix core and scaled once in fp32), eager always.
        * GEMM and the generic matrix-core kernel: eager only (dequantised fp16 fragments feed the MFMA)."""
        nbits, gs = self.qtile_b.nbits, self._gs
        chunk = 4 * (128 // tiling.plane_bits(nbits))
        if self.regime == "gemv":
            return ["deferred", "eager"]
        if self.regime == "mgemv":
            return ["deferred", "eager"] if gs % chunk == 0 else ["eager"]
        if self.regime == "skinny":
            return ["deferred", "eager"] if (gs >= 2 * chunk or gs == chunk) else ["eager"]
        return ["eager"]

    def transform(self) -> List[QFunc]:
        return [self.clone(decode_strategy=d) for d in self.decode_strategies()]

    def schedule(self) -> List[QFunc]:
        smem = (False, True) if self.regime == "gemv" and self.output_epilogue == "none" else (False,)
        return [self.clone(l2cache_a=True, l2cache_b=b, smem_quant=s) for b in (False, True) for s in smem]

    def lower(self) -> List[QFunc]:
        p = self.problem
        if self.regime == "gemv":
            cands = tiling.gemv_candidates(p["M"], p["N"], p["K"], p["NBITS"], p["GS"])
        elif self.regime == "mgemv":
            cands = tiling.mgemv_candidates(p["M"], p["N"], p["K"], p["NBITS"], p["GS"])
        elif self.regime == "skinny":
            cands = tiling.skinny_candidates(p["M"], p["N"], p["K"], p["NBITS"], p["GS"])
        elif self.regime == "gemm":
            cands = tiling.gemm_candidates(p["M"], p["N"], p["K"], p["NBITS"], p["GS"])
        else:
            cands = tiling.mfma_candidates(p["M"], p["N"], p["K"], p["NBITS"], p["GS"])
        return [self.clone(tiling_configs=c) for c in cands]

    # -- code generation ----------------------------------------------------------------------
    def emit(self) -> str:
        p = self.problem
        t = self.tiling_configs
        b = lambda x: "true" if x else "false"
        code = "// QFactory-HIP generated translation unit\n\n"
        defines = dict(getattr(self, "defines", {}))                        # kernel-header tuning knobs
        for name in defines:
            if name not in TUNING_DEFINES:
                raise ValueError(f"{name} is not a tuning knob of the kernel headers ({', '.join(TUNING_DEFINES)})")
        if self.decode_strategy not in self.decode_strategies():
            raise ValueError(f"decode_strategy {self.decode_strategy!r} is not implemented by the {self.regime!r} kernel "
                             f"for {p['NBITS']}-bit weights in groups of {p['GS']} (available: {self.decode_strategies()})")
        if self.decode_strategy == "eager" and self.regime in ("gemv", "mgemv", "skinny"):
            defines[{"gemv": "QF_GEMV_EAGER", "mgemv": "QF_MGEMV_EAGER", "skinny": "QF_SKINNY_EAGER"}[self.regime]] = 1
        if self.regime in ("gemm", "mgemv", "skinny"):
            # the matrix-core kernels expose their dequantisation's vector-instruction issue and have
            # registers to spare: the one-instruction mask-and-merge decode pays there (2 - 7 %
            # measured); it does not in the 4-bit GEMV kernel, where it costs a resident wave
            defines.setdefault("QF_FUSED_AND_OR", 1)
        if self.regime == "gemv" and p["NBITS"] in (2, 3) and t["VB"] == 8 and t["MT"] == 1 \
                and self.decode_strategy == "deferred" and not self.smem_quant \
                and tiling.gemv_chunks_per_lane(p["K"], p["NBITS"], t) == 1:
            # 32 fields per lane and row: the compiler-scheduled one-instruction decode and one scale / zero-point
            # load per lane and stage, as for 4 bits below (part of the 8-byte tiling's measured gain)
            defines.setdefault("QF_FUSED_AND_OR", 2)
            defines.setdefault("QF_GEMV_QUANT_DEDUP", 1)
        if self.regime == "gemv" and p["NBITS"] == 2:
            # sixteen fields per word make the 2-bit GEMV decode-bound: measured 7.6 -> 6.9 us at 8192 x 8192
            defines.setdefault("QF_FUSED_AND_OR", 1)
        if self.regime == "gemv" and p["NBITS"] == 4 and self.decode_strategy == "deferred" and not self.smem_quant \
                and tiling.gemv_chunks_per_lane(p["K"], p["NBITS"], t) == 1:
            # one chunk per lane and row (K <= 4096 x waves): the mask-and-merge decode in one instruction with
            # compiler-scheduled operands, and one scale / zero-point load per lane and stage after the group's
            # lanes have added their sums.  Measured against the plain form, cold weights: 12288 x 4096
            # 6.74 -> 6.47 us, 4096 x 4096 4.00 -> 3.74, 22016 x 4096 10.04 -> 9.86, 8192 x 8192 (eight rows per
            # stage) 8.85 -> 8.26; two chunks per lane (K = 28672) lose 6 %, K = 11008 is level.
            defines.setdefault("QF_FUSED_AND_OR", 2)
            defines.setdefault("QF_GEMV_QUANT_DEDUP", 1)
        if self.regime == "mgemv" and t.get("KS", 1) == 1 and t["WK"] <= 10 and t["MT16"] == 1 \
                and self.output_epilogue != "silu_mul":
            # ten waves and fewer leave LDS for eight partial tiles per wave between two block-wide sums instead of
            # four; it pays where a block sweeps many tiles (K = 5120 at M = 16, cold weights: 27648 x 5120 20.6 -> 18.7 us,
            # 55296 x 5120 36.7 -> 33.7; 15360 x 5120 13.0 -> 12.9, 7168 x 5120 level)
            slots = -(-(-(-p["N"] // 16)) // min(-(-p["N"] // 16), t["PB"]))
            if slots >= 6 and tiling.mgemv_lds_bytes(1, t["WK"], t["CH"], p["NBITS"], sb=8) <= 160 * 1024:
                defines.setdefault("QF_MGEMV_SB", 8)
        if self.regime == "mgemv" and t["MT16"] == 1 and t.get("KS", 1) > 1 and "QF_MGEMV_SB" not in defines:
            # K split over blocks and five tiles per block: one batch of five instead of four and one, so that the
            # blocks' sums go into their swaps in one go (M = 4 / 16, cold weights: 10240 x 8192 12.1 / 13.1 -> 11.3 / 12.5 us,
            # 5120 x 14336 12.9 / 13.6 -> 11.1 / 12.1).  Without the split, or with nine tiles (five and four), level.
            slots = -(-(-(-p["N"] // 16)) // min(-(-p["N"] // 16), t["PB"]))
            if slots == 5 and tiling.mgemv_lds_bytes(1, t["WK"], t["CH"], p["NBITS"], sb=5) <= 160 * 1024:
                defines.setdefault("QF_MGEMV_SB", 5)
        if self.regime == "gemm":
            # Block -> tile map that puts the row slabs of one column of tiles on one XCD (its L2 then serves the weights to
            # all of them) instead of the columns of one slab: pays where a launch has a few slabs -- measured, FETCH_SIZE
            # and time, plain against mapped: 22016 x 4096 at 2048 rows 562 -> 471 MB and 380 -> 357 us, 10240 x 8192 at 256
            # rows (two slabs) 125 -> 80 MB and 65.2 -> 62.8 us -- and loses where there are many, because the blocks of
            # an XCD then share no activation slab: 12288 x 4096 at 8192 rows 806 -> 3260 MB, 753 -> 791 us.
            slabs = -(-p["M"] // t["BM"])
            if 2 <= slabs <= 8 and -(-p["N"] // (32 * t["NT32"] * t["WN"])) >= 8:
                defines.setdefault("QF_GEMM_XCD_MAP", 1)
        assert t.get("KS", 1) == 1 or (self.input_prologue == "none" and self.output_epilogue != "silu_mul"), \
            "a block that sees part of K can neither normalise a row nor pair gate with up: build the object with ksplit=False"
        if self.act_dtype == torch.bfloat16:
            defines["QF_OUT_BF16"] = 1
            if self.converts_activations:
                defines["QF_IN_BF16"] = 1
        if self.output_epilogue == "accumulate":
            assert self.regime in ("gemv", "mgemv", "skinny", "gemm") and self.act_dtype == torch.float16, \
                "every kernel but the generic matrix-core fallback, on fp16, can add its result to the output"
            defines["QF_OUT_ACCUMULATE"] = 1
        elif self.output_epilogue != "none":
            assert self.output_epilogue == "silu_mul" and self.regime in ("gemv", "mgemv", "gemm") and self.act_dtype == torch.float16, \
                "only the dot2 GEMV, the A-stationary and the GEMM kernel, on fp16, write silu(gate) * up"
            defines[{"gemv": "QF_GEMV_GATE_UP_SILU", "mgemv": "QF_MGEMV_GATE_UP_SILU", "gemm": "QF_GEMM_GATE_UP_SILU"}[self.regime]] = 1
        if self.input_prologue != "none":
            assert self.input_prologue == "add_rmsnorm" and self.regime in ("gemv", "mgemv") and self.act_dtype == torch.float16, \
                "only the dot2 GEMV kernel and the A-stationary kernel, on fp16, run the residual add and RMSNorm themselves"
            defines["QF_GEMV_NORM_PROLOGUE" if self.regime == "gemv" else "QF_MGEMV_NORM_PROLOGUE"] = 1
        if self.smem_quant and self.regime == "gemv" and self.output_epilogue == "none":
            defines["QF_GEMV_SMEM_QUANT"] = 1
        for name, value in sorted(defines.items()):
            code += f"#define {name} {value}\n"
        if self.regime == "gemv":
            code += '#include "qf_gemv.hip.h"\n'
            cfg = (f"qf::GemvCfg<{p['NBITS']}, {p['GS']}, {b(p['SYM'])}, true, {p['N']}, {p['K']}, "
                   f"{t['MT']}, {t['WK']}, {t['WN']}, {t['U']}, {t['STEPS']}, {t['VB']}, {b(not self.l2cache_b)}>")
            call = "qf::gemv_launch<Cfg>"
        elif self.regime == "mgemv":
            code += '#include "qf_mgemv.hip.h"\n'
            cfg = tiling.mgemv_cfg_string(p, t, not self.l2cache_b)
            call = "qf::mgemv_launch<Cfg>"
        elif self.regime == "skinny":
            code += '#include "qf_skinny.hip.h"\n'
            cfg = tiling.skinny_cfg_string(p, t, not self.l2cache_b)
            call = "qf::skinny_launch<Cfg>"
        elif self.regime == "gemm":
            code += '#include "qf_gemm.hip.h"\n'
            cfg = tiling.gemm_cfg_string(p, t, not self.l2cache_b)
            call = "qf::gemm_launch<Cfg>"
        elif self.regime == "mfma":
            code += '#include "qf_mfma.hip.h"\n'
            cfg = tiling.mfma_cfg_string(p, t, self.decode_strategy, not self.l2cache_b)
            call = "qf::mfma_launch<Cfg>"
        else:
            raise ValueError(f"unknown regime {self.regime}")
        norm_abi = "#define QF_LAUNCH_NORM 1\n" if self.input_prologue == "add_rmsnorm" else ""
        if self.regime == "mgemv" and t.get("KS", 1) > 1:
            norm_abi += "#define QF_LAUNCH_STATIC 1\n"
        code += f'#if __has_include("qfactory_launch.h")\n#define QF_LAUNCH_GROUPED 1\n{norm_abi}#include "qfactory_launch.h"\n#endif\n\n'
        code += f"using Cfg = {cfg};\nconstexpr int M = {p['M']};\n\n"
        args = "_activation, _weight, _output, _scale, _zero"
        code += self._signature("launch", leading_m=False)
        code += f"\t__return_code = {call}({args}, M, (hipStream_t)_stream);\n}}\n\n"
        code += self._signature("launch_m", leading_m=True)
        code += f"\t__return_code = {call}({args}, m, (hipStream_t)_stream);\n}}\n\n"
        if self.regime == "mgemv" and t.get("KS", 1) > 1:
            # An object that splits K over blocks uses scratch memory in device memory, which launch / launch_m allocate
            # at their first call on a device.  For callers that cannot allocate (under HIP-graph capture from the first
            # call on, in loops that forbid it): the same launch on a static device array of this object.
            code += ("// ---- entry point that allocates nothing ----\n"
                     "// Scratch memory of launch_m_static: one copy per GPU, held until the process ends, shared by every call on\n"
                     "// that GPU (calls that overlap in time on one GPU race; calls on one stream do not overlap).  Zero at load;\n"
                     "// every launch leaves the slots in which its blocks exchange their sums zero.\n"
                     "static __device__ __align__(256) unsigned char scratch[qf::mgemv_static_scratch_bytes<Cfg>()];\n\n"
                     "static int qf_static_scratch(qf::MGemvScratch& out) {\n"
                     "\tstatic std::mutex lock;\n\tstatic void* address[64] = {};       // per device: each GPU holds its own copy at its own address\n"
                     "\tint dev = 0;\n"
                     "\tif (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {\n"
                     "\t\tfprintf(stderr, \"qfactory mgemv: cannot tell the current device\\n\");\n\t\treturn 2;\n\t}\n"
                     "\tstd::lock_guard<std::mutex> guard(lock);\n"
                     "\tif (address[dev] == nullptr) {\n"
                     "\t\tvoid* ptr = nullptr;\n"
                     "\t\thipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));\n"
                     "\t\tif (e != hipSuccess || ptr == nullptr) {\n"
                     "\t\t\tfprintf(stderr, \"qfactory mgemv: no address for the static scratch array: %s\\n\", hipGetErrorString(e));\n"
                     "\t\t\treturn 2;\n\t\t}\n"
                     "\t\taddress[dev] = ptr;\n\t}\n"
                     "\tout = qf::mgemv_scratch_at<Cfg>(address[dev]);\n\treturn 0;\n}\n\n")
            code += self._signature("launch_m_static", leading_m=True)
            code += ("\tif (Cfg::SCRATCH_BYTES * qf::kMGemvScratchRowBlocks > qf::kMGemvStaticScratchMax) {\n"
                     "\t\tfprintf(stderr, \"qfactory mgemv: this object needs %zu bytes of scratch memory, the static array holds at most %zu: call launch_m\\n\",\n"
                     "\t\t        (size_t)(Cfg::SCRATCH_BYTES * qf::kMGemvScratchRowBlocks), (size_t)qf::kMGemvStaticScratchMax);\n"
                     "\t\t__return_code = 1;\n\t\treturn;\n\t}\n"
                     "\tqf::MGemvScratch where;\n"
                     "\t__return_code = qf_static_scratch(where);\n"
                     f"\tif (__return_code == 0) __return_code = {call}({args}, m, (hipStream_t)_stream, qf::NormArgs{{}}, &where);\n}}\n\n")
        if self.input_prologue == "add_rmsnorm":
            # the entry point of this object (launch / launch_m return 1: they carry no norm operands)
            code += ('extern "C" void launch_norm (\n\tint m,\n\tvoid* _activation,\n\tvoid* _delta,\n\tvoid* _gamma,\n'
                     '\tvoid* _x_out,\n\tfloat eps,\n\tvoid* _weight,\n\tvoid* _output,\n\tvoid* _scale,\n\tvoid* _zero,\n'
                     '\tvoid* _stream,\n\tint& __return_code\n) {\n'
                     '\tqf::NormArgs norm;\n\tnorm.delta = (const uint16_t*)_delta;\n\tnorm.gamma = (const uint16_t*)_gamma;\n'
                     '\tnorm.x_out = (uint16_t*)_x_out;\n\tnorm.eps = eps;\n'
                     f'\t__return_code = _gamma == nullptr ? 1 : {call}({args}, m, (hipStream_t)_stream, norm);\n}}\n\n')
        desc = (f"regime={self.regime} M={p['M']} N={p['N']} K={p['K']} NBITS={p['NBITS']} GS={p['GS']} "
                f"SYM={int(p['SYM'])} decode={self.decode_strategy} nt_b={int(not self.l2cache_b)} "
                + ("act=bf16 " if self.act_dtype == torch.bfloat16 else "")
                + ("prologue=add_rmsnorm " if self.input_prologue == "add_rmsnorm" else "")
                + (f"epilogue={self.output_epilogue} " if self.output_epilogue != "none" else "")
                + ("smem_quant=1 " if self.smem_quant and self.regime == "gemv" and self.output_epilogue == "none" else "")
                + " ".join(f"{k}={v}" for k, v in sorted(t.items()))
                # the header knobs that change the generated code and are not named above
                + "".join(f" {k}={v}" for k, v in sorted(defines.items())
                          if k in TUNING_DEFINES and k != "QF_GEMM_FULL_DRAIN"))
        wait_desc = " QF_GEMM_WAIT_DESC" if self.regime == "gemm" else ""    # string literal from the header: counted / drain
        code += f'extern "C" const char* qf_describe() {{ return "{desc}"{wait_desc}; }}\n'
        return code


class MatmulQFunc(QFunc):
    """group_size == -1: activation (M,K) fp16 x raw unsigned low-bit weight (N,K) -> (M,N) fp16."""

    def __init__(self, qtile_a, qtile_b, layout):
        self.qtile_a, self.qtile_b, self.layout = qtile_a, qtile_b, layout
        assert qtile_a.quant_method == "none", "Quantization method not supported for A"
        assert qtile_b.quant_method == "none", "Quantization method not supported for B"
        assert layout == "nt", f"Layout {layout} is not supported"
        _problem_of(qtile_a, qtile_b)
        self.regime = "gemv"
        self.parallel_strategy = "row"
        self.tiling_configs = tiling.gemv_tiling(1, qtile_b.shape[0], qtile_b.shape[1], qtile_b.nbits, None)
        self.decode_strategy = "deferred"       # raw fields: there is no scale or zero-point to apply early
        self.l2cache_a = True
        self.l2cache_b = False
        assert qtile_a.dtype in (torch.float16, torch.bfloat16), f"Data type {qtile_a.dtype} is not supported for A"

    @property
    def act_dtype(self):
        return self.qtile_a.dtype

    @property
    def problem(self):
        return {"M": 1, "N": self.qtile_b.shape[0], "K": self.qtile_b.shape[1], "NBITS": self.qtile_b.nbits}

    def arg_name_type(self):
        return [
            ("m", int),
            ("activation", self.act_dtype), ("weight", torch.int8), ("output", self.act_dtype),
            ("stream", torch.cuda.streams.Stream),
        ]

    def schedule(self) -> List[QFunc]:
        return [self.clone(l2cache_a=a, l2cache_b=b) for a in (True, False) for b in (True, False)]

    def lower(self) -> List[QFunc]:
        p = self.problem
        return [self.clone(tiling_configs=c)
                for c in tiling.gemv_candidates(1, p["N"], p["K"], p["NBITS"], None)]

    def emit(self) -> str:
        p = self.problem
        t = self.tiling_configs
        b = lambda x: "true" if x else "false"
        if self.decode_strategy != "deferred":
            raise ValueError(f"decode_strategy {self.decode_strategy!r}: the group_size == -1 kernel has no scale or "
                             "zero-point to apply early (available: ['deferred'])")
        code = "// QFactory-HIP generated translation unit\n\n"
        if self.act_dtype == torch.bfloat16:
            code += "#define QF_IN_BF16 1\n#define QF_OUT_BF16 1\n"
        code += '#include "qf_gemv.hip.h"\n'
        code += '#if __has_include("qfactory_launch.h")\n#define QF_LAUNCH_PLAIN 1\n#include "qfactory_launch.h"\n#endif\n\n'
        code += (f"using Cfg = qf::GemvCfg<{p['NBITS']}, 0, false, false, {p['N']}, {p['K']}, "
                 f"{t['MT']}, {t['WK']}, {t['WN']}, {t['U']}, {t['STEPS']}, {t['VB']}, {b(not self.l2cache_b)}>;\n\n")
        code += self._signature("launch", leading_m=True)
        code += ("\t__return_code = qf::gemv_launch<Cfg>(_activation, _weight, _output, nullptr, nullptr, m, "
                 "(hipStream_t)_stream);\n}\n\n")
        desc = (f"regime=gemv-plain N={p['N']} K={p['K']} NBITS={p['NBITS']} nt_b={int(not self.l2cache_b)} "
                + ("act=bf16 " if self.act_dtype == torch.bfloat16 else "")
                + " ".join(f"{k}={v}" for k, v in sorted(t.items())))
        code += f'extern "C" const char* qf_describe() {{ return "{desc}"; }}\n'
        return code
