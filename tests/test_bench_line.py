"""The line bench.py prints on stdout stays small and complete, whatever the sections hold (no GPU needed)."""
import json
import re

import bench


def _canned_full():
    kernel = "regime=gemv M=1 N=22016 K=4096 NBITS=4 GS=128 SYM=0 decode=deferred nt_b=1 " + "X=1 " * 40
    shapes = [{"name": n, "N": N, "K": K, "M": 1, "us": 9.123, "GB/s": 5123.4, "TFLOP/s": 19.876, "hbm_frac": 0.6404,
               "bytes": 46902272, "kernel": kernel, "stream_read_us": 8.123, "frac_of_stream_read": 0.8904,
               "module_us": 9.5, "module_out_us": 9.4} for n, N, K in bench.SHAPES]
    gemm = [{"name": n, "N": N, "K": K, "M": 256, "us": 230.41, "TFLOP/s": 1043.8, "mfma_frac": 0.4148, "GB/s": 1204.9,
             "hbm_frac": 0.1506, "dense_fp16_us": 260.12, "speedup_over_dense_fp16": 1.129, "kernel": kernel}
            for n, N, K in bench.GEMM_SHAPES]
    small = [{"config": "configs[2]", "M": M, "N": 8192, "K": 8192, "bits": b, "sym": sym, "us": 14.583, "GB/s": 2426.8,
              "hbm_frac": 0.3034, "TFLOP/s": 147.27, "kernel": kernel}
             for M in (1, 4, 16) for b in (2, 3, 4, 8) for sym in (False, True)] * 2
    decode = [{"batch": b, "value": 15732.3456, "decode_step_us": 4068.123, "quantized_linear_share": 0.56789,
               "quantized_linears_us_per_step": 2301.0, "prefill_tokens_per_s": 70494.4, "unit": "tokens/s"} for b in (1, 16, 64)]
    cpu = {"value": 0.1417, "unit": "GB/s", "cores": 16, "kind": "port", "sample": "s" * 160, "dequant_matmul_ms": 743.09,
           "matmul_only_ms": 41.5, "matmul_only_GB/s": 2.5, "cpu_model": "AMD EPYC 9575F 64-Core Processor", "host_cpus": 16,
           "shapes": [{"name": n, "dequant_matmul_us": 1.0} for n, _, _ in bench.SHAPES]}
    return {
        "metric": "W4A16 g128 GEMV (M=1) algorithmic HBM throughput over the Llama-2-7B linear shapes",
        "value": 4193.2, "unit": "GB/s", "n_gpus": 1, "steps": 20, "warmup": 5, "ms_per_step": 0.02508,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "w" * 200, "bits": 4, "group_size": 128, "M": 1, "weight_copies": 8,
                   "bytes_per_step": 105270000, "timed_with": "one HIP graph of all steps"},
        "hbm_frac_whole_step": 0.5242,
        "roofline": {"bound": "hbm", "achieved": 5123.4, "peak": 8000.0, "unit": "GB/s", "frac": 0.6404, "traffic": 47041000,
                     "traffic_source": "t" * 90, "kernel": "qf::gemv_kernel gate_up N=22016 K=4096 M=1", "avg_launch_us": 9.123,
                     "algorithmic_bytes_per_launch": 46902272,
                     "empirical": {"stream_read_GB/s": 5650.1, "stream_read_us": 8.3, "frac_of_stream_read": 0.9,
                                   "what": "w" * 80, "dense_fp16_TFLOP/s": 1090.5, "dense_fp16_what": "d" * 70}},
        "shapes": shapes, "parity": {"max_rel": 0.00048828125, "nrms": 0.00012345678, "mse": 1.2345678e-6},
        "gemm_m256": {"peak_TFLOP/s": 2516.6, "dense_fp16_TFLOP/s_measured": 1090.5, "shapes": gemm},
        "gemm_m32_m64_m128": gemm * 3, "gemm_prefill_m8192": gemm, "small_m": small, "decode": decode, "cpu_baseline": cpu,
        "report_file": "gpurun_out/bench_report.json",
    }


def test_stdout_line_is_compact_and_complete():
    full = _canned_full()
    text = json.dumps(bench.compact_line(full), separators=(",", ":"))
    assert len(text) < 4096, len(text)
    assert "\n" not in text
    line = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in line, key
    assert "workload" in line["config"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in line["roofline"], key
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in line["cpu_baseline"], key
    assert len(line["gemm_m256"]) == 4 and len(line["decode"]) == 3 and len(line["shapes"]) == 4
    assert "kernel" not in line["shapes"][0]


def test_stored_traffic_figure_is_for_the_dominant_kernel_as_built_now():
    """bench.py exits when MEASURED_TRAFFIC has no entry for the dominant kernel's description; a changed default
    tiling must be caught here, not on the GPU."""
    import torch
    from qfactory.core.qfunc import QMatmulQFunc
    from qfactory.core.qtile import AsymQTile, QTile
    name, N, K = next(s for s in bench.SHAPES if s[0] == bench.DOMINANT)
    qfunc = QMatmulQFunc(QTile((1, K), torch.float16, 16), AsymQTile((N, K), torch.int8, bench.NBITS, (1, bench.GS)), "nt")
    description = re.search(r'qf_describe\(\) \{ return "([^"]*)"', qfunc.emit()).group(1)
    assert description in bench.MEASURED_TRAFFIC, description
