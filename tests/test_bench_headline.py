"""The line that bench.py prints last on stdout stays short enough for a log capture to keep it
whole, whatever the run measured: the summary is built here from a detail record with every
benchmark row a full run produces (values made up, keys and counts as bench.py writes them)."""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402  (imports nothing of torch or of the HIP library at module level)


def _linear_row(m, n, k, kernel, bound):
    r = {"m": m, "n": n, "k": k, "layout": "[n_out, k_in]", "n_sets": 64, "us": 123.456789, "weight_gbs": 3456.789012,
         "hbm_frac": 0.43209876, "tflops": 1234.56789, "mfma_frac": 0.4938271}
    r["roofline"] = (bench.hbm_roofline(kernel, 37748736.0, 0.0123456) if bound == "hbm" else bench.mfma_roofline(kernel, 2.7e11, 0.27))
    return r


def _stack(m):
    modes = ("per_launch_graph", "sequence_sequential_block", "sequence_parallel_block", "sequence_parallel_block_fused_qkv",
             "sequence_parallel_block_fused_qkv_ffn_first", "sequence_parallel_block_fused_qkv_ffn_first_streaming_layout",
             "sequence_decoder_data_flow", "sequence_decoder_data_flow_streaming_layout",
             "sequence_decoder_data_flow_joint_output_streaming_layout", "sequence_decoder_data_flow_two_entries_streaming_layout",
             "sequence_no_waits", "sequence_no_waits_streaming_layout", "default_layout_graph", "default_layout_sequence",
             "streaming_layout_two_entries_graph")
    r = {"m": m, "entries": 168, "weight_bytes": 3170893824.0}
    for i, mode in enumerate(modes):
        r[mode] = {"us_per_pass": 1234.56789 - i, "weight_gbs": 2568.123456, "hbm_frac": 0.32101234, "status": 0, "waits_per_pass": 84,
                   "roofline": bench.hbm_roofline("gemv_mfma_kernel / gemv_stream_single_kernel (168 launches)", 3170893824.0, 1.2345),
                   "max_error_vs_single_call": 0.000123456}
    return r


def full_detail():
    shapes = ((4096, 4096), (16384, 4096), (4096, 16384))
    extra = {
        "calibrate_copy": {"bytes_read": 1 << 27, "bytes_written": 1 << 27, "us": 52.123456, "gbs": 5151.123456},
        "gpu_equals_cpu_baseline_bits": True,
        "decompress_transposed": {"rows": 4096, "cols": 16384, "us": 26.3456789, "gbs": 6531.123456, "hbm_frac": 0.81612345,
                                  "roofline": bench.hbm_roofline("decompress_transposed_tile_kernel", 171966464.0, 0.0263)},
        "gemv": [_linear_row(m, n, k, "gemv_mfma_kernel / gemv_stream_single_kernel", "hbm") for n, k in shapes for m in (1, 8)],
        "gemv_streaming_layout": [_linear_row(m, n, k, "gemv_mfma_kernel (streaming layout)", "hbm") for n, k in shapes for m in (1, 8)],
        "linear_kn": [_linear_row(m, n, k, "gemv_kn_kernel", "hbm") for n, k in shapes for m in (1, 8)]
        + [_linear_row(128, 16384, 4096, "gemm_kn_tile_kernel", "mfma")],
        "linear_knp": [_linear_row(m, n, k, "gemv_knp_kernel", "hbm") for n, k in shapes for m in (1, 8)]
        + [_linear_row(m, 16384, 4096, "gemm_pipe2_kn_kernel", "mfma") for m in (128, 512, 2048)],
        "gemm": [_linear_row(m, 16384, 4096, "gemm_pipe2_kernel", "mfma") for m in (128, 512, 2048)],
        "gemm_streaming_layout": [_linear_row(m, 16384, 4096, "gemm_pipe2_kernel (streaming layout)", "mfma") for m in (128, 512, 2048)],
        "gemm_other_shapes": [_linear_row(512, 4096, 4096, "gemm_pipe2_kernel", "mfma") for _ in range(7)],
        "stack": [_stack(m) for m in (1, 4, 8, 16)],
        "bench_wall_s": 123.4,
    }
    for key in ("compress", "compress_f32"):
        extra[key] = {"rows": 4096, "cols": 16384, "input": "float16", "us": 30.6123456, "bytes": 171966464.0, "gbs": 5614.123456,
                      "hbm_frac": 0.70123456, "roofline": bench.hbm_roofline("compress_kernel", 171966464.0, 0.0306)}
    return {
        "metric": "decompress GB/s & %HBM peak; fused dequant-GEMV/GEMM GB/s, TFLOP/s, %roofline",
        "value": 6875.1, "unit": "GB/s", "n_gpus": 1, "steps": 200, "warmup": 20, "ms_per_step": 0.025013024806976317,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "standalone int4->fp16 decompress, 4096x16384, group_size 64, N(0,0.02) + 0.1% outliers at 8 sigma, "
                   "4 rotating buffer sets (688 MB > last-level cache)", "rows": 4096, "cols": 16384, "group_size": 64},
        "roofline": {"bound": "hbm", "achieved": 6875.1, "peak": 8000.0, "unit": "GB/s", "frac": 0.8594, "traffic": 172268442,
                     "traffic_source": "profiles/decompress_kernel_4096x16384.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE at commit 0123456789ab)",
                     "kernel": "decompress_kernel", "algorithmic_bytes_per_launch": 171966464.0},
        "cpu_baseline": {"value": 0.2785381184491455, "unit": "GB/s", "cores": 1, "kind": "port",
                         "sample": "numpy decompress of one 4096x16384 weight (group 64), best of 3, 0.617 s; host has 256 cpus, "
                         "256 usable, numpy elementwise = 1 thread",
                         "legs": [{"workload": "config 3: numpy decompress -> float32 matmul, m=1 [16384x4096]", "seconds": 1.234,
                                   "value": 0.0305, "unit": "GB/s (packed weight bytes)", "tflops": 0.0001, "cores": "decompress 1, BLAS 16"}] * 4},
        "extra": extra,
    }


def test_headline_is_short_and_complete():
    detail = full_detail()
    assert len(json.dumps(detail)) > 3 * bench.HEADLINE_LIMIT  # (the detail itself is what no longer fits a line)
    head = bench.headline(detail)
    line = json.dumps(head, separators=(",", ":"))
    assert len(line) < bench.HEADLINE_LIMIT, len(line)
    assert "\n" not in line
    back = json.loads(line)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "roofline", "cpu_baseline", "extra"):
        assert key in back, key
    assert back["value"] == detail["value"] and back["ms_per_step"] == detail["ms_per_step"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert back["roofline"][key] == detail["roofline"][key]
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert back["cpu_baseline"][key] == detail["cpu_baseline"][key]
    assert "legs" not in back["cpu_baseline"]
    # one short record per benchmark shape of configurations 3, 4 and 5
    assert len(back["extra"]["c3_gemv"]) == 6 and len(back["extra"]["c3_gemv_default_layout"]) == 6
    assert len(back["extra"]["c3_gemv_streaming_layout"]) == 6
    assert "c3_gemv_default_layout_variables" not in back["extra"]  # (the kernels on the default layout's variables: detail file only)
    assert [r["m"] for r in back["extra"]["c4_gemm"]] == [128, 512, 2048]
    assert [r["m"] for r in back["extra"]["c4_gemm_default_layout"]] == [128, 512, 2048]
    assert [r["m"] for r in back["extra"]["c4_gemm_streaming_layout"]] == [128, 512, 2048]
    assert [r["m"] for r in back["extra"]["c5_stack"]] == [1, 4, 8, 16]
    for r in back["extra"]["c5_stack"]:
        assert set(r) >= {"decoder", "no_waits", "per_launch_graph"}
        assert r["decoder"]["schedule"] == "streaming_layout_two_entries_graph"  # (the fastest of the made-up rows)


def test_emit_prints_the_headline_last(tmp_path, capsys):
    detail = full_detail()
    path = tmp_path / "out" / "detail.json"
    bench.emit(detail, str(path))
    captured = capsys.readouterr()
    lines = captured.out.strip().split("\n")
    assert len(lines) == 1 and len(lines[0]) < bench.HEADLINE_LIMIT
    assert json.loads(lines[0])["extra"]["detail_file"] == str(path)
    assert json.load(open(path))["extra"]["stack"][0]["entries"] == 168  # every figure is in the file ...
    assert "sequence_sequential_block" in captured.err  # ... and on stderr


def test_headline_without_optional_parts():
    detail = full_detail()
    detail["cpu_baseline"] = None
    detail["extra"] = {"bench_wall_s": 1.0}
    head = bench.headline(detail)
    assert head["cpu_baseline"] is None and head["extra"] == {"bench_wall_s": 1.0}
