"""The one JSON line bench.py prints must stay small enough for a harness that keeps only the tail of stdout,
whatever the size of the tables behind it (those go to a side file)."""
import json
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import bench  # noqa: E402


def _dominant(kernel, bound="mfma"):
    return dict(bound=bound, achieved=114.09, peak=416.7, unit="TFLOP/s", frac=0.2738, traffic=None,
                peak_basis="bf16 matrix-core peak 2500 TFLOP/s / 6 term products per fp32 multiply",
                executed_bf16_tflops=684.5, frac_of_fp32_mfma_peak=0.7253, kernel=kernel, us=42.35,
                algorithmic_bytes=58937344, algorithmic_flops=4831838208, us_back_to_back=47.59, us_empty_event_pair=4.45)


def _net_config(name, densities, kernel):
    rows = {p: dict(ms_per_step=2.4918, frames_per_s=3210.5, repeats_ms=[2.5152] * 10, measured_pixel_density=0.01,
                    algorithmic_gflop_per_step=31.3, algorithmic_mb_per_step=253.0, hbm_frac_whole_step=0.0519,
                    dominant=_dominant(kernel)) for p in densities}
    return dict(workload=name, densities=rows, dense_same_kernels_ms=0.6094)


def canned_detail(n_layers=60, n_lossy=12):
    """A result of the shape bench.main() builds, with tables at least as long as a real run's."""
    conv_form = dict(us=8.1, algorithmic_bytes=3000000, algorithmic_flops=110000000, gbs=370.0, hbm_frac=0.0463,
                     tflops=13.6, active_pixels_in=4646, active_pixels_out=6000, active_tiles=230, tiles=1452)
    lossy_rows = [dict(method="exact", param=None, ms_per_step=0.624, speedup=1.0, mean_active_tile_fraction=0.9,
                       max_abs_deviation=0.0, mean_abs_deviation=0.0, stages={"layer%d" % i: 0.9 for i in range(16)})]
    for i in range(n_lossy):
        lossy_rows.append(dict(method="threshold", param=[1e-4, 1e-3, 1e-2, 3e-2, 1e-1][i % 5], ms_per_step=0.5 - 0.01 * i,
                               speedup=1.0 + 0.05 * i, mean_active_tile_fraction=0.5, max_abs_deviation=0.04,
                               mean_abs_deviation=0.004, stages={"layer%d" % j: 0.5 for j in range(16)}))
    return {
        "metric": "incremental frames/s + HBM GB/s, E2Depth-incr 264x352 @5% delta density",
        "value": 1745.2, "unit": "frames/s", "n_gpus": 1, "steps": 200, "warmup": 20, "ms_per_step": 0.573,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "E2Depth-incr recurrent UNet, random init, 1x5x264x352 event voxel deltas, 5% active "
                               "pixels, 1 dense refresh then incremental steps", "density": 0.05, "height": 264,
                   "width": 352, "batch": 1, "graph": True, "timing": "median of 10 repeats of 200 steps",
                   "f32_matmul": "bf16x3", "arithmetic": bench.ARITHMETIC["bf16x3"],
                   "mask_planning": "second stream, builds first"},
        "roofline": dict(_dominant("mie_upconv_masked up2x+5x5 s1 256->128 @66x88"), traffic=40120521),
        "cpu_baseline": dict(value=25.3, unit="frames/s", cores=16, kind="port", ms_per_step=39.5,
                             sample="400 incremental steps of the same E2Depth-incr 264x352 workload (dense F.conv2d on "
                                    "the delta, as the reference executes it), torch-CPU fp32"),
        "repeats_ms_per_step": [0.573] * 10,
        "whole_frame": dict(algorithmic_mb=258.5, algorithmic_gflop=53.3, hbm_gbs=451.0, hbm_frac=0.0564,
                            mfma_tflops=93.0, mfma_frac=0.2232, mfma_peak_tflops=416.7, sum_eager_launch_us=512.0),
        "f32_native_mfma": dict(ms_per_step=0.809, frames_per_s=1236.0),
        "dense_same_kernels_ms": 0.618, "speedup_vs_dense": 1.079,
        "density_sweep": {p: dict(ms_per_step=0.55, frames_per_s=1800.0) for p in ("0.01", "0.05", "0.20")},
        "refresh": dict(ms_eager=0.62, ms_graph=0.58),
        "lossy_frontier": dict(steps=50, exact_inline_ms_per_step=0.624, captured=True, note="x" * 150, reaches_5x=[],
                               points=lossy_rows),
        "configs": {
            "c1_single_conv3x3_32to32_264x352_d05": dict(delta_only=conv_form, fused_reservoir_relu=conv_form,
                                                         build_mask_tiles_us=5.7, dense_bytes=1, dense_flops=2),
            "c2_conv_leakyrelu_relu_64ch_132x176": {p: dict(us_per_step=21.0, algorithmic_bytes=1, gbs=100.0, hbm_frac=0.02)
                                                    for p in ("0.01", "0.05", "0.20")},
            "c4_evflownet_incr_256x256_transposed": _net_config("EVFlowNet-incr", ["0.03"], "mie_tconv2x_masked tconv 3x3 s2 128->32 @256x256"),
            "c4_evflownet_incr_256x256_upsample": _net_config("EVFlowNet-incr", ["0.03"], "mie_conv_masked 3x3 s1 128->32 @256x256"),
            "c5_e2depth_incr_bf16_8x480x640": _net_config("E2Depth-incr bf16", ["0.01", "0.20"], "mie_upconv_masked up2x+5x5 s1 64->32 @480x640"),
        },
        "output_check": dict(max_abs_diff=0.0, frames=4, steps_before=2230, against="same network, eager launches, inline mask planning"),
        "oracle_check": dict(max_abs_diff=1.8e-7, steps=3, rtol=1e-4, atol=1e-5, against="CPU oracle"),
        "layers": [dict(op="conv_masked", shape="up2x+5x5 s1 256->128 @66x88", us=74.3, gbs=204.0, tflops=128.0,
                        bytes=15156144, flops=9515827200, active_tiles=99, tiles=99) for _ in range(n_layers)],
    }


def test_line_is_short_and_parses():
    detail = canned_detail()
    assert len(json.dumps(detail)) > 20000           # the tables a real run carries do not fit a line
    text = bench.compact_line(detail, "gpurun_out/bench_detail.json")
    assert "\n" not in text and len(text) < bench.LINE_LIMIT <= 6000
    line = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in line, key
    assert line["value"] == detail["value"] and line["ms_per_step"] == detail["ms_per_step"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert line["roofline"][key] == detail["roofline"][key]
    assert line["roofline"]["frac"] == round(line["roofline"]["achieved"] / line["roofline"]["peak"], 4)
    assert line["cpu_baseline"] == detail["cpu_baseline"]
    assert "layers" not in line and "lossy_frontier" not in line and "repeats_ms_per_step" not in line
    # every configuration and density of the run is still named, reduced to time + roofline fraction
    cfg = line["configs"]
    assert cfg["c5_e2depth_incr_bf16_8x480x640@0.20"]["ms_per_step"] == 2.4918
    assert set(cfg["c1_single_conv3x3_32to32_264x352_d05/delta_only"]) == {"us", "frac", "bound", "kernel"}
    assert line["whole_frame"]["mfma_peak_tflops"] == line["roofline"]["peak"]      # one basis for both fractions
    assert line["oracle_check"]["steps"] == 3


def test_line_survives_oversized_tables():
    detail = canned_detail()
    for i in range(200):                              # a run with far more configurations than today's
        detail["configs"]["extra_%d" % i] = _net_config("x", ["0.05"], "k" * 60)
    text = bench.compact_line(detail, None)
    assert len(text) < bench.LINE_LIMIT
    line = json.loads(text)
    assert line["roofline"]["frac"] == detail["roofline"]["frac"] and line["cpu_baseline"] is not None


def test_line_of_a_minimal_run():
    detail = canned_detail()
    for key in ("f32_native_mfma", "density_sweep", "refresh", "lossy_frontier", "configs", "cpu_baseline", "oracle_check"):
        detail[key] = None
    detail["dense_same_kernels_ms"] = detail["speedup_vs_dense"] = None
    line = json.loads(bench.compact_line(detail, None))
    assert line["cpu_baseline"] is None and line["value"] == detail["value"]
