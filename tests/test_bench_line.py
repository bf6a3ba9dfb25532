"""The benchmark's stdout line: short enough for a harness that keeps a few KB of
stdout, valid JSON, and carrying the headline, roofline and CPU-baseline objects."""
import json

import bench


def _canned(n_configs):
    r = dict(entry="triton_rms_norm_and_block_quant_forward(output_mode=2) two passes", shape=[8192, 2048],
             algorithmic_bytes=68194304, algorithmic_bytes_read=33558528, algorithmic_bytes_written=34635776,
             us_per_call=18.184, us_per_call_min=18.001, us_per_call_max=18.9, timed_loops=7, preroll_calls=77,
             gb_per_s=3750.2, frac_of_hbm_peak=0.4688, us_per_call_hot=15.1, gb_per_s_hot=4516.2,
             us_single_call_median=20.4, us_single_call_trimmed_mean=20.5, buffer_sets=9,
             us_per_call_from_idle=18.57, stream_us=12.2, stream_gb_per_s=5590.0, frac_of_stream=0.6709,
             hbm_traffic_bytes=102400000.0, hbm_fetched_bytes=67500000.0, hbm_written_bytes=34900000.0,
             cpu_us_per_call=54000.0, cpu_threads=16)
    out = {}
    for i, name in enumerate(bench.ALL[:n_configs]):
        out[name] = dict(r, us_per_call=18.184 + i)
    return out


def test_headline_line_is_short_and_complete():
    results = _canned(len(bench.ALL))
    text = bench.encode_line(bench.headline_line(results, 20, 5, 1500.0))
    assert len(text) < bench.MAX_LINE_CHARS
    assert "\n" not in text
    line = json.loads(text)
    assert json.loads(json.dumps(line)) == line
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "preroll_calls",
                "us_per_call_from_idle"):
        assert key in line, key
    assert line["value"] == 18.184 and line["ms_per_step"] == round(18.184 / 1000, 6)
    assert set(line["roofline"]) >= {"bound", "achieved", "peak", "unit", "frac", "traffic", "copy_ceiling"}
    assert set(line["cpu_baseline"]) >= {"value", "unit", "cores", "kind", "sample"}
    assert "workload" in line["config"] and "model" not in line["config"]
    assert set(line["configs"]) == set(bench.ALL)
    assert all(len(v) == 3 for v in line["configs"].values())


def test_headline_line_sheds_extras_before_it_outgrows_the_window():
    results = _canned(len(bench.ALL))
    for i in range(300):  # far more configurations than the benchmark has
        results["extra_configuration_%03d" % i] = dict(results["cfg1"])
    text = bench.encode_line(bench.headline_line(results, 20, 5, 1500.0))
    assert len(text) < bench.MAX_LINE_CHARS
    line = json.loads(text)
    assert "roofline" in line and "cpu_baseline" in line and line["value"] == 18.184
