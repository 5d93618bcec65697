"""The benchmark's command-line contract: more than one GPU is refused with a message (CPU), and one short run prints
ONE JSON line carrying the agreed keys, the roofline of the dominant kernel and the CPU baseline (GPU)."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "one GPU" in r.stderr and r.stdout.strip() == ""


@pytest.mark.gpu
def test_one_json_line_with_roofline_and_cpu_baseline():
    print("\n[case] bench.py --steps 20 --warmup 3", flush=True)
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "20", "--warmup", "3"], capture_output=True, text=True,
                       timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 20 and d["warmup"] == 3 and d["vs_baseline"] is None and d["higher_is_better"] is False
    assert d["unit"] == "us/layer" and abs(d["value"] - d["ms_per_step"] * 1e3) < 1e-6 and "config2" in d["config"]["workload"]
    rf = d["roofline"]
    assert rf["bound"] == "hbm" and rf["peak"] == 8000.0 and rf["unit"] == "GB/s" and abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-9
    assert 0.3 < rf["frac"] < 1.0 and rf["traffic"] is not None
    cb = d["cpu_baseline"]
    assert cb["kind"] == "port" and cb["cores"] >= 1 and cb["value"] > d["value"] and "sample" in cb
    assert d["graph_replay_matches_eager"] is True
    # the other named configurations, the decoder step and the patched transformers model ride on the same line
    assert set(d["other_configs"]) == {"config1", "config3", "config4"}
    for name, o in d["other_configs"].items():
        for key in ("us_per_layer", "hbm_frac_step", "speedup_vs_dense", "roofline", "graph_replay_matches_eager"):
            assert key in o, (name, key)
        assert 0.05 < o["roofline"]["frac"] < 1.0 and 0.0 < o["hbm_frac_step"] < 1.0 and o["graph_replay_matches_eager"] is True
    dec = d["decoder_config3"]
    for key in ("tokens_per_s", "ms_per_step", "generation_loop_ms"):
        assert dec[key] > 0
    hf = d["patched_transformers_model_config3"]
    assert hf["ms_per_token_step"] > 0 and "patched_preallocated_us_per_layer" in hf["per_layer_slope"]
    assert hf["workload"].startswith("config3 ") and "B=4 " in hf["workload"]
    assert "patched_preallocated_attention_module_only_us_per_layer" in hf["per_layer_slope"]
    # a left-padded batch is timed next to it (the difference of two short runs: no ratio is asserted on it)
    assert hf["per_layer_slope"]["patched_left_padded_batch_us_per_layer"] > 0
    assert hf["per_layer_slope"]["patched_dynamic_cache_adopted_us_per_layer"] < 0.5 * hf["per_layer_slope"]["patched_dynamic_cache_us_per_layer"]
    assert d["paged_cache_identity_table"]["same_bits_as_unpaged"] is True
    for rows in ("rows_8", "rows_64"):
        assert 0.2 < d["chunked_decode"][rows]["gather_hbm_frac_of_whole_chunk_step"] < 1.0
