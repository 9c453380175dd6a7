"""The command line, started as a user would."""
import json
import os
import subprocess
import sys

import pytest

import plain_qwen3 as plain

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args, timeout=600):
    proc = subprocess.run([sys.executable, "-m", "nanohybrid_vlm_amd", *args], cwd=REPO, capture_output=True, text=True,
                          timeout=timeout)
    assert proc.returncode == 0, proc.stderr[-3000:]
    return proc.stdout


def test_random_model_command(tmp_path):
    out = str(tmp_path / "m")
    _run("random-model", "--out", out, "--shape", "tinyB", "--seed", "3")
    cfg, w = plain.read_model_folder(out)
    assert cfg["hidden_size"] == 96 and "lm_head.weight" in w
    assert plain.logits(cfg, w, [1, 2, 3]).shape == (3, 389)


@pytest.mark.gpu
def test_generate_and_bench_commands(model_folders, tmp_path):
    folder = model_folders["A"]
    cfg, w = plain.read_model_folder(folder)
    out = json.loads(_run("generate", "--model", folder, "--dtype", "float32", "--prompt-ids", "5 17 3", "--prompt-ids",
                          "9,8,7,6", "--output-tokens", "5", "--temperature", "0", "--ignore-eos", "--block-size", "8",
                          "--num-blocks", "16", "--max-model-len", "64", "--quiet"))
    assert [o["token_ids"] for o in out] == [plain.greedy_generate(cfg, w, p, 5) for p in ([5, 17, 3], [9, 8, 7, 6])]
    result = str(tmp_path / "bench.json")
    _run("bench", "--model", folder, "--cases", "16:2", "40:3", "--output-tokens", "6", "--repeats", "1",
         "--warmup-output-tokens", "2", "--token-budget", "32", "--block-size", "8", "--num-blocks", "64",
         "--max-model-len", "128", "--label", "tiny", "--mode", "graph", "--output", result)
    data = json.loads(open(result).read())
    assert len(data["results"]) == 2 and all(r["decode_tok_s"] > 0 and r["ttft_ms_mean"] > 0 for r in data["results"])
    out = _run("bench", "--model", folder, "--cases", "16:2", "--output-tokens", "4", "--repeats", "1", "--block-size", "8",
               "--num-blocks", "32", "--max-model-len", "64", "--mode", "eager", "--kernel-times")
    assert "nhv_paged_attention" in out or "nhv_decode_attention_bf16" in out
    assert "nhv_rmsnorm" in out and '"memory"' in out
    # random weights drawn on the device, and the prefix cache switched on
    out = json.loads(_run("generate", "--random-weights", "4", "--shape", "tinyB", "--prompt-ids", "5 17 3",
                          "--output-tokens", "4", "--temperature", "0", "--ignore-eos", "--block-size", "8", "--num-blocks",
                          "16", "--max-model-len", "64", "--enable-prefix-cache", "--quiet"))
    assert len(out[0]["token_ids"]) == 4


def test_model_or_random_weights_is_needed():
    proc = subprocess.run([sys.executable, "-m", "nanohybrid_vlm_amd", "generate", "--prompt-ids", "1"], cwd=REPO,
                          capture_output=True, text=True, timeout=120)
    assert proc.returncode != 0 and "--model DIR or --random-weights SEED" in proc.stderr


def test_bench_refuses_more_than_one_gpu():
    """The measurement program is for one GPU: for more it says so in one line and exits with 2."""
    proc = subprocess.run([sys.executable, os.path.join(REPO, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                          cwd=REPO, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 2
    assert len(proc.stdout.strip().splitlines()) == 1 and "one GPU" in proc.stdout


def _bench(*args, timeout=600):
    proc = subprocess.run([sys.executable, os.path.join(REPO, "bench.py"), *args], cwd=REPO, capture_output=True, text=True,
                          timeout=timeout)
    assert proc.returncode == 0, proc.stderr[-3000:]
    lines = [line for line in proc.stdout.splitlines() if line.startswith("{")]
    assert len(lines) == 1, proc.stdout[-2000:]
    return json.loads(lines[0]), proc.stdout


@pytest.mark.gpu
def test_bench_program_on_a_tiny_shape():
    """The measurement program's three kinds of run, on a tiny shape: the line's fields are there and add up."""
    line, _ = _bench("--shape", "tinyB", "--steps", "6", "--warmup", "2", "--batch", "3", "--prompt-tokens", "40",
                     "--context", "64", "--block-size", "16")
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points", "step_ms", "measured"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 6 and line["dtype"] == "bf16" and line["value"] > 0
    assert abs(line["value"] - 3 / (line["ms_per_step"] * 1e-3)) <= 0.01 * line["value"]
    config = line["config"]
    assert len(config) <= 20 and all(not isinstance(v, (dict, list)) for v in config.values())
    assert config["hidden"] == 96 and config["layers"] == config["layers_of_shape"] == 3 and config["vocab"] == 389
    assert set(line["prefill"]) == {"value", "tokens", "ms", "frac"} and line["prefill"]["tokens"] == 40
    roofline = line["roofline"]
    assert roofline["bound"] == "hbm" and roofline["peak"] == 8000.0
    assert abs(roofline["frac"] - roofline["achieved"] / roofline["peak"]) < 1e-3
    assert set(line["points"]) == {"decode_b1", "decode_b64"} and all(v > 0 for v in line["points"].values())
    # the timed window holds as many steps of GPU work as it counts: with steps issued ahead the mean over the window
    # and the median of the steps agree (a window that starts after a step issued ahead is done, and ends on a step
    # that issues none, would be one step short: 20/19 at 20 steps)
    line, _ = _bench("--shape", "0.6b", "--layers", "8", "--steps", "20", "--warmup", "5", "--batch", "8", "--prompt-tokens",
                     "512", "--context", "1024", "--no-points", "--no-measured-peaks")
    assert abs(line["ms_per_step"] - line["step_ms"]["p50"]) / line["step_ms"]["p50"] < 0.05, line
    # a serving workload: every request queued at once, prompts in portions beside decoding requests
    line, _ = _bench("--shape", "tinyB", "--workload", "serving", "--batch", "5", "--prompt-tokens", "150",
                     "--output-tokens", "8", "--block-size", "16", "--no-measured-peaks")
    assert line["value"] > 0 and line["points"]["decode_only_tok_s"] > 0 and len(line["config"]) <= 20
    # the diagnosis of a layer's products
    line, text = _bench("--shape", "tinyB", "--workload", "projections", "--batch", "1,5")
    assert set(line["table"]) == {f"{name}_m{m}" for name in ("qkv", "o", "gate_up", "down", "head") for m in (1, 5)}
    assert all(v["engine_us"] > 0 and v["read_us"] > 0 for v in line["table"].values())
    assert "a layer's four products at 5 rows" in text
