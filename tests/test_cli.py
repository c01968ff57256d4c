"""The command line's host-side commands (no GPU)."""
import json
import os
import subprocess
import sys

import helpers

ROOT = os.path.normpath(os.path.join(os.path.dirname(__file__), ".."))


def run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bin", "deliverance"), *args], capture_output=True, text=True, timeout=300)


def test_random_then_inspect(tmp_path):
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(helpers.CONFIG_B))
    out = tmp_path / "model"
    p = run("random", "--config", str(cfg), "--seed", "7", "--out", str(out))
    assert p.returncode == 0, p.stderr
    assert (out / "config.json").exists() and (out / "model.safetensors").exists()
    p = run("inspect", str(out))
    assert p.returncode == 0, p.stderr
    assert "architecture GPT2LMHeadModel: 3 layers, width 96, vocabulary 1000, 96 positions" in p.stdout
    assert "h.2.mlp.c_fc.weight" in p.stdout and "[96, 200]" in p.stdout


def test_random_then_inspect_another_design(tmp_path):
    """The same commands on a Virudra configuration: the registry picks the design by config.json."""
    from virudra_models import CONFIG_Y
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(CONFIG_Y))
    out = tmp_path / "model"
    p = run("random", "--config", str(cfg), "--seed", "3", "--out", str(out))
    assert p.returncode == 0, p.stderr
    p = run("inspect", str(out))
    assert p.returncode == 0, p.stderr
    assert "architecture Virudra: 3 layers, width 96, vocabulary 200" in p.stdout and "3 layer calls, 3 cache slots" in p.stdout
    assert "l0.mlp.e2.down" in p.stdout and "l2.mlp.table" in p.stdout and "l1.mix.rel" in p.stdout and "[32, 2]" in p.stdout


def test_random_then_inspect_a_design_with_shared_weights_and_states(tmp_path):
    """... and on a Pedatar configuration: layers on another layer's weights store no tensors and keep a cache slot."""
    from pedatar_models import CONFIG_P
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(CONFIG_P))
    out = tmp_path / "model"
    p = run("random", "--config", str(cfg), "--seed", "4", "--out", str(out))
    assert p.returncode == 0, p.stderr
    p = run("inspect", str(out))
    assert p.returncode == 0, p.stderr
    assert "architecture Pedatar: 2 layers, width 64, vocabulary 300" in p.stdout and "4 layer calls, 4 cache slots" in p.stdout
    assert "l0.mix.dkv.norm" in p.stdout and "l1.mix.A_log" in p.stdout and "l1.mlp.shared.down" in p.stdout and "l2." not in p.stdout


def test_random_then_inspect_a_design_with_parallel_mixers(tmp_path):
    """... and on a Pafolorn configuration: a parallel layer keeps two cache slots, a delta rule's low ranks are named."""
    from pafolorn_models import CONFIG_F
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(CONFIG_F))
    out = tmp_path / "model"
    p = run("random", "--config", str(cfg), "--seed", "5", "--out", str(out))
    assert p.returncode == 0, p.stderr
    p = run("inspect", str(out))
    assert p.returncode == 0, p.stderr
    n = len(CONFIG_F["layers"])
    slots = sum(2 if L["type"] == "parallel" else 1 for L in CONFIG_F["layers"])
    assert f"architecture Pafolorn: {n} layers, width {CONFIG_F['width']}, vocabulary {CONFIG_F['vocab']}" in p.stdout
    assert f"{n} layer calls, {slots} cache slots" in p.stdout
    assert "l0.mix.left.q.norm" in p.stdout and "l0.mix.right.A_log" in p.stdout and "l0.ls1" in p.stdout and "embed.norm" in p.stdout


def test_random_then_inspect_a_design_with_a_loop_of_layers(tmp_path):
    """... and on a Salivik configuration: a looped layer stores its tensors once and keeps a cache slot a pass."""
    from salivik_models import CONFIG_S
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(CONFIG_S))
    out = tmp_path / "model"
    p = run("random", "--config", str(cfg), "--seed", "6", "--out", str(out))
    assert p.returncode == 0, p.stderr
    p = run("inspect", str(out))
    assert p.returncode == 0, p.stderr
    assert "architecture Salivik: 4 layers, width 64, vocabulary 300" in p.stdout and "8 layer calls, 8 cache slots" in p.stdout
    assert "loop.in" in p.stdout and "l1.mix.sink" in p.stdout and "l2.mix.g" in p.stdout and "l1.mlp.router.b" in p.stdout
    assert "l0.mix.v" in p.stdout and "l2.mix.v" not in p.stdout and "embed.norm" in p.stdout


def test_help_names_the_reference_options():
    p = run("generate", "--help")
    for opt in ("--model", "--working-dtype", "--max-tokens", "--temperature", "--seed", "--warmup-cases", "--max-cases",
                "--kv-context-rows-per-page", "--model-config", "--profile-stages", "--kernels", "--suite-file", "--output", "--jsonl-output"):
        assert opt in p.stdout
    p = run("generate", "--model", "/nonexistent")
    assert p.returncode != 0


def test_bench_measures_one_gpu_only():
    """With more than one GPU asked for, bench.py says so in one line and exits with 2."""
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert p.returncode == 2
    assert len(p.stdout.strip().splitlines()) == 1 and "--gpus 2" in p.stdout


def test_trace_run_without_a_gpu_says_so(tmp_path):
    """The replay program drives the GPU engine only: without a GPU it ends with a message, not a traceback."""
    import torch
    if torch.cuda.is_available():
        return
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(tmp_path), "--dtype", "float32",
                        "--out", str(tmp_path / "o"), "--max-tokens", "64"], input="", capture_output=True, text=True, timeout=300)
    assert p.returncode != 0 and "no GPU is visible" in p.stderr and "Traceback" not in p.stderr
