"""The engine's HIP kernels on the CPU: the kernel sources compiled for the host and run thread by
thread (tests/simt), every operand of every kernel call between protected pages.  An access outside
an operand ends the child process with a message that names the kernel, the workgroup, the thread
and the operand.  The children run the GPU test files themselves (the same cases, with CPU tensors),
so what the GPU tests cover for results, these runs cover for addresses.

Set DELIVERANCE_SIMT_FULL=1 to run everything the simulated kernels can run (a quarter of an hour
on 8 cores); the default is a selection that takes about a minute.
"""
import os
import subprocess
import sys

import pytest

from simt import harness

pytestmark = pytest.mark.skipif(not harness.available(), reason="needs clang++ on x86-64 Linux")
FULL = os.environ.get("DELIVERANCE_SIMT_FULL") == "1"

# name -> pytest arguments of the child.  The default selection: the cases marked for it in the GPU test files
# (simt_quick, or simt_a and simt_b where two parameter lists cross).
QUICK = "gpu and (simt_quick or (simt_a and simt_b))"
RUNS = {
    # the regression for the block-tile product's loads past K with K below one slab (K = 24, 65 rows and more)
    "tile_product_small_k": ["tests/test_kernels_gpu.py", "-k", "matrix_cores and 50-24", "-n", "2"],
    "kernels": ["tests/test_kernels_gpu.py", "-n", "4"] + ([] if FULL else ["-m", QUICK]),
    "parts": ["tests/test_parts_gpu.py"],
    # another design's kernels and parts (norms, attention with a bias by distance, gated and expert feed-forwards)
    # and one of its models through the step function
    "virudra": ["tests/test_virudra_gpu.py", "-n", "4"] if FULL else
               ["tests/test_virudra_gpu.py", "-n", "3", "-k",
                "(rms_norm_kernels and 64) or (every_edge and bfloat16) or (experts_feed_forward_part and (64-24 or 300) and bfloat16) "
                "or (gated_feed_forward_part and 64-40) or (attention_with_bias and bfloat16 and 4-2-16-16) or softcap "
                "or (whole_prompts and Z and bfloat16)"],
    # a third design's kernels and parts (rotation, latent attention on its plain and matrix-core forms, the short
    # filter and the scan, routed experts) and two of its models through the step function
    "pedatar": ["tests/test_pedatar_gpu.py", "-n", "4"] if FULL else
               ["tests/test_pedatar_gpu.py", "-n", "3", "-k",
                "rotation or filter or router_takes or (squared_ramp and bfloat16) or (routed_feed_forward and bfloat16 and not 300) "
                "or (selective_scan and bfloat16) or (far_key and 31 and bfloat16) or (latent_attention_part and bfloat16 and m0) "
                "or (whole_prompts and (P or R) and bfloat16) or (mixed_batches and R and bfloat16)"],
    # a fourth design's kernels and parts (the gated delta rule, its read-out norm, the norm and turn of queries and
    # keys, attention over a window with kept first keys on its plain and matrix-core forms, parallel mixers) and its
    # models through the step function
    "pafolorn": ["tests/test_pafolorn_gpu.py", "-n", "4"] if FULL else
                ["tests/test_pafolorn_gpu.py", "-n", "3", "-m", QUICK, "-k",
                 "not token_by_token and not (mixed_batches and (F or G)) and not (portions and sizes0)"],
    # a fifth design's kernels and parts (retention, attention whose keys are its values with a term without a key and
    # an output gate, latent attention with a window and a learned sink, capped gated feed-forwards, a router that
    # weighs the chosen logits among themselves) and its models through the step function
    "salivik": ["tests/test_salivik_gpu.py", "-n", "4"] if FULL else
               ["tests/test_salivik_gpu.py", "-n", "3", "-m", QUICK, "-k",
                "not (portions and sizes0) and not token_by_token and not (mixed_batches and (S or float32)) "
                "and not ((portions or whole_prompts) and S and float32)"],
    "replay": ["tests/test_replay_gpu.py", "-n", "4"] if FULL else
              ["tests/test_replay_gpu.py", "-n", "2", "-k", "(mixed and (A or B) and not 32) or want_subset or errors_leave or first_tokens"],
    # inner sizes of 32 in an engine step: qkv and fc of seed 11 (and, in the full run, proj of seed 5)
    "random_configurations": ["tests/test_random_configs_gpu.py", "-n", "4"] if FULL else
                             ["tests/test_random_configs_gpu.py", "-k", "11"],
}
if FULL:
    RUNS["toy_parts"] = ["tests/test_toy_parts_gpu.py", "tests/test_toy_parts2_gpu.py", "-n", "4"]
    RUNS["engine_paths"] = ["tests/test_engine_paths_gpu.py", "-n", "4"]


@pytest.fixture(scope="module")
def children():
    """All children start together (they are independent processes) and are waited for one by one."""
    harness.build()
    env = dict(os.environ)
    env["DELIVERANCE_SIMT"] = "1"
    procs = {}
    for name, args in RUNS.items():
        marks = [] if "-m" in args else ["-m", "gpu"]
        procs[name] = subprocess.Popen([sys.executable, "-m", "pytest", "-x", "-q", *marks, "-p", "no:cacheprovider",
                                        "-s", *args], cwd=harness.REPO, env=env, stdout=subprocess.PIPE,
                                       stderr=subprocess.STDOUT, text=True)
    yield procs
    for p in procs.values():
        if p.poll() is None:
            p.kill()


@pytest.mark.parametrize("name", sorted(RUNS))
def test_simulated_kernels_stay_inside_their_operands(children, name):
    p = children[name]
    out, _ = p.communicate(timeout=3000 if FULL else 900)
    assert p.returncode == 0, f"simulated run '{name}' ended with status {p.returncode}:\n{out[-3000:]}"
    assert " passed" in out and " failed" not in out, out[-2000:]
