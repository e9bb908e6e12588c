"""bench.py's command-line contract that can be checked without a GPU."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "1"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "ONE GPU" in r.stderr
    assert r.stdout.strip() == ""


def test_token_bytes_formula_matches_the_published_roofline():
    sys.path.insert(0, ROOT)
    import bench
    cfg = bench.CFG
    # packed weights of the 7B Q4_K_M-style model (Q6_K v-proj and output) + norm vectors, positions 64..319, fp16 cache
    tb = bench.token_bytes(cfg, 3888685056 + 1064960, 64, 319)
    assert abs(tb - 3.991e9) < 0.01e9
    assert abs(bench.HBM_PEAK_GBS * 1e9 / tb - 2004) < 5


def test_step_bytes_add_up_to_the_token():
    """The per-launch algorithmic bytes bench.py prices the steps of a layer with, summed over a token, are the token's
    bytes (weights, vectors, cache rows) to within the vectors the per-token formula leaves out (< 0.5 %)."""
    sys.path.insert(0, ROOT)
    import bench
    cfg = bench.CFG
    sb = bench.step_bytes(cfg, 191)
    per_layer = sum(sb[k] for k in ("llama2 qkv + attention", "llama2 attn_output", "llama2 ffn gate/up", "llama2 ffn_down"))
    total = 32 * per_layer + sb["llama2 output"]
    tb = bench.token_bytes(cfg, 3888685056 + 1064960, 191, 191)
    assert abs(total - tb) / tb < 0.005, (total, tb)
    assert sb["llama2 ffn gate/up"] == 50801664 + 1024      # the figure the gate/up profile is quoted on, + the sums of 16
