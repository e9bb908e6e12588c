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


def test_the_emitted_line_keeps_the_drivers_keys_and_types():
    """The JSON line as bench.py builds it (no device needed): the step count is an integer under "steps", the per-launch
    table has a key of its own, every key is there once, and the line survives a JSON round trip."""
    sys.path.insert(0, ROOT)
    import bench
    table = [dict(step="llama2 qkv + attention", us_per_launch=15.0, launches_per_token=32)]
    out = bench.bench_line(K=20, W=5, ms_per_step=1.25, tb=3.95e9, n_layers=32, distinct_layers=4, pos0=68, seq_len=512, form=0, step_times=table,
                           roofline=dict(bound="hbm", achieved=2400.0, peak=8000.0, unit="GB/s", frac=0.3, traffic=None),
                           cpu=dict(value=9.8, unit="tok/s", cores=16, kind="port", sample="x"))
    back = json.loads(json.dumps(out))
    assert isinstance(back["steps"], int) and back["steps"] == 20 and isinstance(back["warmup"], int) and back["warmup"] == 5
    assert back["step_times"] == table
    for key in ("metric", "value", "unit", "n_gpus", "ms_per_step", "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config",
                "roofline", "cpu_baseline", "config1", "config3", "config5"):
        assert key in back, key
    assert back["value"] == 800.0 and back["vs_baseline"] is None and "workload" in back["config"] and "model" not in back["config"]
    assert set(back["roofline"]) >= {"bound", "achieved", "peak", "unit", "frac", "traffic"}
    # no key twice in the source of the line: a later duplicate would silently replace the step count
    import ast
    import inspect
    tree = ast.parse(inspect.getsource(bench.bench_line))
    for node in ast.walk(tree):
        if isinstance(node, ast.Dict):
            keys = [k.value for k in node.keys if isinstance(k, ast.Constant)]
            assert len(keys) == len(set(keys)), keys
