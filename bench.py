#!/usr/bin/env python3
"""Decode benchmark: Llama-2-7B-shape, Q4_K_M-style weights (Q4_K; Q6_K for v-proj and output),
fp16 KV cache, batch 1 -- BASELINE configuration 4.

One "step" = one token through the whole layer stack (greedy decode loop on the device).  The
64 prompt positions of the configuration are always processed first, untimed (62 of them in chunks
through slai_llama2_prefill); then W = --warmup tokens are decoded untimed (the first of them from the
last prompt token: the reference excludes the first generated token as well), and the next K = --steps
generated tokens are timed with HIP events on the library's stream, with inputs and weights resident
in HBM.  The default W = 1, K = 256 times exactly the positions the metric is quoted on (64 .. 319).
Prints ONE JSON line.

Also measured here:
  * roofline: the dominant kernel.  When the model takes the one-launch-per-token form, that launch IS
    the token (every layer and the output matrix): achieved = the token's algorithmic bytes / the
    launch's mean duration inside the timed loop.  Otherwise the two largest kernels of a token are
    timed alone with HIP events while rotating over enough distinct weight copies to defeat the
    256 MB Infinity Cache.  peak = 8 TB/s.
  * cpu_baseline: the CPU oracle (a C restatement of the reference's CPU path) on the host cores:
    configuration 1 in full on one thread (the reference's CPU path is single-threaded) and on all
    cores, and a bounded sample of the headline shapes (depth 2 and 6, a few tokens) extrapolated to
    32 layers.  A reported baseline, not the target.
  * config1, config3, config5: the other decode configurations through the same C ABI (tiny Llama and the
    GPT-2-small shape in full; the long-context one with attention and GEMV rates apart).
"""
import argparse
import math
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
TRAFFIC_PROFILE = os.path.join("profiles", "gate_up_gemv_q4k_hbm_counters.md")
RESIDENT_TRAFFIC_PROFILE = os.path.join("profiles", "resident_decode_llama2_7b_q4k_hbm_counters.md")


def dominant_kernel_traffic():
    """HBM bytes one launch of the dominant kernel moves, read from the committed counter summary (rocprofv3 FETCH_SIZE +
    WRITE_SIZE per dispatch of `bench.py --probe`, each scaled by what the same counter reads for the probe's 64 MiB copy
    kernel): the bold `= **N B**` figure of that file, or None when the file is not there."""
    import re
    try:
        m = re.search(r"=\s*\*\*(\d+) B\*\*", open(os.path.join(ROOT, TRAFFIC_PROFILE)).read())
        return int(m.group(1)) if m else None
    except OSError:
        return None


def resident_kernel_traffic():
    """The same for the resident launch of a whole token (`bench.py --probe-resident` under the counters)."""
    import re
    try:
        m = re.search(r"=\s*\*\*(\d+) B\*\*", open(os.path.join(ROOT, RESIDENT_TRAFFIC_PROFILE)).read())
        return int(m.group(1)) if m else None
    except OSError:
        return None


CFG = dict(dim=4096, hidden_dim=11008, n_layers=32, n_heads=32, n_kv_heads=32, vocab=32000)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def token_bytes(cfg, weight_bytes, pos_lo, pos_hi, kv_bytes=2):
    """Algorithmic HBM bytes per token: packed weights + norm vectors (both in weight_bytes) +
    KV read 2*L*(pos+1)*kv_dim*kv_bytes averaged over the timed positions + KV write."""
    kv_dim = cfg["dim"] * cfg["n_kv_heads"] // cfg["n_heads"]
    mean_t = (pos_lo + pos_hi) / 2.0 + 1.0
    kv_read = 2 * cfg["n_layers"] * mean_t * kv_dim * kv_bytes
    kv_write = 2 * cfg["n_layers"] * kv_dim * kv_bytes
    return weight_bytes + kv_read + kv_write


BLOCK_BYTES = {12: (144, 256), 14: (210, 256), 8: (34, 32), 13: (176, 256), 2: (18, 32)}      # ggml type: bytes per block, weights per block


def packed_bytes(ggml_type, nrows, ncols):
    b, w = BLOCK_BYTES[ggml_type]
    return nrows * ncols // w * b


def step_bytes(cfg, pos, kv_bytes=2):
    """Algorithmic HBM bytes of one launch of each step of a layer (and of the output matrix) in the headline model: packed
    weights + the vectors read and written (+ the cache rows 0..pos and the new row for the launch that holds the attention)."""
    d, h, v = cfg["dim"], cfg["hidden_dim"], cfg["vocab"]
    kv_dim = d * cfg["n_kv_heads"] // cfg["n_heads"]
    vec = 4 * d + 4 * d // 16                                   # a weighted activation vector and its sums of 16
    return {
        "llama2 qkv + attention": packed_bytes(12, d, d) + packed_bytes(12, kv_dim, d) + packed_bytes(14, kv_dim, d) + 4 * d + vec
                                  + 2 * (pos + 1) * kv_dim * kv_bytes + 4 * d,
        "llama2 attn_output": packed_bytes(12, d, d) + 4 * d + 8 * d + vec,
        "llama2 ffn gate/up": 2 * packed_bytes(12, h, d) + 4 * d + vec + 4 * h,
        "llama2 ffn_down": packed_bytes(12, d, h) + 4 * h + 8 * d + vec,
        "llama2 output": packed_bytes(14, v, d) + 4 * d + vec + 4 * v,
    }


def measure_dominant_kernel(backend, reps=20):
    """Mean launch duration of the fused gate/up GEMV (Q4_K, 11008x4096 twice) over distinct copies, launched the way
    the decode loop launches it: 64-row-tile layout, activations in the prepared form left by the preceding GEMV."""
    from slai_amd import _ffi, synth
    from slai_amd.runtime import GpuQuantMatrix, GpuTensor, LlmContext
    dim, hid, t = CFG["dim"], CFG["hidden_dim"], 12
    ncopies = 8                                     # 8 x 50.7 MB = 406 MB > 256 MB Infinity Cache
    base = synth.normal_quantized(4242, t, hid, dim, 0.02)
    rb = base.size // hid
    mats = []
    for i in range(2 * ncopies):
        mats.append(GpuQuantMatrix(backend, t, hid, dim, np.roll(base.reshape(hid, rb), i + 1, axis=0), layout=_ffi.LAYOUT_TILE64))
    x = GpuTensor.vector(backend, synth.normal(7, dim, 1.0))
    w = GpuTensor.vector(backend, np.ones(dim, np.float32))
    hb = GpuTensor(backend, hid)
    prep = GpuTensor(backend, dim + dim // 16)
    ctxt = LlmContext(backend)
    ctxt.rms_norm_prepare(prep, x, w)
    for i in range(ncopies):
        ctxt.ffn_gate_up_silu_prepared(hb, mats[2 * i], mats[2 * i + 1], x, prep, 1e-5)
    backend.synchronize()
    backend.timer_begin()
    for _ in range(reps):
        for i in range(ncopies):
            ctxt.ffn_gate_up_silu_prepared(hb, mats[2 * i], mats[2 * i + 1], x, prep, 1e-5)
    ms = backend.timer_end() / (reps * ncopies)
    algo = 2 * mats[0].device_bytes() + dim * 4 * 2 + hid * 4     # 2 packed matrices + x + its weighted copy + out
    for o in mats + [x, w, hb, prep]:
        o.destroy()
    return ms, algo


def counter_probe(backend):
    """For hardware-counter runs: 64 launches of a plain copy kernel of known size (64 MiB read, 64 MiB
    written) and the dominant-kernel loop, nothing else, so that per-dispatch FETCH_SIZE / WRITE_SIZE of
    the GEMV can be scaled by what the same counter reads for the copy."""
    from slai_amd.runtime import GpuTensor, LlmContext
    n = 16 * 1024 * 1024
    a = GpuTensor(backend, n)
    b = GpuTensor(backend, n)
    ctxt = LlmContext(backend)
    for _ in range(64):
        ctxt.copy(a, b)
    backend.synchronize()
    ms, algo = measure_dominant_kernel(backend, reps=8)
    a.destroy(); b.destroy()
    print(json.dumps({"probe": "copy kernel 67108864 B read + 67108864 B written per launch (64 launches); "
                               "gate/up GEMV %d algorithmic bytes per launch" % algo,
                      "gemv_launch_us": round(ms * 1000, 2)}))


def counter_probe_resident(backend, seed, pos=192, reps=8):
    """For hardware-counter runs of the resident launch: 64 launches of the copy kernel of known size, then the
    configuration-4 model (all 32 layers), 64 prompt positions through the chunked pass, and `reps` + 3 tokens at one
    position launched from the host (embedding row, emptying of the hand-off buffers, the resident launch), nothing else."""
    from slai_amd import _ffi
    from slai_amd import gguf_writer as gw
    from slai_amd.runtime import Gguf, GpuTensor, Llama2, LlmContext
    n = 16 * 1024 * 1024
    a = GpuTensor(backend, n)
    b = GpuTensor(backend, n)
    ctxt = LlmContext(backend)
    for _ in range(64):
        ctxt.copy(a, b)
    backend.synchronize()
    a.destroy(); b.destroy()
    data = gw.llama_gguf(dim=CFG["dim"], hidden_dim=CFG["hidden_dim"], n_layers=CFG["n_layers"], n_heads=CFG["n_heads"], n_kv_heads=CFG["n_kv_heads"],
                         vocab=CFG["vocab"], seq_len=512, wtype=12, v_type=14, out_type=14, embd_type=12, seed=seed, distinct_layers=4)
    g = Gguf(data)
    m = Llama2(backend, g, _ffi.MODEL_LLAMA, _ffi.KV_F16)
    assert m.decode_form() == 1, "the model did not take the resident launch"
    prompt = np.random.Generator(np.random.PCG64(seed)).integers(0, CFG["vocab"], pos).astype(np.int32)
    m.prefill(prompt, 0, 0)
    steps = m.time_steps(pos, 17, reps=reps)
    tb = token_bytes(CFG, m.weight_bytes(), pos, pos)
    m.destroy(); g.close()
    print(json.dumps({"probe": "copy kernel 67108864 B read + 67108864 B written per launch (64 launches); resident launch of a token at position %d, "
                               "%d algorithmic bytes per launch (%d launches)" % (pos, tb, reps + 3),
                      "launches_us": {name: round(us, 2) for name, us, _, _ in steps}}))


def counter_probe_gqa(backend, seed, pos=4047, n_caches=10, rounds=4):
    """For hardware-counter runs of the attention of a grouped-query model: 64 launches of the copy kernel of known size,
    then the attention operator on a Qwen2-7B-shaped layer (28 query heads on 4 kv heads of 128, fp16 cache, context 4096)
    at position `pos`, over `n_caches` distinct cache pairs, launched from the host.  SLAI_GQA_ON_DIE=0 in the environment
    gives the plain workgroup order for comparison."""
    from slai_amd import _ffi
    from slai_amd.runtime import GpuTensor, LlmContext
    n = 16 * 1024 * 1024
    a = GpuTensor(backend, n)
    b = GpuTensor(backend, n)
    ctxt = LlmContext(backend)
    for _ in range(64):
        ctxt.copy(a, b)
    backend.synchronize()
    a.destroy(); b.destroy()
    nh, nkv, hs, seq_len = 28, 4, 128, 4096
    kv_dim = nkv * hs
    rng = np.random.Generator(np.random.PCG64(seed))
    caches = [(GpuTensor(backend, kv_dim, seq_len, _ffi.DT_F16, data=rng.standard_normal((seq_len, kv_dim), dtype=np.float32).astype(np.float16)),
               GpuTensor(backend, kv_dim, seq_len, _ffi.DT_F16, data=rng.standard_normal((seq_len, kv_dim), dtype=np.float32).astype(np.float16))) for _ in range(n_caches)]
    params = _ffi.AttnParams(seq_len, kv_dim, nh // nkv, nh, hs, pos, (0, 0))
    gparams = GpuTensor.scalar(backend, params)
    gq = GpuTensor.vector(backend, rng.standard_normal(nh * hs, dtype=np.float32))
    gatt, gxb = GpuTensor(backend, seq_len, nh), GpuTensor(backend, nh * hs)
    backend.timer_begin()
    for _ in range(rounds):
        for kc, vc in caches:
            ctxt.attention(params, gparams, gq, kc, vc, gatt, gxb)
    us = backend.timer_end() * 1000.0 / (rounds * n_caches)
    print(json.dumps({"probe": "copy kernel 67108864 B read + 67108864 B written per launch (64 launches); attention of 28 query heads on 4 kv heads of 128 "
                               "at position %d, fp16 cache: %d algorithmic bytes per call (%d calls over %d cache pairs)"
                               % (pos, 2 * (pos + 1) * kv_dim * 2, rounds * n_caches, n_caches),
                      "us_per_call": round(us, 2), "on_die": os.environ.get("SLAI_GQA_ON_DIE", "1")}))


EAGER = False        # --eager: launch from the host instead of replaying a HIP graph (for runs under the kernel tracer)


def graph_time_us(backend, enqueue, n_launches, reps=20):
    """Mean time per launch of `enqueue` (which issues n_launches kernels) captured in a HIP graph and replayed."""
    enqueue()                                   # eager once: sizes scratch buffers outside the capture
    backend.synchronize()
    if EAGER:
        backend.timer_begin()
        for _ in range(reps):
            enqueue()
        return backend.timer_end() * 1000.0 / (reps * n_launches)
    backend.graph_begin_capture()
    enqueue()
    g = backend.graph_end_capture()
    backend.graph_launch(g)
    backend.synchronize()
    backend.timer_begin()
    for _ in range(reps):
        backend.graph_launch(g)
    ms = backend.timer_end()
    backend.graph_destroy(g)
    return ms * 1000.0 / (reps * n_launches)


def sweep(backend):
    """Config 2 (stand-alone GEMV, every block format, two shapes) and the attention kernel at long context (config 5
    shape): per-launch time and GB/s over rotating weight copies (> 512 MB, so reads come from HBM), launched from a
    HIP graph so that the host is not in the loop.  Algorithmic bytes = packed W + 4*ncols + 4*nrows."""
    from slai_amd import _ffi, synth
    from slai_amd.runtime import GpuQuantMatrix, GpuTensor, LlmContext
    ctxt = LlmContext(backend)
    names = {2: "Q4_0", 12: "Q4_K", 13: "Q5_K", 14: "Q6_K", 8: "Q8_0"}
    rows = []
    if EAGER:
        # under a profiler: a plain copy of known size first (64 MiB read, 64 MiB written per launch), against which
        # the byte counters of the other kernels are scaled
        n = 16 * 1024 * 1024
        ca, cb = GpuTensor(backend, n), GpuTensor(backend, n)
        for _ in range(16):
            ctxt.copy(ca, cb)
        backend.synchronize()
        ca.destroy(); cb.destroy()
    for (nrows, ncols) in ((4096, 4096), (11008, 4096)):
        for t in (2, 12, 13, 14, 8):
            base = synth.normal_quantized(4242 + t, t, nrows, ncols, 0.02)
            rb = base.size // nrows
            ncopies = int(math.ceil(560e6 / base.size))
            x = GpuTensor.vector(backend, synth.normal(7, ncols, 1.0))
            ones = GpuTensor.vector(backend, np.ones(ncols, np.float32))
            prep = GpuTensor(backend, ncols + ncols // 16)
            ctxt.rms_norm_prepare(prep, x, ones)
            out = GpuTensor(backend, nrows)
            res = {"format": names[t], "nrows": nrows, "ncols": ncols, "copies": ncopies}
            algo = base.size + 4 * ncols + 4 * nrows
            for layout, label in ((_ffi.LAYOUT_TILE16, "tile16"), (_ffi.LAYOUT_TILE64, "tile64")):
                mats = [GpuQuantMatrix(backend, t, nrows, ncols, np.roll(base.reshape(nrows, rb), i + 1, axis=0), layout=layout)
                        for i in range(ncopies)]
                if layout == _ffi.LAYOUT_TILE64:
                    us = graph_time_us(backend, lambda: [ctxt.matmul_quant_assign_prepared(out, m, prep) for m in mats], ncopies)
                else:
                    us = graph_time_us(backend, lambda: [ctxt.matmul_quant_assign(out, m, x) for m in mats], ncopies)
                res[label + "_us"] = round(us, 2)
                res[label + "_gbs"] = round(algo / us / 1e3, 1)
                for m in mats:
                    m.destroy()
            res["algorithmic_bytes"] = algo
            rows.append(res)
            log("gemv %-5s %5dx%-5d  16-row tiles %6.2f us %7.1f GB/s | 64-row tiles %6.2f us %7.1f GB/s"
                % (names[t], nrows, ncols, res["tile16_us"], res["tile16_gbs"], res["tile64_us"], res["tile64_gbs"]))
            for o in (x, ones, prep, out):
                o.destroy()
    # attention, config 5 shape: 32 heads x 128, fp16 cache, positions ~4000 of 4096
    AttnParams = _ffi.AttnParams
    nh, hs, seq = 32, 128, 4096
    kv_dim = nh * hs
    rng = np.random.Generator(np.random.PCG64(5))
    ncopies = 10                                 # 10 x 2 x 32 MiB of cache > 512 MB
    caches = [(GpuTensor(backend, kv_dim, seq, _ffi.DT_F16, data=rng.standard_normal((seq, kv_dim), dtype=np.float32).astype(np.float16)),
               GpuTensor(backend, kv_dim, seq, _ffi.DT_F16, data=rng.standard_normal((seq, kv_dim), dtype=np.float32).astype(np.float16)))
              for _ in range(ncopies)]
    gq = GpuTensor.vector(backend, rng.standard_normal(nh * hs, dtype=np.float32))
    gatt, gxb = GpuTensor(backend, seq, nh), GpuTensor(backend, nh * hs)
    att = []
    for pos in (1023, 4047):
        params = AttnParams(seq, kv_dim, 1, nh, hs, pos, (0, 0))
        gparams = GpuTensor.scalar(backend, params)
        us = graph_time_us(backend, lambda: [ctxt.attention(params, gparams, gq, k, v, gatt, gxb) for (k, v) in caches], ncopies)
        algo = 2 * (pos + 1) * kv_dim * 2
        att.append({"pos": pos, "us": round(us, 2), "gbs": round(algo / us / 1e3, 1), "algorithmic_bytes": algo})
        log("attention 32x128 f16, pos %4d: %6.2f us (attention + combine) %7.1f GB/s" % (pos, us, algo / us / 1e3))
        gparams.destroy()
    for o in [gq, gatt, gxb] + [t for kv in caches for t in kv]:
        o.destroy()
    print(json.dumps({"sweep": "stand-alone GEMV per block format (BASELINE config 2) and long-context attention (config 5 shape)",
                      "peak_gbs": HBM_PEAK_GBS, "gemv": rows, "attention": att}), flush=True)


def cpu_config1(seed):
    """BASELINE configuration 1 in full on the oracle: tiny Llama (dim 288, 6 layers, Q8_0), 16 prompt ids + 128 greedy
    tokens, on ONE thread (the reference's CPU path is single-threaded nalgebra, models/llama2/cpu.rs:370-376) and on all
    cores; tok/s over the 143 forward passes of the run (the reference feeds a prompt token by token, chat_llama2.rs:105-158)."""
    import oracle
    from slai_amd import gguf_writer as gw
    L = oracle.load()
    data = gw.tiny_llama_gguf(seed=seed)
    err = C.c_int(0)
    g = L.slo_gguf_parse(data.ctypes.data, data.size, C.byref(err))
    prompt = np.random.Generator(np.random.PCG64(seed)).integers(0, 32000, 16).astype(np.int32)
    out = {}
    ncores = os.cpu_count() or 1
    n = 16 + 128 - 1                              # forward passes of the configuration: 16 prompt ids, 128 tokens out
    for label, threads in (("one_thread", 1), ("all_cores", min(16, ncores))):
        L.slo_set_threads(threads)
        m = L.slo_llama2_from_gguf(g, b"llama", 0, 0, 0)
        toks = np.zeros(n, np.int32)
        t0 = time.perf_counter()
        L.slo_llama2_generate(m, prompt.ctypes.data, 16, 0, n, -1, toks.ctypes.data, None)
        dt = time.perf_counter() - t0
        L.slo_llama2_free(m)
        out[label] = dict(tok_s=round(n / dt, 2), threads=threads, forward_passes=n)
    L.slo_gguf_free(g)
    out["nproc"] = ncores
    return out


def cpu_baseline(seed, n_tokens=32):
    """Oracle decode of the headline layer shapes at depth 2 and 6, extrapolated linearly to 32 layers; beside it
    configuration 1 in full (cpu_config1)."""
    import oracle
    from slai_amd import gguf_writer as gw
    L = oracle.load()
    threads = min(16, os.cpu_count() or 1)
    L.slo_set_threads(threads)
    times = {}
    for nl in (2, 6):
        data = gw.llama_gguf(dim=CFG["dim"], hidden_dim=CFG["hidden_dim"], n_layers=nl, n_heads=CFG["n_heads"],
                             n_kv_heads=CFG["n_kv_heads"], vocab=CFG["vocab"], seq_len=128, wtype=12, v_type=14,
                             out_type=14, embd_type=12, seed=seed, with_output=True, distinct_layers=2)
        err = C.c_int(0)
        g = L.slo_gguf_parse(data.ctypes.data, data.size, C.byref(err))
        m = L.slo_llama2_from_gguf(g, b"llama", 1, 0, 1)
        prompt = np.random.Generator(np.random.PCG64(seed)).integers(0, CFG["vocab"], 2).astype(np.int32)
        out = np.zeros(n_tokens + 2, np.int32)
        L.slo_llama2_generate(m, prompt.ctypes.data, 2, 0, 2, -1, out.ctypes.data, None)       # untimed
        t0 = time.perf_counter()
        seq = np.concatenate([prompt, out[:2]]).astype(np.int32)
        L.slo_llama2_generate(m, seq.ctypes.data, seq.size, 2, n_tokens, -1, out.ctypes.data, None)
        times[nl] = (time.perf_counter() - t0) / n_tokens
        L.slo_llama2_free(m); L.slo_gguf_free(g)
        del data
    per_layer = (times[6] - times[2]) / 4.0
    head = max(times[2] - 2 * per_layer, 0.0)
    full = head + CFG["n_layers"] * per_layer
    return dict(value=1.0 / full, unit="tok/s", cores=threads, kind="port", nproc=os.cpu_count() or 1,
                sample="oracle (C restatement of models/llama2/cpu.rs, OpenMP over GEMV rows) on the same layer shapes and "
                       "quantization at depth 2 and 6, %d tokens each; %.2f ms per layer + %.2f ms embedding/head per token, "
                       "extrapolated to 32 layers" % (n_tokens, per_layer * 1e3, head * 1e3),
                config1=cpu_config1(seed))


def config5_block(backend, seed, n_steps=96):
    """BASELINE configuration 5: the 7B shape with Q8_0 weights and an fp16 cache pre-filled to 4000 positions with seeded
    N(0,1) rows, 96 tokens decoded up to the 4096th position.  Attention rate: the attention kernels (split + combine)
    timed alone at position 4047 over rotating caches; GEMV rate: the weight bytes over what is left of the token."""
    from slai_amd import _ffi
    from slai_amd import gguf_writer as gw
    from slai_amd.runtime import Gguf, GpuTensor, Llama2, LlmContext
    t0 = time.perf_counter()
    data = gw.llama_gguf(dim=CFG["dim"], hidden_dim=CFG["hidden_dim"], n_layers=CFG["n_layers"], n_heads=CFG["n_heads"], n_kv_heads=CFG["n_kv_heads"],
                         vocab=CFG["vocab"], seq_len=4096, wtype=8, seed=seed + 5, distinct_layers=2)
    g = Gguf(data)
    m = Llama2(backend, g, _ffi.MODEL_LLAMA, _ffi.KV_F16)
    rng = np.random.Generator(np.random.PCG64(seed + 6))
    fills = [(rng.standard_normal((4000, CFG["dim"]), dtype=np.float32).astype(np.float16),
              rng.standard_normal((4000, CFG["dim"]), dtype=np.float32).astype(np.float16)) for _ in range(4)]
    for l in range(CFG["n_layers"]):
        m.write_kv(l, *fills[l % 4])
    log("config 5 model: %.2f GB, set up in %.1f s" % (data.size / 1e9, time.perf_counter() - t0))
    seq = np.zeros(4001, np.int32); seq[4000] = 17
    m.generate(seq, 8, start_pos=4000)                                    # untimed: graph capture, first touch
    _, ms = m.generate(seq, n_steps, start_pos=4000)
    ms_tok = ms / n_steps
    wbytes = m.weight_bytes()
    kv_dim = CFG["dim"]
    kv_read = 2 * CFG["n_layers"] * (4000 + (n_steps + 1) / 2.0) * kv_dim * 2
    form = m.decode_form()
    m.destroy(); g.close(); del data
    # the attention kernels alone at position 4047 (the mean of the 96 positions), rotating over > 512 MB of caches
    ctxt = LlmContext(backend)
    nh, hs, seq_len, pos = CFG["n_heads"], CFG["dim"] // CFG["n_heads"], 4096, 4047
    caches = [(GpuTensor(backend, kv_dim, seq_len, _ffi.DT_F16, data=np.resize(fills[i % 4][0], (seq_len, kv_dim))),
               GpuTensor(backend, kv_dim, seq_len, _ffi.DT_F16, data=np.resize(fills[i % 4][1], (seq_len, kv_dim)))) for i in range(10)]
    params = _ffi.AttnParams(seq_len, kv_dim, 1, nh, hs, pos, (0, 0))
    gparams = GpuTensor.scalar(backend, params)
    gq = GpuTensor.vector(backend, rng.standard_normal(nh * hs, dtype=np.float32))
    gatt, gxb = GpuTensor(backend, seq_len, nh), GpuTensor(backend, nh * hs)
    us = graph_time_us(backend, lambda: [ctxt.attention(params, gparams, gq, kc, vc, gatt, gxb) for (kc, vc) in caches], len(caches))
    attn_bytes = 2 * (pos + 1) * kv_dim * 2
    for o in [gparams, gq, gatt, gxb] + [t for kv in caches for t in kv]:
        o.destroy()
    attn_ms_tok = us * CFG["n_layers"] / 1000.0
    rest_ms = max(ms_tok - attn_ms_tok, 1e-6)
    total = wbytes + kv_read
    return dict(workload="7B shape, Q8_0, fp16 cache pre-filled to 4000 positions, %d tokens at positions 4000..%d" % (n_steps, 3999 + n_steps),
                tok_s=round(1000.0 / ms_tok, 1), ms_per_step=round(ms_tok, 4), token_bytes=int(total),
                hbm_gbs=round(total / ms_tok / 1e6, 1), hbm_roofline_frac=round(total / ms_tok / 1e6 / HBM_PEAK_GBS, 4),
                attention=dict(us_per_layer=round(us, 2), gbs=round(attn_bytes / us / 1e3, 1), frac=round(attn_bytes / us / 1e3 / HBM_PEAK_GBS, 4),
                               algorithmic_bytes=attn_bytes, how="split + combine kernels alone at position %d over 10 rotating cache pairs" % pos),
                gemv=dict(gbs=round(wbytes / rest_ms / 1e6, 1), frac=round(wbytes / rest_ms / 1e6 / HBM_PEAK_GBS, 4), weight_bytes=int(wbytes),
                          how="weight bytes over the token time less 32 x the attention time"),
                decode_form=form)


def small_config_blocks(backend, seed):
    """BASELINE configurations 1 (tiny Llama, Q8_0, 16 prompt ids + 128 tokens) and 3 (GPT-2-small shape, Q8_0, 32 prompt
    ids + 256 tokens) through the C ABI: tok/s over the generated tokens of the device-resident greedy loop, the prompt
    fed token by token as the reference does (chat_llama2.rs:105-158), second run timed (the first captures the graph)."""
    from slai_amd import _ffi
    from slai_amd import gguf_writer as gw
    from slai_amd.runtime import Gguf, Gpt2, Llama2
    out = {}
    for name, make, cls, vocab, n_prompt, n_tokens in (
            ("config1", lambda: gw.tiny_llama_gguf(seed=seed), lambda g: Llama2(backend, g, _ffi.MODEL_LLAMA, _ffi.KV_F32), 32000, 16, 128),
            ("config3", lambda: gw.gpt2_gguf(seed=seed), lambda g: Gpt2(backend, g), 50257, 32, 256)):
        data = make()
        g = Gguf(data)
        m = cls(g)
        prompt = np.random.Generator(np.random.PCG64(seed)).integers(0, vocab, n_prompt).astype(np.int32)
        m.generate(prompt, n_prompt + 8)                                        # untimed: graph capture, first touch
        first, _ = m.generate(prompt, n_prompt - 1)                             # the prompt, untimed (caches only)
        seq = np.concatenate([prompt, np.zeros(1, np.int32)])
        _, ms = m.generate(seq, n_tokens, start_pos=n_prompt - 1)               # timed: the generated tokens
        wbytes = m.weight_bytes()
        m.destroy(); g.close(); del data
        out[name] = dict(tok_s=round(1000.0 * n_tokens / ms, 1), ms_per_step=round(ms / n_tokens, 4), tokens=n_tokens, prompt=n_prompt,
                         weight_bytes=int(wbytes), hbm_gbs=round(wbytes / (ms / n_tokens) / 1e6, 1))
    out["config1"]["workload"] = "tiny Llama-2: dim 288, 6 layers, 6 heads, FFN 768, vocab 32000, Q8_0, f32 cache"
    out["config3"]["workload"] = "GPT-2-small shape: dim 768, 12 layers, 12 heads, FFN 3072, vocab 50257, context 1024, Q8_0"
    return out


def bench_line(K, W, ms_per_step, tb, n_layers, distinct_layers, pos0, seq_len, form, step_times=None, sampled=None, prompt_chunks=None,
               config5=None, small=None, roofline=None, cpu=None):
    """The one JSON line of the benchmark as a dict (no device needed to build it)."""
    tok_s = 1000.0 / ms_per_step
    small = small or {}
    return {
        "metric": "decode tok/s & % of HBM roofline, Llama-2-7B-shape Q4_K, batch 1",
        "value": round(tok_s, 2), "unit": "tok/s", "n_gpus": 1, "steps": int(K), "warmup": int(W),
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic: seeded N(0,0.02) weights quantized with ggml's reference algorithm "
                                "(%d layers generated, the rest are row-rotated copies in distinct memory), seeded prompt ids"
                                % distinct_layers,
        "config": {"workload": "BASELINE config 4: Llama-2-7B-shape greedy decode, dim 4096, %d layers, 32 heads, FFN 11008, "
                               "vocab 32000, Q4_K weights (Q6_K v-proj/output), fp16 KV; 64 prompt positions processed untimed, "
                               "%d token(s) decoded untimed, then %d tokens timed at positions %d..%d"
                               % (n_layers, W, K, pos0, pos0 + K - 1), "batch": 1, "kv_dtype": "f16", "context": seq_len,
                   "decode_form": "one resident launch per token" if form else "one launch per step"},
        "token_bytes": int(tb), "hbm_gbs": round(tb / ms_per_step / 1e6, 1),
        "hbm_roofline_frac": round(tb / ms_per_step / 1e6 / HBM_PEAK_GBS, 4),
        "roofline_tok_s": round(HBM_PEAK_GBS * 1e9 / tb, 1),
        "step_times": step_times, "sampled_decode": sampled, "prompt_chunks": prompt_chunks,
        "config1": small.get("config1"), "config3": small.get("config3"), "config5": config5,
        "roofline": roofline, "cpu_baseline": cpu,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--layers", type=int, default=CFG["n_layers"], help="depth (32 = the benchmark configuration)")
    ap.add_argument("--distinct-layers", type=int, default=4)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-roofline", action="store_true")
    ap.add_argument("--no-side", action="store_true", help="only the headline decode (no sampled decode, prompt chunks, config 5)")
    ap.add_argument("--probe", action="store_true", help="counter probe: copy kernel + dominant GEMV only")
    ap.add_argument("--probe-resident", action="store_true", help="counter probe: copy kernel + the resident launch of a few tokens only")
    ap.add_argument("--probe-gqa", action="store_true", help="counter probe: copy kernel + the attention of a grouped-query layer only")
    ap.add_argument("--sweep", action="store_true", help="per-format GEMV sweep and long-context attention instead of the decode run")
    ap.add_argument("--eager", action="store_true", help="with --sweep: launch from the host, no HIP graph (the kernel tracer cannot follow graph launches here)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs the decode path on ONE GPU (batch-1 decode does not shard usefully); "
              "--gpus %d is not supported" % args.gpus, file=sys.stderr)
        sys.exit(2)
    if args.probe or args.probe_resident or args.probe_gqa or args.sweep:
        global EAGER
        EAGER = args.eager
        from slai_amd.runtime import Backend
        backend = Backend(0)
        if args.probe_gqa:
            counter_probe_gqa(backend, args.seed)
        elif args.probe or args.probe_resident:
            counter_probe_resident(backend, args.seed) if args.probe_resident else counter_probe(backend)
        else:
            sweep(backend)
        backend.close()
        return
    K, W = args.steps, max(args.warmup, 1)
    P = 64                                       # prompt positions of the configuration, always processed first
    cfg = dict(CFG, n_layers=args.layers)
    seq_len = max(512, ((P + W + K + 63) // 64) * 64)

    from slai_amd import _ffi
    from slai_amd import gguf_writer as gw
    from slai_amd.runtime import Backend, Gguf, Llama2

    t0 = time.perf_counter()
    data = gw.llama_gguf(dim=cfg["dim"], hidden_dim=cfg["hidden_dim"], n_layers=cfg["n_layers"], n_heads=cfg["n_heads"],
                         n_kv_heads=cfg["n_kv_heads"], vocab=cfg["vocab"], seq_len=seq_len, wtype=12, v_type=14, out_type=14,
                         embd_type=12, seed=args.seed, distinct_layers=min(args.distinct_layers, cfg["n_layers"]))
    log("model file: %.2f GB in %.1f s" % (data.size / 1e9, time.perf_counter() - t0))
    backend = Backend(0)
    t0 = time.perf_counter()
    g = Gguf(data)
    model = Llama2(backend, g, _ffi.MODEL_LLAMA, _ffi.KV_F16)
    form = model.decode_form()
    log("upload: %.1f s, weights %.3f GB, decode form %d (%s)" % (time.perf_counter() - t0, model.weight_bytes() / 1e9, form,
                                                                  "one resident launch per token" if form else "one launch per step"))

    prompt = np.random.Generator(np.random.PCG64(args.seed)).integers(0, cfg["vocab"], P).astype(np.int32)
    # untimed: prompt positions 0 .. P-2 in chunks (caches only), then W tokens decoded from the last prompt token on
    model.prefill(prompt[:P - 1], 0, 0)
    warm, _ = model.generate(prompt, W, start_pos=P - 1)
    seq = np.concatenate([prompt, warm]).astype(np.int32)
    # timed: K tokens at positions P-1+W .. P-2+W+K
    pos0 = P - 1 + W
    wall0 = time.perf_counter()
    toks, ms = model.generate(seq, K, start_pos=pos0)
    wall = time.perf_counter() - wall0
    ms_per_step = ms / K
    tok_s = 1000.0 / ms_per_step
    tb = token_bytes(cfg, model.weight_bytes(), pos0, pos0 + K - 1)
    log("decode: %.3f ms/token (events), wall %.3f ms/token, %.1f tok/s, %.2f GB/token -> %.1f GB/s"
        % (ms_per_step, wall * 1000 / K, tok_s, tb / 1e9, tb / ms_per_step / 1e6))
    steps = None
    resident_us = None
    if form == 1 and not args.no_roofline:
        # the launches of a token with an event after each (launched from the host, 8 tokens at the middle position): the
        # embedding row, the emptying of the hand-off buffers, the resident launch of the layer stack and the output matrix
        mid = pos0 + K // 2
        steps = [dict(step=name, us_per_launch=round(us, 2), launches_per_token=per, us_between_events_in_a_token=round(us, 2))
                 for name, us, per, _ in model.time_steps(mid, int(toks[K // 2 - 1]), reps=8)]
        resident_us = next(e["us_per_launch"] for e in steps if e["step"] == "llama2 resident token")
        log("launches of a token: " + "; ".join("%s %.2f us" % (e["step"], e["us_per_launch"]) for e in steps))
    if form == 0 and not args.no_roofline:
        # every launch of a token, timed with an event after each (launched from the host, 8 tokens at the middle position)
        mid = pos0 + K // 2
        sb = step_bytes(cfg, mid)
        steps = []
        for name, us, per, alone in model.time_steps(mid, int(toks[K // 2 - 1]), reps=8):
            e = dict(step=name, us_per_launch=round(alone, 2), launches_per_token=per, us_between_events_in_a_token=round(us, 2))
            if name in sb:
                e.update(algorithmic_bytes=int(sb[name]), gbs=round(sb[name] / alone / 1e3, 1), frac=round(sb[name] / alone / 1e3 / HBM_PEAK_GBS, 4))
            steps.append(e)
        log("steps (each alone, one launch per layer back to back): " + "; ".join("%s %.2f us x %d" % (e["step"], e["us_per_launch"], e["launches_per_token"]) for e in steps))
    sampled = prompt_chunks = None
    if not args.no_side:
        # the same K positions with the chat's sampler (temperature 0.7, top-p 0.95) picked on the device: reported beside
        # the headline, never as it.  Random weights give nearly flat logits, the slow case of the nucleus search.
        _, ms_s = model.generate_sampled(seq, K, 0.7, 0.95, args.seed, start_pos=pos0)
        sampled = dict(tok_s=round(1000.0 * K / ms_s, 2), ms_per_step=round(ms_s / K, 4), temperature=0.7, top_p=0.95)
        log("sampled decode (device sampler, T=0.7, top-p 0.95): %.3f ms/token, %.1f tok/s" % (ms_s / K, 1000.0 * K / ms_s))
        # prompt processing, reported beside the headline: the reference feeds a prompt token by token (chat_llama2.rs:105-158);
        # the chunked pass runs 32 tokens per pass over the weights on the matrix cores and computes no logits
        n_prompt = min(256, seq_len)
        ptoks = np.random.Generator(np.random.PCG64(args.seed + 1)).integers(0, cfg["vocab"], n_prompt).astype(np.int32)
        model.prefill(ptoks, 0, 0)                                   # untimed: buffers, first touch
        ms_p = min(model.prefill(ptoks, 0, 0) for _ in range(3))
        ms_loop = model.prefill(ptoks[:64], 0, 1)
        prompt_chunks = dict(tok_s=round(1000.0 * n_prompt / ms_p, 1), tokens=n_prompt, ms=round(ms_p, 3), path=model.prefill_path(),
                             token_by_token_tok_s=round(1000.0 * 64 / ms_loop, 1), fp32_repeats=model.prefill_fp32_repeats())
        log("prompt: %d tokens in %.2f ms (%.0f tok/s) in chunks; token by token %.0f tok/s" % (n_prompt, ms_p, 1000.0 * n_prompt / ms_p, 1000.0 * 64 / ms_loop))
    model.destroy(); g.close(); del data

    roof = None
    if not args.no_roofline:
        if form == 1:
            # the resident launch is nearly the whole token: its bytes are the token's bytes less the embedding row
            ach = tb / (resident_us * 1e-6) / 1e9
            roof = dict(bound="hbm", kernel="llama_decode_persistent_kernel (all 32 layers: RMSNorm + q/k/v + RoPE + cache write, attention, output projection, "
                                            "RMSNorm + gate/up + SiLU, down projection; final norm + output matrix): one launch per token",
                        achieved=round(ach, 1), peak=HBM_PEAK_GBS, unit="GB/s", frac=round(ach / HBM_PEAK_GBS, 4), traffic=resident_kernel_traffic(),
                        traffic_source=RESIDENT_TRAFFIC_PROFILE, launch_us=resident_us, algorithmic_bytes=int(tb),
                        how="HIP events on the library's stream before and after the launch, 8 tokens at position %d launched from the host" % (pos0 + K // 2))
        else:
            kms, kalgo = measure_dominant_kernel(backend)
            ach = kalgo / (kms * 1e-3) / 1e9
            gate_up = dict(kernel="gemv_rowtile_kernel<Q4_K, gated pair> (RMSNorm + gate/up GEMV + SiLU, 2x 11008x4096), alone over 8 rotating weight copies",
                           achieved=round(ach, 1), frac=round(ach / HBM_PEAK_GBS, 4), traffic=dominant_kernel_traffic(), traffic_source=TRAFFIC_PROFILE,
                           launch_us=round(kms * 1000, 2), algorithmic_bytes=kalgo)
            top = max((e for e in steps if "algorithmic_bytes" in e), key=lambda e: e["us_per_launch"] * e["launches_per_token"]) if steps else None
            if top and top["step"] == "llama2 qkv + attention":
                # the launch that takes the largest share of a token: q/k/v projections and the attention in one kernel.  It
                # is not an operator of its own: slai_llama2_time_steps launches it alone, layer after layer.
                roof = dict(bound="hbm", kernel="qkv_attention_kernel (RMSNorm + q/k/v GEMV, RoPE, cache write, attention; 32 launches per token)",
                            achieved=top["gbs"], peak=HBM_PEAK_GBS, unit="GB/s", frac=top["frac"], traffic=None,
                            launch_us=top["us_per_launch"], algorithmic_bytes=top["algorithmic_bytes"],
                            how="its 32 launches of a token (one per layer, each layer's own weights and cache) back to back from the host at position %d, "
                                "HIP events before the first and after the last, 8 repetitions" % (pos0 + K // 2),
                            second_kernel=gate_up)
            else:
                roof = dict(bound="hbm", peak=HBM_PEAK_GBS, unit="GB/s", **gate_up)
        log("dominant kernel: %s us/launch, %.1f GB/s" % (roof["launch_us"], roof["achieved"]))
    c5 = small = None
    if not args.no_side:
        small = small_config_blocks(backend, args.seed)
        log("config 1: %.1f tok/s (%.4f ms/token); config 3: %.1f tok/s (%.4f ms/token)"
            % (small["config1"]["tok_s"], small["config1"]["ms_per_step"], small["config3"]["tok_s"], small["config3"]["ms_per_step"]))
        c5 = config5_block(backend, args.seed)
        log("config 5: %.1f tok/s (%.3f ms/token); attention %.2f us/layer = %.1f GB/s; GEMV %.1f GB/s"
            % (c5["tok_s"], c5["ms_per_step"], c5["attention"]["us_per_layer"], c5["attention"]["gbs"], c5["gemv"]["gbs"]))
    backend.close()

    cpu = None
    if not args.no_cpu_baseline:
        t0 = time.perf_counter()
        cpu = cpu_baseline(args.seed)
        log("cpu baseline: %.3f tok/s on %d threads (%.1f s); config 1 in full: %s" % (cpu["value"], cpu["cores"], time.perf_counter() - t0, cpu["config1"]))

    out = bench_line(K, W, ms_per_step, tb, cfg["n_layers"], min(args.distinct_layers, cfg["n_layers"]), pos0, seq_len, form, step_times=steps,
                     sampled=sampled, prompt_chunks=prompt_chunks, config5=c5, small=small, roofline=roof, cpu=cpu)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
