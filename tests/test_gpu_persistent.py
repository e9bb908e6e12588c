"""The one-launch-per-token form of the Llama-2 layer stack (kernels_decode_persistent.hip) against the oracle and against
the launch-per-step form it replaces, on models of the shapes it covers (as many cache heads as query heads of size 128,
width a multiple of 1024, Q4_K / Q6_K mixes, projections in 16-row tiles).  Same bars as the other model tests: logits
within 1e-2 of the oracle's (1e-3 of the other device path), greedy ids identical; every test asserts that the model took
the resident form.  The kernel's addresses are checked on the CPU in tests/test_resident_plan.py."""
import os

import numpy as np
import pytest

from gpu_common import rel_err
from slai_amd import _ffi
from slai_amd import gguf_writer as gw
from test_gpu_models import check_llama

pytestmark = pytest.mark.gpu


def backend_with(persistent, resident_max_pos=None):
    from slai_amd.runtime import Backend
    os.environ["SLAI_PERSISTENT"] = "1" if persistent else "0"
    if resident_max_pos is not None:
        os.environ["SLAI_RESIDENT_MAX_POS"] = str(resident_max_pos)
    try:
        return Backend(0)
    finally:
        del os.environ["SLAI_PERSISTENT"]
        os.environ.pop("SLAI_RESIDENT_MAX_POS", None)


@pytest.mark.parametrize("kv_f16", [True, False])
def test_persistent_small_model_vs_oracle(kv_f16):
    """dim 1024 (8 heads of 128), hidden 3072, 3 layers, vocabulary with a row tail, Q4_K with Q6_K v-proj / output /
    down: logits step by step and 40 greedy ids against the oracle."""
    b = backend_with(True)
    try:
        data = gw.llama_gguf(dim=1024, hidden_dim=3072, n_layers=3, n_heads=8, n_kv_heads=8, vocab=2000, seq_len=256, wtype=12, v_type=14,
                             out_type=14, embd_type=12, seed=71, std=0.05, norm_random=True)
        worst = check_llama(b, data, [5, 1000, 1999, 9, 77, 3], 40, kv_f16=kv_f16, check_logit_steps=12, decode_form=1)
        print("worst logits rel err", worst)
    finally:
        b.close()


@pytest.mark.parametrize("kv_f16", [True, False])
def test_persistent_long_context_vs_oracle(kv_f16):
    """600 steps on the small model: the attention asks for the first 384 cached positions (f16 cache; 128 with an f32
    cache) before the query exists and walks the rest in passes of 128 with one pass in flight; positions 128, 129, 384,
    385, 512, 513 are where those paths change.  Beyond position 512 (256 with an f32 cache) the host launches the
    variant of the kernel whose unit workgroups touch the far cache rows into the die's L2."""
    b = backend_with(True)
    try:
        data = gw.llama_gguf(dim=1024, hidden_dim=3072, n_layers=2, n_heads=8, n_kv_heads=8, vocab=2000, seq_len=640, wtype=12, v_type=14,
                             out_type=14, embd_type=12, seed=77, std=0.05, norm_random=True)
        check_llama(b, data, [5, 1000, 1999], 600, kv_f16=kv_f16, check_logit_steps=4, decode_form=1)
    finally:
        b.close()


@pytest.mark.parametrize("kv_f16", [True, False])
def test_launch_form_changes_with_the_position(kv_f16):
    """A model with a context of 2048 takes the resident launch for its first positions and one launch per step beyond
    (here from position 21 on, so that the prompt, the step-by-step logits and the generated ids all cross the change):
    both forms keep the same caches and loop state, and the ids and logits follow the oracle's throughout."""
    b = backend_with(True, resident_max_pos=21)
    try:
        data = gw.llama_gguf(dim=1024, hidden_dim=3072, n_layers=2, n_heads=8, n_kv_heads=8, vocab=2000, seq_len=2048, wtype=12, v_type=14,
                             out_type=14, embd_type=12, seed=91, std=0.05, norm_random=True)
        check_llama(b, data, [5, 1000, 1999, 9, 77, 3, 8, 21], 40, kv_f16=kv_f16, check_logit_steps=30, decode_form=1)
    finally:
        b.close()


def test_persistent_other_kquant_mixes():
    """The block formats the resident launch takes besides the headline mix: Q6_K in the two projections into the residual
    (16-row tiles on the matrix cores), Q5_K q and k (the vector-unit path with wave-uniform activations), Q6_K q, f32 cache."""
    b = backend_with(True)
    try:
        for seed, types, kv_f16 in ((81, {"attn_output": 14, "ffn_down": 14}, True), (82, {"attn_q": 13, "attn_k": 13, "ffn_down": 14}, False),
                                    (83, {"attn_q": 14, "attn_output": 14}, True)):
            data = gw.llama_gguf(dim=1024, hidden_dim=3072, n_layers=2, n_heads=8, n_kv_heads=8, vocab=1500, seq_len=320, wtype=12, v_type=14,
                                 out_type=12, embd_type=12, seed=seed, std=0.05, norm_random=True, tensor_types=types)
            check_llama(b, data, [5, 1000, 1499, 9], 24, kv_f16=kv_f16, check_logit_steps=6, decode_form=1)
    finally:
        b.close()


def test_persistent_qwen2_bias_and_neox_pairs():
    """The Qwen2 variant in the resident form: q / k / v biases and NeoX rotary pairs (i, i + 64), which the workgroups that
    multiply q and k rotate themselves (their units hold rows {0..31, 64..95} / {32..63, 96..127} of a head)."""
    b = backend_with(True)
    try:
        data = gw.llama_gguf(dim=1024, hidden_dim=3072, n_layers=3, n_heads=8, n_kv_heads=8, vocab=2000, seq_len=256, wtype=12, v_type=14,
                             out_type=14, embd_type=12, seed=75, std=0.05, arch="qwen2", bias=True, norm_random=True, rope_base=1000000.0, rms_eps=1e-6)
        check_llama(b, data, [5, 1000, 1999, 9], 40, kv_f16=True, model_type=_ffi.MODEL_QWEN2, neox=1, name=b"qwen2", check_logit_steps=12, decode_form=1)
    finally:
        b.close()


def test_persistent_small_model_behind_large_allocations():
    """The small model again, loaded after 5 GB of other allocations in steps of 640 MB: its buffers then lie at
    addresses whose lower 32 bits are spread over the whole range, bit 31 included (the first version of the kernel
    rebuilt pointers from two words with the lower one sign-extended, which only such addresses expose)."""
    from slai_amd.runtime import GpuTensor
    b = backend_with(True)
    try:
        pads = [GpuTensor(b, 160 * 1024 * 1024) for _ in range(8)]
        data = gw.llama_gguf(dim=1024, hidden_dim=3072, n_layers=3, n_heads=8, n_kv_heads=8, vocab=2000, seq_len=256, wtype=12, v_type=14,
                             out_type=14, embd_type=12, seed=73, std=0.05, norm_random=True)
        check_llama(b, data, [5, 1000, 1999, 9, 77, 3], 24, kv_f16=True, check_logit_steps=6, decode_form=1)
        for t in pads:
            t.destroy()
    finally:
        b.close()


def test_persistent_matches_launch_per_step_form():
    """The same model through both forms on the device: ids identical over 48 steps, logits within 1e-3."""
    from slai_amd.runtime import Gguf, Llama2
    data = gw.llama_gguf(dim=2048, hidden_dim=5632, n_layers=4, n_heads=16, n_kv_heads=16, vocab=4096, seq_len=512, wtype=12, v_type=14,
                         out_type=14, embd_type=12, seed=72, std=0.04, norm_random=True)
    prompt = np.array([7, 4000, 123, 9], np.int32)
    out = {}
    for persistent in (False, True):
        b = backend_with(persistent)
        try:
            g = Gguf(data)
            m = Llama2(b, g, _ffi.MODEL_LLAMA, _ffi.KV_F16)
            assert m.decode_form() == int(persistent)
            ids, ms = m.generate(prompt, 48)
            logits = m.forward_logits(48, int(ids[47]))
            out[persistent] = (ids, logits, ms / 48)
            m.destroy(); g.close()
        finally:
            b.close()
    assert np.array_equal(out[True][0], out[False][0]), (out[True][0].tolist(), out[False][0].tolist())
    assert rel_err(out[True][1], out[False][1]) < 1e-3
    print("ms/token: per-step launches %.3f, one launch %.3f" % (out[False][2], out[True][2]))


def test_persistent_width_3072_vs_oracle():
    """dim 3072 (24 heads), FFN 12288, 2 layers: twelve super-blocks per row (twelve of the sixteen waves multiply a
    64-row unit, three waves a 16-row tile of the output projection, twelve one of the down projection) and gate / up units
    of 64 rows -- the decomposition between the test shapes above and the headline's."""
    b = backend_with(True)
    try:
        data = gw.llama_gguf(dim=3072, hidden_dim=12288, n_layers=2, n_heads=24, n_kv_heads=24, vocab=1000, seq_len=128, wtype=12, v_type=14,
                             out_type=14, embd_type=12, seed=43, std=0.03, norm_random=True)
        check_llama(b, data, [5, 999, 77, 3], 24, kv_f16=True, check_logit_steps=8, decode_form=1)
    finally:
        b.close()


def test_persistent_7b_width_two_layers_vs_oracle():
    """The headline shapes (dim 4096, hidden 11008, 32 heads, vocab 32000) at depth 2 against the oracle."""
    b = backend_with(True)
    try:
        data = gw.llama_gguf(dim=4096, hidden_dim=11008, n_layers=2, n_heads=32, n_kv_heads=32, vocab=32000, seq_len=128, wtype=12, v_type=14,
                             out_type=14, embd_type=12, seed=41)
        prompt = np.random.Generator(np.random.PCG64(41)).integers(0, 32000, 8)
        check_llama(b, data, prompt, 40, kv_f16=True, check_logit_steps=10, decode_form=1)
    finally:
        b.close()
