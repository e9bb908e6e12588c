"""Every address of the resident decode kernel on the CPU: tests/native/resident_bounds.cpp walks the index arithmetic
the kernel itself uses (slai_amd/csrc/resident_plan.h) for every workgroup, wave, lane and layer of a launch and checks
each access against the allocation it goes to, with the buffers placed below and above 0x80000000 in the lower address
word.  The sign-extending join of an address's two words (the defect an earlier form of the kernel had) is the negative
control: it must be caught.  No GPU needed."""
import ctypes as C
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
Q4_K, Q5_K, Q6_K = 12, 13, 14


@pytest.fixture(scope="module")
def rb(tmp_path_factory):
    out = str(tmp_path_factory.mktemp("rb") / "libresident_bounds.so")
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-I", os.path.join(ROOT, "slai_amd", "csrc"),
                           os.path.join(HERE, "native", "resident_bounds.cpp"), "-o", out])
    L = C.CDLL(out)
    L.rb_audit.restype = C.c_ulonglong
    L.rb_audit.argtypes = [C.c_uint32] * 7 + [C.c_int] * 7 + [C.c_uint32, C.c_int, C.c_int, C.c_int, C.c_int, C.c_char_p, C.c_size_t, C.POINTER(C.c_ulonglong)]
    L.rb_shape.argtypes = [C.c_uint32] * 4 + [C.POINTER(C.c_uint32)] * 3
    return L


def audit(rb, dim, hidden, n_heads, n_layers, vocab, seq_len, grid=0, types=(Q4_K, Q4_K, Q6_K, Q4_K, Q4_K, Q4_K, Q6_K), kv_bytes=2, high=0, sign_ext=0, neox=0):
    msg = C.create_string_buffer(400)
    checked = C.c_ulonglong()
    bad = rb.rb_audit(dim, hidden, n_heads, n_layers, vocab, seq_len, grid, *types, max(n_heads, 256), kv_bytes, high, sign_ext, neox, msg, 400, C.byref(checked))
    return bad, msg.value.decode(), checked.value


# the shapes of tests/test_gpu_persistent.py and the headline configuration (BASELINE config 4: 32 layers, context 512)
SHAPES = {
    "small (dim 1024, Q6_K down)": dict(dim=1024, hidden=3072, n_heads=8, n_layers=3, vocab=2000, seq_len=256, types=(Q4_K, Q4_K, Q6_K, Q4_K, Q4_K, Q6_K, Q6_K)),
    "small, f32 cache": dict(dim=1024, hidden=3072, n_heads=8, n_layers=3, vocab=2000, seq_len=256, types=(Q4_K, Q4_K, Q6_K, Q4_K, Q4_K, Q6_K, Q6_K), kv_bytes=4),
    "dim 2048": dict(dim=2048, hidden=5632, n_heads=16, n_layers=4, vocab=4096, seq_len=512),
    "7B width, 2 layers": dict(dim=4096, hidden=11008, n_heads=32, n_layers=2, vocab=32000, seq_len=128),
    "config 4": dict(dim=4096, hidden=11008, n_heads=32, n_layers=32, vocab=32000, seq_len=512),
    "7B width, context 4096, f32 cache": dict(dim=4096, hidden=11008, n_heads=32, n_layers=2, vocab=32000, seq_len=4096, kv_bytes=4),
    "dim 3072": dict(dim=3072, hidden=12288, n_heads=24, n_layers=2, vocab=1000, seq_len=128),
    "NeoX rotary pairs": dict(dim=2048, hidden=5632, n_heads=16, n_layers=2, vocab=4096, seq_len=300, neox=1),
    "wide FFN (12 column groups in the down projection)": dict(dim=3072, hidden=12288, n_heads=24, n_layers=2, vocab=1000, seq_len=64, types=(Q5_K, Q4_K, Q4_K, Q6_K, Q4_K, Q4_K, Q4_K)),
}


@pytest.mark.parametrize("name", list(SHAPES))
@pytest.mark.parametrize("high", [0, 1], ids=["bases below 0x80000000", "bases above 0x80000000"])
def test_every_access_lies_inside_its_allocation(rb, name, high):
    bad, msg, checked = audit(rb, high=high, **SHAPES[name])
    assert bad == 0, msg
    assert checked > 500_000


def test_the_decomposition_gives_every_workgroup_a_role_in_every_phase(rb):
    """The headline shapes: 256 workgroups = the 16-row tiles of the projections = seven q / k / v units (v in three) + one
    attention workgroup per head = gate / up in 256 units of 43 rows.  Narrower models take fewer workgroups."""
    g, r, n = C.c_uint32(), C.c_uint32(), C.c_uint32()
    rb.rb_shape(4096, 11008, 32, 0, C.byref(g), C.byref(r), C.byref(n))
    assert (g.value, r.value, n.value) == (256, 43, 256)
    rb.rb_shape(1024, 3072, 8, 0, C.byref(g), C.byref(r), C.byref(n))
    assert (g.value, r.value, n.value) == (64, 48, 64)
    rb.rb_shape(2048, 5632, 16, 0, C.byref(g), C.byref(r), C.byref(n))
    assert (g.value, r.value, n.value) == (128, 44, 128)
    bad, msg, _ = audit(rb, grid=224, **SHAPES["7B width, 2 layers"])       # any other grid is refused
    assert bad and "shape_ok" in msg


def test_unsupported_shapes_are_refused(rb):
    for kw in (dict(dim=4096, hidden=11008, n_heads=32, n_layers=2, vocab=32000, seq_len=100000),    # context beyond what the plan admits
               dict(dim=5120, hidden=13824, n_heads=40, n_layers=2, vocab=32000, seq_len=512),       # width beyond four staging pieces per lane
               dict(dim=3072, hidden=4096, n_heads=24, n_layers=2, vocab=100, seq_len=64),           # 192 workgroups: units of 22 rows cover 4096 rows with 187
               dict(dim=1024, hidden=2800, n_heads=8, n_layers=2, vocab=100, seq_len=64)):            # FFN width not in super-blocks
        bad, msg, _ = audit(rb, **kw)
        assert bad and "shape_ok" in msg, (kw, msg)


def test_the_sign_extending_join_is_caught(rb):
    """Negative control: with an address's lower word widened as a signed int, buffers at or above 0x80000000 in the lower
    word are addressed at 0xffffffff........; the audit reports it (and stays silent for buffers below)."""
    bad, msg, _ = audit(rb, high=1, sign_ext=1, **SHAPES["small (dim 1024, Q6_K down)"])
    assert bad > 0 and "0xffffffff" in msg, msg
    bad, msg, _ = audit(rb, high=0, sign_ext=1, **SHAPES["small (dim 1024, Q6_K down)"])
    assert bad == 0, msg
