"""The generator of the 4-wave kernels' K loop proves its own wait counts: every `s_waitcnt vmcnt(n)` it
writes is replayed against the instruction stream of every history a tile can have (first tile of a
workgroup, after compiled epilogue stores, after a fused epilogue) and must not allow more operations
in flight than were issued after the copies it waits for."""
import importlib.util
import os
import re

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
GEN = os.path.join(os.path.dirname(HERE), "tritonblas_amd", "csrc", "gen_w4.py")


def _load():
    spec = importlib.util.spec_from_file_location("gen_w4", GEN)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.mark.parametrize("kind", ["fp8", "e5m2", "e4e5", "e5e4", "fp4", "bf16", "f16", "i8"])
def test_wait_counts_hold_for_every_history(kind):
    gen = _load()
    slack = gen.Gen(kind).check()
    assert slack and min(slack.values()) >= 0


def test_checker_catches_a_wait_that_is_too_loose():
    """the same replay with one wait loosened by one must fail"""
    gen = _load()
    g = gen.Gen("fp8")
    parts = g.parts()
    waits = [o for o in parts["steady1"] if isinstance(o, gen.WaitVm)]
    assert waits
    g.parts = lambda: parts
    for k in waits[0].vals:
        waits[0].vals[k] += 1
    with pytest.raises(AssertionError):
        g.check()


@pytest.mark.parametrize("kind", ["fp8", "e5m2", "fp4", "bf16", "i8"])
def test_program_shape(kind):
    """one MFMA per accumulator tile and K slice in every step; the fused epilogue stores 32 times"""
    gen = _load()
    g = gen.Gen(kind)
    parts = g.parts()
    per_step = 64 if kind in ("fp8", "e5m2") else 128
    for name in ("first0", "first0_fe", "first0_fe16", "first1", "steady0", "steady1", "last0", "last1"):
        assert sum(1 for o in parts[name] if not isinstance(o, gen.WaitVm) and o.text.startswith("v_mfma")) == per_step, name
    for fe in ("first0_fe", "first0_fe16"):
        stores = [o for o in parts[fe] if not isinstance(o, gen.WaitVm) and o.text.startswith("global_store")]
        assert len(stores) == 32
    # the two fused epilogues differ in the conversion only
    a = [o.text for o in parts["first0_fe"] if not isinstance(o, gen.WaitVm)]
    b = [o.text for o in parts["first0_fe16"] if not isinstance(o, gen.WaitVm)]
    assert len(a) == len(b) and all(x == y or (x.startswith("v_cvt_pk_bf16_f32") and y == x.replace("bf16", "f16")) or x.startswith(";")
                                    for x, y in zip(a, b))
    assert not any(o.text.startswith("global_store") for o in parts["first0"] if not isinstance(o, gen.WaitVm))
    # the first K step starts every sum from zero, the others accumulate
    first = [o.text for o in parts["first0"] if not isinstance(o, gen.WaitVm) and o.text.startswith("v_mfma")]
    assert sum(1 for t in first if t.count("a[") == 1) == 64          # (no accumulator among the sources)
    steady = [o.text for o in parts["steady0"] if not isinstance(o, gen.WaitVm) and o.text.startswith("v_mfma")]
    assert all(t.count("a[") == 2 for t in steady)


@pytest.mark.parametrize("kind,fields", [("e5m2", " cbsz:1 blgp:1"), ("e4e5", " cbsz:1"), ("e5e4", " blgp:1")])
def test_8bit_float_kinds_differ_from_e4m3_only_in_the_format_fields(kind, fields):
    """cbsz is the format of the MFMA's first source, which is the B fragment, blgp that of the second, the A
    fragment: e4e5 (A in e4m3, B in e5m2) sets cbsz alone, e5e4 blgp alone."""
    gen = _load()
    a, b = gen.Gen("fp8").program(), gen.Gen(kind).program()
    assert len(a) == len(b)
    for x, y in zip(a, b):
        if x.startswith("v_mfma"):
            assert y == x + fields
            assert re.match(r"v_mfma_f32_16x16x128_f8f6f4 a\[\d+:\d+\], v\[(\d+):\d+\], v\[(\d+):\d+\]", x)
        else:
            assert x == y
