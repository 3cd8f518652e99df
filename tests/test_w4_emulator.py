"""Address and data-flow replay of the generated K loops on the CPU (tests/w4_emulator.py): every copy inside its
operand, every LDS access inside its area and after the copy it depends on, every MFMA on the right fragments
of the right K step, every fused-epilogue store inside the previous tile -- for tiles of 4, 6 and 8 K steps,
whole and ragged, with and without a next tile, and every history of the wait counts."""
import pytest

from w4_emulator import Fail, replay

KINDS = ["fp8", "fp4", "bf16", "i8"]


def _steps(kind):
    return (4, 6, 8)


@pytest.mark.parametrize("kind", KINDS)
def test_whole_tiles_fused_epilogues(kind):
    """first tile, then tiles whose predecessor's epilogue is fused into them, the last one without a next tile"""
    for ks in _steps(kind):
        n = replay(kind, 512, 768, ks, [(0, 0), (256, 0), (0, 256), (256, 512)])
        assert n > 0


@pytest.mark.parametrize("kind", KINDS)
def test_ragged_tiles_and_compiled_epilogues(kind):
    """ragged row and column blocks (clamped copies, compiled epilogues with an unknown number of stores) between
    whole tiles, and padded row strides"""
    ks = _steps(kind)[0]
    replay(kind, 600, 520, ks, [(0, 0), (512, 0), (256, 256), (0, 512), (512, 512), (256, 0)], pad=64)


@pytest.mark.parametrize("kind", ["fp8", "fp4", "bf16"])
def test_fast_compiled_epilogues(kind):
    """fp16 output: whole tiles take the compiled fast epilogue (exactly 32 stores per wave), nothing is fused"""
    ks = _steps(kind)[-1]
    replay(kind, 512, 512, ks, [(0, 0), (256, 0), (0, 256)], c_bf16=False)


@pytest.mark.parametrize("kind", ["fp8", "fp4", "bf16"])
def test_stream_k_pieces(kind):
    """a work list as the Stream-K schedule deals it out: whole tiles, then pieces of a tile's K range (multiples of
    four K steps) whose copies start inside the operand rows -- including the look-ahead into the next piece"""
    replay(kind, 512, 512, 16, [(0, 0), (256, 0, 8, 16), (0, 256, 4, 12), (256, 256, 0, 4), (256, 256)])


def test_single_tile_workgroup():
    for kind in ("fp8", "fp4"):
        replay(kind, 256, 256, _steps(kind)[0], [(0, 0)])


@pytest.mark.parametrize("kind", ["fp8", "fp4"])
def test_replay_catches_a_copy_cursor_that_runs_ahead(kind, monkeypatch):
    """the replay must fail when the K loop is broken: copies that advance 256 bytes per K step instead of 128
    run past the end of the operand rows and feed the wrong K step"""
    import w4_emulator as E
    gen = E.load_generator()
    orig = gen.Gen.dma_advance

    def broken(self):
        return [gen.Op(o.text.replace(", 128", ", 256")) for o in orig(self)]
    real_load = E.load_generator

    def patched():
        g = real_load()
        g.Gen.dma_advance = broken
        return g
    monkeypatch.setattr(E, "load_generator", patched)
    with pytest.raises(Fail):
        E.replay(kind, 512, 512, _steps(kind)[-1], [(0, 0), (256, 0)])


def test_replay_catches_a_wait_that_is_too_loose(monkeypatch):
    """a vmcnt that allows one more operation in flight lets an LDS read see bytes whose copy may not have landed"""
    import w4_emulator as E
    real_load = E.load_generator

    def patched():
        g = real_load()
        solve = g.Gen.solve

        def loose(self, P):
            solve(self, P)
            w = [o for o in P["steady1"] if isinstance(o, g.WaitVm)][0]
            for k in w.vals:
                w.vals[k] += 1
        g.Gen.solve = loose
        return g
    monkeypatch.setattr(E, "load_generator", patched)
    with pytest.raises(Fail):
        E.replay("fp8", 512, 512, 8, [(0, 0), (256, 0)])
