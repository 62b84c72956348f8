"""Selection rectangles and the ring write on the device against the CPU oracle: integer and
copy work, so bit-exact. The cases are the reference's own
(crates/engine/src/v4/select.rs:514-808) plus the shipped geometry (window 128, ratios 4 and
128, index_topk 512) at prompt lengths the oracle still finishes in seconds."""
import numpy as np
import pytest

from rivoli_amd import hip
from tests.gpu_util import back, dev, dzeros

pytestmark = pytest.mark.gpu


def device_gather(win, ratio, topk, seqlen, start):
    rows, cols = hip.sel_shape(win, ratio, topk, seqlen, start)
    out = dzeros(rows * cols * 4 + 64, 0xEE)
    assert hip.launch_sel_gather(win, ratio, topk, seqlen, start, out) == (rows, cols)
    raw = back(out, np.int32)
    assert (raw[rows * cols:] == np.int32(-286331154)).all()          # 0xEEEEEEEE: nothing past the rectangle
    return raw[:rows * cols].reshape(rows, cols)


@pytest.mark.parametrize("win,ratio,topk,seqlen,start", [
    (4, 0, 512, 1, 6), (4, 0, 512, 1, 2), (4, 0, 512, 1, 3), (100, 2, 512, 6, 0), (4, 0, 512, 7, 0),
    (8, 0, 512, 5, 0), (8, 0, 512, 1, 9), (8, 4, 512, 12, 0), (8, 4, 512, 1, 19), (8, 128, 512, 1, 300),
    (128, 4, 512, 2048, 0), (128, 128, 512, 3000, 0), (128, 4, 512, 1, 2047), (128, 128, 512, 1, 60000),
    (128, 0, 512, 700, 0), (1, 4, 512, 9, 0), (300, 4, 512, 1, 100), (128, 128, 512, 70000, 0)])
def test_positional_rectangle(oracle, win, ratio, topk, seqlen, start):
    code, want = oracle.sel_gather(win, ratio, topk, seqlen, start)
    assert code == 0
    assert np.array_equal(device_gather(win, ratio, topk, seqlen, start), want)


@pytest.mark.parametrize("win,ratio,topk,seqlen,start,n_comp", [
    (8, 4, 512, 1, 19, 5), (8, 4, 512, 12, 0, 3), (4, 4, 3, 1, 19, 5), (128, 4, 512, 4096, 0, 1024),
    (128, 4, 512, 1, 40000, 10000), (128, 4, 64, 1, 5000, 1250), (128, 4, 512, 1, 100, 0), (8, 4, 1, 8, 0, 2)])
def test_scored_rectangle(oracle, win, ratio, topk, seqlen, start, n_comp):
    rows = seqlen if start == 0 else 1
    rng = np.random.default_rng(seqlen + start)
    scores = rng.standard_normal((rows, n_comp)).astype(np.float32)
    if n_comp:
        scores[:, rng.integers(0, n_comp, max(1, n_comp // 8))] = 1.0      # ties
    code, want = oracle.sel_gather_scored(scores, win, ratio, topk, seqlen, start)
    assert code == 0
    out = dzeros(want.size * 4 + 64, 0xEE)
    shape = hip.launch_sel_gather_scored(dev(scores) if n_comp else None, n_comp, win, ratio, topk, seqlen, start,
                                         out)
    assert shape == want.shape
    raw = back(out, np.int32)
    assert np.array_equal(raw[:want.size].reshape(want.shape), want)
    assert (raw[want.size:] == np.int32(-286331154)).all()


def test_random_rectangles(oracle):
    """150 random (window, ratio, phase, length) shapes, positional and scored."""
    rng = np.random.default_rng(0x5E1)
    for case in range(150):
        win = int(rng.integers(1, 200))
        ratio = int(rng.choice([0, 2, 4, 4, 8, 128]))
        if rng.random() < 0.5:
            seqlen, start = int(rng.integers(1, 600)), 0
        else:
            seqlen, start = 1, int(rng.integers(1, 5000))
        rows = seqlen if start == 0 else 1
        if ratio and rng.random() < 0.5:
            n_comp = (start + rows) // ratio
            cap = int(rng.integers(1, 40))
            scores = rng.standard_normal((rows, n_comp)).astype(np.float32).round(1)      # rounded: ties
            code, want = oracle.sel_gather_scored(scores, win, ratio, cap, seqlen, start)
            out = dzeros(want.size * 4 + 16, 0xEE)
            shape = hip.launch_sel_gather_scored(dev(scores) if n_comp else None, n_comp, win, ratio, cap, seqlen,
                                                 start, out)
        else:
            code, want = oracle.sel_gather(win, ratio, 10 ** 6, seqlen, start)
            out = dzeros(want.size * 4 + 16, 0xEE)
            shape = hip.launch_sel_gather(win, ratio, 10 ** 6, seqlen, start, out)
        assert code == 0 and shape == want.shape, (case, win, ratio, seqlen, start)
        assert np.array_equal(back(out, np.int32)[:want.size].reshape(want.shape), want), (case, win, ratio, seqlen, start)


def test_scored_equals_positional_below_the_cap(oracle):
    """select.rs:645-677 on the device, both phases."""
    for seqlen, start in ((1, 19), (12, 0), (1500, 0)):
        pos = device_gather(128, 4, 512, seqlen, start)
        rows, cols = pos.shape
        n_comp = (start + rows) // 4
        scores = np.arange(rows * n_comp, dtype=np.float32).reshape(rows, n_comp)
        out = dzeros(pos.size * 4)
        assert hip.launch_sel_gather_scored(dev(scores), n_comp, 128, 4, 512, seqlen, start, out) == (rows, cols)
        assert np.array_equal(back(out, np.int32).reshape(rows, cols), pos)


def test_selection_guards():
    b = dzeros(4096)

    def code_of(fn, *args):
        with pytest.raises(hip.LaunchError) as e:
            fn(*args)
        return e.value.code

    assert code_of(hip.sel_shape, 8, 0, 512, 3, 5) == 1005
    assert code_of(hip.sel_shape, 0, 0, 512, 1, 5) == 1001
    assert code_of(hip.sel_shape, 8, 4, 2, 1, 12) == 1006
    assert hip.sel_shape(8, 4, 2, 1, 10) == (1, 10) and hip.sel_shape(8, 2, 2, 1, 48) == (1, 8 + 24)
    assert code_of(hip.launch_sel_gather, 8, 4, 2, 1, 12, b) == 1006
    assert code_of(hip.launch_sel_gather, 8, 4, 512, 1, 12, None) == 1001
    assert code_of(hip.launch_sel_gather_scored, b, 5, 8, 0, 3, 1, 19, b) == 1001
    assert code_of(hip.launch_sel_gather_scored, b, 5, 8, 4, 3, 2, 19, b) == 1005
    assert code_of(hip.launch_sel_gather_scored, None, 5, 8, 4, 3, 1, 19, b) == 1001


@pytest.mark.parametrize("win,hd,seqlen,start", [(8, 6, 1, 5), (8, 6, 1, 21), (8, 6, 5, 0), (8, 6, 8, 0), (8, 6, 19, 0),
                                                  (8, 6, 16, 0), (128, 512, 300, 0), (128, 512, 1, 77777),
                                                  (128, 512, 100, 0), (128, 511, 257, 0)])
def test_ring_write(oracle, win, hd, seqlen, start):
    rng = np.random.default_rng(seqlen * 7 + start)
    kv = rng.standard_normal((seqlen, hd)).astype(np.float32)
    cache = rng.standard_normal((win, hd)).astype(np.float32)
    want = cache.copy()
    assert oracle.ring_write(kv, want, win, seqlen, start) == 0
    d_cache = dev(cache)
    hip.launch_kv_ring_write(dev(kv), d_cache, win, hd, seqlen, start)
    assert np.array_equal(back(d_cache, np.uint32), want.view(np.uint32).ravel())
    with pytest.raises(hip.LaunchError) as e:
        hip.launch_kv_ring_write(dev(kv), d_cache, win, hd, 2, 3)
    assert e.value.code == 1005
