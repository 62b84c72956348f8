"""The compressor's pooling stage on the device against the CPU oracle. The deposit is copies
and one add: bit-exact. Pooling, norm and rotation go through expf and a block reduction, so
the bar is the reference's own for these kernels: at most 2 bf16 codes apart
(crates/engine/tests/v4_compressor/metric.rs, CLEAN_ULP = 2), with almost every element equal;
values that cancelled to almost nothing are compared absolutely (tests/v4_cases.py)."""
import ctypes as C

import numpy as np
import pytest

from oracle.kvoracle import CompGeom as OracleGeom
from rivoli_amd import hip
from tests.gpu_util import back, dev, dzeros, need_ref
from tests.v4_cases import compress_gap, compress_inputs

pytestmark = pytest.mark.gpu
CLEAN_ULP = 2


def geoms(ratio, d, rd):
    return OracleGeom.attention(ratio, d, rd), hip.CompGeom.build(ratio, d, rd, 1e-6)


def fresh_states(g):
    """kv zeroed, scores -inf (crates/engine/src/v4/kvcompress.rs:222)."""
    return [np.zeros((g.coff * g.ratio, g.cd), np.float32),
            np.full((g.coff * g.ratio, g.cd), -np.inf, np.float32)]


def device_prefill(hg, kv, score, ape, norm, freqs, nblk, launch=None):
    out = dzeros(nblk * hg.d * 4, 0xEE)
    bufs = [dev(a) for a in (kv, score, ape, norm, freqs)]
    fin = hip.CompFinish.of(bufs[3], bufs[4], out)
    if launch is None:
        hip.launch_kv_compress_prefill(bufs[0], bufs[1], bufs[2], fin, hg, nblk)
    else:
        assert launch(bufs[0].data_ptr(), bufs[1].data_ptr(), bufs[2].data_ptr(), C.byref(fin),
                      C.byref(hg), nblk, None) == 0
    return back(out, np.float32).reshape(nblk, hg.d)


def assert_clean(oracle, got, want, what, rd):
    gap = compress_gap(oracle, got, want, rd)
    assert gap.max() <= CLEAN_ULP and np.mean(gap > 0) < 0.01, (what, int(gap.max()), float(np.mean(gap > 0)))


@pytest.mark.parametrize("ratio,d,rd,s", [(4, 512, 64, 1024), (128, 512, 64, 1024), (4, 64, 16, 45),
                                          (8, 34, 8, 80), (16, 128, 32, 160), (32, 130, 64, 96),
                                          (4, 2048, 64, 64)])
def test_prefill_matches_oracle(oracle, ratio, d, rd, s):
    """The shipped geometries (overlapping ratio 4, ratio 128) and odd ones: widths that are
    not a multiple of four, a window of exactly 16, a row wider than one pass of the workgroup."""
    og, hg = geoms(ratio, d, rd)
    kv, score, ape, norm, freqs = compress_inputs(og, s, seed=ratio * 31 + d)
    nblk = s // ratio
    code, want = oracle.kv_compress_prefill(kv, score, ape, norm, freqs, og, nblk)
    assert code == 0
    got = device_prefill(hg, kv, score, ape, norm, freqs, nblk)
    assert_clean(oracle, got, want, f"ratio {ratio} d {d}", rd)


@pytest.mark.parametrize("ratio,d,rd,s", [(4, 512, 64, 1024), (128, 512, 64, 1024), (4, 64, 16, 45),
                                          (8, 34, 8, 80), (16, 128, 32, 160), (32, 130, 64, 96)])
def test_reference_prefill_agrees_with_the_oracle(oracle, ratio, d, rd, s):
    """The reference's own kernel (kvcompress.hip compiled for this GPU; widths it accepts)."""
    ref = need_ref("rivoli_kv_compress_prefill")
    og, hg = geoms(ratio, d, rd)
    kv, score, ape, norm, freqs = compress_inputs(og, s, seed=ratio * 31 + d)
    nblk = s // ratio
    code, want = oracle.kv_compress_prefill(kv, score, ape, norm, freqs, og, nblk)
    assert code == 0
    theirs = device_prefill(hg, kv, score, ape, norm, freqs, nblk, launch=ref.rivoli_kv_compress_prefill)
    assert_clean(oracle, theirs, want, f"reference kernel, ratio {ratio} d {d}", rd)


def test_masked_and_peaked_windows(oracle):
    og, hg = geoms(4, 512, 64)
    kv, score, ape, norm, freqs = compress_inputs(og, 64, seed=77)
    score[20:24] = -np.inf                                # a whole block of masked rows
    score[30, :] = 90.0                                   # one row dominates both its windows
    score[40, 100:200] = -np.inf
    code, want = oracle.kv_compress_prefill(kv, score, ape, norm, freqs, og, 16)
    got = device_prefill(hg, kv, score, ape, norm, freqs, 16)
    assert code == 0 and np.isfinite(want).all()
    assert_clean(oracle, got, want, "masked / peaked", 64)


@pytest.mark.parametrize("ratio,d,rd,s,s0", [(4, 512, 64, 45, 14), (4, 64, 16, 30, 2), (128, 512, 64, 400, 130),
                                              (8, 32, 8, 50, 19)])
def test_deposit_and_decode_follow_the_state_machine(oracle, ratio, d, rd, s, s0):
    """Prefill s0 tokens, then one token at a time. The deposit is bit-exact against the oracle
    at every step; every emitted block is within the bar of the oracle's AND bit-identical to
    the device's own prefill of the whole sequence (both arms run the same fold)."""
    og, hg = geoms(ratio, d, rd)
    kv, score, ape, norm, freqs = compress_inputs(og, s, seed=s + ratio)
    want_states = fresh_states(og)
    st = [dev(a) for a in want_states]
    kv_d, sc_d, ape_d, norm_d, freqs_d = (dev(a) for a in (kv, score, ape, norm, freqs))
    row_bytes = og.cd * 4

    def check_states(what):
        for name, d_buf, w in (("kv", st[0], want_states[0]), ("score", st[1], want_states[1])):
            assert np.array_equal(back(d_buf, np.uint32), w.view(np.uint32).ravel()), (what, name)

    hip.launch_kv_compress_deposit(kv_d, sc_d, ape_d, st[0], st[1], hg, s0, 0)
    assert oracle.kv_compress_deposit(kv[:s0], score[:s0], ape, want_states[0], want_states[1], og, s0, 0) == 0
    check_states("prefill deposit")
    blocks, want_blocks = [], []
    if s0 >= ratio:
        blocks += list(device_prefill(hg, kv[:s0], score[:s0], ape, norm, freqs, s0 // ratio))
        want_blocks += list(oracle.kv_compress_prefill(kv[:s0], score[:s0], ape, norm, freqs, og, s0 // ratio)[1])
    out = dzeros(og.d * 4)
    fin = hip.CompFinish.of(norm_d, freqs_d, out)
    for pos in range(s0, s):
        hip.launch_kv_compress_deposit(kv_d.data_ptr() + pos * row_bytes, sc_d.data_ptr() + pos * row_bytes,
                                       ape_d, st[0], st[1], hg, 1, pos % ratio)
        assert oracle.kv_compress_deposit(kv[pos:pos + 1], score[pos:pos + 1], ape, want_states[0],
                                          want_states[1], og, 1, pos % ratio) == 0
        if (pos + 1) % ratio == 0:
            hip.launch_kv_compress_decode(st[0], st[1], fin, hg, pos)
            blocks.append(back(out, np.float32).copy())
            code, w = oracle.kv_compress_decode(want_states[0], want_states[1], norm, freqs, og, pos)
            assert code == 0
            want_blocks.append(w)
            check_states(f"after the block at {pos}")     # the slide is bit-exact too
    blocks, want_blocks = np.array(blocks), np.array(want_blocks)
    assert_clean(oracle, blocks, want_blocks, "stepped blocks", rd)
    whole = device_prefill(hg, kv, score, ape, norm, freqs, s // ratio)
    assert np.array_equal(blocks.view(np.uint32), whole.view(np.uint32))


def test_compress_guards():
    hg = hip.CompGeom.build(4, 32, 8, 1e-6)
    b = dzeros(1 << 16)
    fin = hip.CompFinish.of(b, b, b)

    def code_of(fn, *args):
        with pytest.raises(hip.LaunchError) as e:
            fn(*args)
        return e.value.code

    assert code_of(hip.launch_kv_compress_deposit, b, b, b, b, b, None, 1, 0) == 1000
    assert code_of(hip.launch_kv_compress_prefill, b, b, b, None, hg, 1) == 1000
    assert code_of(hip.launch_kv_compress_decode, b, b, fin, None, 3) == 1000
    for geom, code in ((hip.CompGeom(1, 1, 32, 32, 1, 8, 1e-6), 1001), (hip.CompGeom(4, 2, 32, 64, 8, 7, 1e-6), 1002),
                       (hip.CompGeom(4, 2, 32, 32, 8, 8, 1e-6), 1003), (hip.CompGeom(256, 1, 32, 32, 256, 8, 1e-6), 1004),
                       (hip.CompGeom(8, 2, 32, 64, 16, 8, 1e-6), 1010)):
        assert code_of(hip.launch_kv_compress_prefill, b, b, b, fin, geom, 1) == code
        assert code_of(hip.launch_kv_compress_deposit, b, b, b, b, b, geom, 1, 0) == code
        assert code_of(hip.launch_kv_compress_decode, b, b, fin, geom, 3) == code
    assert code_of(hip.launch_kv_compress_deposit, b, b, b, b, b, hg, 0, 0) == 1005
    assert code_of(hip.launch_kv_compress_deposit, b, b, b, b, b, hg, 3, 2) == 1008
    assert code_of(hip.launch_kv_compress_deposit, None, b, b, b, b, hg, 1, 0) == 1001
    assert code_of(hip.launch_kv_compress_prefill, b, b, b, fin, hg, 0) == 1006
    assert code_of(hip.launch_kv_compress_prefill, b, b, b, hip.CompFinish.of(b, b, None), hg, 1) == 1001
    assert code_of(hip.launch_kv_compress_decode, b, b, fin, hg, 0) == 1007
    assert code_of(hip.launch_kv_compress_decode, b, b, fin, hg, 5) == 1009
    assert code_of(hip.launch_kv_compress_prefill, b, b, b, fin, hip.CompGeom.build(4, 16384, 8, 1e-6), 1) == 1002
