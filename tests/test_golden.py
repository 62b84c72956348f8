"""The committed golden vectors (tests/golden/kvcache_golden.json, written by
tests/golden/make_golden.py): the oracle must still reproduce them, and the device path must
reproduce them through the C ABI without the oracle in the loop."""
import json
import os

import numpy as np
import pytest

from tests.golden import inputs
from tests.golden.make_golden import (OUT, PT, W, block_index_inputs, build_cases, consumer_inputs, fnv, hexs,
                                      second_format_inputs)
from tests.test_oracle_quant import fixture_a99e
from tests.topk_cases import reference_topk_cases


@pytest.fixture(scope="module")
def golden():
    assert os.path.exists(OUT), "run python -m tests.golden.make_golden"
    with open(OUT) as f:
        return json.load(f)


def test_oracle_reproduces_golden(oracle, golden):
    got = build_cases(oracle)
    assert sorted(got) == sorted(golden)
    for key in golden:
        assert got[key] == golden[key], key


def test_golden_known_values(golden):
    """Values in the file that the reference documents itself: decode(0x38) = 1.0,
    decode(0x7e) = 448, decode(0xc0) = -2.0 (crates/core/src/routing.rs:338-362); the
    half-away subnormal ties; the top-k KAT's shape (k clamps to nt)."""
    table = np.frombuffer(bytes.fromhex(golden["e4m3_decode_table_u32"]), np.uint32).view(np.float32)
    assert table[0x38] == 1.0 and table[0x7E] == 448.0 and table[0xC0] == -2.0
    assert table[0x3C] == 1.5 and table[0x18] == 0.0625 and np.isnan(table[0x7F])
    assert golden["subnormal_tie_codes"] == [1, 3, 5, 7, 8]
    assert golden["index_topk_cases"]["k > nt (wrapper clamp)"]["n"] == 500
    assert golden["index_topk_cases"]["ReLU-sparse (prefix answer)"]["head"] == [0, 1, 2, 3, 4, 5]
    # second cache format: the tie block's 448 survives, its half quanta went to the even side
    # (crates/engine/tests/kernel_v4_quant.rs:283-343); a prefill row of the selection is the
    # positional fill while its limit is within the cap (crates/engine/src/v4/select.rs:645-676)
    tie = np.frombuffer(bytes.fromhex(golden["act_quant_tie_block_u32"]), np.uint32).view(np.float32)
    q = 2.0 ** -9
    assert tie[0] == 448.0 and (tie[[2, 4, 6, 8, 10]] / q).tolist() == [-0.0, -2.0, -2.0, -4.0, -4.0]
    assert golden["scored_rows"]["prefill_row9"] == [128, 129, -1, -1]
    assert sorted(golden["scored_rows"]["prefill_row23"]) == golden["scored_rows"]["prefill_row23"]


@pytest.mark.gpu
def test_device_reproduces_golden(oracle, golden):
    """Same inputs (their hashes are checked first), outputs from the HIP library only."""
    from rivoli_amd import hip
    from tests.gpu_util import back, dev, dzeros

    # codecs
    sweep = (np.arange(1 << 16, dtype=np.uint32) << np.uint32(16)).view(np.float32)
    finite = sweep[np.isfinite(sweep)]
    codes = dzeros(finite.size)
    hip.launch_codec_e4m3_encode(dev(finite), codes, finite.size)
    assert fnv(oracle, back(codes)) == golden["e4m3_encode_all_bf16_values"]["fnv"]
    dec = dzeros(256 * 2)
    hip.launch_codec_e4m3_dequant_bf16(dev(np.arange(256, dtype=np.uint8)), 1.0, dec, 256)
    table = np.frombuffer(bytes.fromhex(golden["e4m3_decode_table_u32"]), np.uint32)
    finite_codes = (np.arange(256) & 0x7F) != 0x7F
    assert np.array_equal(back(dec, np.uint16)[finite_codes], (table >> 16).astype(np.uint16)[finite_codes])

    # the reference's append_kv fixture
    g = golden["append_kv_a99e"]
    rows, kvl, ropn, pos, nb = 5, 256, 64, 3, 2
    latent, rope = fixture_a99e(oracle)
    assert fnv(oracle, latent) == g["latent_fnv"] and fnv(oracle, rope) == g["rope_fnv"]
    c8, ls, rc = dzeros(rows * kvl), dzeros(rows * nb * 4), dzeros(rows * ropn * 2)
    hip.launch_append_kv(dev(latent), dev(rope), c8, ls, rc, pos, kvl, ropn, nb)
    assert hexs(back(c8)[pos * kvl:(pos + 1) * kvl]) == g["codes_row3"]
    assert hexs(back(ls, np.uint32)[pos * nb:(pos + 1) * nb]) == g["scales_row3_u32"]
    assert hexs(back(rc, np.uint16)[pos * ropn:(pos + 1) * ropn]) == g["rope_row3_bf16"]

    # the ten index_topk cases
    for name, scores, k in reference_topk_cases(oracle):
        c = golden["index_topk_cases"][name]
        assert fnv(oracle, scores) == c["scores_fnv"], name
        out = dzeros(max(scores.size, k) * 4, 0xFF)
        hip.launch_index_topk(dev(scores), scores.size, k, out)
        sel = back(out, np.uint32)[:c["n"]]
        assert fnv(oracle, sel) == c["fnv"], name
        assert [int(v) for v in sel[:6]] == c["head"] and [int(v) for v in sel[-3:]] == c["tail"], name

    # configuration 1: all but the last token, then the last token, then the full gather
    g = golden["config1"]
    rows1, table1, slots1 = inputs.config1(oracle)
    assert fnv(oracle, rows1) == g["rows_fnv"] and fnv(oracle, table1) == g["table_fnv"]
    n, pb = rows1.shape[0], hip.kv_page_bytes(PT, W)
    pool, rows_d, slots_d = dzeros(table1.size * pb), dev(rows1), dev(slots1)
    hip.launch_kv_append_paged(rows_d, slots_d, pool, n - 1, W, PT, table1.size)
    assert fnv(oracle, back(pool)) == g["pool_before_last_fnv"]
    hip.launch_kv_append_paged(rows_d[(n - 1) * W * 2:], slots_d[(n - 1) * 4:], pool, 1, W, PT, table1.size)
    assert fnv(oracle, back(pool)) == g["pool_fnv"]
    out = dzeros(n * W * 2)
    lens = np.array([n], np.int32)
    hip.launch_kv_gather_paged(pool, dev(table1), dev(lens), dev(np.array([0, n], np.int32)), out, 1,
                               table1.shape[1], W, PT, table1.size)
    got = back(out, np.uint16).reshape(n, W)
    assert fnv(oracle, got) == g["gather_fnv"] and hexs(got[0, :8]) == g["gather_row0_head"]

    # configuration 2
    g = golden["config2"]
    rows2, table2, slots2 = inputs.config2(oracle)
    assert fnv(oracle, rows2) == g["rows_fnv"] and fnv(oracle, slots2) == g["slots_fnv"]
    pool2 = dzeros(table2.size * pb)
    hip.launch_kv_append_paged(dev(rows2), dev(slots2), pool2, rows2.shape[0], W, PT, table2.size)
    assert fnv(oracle, back(pool2)) == g["pool_fnv"]

    # configuration 4, small
    g = golden["config4_small"]
    rows4, table4, slots4, scores4, k4 = inputs.config4_small(oracle)
    assert fnv(oracle, rows4) == g["rows_fnv"] and fnv(oracle, scores4) == g["scores_fnv"]
    assert fnv(oracle, table4) == g["table_fnv"]
    n_q, nt = scores4.shape
    pool4 = dzeros(table4.size * pb)
    hip.launch_kv_append_paged(dev(rows4), dev(slots4), pool4, rows4.shape[0], W, PT, table4.size)
    assert fnv(oracle, back(pool4)) == g["pool_fnv"]
    sel = dzeros(n_q * k4 * 4, 0xFF)
    hip.launch_index_topk_batched(dev(scores4), n_q, nt, None, nt, k4, sel)
    sel_np = back(sel, np.uint32).reshape(n_q, k4)
    assert fnv(oracle, sel_np) == g["selected_fnv"]
    assert [int(v) for v in sel_np[0, :6]] == g["selected_q0_head"]
    out4 = dzeros(n_q * k4 * W * 2)
    hip.launch_kv_gather_rows_paged(pool4, dev(table4), sel, None, out4, n_q, k4, table4.shape[1], W, PT,
                                    table4.size)
    assert fnv(oracle, back(out4, np.uint16)) == g["gather_rows_fnv"]


@pytest.mark.gpu
def test_device_reproduces_second_format_golden(oracle, golden):
    from rivoli_amd import hip
    from tests.gpu_util import back, dev, dzeros
    from tests.test_oracle_v4 import reference_tie_block
    from tests.v4_cases import compress_gap

    rows, scores, (geom, kv, score, ape, norm, freqs) = second_format_inputs(oracle)
    tie = dev(reference_tie_block())
    hip.launch_act_quant_f8_prefix(tie, tie, 1, 64, 64, 64)
    assert hexs(back(tie, np.uint32)) == golden["act_quant_tie_block_u32"]
    g = golden["act_quant_rows"]
    assert fnv(oracle, rows) == g["rows_fnv"]
    rows_d = dev(rows)
    hip.launch_act_quant_f8_prefix(rows_d, rows_d, 24, 512, 448, 64)
    got = back(rows_d, np.uint32).reshape(24, 512)
    assert fnv(oracle, got) == g["fnv"] and hexs(got[0, :8]) == g["row0_head_u32"]

    g = golden["scored_rows"]
    assert fnv(oracle, scores) == g["scores_fnv"]
    for prefill, cap, key, row, idx in ((True, 4, "prefill_fnv", "prefill_row23", 23),
                                        (False, 6, "decode_fnv", "decode_row0", 0)):
        out = dzeros(24 * cap * 4, 0xEE)
        hip.launch_index_select_blocks(dev(scores), 24, 40, 4, cap, prefill, 128, out)
        sel = back(out, np.int32).reshape(24, cap)
        assert fnv(oracle, sel) == g[key] and [int(v) for v in sel[idx]] == g[row]

    g = golden["compress_prefill_ratio4"]
    assert fnv(oracle, kv) == g["kv_fnv"] and fnv(oracle, score) == g["score_fnv"]
    out = dzeros(4 * geom.d * 4)
    norm_d, freqs_d = dev(norm), dev(freqs)
    hip.launch_kv_compress_prefill(dev(kv), dev(score), dev(ape), hip.CompFinish.of(norm_d, freqs_d, out),
                                   hip.CompGeom.build(4, 64, 16, 1e-6), 4)
    want = np.frombuffer(bytes.fromhex(g["out_u32"]), np.uint32).view(np.float32).reshape(4, geom.d)
    assert compress_gap(oracle, back(out, np.float32).reshape(4, geom.d), want, 16).max() <= 2


def test_golden_consumer_known_values(golden):
    """What the reference's own unit cases fix about these vectors
    (crates/engine/src/v4/select.rs:533-553): a prefill row reads the last `win` positions up to
    its own, then the blocks that have closed, shifted past the prompt; a decode row reads the
    full ring oldest first."""
    g = golden["selection_rectangles"]
    assert g["prefill_shape"] == [24, 8 + 6]
    assert g["prefill_row10"] == [3, 4, 5, 6, 7, 8, 9, 10] + [24, 25, -1, -1, -1, -1]
    assert g["decode_row"] == [6, 7, 0, 1, 2, 3, 4, 5] + [8, 9, 10, 11, 12]
    assert g["scored_shape"] == [24, 8 + 3] and g["scored_row23"][:8] == list(range(16, 24))
    assert all(24 <= v < 30 for v in g["scored_row23"][8:]) and g["scored_row23"][8:] == sorted(g["scored_row23"][8:])


@pytest.mark.gpu
def test_device_reproduces_consumer_golden(oracle, golden):
    from rivoli_amd import hip
    from tests.gpu_util import back, dev, dzeros

    n, h, d, kv, q, sink, scores = consumer_inputs(oracle)
    g = golden["selection_rectangles"]
    rows, cols = g["prefill_shape"]
    out = dzeros(rows * cols * 4, 0xEE)
    assert hip.launch_sel_gather(8, 4, 512, n, 0, out) == (rows, cols)
    pos = back(out, np.int32).reshape(rows, cols)
    assert fnv(oracle, pos) == g["prefill_fnv"] and [int(v) for v in pos[10]] == g["prefill_row10"]
    out = dzeros(13 * 4, 0xEE)
    assert hip.launch_sel_gather(8, 4, 512, 1, 21, out) == (1, 13)
    assert [int(v) for v in back(out, np.int32)] == g["decode_row"]
    rows, cols = g["scored_shape"]
    idx_d = dzeros(rows * cols * 4, 0xEE)
    assert hip.launch_sel_gather_scored(dev(scores), n // 4, 8, 4, 3, n, 0, idx_d) == (rows, cols)
    scored = back(idx_d, np.int32).reshape(rows, cols)
    assert fnv(oracle, scored) == g["scored_fnv"] and [int(v) for v in scored[23]] == g["scored_row23"]
    ring = dzeros(8 * d * 4)
    hip.launch_kv_ring_write(dev(kv[:n]), ring, 8, d, n, 0)
    assert fnv(oracle, back(ring, np.float32).reshape(8, d)) == golden["ring_after_prefill_fnv"]
    g = golden["gather_attn"]
    assert fnv(oracle, q) == g["q_fnv"] and fnv(oracle, kv) == g["kv_fnv"]
    o = dzeros(n * h * d * 4)
    hip.launch_gather_attn_shared_kv(dev(q), dev(kv), dev(sink), idx_d, n, h, d, cols, d ** -0.5, o)
    got = back(o, np.float32).reshape(n, h, d)
    want = np.frombuffer(bytes.fromhex(g["row23_head0_u32"]), np.uint32).view(np.float32)
    # the reference's bar for this kernel: 1/128 of the largest expected element
    assert np.max(np.abs(got[23, 0] - want)) <= np.max(np.abs(want)) / 128.0


@pytest.mark.gpu
def test_device_reproduces_block_index_golden(oracle, golden):
    """The Hadamard + fp4 spread and the block scores from the HIP library only."""
    from rivoli_amd import hip
    from tests.gpu_util import back, dev, dzeros

    g = golden["block_index"]
    q, kv, w = block_index_inputs(oracle)
    assert (fnv(oracle, q), fnv(oracle, kv), fnv(oracle, w)) == (g["q_fnv"], g["kv_fnv"], g["w_fnv"])
    q_d, kv_d = dev(q), dev(kv)
    hip.launch_act_quant_f4_rotated(q_d, 12, 128)
    hip.launch_act_quant_f4_rotated(kv_d, 20, 128)
    sq = back(q_d, np.uint32).reshape(12, 128)
    assert fnv(oracle, sq) == g["spread_q_fnv"] and hexs(sq[0, :8]) == g["spread_q_row0_head_u32"]
    assert fnv(oracle, back(kv_d, np.uint32)) == g["spread_kv_fnv"]
    out = dzeros(3 * 20 * 4, 0x5A)
    hip.launch_index_score_blocks(q_d, kv_d, dev(w), out, 3, 20, 4, 128)
    assert hexs(back(out, np.uint32)) == g["scores_u32"]
