"""Writes tests/golden/kvcache_golden.json from the CPU oracle.

The reference stores no vectors for this path (its tests compute every expectation at run
time), so the committed vectors are the oracle's own outputs, taken only AFTER the oracle has
passed the reference's known answers and the invariant checks in tests/test_oracle_*.py —
this script runs those first and refuses to write when any fails. Small outputs are stored
in full (hex); large ones as the reference's own pinning idiom, an FNV-1a hash of the bytes
(crates/core/src/hash.rs:1-25), together with a few leading values.

    python -m tests.golden.make_golden
"""
import json
import os
import subprocess
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
OUT = os.path.join(HERE, "kvcache_golden.json")
W, PT = 576, 64


def fnv(oracle, a) -> str:
    return f"{oracle.fnv1a(np.ascontiguousarray(a).tobytes()):016x}"


def hexs(a) -> str:
    return np.ascontiguousarray(a).tobytes().hex()


def build_cases(oracle) -> dict:
    """Every golden case, computed by the oracle. Shared with the tests, which recompute the
    same dict (from the oracle, or from the device) and compare it with the stored one."""
    from tests.golden import inputs
    from tests.test_oracle_quant import fixture_a99e
    from tests.topk_cases import reference_topk_cases

    g = {}
    # -- codecs: the whole decode table and an encode sweep over every f32 exponent ----------
    codes = np.arange(256, dtype=np.uint8)
    g["e4m3_decode_table_u32"] = hexs(oracle.e4m3_to_f32(codes).view(np.uint32))
    sweep = (np.arange(1 << 16, dtype=np.uint32) << np.uint32(16)).view(np.float32)  # all bf16 values
    finite = sweep[np.isfinite(sweep)]
    g["e4m3_encode_all_bf16_values"] = {"n": int(finite.size), "fnv": fnv(oracle, oracle.f32_to_e4m3(finite))}
    g["subnormal_tie_codes"] = [int(c) for c in oracle.f32_to_e4m3(
        np.array([1, 5, 9, 13, 15], np.float32) * np.float32(2.0 ** -10))]

    # -- the reference's append_kv fixture (crates/engine/tests/fwd_kernel.rs:139-214) -------
    rows, kvl, ropn, pos, nb = 5, 256, 64, 3, 2
    latent, rope = fixture_a99e(oracle)
    lc8, ls, rc = np.zeros(rows * kvl, np.uint8), np.zeros(rows * nb, np.float32), np.zeros(rows * ropn, np.uint16)
    assert oracle.append_kv(latent, rope, lc8, ls, rc, pos, kvl, ropn, nb) == 0
    g["append_kv_a99e"] = {
        "latent_fnv": fnv(oracle, latent), "rope_fnv": fnv(oracle, rope),
        "codes_row3": hexs(lc8[pos * kvl:(pos + 1) * kvl]),
        "scales_row3_u32": hexs(ls[pos * nb:(pos + 1) * nb].view(np.uint32)),
        "rope_row3_bf16": hexs(rc[pos * ropn:(pos + 1) * ropn]),
    }

    # -- the ten index_topk cases (crates/engine/tests/kernel_vector.rs:132-170) -------------
    tk = {}
    for name, scores, k in reference_topk_cases(oracle):
        sel = oracle.topk(scores, k)
        tk[name] = {"scores_fnv": fnv(oracle, scores), "n": int(sel.size), "fnv": fnv(oracle, sel),
                    "head": [int(v) for v in sel[:6]], "tail": [int(v) for v in sel[-3:]]}
    g["index_topk_cases"] = tk

    # -- benchmark configuration 1: append the last token, gather the whole context ----------
    rows1, table1, slots1 = inputs.config1(oracle)
    pb = oracle.kv_page_bytes(PT, W)
    pool = np.zeros(table1.size * pb, np.uint8)
    oracle.kv_append_paged(rows1[:-1], slots1[:-1], pool, W, PT, table1.size)
    before = fnv(oracle, pool)
    oracle.kv_append_paged(rows1[-1:], slots1[-1:], pool, W, PT, table1.size)
    out1 = oracle.kv_gather_paged(pool, table1, np.array([rows1.shape[0]], np.int32), W, PT)
    g["config1"] = {"rows_fnv": fnv(oracle, rows1), "table_fnv": fnv(oracle, table1),
                    "pool_before_last_fnv": before, "pool_fnv": fnv(oracle, pool),
                    "gather_fnv": fnv(oracle, out1), "gather_row0_head": hexs(out1[0, :8]),
                    "last_scale_u32": hexs(pool[int(slots1[-1]) // PT * pb + PT * W + (int(slots1[-1]) % PT) * 4:][:4])}

    # -- benchmark configuration 2: bulk append with x50 outlier rows ------------------------
    rows2, table2, slots2 = inputs.config2(oracle)
    pool2 = np.zeros(table2.size * pb, np.uint8)
    oracle.kv_append_paged(rows2, slots2, pool2, W, PT, table2.size)
    g["config2"] = {"rows_fnv": fnv(oracle, rows2), "slots_fnv": fnv(oracle, slots2),
                    "pool_fnv": fnv(oracle, pool2)}

    # -- benchmark configuration 4, small: top-k then sparse gather --------------------------
    rows4, table4, slots4, scores4, k4 = inputs.config4_small(oracle)
    pool4 = np.zeros(table4.size * pb, np.uint8)
    oracle.kv_append_paged(rows4, slots4, pool4, W, PT, table4.size)
    sel4 = oracle.topk_batched(scores4, k4)
    out4 = oracle.kv_gather_rows_paged(pool4, table4, sel4, W, PT)
    g["config4_small"] = {"rows_fnv": fnv(oracle, rows4), "scores_fnv": fnv(oracle, scores4),
                          "table_fnv": fnv(oracle, table4), "pool_fnv": fnv(oracle, pool4),
                          "selected_fnv": fnv(oracle, sel4), "selected_q0_head": [int(v) for v in sel4[0, :6]],
                          "gather_rows_fnv": fnv(oracle, out4)}
    g.update(second_format_cases(oracle))
    return g


def second_format_inputs(oracle):
    """Seeded inputs of the second cache format's cases, from the reference tests' own
    generator (crates/engine/tests/common/reference.rs:141-162)."""
    from oracle.kvoracle import CompGeom

    lcg = oracle.lcg(0x5EED0006)
    rows = (lcg.fill(24 * 512) * np.float32(2.0)).reshape(24, 512)
    rows[3, 64:128] = 0.0                                   # an all-zero block: the amax floor
    rows[5] *= np.float32(200.0)
    scores = lcg.fill(24 * 40).reshape(24, 40)
    scores[:, ::5] = np.float32(0.25)                       # ties
    geom = CompGeom.attention(4, 64, 16)
    kv, score = lcg.fill(16 * geom.cd).reshape(16, geom.cd), lcg.fill(16 * geom.cd).reshape(16, geom.cd)
    ape, norm = lcg.fill(4 * geom.cd).reshape(4, geom.cd), np.float32(1.0) + np.float32(0.1) * lcg.fill(geom.d)
    ang = np.arange(16, dtype=np.float64)[:, None] * (10000.0 ** (-np.arange(8) / 8.0))[None, :]
    freqs = np.stack([np.cos(ang), np.sin(ang)], axis=-1).reshape(16, 16).astype(np.float32)
    return rows, scores, (geom, kv, score, ape, norm, freqs)


def second_format_cases(oracle) -> dict:
    from tests.test_oracle_v4 import reference_tie_block

    rows, scores, (geom, kv, score, ape, norm, freqs) = second_format_inputs(oracle)
    g = {}
    # the reference's tie fixture (crates/engine/tests/kernel_v4_quant.rs:283-296), in full
    code, tie = oracle.act_quant_f8_prefix(reference_tie_block()[None, :], 64, 64)
    assert code == 0
    g["act_quant_tie_block_u32"] = hexs(tie.view(np.uint32))
    code, q = oracle.act_quant_f8_prefix(rows, 448, 64)
    assert code == 0
    g["act_quant_rows"] = {"rows_fnv": fnv(oracle, rows), "fnv": fnv(oracle, q),
                           "row0_head_u32": hexs(q[0, :8].view(np.uint32))}
    sel_p = oracle.v4_scored_rows(scores, 4, 4, True, 128)
    sel_d = oracle.v4_scored_rows(scores, 4, 6, False, 128)
    g["scored_rows"] = {"scores_fnv": fnv(oracle, scores), "prefill_fnv": fnv(oracle, sel_p),
                        "prefill_row23": [int(v) for v in sel_p[23]], "prefill_row9": [int(v) for v in sel_p[9]],
                        "decode_fnv": fnv(oracle, sel_d), "decode_row0": [int(v) for v in sel_d[0]]}
    # the compressor pooling: a small overlapping case in full (the device matches it to within
    # two bf16 codes, not bit for bit)
    code, out = oracle.kv_compress_prefill(kv, score, ape, norm, freqs, geom, 4)
    assert code == 0
    g["compress_prefill_ratio4"] = {"kv_fnv": fnv(oracle, kv), "score_fnv": fnv(oracle, score),
                                    "out_u32": hexs(out.view(np.uint32))}
    g.update(consumer_cases(oracle))
    g.update(block_index_cases(oracle))
    return g


def block_index_inputs(oracle):
    """Seeded inputs of the block indexer's cases: 3 queries x 4 index heads and 20 block rows
    of 128 bf16 values, rows scaled over several binades; signed bf16 head weights."""
    lcg = oracle.lcg(0x5EED0009)

    def bf16_values(x):
        return (oracle.f32_to_bf16(x).astype(np.uint32) << 16).view(np.float32)

    q = bf16_values(lcg.fill(12 * 128).reshape(12, 128) * (np.float32(2.0) ** np.arange(-6, 6))[:, None].astype(np.float32))
    kv = bf16_values(lcg.fill(20 * 128).reshape(20, 128) * np.float32(3.0))
    w = bf16_values(lcg.fill(3 * 4).reshape(3, 4) * np.float32(0.1))
    return q, kv, w


def block_index_cases(oracle) -> dict:
    q, kv, w = block_index_inputs(oracle)
    (cq, sq), (ck, skv) = oracle.act_quant_f4_rotated(q), oracle.act_quant_f4_rotated(kv)
    cs, score = oracle.index_score_blocks(sq.reshape(3, 4, 128), skv, w)
    assert cq == ck == cs == 0
    return {"block_index": {"q_fnv": fnv(oracle, q), "kv_fnv": fnv(oracle, kv), "w_fnv": fnv(oracle, w),
                            "spread_q_fnv": fnv(oracle, sq), "spread_q_row0_head_u32": hexs(sq[0, :8].view(np.uint32)),
                            "spread_kv_fnv": fnv(oracle, skv), "scores_u32": hexs(score.view(np.uint32))}}


def consumer_inputs(oracle):
    """Seeded inputs of the selection / ring / attention cases: a 24-token prompt on the indexed
    class (window 8, ratio 4), 4 heads of width 64; cache rows and q are bf16 values."""
    lcg = oracle.lcg(0x5EED0008)
    n, h, d = 24, 4, 64
    def bf16_values(x):
        return (oracle.f32_to_bf16(x).astype(np.uint32) << 16).view(np.float32)

    kv = bf16_values(lcg.fill((n + n // 4) * d)).reshape(n + n // 4, d)
    q = bf16_values(lcg.fill(n * h * d) * np.float32(2.0)).reshape(n, h, d)
    sink = lcg.fill(h)
    scores = lcg.fill(n * (n // 4)).reshape(n, n // 4)
    return n, h, d, kv, q, sink, scores


def consumer_cases(oracle) -> dict:
    n, h, d, kv, q, sink, scores = consumer_inputs(oracle)
    g = {}
    code, pos = oracle.sel_gather(8, 4, 512, n, 0)
    assert code == 0
    code, dec = oracle.sel_gather(8, 4, 512, 1, 21)
    assert code == 0
    code, scored = oracle.sel_gather_scored(scores, 8, 4, 3, n, 0)
    assert code == 0
    g["selection_rectangles"] = {"prefill_shape": list(pos.shape), "prefill_fnv": fnv(oracle, pos),
                                 "prefill_row10": [int(v) for v in pos[10]],
                                 "decode_row": [int(v) for v in dec[0]],
                                 "scored_shape": list(scored.shape), "scored_fnv": fnv(oracle, scored),
                                 "scored_row23": [int(v) for v in scored[23]]}
    ring = np.zeros((8, d), np.float32)
    assert oracle.ring_write(kv[:n], ring, 8, n, 0) == 0
    g["ring_after_prefill_fnv"] = fnv(oracle, ring)
    out = oracle.sparse_attn(q, kv, sink, scored, d ** -0.5)
    # the device matches this to the reference's bar (1/128 of the largest element), not bit for bit
    g["gather_attn"] = {"q_fnv": fnv(oracle, q), "kv_fnv": fnv(oracle, kv),
                        "row23_head0_u32": hexs(out[23, 0].view(np.uint32)), "out_fnv": fnv(oracle, out)}
    return g


def main() -> None:
    sys.path.insert(0, ROOT)
    rc = subprocess.run([sys.executable, "-m", "pytest", "-q", "-x", "-m", "not gpu",
                         os.path.join(ROOT, "tests", "test_oracle_codecs.py"),
                         os.path.join(ROOT, "tests", "test_oracle_quant.py"),
                         os.path.join(ROOT, "tests", "test_oracle_topk_hash.py"),
                         os.path.join(ROOT, "tests", "test_oracle_v4.py"),
                         os.path.join(ROOT, "tests", "test_oracle_v4_compress.py"),
                         os.path.join(ROOT, "tests", "test_oracle_v4_select.py"),
                         os.path.join(ROOT, "tests", "test_oracle_v4_blockindex.py")], cwd=ROOT).returncode
    if rc != 0:
        sys.exit("the oracle does not pass its known-answer tests: no vectors written")
    from oracle.kvoracle import oracle as get_oracle

    g = build_cases(get_oracle())
    with open(OUT, "w") as f:
        json.dump(g, f, indent=1, sort_keys=True)
        f.write("\n")
    print("wrote", OUT, os.path.getsize(OUT), "bytes")


if __name__ == "__main__":
    main()
