"""Pins the attention oracle: against an independent float64 restatement, against closed
forms a wrong index, a dropped term or a transposed operand cannot satisfy, and the paged and
linear forms against each other. The reference computes its own expectation for this kernel
with the same formula at test time (crates/engine/tests/kernel_attend.rs:201-226) and stores
no vectors, so there is nothing else to compare with."""
import numpy as np
import pytest

from tests.attend_cases import attend_f64, paged_case, reference_attend_case, widen_linear, widen_paged

REFERENCE_SHAPES = [  # crates/engine/tests/kernel_attend.rs:270-307: seed, h, nt, kvl, rope
    (0x0A5E1102, 64, 300, 512, 64),
    (0x5F117BAD, 64, 704, 512, 64),
    (0x00C0FFEE, 4, 1, 128, 8),
    (0xB10CC0DE, 20, 130, 512, 64),
]


def rel_err(got, want):
    return float(np.abs(got.astype(np.float64) - want).max() / max(np.abs(want).max(), 1e-30))


@pytest.mark.parametrize("seed,h,nt,kvl,rope", REFERENCE_SHAPES)
def test_linear_form_matches_float64_on_the_reference_shapes(oracle, seed, h, nt, kvl, rope):
    qabs, qrope, lc8, lscale, rc, nb, scale = reference_attend_case(oracle, seed, h, nt, kvl, rope)
    code, got = oracle.mla_attend(qabs, qrope, lc8, lscale, rc, None, h, nt, kvl, rope, nb, scale)
    assert code == 0
    lat, rk = widen_linear(oracle, lc8, lscale, rc, nt, kvl, rope, nb)
    assert rel_err(got, attend_f64(qabs, qrope, lat, rk, scale)) < 1e-5
    # and the widened-rows entry point is the same computation
    assert np.array_equal(got, oracle.mla_attend_dense(qabs, qrope, lat, rk, scale))


def test_closed_forms(oracle):
    rng = np.random.default_rng(7)
    H, nr, kvl, rope = 3, 50, 128, 16
    lat = rng.standard_normal((nr, kvl)).astype(np.float32)
    rk = rng.standard_normal((nr, rope)).astype(np.float32)
    zero_a, zero_r = np.zeros((H, kvl), np.float32), np.zeros((H, rope), np.float32)
    # all scores equal -> the plain mean of the latent rows, for every head
    got = oracle.mla_attend_dense(zero_a, zero_r, lat, rk, 0.3)
    assert np.allclose(got, np.broadcast_to(lat.mean(0), (H, kvl)), atol=2e-6)
    # a rope-only query picks by the roped key alone: make row 17's key dominate
    rk2 = rk.copy()
    rk2[17] = 0
    rk2[17, 5] = 100.0
    qr = zero_r.copy()
    qr[:, 5] = 10.0
    got = oracle.mla_attend_dense(zero_a, qr, lat, rk2, 1.0)
    assert np.allclose(got, np.broadcast_to(lat[17], (H, kvl)), atol=1e-6)
    # a latent-only query: head h is aligned with row 3+h
    lat3 = lat.copy()
    qa = zero_a.copy()
    for h in range(H):
        qa[h] = lat3[3 + h] * 50.0
    got = oracle.mla_attend_dense(qa, zero_r, lat3, rk, 1.0)
    for h in range(H):
        assert np.allclose(got[h], lat3[3 + h], atol=1e-5)
    # one row attends to itself whatever the query; scale 0 is the mean again
    got = oracle.mla_attend_dense(qa, qr, lat[:1], rk[:1], 1.0)
    assert np.array_equal(got, np.broadcast_to(lat[0], (H, kvl)))
    got = oracle.mla_attend_dense(qa, qr, lat, rk, 0.0)
    assert np.allclose(got, np.broadcast_to(lat.mean(0), (H, kvl)), atol=2e-6)


def test_rows_argument_and_guards(oracle):
    seed, h, nt, kvl, rope = 0xB10CC0DE, 20, 130, 512, 64
    qabs, qrope, lc8, lscale, rc, nb, scale = reference_attend_case(oracle, seed, h, nt, kvl, rope)
    rows = np.array([5, 0, 129, 77, 3, 64], np.uint32)
    code, got = oracle.mla_attend(qabs, qrope, lc8, lscale, rc, rows, h, rows.size, kvl, rope, nb, scale)
    assert code == 0
    lat, rk = widen_linear(oracle, lc8, lscale, rc, nt, kvl, rope, nb)
    assert np.array_equal(got, oracle.mla_attend_dense(qabs, qrope, lat[rows], rk[rows], scale))
    # launcher guards, crates/backend/kernels/attn.hip:284-293
    assert oracle.mla_attend(qabs, qrope, lc8, lscale, rc, None, 0, nt, kvl, rope, nb, scale)[0] == 1001
    assert oracle.mla_attend(qabs, qrope, lc8, lscale, rc, None, h, nt, 640, rope, 5, scale)[0] == 1004
    assert oracle.mla_attend(qabs, qrope, lc8, lscale, rc, None, h, nt, 160, rope, 1, scale)[0] == 1004


def test_paged_form(oracle):
    c = paged_case(oracle, [130, 1, 0, 257], H=5, seed=41)
    got = oracle.mla_attend_paged(c["qabs"], c["qrope"], c["pool"], c["table"], c["lens"], None, None,
                                  512, 64, 64, c["scale"], n_threads=3)
    for s, n in enumerate(c["lens"]):
        if n == 0:
            assert not got[s].any()
            continue
        lat, rk = widen_paged(oracle, c["pool"], c["table"][s], np.arange(n))
        assert np.array_equal(got[s], oracle.mla_attend_dense(c["qabs"][s], c["qrope"][s], lat, rk, c["scale"]))
        assert rel_err(got[s], attend_f64(c["qabs"][s], c["qrope"][s], lat, rk, c["scale"])) < 1e-5
    # sparse: a row list per sequence, ragged through n_rows
    k = 16
    rng = np.random.default_rng(3)
    rows = np.zeros((4, k), np.uint32)
    n_rows = np.array([16, 1, 0, 9], np.int32)
    for s, n in enumerate(c["lens"]):
        if n:
            rows[s, :min(k, n)] = np.sort(rng.choice(n, min(k, n), replace=False))
    got = oracle.mla_attend_paged(c["qabs"], c["qrope"], c["pool"], c["table"], None, rows, n_rows,
                                  512, 64, 64, c["scale"])
    for s in range(4):
        if n_rows[s] == 0:
            assert not got[s].any()
            continue
        lat, rk = widen_paged(oracle, c["pool"], c["table"][s], rows[s, :n_rows[s]])
        assert np.array_equal(got[s], oracle.mla_attend_dense(c["qabs"][s], c["qrope"][s], lat, rk, c["scale"]))
