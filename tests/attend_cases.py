"""Inputs for the MLA attention tests.

`reference_attend_case` redraws what crates/engine/tests/kernel_attend.rs:228-245 (check_attend)
draws from its seeded stream, in the same order: qabs, qrope, the e4m3 latent bytes, the
positive per-128 block scales, the bf16 roped keys. `attend_f64` is the same formula in float64
with numpy — an independent restatement the oracle is checked against."""
import numpy as np

from tests.util import bf16_to_f32, make_rows_bf16, shuffled_block_tables, slots_for


def reference_attend_case(oracle, seed, h, nt, kvl, rope):
    r = oracle.lcg(seed)
    nb = kvl // 128
    qabs = r.fill(h * kvl).reshape(h, kvl)
    qrope = r.fill(h * rope).reshape(h, rope)
    lc8 = oracle.f32_to_e4m3(r.fill(nt * kvl))
    lscale = (np.abs(r.fill(nt * nb) * np.float32(0.1)) + np.float32(0.01)).astype(np.float32)
    rc = oracle.f32_to_bf16(r.fill(nt * rope))
    scale = np.float32(1.0) / np.sqrt(np.float32(kvl + rope))
    return qabs, qrope, lc8, lscale, rc, nb, float(scale)


def widen_linear(oracle, lc8, lscale, rc, nt, kvl, rope, nb):
    """The kernel's own dequant (crates/engine/tests/kernel_attend.rs:243-245): one f32 product."""
    lat = oracle.e4m3_to_f32(lc8).reshape(nt, kvl) * np.repeat(lscale.reshape(nt, nb), 128, axis=1)
    return lat.astype(np.float32), bf16_to_f32(rc).reshape(nt, rope)


def attend_f64(qabs, qrope, lat, rk, scale):
    qa, qr = qabs.astype(np.float64), qrope.astype(np.float64)
    L, R = lat.astype(np.float64), rk.astype(np.float64)
    s = (qa @ L.T + qr @ R.T) * float(scale)
    s -= s.max(axis=1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=1, keepdims=True)
    return p @ L


def widen_paged(oracle, pool, table_row, tokens, kvl=512, rope=64, page_tokens=64):
    """Rows `tokens` of one sequence of the paged cache as f32: e4m3_to_f32(code) * scale."""
    width = kvl + rope
    pb = oracle.kv_page_bytes(page_tokens, width)
    tokens = np.asarray(tokens, np.int64)
    pages = table_row[tokens // page_tokens].astype(np.int64)
    offs = tokens % page_tokens
    codes = np.stack([pool[p * pb + o * width: p * pb + (o + 1) * width] for p, o in zip(pages, offs)])
    scl = np.array([pool[p * pb + page_tokens * width + o * 4:][:4].view(np.float32)[0]
                    for p, o in zip(pages, offs)], np.float32)
    wide = oracle.e4m3_to_f32(codes) * scl[:, None]
    return wide[:, :kvl].astype(np.float32), wide[:, kvl:].astype(np.float32)


def paged_case(oracle, lens, H, seed, n_spare_pages=3, kvl=512, rope=64, page_tokens=64, q_gain=1.0,
               outlier_frac=0.01):
    """A paged cache holding len(lens) sequences on shuffled pages, plus queries.
    Returns dict(pool, table, lens, qabs, qrope, scale, n_pages)."""
    width = kvl + rope
    rng = np.random.default_rng(seed)
    blocks = max(1, -(-max(lens) // page_tokens))
    n_pages = len(lens) * blocks + n_spare_pages
    table = shuffled_block_tables(len(lens), blocks, n_pages, seed + 1)
    pool = np.zeros(n_pages * oracle.kv_page_bytes(page_tokens, width), np.uint8)
    for s, n in enumerate(lens):
        if n == 0:
            continue
        rows = make_rows_bf16(n, width, seed=seed + 10 + s, outlier_frac=outlier_frac, outlier_mul=30.0)
        oracle.kv_append_paged(rows, slots_for(table[s], np.arange(n), page_tokens), pool, width,
                               page_tokens, n_pages)
    qabs = (rng.standard_normal((len(lens), H, kvl)) * q_gain).astype(np.float32)
    qrope = (rng.standard_normal((len(lens), H, rope)) * q_gain).astype(np.float32)
    return dict(pool=pool, table=table, lens=np.asarray(lens, np.int32), qabs=qabs, qrope=qrope,
                scale=float(np.float32(1.0) / np.sqrt(np.float32(width))), n_pages=n_pages)
