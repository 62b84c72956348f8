"""Inputs and independent restatements for the second cache format's compressor tests."""
import numpy as np

from oracle.kvoracle import CompGeom


def compress_inputs(geom: CompGeom, s: int, seed: int, positions: int = 0):
    """Projected kv / gate scores for s tokens, the position-in-block embedding, the norm weight
    and a rotation table of (cos, sin) pairs for `positions` positions (at least s)."""
    rng = np.random.default_rng(seed)
    kv = rng.standard_normal((s, geom.cd)).astype(np.float32)
    score = (rng.standard_normal((s, geom.cd)) * 2.0).astype(np.float32)
    ape = rng.standard_normal((geom.ratio, geom.cd)).astype(np.float32)
    norm = (1.0 + 0.1 * rng.standard_normal(geom.d)).astype(np.float32)
    n_pos = max(positions, s, 1)
    inv = 160000.0 ** (-np.arange(geom.rd // 2, dtype=np.float64) * 2.0 / geom.rd)
    ang = np.arange(n_pos, dtype=np.float64)[:, None] * inv[None, :]
    freqs = np.stack([np.cos(ang), np.sin(ang)], axis=-1).reshape(n_pos, geom.rd).astype(np.float32)
    return kv, score, ape, norm, freqs


def bf16_gap(oracle, a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """Distance in bf16 codes under a monotone ordering (crates/engine/tests/v4_compressor/
    metric.rs: 0 is bit-identical, 1 is adjacent representable values)."""
    def ordered(x):
        c = oracle.f32_to_bf16(np.ascontiguousarray(x, np.float32)).astype(np.int64)
        return np.where(c & 0x8000, -(c & 0x7FFF), c)
    return np.abs(ordered(a) - ordered(b))


def literal_pooling(geom: CompGeom, kv, score, ape, nblk: int) -> np.ndarray:
    """model.py's own order of operations in float64: add the position embedding to the scores,
    materialise overlap_transform's [nblk, ents, d] tensors (zero / -inf where block 0 has no
    previous block), softmax over the entry axis, weighted sum."""
    r, d, cd = geom.ratio, geom.d, geom.cd
    kv64 = kv[: nblk * r].astype(np.float64).reshape(nblk, r, cd)
    sc64 = (score[: nblk * r].astype(np.float32).reshape(nblk, r, cd) + ape[None, :, :]).astype(np.float64)
    if geom.coff == 2:
        kb = np.zeros((nblk, 2 * r, d))
        sb = np.full((nblk, 2 * r, d), -np.inf)
        kb[:, r:] = kv64[:, :, d:]
        sb[:, r:] = sc64[:, :, d:]
        kb[1:, :r] = kv64[:-1, :, :d]
        sb[1:, :r] = sc64[:-1, :, :d]
    else:
        kb, sb = kv64, sc64
    w = np.exp(sb - sb.max(axis=1, keepdims=True))
    w /= w.sum(axis=1, keepdims=True)
    return (kb * w).sum(axis=1)


def literal_finish(oracle, geom: CompGeom, pooled, norm, freqs, first_pos: int) -> np.ndarray:
    """bf16 store, RMSNorm in float64 with the bf16 store, complex rotation of the last rd dims
    at each block's first position, bf16 store."""
    rb = lambda x: oracle.e4m3_to_f32(np.zeros(0, np.uint8)) if x.size == 0 else \
        (oracle.f32_to_bf16(x.astype(np.float32)).astype(np.uint32) << 16).view(np.float32)
    d, rd, r = geom.d, geom.rd, geom.ratio
    x = rb(pooled).astype(np.float64)
    rs = 1.0 / np.sqrt((x * x).mean(axis=1, keepdims=True) + np.float64(np.float32(geom.eps)))
    x = rb(norm.astype(np.float64)[None, :] * (x * rs)).astype(np.float64)
    pos = first_pos + np.arange(x.shape[0]) * r
    t = freqs[pos].astype(np.float64).reshape(-1, rd // 2, 2)
    z = (x[:, d - rd::2] + 1j * x[:, d - rd + 1::2]) * (t[:, :, 0] + 1j * t[:, :, 1])
    x[:, d - rd::2], x[:, d - rd + 1::2] = z.real, z.imag
    return rb(x)


def compress_gap(oracle, got: np.ndarray, want: np.ndarray, rd: int) -> np.ndarray:
    """bf16 code distance between two sets of compressed rows, with the two places where a code
    distance says nothing taken out: a value that is tiny against its row because the weighted
    sum (or the rotation's a*c - b*s) cancelled carries an absolute error of the terms' size,
    which is many codes of the small result. Such elements count as equal when they agree to
    2^-14 of the row's largest value (2^-8 in the rotated tail, where a one-code difference of
    an input passes straight through)."""
    gap = bf16_gap(oracle, got, want)
    top = np.abs(want).max(axis=1, keepdims=True)
    tail = (np.arange(got.shape[1]) >= got.shape[1] - rd)[None, :]
    near = np.abs(got - want) <= top * np.where(tail, 2.0 ** -8, 2.0 ** -14)
    return np.where(near, np.minimum(gap, 2), gap)


def literal_sel_gather(win, ratio, seqlen, start_pos):
    """One selection rectangle cell by cell from the rule as the reference words it
    (crates/engine/src/v4/select.rs:195-241): at prefill the last `win` absolute positions up
    to the query's own; at decode the ring's slots oldest first, slot p % win holding position
    p; then every compressed block that has closed, shifted past the window region."""
    prefill = start_pos == 0
    rows = seqlen if prefill else 1
    out = []
    for t in range(rows):
        if prefill:
            width = min(seqlen, win)
            live = list(range(max(0, t - win + 1), t + 1))
            if t >= win - 1:
                row = live
            else:
                row = [v if v <= t else -1 for v in range(width)]
        else:
            positions = list(range(max(0, start_pos - win + 1), start_pos + 1))   # oldest first
            row = [p % win for p in positions] + [-1] * (win - len(positions))
        if ratio:
            if prefill:
                closed = (t + 1) // ratio
                row += [seqlen + c if c < closed else -1 for c in range(seqlen // ratio)]
            else:
                row += [win + c for c in range((start_pos + 1) // ratio)]
        out.append(row)
    return np.array(out, np.int32).reshape(rows, -1)


def sparse_attn_f64(q, kv, sink, idxs, scale):
    """The index-list attention in float64 with a library softmax shape: masked slots (-1) out,
    the sink in the denominator only (crates/backend/kernels/attn.hip:333-343)."""
    q, kv, sink = np.asarray(q, np.float64), np.asarray(kv, np.float64), np.asarray(sink, np.float64)
    m, h, d = q.shape
    out = np.empty((m, h, d))
    for t in range(m):
        live = [int(i) for i in idxs[t] if i >= 0]
        rows = kv[live]
        for hh in range(h):
            logit = rows @ q[t, hh] * float(np.float32(scale))
            mx = logit.max()
            e = np.exp(logit - mx)
            out[t, hh] = (e @ rows) / (e.sum() + np.exp(sink[hh] - mx))
    return out


def bf16_round(x):
    """f32 -> nearest-even bf16 value, as f32 (finite inputs)."""
    b = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return (((b + 0x7FFF + ((b >> 16) & 1)) >> 16) << 16).astype(np.uint32).view(np.float32).reshape(np.shape(x))


def attend_inputs(oracle, m, h, d, rows, seed, cache_like=True, q_scale=1.0):
    """q [m, h, d], kv [rows, d], sink [h]. cache_like: what the model hands the kernel — q
    rounded to bf16 after its rotary, kv rows whose first d - 64 dims went through the block-64
    fp8 quantize-dequantize and whose last 64 are bf16 values
    (crates/engine/src/v4/attn.rs:272-290); otherwise arbitrary f32."""
    rng = np.random.default_rng(seed)
    q = (rng.standard_normal((m, h, d)) * q_scale).astype(np.float32)
    kv = rng.standard_normal((rows, d)).astype(np.float32)
    # outlier rows; milder where the kernel will round the rows to bf16 on load, which moves
    # a logit by ~2^-9 of its size
    kv[rng.integers(0, rows, max(1, rows // 50))] *= 8.0 if cache_like else 3.0
    sink = rng.standard_normal(h).astype(np.float32)
    if cache_like:
        q, kv = bf16_round(q), bf16_round(kv)
        n = d - 64 if d > 64 and (d - 64) % 64 == 0 else 0
        if n:
            code, kv = oracle.act_quant_f8_prefix(kv, n, 64)
            assert code == 0
    return q, kv, sink
