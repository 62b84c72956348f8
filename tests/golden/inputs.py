"""Seeded inputs of the golden cases, rebuilt identically wherever the tests run.

Everything is drawn from the reference tests' own generator (`Lcg`,
crates/engine/tests/common/reference.rs:141-162) so a case is a seed, not a data file:
uniforms straight from the stream, normals by Box-Muller over pairs of uniforms (evaluated
in float64, narrowed to f32, then rounded to bf16 — that bf16 tensor is the input),
permutations by Fisher-Yates over the same stream. The golden file stores a hash of every
input next to the hash of the expected output, so a platform whose libm moved an input by an
ulp is reported as such and not as a kernel failure.
"""
import numpy as np

from tests.util import f32_to_bf16_rne

SEED_BASE = 0x5EED0000


def uniforms(lcg, n):
    """n draws in [-1, 1)."""
    return lcg.fill(n)


def normals_f32(lcg, n):
    """n N(0,1) samples from 2*ceil(n/2) uniforms (Box-Muller, both branches used)."""
    m = (n + 1) // 2
    u = lcg.fill(2 * m).astype(np.float64)
    a = (u[0::2] + 1.0) * 0.5            # [0, 1)
    b = (u[1::2] + 1.0) * 0.5
    r = np.sqrt(-2.0 * np.log1p(-a))     # 1 - a in (0, 1]
    z = np.concatenate([r * np.cos(2.0 * np.pi * b), r * np.sin(2.0 * np.pi * b)])
    return z[:n].astype(np.float32)


def permutation(lcg, n):
    """Fisher-Yates driven by the stream: j = floor((u + 1) / 2 * (i + 1))."""
    u = (lcg.fill(n).astype(np.float64) + 1.0) * 0.5
    p = np.arange(n, dtype=np.int32)
    for i in range(n - 1, 0, -1):
        j = int(u[i] * (i + 1))
        p[i], p[j] = p[j], p[i]
    return p


def rows_bf16(lcg, n, width, outlier_frac=0.0, outlier_mul=1.0):
    """[n, width] bf16 bit patterns ~N(0,1), a seeded fraction of ROWS multiplied in f32."""
    x = normals_f32(lcg, n * width).reshape(n, width)
    if outlier_frac > 0:
        hit = (lcg.fill(n) + 1.0) * 0.5 < outlier_frac
        x[hit] *= np.float32(outlier_mul)
    return f32_to_bf16_rne(x)


def config1(oracle, ctx=4096, width=576, page_tokens=64):
    """Benchmark configuration 1: one sequence of `ctx` tokens, block table = a seeded
    permutation of ctx/page_tokens pages; the last token is the appended one."""
    lcg = oracle.lcg(SEED_BASE + 1)
    rows = rows_bf16(lcg, ctx, width)
    table = permutation(lcg, ctx // page_tokens)
    pos = np.arange(ctx)
    slots = (table[pos // page_tokens] * page_tokens + pos % page_tokens).astype(np.int32)
    return rows, table.reshape(1, -1), slots


def config2(oracle, n=8192, width=576, page_tokens=64):
    """Benchmark configuration 2: n new rows, 0.5% of rows x50, into shuffled pages."""
    lcg = oracle.lcg(SEED_BASE + 2)
    rows = rows_bf16(lcg, n, width, outlier_frac=0.005, outlier_mul=50.0)
    table = permutation(lcg, n // page_tokens)
    pos = np.arange(n)
    slots = (table[pos // page_tokens] * page_tokens + pos % page_tokens).astype(np.int32)
    return rows, table.reshape(1, -1), slots


def config4_small(oracle, n_q=4, nt=8192, k=512, width=576, page_tokens=64):
    """Benchmark configuration 4 at a size the oracle finishes at once: per query nt scores
    ~N(0,1) with +4 on the last 64 tokens, fragmented pages, top-k then sparse gather."""
    lcg = oracle.lcg(SEED_BASE + 4)
    rows = rows_bf16(lcg, n_q * nt, width)
    blocks = nt // page_tokens
    table = permutation(lcg, n_q * blocks).reshape(n_q, blocks)
    pos = np.arange(nt)
    slots = np.concatenate([table[q][pos // page_tokens] * page_tokens + pos % page_tokens
                            for q in range(n_q)]).astype(np.int32)
    scores = normals_f32(lcg, n_q * nt).reshape(n_q, nt)
    scores[:, -64:] += np.float32(4.0)
    return rows, table, slots, scores, k
