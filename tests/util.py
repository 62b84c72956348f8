"""Seeded synthetic inputs shared by the oracle and GPU parity tests (numpy only)."""
import numpy as np


def f32_to_bf16_rne(x: np.ndarray) -> np.ndarray:
    """Textbook integer round-to-nearest-even; finite inputs only."""
    b = np.ascontiguousarray(x, np.float32).view(np.uint32)
    # uint32 arithmetic cannot wrap for finite inputs (|bits| <= 0x7f7fffff before the add)
    r = (b >> np.uint32(16)) & np.uint32(1)
    r += np.uint32(0x7FFF)
    r += b
    r >>= np.uint32(16)
    return r.astype(np.uint16)


def bf16_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def make_rows_bf16(n, width=576, seed=0, outlier_frac=0.0, outlier_mul=1.0) -> np.ndarray:
    """[n, width] bf16 bit patterns: N(0,1) in f32, a fraction of ROWS scaled, then RNE to bf16.
    That bf16 tensor is the input both the oracle and the kernels receive."""
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((n, width), dtype=np.float32)
    if outlier_frac > 0:
        hit = rng.random(n) < outlier_frac
        x[hit] *= np.float32(outlier_mul)
    return f32_to_bf16_rne(x)


def shuffled_block_tables(n_seqs, blocks_per_seq, n_pages, seed):
    """Disjoint pages for every sequence, drawn from one shuffled global pool."""
    rng = np.random.default_rng(seed)
    perm = rng.permutation(n_pages).astype(np.int32)
    assert n_seqs * blocks_per_seq <= n_pages
    return perm[: n_seqs * blocks_per_seq].reshape(n_seqs, blocks_per_seq).copy()


def slots_for(table_row, positions, page_tokens=64):
    positions = np.asarray(positions)
    return (table_row[positions // page_tokens] * page_tokens + positions % page_tokens).astype(np.int32)
