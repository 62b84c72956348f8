"""The ten index_topk cases of crates/engine/tests/kernel_vector.rs:132-170, regenerated from
the same seeded stream (data, not code: closed-form ramps and Lcg(0x7071_C0DE) draws)."""
import numpy as np


def reference_topk_cases(oracle):
    rng = oracle.lcg(0x7071C0DE)
    nt = 5185
    relu_sparse = np.zeros(nt, np.float32)
    relu_sparse[:300] = (300 - np.arange(300)).astype(np.float32) * np.float32(0.25)
    scattered = np.zeros(nt, np.float32)
    for j in range(300):
        scattered[(j * 7919) % nt] = np.float32(300 - j) * np.float32(0.25)
    dense = rng.fill(nt) * np.float32(8.0)
    heavy_ties = np.floor(rng.fill(nt) * np.float32(4.0)).astype(np.float32)
    ramp = lambda n, m: (np.arange(n) % m).astype(np.float32)
    signed_zeros = np.where(np.arange(4096) % 3 == 0, np.float32(-0.0), np.float32(0.0)).astype(np.float32)
    negatives = (-(np.arange(4096) % 11)).astype(np.float32)
    return [
        ("mixed +0.0/-0.0", signed_zeros, 2048),
        ("negatives only", negatives, 2048),
        ("k == nt", ramp(2048, 7), 2048),
        ("k == nt - 1", ramp(2049, 7), 2048),
        ("k > nt (wrapper clamp)", ramp(500, 7), 2048),
        ("single block", ramp(200, 5), 64),
        ("ReLU-sparse (prefix answer)", relu_sparse, 2048),
        ("scattered zeros (non-prefix answer)", scattered, 2048),
        ("dense random", dense, 2048),
        ("heavy ties", heavy_ties, 2048),
    ]


def brute_force_topk(scores: np.ndarray, k: int) -> np.ndarray:
    """Full lexicographic sort by (-score, index) with -0.0 == +0.0; first k, ascending."""
    s = scores.astype(np.float64) + 0.0  # -0.0 + 0.0 == +0.0
    order = np.lexsort((np.arange(s.size), -s))
    return np.sort(order[: min(k, s.size)]).astype(np.uint32)
