"""benchmark configuration 5 as a seeded event stream: a 2048-page pool kept ~80% full by up to 64
sequences of 512 to 128K tokens, decode appends interleaved with whole-sequence frees whose
pages are reused LIFO; 1% of tokens are x200 outliers. Shared by the CPU and GPU tests."""
import numpy as np

from rivoli_amd.pagepool import PagePool, PoolExhausted
from tests.util import f32_to_bf16_rne

W, PT, N_PAGES, MAX_SEQS = 576, 64, 2048, 64


_BANK = None


def token_rows(rng, n):
    """n rows drawn (with repetition) from a fixed bank of 32768 N(0,1) rows, 1% of which are
    x200 outliers; drawing from a bank keeps a 10k-step stream cheap to generate."""
    global _BANK
    if _BANK is None:
        brng = np.random.default_rng(0xBA2C)
        x = brng.standard_normal((32768, W), dtype=np.float32)
        x[brng.random(32768) < 0.01] *= np.float32(200.0)
        _BANK = f32_to_bf16_rne(x)
    return _BANK[rng.integers(0, 32768, n)]


def churn_events(steps, seed):
    """Yields ("append", slots[int32 n], rows[uint16 n x W]) and ("free", seq) events, and at
    the end ("final", {seq: (block_table, length)}). The allocator is the product's own
    (host C++); the stream is deterministic for a seed."""
    rng = np.random.default_rng(seed)
    pool = PagePool(N_PAGES, PT)
    live = []
    stats = {"appended": 0, "freed_seqs": 0, "evictions": 0, "max_len": 0}

    def admit():
        free_tokens = pool.pages_free * PT
        want = int(512 * 2.0 ** (8.0 * rng.random() ** 3))    # 512..128K, mostly short
        n = min(want, free_tokens - PT)
        if n < 512 or len(live) >= MAX_SEQS:
            return None
        s = pool.seq_create()
        live.append(s)
        return s, pool.seq_extend(s, n)

    for _ in range(steps):
        fill = pool.pages_owned / N_PAGES
        if fill < 0.8 and len(live) < MAX_SEQS:
            got = admit()
            if got is not None:
                s, slots = got
                stats["appended"] += slots.size
                stats["max_len"] = max(stats["max_len"], slots.size)
                yield "append", slots, token_rows(rng, slots.size)
                continue
        if live and rng.random() < 0.04:
            s = live.pop(int(rng.integers(len(live))))
            pool.seq_free(s)
            stats["freed_seqs"] += 1
            yield "free", s
            continue
        # decode step: one token for every live sequence (evict a random one if the pool is full)
        slots = []
        for s in list(live):
            if s not in live:      # evicted earlier in this very step
                continue
            try:
                slots.append(pool.seq_extend(s, 1))
            except PoolExhausted:
                victim = live.pop(int(rng.integers(len(live))))
                pool.seq_free(victim)
                stats["evictions"] += 1
                yield "free", victim
                if victim != s and s in live:
                    slots.append(pool.seq_extend(s, 1))
        if slots:
            slots = np.concatenate(slots)
            stats["appended"] += slots.size
            yield "append", slots, token_rows(rng, slots.size)
    yield "final", {s: (pool.block_table(s), pool.seq_len(s)) for s in live}, stats
