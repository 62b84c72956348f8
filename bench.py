"""Benchmark of the fp8 MLA KV-cache hot path on one MI355X.

Workload (default): BASELINE config 3 at its metric point — 48 layers, batch 32, every
sequence at 32768 tokens of context, pages of 64 tokens drawn from a shuffled global pool. One
"step" is one decode step's KV work: per layer, quantize-append one new 576-wide row per
sequence, then gather + dequantize every sequence's full context to bf16. All inputs are
resident in HBM before the timed region; timing is HIP events on the launch stream.

Prints one JSON line: value = algorithmic bytes moved per step / step time (GB/s);
`roofline` prices the gather kernel (the dominant one) against 8 TB/s using per-launch event
timings taken inside the timed region; `cpu_baseline` times the CPU oracle's gather on the
host cores over a bounded sample of the same workload (and doubles as a full-size parity
check of one layer).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

W, PT = 576, 64
ROW_IN = W * 2            # bf16 row
REC = W + 4               # stored record: codes + one f32 scale
HBM_PEAK = 8.0e12


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--layers", type=int, default=48)
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--ctx", type=int, default=32768)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    return ap.parse_args()


def main():
    a = parse()
    if a.gpus != 1:
        sys.exit("bench.py measures one GPU: this path shards by layer or by sequence with no "
                 "exchange step, and no multi-GPU figure is produced (run with --gpus 1)")
    import torch

    from rivoli_amd import hip

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (cuda:0); there is no CPU fallback for the product path")
    torch.cuda.set_device(0)
    hip.lib()
    L, B, ctx = a.layers, a.batch, a.ctx
    blocks = -(-ctx // PT)
    n_pages = B * blocks
    page_bytes = hip.kv_page_bytes(PT, W)
    n_tok = B * ctx

    # ---- synthetic, seeded, resident inputs ------------------------------------------------
    g = torch.Generator(device="cuda")
    g.manual_seed(0x5EED0003)
    rng = np.random.default_rng(0x5EED0003)
    perm = rng.permutation(n_pages).astype(np.int32)            # shuffled global pool
    tables_np = perm.reshape(B, blocks)
    pos = np.arange(ctx)
    slots_np = np.concatenate([tables_np[s][pos // PT] * PT + pos % PT for s in range(B)]).astype(np.int32)
    tables = torch.from_numpy(tables_np.copy()).cuda()
    slots_all = torch.from_numpy(slots_np).cuda()
    seq_lens_np = np.full(B, ctx, np.int32)
    cu_np = np.concatenate([[0], np.cumsum(seq_lens_np)]).astype(np.int32)
    seq_lens, cu = torch.from_numpy(seq_lens_np).cuda(), torch.from_numpy(cu_np).cuda()
    # the step's new tokens: the last position of every sequence
    new_slots = torch.from_numpy(slots_np.reshape(B, ctx)[:, -1].copy()).cuda()

    kv_rows = torch.randn(n_tok, W, generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    pools = []
    for layer in range(L):
        pool = torch.empty(n_pages * page_bytes, dtype=torch.uint8, device="cuda")
        hip.launch_kv_append_paged(kv_rows, slots_all, pool, n_tok, W, PT, n_pages)
        pools.append(pool)
    new_rows = [torch.randn(B, W, generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
                for _ in range(L)]
    out = torch.empty(n_tok * W, dtype=torch.bfloat16, device="cuda")
    torch.cuda.synchronize()

    stream = torch.cuda.Stream()
    sh = stream.cuda_stream

    def step(events=None):
        for layer in range(L):
            hip.launch_kv_append_paged(new_rows[layer], new_slots, pools[layer], B, W, PT, n_pages,
                                       None, sh)
            if events is not None:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
            hip.launch_kv_gather_paged(pools[layer], tables, seq_lens, cu, out, B, blocks, W, PT,
                                       n_pages, None, sh)
            if events is not None:
                e1.record(stream)
                events.append((e0, e1))

    for _ in range(a.warmup):
        step()
    stream.synchronize()
    torch.cuda.synchronize()
    t_begin, t_end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    events = []
    t_begin.record(stream)
    for _ in range(a.steps):
        step(events)
    t_end.record(stream)
    stream.synchronize()
    torch.cuda.synchronize()
    ms_per_step = t_begin.elapsed_time(t_end) / a.steps
    gather_ms = float(np.mean([e0.elapsed_time(e1) for e0, e1 in events]))

    append_bytes = L * B * (ROW_IN + 4 + REC)                   # row + slot in, record out
    gather_bytes_layer = n_tok * (REC + ROW_IN) + B * blocks * 4  # records + table in, bf16 out
    step_bytes = append_bytes + L * gather_bytes_layer
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    achieved = gather_bytes_layer / (gather_ms * 1e-3) / 1e9

    result = {
        "metric": "kv_append_gather_GBps", "value": round(value, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "batched decode (BASELINE config 3, metric point): append 1 token/"
                               "seq/layer then gather+dequantize every sequence's full context",
                   "layers": L, "batch": B, "ctx": ctx, "page_tokens": PT, "width": W,
                   "stored": "fp8 e4m3 + 1 f32 scale/token", "out": "bf16"},
        "decode_step_kv_ms": round(ms_per_step, 4),
        "tokens_per_s": round(L * n_tok / (ms_per_step * 1e-3), 1),
        "hbm_peak_frac": round(value * 1e9 / HBM_PEAK, 4),
        "roofline": {"bound": "hbm", "kernel": "kv_gather_paged_kernel", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": round(achieved * 1e9 / HBM_PEAK, 4),
                     "avg_launch_ms": round(gather_ms, 5), "bytes_per_launch": gather_bytes_layer,
                     "traffic": None},
    }

    if not a.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(pools[0], tables_np, seq_lens_np, out, a.cpu_seconds,
                                              hip, tables, seq_lens, cu, B, blocks, n_pages)
    print(json.dumps(result), flush=True)


def cpu_baseline(pool0, tables_np, seq_lens_np, out, budget_s, hip, tables, seq_lens, cu, B, blocks,
                 n_pages):
    """The CPU oracle's gather over layer 0 of the same pool, on the host cores, repeated until
    about `budget_s` seconds have been spent; its output is also compared with the GPU's."""
    import torch

    from oracle.kvoracle import oracle as get_oracle

    ora = get_oracle()
    cores = max(1, min(16, os.cpu_count() or 1))
    pool_host = pool0.cpu().numpy()
    n_tok = int(seq_lens_np.sum())
    out_host = np.empty((n_tok, W), np.uint16)
    reps, spent = 0, 0.0
    while spent < budget_s and reps < 50:
        t0 = time.perf_counter()
        ora.kv_gather_paged(pool_host, tables_np, seq_lens_np, W, PT, n_threads=cores, out=out_host)
        spent += time.perf_counter() - t0
        reps += 1
    per_layer_s = spent / reps
    bytes_layer = n_tok * (REC + ROW_IN) + tables_np.size * 4
    # full-size parity of one layer: GPU gather of the same pool vs the oracle's bytes
    hip.launch_kv_gather_paged(pool0, tables, seq_lens, cu, out, B, blocks, W, PT, n_pages)
    torch.cuda.synchronize()
    same = bool(np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1, W),
                               out_host))
    if not same:
        raise SystemExit("bench: GPU gather differs from the CPU oracle at full size")
    return {"value": round(bytes_layer / per_layer_s / 1e9, 3), "unit": "GB/s", "cores": cores,
            "kind": "port",
            "sample": f"gather+dequantize of one layer ({n_tok} tokens, same pool and block "
                      f"tables) x{reps} reps, {cores} host threads; GPU output checked equal",
            "tokens_per_s": round(n_tok / per_layer_s, 1)}


if __name__ == "__main__":
    main()
