"""Benchmark of the fp8 MLA KV-cache hot path on one MI355X.

Workload (default): benchmark configuration 3 at its metric point — 48 layers, batch 32, every
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
import re
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
    ap.add_argument("--workload", choices=["all", "decode", "prefill", "dsa", "dsa_scored", "dsa_attend", "attend", "v4",
                                           "v4_attend", "v4_index"],
                    default="all",
                    help="all (default) = the headline line with every other configuration attached under `configs`; decode = configuration 3 (the headline line) alone; prefill = configuration 2 "
                         "bulk append; dsa = configuration 4 top-k + sparse gather on synthetic "
                         "scores; dsa_scored = the same with the scores computed on the device; "
                         "dsa_attend = configuration 4 with the sparse gather replaced by MLA decode "
                         "attention over the selected rows; "
                         "attend = configuration 3 with the gather replaced by MLA decode "
                         "attention reading the fp8 pages directly; "
                         "v4 = the second cache format's prefill ops: block-64 quantize-dequantize "
                         "of `tokens` f32 cache rows, then the scored block selection for every "
                         "query row (ratio 4, cap --index-topk); "
                         "v4_attend = the second cache format's consumer at prefill: ring write, the "
                         "[window | scored blocks] selection rectangle, and the index-list attention "
                         "of `tokens` queries x --heads heads over it; "
                         "v4_index = the second cache format's block indexer at prefill: the Hadamard + "
                         "fp4 spread of `tokens` x --heads query rows of 128 and the block scores of "
                         "every query against the tokens / 4 compressed blocks")
    ap.add_argument("--index-topk", type=int, default=512, help="v4: blocks kept per query row")
    ap.add_argument("--heads", type=int, default=64, help="attend: query heads")
    ap.add_argument("--precise", type=int, default=2, choices=[0, 1, 2, 3, 4],
                    help="attend: 2 = q and softmax weights as bf16 hi+lo (parity mode), "
                         "1 = q only, 0 = plain bf16; on the 8-bit matrix instructions: 4 = q as three "
                         "e4m3 terms and the weights as two (inside the reference's bar), 3 = two and two "
                         "(bf16-class)")
    ap.add_argument("--ragged", action="store_true",
                    help="decode / attend: per-sequence context drawn uniformly from [1024, ctx] "
                         "(configuration 3 as written) instead of every sequence at ctx (its metric point)")
    ap.add_argument("--table-blocks", type=int, default=0,
                    help="decode: columns of the block tables (default: what ctx needs); more = tables sized "
                         "for a context limit above ctx, their extra columns unused")
    ap.add_argument("--gather-form", choices=["packed", "grid"], default="packed",
                    help="decode: rivoli_kv_gather_paged_packed (the caller passes the batch's token count) "
                         "or rivoli_kv_gather_paged")
    ap.add_argument("--tokens", type=int, default=8192, help="prefill: new tokens per step")
    ap.add_argument("--topk", type=int, default=2048)
    ap.add_argument("--unfused", action="store_true",
                    help="dsa / dsa_scored: run the selection and the sparse gather as two separate "
                         "entry points instead of the one fused call")
    ap.add_argument("--one-launch", action="store_true",
                    help="decode: the step's append and gather as one launch (rivoli_kv_append_gather_paged) "
                         "instead of two calls; it pays where the step is launch-bound (configuration 1), and "
                         "measures equal at configuration 3's size")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 1 GiB device copy (a known-size kernel to scale "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings by)")
    ap.add_argument("--full-scores", action="store_true",
                    help="v4_index: score every query against every block (the reference's rectangle) instead "
                         "of the entries a prefill's selection can rank")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    return ap.parse_args()


def context_lengths(a, rng):
    """Every sequence at ctx (the metric point), or ~U[1024, ctx] with --ragged."""
    if not a.ragged:
        return np.full(a.batch, a.ctx, np.int32)
    return rng.integers(min(1024, a.ctx), a.ctx + 1, size=a.batch).astype(np.int32)


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
    if a.calibrate_copy:
        src = torch.zeros(1 << 30, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if a.workload != "all":
        res = run_workload(a.workload, a, torch, hip)
        print(json.dumps(res), flush=True)
        return
    # the default run: the headline (configuration 3 at its metric point) and, in the same
    # line, the other configurations, each with its own oracle check
    res = bench_decode(a, torch, hip)
    short = min(a.cpu_seconds, 2.0)
    small = dict(layers=1, batch=1, ctx=4096, steps=200, warmup=20, cpu_seconds=short)
    others = (("cfg3_ragged", "decode", dict(ragged=True, cpu_seconds=short)),
              # configuration 1 (append one token, gather 4096): as two calls and as one launch
              ("cfg1_step", "decode", small),
              ("cfg1_step_one_launch", "decode", dict(small, one_launch=True)),
              ("cfg4_dsa", "dsa", dict(cpu_seconds=short)),
              ("cfg4_dsa_scored", "dsa_scored", dict(cpu_seconds=short)),
              ("cfg4_dsa_attend", "dsa_attend", dict(precise=4)),
              ("cfg2_prefill_8192", "prefill", dict(tokens=8192, cpu_seconds=short)),
              ("cfg2_prefill_1048576", "prefill", dict(tokens=1048576, cpu_seconds=short)),
              # the cache's consumer at configuration 3's shape: inside the reference's own bar on
              # the 8-bit matrix instructions, and the tighter bf16 hi + lo mode
              ("attend_decode", "attend", dict(precise=4)),
              ("attend_decode_bf16x2", "attend", dict(precise=2)),
              # the second cache format's own operators, at prefill
              # (one layer a step, a millisecond or so: more steps than the default three, so that
              # the first launches' cold caches do not set the figure)
              ("v4_prefill_32768", "v4", dict(tokens=32768, steps=20, warmup=3)),
              ("v4_attend_prefill_8192", "v4_attend", dict(tokens=8192, precise=2, steps=20, warmup=3)),
              ("v4_index_prefill_4096", "v4_index", dict(tokens=4096, steps=20, warmup=3)))
    res["configs"] = {}
    for name, workload, over in others:
        torch.cuda.empty_cache()
        sub = run_workload(workload, argparse.Namespace(**{**vars(a), **over}), torch, hip)
        res["configs"][name] = brief(sub)
    print(json.dumps(res), flush=True)


def run_workload(workload, a, torch, hip):
    if workload == "decode":
        return bench_decode(a, torch, hip)
    if workload == "prefill":
        return bench_prefill(a, torch, hip)
    if workload in ("dsa", "dsa_scored", "dsa_attend"):
        return bench_dsa(a, torch, hip, scored=workload == "dsa_scored", attend=workload == "dsa_attend")
    if workload == "attend":
        return bench_attend(a, torch, hip)
    if workload == "v4":
        return bench_v4(a, torch, hip)
    if workload == "v4_attend":
        return bench_v4_attend(a, torch, hip)
    if workload == "v4_index":
        return bench_v4_index(a, torch, hip)
    raise SystemExit(f"unknown workload {workload}")


def brief(res):
    """What a secondary configuration contributes to the default run's line: the figures, not
    the prose (`--workload X` prints the full record of one configuration). frac = the dominant
    kernel's algorithmic bytes (or flops) per launch / its bracketed launch time / the peak;
    frac_step, where present, is the same bytes over the step time per launch (the plain pass,
    whose launches queue ahead of the device). checked: how the GPU result compared with the
    CPU oracle ("equal", or the error it stayed within); cpu: the oracle's rate in `unit`
    (GB/s where no unit is given)."""
    r = res.get("roofline", {})
    out = {"value": res["value"], "ms": res["ms_per_step"]}
    if res["unit"] != "GB/s":  # (the headline's unit is the default)
        out["unit"] = res["unit"]
    if "layer_us" in res:
        out["layer_us"] = res["layer_us"]
    out["kernel"] = (r.get("kernel") or "").split(" (")[0]
    if r.get("bound", "hbm") != "hbm":
        out["bound"] = r["bound"]
    out["frac"] = r.get("frac")
    if "frac_step" in r:
        out["frac_step"] = r["frac_step"]
    out["launch_ms"] = r.get("avg_launch_ms")
    per_launch = r.get("bytes_per_launch", r.get("flops_per_launch"))
    if per_launch is not None:
        out["per_launch"] = int(per_launch)
    if r.get("traffic") is not None:  # (absent: not measured for this shape)
        out["traffic"] = r["traffic"]
    elif "index_score" in res and res["index_score"].get("traffic") is not None:
        out["score_traffic"] = res["index_score"]["traffic"]
    if "kernels_ms" in res:
        out["kernels_ms"] = res["kernels_ms"]
    elif "kernels" in res:
        out["kernels_ms"] = {k: v["avg_launch_ms"] for k, v in res["kernels"].items()}
    if "index_score" in res:
        out["score_frac"] = res["index_score"]["frac"]
    if "decode_one_query_us" in res:
        out["decode_one_query_us"] = res["decode_one_query_us"]
    cfg = res.get("config", {})
    out["shape"] = " ".join(f"{k}={v}" for k, v in cfg.items()
                            if isinstance(v, (int, float)) and not isinstance(v, bool)
                            and k not in ("width", "page_tokens", "head_dim", "quantized_dims", "block",
                                          "table_blocks", "launches_per_layer", "live_slots", "scores_computed",
                                          "pages", "slots_per_query"))
    if "cpu_baseline" in res:
        c = res["cpu_baseline"]
        m = re.search(r"within ([0-9.e+-]+)", c["sample"])
        out["checked"] = m.group(1) if m else "equal"
        out["cpu"] = {"value": c["value"], "cores": c["cores"]}
        if c["unit"] != res["unit"]:
            out["cpu"]["unit"] = c["unit"]
    return out


def host_threads():
    """(threads the CPU baseline uses, processors this process may run on, processors the box has)."""
    try:
        usable = len(os.sched_getaffinity(0))
    except AttributeError:
        usable = os.cpu_count() or 1
    return max(1, min(16, usable)), usable, os.cpu_count() or 1


_TRAFFIC = None


def measured_traffic(key):
    """HBM bytes per launch of a workload's dominant kernel, from rocprofv3 --pmc FETCH_SIZE and
    WRITE_SIZE runs of that workload scaled by a plain copy of known size. Counters cannot be
    read from inside the process, so the figures are kept in profiles/traffic.json by shape;
    a shape that was not measured reports null."""
    global _TRAFFIC
    if _TRAFFIC is None:
        try:
            with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
                _TRAFFIC = json.load(f)
        except (OSError, ValueError):
            _TRAFFIC = {}
    entry = _TRAFFIC.get(key)
    return entry["bytes"] if isinstance(entry, dict) else None


def bench_decode(a, torch, hip):
    """Benchmark configuration 3: per layer, append one token per sequence, then gather and
    dequantize every sequence's context."""
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
    cols = max(blocks, a.table_blocks)
    if cols > blocks:
        tables_np = np.concatenate([tables_np, np.full((B, cols - blocks), -1, np.int32)], axis=1)
    tables = torch.from_numpy(tables_np.copy()).cuda()
    slots_all = torch.from_numpy(slots_np).cuda()
    seq_lens_np = context_lengths(a, rng)
    cu_np = np.concatenate([[0], np.cumsum(seq_lens_np)]).astype(np.int32)
    seq_lens, cu = torch.from_numpy(seq_lens_np).cuda(), torch.from_numpy(cu_np).cuda()
    # the step's new tokens: the last position of every sequence
    new_slots = torch.from_numpy(slots_np.reshape(B, ctx)[np.arange(B), seq_lens_np - 1].copy()).cuda()
    n_att = int(seq_lens_np.sum())                              # tokens gathered per layer

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

    fused = a.one_launch and a.gather_form == "packed"

    def step(events=None):
        for layer in range(L):
            if not fused:
                hip.launch_kv_append_paged(new_rows[layer], new_slots, pools[layer], B, W, PT, n_pages,
                                           None, sh)
            if events is not None:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
            if fused:    # the step's two calls as one launch
                hip.launch_kv_append_gather_paged(new_rows[layer], new_slots, pools[layer], tables, seq_lens, cu,
                                                  out, B, cols, n_att, W, PT, n_pages, None, None, sh)
            elif a.gather_form == "packed":
                hip.launch_kv_gather_paged_packed(pools[layer], tables, seq_lens, cu, out, B, cols, n_att, W,
                                                  PT, n_pages, None, sh)
            else:
                hip.launch_kv_gather_paged(pools[layer], tables, seq_lens, cu, out, B, cols, W, PT, n_pages,
                                           None, sh)
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
    table_entries = int((-(-seq_lens_np // PT)).sum())
    gather_bytes_layer = n_att * (REC + ROW_IN) + table_entries * 4  # records + table in, bf16 out
    step_bytes = append_bytes + L * gather_bytes_layer
    if fused:  # the launch that is bracketed also appends: its new rows in, their records out
        # (the new tokens' bf16 rows come from the rows just quantized, not from their records)
        gather_bytes_layer += B * (ROW_IN + 4 + REC) - B * REC
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    achieved = gather_bytes_layer / (gather_ms * 1e-3) / 1e9

    result = {
        "metric": "kv_append_gather_GBps", "value": round(value, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": ("cfg3 batched decode, contexts ~U[1024, ctx]" if a.ragged else
                                "cfg3 batched decode at its metric point") +
                               ": per layer append 1 token/seq, gather+dequantize every context",
                   "layers": L, "batch": B, "ctx": ctx, "page_tokens": PT, "width": W,
                   "stored": "fp8 e4m3 + 1 f32 scale/token", "out": "bf16",
                   "contexts": "uniform in [1024, ctx]" if a.ragged else "all at ctx",
                   "tokens_per_layer": n_att, "table_blocks": cols, "gather_form": a.gather_form,
                   "launches_per_layer": 1 if fused else 2},
        "decode_step_kv_ms": round(ms_per_step, 4),
        "tokens_per_s": round(L * n_att / (ms_per_step * 1e-3), 1),
        "hbm_peak_frac": round(value * 1e9 / HBM_PEAK, 4),
        # rivoli_kv_gather_paged_packed takes the launch sized by the token count when the batch fills
        # less than 0.7 of what its block tables could hold (kv_gather.hip: gather_paged_launch)
        "roofline": {"bound": "hbm",
                     "kernel": ("kv_gather_flat_kernel" if a.gather_form == "packed" and n_att * 10 < B * cols * PT * 7
                                else "kv_gather_paged_kernel") + (" (with the step's appends)" if fused else ""),
                     "achieved": round(achieved, 1),
                     "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": round(achieved * 1e9 / HBM_PEAK, 4),
                     "avg_launch_ms": round(gather_ms, 5), "bytes_per_launch": gather_bytes_layer,
                     "traffic": measured_traffic(f"decode:b{B}:ctx{ctx}:{'ragged' if a.ragged else 'uniform'}")},
    }

    if not a.no_cpu_baseline:
        regather = None
        if fused:   # layer 0's step again: the append rewrites the same record, the gather is checked
            regather = lambda: hip.launch_kv_append_gather_paged(new_rows[0], new_slots, pools[0], tables, seq_lens,
                                                                 cu, out, B, cols, n_att, W, PT, n_pages)
        result["cpu_baseline"] = cpu_baseline(pools[0], tables_np, seq_lens_np, out, a.cpu_seconds,
                                              hip, tables, seq_lens, cu, B, cols, n_pages, regather)
    return result


def timed(torch, stream, steps, warmup, step):
    """Warm up, time `steps` calls of step(None) with one HIP event pair around all of them (the
    step time), then run the same `steps` calls again as step(events) with every kernel
    bracketed by its own event pair (the per-kernel times). The two passes are separate because
    an event pair per launch keeps the launches of a short step from queueing ahead of the
    device: the bracketed pass of the configuration 4 step takes 2.9 ms where the plain one
    takes 2.1 ms."""
    for _ in range(warmup):
        step(None)
    stream.synchronize()
    torch.cuda.synchronize()
    t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0.record(stream)
    for _ in range(steps):
        step(None)
    t1.record(stream)
    stream.synchronize()
    torch.cuda.synchronize()
    events = {}
    for _ in range(steps):
        step(events)
    stream.synchronize()
    torch.cuda.synchronize()
    per_kernel = {k: float(np.mean([a.elapsed_time(b) for a, b in v])) for k, v in events.items()}
    return t0.elapsed_time(t1) / steps, per_kernel


def bracket(torch, stream, events, name, launch):
    if events is None:
        return launch()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    launch()
    e1.record(stream)
    events.setdefault(name, []).append((e0, e1))


def bench_prefill(a, torch, hip):
    """benchmark configuration 2: `tokens` new 576-wide bf16 rows (0.5% of rows x50) quantize-appended
    into shuffled pages, one layer, one launch per step."""
    n = a.tokens
    n_pages = -(-n // PT)
    page_bytes = hip.kv_page_bytes(PT, W)
    g = torch.Generator(device="cuda")
    g.manual_seed(0x5EED0002)
    rng = np.random.default_rng(0x5EED0002)
    rows = torch.randn(n, W, generator=g, device="cuda", dtype=torch.float32)
    hit = torch.rand(n, generator=g, device="cuda") < 0.005
    rows[hit] *= 50.0
    rows = rows.to(torch.bfloat16)
    table = rng.permutation(n_pages).astype(np.int32)
    pos = np.arange(n)
    slots = torch.from_numpy((table[pos // PT] * PT + pos % PT).astype(np.int32)).cuda()
    pool = torch.zeros(n_pages * page_bytes, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.Stream()
    sh = stream.cuda_stream

    def step(events):
        bracket(torch, stream, events, "append",
                lambda: hip.launch_kv_append_paged(rows, slots, pool, n, W, PT, n_pages, None, sh))

    ms, per = timed(torch, stream, a.steps, a.warmup, step)
    nbytes = n * (ROW_IN + 4 + REC)
    res = {"metric": "kv_append_GBps", "value": round(nbytes / (ms * 1e-3) / 1e9, 2), "unit": "GB/s",
           "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms, 5),
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
           "data": "synthetic",
           "config": {"workload": "prefill bulk append (benchmark configuration 2)", "tokens": n,
                      "pages": n_pages, "width": W, "page_tokens": PT},
           "tokens_per_s": round(n / (ms * 1e-3), 1),
           # (kv_append.hip picks the kernel by the batch's size)
           "roofline": {"bound": "hbm",
                        "kernel": ("kv_append_paged_token_kernel<2>" if n < 512 else
                                   "kv_append_paged_wide_kernel" if n < 20480 else "kv_append_paged_kernel<72>"),
                        "achieved": round(nbytes / (per["append"] * 1e-3) / 1e9, 2),
                        "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                        "frac": round(nbytes / (per["append"] * 1e-3) / HBM_PEAK, 5),
                        "frac_step": round(nbytes / (ms * 1e-3) / HBM_PEAK, 5),
                        "avg_launch_ms": round(per["append"], 5), "bytes_per_launch": nbytes,
                        "traffic": measured_traffic(f"prefill:tokens{n}")}}
    if not a.no_cpu_baseline:
        from oracle.kvoracle import oracle as get_oracle

        ora = get_oracle()
        cores, usable, nproc = host_threads()
        rows_h = rows.view(torch.int16).cpu().numpy().view(np.uint16)
        slots_h, pool_h = slots.cpu().numpy(), np.zeros(n_pages * page_bytes, np.uint8)
        reps, spent = 0, 0.0
        while spent < a.cpu_seconds and reps < 200:
            t0 = time.perf_counter()
            ora.kv_append_paged(rows_h, slots_h, pool_h, W, PT, n_pages, n_threads=cores)
            spent += time.perf_counter() - t0
            reps += 1
        if not np.array_equal(pool.cpu().numpy(), pool_h):
            raise SystemExit("bench: GPU append differs from the CPU oracle")
        res["cpu_baseline"] = {"value": round(nbytes / (spent / reps) / 1e9, 3), "unit": "GB/s",
                               "cores": cores, "nproc": nproc, "usable": usable, "kind": "port",
                               "sample": f"the same {n}-token append x{reps} reps, {cores} host "
                                         "threads; GPU pool bytes checked equal"}
    return res


def ordered_bf16(ora, x):
    """bf16 codes under a monotone ordering, for code-distance comparisons."""
    c = ora.f32_to_bf16(np.ascontiguousarray(x, np.float32)).astype(np.int64)
    return np.where(c & 0x8000, -(c & 0x7FFF), c)


def bench_v4(a, torch, hip):
    """The second cache format at prefill: `tokens` new f32 cache rows of 512 dims are quantized
    and dequantized in place over their first 448 dims at block 64 (the rotated tail keeps its
    precision), and every query row selects its best `index_topk` closed blocks (ratio 4) from
    its row of the [tokens, tokens / 4] score matrix."""
    n, hd, nq, blk, ratio = a.tokens, 512, 448, 64, 4
    n_comp, cap, offset = n // ratio, a.index_topk, 128
    k = min(cap, n_comp)
    g = torch.Generator(device="cuda")
    g.manual_seed(0x5EED0006)
    fresh = torch.randn(n, hd, generator=g, device="cuda", dtype=torch.float32)
    hit = torch.rand(n, generator=g, device="cuda") < 0.01
    fresh[hit] *= 200.0
    kv = fresh.clone()
    scores = torch.randn(n, n_comp, generator=g, device="cuda", dtype=torch.float32)
    sel = torch.empty(n, k, dtype=torch.int32, device="cuda")
    stream = torch.cuda.Stream()
    sh = stream.cuda_stream

    # the attention compressor at ratio 4 (overlapping windows): the projections' outputs for the
    # same tokens, pooled into n / 4 compressed rows
    geom = hip.CompGeom.build(ratio, hd, hd - nq, 1e-6)
    c_kv = torch.randn(n, geom.cd, generator=g, device="cuda", dtype=torch.float32)
    c_score = torch.randn(n, geom.cd, generator=g, device="cuda", dtype=torch.float32) * 2.0
    c_ape = torch.randn(ratio, geom.cd, generator=g, device="cuda", dtype=torch.float32)
    c_norm = 1.0 + 0.1 * torch.randn(hd, generator=g, device="cuda", dtype=torch.float32)
    inv = 160000.0 ** (-torch.arange(geom.rd // 2, device="cuda", dtype=torch.float64) * 2.0 / geom.rd)
    ang = torch.arange(n, device="cuda", dtype=torch.float64)[:, None] * inv[None, :]
    c_freqs = torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1).reshape(n, geom.rd).float().contiguous()
    c_out = torch.empty(n_comp, hd, dtype=torch.float32, device="cuda")
    c_fin = hip.CompFinish.of(c_norm, c_freqs, c_out)

    def step(events):
        bracket(torch, stream, events, "compress",
                lambda: hip.launch_kv_compress_prefill(c_kv, c_score, c_ape, c_fin, geom, n_comp, sh))
        bracket(torch, stream, events, "quant",
                lambda: hip.launch_act_quant_f8_prefix(kv, kv, n, hd, nq, blk, sh))
        bracket(torch, stream, events, "select",
                lambda: hip.launch_index_select_blocks(scores, n, n_comp, ratio, cap, True, offset, sel, sh))

    ms, per = timed(torch, stream, a.steps, a.warmup, step)
    limit = np.minimum((np.arange(n) + 1) // ratio, n_comp)
    quant_bytes = n * nq * 8                                       # f32 in, f32 out
    select_bytes = int(limit[limit > k].sum()) * 4 + n * k * 4     # ranked rows' legal scores in, rows out
    compress_bytes = 2 * n * geom.cd * 4 + n_comp * hd * 4         # kv + score windows in, rows out
    names = {"select": ("block_select_kernel", select_bytes), "quant": ("act_quant_kernel", quant_bytes),
             "compress": ("kv_compress_prefill_kernel", compress_bytes)}
    dom = max(names, key=lambda k_: per[k_])
    dom_bytes = names[dom][1]
    res = {"metric": "v4_cache_compress_quant_select_GBps",
           "value": round((compress_bytes + quant_bytes + select_bytes) / (ms * 1e-3) / 1e9, 1), "unit": "GB/s",
           "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms, 5),
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
           "data": "synthetic",
           "config": {"workload": "second cache format, prefill: pooling of the tokens into compressed rows "
                                  "(ratio 4, overlapping windows), block-64 quantize-dequantize of the "
                                  "new cache rows, scored block selection per query row",
                      "tokens": n, "head_dim": hd, "quantized_dims": nq, "block": blk, "ratio": ratio,
                      "n_comp": n_comp, "index_topk": cap},
           "tokens_per_s": round(n / (ms * 1e-3), 1),
           "kernels": {"kv_compress_prefill_kernel": {"avg_launch_ms": round(per["compress"], 5),
                                                      "bytes_per_launch": compress_bytes,
                                                      "GBps": round(compress_bytes / (per["compress"] * 1e-3) / 1e9, 1)},
                       "act_quant_kernel": {"avg_launch_ms": round(per["quant"], 5), "bytes_per_launch": quant_bytes,
                                            "GBps": round(quant_bytes / (per["quant"] * 1e-3) / 1e9, 1)},
                       "block_select_kernel": {"avg_launch_ms": round(per["select"], 5),
                                               "bytes_per_launch": select_bytes,
                                               "GBps": round(select_bytes / (per["select"] * 1e-3) / 1e9, 1)}},
           "roofline": {"bound": "hbm", "kernel": names[dom][0],
                        "achieved": round(dom_bytes / (per[dom] * 1e-3) / 1e9, 1), "peak": HBM_PEAK / 1e9,
                        "unit": "GB/s", "frac": round(dom_bytes / (per[dom] * 1e-3) / HBM_PEAK, 4),
                        "avg_launch_ms": round(per[dom], 5), "bytes_per_launch": dom_bytes,
                        # measured the same way for the selection at 32 768 tokens, cap 512 (profiles/)
                        "traffic": 604300000 if (dom, n, cap) == ("select", 32768, 512) else None}}
    if not a.no_cpu_baseline:
        from oracle.kvoracle import oracle as get_oracle

        ora = get_oracle()
        # bounded sample: the first rows of the same inputs, one host thread; the sample doubles
        # as a parity check of both kernels
        nr = min(n, 2048)
        x_h, s_h = fresh[:nr].cpu().numpy(), scores[:nr].cpu().numpy()
        t0 = time.perf_counter()
        code, want_kv = ora.act_quant_f8_prefix(x_h, nq, blk)
        want_sel = ora.v4_scored_rows(s_h, ratio, cap, True, offset)
        from oracle.kvoracle import CompGeom as OracleGeom

        og = OracleGeom.attention(ratio, hd, hd - nq)
        code_c, want_c = ora.kv_compress_prefill(c_kv[:nr].cpu().numpy(), c_score[:nr].cpu().numpy(),
                                                 c_ape.cpu().numpy(), c_norm.cpu().numpy(),
                                                 c_freqs[:nr].cpu().numpy(), og, nr // ratio)
        spent = time.perf_counter() - t0
        got_kv, got_sel = kv[:nr].cpu().numpy(), sel[:nr].cpu().numpy()
        if code != 0 or not np.array_equal(got_kv.view(np.uint32), want_kv.view(np.uint32)):
            raise SystemExit("bench: GPU quantize-dequantize differs from the CPU oracle")
        if not np.array_equal(got_sel, want_sel):
            raise SystemExit("bench: GPU block selection differs from the CPU oracle")
        got_c = c_out[: nr // ratio].cpu().numpy()
        gap = np.abs(ordered_bf16(ora, got_c) - ordered_bf16(ora, want_c))
        # a value that cancelled to almost nothing against its row carries the terms' absolute
        # error, which is many codes of the small result: those are compared absolutely, to
        # 2^-14 of the row's largest value (2^-8 in the rotated tail)
        top = np.abs(want_c).max(axis=1, keepdims=True)
        near = np.abs(got_c - want_c) <= top * np.where((np.arange(hd) >= nq)[None, :], 2.0 ** -8, 2.0 ** -14)
        gap = np.where(near, np.minimum(gap, 2), gap)
        if code_c != 0 or gap.max() > 2 or np.mean(gap > 0) > 0.01:
            raise SystemExit(f"bench: GPU compressor pooling is more than 2 bf16 codes from the CPU oracle "
                             f"(code {code_c}, max gap {gap.max()}, differing {np.mean(gap > 0):.4f})")
        sample_bytes = (nr * nq * 8 + int(limit[:nr][limit[:nr] > k].sum()) * 4 + nr * k * 4
                        + 2 * nr * geom.cd * 4 + (nr // ratio) * hd * 4)
        res["cpu_baseline"] = {"value": round(sample_bytes / spent / 1e9, 3), "unit": "GB/s", "cores": 1,
                               "kind": "port",
                               "sample": f"the first {nr} rows of the same inputs through the oracle's "
                                         "compressor pooling, act_quant and scored_rows, one host thread; "
                                         "GPU results checked (pooling within 2 bf16 codes, the others equal)"}
    return res


def bench_v4_index(a, torch, hip):
    """The second cache format's block indexer at prefill (crates/engine/src/v4/blocksel.rs:218-248):
    `tokens` queries x `heads` index heads of 128 are spread in place (Hadamard + simulated fp4),
    then every query is scored against the tokens / 4 compressed blocks (spread rows as well)."""
    s, heads, hd, ratio = a.tokens, a.heads, 128, 4
    n_comp = max(s // ratio, 1)
    g = torch.Generator(device="cuda")
    g.manual_seed(0x5EED0007)
    q_raw = torch.randn(s * heads, hd, generator=g, device="cuda", dtype=torch.float32).bfloat16().float()
    kv = torch.randn(n_comp, hd, generator=g, device="cuda", dtype=torch.float32).bfloat16().float()
    w = (torch.randn(s, heads, generator=g, device="cuda", dtype=torch.float32) * hd ** -0.5).bfloat16().float()
    hip.launch_act_quant_f4_rotated(kv, n_comp, hd)     # the indexer compressor's finish
    q = q_raw.clone()
    score = torch.empty(s, n_comp, dtype=torch.float32, device="cuda")
    stream = torch.cuda.Stream()
    sh = stream.cuda_stream

    def step(events):
        bracket(torch, stream, events, "spread", lambda: hip.launch_act_quant_f4_rotated(q, s * heads, hd, sh))
        if a.full_scores:   # the reference's rectangle: every query against every block
            bracket(torch, stream, events, "score",
                    lambda: hip.launch_index_score_blocks(q, kv, w, score, s, n_comp, heads, hd, sh))
        else:               # what a prefill's selection can rank: block < (t + 1) / ratio
            bracket(torch, stream, events, "score",
                    lambda: hip.launch_index_score_blocks_prefill(q, kv, w, score, s, n_comp, heads, hd, ratio, sh))

    ms, per = timed(torch, stream, a.steps, a.warmup, step)
    spread_bytes = s * heads * hd * 8                                   # f32 in, f32 out
    limit = np.minimum((np.arange(s) + 1) // ratio, n_comp)
    scored = s * n_comp if a.full_scores else int((-(-limit // 64) * 64).clip(max=-(-n_comp // 64) * 64).sum())
    score_flops = 2 * scored * heads * hd                               # one multiply and one add per term
    score_bytes = s * heads * hd * 4 + n_comp * hd * 4 + s * n_comp * 4
    # the timed steps spread the same buffer again and again; the check runs one step on a fresh copy
    q.copy_(q_raw)
    torch.cuda.synchronize()
    step(None)
    stream.synchronize()
    legal = s * n_comp if a.full_scores else int(limit.sum())
    res = {"metric": "v4_block_index_scores_per_s", "value": round(legal / (ms * 1e-3), 1), "unit": "scores/s",
           "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms, 5),
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "second cache format, prefill: Hadamard + fp4 spread of the index queries, block "
                                  "scores of every query against every compressed block (sequential f32 folds, "
                                  "bit-identical to the reference's kernel)",
                      "tokens": s, "heads": heads, "head_dim": hd, "ratio": ratio, "n_comp": n_comp,
                      "entries": "all" if a.full_scores else "legal (block < (t + 1) / ratio), in groups of 64 blocks",
                      "scores_per_step": legal, "scores_computed": scored},
           "tokens_per_s": round(s / (ms * 1e-3), 1),
           "kernels": {"f4_rotated_kernel": {"avg_launch_ms": round(per["spread"], 5), "bytes_per_launch": spread_bytes,
                                             "GBps": round(spread_bytes / (per["spread"] * 1e-3) / 1e9, 1)},
                       "index_score_blocks_kernel": {"avg_launch_ms": round(per["score"], 5),
                                                     "flops_per_launch": score_flops, "bytes_per_launch": score_bytes,
                                                     "TFLOPps": round(score_flops / (per["score"] * 1e-3) / 1e12, 2)}},
           # the scorer is bound by vector issue, not by memory or the matrix cores: the published
           # fp32 vector peak counts a fused multiply-add on packed pairs as four operations per lane
           # and cycle; the reference's two roundings per term allow one
           "roofline": {"bound": "fp32", "kernel": "index_score_blocks_kernel",
                        "achieved": round(score_flops / (per["score"] * 1e-3) / 1e12, 2), "peak": 157.3,
                        "unit": "TFLOP/s", "frac": round(score_flops / (per["score"] * 1e-3) / 157.3e12, 4),
                        "unfused_unpacked_peak": 39.3,
                        "frac_of_unfused_unpacked_peak": round(score_flops / (per["score"] * 1e-3) / 39.3e12, 4),
                        "avg_launch_ms": round(per["score"], 5), "traffic": None}}
    # a decode step of the same layer: one query against the ctx / ratio blocks of a long context
    d_comp = max(a.ctx // ratio, 1)
    d_kv = torch.randn(d_comp, hd, generator=g, device="cuda", dtype=torch.float32).bfloat16().float()
    hip.launch_act_quant_f4_rotated(d_kv, d_comp, hd)
    d_q = q_raw[:heads].clone()
    d_score = torch.empty(d_comp, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()

    def decode_step(events):
        bracket(torch, stream, events, "spread", lambda: hip.launch_act_quant_f4_rotated(d_q, heads, hd, sh))
        bracket(torch, stream, events, "score",
                lambda: hip.launch_index_score_blocks(d_q, d_kv, w, d_score, 1, d_comp, heads, hd, sh))

    d_ms, d_per = timed(torch, stream, max(a.steps, 20), a.warmup, decode_step)
    res["decode_one_query_us"] = {"blocks": d_comp, "step": round(d_ms * 1e3, 2),
                                  "spread": round(d_per["spread"] * 1e3, 2), "score": round(d_per["score"] * 1e3, 2)}
    if not a.no_cpu_baseline:
        from oracle.kvoracle import oracle as get_oracle

        ora = get_oracle()
        d_q.copy_(q_raw[:heads])
        torch.cuda.synchronize()
        decode_step(None)
        stream.synchronize()
        code_d, want_d = ora.index_score_blocks(ora.act_quant_f4_rotated(q_raw[:heads].cpu().numpy())[1][None],
                                                d_kv.cpu().numpy(), w[:1].cpu().numpy())
        if code_d != 0 or not np.array_equal(d_score.cpu().numpy().view(np.uint32), want_d.view(np.uint32).ravel()):
            raise SystemExit("bench: GPU decode block scores differ from the CPU oracle")
        rows = sorted({0, 1, s // 2, s - 1} | set(range(min(s, 12))))
        q_h = q_raw.view(s, heads, hd)[rows].cpu().numpy()
        kv_h, w_h = kv.cpu().numpy(), w[rows].cpu().numpy()
        t0 = time.perf_counter()
        code_q, want_q = ora.act_quant_f4_rotated(q_h.reshape(-1, hd))
        code_s, want_s = ora.index_score_blocks(want_q.reshape(len(rows), heads, hd), kv_h, w_h)
        spent = time.perf_counter() - t0
        got_q = q.view(s, heads, hd)[rows].cpu().numpy().reshape(-1, hd)
        got_s = score[rows].cpu().numpy()
        if not a.full_scores:   # only the legal entries are defined
            keep = np.arange(n_comp)[None, :] < limit[rows][:, None]
            got_s, want_s = np.where(keep, got_s, 0.0).astype(np.float32), np.where(keep, want_s, 0.0).astype(np.float32)
        if code_q != 0 or not np.array_equal(got_q.view(np.uint32), want_q.view(np.uint32)):
            raise SystemExit("bench: GPU spread differs from the CPU oracle")
        if code_s != 0 or not np.array_equal(got_s.view(np.uint32), want_s.view(np.uint32)):
            raise SystemExit("bench: GPU block scores differ from the CPU oracle")
        res["cpu_baseline"] = {"value": round(len(rows) * n_comp / spent, 1), "unit": "scores/s", "cores": 1,
                               "kind": "port",
                               "sample": f"{len(rows)} query rows of the same inputs through the oracle's spread and "
                                         "block scorer, one host thread; GPU results bit-equal"}
        res["cpu_baseline"]["nproc"] = host_threads()[2]
    return res


def bench_v4_attend(a, torch, hip):
    """The second cache format's consumer at prefill, one layer of the indexed class (window 128,
    ratio 4): the prompt's last 128 rows go into the ring, every query row gets its
    [window | best index_topk closed blocks] index list, and all heads of every query attend over
    those rows of the [prompt rows | compressed rows] buffer (key = value = the 512-wide row)."""
    n, h, d, win, ratio, cap = a.tokens, a.heads, 512, 128, 4, a.index_topk
    n_comp = n // ratio
    g = torch.Generator(device="cuda")
    g.manual_seed(0x5EED0007)
    # what the model hands over: q rounded to bf16 after its rotary; cache rows quantized and
    # dequantized over their first 448 dims, bf16 values in the rotated tail
    q = torch.randn(n, h, d, generator=g, device="cuda", dtype=torch.float32).bfloat16().float()
    kv = torch.randn(n + n_comp, d, generator=g, device="cuda", dtype=torch.float32).bfloat16().float()
    hip.launch_act_quant_f8_prefix(kv, kv, n + n_comp, d, 448, 64)
    sink = torch.randn(h, generator=g, device="cuda", dtype=torch.float32)
    scores = torch.randn(n, n_comp, generator=g, device="cuda", dtype=torch.float32)
    cols = min(n, win) + min(cap, n_comp)
    idx = torch.empty(n, cols, dtype=torch.int32, device="cuda")
    ring = torch.zeros(win, d, dtype=torch.float32, device="cuda")
    o = torch.empty(n, h, d, dtype=torch.float32, device="cuda")
    scale = d ** -0.5
    stream = torch.cuda.Stream()
    sh = stream.cuda_stream

    def step(events):
        bracket(torch, stream, events, "ring", lambda: hip.launch_kv_ring_write(kv, ring, win, d, n, 0, sh))
        bracket(torch, stream, events, "select",
                lambda: hip.launch_sel_gather_scored(scores, n_comp, win, ratio, cap, n, 0, idx, sh))
        bracket(torch, stream, events, "attend",
                lambda: hip.launch_gather_attn_shared_kv(q, kv, sink, idx, n, h, d, cols, scale, o, sh,
                                                         precise=a.precise))

    ms, per = timed(torch, stream, a.steps, a.warmup, step)
    live = int((idx >= 0).sum().item())
    flops = 4.0 * h * d * live                                    # scores and values, 2 flops per multiply-add
    hbm_bytes = 2 * n * h * d * 4 + (n + n_comp) * d * 4 + n * cols * 4   # q in, o out, every row once, the lists
    att = per["attend"] * 1e-3
    res = {"metric": "v4_gather_attn_TFLOPs", "value": round(flops / (ms * 1e-3) / 1e12, 2), "unit": "TFLOP/s",
           "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms, 5),
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
           "data": "synthetic",
           "config": {"workload": "second cache format, prefill consumer: ring write, [window | scored blocks] "
                                  "selection, index-list attention with shared key/value rows",
                      "tokens": n, "heads": h, "head_dim": d, "window": win, "ratio": ratio, "index_topk": cap,
                      "slots_per_query": cols, "live_slots": live, "precise": a.precise},
           "queries_per_s": round(n / (ms * 1e-3), 1),
           "kernels_ms": {k_: round(v, 5) for k_, v in per.items()},
           "roofline": {"bound": "mfma", "kernel": "gather_attn_d512_kernel",
                        "achieved": round(flops / att / 1e12, 2), "peak": 2500.0, "unit": "TFLOP/s",
                        "frac": round(flops / att / 2.5e15, 4), "avg_launch_ms": round(per["attend"], 5),
                        "flops_per_launch": flops,
                        # HBM bytes per launch by rocprofv3 FETCH_SIZE + WRITE_SIZE on this workload,
                        # each scaled by its reading for a known 1 GiB copy (profiles/); it cannot
                        # be read from inside the process
                        "traffic": 2917700000 if (n, h, cap) == (8192, 64, 512) else None,
                        "hbm": {"bytes_per_launch": hbm_bytes, "achieved_GBps": round(hbm_bytes / att / 1e9, 1),
                                "frac": round(hbm_bytes / att / HBM_PEAK, 4)}}}
    # the reference's decode shape: ONE query row over the same 640-slot list, with the list
    # shared among workgroups through a partial buffer, and without
    part = torch.empty(max(hip.gather_attn_scratch_floats(1, h, d, cols), 4), dtype=torch.float32, device="cuda")
    o1 = torch.empty(h, d, dtype=torch.float32, device="cuda")

    def decode_step(events):
        bracket(torch, stream, events, "split",
                lambda: hip.launch_gather_attn_shared_kv(q[n - 1], kv, sink, idx[n - 1], 1, h, d, cols, scale, o1,
                                                         sh, precise=a.precise, partial=part))
        bracket(torch, stream, events, "whole",
                lambda: hip.launch_gather_attn_shared_kv(q[n - 1], kv, sink, idx[n - 1], 1, h, d, cols, scale, o1,
                                                         sh, precise=a.precise))

    _, per_decode = timed(torch, stream, 20, 3, decode_step)
    res["decode_one_query_us"] = {"split_over_slots": round(per_decode["split"] * 1e3, 2),
                                  "one_workgroup": round(per_decode["whole"] * 1e3, 2)}
    if not a.no_cpu_baseline:
        from oracle.kvoracle import oracle as get_oracle

        ora = get_oracle()
        # bounded sample: the last queries of the prompt (full index lists), one host thread;
        # doubles as the parity check, at the reference's bar for this kernel
        nq = min(n, 48)
        q_h, idx_h = q[n - nq:].cpu().numpy(), idx[n - nq:].cpu().numpy()
        kv_h, sink_h = kv.cpu().numpy(), sink.cpu().numpy()
        t0 = time.perf_counter()
        want = ora.sparse_attn(q_h, kv_h, sink_h, idx_h, scale)
        spent = time.perf_counter() - t0
        got = o[n - nq:].cpu().numpy()
        err = float(np.max(np.abs(got - want)) / np.max(np.abs(want)))
        if not err <= 1.0 / 128.0:
            raise SystemExit(f"bench: GPU index-list attention is {err:.4g} of the largest element from the CPU "
                             "oracle (bar 1/128)")
        want_idx = ora.sel_gather_scored(scores[n - nq:].cpu().numpy() if n == nq else scores.cpu().numpy(), win,
                                         ratio, cap, n, 0)[1] if n <= 4096 else None
        if want_idx is not None and not np.array_equal(idx.cpu().numpy(), want_idx):
            raise SystemExit("bench: GPU selection rectangle differs from the CPU oracle")
        sample_flops = 4.0 * h * d * int((idx_h >= 0).sum())
        res["cpu_baseline"] = {"value": round(sample_flops / spent / 1e12, 6), "unit": "TFLOP/s", "cores": 1,
                               "kind": "port",
                               "sample": f"the last {nq} queries of the same inputs through the oracle's "
                                         f"sparse_attn, one host thread; GPU output within {err:.2g} of the "
                                         "largest element (bar 1/128)"}
    return res


def bench_dsa(a, torch, hip, scored=False, attend=False):
    """benchmark configuration 4: per layer, select the top-k of 65536 indexer scores for each of 16
    queries (ties to the lowest index), then gather + dequantize those rows from fragmented
    pages. One step = all layers."""
    L, B, nt, k = a.layers, (16 if a.batch == 32 else a.batch), (65536 if a.ctx == 32768 else a.ctx), a.topk
    blocks = -(-nt // PT)
    n_pages = B * blocks
    page_bytes = hip.kv_page_bytes(PT, W)
    g = torch.Generator(device="cuda")
    g.manual_seed(0x5EED0004)
    rng = np.random.default_rng(0x5EED0004)
    tables_np = rng.permutation(n_pages).astype(np.int32).reshape(B, blocks)
    pos = np.arange(nt)
    slots_np = np.concatenate([tables_np[s][pos // PT] * PT + pos % PT for s in range(B)]).astype(np.int32)
    tables, slots_all = torch.from_numpy(tables_np.copy()).cuda(), torch.from_numpy(slots_np).cuda()
    kv_rows = torch.randn(B * nt, W, generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    pools = []
    for _ in range(L):
        pool = torch.empty(n_pages * page_bytes, dtype=torch.uint8, device="cuda")
        hip.launch_kv_append_paged(kv_rows, slots_all, pool, B * nt, W, PT, n_pages)
        pools.append(pool)
    del kv_rows
    scores = []
    NH, HD = 64, 128                                             # indexer heads x head dim
    if scored:
        # one paged bf16 key cache per layer (same block tables), filled by index_append_paged;
        # every layer gets its own queries and head weights
        keys = torch.randn(B * nt, HD, generator=g, device="cuda", dtype=torch.float32)
        kpools, qs, ws = [], [], []
        for _ in range(L):
            kp = torch.empty(n_pages * PT * HD, dtype=torch.bfloat16, device="cuda")
            hip.launch_index_append_paged(keys, slots_all, kp, B * nt, HD, PT, n_pages)
            kpools.append(kp)
            qs.append(torch.randn(B, NH, HD, generator=g, device="cuda", dtype=torch.float32))
            ws.append(torch.rand(B, NH, generator=g, device="cuda", dtype=torch.float32))
        del keys
        score_buf = torch.empty(B, nt, dtype=torch.float32, device="cuda")
    else:
        for _ in range(L):
            sc = torch.randn(B, nt, generator=g, device="cuda", dtype=torch.float32)
            sc[:, -64:] += 4.0                                   # recency boost
            scores.append(sc)
    sel = torch.empty(B * k, dtype=torch.int32, device="cuda")
    out = torch.empty(B * k * W, dtype=torch.bfloat16, device="cuda")
    H = a.heads
    if attend:
        qabs = [torch.randn(B, H, 512, generator=g, device="cuda", dtype=torch.float32) for _ in range(L)]
        qrope = [torch.randn(B, H, 64, generator=g, device="cuda", dtype=torch.float32) for _ in range(L)]
        clat = torch.empty(B, H, 512, dtype=torch.float32, device="cuda")
        partial = torch.empty(max(hip.mla_attend_paged_scratch_floats(B, H, k), 1), dtype=torch.float32,
                              device="cuda")
    ws_topk = torch.zeros(hip.index_topk_workspace_bytes(B, nt), dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    sh = stream.cuda_stream

    fused = not attend and not a.unfused

    score = hip.launch_index_score_paged_hist if fused else hip.launch_index_score_paged

    def step(events):
        for layer in range(L):
            if scored:
                tail = (ws_topk, sh) if fused else (sh,)
                bracket(torch, stream, events, "score",
                        lambda: score(qs[layer], ws[layer], kpools[layer], tables, None, None, B, blocks, nt,
                                      nt, NH, NH, HD, PT, n_pages, HD ** -0.5, 1.0, score_buf, *tail))
            sc_in = score_buf if scored else scores[layer]
            if fused:
                bracket(torch, stream, events, "select_gather",
                        lambda: hip.launch_dsa_select_gather_paged(sc_in, B, nt, None, nt, k, sel, ws_topk, scored,
                                                                   pools[layer], tables, out, blocks, W, PT,
                                                                   n_pages, None, sh))
                continue
            bracket(torch, stream, events, "topk",
                    lambda: hip.launch_index_topk_batched(sc_in, B, nt, None, nt, k, sel, ws_topk, sh))
            if attend:
                bracket(torch, stream, events, "attend_rows",
                        lambda: hip.launch_mla_attend_paged(qabs[layer], qrope[layer], pools[layer], tables, None,
                                                            sel, None, B, H, k, blocks, 512, 64, PT, n_pages,
                                                            float(W) ** -0.5, a.precise, clat, partial, None, sh))
            else:
                bracket(torch, stream, events, "gather_rows",
                        lambda: hip.launch_kv_gather_rows_paged(pools[layer], tables, sel, None, out, B, k,
                                                                blocks, W, PT, n_pages, None, sh))

    ms, per = timed(torch, stream, a.steps, a.warmup, step)
    topk_bytes = B * nt * 4 + B * k * 4
    rows_bytes = B * k * (4 + REC + ROW_IN) + B * blocks * 4
    if attend:  # row list, records and table in, q in, clat out; no bf16 rows are written
        rows_bytes = B * k * (4 + REC) + B * blocks * 4 + B * H * (W + 512) * 4
    rows_kernel = "attend_rows" if attend else ("select_gather" if fused else "gather_rows")
    score_bytes = (B * nt * (HD * 2 + 4) + B * NH * (HD + 1) * 4 + B * blocks * 4) if scored else 0
    layer_bytes = topk_bytes + rows_bytes + score_bytes
    dom_bytes = topk_bytes + rows_bytes if fused else rows_bytes
    res = {"metric": "kv_dsa_topk_gather_GBps", "value": round(L * layer_bytes / (ms * 1e-3) / 1e9, 2),
           "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
           "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "DSA sparse path (benchmark configuration 4): top-k then sparse row gather"
                                  + (", one fused call per layer" if fused else ""),
                      "layers": L, "batch": B, "ctx": nt, "k": k, "width": W, "page_tokens": PT},
           "rows_per_s": round(L * B * k / (ms * 1e-3), 1),
           "layer_us": round(ms * 1e3 / L, 2), "hbm_peak_frac": round(L * layer_bytes / (ms * 1e-3) / HBM_PEAK, 4),
           "kernels_ms": {n: round(v, 5) for n, v in per.items()},
           "roofline": {"bound": "hbm",
                        "kernel": "mla_attend_paged_kernel" if attend else
                                  ("topk_hist + topk_cand + topk_finish_bits (select and gather)" if fused
                                   else "kv_gather_rows_kernel"),
                        "achieved": round(dom_bytes / (per[rows_kernel] * 1e-3) / 1e9, 2),
                        "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                        "frac": round(dom_bytes / (per[rows_kernel] * 1e-3) / HBM_PEAK, 5),
                        "avg_launch_ms": round(per[rows_kernel], 5),
                        "bytes_per_launch": dom_bytes,
                        "traffic": measured_traffic(f"dsa:b{B}:ctx{nt}:k{k}") if fused and not scored else None}}
    if fused and not scored:  # the step IS one such call per layer
        res["roofline"]["frac_step"] = round(dom_bytes / (ms * 1e-3 / L) / HBM_PEAK, 5)
    if not fused:
        res["topk"] = {"achieved": round(topk_bytes / (per["topk"] * 1e-3) / 1e9, 2), "unit": "GB/s",
                       "avg_launch_ms": round(per["topk"], 5), "bytes_per_launch": topk_bytes}
    if scored:
        res["config"]["workload"] = ("DSA sparse path with device scores: index_score (64 heads x "
                                     "128, paged bf16 keys) -> top-k -> sparse row gather")
        res["index_score"] = {"achieved": round(score_bytes / (per["score"] * 1e-3) / 1e9, 2),
                              "unit": "GB/s", "frac": round(score_bytes / (per["score"] * 1e-3) / HBM_PEAK, 4),
                              "avg_launch_ms": round(per["score"], 5), "bytes_per_launch": score_bytes,
                              "tflops": round(B * nt * NH * HD * 2 * 2 / (per["score"] * 1e-3) / 1e12, 1),
                              "traffic": measured_traffic(f"dsa_scored:b{B}:ctx{nt}:h{NH}")}
    if attend:
        res["metric"] = "kv_dsa_topk_attend_GBps"
        res["config"]["workload"] = ("DSA sparse path with the consumer fused: top-k, then MLA latent attention "
                                     "over the selected rows straight from the fp8 pages")
        res["config"]["heads"], res["config"]["precise"] = H, a.precise
    if not a.no_cpu_baseline:
        from oracle.kvoracle import oracle as get_oracle

        ora = get_oracle()
        cores, usable, nproc = host_threads()
        pool_h = pools[0].cpu().numpy()
        note = ""
        if scored:
            # layer 0's scores as the device computed them: a sample of them against the oracle's
            # scorer (the reference's bar for that kernel, 1e-5 of the largest score:
            # crates/engine/tests/indexer_kernel.rs:351-366), then the selection and the gather
            # on exactly those scores
            score(qs[0], ws[0], kpools[0], tables, None, None, B, blocks, nt, nt, NH, NH, HD, PT, n_pages,
                  HD ** -0.5, 1.0, score_buf, *((ws_topk,) if fused else ()))
            torch.cuda.synchronize()
            sc_h = score_buf.cpu().numpy()
            n_s = 4096
            want_sc = ora.index_score_paged(qs[0][:1].cpu().numpy(), ws[0][:1].cpu().numpy(),
                                            kpools[0].view(torch.int16).cpu().numpy().view(np.uint16),
                                            tables_np[:1], np.array([n_s], np.int32), None, n_s, HD, PT,
                                            HD ** -0.5, 1.0, n_threads=cores)
            err = float(np.abs(sc_h[0, :n_s] - want_sc[0]).max() / np.abs(want_sc[0]).max())
            if not err <= 1e-5:
                raise SystemExit(f"bench: device scores differ from the CPU oracle ({err:.2e} of the largest)")
            note = f"; device scores of query 0's first {n_s} tokens: error {err:.1e} of the largest (bar 1e-5)"
        else:
            sc_h = scores[0].cpu().numpy()
        reps, spent = 0, 0.0
        while spent < a.cpu_seconds and reps < 50:
            t0 = time.perf_counter()
            want_sel = ora.topk_batched(sc_h, k, n_threads=cores)
            want_rows = None if attend else ora.kv_gather_rows_paged(pool_h, tables_np, want_sel, W, PT)
            spent += time.perf_counter() - t0
            reps += 1
        sc_d = score_buf if scored else scores[0]
        if fused:
            hip.launch_dsa_select_gather_paged(sc_d, B, nt, None, nt, k, sel, ws_topk, scored, pools[0], tables,
                                               out, blocks, W, PT, n_pages)
        else:
            hip.launch_index_topk_batched(sc_d, B, nt, None, nt, k, sel, ws_topk)
            if not attend:
                hip.launch_kv_gather_rows_paged(pools[0], tables, sel, None, out, B, k, blocks, W, PT, n_pages)
        torch.cuda.synchronize()
        if not np.array_equal(sel.cpu().numpy().view(np.uint32).reshape(B, k), want_sel):
            raise SystemExit("bench: GPU top-k differs from the CPU oracle")
        if attend:
            # the attention over the selected rows: two queries through the oracle (the reference's
            # bar for that kernel, crates/engine/tests/kernel_attend.rs:267)
            n_chk = 2
            hip.launch_mla_attend_paged(qabs[0], qrope[0], pools[0], tables, None, sel, None, B, H, k, blocks, 512,
                                        64, PT, n_pages, float(W) ** -0.5, a.precise, clat, partial)
            torch.cuda.synchronize()
            want_att = ora.mla_attend_paged(qabs[0][:n_chk].cpu().numpy(), qrope[0][:n_chk].cpu().numpy(), pool_h,
                                            tables_np[:n_chk], np.full(n_chk, nt, np.int32), want_sel[:n_chk], None,
                                            512, 64, PT, float(W) ** -0.5, n_threads=cores)
            got_att = clat.cpu().numpy()[:n_chk]
            err = float(np.abs(got_att - want_att).max() / np.abs(want_att).max())
            if not err <= 1e-3:
                raise SystemExit(f"bench: attention over the selected rows differs from the oracle ({err:.2e})")
            sample = (f"one layer's top-k on {cores} host threads x{reps} reps, GPU indices checked equal; attention "
                      f"of {n_chk} queries over their {k} rows within {err:.1e} of the oracle's")
            cpu_bytes = topk_bytes
        else:
            if not np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16).reshape(B, k, W), want_rows):
                raise SystemExit("bench: GPU sparse gather differs from the CPU oracle")
            sample = (f"one layer (top-k on {cores} host threads, sparse gather single-threaded) x{reps} reps; "
                      "GPU indices and rows checked equal" + note)
            cpu_bytes = topk_bytes + rows_bytes
        res["cpu_baseline"] = {"value": round(cpu_bytes / (spent / reps) / 1e9, 3), "unit": "GB/s",
                               "cores": cores, "nproc": nproc, "usable": usable, "kind": "port",
                               "sample": sample}
    return res


def bench_attend(a, torch, hip):
    """benchmark configuration 3 with the consumer fused in: per layer, append one token per sequence,
    then MLA decode attention for `heads` query heads over every sequence's full context,
    straight from the fp8 pages (no bf16 copy of the cache is made)."""
    L, B, ctx, H = a.layers, a.batch, a.ctx, a.heads
    KVL, ROPE = 512, 64
    blocks = -(-ctx // PT)
    n_pages = B * blocks
    page_bytes = hip.kv_page_bytes(PT, W)
    n_tok = B * ctx
    g = torch.Generator(device="cuda")
    g.manual_seed(0x5EED0003)
    rng = np.random.default_rng(0x5EED0003)
    tables_np = rng.permutation(n_pages).astype(np.int32).reshape(B, blocks)
    pos = np.arange(ctx)
    slots_np = np.concatenate([tables_np[s][pos // PT] * PT + pos % PT for s in range(B)]).astype(np.int32)
    tables, slots_all = torch.from_numpy(tables_np.copy()).cuda(), torch.from_numpy(slots_np).cuda()
    seq_lens_np = context_lengths(a, rng)
    seq_lens = torch.from_numpy(seq_lens_np).cuda()
    new_slots = torch.from_numpy(slots_np.reshape(B, ctx)[np.arange(B), seq_lens_np - 1].copy()).cuda()
    n_att = int(seq_lens_np.sum())
    kv_rows = torch.randn(n_tok, W, generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    pools = []
    for _ in range(L):
        pool = torch.empty(n_pages * page_bytes, dtype=torch.uint8, device="cuda")
        hip.launch_kv_append_paged(kv_rows, slots_all, pool, n_tok, W, PT, n_pages)
        pools.append(pool)
    del kv_rows
    new_rows = [torch.randn(B, W, generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
                for _ in range(L)]
    qabs = [torch.randn(B, H, KVL, generator=g, device="cuda", dtype=torch.float32) for _ in range(L)]
    qrope = [torch.randn(B, H, ROPE, generator=g, device="cuda", dtype=torch.float32) for _ in range(L)]
    clat = torch.empty(B, H, KVL, dtype=torch.float32, device="cuda")
    n_scratch = hip.mla_attend_paged_scratch_floats(B, H, ctx)
    partial = torch.empty(max(n_scratch, 1), dtype=torch.float32, device="cuda")
    sm_scale = float(W) ** -0.5
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    sh = stream.cuda_stream

    def attend(layer, lens, max_rows, st):
        hip.launch_mla_attend_paged(qabs[layer], qrope[layer], pools[layer], tables, lens, None, None, B, H,
                                    max_rows, blocks, KVL, ROPE, PT, n_pages, sm_scale, a.precise, clat,
                                    partial, None, st)

    def step(events):
        for layer in range(L):
            hip.launch_kv_append_paged(new_rows[layer], new_slots, pools[layer], B, W, PT, n_pages, None, sh)
            bracket(torch, stream, events, "attend", lambda: attend(layer, seq_lens, ctx, sh))

    ms, per = timed(torch, stream, a.steps, a.warmup, step)
    table_entries = int((-(-seq_lens_np // PT)).sum())
    attend_bytes = n_att * REC + table_entries * 4 + B * H * (W + KVL) * 4   # records, table, q in, clat out
    append_bytes = B * (ROW_IN + 4 + REC)
    flops = 2.0 * n_att * H * (W + KVL)
    res = {"metric": "kv_append_attend_GBps", "value": round(L * (attend_bytes + append_bytes) / (ms * 1e-3) / 1e9, 1),
           "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms, 4),
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16 x f32-accumulate",
           "data": "synthetic",
           "config": {"workload": "batched decode (benchmark configuration 3 shape) with the cache consumer "
                                  "fused: append 1 token/seq/layer, then MLA latent attention over every "
                                  "sequence's full context straight from the fp8 pages",
                      "layers": L, "batch": B, "ctx": ctx, "heads": H, "page_tokens": PT, "width": W,
                      "precise": a.precise, "contexts": "uniform in [1024, ctx]" if a.ragged else "all at ctx",
                      "tokens_per_layer": n_att},
           "decode_step_kv_ms": round(ms, 4),
           "tokens_per_s": round(L * n_att / (ms * 1e-3), 1),
           "roofline": {"bound": "hbm", "kernel": "mla_attend_paged_kernel",
                        "achieved": round(attend_bytes / (per["attend"] * 1e-3) / 1e9, 1),
                        "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                        "frac": round(attend_bytes / (per["attend"] * 1e-3) / HBM_PEAK, 4),
                        "avg_launch_ms": round(per["attend"], 5), "bytes_per_launch": attend_bytes,
                        "traffic": measured_traffic(f"attend:b{B}:ctx{ctx}:h{H}:{'ragged' if a.ragged else 'uniform'}"),
                        "tflops": round(flops / (per["attend"] * 1e-3) / 1e12, 1)}}
    if not a.no_cpu_baseline:
        from oracle.kvoracle import oracle as get_oracle

        ora = get_oracle()
        cores, usable, nproc = host_threads()
        # bounded sample: the first `cores` sequences cut to 2048 tokens, all heads, layer 0
        ns, cut = min(B, cores), min(ctx, 2048)
        lens_cut = np.zeros(B, np.int32)
        lens_cut[:ns] = cut
        pool_h = pools[0].cpu().numpy()
        qa_h, qr_h = qabs[0].cpu().numpy(), qrope[0].cpu().numpy()
        t0 = time.perf_counter()
        want = ora.mla_attend_paged(qa_h[:ns], qr_h[:ns], pool_h, tables_np[:ns], lens_cut[:ns], None, None,
                                    KVL, ROPE, PT, sm_scale, n_threads=cores)
        spent = time.perf_counter() - t0
        attend(0, torch.from_numpy(lens_cut).cuda(), ctx, None)
        torch.cuda.synchronize()
        got = clat.cpu().numpy()[:ns]
        err, mx = float(np.abs(got - want).max()), float(np.abs(want).max())
        bar = {2: 1e-4, 1: 2e-3, 0: 3e-2, 3: 3e-2, 4: 1e-3}[a.precise] * mx
        if not err <= bar:
            raise SystemExit(f"bench: GPU attention differs from the CPU oracle: err={err:.3e} max={mx:.3e}")
        sample_bytes = ns * cut * REC + ns * H * (W + KVL) * 4
        res["cpu_baseline"] = {"value": round(sample_bytes / spent / 1e9, 4), "unit": "GB/s", "cores": cores,
                               "nproc": nproc, "usable": usable, "kind": "port",
                               "sample": f"attention of {ns} sequences x {cut} tokens x {H} heads (layer 0, same "
                                         f"pool) on {cores} host threads; GPU output within {err / mx:.1e} of it",
                               "tokens_per_s": round(ns * cut / spent, 1)}
    return res


def cpu_baseline(pool0, tables_np, seq_lens_np, out, budget_s, hip, tables, seq_lens, cu, B, blocks,
                 n_pages, regather=None):
    """The CPU oracle's gather over layer 0 of the same pool, on the host cores, repeated until
    about `budget_s` seconds have been spent; its output is also compared with the GPU's."""
    import torch

    from oracle.kvoracle import oracle as get_oracle

    ora = get_oracle()
    cores, usable, nproc = host_threads()
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
    # the same oracle on ONE host thread, over the first sequence only (a bounded sample)
    one_len = seq_lens_np[:1].copy()
    one_out = np.empty((int(one_len[0]), W), np.uint16)
    t0 = time.perf_counter()
    ora.kv_gather_paged(pool_host, tables_np[:1], one_len, W, PT, n_threads=1, out=one_out)
    one_s = time.perf_counter() - t0
    one_bytes = int(one_len[0]) * (REC + ROW_IN)
    # full-size parity of one layer: GPU gather of the same pool vs the oracle's bytes (through
    # the entry point that was timed, when the caller hands it over)
    out.fill_(0)
    if regather is not None:
        regather()
    else:
        hip.launch_kv_gather_paged(pool0, tables, seq_lens, cu, out, B, blocks, W, PT, n_pages)
    torch.cuda.synchronize()
    same = bool(np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16).reshape(-1, W)[:n_tok],
                               out_host))
    if not same:
        raise SystemExit("bench: GPU gather differs from the CPU oracle at full size")
    return {"value": round(bytes_layer / per_layer_s / 1e9, 3), "unit": "GB/s", "cores": cores, "nproc": nproc,
            "usable": usable, "kind": "port",
            "sample": f"one layer's gather+dequantize ({n_tok} tokens, same pool and tables) x{reps}, "
                      f"{cores} threads; GPU output equal",
            "tokens_per_s": round(n_tok / per_layer_s, 1),
            "one_thread": {"value": round(one_bytes / one_s / 1e9, 3), "unit": "GB/s",
                           "sample": f"the layer's first sequence ({int(one_len[0])} tokens), once"}}


if __name__ == "__main__":
    main()
