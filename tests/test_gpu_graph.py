"""The launchers only launch (no allocation, no copy, no synchronisation), so a decode step made
of them can be captured into a HIP graph and replayed. The step here is the whole path — append
one token per sequence, gather the contexts, select rows, gather them, attend over them — and
every replay, with the program's own eager work and synchronisations between replays, must
reproduce the eager result of the same inputs bit for bit."""
import numpy as np
import pytest

from rivoli_amd import hip
from tests.attend_cases import paged_case
from tests.gpu_util import dev, torch_cuda
from tests.util import make_rows_bf16, slots_for

pytestmark = pytest.mark.gpu
W, KVL, ROPE, PT, H, K = 576, 512, 64, 64, 64, 256


def test_decode_step_replays_from_a_graph(oracle):
    torch = torch_cuda()
    lens = [700, 1500, 900]
    c = paged_case(oracle, [n + 3 for n in lens], H=H, seed=91)     # room for three more tokens
    n_seqs, blocks, n_pages = len(lens), c["table"].shape[1], c["n_pages"]
    pool, table = dev(c["pool"]), dev(c["table"])
    qabs, qrope = dev(c["qabs"]), dev(c["qrope"])
    max_ctx = max(lens) + 3
    # the step's inputs live in fixed device buffers that the host refills between replays
    new_rows = torch.zeros(n_seqs * W * 2, dtype=torch.uint8, device="cuda")
    new_slots = torch.zeros(n_seqs * 4, dtype=torch.uint8, device="cuda")
    seq_lens = torch.zeros(n_seqs * 4, dtype=torch.uint8, device="cuda")
    cu = torch.zeros((n_seqs + 1) * 4, dtype=torch.uint8, device="cuda")
    scores = torch.zeros(n_seqs * max_ctx * 4, dtype=torch.uint8, device="cuda")
    gathered = torch.zeros(n_seqs * max_ctx * W * 2, dtype=torch.uint8, device="cuda")
    sel = torch.zeros(n_seqs * K * 4, dtype=torch.uint8, device="cuda")
    picked = torch.zeros(n_seqs * K * W * 2, dtype=torch.uint8, device="cuda")
    clat = torch.zeros(n_seqs * H * KVL * 4, dtype=torch.uint8, device="cuda")
    partial = torch.zeros(max(hip.mla_attend_paged_scratch_floats(n_seqs, H, K), 1) * 4, dtype=torch.uint8,
                          device="cuda")

    def step(stream):
        hip.launch_kv_append_paged(new_rows, new_slots, pool, n_seqs, W, PT, n_pages, None, stream)
        hip.launch_kv_gather_paged(pool, table, seq_lens, cu, gathered, n_seqs, blocks, W, PT, n_pages, None, stream)
        hip.launch_index_topk_batched(scores, n_seqs, max_ctx, seq_lens, max_ctx, K, sel, None, stream)
        hip.launch_kv_gather_rows_paged(pool, table, sel, None, picked, n_seqs, K, blocks, W, PT, n_pages, None, stream)
        hip.launch_mla_attend_paged(qabs, qrope, pool, table, seq_lens, sel, None, n_seqs, H, K, blocks, KVL, ROPE,
                                    PT, n_pages, c["scale"], 2, clat, partial, None, stream)

    def load_inputs(t):
        """Token t of the continuation: one new row per sequence at position lens[s] + t."""
        now = np.array([n + t + 1 for n in lens], np.int32)
        rows = make_rows_bf16(n_seqs, W, seed=500 + t)
        slots = np.array([slots_for(c["table"][s], np.array([lens[s] + t]), PT)[0] for s in range(n_seqs)], np.int32)
        sc = np.random.default_rng(600 + t).standard_normal((n_seqs, max_ctx)).astype(np.float32)
        for buf, a in ((new_rows, rows), (new_slots, slots), (seq_lens, now),
                       (cu, np.concatenate([[0], np.cumsum(now)]).astype(np.int32)), (scores, sc)):
            buf.copy_(dev(a))

    def outputs():
        torch.cuda.synchronize()
        return [b.clone() for b in (pool, gathered, sel, picked, clat)]

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        load_inputs(0)
        step(stream.cuda_stream)                                   # warm-up outside the capture
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            step(torch.cuda.current_stream().cuda_stream)
        for t in range(3):
            pool_before = pool.clone()
            load_inputs(t)
            for b in (gathered, sel, picked, clat):                # what a launch leaves unwritten stays 0xEE
                b.fill_(0xEE)
            step(stream.cuda_stream)                               # eager, for the expectation
            want = outputs()
            pool.copy_(pool_before)                                # undo the append, then replay
            for b in (gathered, sel, picked, clat):
                b.fill_(0xEE)
            graph.replay()
            got = outputs()
            for name, g, w in zip(("pool", "gathered", "selection", "selected rows", "attention"), got, want):
                assert torch.equal(g, w), (t, name)
    # and the eager results are the oracle's: the last step's selection against the CPU rule
    now = np.array([n + 3 for n in lens], np.int32)
    sc = np.random.default_rng(602).standard_normal((n_seqs, max_ctx)).astype(np.float32)
    assert np.array_equal(got[2].cpu().numpy().view(np.uint32).reshape(n_seqs, K),
                          oracle.topk_batched(sc, K, nts=now))


def test_second_format_decode_step_replays_from_a_graph(oracle):
    """The second cache format's decode step — quantize the new entry, write it into the ring,
    deposit into the compressor (and pool the block this position closes), spread the index
    queries and score the blocks, build the [ring | scored blocks] rectangle from those scores,
    attend with the list shared among workgroups — captured
    once at a position that closes a block and replayed on fresh inputs."""
    from oracle.kvoracle import CompGeom as OracleGeom
    from tests.v4_cases import bf16_round, compress_inputs

    torch = torch_cuda()
    win, ratio, d, rd, heads, cap, pos = 128, 4, 512, 64, 64, 64, 1023      # position 1023 closes block 255
    n_comp = (pos + 1) // ratio
    og, hg = OracleGeom.attention(ratio, d, rd), hip.CompGeom.build(ratio, d, rd, 1e-6)
    rng = np.random.default_rng(5)
    _, _, ape, norm, freqs = compress_inputs(og, 8, seed=3, positions=pos + 1)
    cache0 = bf16_round(rng.standard_normal((win + 512, d)).astype(np.float32))
    cache, state_kv = dev(cache0), dev(rng.standard_normal((og.coff * ratio, og.cd)).astype(np.float32))
    state_sc = dev(rng.standard_normal((og.coff * ratio, og.cd)).astype(np.float32))
    ape_d, norm_d, freqs_d, sink = dev(ape), dev(norm), dev(freqs), dev(rng.standard_normal(heads).astype(np.float32))
    # the step's inputs live in fixed device buffers that the host refills between replays
    entry = torch.zeros(d * 4, dtype=torch.uint8, device="cuda")
    ckv = torch.zeros(og.cd * 4, dtype=torch.uint8, device="cuda")
    csc = torch.zeros(og.cd * 4, dtype=torch.uint8, device="cuda")
    q = torch.zeros(heads * d * 4, dtype=torch.uint8, device="cuda")
    scores = torch.zeros(n_comp * 4, dtype=torch.uint8, device="cuda")
    # the block indexer that makes the scores: 64 index heads of 128, the blocks' spread rows
    iheads, ihd = 64, 128
    iq = torch.zeros(iheads * ihd * 4, dtype=torch.uint8, device="cuda")
    iw = torch.zeros(iheads * 4, dtype=torch.uint8, device="cuda")
    ikv_h = bf16_round(rng.standard_normal((n_comp, ihd)).astype(np.float32))
    ikv = dev(ikv_h)
    hip.launch_act_quant_f4_rotated(ikv, n_comp, ihd)
    cols = win + cap
    idx = torch.zeros(cols * 4, dtype=torch.uint8, device="cuda")
    o = torch.zeros(heads * d * 4, dtype=torch.uint8, device="cuda")
    part = torch.zeros(max(hip.gather_attn_scratch_floats(1, heads, d, cols), 4) * 4, dtype=torch.uint8, device="cuda")
    first, _ = hip.compress_dst(ratio, win, 1, pos)
    block_row = cache[first * d * 4:(first + 1) * d * 4]                 # the pooled block's home, by position
    fin = hip.CompFinish.of(norm_d, freqs_d, block_row)

    def step(stream):
        hip.launch_act_quant_f8_prefix(entry, entry, 1, d, d - rd, 64, stream)
        hip.launch_kv_ring_write(entry, cache, win, d, 1, pos, stream)
        hip.launch_kv_compress_deposit(ckv, csc, ape_d, state_kv, state_sc, hg, 1, pos % ratio, stream)
        hip.launch_kv_compress_decode(state_kv, state_sc, fin, hg, pos, stream)
        hip.launch_act_quant_f8_prefix(block_row, block_row, 1, d, d - rd, 64, stream)
        hip.launch_act_quant_f4_rotated(iq, iheads, ihd, stream)
        hip.launch_index_score_blocks(iq, ikv, iw, scores, 1, n_comp, iheads, ihd, stream)
        hip.launch_sel_gather_scored(scores, n_comp, win, ratio, cap, 1, pos, idx, stream)
        hip.launch_gather_attn_shared_kv(q, cache, sink, idx, 1, heads, d, cols, d ** -0.5, o, stream, partial=part)

    def load_inputs(t):
        r = np.random.default_rng(900 + t)
        for buf, a in ((entry, bf16_round(r.standard_normal(d).astype(np.float32))),
                       (ckv, r.standard_normal(og.cd).astype(np.float32)),
                       (csc, r.standard_normal(og.cd).astype(np.float32)),
                       (q, bf16_round(r.standard_normal((heads, d)).astype(np.float32))),
                       (iq, bf16_round(r.standard_normal((iheads, ihd)).astype(np.float32))),
                       (iw, bf16_round((r.standard_normal(iheads) * 0.1).astype(np.float32)))):
            buf.copy_(dev(a))

    state = (cache, state_kv, state_sc)

    def outputs():
        torch.cuda.synchronize()
        return [b.clone() for b in (cache, state_kv, state_sc, idx, o)]

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        load_inputs(0)
        saved = [b.clone() for b in state]
        step(stream.cuda_stream)                                   # warm-up outside the capture
        stream.synchronize()
        for b, s in zip(state, saved):
            b.copy_(s)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            step(torch.cuda.current_stream().cuda_stream)
        for b, s in zip(state, saved):                             # the capture ran nothing; start clean anyway
            b.copy_(s)
        for t in range(3):
            before = [b.clone() for b in state]
            load_inputs(t)
            entry_in, iq_in = entry.clone(), iq.clone()
            for b in (idx, o):
                b.fill_(0xEE)
            step(stream.cuda_stream)                               # eager, for the expectation
            want = outputs()
            for b, s in zip(state, before):                        # undo the step, then replay it
                b.copy_(s)
            entry.copy_(entry_in)
            iq.copy_(iq_in)
            for b in (idx, o):
                b.fill_(0xEE)
            graph.replay()
            got = outputs()
            for name, g, w in zip(("cache", "compressor kv state", "compressor score state", "rectangle", "attention"),
                                  got, want):
                assert torch.equal(g, w), (t, name)
    # and the eager result is the oracle's: the last rectangle against the CPU chain (spread the
    # index queries, score the blocks, select)
    r = np.random.default_rng(902)                                  # load_inputs(2): iq and iw are its last two draws
    for n in (d, og.cd, og.cd, heads * d):
        r.standard_normal(n)
    iq_h = bf16_round(r.standard_normal((iheads, ihd)).astype(np.float32))
    iw_h = bf16_round((r.standard_normal(iheads) * 0.1).astype(np.float32))
    code_s, want_scores = oracle.index_score_blocks(oracle.act_quant_f4_rotated(iq_h)[1][None],
                                                    oracle.act_quant_f4_rotated(ikv_h)[1], iw_h[None, :])
    assert code_s == 0 and np.array_equal(scores.cpu().numpy().view(np.uint32), want_scores.view(np.uint32).ravel())
    code, want_rect = oracle.sel_gather_scored(want_scores, win, ratio, cap, 1, pos)
    assert code == 0 and np.array_equal(got[3].cpu().numpy().view(np.int32).reshape(1, cols), want_rect)
