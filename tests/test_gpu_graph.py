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
