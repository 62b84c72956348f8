"""The decode step's cache work as one launch (rivoli_kv_append_gather_paged) against the two
calls it replaces and against the oracle: pool bytes and gathered rows equal, bit for bit,
through both launch forms (the grid over the block tables, the flat grid sized by the batch's
token count)."""
import numpy as np
import pytest

from rivoli_amd import hip
from tests.gpu_util import back, dev, dzeros
from tests.test_gpu_gather import build_pool
from tests.util import make_rows_bf16, slots_for

pytestmark = pytest.mark.gpu
W, PT = 576, 64


def step_both_ways(oracle, pool_h, tables, lens_before, new_rows, new_slots, width=W, pt=PT, wide=False,
                   total=None):
    """Appends new_rows at new_slots and gathers lens_before + (slot >= 0): the oracle, the two
    separate device calls, and the fused call. Returns (want_pool, want_out, sep, fused) where
    sep / fused = (pool, out, bad_slots, bad_pages)."""
    n_seqs = len(lens_before)
    n_pages = pool_h.size // (pt * (width + 4))
    in_pool = (new_slots >= 0) & (new_slots < n_pages * pt)
    lens = (np.asarray(lens_before) + (new_slots >= 0)).astype(np.int32)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    want_pool = pool_h.copy()
    oracle.kv_append_paged(new_rows, new_slots, want_pool, width, pt, n_pages)
    want_out = oracle.kv_gather_paged(want_pool, tables, lens, width, pt)
    if wide:   # unused table columns: the batch fills little of what the tables could hold
        t = np.full((n_seqs, 4 * tables.shape[1] + 1), -1, np.int32)
        t[:, : tables.shape[1]] = tables
        tables = t
    tot = int(cu[-1]) if total is None else total
    results = []
    for fused in (False, True):
        pool, out = dev(pool_h), dzeros(max(int(cu[-1]), 1) * width * 2, 0x5A)
        bad_s, bad_p = dzeros(4), dzeros(4)
        args = (pool, dev(tables), dev(lens), dev(cu), out, n_seqs, tables.shape[1], tot, width, pt, n_pages)
        if fused:
            hip.launch_kv_append_gather_paged(dev(new_rows), dev(new_slots), *args, bad_s, bad_p)
        else:
            hip.launch_kv_append_paged(dev(new_rows), dev(new_slots), pool, n_seqs, width, pt, n_pages, bad_s)
            if tot < 0:
                hip.launch_kv_gather_paged(*args[:7], width, pt, n_pages, bad_p)
            else:
                hip.launch_kv_gather_paged_packed(*args, bad_p)
        results.append((back(pool).copy(), back(out, np.uint16).reshape(-1, width).copy(),
                        int(back(bad_s, np.uint32)[0]), int(back(bad_p, np.uint32)[0])))
    assert int((~in_pool & (new_slots >= 0)).sum()) == results[0][2]
    return want_pool, want_out, results[0], results[1]


def check(want_pool, want_out, sep, fused):
    assert np.array_equal(sep[0], want_pool) and np.array_equal(sep[1][: want_out.shape[0]], want_out)
    assert np.array_equal(fused[0], sep[0]), "pool bytes differ from append-then-gather"
    assert np.array_equal(fused[1], sep[1]), "gathered rows differ from append-then-gather"
    assert fused[2:] == sep[2:]


@pytest.mark.parametrize("total", ["exact", "unknown"])
@pytest.mark.parametrize("wide", [False, True])
def test_config1_step(oracle, wide, total):
    """benchmark configuration 1: 4095 cached tokens on 64 shuffled pages, append the 4096th,
    gather all 4096."""
    pool, tables = build_pool(oracle, [4095], 64, seed=0x5EED0001 % 10007)
    new = make_rows_bf16(1, W, seed=4095)
    slot = slots_for(tables[0], np.array([4095]), PT).astype(np.int32)
    check(*step_both_ways(oracle, pool, tables, [4095], new, slot, wide=wide,
                          total=-1 if total == "unknown" else None))


@pytest.mark.parametrize("wide", [False, True])
def test_ragged_batch_page_boundaries_padding_and_outliers(oracle, wide):
    """New tokens that open a page, close one, sit mid-page; a sequence of one token (the new
    one); sequences without a new token (slot -1); a slot outside the pool; an outlier row and
    an all-zero row among the new ones."""
    before = [0, 63, 64, 65, 700, 1023, 2049, 5, 300, 127]
    n_pages = 400
    pool, tables = build_pool(oracle, [n + 1 for n in before], n_pages, seed=77, outlier_frac=0.01,
                              outlier_mul=200.0)
    # build_pool wrote one token too many per sequence: zero the record of the last one, so that
    # the step below really brings it (codes and scale)
    rec = W + 4
    new = make_rows_bf16(len(before), W, seed=5)
    new[4, :] = 0                                          # all zero: scale 1.0
    b = new[5].astype(np.uint32) << 16
    new[5] = ((b.view(np.float32) * np.float32(200.0)).view(np.uint32) >> 16).astype(np.uint16)
    slots = np.array([slots_for(tables[s], np.array([before[s]]), PT)[0] for s in range(len(before))], np.int32)
    page_bytes = oracle.kv_page_bytes(PT, W)
    for s, slot in enumerate(slots):
        page, off = divmod(int(slot), PT)
        pool[page * page_bytes + off * W: page * page_bytes + (off + 1) * W] = 0xCC
        pool[page * page_bytes + PT * W + 4 * off: page * page_bytes + PT * W + 4 * off + 4] = 0xCC
    slots[7] = -1                                          # no new token: 5 tokens gathered
    slots[8] = n_pages * PT + 3                            # outside the pool: counted, gathered whole
    want_pool, want_out, sep, fused = step_both_ways(oracle, pool, tables, before, new, slots, wide=wide)
    check(want_pool, want_out, sep, fused)
    assert sep[2] == 1 and sep[3] == 0


def test_other_widths_and_page_sizes(oracle):
    for width, pt, before in ((128, 16, [15, 16, 40]), (1024, 64, [100, 3]), (64, 4, [7, 8, 1])):
        n_pages = 64
        pool, tables = build_pool(oracle, [n + 1 for n in before], n_pages, seed=width, width=width, pt=pt)
        new = make_rows_bf16(len(before), width, seed=9)
        slots = np.array([slots_for(tables[s], np.array([before[s]]), pt)[0] for s in range(len(before))], np.int32)
        check(*step_both_ways(oracle, pool, tables, before, new, slots, width=width, pt=pt))


def test_guards():
    b = dzeros(1 << 16)
    def call(**kw):
        a = dict(new_rows=b, slot_mapping=b, pool=b, block_table=b, seq_lens=b, cu_seqlens=b, out=b, n_seqs=2,
                 max_blocks_per_seq=4, total_tokens=100, width=W, page_tokens=PT, n_pages=8)
        a.update(kw)
        hip.launch_kv_append_gather_paged(**a)
    call()
    for kw, code in ((dict(new_rows=None), 1001), (dict(slot_mapping=None), 1001), (dict(pool=None), 1001),
                     (dict(n_seqs=0), 1001), (dict(width=2048), 1002), (dict(width=100), 1004),
                     (dict(new_rows=b.data_ptr() + 2), 1004)):
        with pytest.raises(hip.LaunchError) as e:
            call(**kw)
        assert e.value.code == code, kw


def test_the_one_launch_step_replays_from_a_graph(oracle):
    """A serving loop's use: the call captured once, replayed per token on inputs the host
    refills in place; every replay equals append-then-gather launched eagerly."""
    from tests.gpu_util import torch_cuda

    torch = torch_cuda()
    lens0 = [700, 64, 1500, 129]
    n_seqs = len(lens0)
    n_pages = n_seqs * -(-(max(lens0) + 4) // PT) + 3
    pool_h, tables = build_pool(oracle, lens0, n_pages, seed=404)
    blocks = tables.shape[1]
    max_tok = sum(lens0) + 4 * n_seqs
    pool, table_d = dev(pool_h), dev(tables)
    new_rows = torch.zeros(n_seqs * W * 2, dtype=torch.uint8, device="cuda")
    new_slots = torch.zeros(n_seqs * 4, dtype=torch.uint8, device="cuda")
    seq_lens = torch.zeros(n_seqs * 4, dtype=torch.uint8, device="cuda")
    cu = torch.zeros((n_seqs + 1) * 4, dtype=torch.uint8, device="cuda")
    out = torch.zeros(max_tok * W * 2, dtype=torch.uint8, device="cuda")

    def load_inputs(t):
        now = np.array([n + t + 1 for n in lens0], np.int32)
        rows = make_rows_bf16(n_seqs, W, seed=900 + t)
        slots = np.array([slots_for(tables[s], np.array([lens0[s] + t]), PT)[0] for s in range(n_seqs)], np.int32)
        for buf, a in ((new_rows, rows), (new_slots, slots), (seq_lens, now),
                       (cu, np.concatenate([[0], np.cumsum(now)]).astype(np.int32))):
            buf.copy_(dev(a))
        return int(now.sum())

    # the captured call is told the largest token count the graph will see: the flat grid is sized
    # by it, and units past the batch's real end find no sequence and leave
    def fused(stream):
        hip.launch_kv_append_gather_paged(new_rows, new_slots, pool, table_d, seq_lens, cu, out, n_seqs, blocks,
                                          max_tok, W, PT, n_pages, None, None, stream)

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        load_inputs(0)
        pool_start = pool.clone()
        fused(stream.cuda_stream)                                  # warm-up outside the capture
        stream.synchronize()
        pool.copy_(pool_start)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            fused(torch.cuda.current_stream().cuda_stream)
        for t in range(3):
            n_now = load_inputs(t)
            pool_before = pool.clone()
            out.fill_(0xEE)
            hip.launch_kv_append_paged(new_rows, new_slots, pool, n_seqs, W, PT, n_pages, None, stream.cuda_stream)
            hip.launch_kv_gather_paged_packed(pool, table_d, seq_lens, cu, out, n_seqs, blocks, max_tok, W, PT,
                                              n_pages, None, stream.cuda_stream)
            torch.cuda.synchronize()
            want_pool, want_out = pool.clone(), out.clone()
            pool.copy_(pool_before)
            out.fill_(0xEE)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(pool, want_pool), t
            assert torch.equal(out[: n_now * W * 2], want_out[: n_now * W * 2]), t
