"""The select-and-gather call that allocates nothing (its workspace is an array inside the
library's device image) against the form that takes a caller's workspace: bit for bit, on
calls that follow each other with different shapes."""
import numpy as np
import pytest

from rivoli_amd import hip
from tests.gpu_util import back, dev, dzeros
from tests.test_gpu_dsa_fused import PT, W, check_against_oracle, paged_cache, run_fused

pytestmark = pytest.mark.gpu


def run_noalloc(scores, nts, k, tables, n_pages, pool_d):
    n_q, stride = scores.shape
    rows = dzeros(n_q * k * 4, 0xFF)
    out = dzeros(n_q * k * W * 2, 0xEE)
    bad = dzeros(4)
    hip.launch_dsa_select_gather_paged_noalloc(
        dev(scores), n_q, stride, None if nts is None else dev(np.asarray(nts, np.int32)), stride, k, rows,
        pool_d, dev(tables), out, tables.shape[1], W, PT, n_pages, bad)
    return (back(rows, np.uint32).reshape(n_q, k), back(out, np.uint16).reshape(n_q, k, W),
            int(back(bad, np.uint32)[0]))


def test_noalloc_equals_the_workspace_form_on_successive_calls(oracle):
    rng = np.random.default_rng(2024)
    # a larger call, a smaller one of another shape (its histograms sit where the first left
    # lists), a ragged one, one that needs no workspace, and the first shape again
    cases = [(4, 50000, 1024, None), (2, 20000, 300, None), (3, 40000, 512, [40000, 0, 16500]),
             (2, 3000, 256, None), (4, 50000, 1024, None)]
    for n_q, nt, k, nts in cases:
        tables, n_pages, pool_h = paged_cache(oracle, rng, n_q, nt)
        s = rng.standard_normal((n_q, nt), dtype=np.float32)
        s[0, ::5] = np.float32(0.5)                          # ties across the pivot
        pool_d = dev(pool_h)
        want_rows, want_out, want_bad = run_fused(s, nts, k, tables, n_pages, pool_d, split=True)
        got_rows, got_out, got_bad = run_noalloc(s, nts, k, tables, n_pages, pool_d)
        assert np.array_equal(got_rows, want_rows), (n_q, nt, k)
        assert np.array_equal(got_out, want_out), (n_q, nt, k)
        assert got_bad == want_bad == 0
        check_against_oracle(oracle, s, nts, k, tables, pool_h, got_rows, got_out)


def test_noalloc_size_limit_and_guards():
    b = dzeros(1 << 16)
    def call(**kw):
        a = dict(scores=b, n_queries=1, stride=20000, nts=None, nt=20000, k=8, rows=b, pool=b, block_table=b,
                 out=b, max_blocks_per_seq=400, width=W, page_tokens=PT, n_pages=10)
        a.update(kw)
        hip.launch_dsa_select_gather_paged_noalloc(**a)
    for kw, code in ((dict(n_queries=17, nt=65536, stride=65536), 1002),      # one query more than fits
                     (dict(n_queries=1, nt=1 << 22, stride=1 << 22), 1002),
                     (dict(pool=None), 1001), (dict(k=0), 1001), (dict(stride=100), 1002), (dict(width=100), 1004)):
        with pytest.raises(hip.LaunchError) as e:
            call(**kw)
        assert e.value.code == code, kw


def test_noalloc_call_replays_from_a_graph(oracle):
    """The callers it is for: the call captured into a HIP graph (the first call on the device,
    which looks the array's address up, made before the capture) and replayed on fresh scores,
    with eager work between the replays; every replay equals the workspace form."""
    from tests.gpu_util import torch_cuda

    torch = torch_cuda()
    rng = np.random.default_rng(77)
    n_q, nt, k = 3, 30000, 400
    tables, n_pages, pool_h = paged_cache(oracle, rng, n_q, nt)
    pool_d, tables_d = dev(pool_h), dev(tables)
    scores = torch.zeros(n_q * nt * 4, dtype=torch.uint8, device="cuda")
    rows, out = dzeros(n_q * k * 4, 0xFF), dzeros(n_q * k * W * 2, 0xEE)

    def call(stream):
        hip.launch_dsa_select_gather_paged_noalloc(scores, n_q, nt, None, nt, k, rows, pool_d, tables_d, out,
                                                   tables.shape[1], W, PT, n_pages, None, stream)

    call(hip.NULL_STREAM)                                      # the address lookup happens here
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            call(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for t in range(3):                                         # replays on the null stream, like the eager work
        s = rng.standard_normal((n_q, nt), dtype=np.float32)
        s[1, ::7] = np.float32(0.25)
        scores.copy_(dev(s))
        rows.fill_(0xFF)
        out.fill_(0xEE)
        graph.replay()
        torch.cuda.synchronize()
        got_rows, got_out = back(rows, np.uint32).reshape(n_q, k), back(out, np.uint16).reshape(n_q, k, W)
        want_rows, want_out, _ = run_fused(s, None, k, tables, n_pages, pool_d, split=True)   # eager work between
        assert np.array_equal(got_rows, want_rows), t
        assert np.array_equal(got_out, want_out), t
