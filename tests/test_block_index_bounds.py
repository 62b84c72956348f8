"""Host-side restatement of the index arithmetic of the block scorer's head-split kernel
(rivoli_amd/csrc/block_index.hip: index_score_blocks_128_split_kernel + walk_pairs): which
floats of q a wave requests, for head counts that leave some of the eight waves without a head.
Every request must stay inside q[s][heads][128]; a wave without heads requests nothing."""
import pytest

WAVES, HD, CHUNK = 8, 128, 32


def wave_requests(s, heads, wave, t, guard=True):
    """(first, last) float offsets of every chunk the wave requests for query t."""
    per = -(-heads // WAVES)
    h0 = min(wave * per, heads)
    h1 = min(h0 + per, heads)
    g0, g1 = t * heads + h0, t * heads + h1
    if guard and g0 >= g1:
        return []
    out = []
    qp = g0 * HD
    out.append((qp, qp + CHUNK - 1))                      # the first chunk, before the loop
    for g in range(g0, g1):
        for off in (32, 64, 96):
            out.append((qp + off, qp + off + CHUNK - 1))
        nxt = qp + HD if g + 1 < g1 else qp               # the next pair's first chunk, or its own again
        out.append((nxt, nxt + CHUNK - 1))
        qp += HD
    return out


@pytest.mark.parametrize("heads", [1, 2, 5, 7, 8, 9, 11, 17, 20, 63, 64, 65, 128])
@pytest.mark.parametrize("s", [1, 2, 65])
def test_every_request_stays_inside_q(s, heads):
    size = s * heads * HD
    covered = set()
    for t in range(s):
        for wave in range(WAVES):
            for first, last in wave_requests(s, heads, wave, t):
                assert 0 <= first and last < size, (s, heads, wave, t, first, last, size)
                covered.update(range(first // CHUNK, last // CHUNK + 1))
    assert covered == set(range(size // CHUNK))           # and every chunk of q is read by someone


def test_a_wave_without_heads_would_read_past_the_end_without_the_guard():
    s, heads = 2, 5                                       # per = 1: waves 5..7 have no head
    size = s * heads * HD
    assert wave_requests(s, heads, 7, s - 1) == []
    first, last = wave_requests(s, heads, 7, s - 1, guard=False)[0]
    assert last >= size                                   # what the guard is there for
