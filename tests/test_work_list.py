"""How a step's prompt rows are cut for the attention kernel (host side, no GPU): the work list."""
import random
import types

import pytest

from bare_cuda_4gib_amd.csrc import ops


def batch_of(requests):
    """requests: [(cached tokens, new tokens)]."""
    start = [0]
    for _, new in requests:
        start.append(start[-1] + new)
    return types.SimpleNamespace(n_seqs=len(requests), n_tokens=start[-1], seq_start=start, seq_ctx=[c for c, _ in requests])


def pieces_of(batch, piece, skip=()):
    starts = [0]
    for s in range(batch.n_seqs):
        new = batch.seq_start[s + 1] - batch.seq_start[s]
        starts.append(starts[-1] + (0 if s in skip else -(-new // piece)))
    return starts


@pytest.mark.parametrize("seed", range(6))
def test_every_part_of_every_piece_once_and_the_longest_first(seed):
    rng = random.Random(seed)
    piece = rng.choice([4, 16, 32])
    window = rng.choice([0, 0, 100])
    requests = [(rng.randrange(0, 3000), rng.randrange(1, 700)) for _ in range(rng.randrange(1, 9))]
    batch = batch_of(requests)
    skip = {s for s in range(batch.n_seqs) if rng.random() < 0.2}                 # requests another launch serves
    starts = pieces_of(batch, piece, skip)
    items, row_parts, most = ops.prompt_work_list(batch, starts, piece, rng.choice([1, 4, 8]), window)
    seen = {}
    for it in items:
        index, part, parts = it & 0xfffff, (it >> 20) & 15, it >> 24
        assert 0 <= part < parts <= ops.ATTENTION_MAX_PROMPT_SPLITS and 0 <= index < starts[-1]
        assert (index, part) not in seen
        seen[(index, part)] = parts
    for index in range(starts[-1]):                                                # every part of every piece
        parts = seen[(index, 0)]
        assert all(seen[(index, z)] == parts for z in range(parts))
    assert len(seen) == sum(seen[(i, 0)] for i in range(starts[-1]))
    assert most == max([1] + list(seen.values())) and len(row_parts) == batch.n_tokens
    # rows: the parts of their piece; rows of requests without pieces: one
    for s in range(batch.n_seqs):
        first, new = batch.seq_start[s], batch.seq_start[s + 1] - batch.seq_start[s]
        for r in range(new):
            want = 1 if s in skip else seen[(starts[s] + r // piece, 0)]
            assert row_parts[first + r] == want
    # the longest walks first: a part's length never grows along the list
    def length(it):
        index, parts = it & 0xfffff, it >> 24
        s = max(q for q in range(batch.n_seqs) if starts[q] <= index and starts[q + 1] > index)
        j = index - starts[s]
        ctx0, new = batch.seq_ctx[s], batch.seq_start[s + 1] - batch.seq_start[s]
        lo = max(0, ctx0 + j * piece - window + 1) if window else 0
        tiles = (ctx0 + min(new, (j + 1) * piece) - 1) // 32 - lo // 32 + 1
        return -(-tiles // parts)
    lengths = [length(it) for it in items]
    assert lengths == sorted(lengths, reverse=True)


def test_a_long_prompt_alone_is_cut_by_an_even_share():
    """2,048 tokens, 32-token pieces, four head blocks: 8,320 key tiles over 512 places are 16.25 each; parts hold
    at most half more (25), so the last piece's 64 tiles go in three parts and the first 25 pieces in one."""
    batch = batch_of([(0, 2048)])
    items, row_parts, most = ops.prompt_work_list(batch, [0, 64], 32, 4, 0)
    assert most == 3 and row_parts[0] == 1 and row_parts[25 * 32 - 1] == 1 and row_parts[25 * 32] == 2 and row_parts[-1] == 3
    assert len(items) == 25 + 25 * 2 + 14 * 3                          # pieces 0-24, 25-49, 50-63
    # a short prompt is cut down to the least walk, a very long one not at all
    assert ops.prompt_work_list(batch_of([(0, 512)]), [0, 16], 32, 4, 0)[2] == 4
    assert ops.prompt_work_list(batch_of([(0, 8192)]), [0, 256], 32, 4, 0)[2] == 1
