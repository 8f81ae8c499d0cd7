"""The packed launch's tile deal, restated on the host.

The matrix-core kernel deals the tiles of a packed batch to its persistent workgroups by itself (the set-up
of `srt_seq` / `seq_pre`, `dealt_tile`, `take` in turbodeberta_amd/csrc/attn_mfma.hip): the tiles are listed by
decreasing length of their sequence and dealt to the workgroups back and forth, round after round.  This file
restates that arithmetic step by step and checks, for grid sizes the GPU tests cannot all reach, that every
tile of the batch is dealt to exactly one workgroup -- the packed encoder allocates its output
uninitialised, so a tile nobody took would be garbage.  The device code itself is exercised at grids of 8,
24, 40, 248 and 256 workgroups by tests/test_ops_gpu.py::test_packed_tile_deal_at_other_grid_sizes."""
import numpy as np
import pytest

BM, BN = 128, 64


def tiles_of(n):
    return (n + BM - 1) // BM


def cost_of(n):
    """What a tile of a sequence of n tokens costs, in eighths of a key step (about 3 steps beside its own)."""
    return 8 * ((n + BN - 1) // BN) + 24


def deal_of_workgroup(seq_n, heads, grid, block):
    """Tiles (head, sequence, first row) that the workgroup with block id `block` of `grid` processes, in order."""
    assert len(seq_n) == 64 and grid % 8 == 0
    # set-up: rank of every sequence by decreasing length (ties: lower index first), then the sequence and the
    # tile count (all heads) at each rank, and the inclusive prefix sum of the counts
    rank = [sum(1 for b2 in range(64) if seq_n[b2] > seq_n[b] or (seq_n[b2] == seq_n[b] and b2 < b))
            for b in range(64)]
    srt_seq = [0] * 64
    for b in range(64):
        srt_seq[rank[b]] = b
    seq_pre = np.cumsum([tiles_of(seq_n[srt_seq[r]]) * heads for r in range(64)]).tolist()

    g = (block & 7) * (grid >> 3) + (block >> 3)             # neighbours in the deal share an XCD
    mine = []
    j = 0
    while True:                                              # dealt_tile(j), j = 0, 1, ... until there is none
        k = j * grid + (grid - 1 - g if j & 1 else g)
        if k >= seq_pre[63]:
            break
        r = next(i for i in range(64) if seq_pre[i] > k)
        b = srt_seq[r]
        per_head = tiles_of(seq_n[b])
        assert per_head > 0
        within = k - (seq_pre[r] - per_head * heads)
        head = within // per_head
        assert 0 <= within and head < heads
        mine.append((head, b, (within - head * per_head) * BM))
        j += 1
    return mine


def all_tiles(seq_n, heads):
    return sorted((h, b, BM * i) for h in range(heads) for b, n in enumerate(seq_n) for i in range(tiles_of(n)))


@pytest.mark.parametrize("grid", [8, 24, 40, 64, 248, 256, 304])
@pytest.mark.parametrize("heads", [1, 12, 16])
def test_every_tile_is_dealt_exactly_once(grid, heads):
    rs = np.random.RandomState(grid * 31 + heads)
    for trial in range(6):
        count = [64, 64, 17, 1, 40, 64][trial]
        hi = [513, 200, 4097, 130, 65, 2][trial]
        lengths = rs.randint(0 if trial else 1, hi, size=count).tolist()
        if trial == 1:
            for i in (0, 5, 31, 63):
                lengths[i] = 0
        seq_n = lengths + [0] * (64 - count)
        dealt = [t for g in range(grid) for t in deal_of_workgroup(seq_n, heads, grid, g)]
        assert sorted(dealt) == all_tiles(seq_n, heads), (grid, heads, trial)


def test_empty_batch_has_no_tiles():
    assert all(deal_of_workgroup([0] * 64, 12, 256, g) == [] for g in range(0, 256, 37))


def test_balance_of_the_benchmark_batch():
    """64 sequences of 16..512 tokens, 12 heads, 256 workgroups: the heaviest workgroup carries at most 1.08x
    the mean cost, whatever the draw of the lengths."""
    for seed in range(8):
        lengths = np.random.RandomState(seed).randint(16, 513, size=64).tolist()
        cost = [sum(cost_of(lengths[b]) for _, b, _ in deal_of_workgroup(lengths, 12, 256, g)) for g in range(256)]
        assert max(cost) <= 1.08 * (sum(cost) / 256), (seed, max(cost) / (sum(cost) / 256))


def test_query_tiles_of_a_sequence_and_head_share_an_xcd():
    """Sequences of one length: the 4 query tiles of a (sequence, head) that are dealt in one round go to block ids that
    agree modulo 8, the XCD a block runs on."""
    seq_n = [512] * 64
    owner = {}
    for block in range(256):
        for j, t in enumerate(deal_of_workgroup(seq_n, 12, 256, block)):
            owner[t] = block & 7
    for h in range(12):
        for b in range(64):
            assert len({owner[(h, b, BM * i)] for i in range(4)}) == 1, (h, b)
