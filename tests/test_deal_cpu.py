"""The packed launch's tile deal, restated on the host.

The matrix-core kernel deals the tiles of a packed batch to its persistent workgroups by itself
(`first_balanced`, `take`, `settle` in turbodeberta_amd/csrc/attn_mfma.hip): teams of workgroups own
contiguous cost intervals of the tile list, and inside a team every tile goes to the member with the least
cost so far.  This file restates that arithmetic step by step and checks, for grid sizes the GPU tests
cannot all reach, that every tile of the batch is dealt to exactly one workgroup -- the packed encoder
allocates its output uninitialised, so a tile nobody took would be garbage.  The device code itself is
exercised at grids of 8, 24, 40, 248 and 256 workgroups by
tests/test_ops_gpu.py::test_packed_tile_deal_at_other_grid_sizes."""
import numpy as np
import pytest

BM, BN, TEAM = 128, 64, 2
INF = (1 << 63) - 1


def tiles_of(n):
    return (n + BM - 1) // BM


def cost_of(n):
    return 8 * ((n + BN - 1) // BN) + 24


def ctz(x):
    return (x & -x).bit_length() - 1


class Cursor:
    __slots__ = ("vb", "head", "b", "row0", "len", "cost")

    def __init__(self):
        self.vb, self.head, self.b, self.row0, self.len, self.cost = -1, 0, 0, 0, 0, 0

    def copy(self):
        c = Cursor()
        for k in self.__slots__:
            setattr(c, k, getattr(self, k))
        return c


def deal_of_workgroup(seq_n, heads, grid, g):
    """Tiles (head, sequence, first row) that workgroup `g` of `grid` processes, in order."""
    assert len(seq_n) == 64 and grid % 8 == 0
    pre = np.cumsum([tiles_of(n) * cost_of(n) for n in seq_n]).tolist()
    cost_per_head = pre[63]
    have = sum(1 << b for b, n in enumerate(seq_n) if n > 0)

    def settle(t, tile_in_seq, cost_end):
        while t.head < heads:
            n = t.len if t.len > 0 else seq_n[t.b]
            if tile_in_seq < tiles_of(n):
                t.row0, t.len = tile_in_seq * BM, n
                t.vb = 0 if t.cost < cost_end else -1
                return t
            later = 0 if t.b >= 63 else have & ~((2 << t.b) - 1)
            tile_in_seq, t.len = 0, 0
            if later:
                t.b = ctz(later)
            else:
                t.head += 1
                t.b = ctz(have)
                t.cost = t.head * cost_per_head
        t.vb = -1
        return t

    team_size = TEAM if grid % (8 * TEAM) == 0 else 1
    member = (g >> 3) % team_size
    load = [0 if m < team_size else INF for m in range(TEAM)]
    if cost_per_head <= 0:
        return []
    teams = grid // team_size
    team = (g & 7) * (teams // 8) + (g >> 3) // team_size
    total = cost_per_head * heads
    start = total // teams * team + total % teams * team // teams
    cost_end = total // teams * (team + 1) + total % teams * (team + 1) // teams
    t = Cursor()
    t.head = start // cost_per_head
    rem = start - t.head * cost_per_head
    t.b = next(b for b in range(64) if pre[b] > rem)
    n = seq_n[t.b]
    before = pre[t.b] - tiles_of(n) * cost_of(n)
    tile_in_seq = (rem - before + cost_of(n) - 1) // cost_of(n)          # first tile starting at or after rem
    t.cost = t.head * cost_per_head + before + tile_in_seq * cost_of(n)
    cursor = settle(t, tile_in_seq, cost_end)

    mine = []
    while cursor.vb >= 0:                                               # take(), until the list is exhausted
        t = cursor.copy()
        m = min(range(TEAM), key=lambda i: (load[i], i))                # the first of the least loaded members
        c = cost_of(t.len)
        load[m] += c
        cursor.cost += c
        cursor = settle(cursor, t.row0 // BM + 1, cost_end)
        if m == member:
            mine.append((t.head, t.b, t.row0))
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
    """64 sequences of 16..512 tokens, 12 heads, 256 workgroups: the heaviest workgroup carries at most 1.15x
    the mean cost (the figure the packed profile quotes is 1.12)."""
    lengths = np.random.RandomState(0).randint(16, 513, size=64).tolist()
    cost = [sum(cost_of(lengths[b]) for _, b, _ in deal_of_workgroup(lengths, 12, 256, g)) for g in range(256)]
    assert max(cost) <= 1.15 * (sum(cost) / 256), max(cost) / (sum(cost) / 256)
