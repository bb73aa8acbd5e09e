"""CPU: the work-item tables of the column kernel of the fused attention backward pass (host logic only)."""
import pytest
import torch

from torch_blocksparse.attention_core import _ColumnTable, _GatheredTiles


@pytest.mark.parametrize('seed,shape,density,part', [(0, (2, 8, 8), 0.5, 3), (1, (3, 40, 24), 0.7, 16), (2, (1, 5, 9), 0.2, 2), (3, (2, 33, 7), 1.0, 8)])
def test_items_cover_every_column_in_row_order(seed, shape, density, part):
    torch.manual_seed(seed)
    H, R, C = shape
    lay = (torch.rand(H, R, C) < density).long()
    lay[0, :, 0] = 1                                    # one long column
    lay[:, :, C - 1] = 0                                # and an empty one in every head
    ct = _ColumnTable(lay, 'cpu', part)
    t = ct.items.tolist()
    ids = {tuple(x): i for i, x in enumerate(lay.nonzero().tolist())}
    assert ct.columns == C and ct.n_items >= H * C
    seen = {}
    slots = []
    for i in range(ct.n_items):
        count, offset, h, c, slot = t[12 * i:12 * i + 5]
        assert t[12 * i + 5:12 * i + 12] == [0, 0, 0, c, c, c, c]
        assert 0 <= count <= part
        blocks = [t[offset + 4 * b:offset + 4 * b + 4] for b in range(count)]
        for bid, r, cc, hh in blocks:
            assert (cc, hh) == (c, h) and ids[(h, r, c)] == bid
        seen.setdefault((h, c), []).append((slot, [b[1] for b in blocks]))
        if slot >= 0:
            slots.append(slot)
    assert slots == list(range(ct.n_slots))             # parts of a column follow each other, slots in order
    assert len(seen) == H * C
    split = {}
    if ct.n_split:
        s = ct.split.tolist()
        split = {(s[8 * i], s[8 * i + 1]): (s[8 * i + 2], s[8 * i + 3]) for i in range(ct.n_split)}
        assert all(s[8 * i + 4:8 * i + 8] == [s[8 * i + 1]] * 4 for i in range(ct.n_split))
    for (h, c), parts in seen.items():
        rows = [r for _, rs in parts for r in rs]
        assert rows == lay[h, :, c].nonzero().flatten().tolist()       # every block once, by row
        if len(parts) == 1:
            assert parts[0][0] == -1 and (h, c) not in split
            assert len(rows) <= part
        else:
            assert len(rows) > part
            first, n = split[(h, c)]
            assert n == len(parts) and [p[0] for p in parts] == list(range(first, first + n))
            sizes = [len(rs) for _, rs in parts]
            assert max(sizes) - min(sizes) <= 1 and min(sizes) >= 1
    assert len(split) == sum(1 for p in seen.values() if len(p) > 1)


def _ids_of(lay):
    ids = torch.full(lay.shape, -1, dtype=torch.int64)
    ids[lay] = torch.arange(int(lay.sum()))
    return ids


@pytest.mark.parametrize('S,seed,density', [(2, 0, 0.3), (4, 1, 0.3), (4, 2, 0.05), (2, 3, 0.9)])
def test_gathered_tiles_hold_every_block_once(S, seed, density):
    """A line of tiles = S block-rows; its tiles take the block-columns that hold a block in any of them, ascending, S per
    tile; padding slots repeat a valid column and carry no block."""
    torch.manual_seed(seed)
    H, R, C = 2, 4 * S, 6 * S + 1
    lay = torch.rand(H, R, C) < density
    lay[0, :S] = False                                   # an empty line
    lay[1, S, :] = True                                  # a full block-row
    ids = _ids_of(lay)
    g = _GatheredTiles(lay, ids, S)
    assert g.entries().shape == (g.n_tiles, 8 + S * S)
    seen = set()
    for line in range(H * (R // S)):
        h, t = divmod(line, R // S)
        want = lay[h, t * S:(t + 1) * S].any(0).nonzero().flatten().tolist()
        assert int(g.sizes[line]) == -(-len(want) // S)
        got = []
        for k in range(int(g.sizes[line])):
            tile = int(g.starts[line]) + k
            e = g.entries()[tile].tolist()
            assert e[:4] == [tile, 0, t, h] and e[4:4 + S] == g.cols[tile].tolist() and e[8:] == g.ids[tile].flatten().tolist()
            for slot in range(S):
                c = int(g.cols[tile, slot])
                assert 0 <= c < C
                blocks = [int(g.ids[tile, i, slot]) for i in range(S)]
                if len(got) < len(want) and c == want[len(got)]:
                    for i, b in enumerate(blocks):
                        assert b == int(ids[h, t * S + i, c])
                        if b >= 0:
                            assert b not in seen
                            seen.add(b)
                    got.append(c)
                else:
                    assert blocks == [-1] * S            # padding
        assert got == want
    assert len(seen) == int(lay.sum())


@pytest.mark.parametrize('S,seed', [(2, 0), (4, 1)])
def test_column_table_of_small_blocks(S, seed):
    """Columns of tiles = S block-columns, the long ones together (every block-column in exactly one), their tiles gather
    block-rows; ids per tile as [gathered block-row][block-column of the group]; every block once."""
    torch.manual_seed(seed)
    H, R, C = 2, 9 * S, 5 * S
    lay = torch.rand(H, R, C) < 0.1
    lay[:, :, 1] = True                                  # a long column
    lay[:, :, 2 * S + 1] = True                          # and another one, in another aligned group of S
    ids = _ids_of(lay)
    ct = _ColumnTable(lay.long(), 'cpu', part=3, S=S, ids=ids)
    t = ct.items.tolist()
    ES = 8 + S * S
    assert ct.columns == C // S
    seen, cols_seen = set(), {h: [] for h in range(H)}
    per_column = {}
    for i in range(ct.n_items):
        count, offset, h, c, slot = t[12 * i:12 * i + 5]
        groups = t[12 * i + 8:12 * i + 8 + S]
        per_column.setdefault((h, c), (groups, []))
        assert per_column[(h, c)][0] == groups
        for e in range(count):
            tile, _, c2, h2 = t[offset + ES * e:offset + ES * e + 4]
            rows = t[offset + ES * e + 4:offset + ES * e + 4 + S]
            tiles = t[offset + ES * e + 8:offset + ES * (e + 1)]
            assert (c2, h2) == (c, h)
            for i2, r in enumerate(rows):
                for gidx, col in enumerate(groups):
                    b = tiles[i2 * S + gidx]
                    if b >= 0:
                        assert bool(lay[h, r, col]) and int(ids[h, r, col]) == b and b not in seen
                        seen.add(b)
            per_column[(h, c)][1].append(rows)
    assert len(seen) == int(lay.sum())
    for (h, c), (groups, _) in per_column.items():
        cols_seen[h] += groups
    for h in range(H):
        assert sorted(cols_seen[h]) == list(range(C))    # a partition of the block-columns
        assert set(per_column[(h, 0)][0][:2]) == {1, 2 * S + 1}          # the two long columns share the first group
        rest = [c for cc in range(1, C // S) for c in per_column[(h, cc)][0]]
        assert rest == sorted(rest) or S == 2            # the others as they lie (S = 2: the first group is the two long ones)
