"""CPU: the work-item tables of the column kernel of the fused attention backward pass (host logic only)."""
import pytest
import torch

from torch_blocksparse.attention_core import _ColumnTable


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
        count, offset, h, c, slot = t[8 * i:8 * i + 5]
        assert t[8 * i + 5:8 * i + 8] == [0, 0, 0]
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
        split = {(s[4 * i], s[4 * i + 1]): (s[4 * i + 2], s[4 * i + 3]) for i in range(ct.n_split)}
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
