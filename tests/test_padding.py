"""How a step is laid into the padded sizes of a recorded step (host arrays only: no GPU)."""
import numpy as np
import pytest

from ginfer_amd.engine.runner import ModelRunner, pad_step
from ginfer_amd.kernels import ops


def host_arrays(q_len, q_start, page=8, want_last=True):
    """What ModelRunner._host_arrays makes for entries of these lengths, one cache group, pages numbered from 1."""
    q_len, q_start = np.asarray(q_len, dtype=np.int64), np.asarray(q_start, dtype=np.int64)
    E, T = len(q_len), int(q_len.sum())
    cu = np.zeros(E + 1, dtype=np.int32)
    np.cumsum(q_len, out=cu[1:])
    ent = np.repeat(np.arange(E, dtype=np.int32), q_len)
    pos = (np.arange(T) - np.repeat(cu[:-1], q_len) + np.repeat(q_start, q_len)).astype(np.int32)
    width = int(-(-(q_start + q_len).max() // page))
    table = np.full((E, width), -1, dtype=np.int32)
    nxt = 1
    for e in range(E):
        for b in range(-(-int(q_start[e] + q_len[e]) // page)):
            table[e, b] = nxt
            nxt += 1
    slots = table[ent, pos // page].astype(np.int64) * page + pos % page
    rows = np.asarray([int(cu[e + 1]) - 1 for e in range(E)] if want_last else [], dtype=np.int32)
    return dict(E=E, T=T, ids=np.arange(1, T + 1, dtype=np.int32), pos=pos, ent=ent, cu=cu, q_start=q_start.astype(np.int32),
                q_len=q_len, rows=rows, width=width, tables=[table], slot_maps=[slots],
                state_slots=np.arange(E, dtype=np.int64), max_kv=int((q_start + q_len).max()),
                decode_info=ModelRunner._decode_info(cu, q_len, q_start, ent, T == E))


@pytest.mark.parametrize("q_len,q_start", [([1, 5, 1, 20], [30, 0, 7, 16]), ([40], [0]), ([1, 1, 2], [3, 9, 0]), ([17, 33, 1], [0, 16, 99])])
def test_a_step_laid_into_padded_sizes(q_len, q_start):
    host = host_arrays(q_len, q_start)
    T, E = host["T"], host["E"]
    t_pad, e_pad, width = 64, 8, 16
    p = pad_step(host, t_pad, e_pad, width, pad_slot=99)
    dummy = e_pad
    # sizes
    assert p["T"] == t_pad and p["E"] == e_pad + 1 and p["width"] == width
    assert all(len(p[k]) == t_pad for k in ("ids", "pos", "ent")) and len(p["slot_maps"][0]) == t_pad
    assert len(p["cu"]) == e_pad + 2 and len(p["q_start"]) == e_pad + 1 and len(p["rows"]) == e_pad
    assert p["tables"][0].shape == (e_pad + 1, width) and p["decode_info"].shape == (e_pad, 4)
    assert p["tiles"].shape == (t_pad // ops.PLAN_TILE_ROWS + e_pad, 4)
    # the step's own part is untouched
    for k in ("ids", "pos", "ent"):
        assert np.array_equal(p[k][:T], host[k])
    assert np.array_equal(p["slot_maps"][0][:T], host["slot_maps"][0]) and np.array_equal(p["rows"][:E], host["rows"])
    assert np.array_equal(p["tables"][0][:E, :host["width"]], host["tables"][0])
    # the padding: tokens of the extra entry at position 0, which write nothing and read page 0 only
    assert (p["ent"][T:] == dummy).all() and (p["pos"][T:] == 0).all() and (p["slot_maps"][0][T:] == -1).all()
    assert p["tables"][0][dummy, 0] == 0 and (p["tables"][0][dummy, 1:] == -1).all() and (p["tables"][0][E:dummy] == -1).all()
    # entries: cu is monotone, the empty entries own nothing, the extra entry owns the padding rows
    assert (np.diff(p["cu"]) >= 0).all() and p["cu"][E] == T and p["cu"][dummy] == T and p["cu"][dummy + 1] == t_pad
    assert int(p["q_len"].sum()) == t_pad and p["q_len"][dummy] == t_pad - T and (p["q_len"][E:dummy] == 0).all()
    # the plan: every own row is covered exactly once by a record of a single token or by a tile; what fills the plan
    # points at the first padding row
    covered = np.zeros(t_pad, dtype=int)
    singles = sum(1 for n in q_len if n == 1)
    for i, (row, pos, entry, _) in enumerate(p["decode_info"]):
        if i < singles:
            assert entry < E and host["q_len"][entry] == 1 and pos == host["q_start"][entry] and row == host["cu"][entry]
            covered[row] += 1
        else:
            assert (row, pos, entry) == (T, 0, dummy)
    for entry, row0, rows, pos0 in p["tiles"]:
        if entry == dummy:
            assert (row0, rows, pos0) == (T, 1, 0)
            continue
        assert 1 <= rows <= ops.PLAN_TILE_ROWS and host["cu"][entry] <= row0 and row0 + rows <= host["cu"][entry + 1]
        assert pos0 == host["q_start"][entry] + row0 - host["cu"][entry]
        covered[row0:row0 + rows] += 1
    assert (covered[:T] == 1).all() and (covered[T:] == 0).all()


def test_rows_go_to_records_and_tiles():
    rows, pos, entries, tiles = ops.plan_rows([1, 20, 1, 3], [5, 0, 8, 40], 16)
    assert rows == [0, 21] and pos == [5, 8] and entries == [0, 2]
    assert sorted(tiles) == [(1, 1, 16, 0), (1, 17, 4, 16), (3, 22, 3, 40)]
    assert tiles[0] == (3, 22, 3, 40)            # the tile with the most keys comes first
