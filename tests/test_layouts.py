"""The two fragment-order layouts, pinned on the CPU element by element: the copy of a matrix
that the decode products read, and the normalised rows of a decode step in the same order.
Both put element (row, k) of a piece of 16 rows x 32 of K at lane (k % 32) / 8 * 16 + row % 16,
value k % 8 of that lane: the order in which a 16x16x32 matrix instruction takes its operands."""
import pytest
import torch

from kappai_amd.kernels import ops


def place_in_piece(row: int, k: int) -> int:
    return ((k % 32) // 8 * 16 + row % 16) * 8 + k % 8


def test_matrix_copy_in_fragment_order():
    N, K = 48, 96
    w = torch.arange(N * K, dtype=torch.float32).remainder(251).to(torch.bfloat16).reshape(N, K)
    flat = ops.fragment_order(w).reshape(-1)
    for n in range(N):
        for k in range(K):
            piece = (n // 16) * (K // 32) + k // 32
            assert flat[piece * 512 + place_in_piece(n, k)] == w[n, k], (n, k)
    assert ops.fragment_order(w[:40]) is None and ops.fragment_order(w[:, :72]) is None
    assert ops.fragment_order(w.float()) is None


@pytest.mark.gpu
def test_rows_in_fragment_order_come_back_as_rows():
    n, D = 11, 96
    rows = torch.arange(n * D, dtype=torch.float32).remainder(241).to(torch.bfloat16).reshape(n, D)
    data = torch.full((16 * D,), -1.0, dtype=torch.bfloat16)
    for i in range(n):
        for k in range(D):
            data[(k // 32) * 512 + place_in_piece(i, k)] = rows[i, k]
    frag = ops.FragmentRows(data.reshape(16, D).to("cuda:0"), n, resid=torch.zeros(n, D))
    assert frag.shape == (n, D) and frag.dtype == torch.bfloat16
    assert torch.equal(frag.materialize().cpu(), rows)
    assert ops.FragmentRows.fits(16, 2048, torch.bfloat16)
    assert not ops.FragmentRows.fits(17, 2048, torch.bfloat16)       # one tile of 16 rows
    assert not ops.FragmentRows.fits(8, 2040, torch.bfloat16)        # whole pieces of 32 of K
    assert not ops.FragmentRows.fits(8, 2048, torch.float32)


def test_row_tables_of_a_step():
    """The int32 tables that ``layout_rows`` makes for a step of two prompt portions and three
    single decoded tokens: rows, positions, segments, and what the attention part's own layout
    adds to them (``AttentionTiles``): tiles of at most 32 rows; and with a limit for lone rows,
    the single tokens leave the tile table once the longest of their contexts reaches it (never in
    a step of single tokens only, where no tiles are used)."""
    import numpy as np
    from kappai_amd.cache import CacheManager, PagedKV
    from kappai_amd.engine.batch import StepEntry, layout_rows
    from kappai_amd.parts.attention import AttentionTiles
    cm = CacheManager([PagedKV(2, 16)], 16, 400, 8)
    held = {"a": 0, "b": 1500, "c": 40, "d": 70, "e": 2999}
    caches = {}
    for name, n in held.items():
        caches[name] = cm.open(name)
        if n:
            cm.extend(caches[name], n)
            cm.commit(caches[name], n)
    new = {"a": 70, "b": 1, "c": 33, "d": 1, "e": 1}
    entries = []
    for name, n in new.items():
        cm.extend(caches[name], n)
        entries.append(StepEntry(caches[name], list(range(n)), [n - 1]))
    arrays, sizes = layout_rows(entries, cm, 100, [AttentionTiles(32)])
    assert sizes["n_rows"] == 106 and sizes["max_segment_rows"] == 70
    assert sizes["max_position"] == 2999 and sizes["numbers"] == {"max_lone_position": -1}
    assert "lone_rows" not in arrays and sizes["extra"] == ["q_tiles"]
    assert arrays["seg_start"].tolist() == [0, 70, 71, 104, 105, 106]
    assert arrays["logit_rows"].tolist() == [69, 70, 103, 104, 105]
    assert arrays["row_pos"][[0, 69, 70, 71, 103, 104, 105]].tolist() == [0, 69, 1500, 40, 72, 70,
                                                                         2999]
    tiles = arrays["q_tiles"].tolist()
    assert [t[:3] for t in tiles] == [[0, 0, 32], [0, 32, 32], [0, 64, 6], [1, 70, 1], [2, 71, 32],
                                      [2, 103, 1], [3, 104, 1], [4, 105, 1]]
    assert [t[3] for t in tiles[:3]] == [0 | 3 << 16, 1 | 3 << 16, 2 | 3 << 16]
    # the longest lone context (3000 keys) reaches the limit: all three single tokens leave
    arrays, sizes = layout_rows(entries, cm, 100, [AttentionTiles(32, 3000)])
    assert arrays["lone_rows"].tolist() == [70, 104, 105]
    assert sizes["numbers"]["max_lone_position"] == 2999
    assert sorted(sizes["extra"]) == ["lone_rows", "q_tiles"]
    assert [t[:3] for t in arrays["q_tiles"].tolist()] == [[0, 0, 32], [0, 32, 32], [0, 64, 6],
                                                           [2, 71, 32], [2, 103, 1]]
    assert arrays["q_tiles"].dtype == np.int32 and arrays["lone_rows"].dtype == np.int32
    # it does not: nothing changes
    arrays, sizes = layout_rows(entries, cm, 100, [AttentionTiles(32, 3001)])
    assert "lone_rows" not in arrays and len(arrays["q_tiles"]) == 8
    # single tokens only: a decode step, which has no use for the list
    singles = [e for e in entries if len(e.tokens) == 1]
    arrays, sizes = layout_rows(singles, cm, 100, [AttentionTiles(32, 100)])
    assert "lone_rows" not in arrays and sizes["numbers"]["max_lone_position"] == -1
    # no part asks for anything: the step's own tables only
    arrays, sizes = layout_rows(entries, cm, 100)
    assert "q_tiles" not in arrays and sizes["extra"] == [] and sizes["numbers"] == {}


def test_tables_of_the_parts_own():
    """Layouts of different families are built side by side; layers that ask for the same family
    differently are brought to one (the attention tiles: one tile size or an error, the single
    rows apart only if all agree); two tables of one name, or a table that is not int32, are
    refused."""
    import numpy as np
    import pytest
    from kappai_amd.cache import CacheManager, PagedKV
    from kappai_amd.engine.batch import StepEntry, layout_rows
    from kappai_amd.parts.attention import AttentionTiles
    from kappai_amd.parts.base import StepTables

    class Chunks(StepTables):
        """The segments cut into chunks of four rows: (segment, first row, rows)."""
        family = "toy_chunks"

        def __init__(self, name="chunks", dtype=np.int32):
            self.name, self.dtype = name, dtype

        def __eq__(self, other):
            return isinstance(other, Chunks) and (self.name, self.dtype) == (other.name, other.dtype)

        def build(self, step):
            ss = step.arrays["seg_start"]
            rows = [(s, r, min(4, int(ss[s + 1]) - r)) for s in range(len(ss) - 1)
                    for r in range(int(ss[s]), int(ss[s + 1]), 4)]
            return {self.name: np.asarray(rows, dtype=self.dtype)}, {"n_chunks": len(rows)}

    cm = CacheManager([PagedKV(2, 16)], 16, 40, 4)
    entries = []
    for name, n in (("a", 9), ("b", 1), ("c", 6)):
        rc = cm.open(name)
        cm.extend(rc, n)
        entries.append(StepEntry(rc, list(range(n)), []))
    arrays, sizes = layout_rows(entries, cm, 100, [AttentionTiles(32), Chunks()])
    assert arrays["chunks"].tolist() == [[0, 0, 4], [0, 4, 4], [0, 8, 1], [1, 9, 1], [2, 10, 4],
                                         [2, 14, 2]]
    assert sizes["numbers"] == {"max_lone_position": -1, "n_chunks": 6}
    assert sizes["extra"] == ["q_tiles", "chunks"]
    with pytest.raises(ValueError, match="are called"):
        layout_rows(entries, cm, 100, [Chunks(), Chunks()])
    with pytest.raises(ValueError, match="are called"):
        layout_rows(entries, cm, 100, [Chunks("row_pos")])
    with pytest.raises(ValueError, match="int32"):
        layout_rows(entries, cm, 100, [Chunks(dtype=np.int64)])
    # what layers ask of one family
    t = AttentionTiles(32, 4096)
    assert t.combine([AttentionTiles(32, 4096)]) == t
    assert t.combine([AttentionTiles(32, None)]) == AttentionTiles(32, None)
    with pytest.raises(ValueError, match="different sizes"):
        t.combine([AttentionTiles(64, 4096)])
    with pytest.raises(ValueError, match="different tables"):
        Chunks().combine([Chunks("other")])
