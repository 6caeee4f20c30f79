"""Pins the routing oracle (oracle/routing.py) against the worked examples in the reference's docstrings,
the padding rule of its top-k test, closed forms and brute force.  CPU only."""
import numpy as np
import pytest
import torch

from oracle import routing as ort


def test_bitmatrix_docstring_example():
    # tensor_details/bitmatrix.py:11-19: 4x7 bitmatrix, nonzeros numbered row-major
    rows = [[2, 4, 5], [1, 5], [0, 1, 2, 6], [2, 4]]
    flat = torch.tensor([c for r in rows for c in r], dtype=torch.int32)
    m = ort.make_bitmatrix_metadata(flat, 7)
    assert m.col_sum.tolist() == [1, 2, 3, 0, 2, 2, 1]
    assert m.col_sorted_indx.tolist() == [5, 3, 6, 0, 7, 9, 1, 10, 2, 4, 8]
    assert m.row_sorted_indx.tolist() == [3, 6, 8, 1, 9, 0, 2, 4, 10, 5, 7]


def test_bitmatrix_dropped_entries_are_compacted():
    # bitmatrix.py:160-162: -1 entries are dropped, the tail is padded with -1
    indx = torch.tensor([[1, 0], [-1, -1], [0, 1]], dtype=torch.int32)
    m = ort.make_bitmatrix_metadata(indx, 3)
    assert m.col_sum.tolist() == [2, 2, 0]
    assert m.col_sorted_indx.tolist()[-2:] == [-1, -1] and m.row_sorted_indx.tolist()[-2:] == [-1, -1]


@pytest.mark.parametrize("T, E, k", [(1, 8, 2), (37, 128, 4), (300, 200, 8), (64, 7, 1)])
def test_bitmatrix_invariants(T, E, k):
    g = torch.Generator().manual_seed(T * 1000 + E)
    logits = torch.randn((T, E), generator=g)
    _, indx, _ = ort.topk(logits, k)
    m = ort.make_bitmatrix_metadata(indx, E)
    R = T * k
    assert int(m.col_sum.sum()) == R
    assert np.array_equal(m.col_sum.numpy(), np.bincount(indx.reshape(-1).numpy(), minlength=E))
    cs, rs = m.col_sorted_indx.long(), m.row_sorted_indx.long()
    assert torch.equal(cs[rs], torch.arange(R)) and torch.equal(rs[cs], torch.arange(R))
    e_sorted = indx.reshape(-1)[cs]
    assert torch.all(e_sorted[1:] >= e_sorted[:-1])
    same = e_sorted[1:] == e_sorted[:-1]
    assert torch.all(cs[1:][same] > cs[:-1][same]), "stable within an expert"


def test_ragged_docstring_block_offs():
    # tensor_details/ragged_tensor.py:16-29 (the block_offs rows; 256 is the extra HIP block size)
    sizes = torch.tensor([15, 17, 0, 127], dtype=torch.int32)
    md = ort.make_ragged_tensor_metadata(sizes, int(sizes.sum()))
    assert md.slice_offs.tolist() == [0, 15, 32, 32, 159]
    expect = {16: [0, 1, 3, 3, 11], 32: [0, 1, 2, 2, 6], 64: [0, 1, 2, 2, 4], 128: [0, 1, 2, 2, 3], 256: [0, 1, 2, 2, 3]}
    for i, bs in enumerate(ort.BLOCK_SIZES):
        assert md.block_offs_data[i].tolist() == expect[bs]
    # schedule entries are (block_in_slice << 16) | slice_id; for 128: (0,0) (0,1) (0,3) then -1
    sch = md.block_schedule_data[ort.BLOCK_SIZES.index(128)].tolist()
    assert sch[:3] == [0, 1, 3] and set(sch[3:]) == {-1}
    sch16 = md.block_schedule_data[0].tolist()
    assert sch16[:4] == [0, 1, (1 << 16) | 1, 3] and sch16[10] == (7 << 16) | 3 and sch16[11] == -1


@pytest.mark.parametrize("E", [1, 7, 33, 911, 1025])
def test_ragged_brute_force(E):
    # tests/test_tensor_details/... brute force of ragged_tensor.py:243-256 over awkward slice counts
    rng = np.random.default_rng(E)
    sizes = rng.integers(0, 200, E).astype(np.int32)
    sizes[rng.integers(0, E, max(1, E // 5))] = 0
    R = int(sizes.sum())
    md = ort.make_ragged_tensor_metadata(torch.from_numpy(sizes), R)
    assert md.slice_offs.tolist() == [0] + np.cumsum(sizes).tolist()
    width = ort.max_n_blocks(E, R)
    assert md.block_schedule_data.shape == (len(ort.BLOCK_SIZES), width)
    for i, bs in enumerate(ort.BLOCK_SIZES):
        want = []
        for e, s in enumerate(sizes.tolist()):
            want += [(b << 16) | e for b in range(-(-s // bs))]
        assert len(want) <= ort.n_blocks(E, R, bs) <= width
        got = md.block_schedule_data[i].tolist()
        assert got[:len(want)] == want and all(v == -1 for v in got[len(want):])
        assert md.block_offs_data[i].tolist() == [0] + np.cumsum(-(-sizes // bs)).tolist()


def test_n_blocks_floor_division():
    # ragged_tensor.py:73-81 uses Python floor division on a negative numerator
    assert ort.n_blocks(128, 16384, 16) == 127 + 1017 == 1144
    assert ort.n_blocks(8, 5, 16) == 5
    for E, R, bs in [(4, 159, 16), (4, 159, 128), (128, 129, 128), (3, 1000, 64)]:
        worst = max(sum(-(-s // bs) for s in split) for split in _splits(E, R, bs))
        assert ort.n_blocks(E, R, bs) == worst


def _splits(E, R, bs):
    # the worst case puts one row in E-1 slices and the rest in one; a few other splits for contrast
    yield [1] * (E - 1) + [R - (E - 1)]
    yield [R] + [0] * (E - 1)
    yield [R // E] * (E - 1) + [R - (R // E) * (E - 1)]


def test_topk_all_equal_padding_rule():
    # tests/test_topk.py:39-51: equal payloads pick experts 0..k-1
    x = torch.full((5, 16), 0.25)
    v, i, bits = ort.topk(x, 4)
    assert i.tolist() == [[0, 1, 2, 3]] * 5
    assert torch.allclose(v, torch.full((5, 4), 0.25))
    assert (bits.view(torch.int32)[:, 0] == 0xF).all()


@pytest.mark.parametrize("T, E, k", [(3, 5, 2), (17, 33, 8), (300, 200, 8)])
def test_topk_brute_force(T, E, k):
    g = torch.Generator().manual_seed(E)
    x = torch.randn((T, E), generator=g)
    x[:, ::3] = x[:, 1:2]  # ties across a third of the experts
    v, indx, bits = ort.topk(x, k, apply_softmax=False)
    for t in range(T):
        cand = sorted(range(E), key=lambda e: (-float(x[t, e]), e))[:k]
        assert indx[t].tolist() == cand
        assert v[t].tolist() == [float(x[t, e]) for e in cand]
        words = bits[t].numpy().view(np.uint32)
        sel = {e for e in range(E) if (int(words[e // 32]) >> (e % 32)) & 1}
        assert sel == set(cand)


def test_topk_softmax_closed_form():
    x = torch.tensor([[0.0, np.log(3.0), -50.0, np.log(3.0)]], dtype=torch.float32)
    v, i, _ = ort.topk(x, 2)
    assert i.tolist() == [[1, 3]] and torch.allclose(v, torch.tensor([[0.5, 0.5]]))
    v, i, _ = ort.topk(x, 4)
    assert i.tolist() == [[1, 3, 0, 2]] and torch.allclose(v[0, :3], torch.tensor([3 / 7, 3 / 7, 1 / 7]), atol=1e-6)


def test_routing_glue():
    # tests/test_distributed.py:203-210: gather = col_sorted // k, scatter = col_sorted, gammas = vals[col_sorted]
    g = torch.Generator().manual_seed(9)
    T, E, k = 50, 12, 4
    logits = torch.randn((T, E), generator=g)
    r = ort.routing(logits, k)
    cs = r.meta.col_sorted_indx.long()
    assert torch.equal(r.gather_indx.long(), cs // k)
    assert torch.equal(r.scatter_indx.long(), cs)
    assert torch.equal(r.gammas, r.vals.reshape(-1)[cs])
    assert torch.allclose(r.vals.sum(-1), torch.ones(T), atol=1e-6)


def test_remap_ragged_metadata_hand_example_and_rebuild():
    """`remap_ragged_tensor_metadata` (ragged_tensor.py:388-433).  Hand-worked: sizes [15, 17, 0, 127] keeping slices 1 and 3
    as local 0 and 1.  Block size 16: blocks per slice [1, 2, 0, 8], offsets [0, 1, 3, 3, 11]; kept offsets are those of
    slices 1 and 3 (1 and 3), then the 10 entries kept, then -1.  Independent check: the compacted schedule equals the
    schedule built from scratch for the kept sizes [17, 127], entry for entry."""
    from oracle import routing as ort
    sizes = torch.tensor([15, 17, 0, 127], dtype=torch.int32)
    md = ort.make_ragged_tensor_metadata(sizes, 159)
    smap = torch.tensor([-1, 0, -1, 1], dtype=torch.int32)
    r = ort.remap_ragged_tensor_metadata(md, smap)
    assert r.slice_sizes.tolist() == [17, 127, -1, -1]
    assert r.slice_offs.tolist() == [15, 32, -1, -1, -1]
    assert r.block_offs_data[0].tolist() == [1, 3, 10, -1, -1]  # block size 16
    assert r.block_offs_data[3].tolist() == [1, 2, 2, -1, -1]  # block size 128: one block each
    s16 = r.block_schedule_data[0].tolist()
    assert s16[:10] == [(0 << 16) | 0, (1 << 16) | 0] + [(b << 16) | 1 for b in range(8)] and set(s16[10:]) <= {-1}
    fresh = ort.make_ragged_tensor_metadata(torch.tensor([17, 127], dtype=torch.int32), 159)
    for i in range(len(ort.BLOCK_SIZES)):
        n = int(fresh.block_offs_data[i][-1])
        assert r.block_schedule_data[i][:n].tolist() == fresh.block_schedule_data[i][:n].tolist()
        assert int(r.block_offs_data[i][2]) == n
    # a permuting map only renames the slice ids inside the schedule
    smap2 = torch.tensor([2, -1, 0, 1], dtype=torch.int32)
    r2 = ort.remap_ragged_tensor_metadata(md, smap2)
    assert r2.slice_sizes.tolist() == [15, 0, 127, -1]
    assert [e & 0xFFFF for e in r2.block_schedule_data[3].tolist() if e != -1] == [2, 1]


@pytest.mark.parametrize("apply_softmax", [True, False])
def test_topk_backward_matches_autograd(apply_softmax):
    """The backward oracle against torch autograd of the forward oracle's definition (values = softmax over the kept
    logits, topk.py:160-174): an independent derivation of the same gradient."""
    from oracle import routing as ort
    g = torch.Generator().manual_seed(3)
    T, E, k = 37, 50, 4
    x = torch.randn((T, E), generator=g, dtype=torch.float64).requires_grad_()
    _, indx, _ = ort.topk(x.detach().float(), k, apply_softmax)
    dy = torch.randn((T, k), generator=g, dtype=torch.float64)
    kept = torch.gather(x, 1, indx.long())
    vals = torch.softmax(kept, dim=1) if apply_softmax else kept
    (vals * dy).sum().backward()
    got = ort.topk_backward(x.detach().float(), indx, dy.float(), apply_softmax)
    assert torch.allclose(got.double(), x.grad, rtol=1e-5, atol=1e-6)
    assert int((got != 0).sum(dim=1).max()) <= k
    part = ort.topk_backward(x.detach().float(), indx, dy.float(), apply_softmax, n_rows=10)
    assert torch.equal(part[:10], got[:10]) and not part[10:].any()
