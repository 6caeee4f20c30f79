"""GPU parity of the router and the routing metadata (through the C ABI) against the CPU oracle.

Cases mirror python/triton_kernels/tests/test_topk.py:11-51 and tests/test_tensor.py:243-302:
indices, bitmatrix, histogram, both permutations and the ragged block schedule are compared bit for bit;
gate values within the float tolerance the reference uses for them."""
import pytest
import torch

from oracle import routing as ort
from oracle.checks import assert_close, assert_equal

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tk(device):
    import triton_amd.tensor as tensor
    import triton_amd.topk as topk
    return topk, tensor


def _logits(T, E, dtype, seed=0, ties=False):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((T, E), generator=g)
    if ties:
        # many equal logits exercise the lower-index tie rule; '+ 0.0' turns -0.0 into +0.0 because the
        # packed integer key orders +0.0 above -0.0 (as the reference kernel does) while argsort ties them
        x = torch.round(x * 2) / 2 + 0.0
    return x.to(dtype)


@pytest.mark.parametrize("T", [1, 7, 256, 300])
@pytest.mark.parametrize("E", [13, 32, 128, 200])
@pytest.mark.parametrize("k", [1, 4, 8])
@pytest.mark.parametrize("softmax", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_topk(tk, device, T, E, k, softmax, dtype):
    topk, _ = tk
    x = _logits(T, E, dtype, seed=T * 1000 + E, ties=(E == 32))
    sm = topk.topk(x.to(device), k, apply_softmax=softmax)
    vals, indx, bits = ort.topk(x, k, apply_softmax=softmax)
    assert sm.indx.dtype == torch.int16 and sm.vals.dtype == dtype
    assert_equal(indx, sm.indx.to(torch.int32), "indx")
    assert_close(vals, sm.vals, what="vals")
    # bitmatrix: shape (T, words) over uint32 storage allocated column-major and padded to 32 rows
    data = sm.mask.storage.data
    words = (E + 31) // 32
    assert tuple(data.shape) == (T, words) and data.stride() == (1, (T + 31) // 32 * 32)
    assert sm.mask.shape == [T, E]
    assert_equal(bits, data.view(torch.int32), "bitmatrix")
    m = ort.make_bitmatrix_metadata(indx, E)
    assert_equal(m.col_sum, sm.mask_metadata.col_sum, "col_sum")
    assert_equal(m.col_sorted_indx, sm.mask_metadata.col_sorted_indx, "col_sorted_indx")
    assert_equal(m.row_sorted_indx, sm.mask_metadata.row_sorted_indx, "row_sorted_indx")


def test_topk_all_equal_picks_lowest_indices(tk, device):
    topk, _ = tk
    x = torch.zeros((5, 40), dtype=torch.float32, device=device)
    sm = topk.topk(x, 8, apply_softmax=False)
    assert sm.indx.to(torch.int32).tolist() == [list(range(8))] * 5


def test_topk_n_rows_and_provided_indx(tk, device):
    topk, _ = tk
    x = _logits(50, 64, torch.float32, seed=5)
    sm = topk.topk(x.to(device), 4, n_rows=37)
    vals, indx, bits = ort.topk(x, 4, n_rows=37)
    assert_equal(indx[:37], sm.indx[:37].to(torch.int32), "indx")
    m = ort.make_bitmatrix_metadata(indx, 64)
    assert_equal(m.col_sum, sm.mask_metadata.col_sum, "col_sum")
    assert_equal(m.col_sorted_indx, sm.mask_metadata.col_sorted_indx, "col_sorted_indx")
    assert_equal(m.row_sorted_indx, sm.mask_metadata.row_sorted_indx, "row_sorted_indx")
    # user-provided indices: values are gathered, softmax still applies
    yi = torch.stack([torch.randperm(64, generator=torch.Generator().manual_seed(i))[:4] for i in range(50)]).to(torch.int16)
    sm2 = topk.topk(x.to(device), 4, y_indx=yi.to(device))
    ref = torch.softmax(torch.gather(x, 1, yi.long()), dim=-1)
    assert_close(ref, sm2.vals, what="vals with provided indx")
    m2 = ort.make_bitmatrix_metadata(yi.int(), 64)
    assert_equal(m2.col_sorted_indx, sm2.mask_metadata.col_sorted_indx, "col_sorted_indx")


@pytest.mark.parametrize("T", [7, 256, 17111])
@pytest.mark.parametrize("E", [13, 32, 128, 811])
@pytest.mark.parametrize("k", [1, 4, 8])
def test_make_bitmatrix_metadata(tk, device, T, E, k):
    _, tensor = tk
    g = torch.Generator().manual_seed(T + E + k)
    indx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(min(T, 512))])
    indx = indx.repeat((T + indx.shape[0] - 1) // indx.shape[0], 1)[:T].to(torch.int32)
    if T > 7:
        indx[T - T // 10:] = -1  # masked tail rows, as `topk(..., n_rows=...)` leaves them
    from triton_amd.tensor_details.dtype import BIT
    bm = tensor.wrap_torch_tensor(torch.empty((T, (E + 31) // 32), dtype=torch.int32, device=device), dtype=BIT, shape=[T, E])
    got = tensor.make_bitmatrix_metadata(indx.to(device), bm)
    ref = ort.make_bitmatrix_metadata(indx, E)
    assert_equal(ref.col_sum, got.col_sum, "col_sum")
    assert_equal(ref.col_sorted_indx, got.col_sorted_indx, "col_sorted_indx")
    assert_equal(ref.row_sorted_indx, got.row_sorted_indx, "row_sorted_indx")
    valid = ref.col_sorted_indx >= 0
    assert int(valid.sum()) == int(ref.col_sum.sum())


def test_make_bitmatrix_metadata_with_dropped_entries(tk, device):
    """Entries equal to -1 in the middle of the index matrix are skipped.  Positions are flat offsets
    t*k+j into the index matrix (what the reference kernel stores, bitmatrix.py:55-73), so the result is
    checked through its defining properties rather than against the compacting torch twin."""
    _, tensor = tk
    T, E, k = 300, 40, 4
    g = torch.Generator().manual_seed(11)
    indx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    indx[torch.rand((T, k), generator=g) < 0.15] = -1
    from triton_amd.tensor_details.dtype import BIT
    bm = tensor.wrap_torch_tensor(torch.empty((T, 2), dtype=torch.int32, device=device), dtype=BIT, shape=[T, E])
    got = tensor.make_bitmatrix_metadata(indx.to(device), bm)
    flat = indx.reshape(-1)
    n_valid = int((flat >= 0).sum())
    col, row = got.col_sorted_indx.cpu(), got.row_sorted_indx.cpu()
    assert torch.equal(got.col_sum.cpu(), torch.bincount(flat[flat >= 0].long(), minlength=E).int())
    assert bool((col[n_valid:] == -1).all()) and bool((col[:n_valid] >= 0).all())
    experts = flat[col[:n_valid].long()]
    assert bool((experts >= 0).all())
    key = experts.long() * flat.numel() + col[:n_valid].long()
    assert bool((key[1:] > key[:-1]).all())  # grouped by expert, flat order inside a group (stable)
    assert bool((row[flat < 0] == -1).all())
    assert torch.equal(col[row[flat >= 0].long()].long(), torch.nonzero(flat >= 0).reshape(-1))


@pytest.mark.parametrize("E", [1, 7, 33, 911, 1025])
def test_make_ragged_tensor_metadata(tk, device, E):
    _, tensor = tk
    g = torch.Generator().manual_seed(E)
    sizes = torch.randint(0, 200, (E, ), generator=g, dtype=torch.int32)
    sizes[torch.rand(E, generator=g) < 0.2] = 0
    R = int(sizes.sum()) + 5
    got = tensor.make_ragged_tensor_metadata(sizes.to(device), R)
    ref = ort.make_ragged_tensor_metadata(sizes, R)
    assert_equal(ref.slice_offs, got.slice_offs, "slice_offs")
    assert_equal(ref.block_offs_data, got.block_offs_data, "block_offs")
    assert_equal(ref.block_schedule_data, got.block_schedule_data, "block_schedule")
    assert got.block_offs(64).shape == (E + 1, )


def test_docstring_examples(tk, device):
    _, tensor = tk
    got = tensor.make_ragged_tensor_metadata(torch.tensor([15, 17, 0, 127], dtype=torch.int32, device=device), 159)
    assert got.block_offs_data.tolist()[:4] == [[0, 1, 3, 3, 11], [0, 1, 2, 2, 6], [0, 1, 2, 2, 4], [0, 1, 2, 2, 3]]
    assert got.slice_offs.tolist() == [0, 15, 32, 32, 159]
    assert got.block_schedule(128).tolist()[:4] == [0, 1, 3, -1]
    assert got.block_schedule(64).tolist()[:5] == [0, 1, 3, (1 << 16) | 3, -1]


def test_baseline_router_shape(tk, device):
    """gpt-oss shape: 4096 tokens, 128 experts, top-4; plus a skewed decode batch."""
    topk, _ = tk
    for T, seed, skew in [(4096, 2, False), (16, 3, True), (1, 3, True), (64, 3, True)]:
        g = torch.Generator().manual_seed(seed)
        x = torch.randn((T, 128), generator=g)
        if skew:
            x = x + torch.randn((128, ), generator=g) * 1.5
        sm = topk.topk(x.to(device), 4)
        r = ort.routing(x, 4)
        assert_equal(r.indx, sm.indx.to(torch.int32), "indx")
        assert_equal(r.meta.col_sum, sm.mask_metadata.col_sum, "col_sum")
        assert_equal(r.meta.col_sorted_indx, sm.mask_metadata.col_sorted_indx, "col_sorted")
        assert_equal(r.meta.row_sorted_indx, sm.mask_metadata.row_sorted_indx, "row_sorted")
        assert_close(r.vals, sm.vals, what="vals")


@pytest.mark.parametrize("n_slices", [9, 32, 911, 1025])
def test_remap_ragged_tensor_metadata(device, n_slices):
    """Mirrors tests/test_tensor.py:259-277 of the reference: random sizes with an empty slice, a random permutation as
    slice map with five entries dropped; every output tensor equals the oracle's."""
    from oracle import routing as ort
    from triton_amd.tensor import make_ragged_tensor_metadata, remap_ragged_tensor_metadata
    g = torch.Generator().manual_seed(n_slices)
    max_slice_size = 200
    n_total_rows = max_slice_size * n_slices
    sizes = torch.randint(0, max_slice_size, (n_slices, ), dtype=torch.int32, generator=g)
    sizes[int(torch.randint(0, n_slices, (1, ), generator=g))] = 0
    smap = torch.randperm(n_slices, generator=g).to(torch.int32)
    smap[torch.randint(0, n_slices, (5, ), generator=g)] = -1
    md = make_ragged_tensor_metadata(sizes.to(device), n_total_rows)
    got = remap_ragged_tensor_metadata(md, smap.to(device))
    ref = ort.remap_ragged_tensor_metadata(ort.make_ragged_tensor_metadata(sizes, n_total_rows), smap)
    assert torch.equal(got.slice_sizes.cpu(), ref.slice_sizes)
    assert torch.equal(got.slice_offs.cpu(), ref.slice_offs)
    assert torch.equal(got.block_offs_data.cpu(), ref.block_offs_data)
    assert torch.equal(got.block_schedule_data.cpu(), ref.block_schedule_data)


def test_matmul_on_remapped_metadata(device):
    """The expert-parallel use (tests/test_distributed.py:236-241 of the reference): global metadata restricted to a
    rank's experts, the rank's weights only; rows of the kept experts sit at their global positions."""
    from oracle import moe as omoe
    from oracle.checks import assert_close
    from triton_amd.matmul import matmul
    from triton_amd.tensor import make_ragged_tensor_metadata, remap_ragged_tensor_metadata
    g = torch.Generator().manual_seed(5)
    E, K, N = 8, 256, 192
    sizes = torch.tensor([40, 17, 0, 130, 33, 5, 64, 11], dtype=torch.int32)
    M = int(sizes.sum())
    local = [1, 3, 4, 6]
    smap = torch.full((E, ), -1, dtype=torch.int32)
    smap[local] = torch.arange(len(local), dtype=torch.int32)
    x = torch.randn((M, K), generator=g).to(torch.bfloat16)
    w = (torch.randn((E, K, N), generator=g) * 0.1).to(torch.bfloat16)
    md = remap_ragged_tensor_metadata(make_ragged_tensor_metadata(sizes.to(device), M), smap.to(device))
    y = matmul(x.to(device), w[local].to(device), None, md).cpu()
    offs = torch.cumsum(torch.cat([torch.zeros(1, dtype=torch.int64), sizes.long()]), 0)
    for e in local:
        lo, hi = int(offs[e]), int(offs[e + 1])
        ref = omoe.matmul(x[lo:hi], w[e:e + 1], None, torch.tensor([hi - lo]))
        assert_close(ref, y[lo:hi], what=f"rows of expert {e}")


@pytest.mark.parametrize("T, E, k", [(1, 8, 2), (300, 200, 8), (4096, 128, 4), (77, 1000, 32)])
@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("apply_softmax", [True, False])
def test_topk_backward(device, T, E, k, dt, apply_softmax):
    """`topk_backward` (topk.py:76-85, _topk_backward.py:5-51) against the oracle, and through autograd of `topk`."""
    from triton_amd.topk import topk, topk_backward
    g = torch.Generator().manual_seed(T + E)
    x = torch.randn((T, E), generator=g).to(dt)
    dy = torch.randn((T, k), generator=g).to(dt)
    _, indx, _ = ort.topk(x, k, apply_softmax)
    n_rows = None if T < 100 else T - 5
    dx = topk_backward(x.to(device), indx.to(torch.int16).to(device), dy.to(device), k, n_rows, apply_softmax)
    ref = ort.topk_backward(x, indx, dy, apply_softmax, n_rows)
    assert dx.dtype == dt and dx.shape == x.shape
    assert torch.equal((dx.cpu() != 0), (ref != 0)) or dt == torch.bfloat16  # same support (bf16 may round tiny values to 0)
    tol = dict(rtol=2e-5, atol=1e-6) if dt == torch.float32 else dict(rtol=2e-2, atol=1e-3)
    assert torch.allclose(dx.cpu().float(), ref.float(), **tol)
    # through autograd: d/dx of sum(vals * dy)
    xg = x.to(device).requires_grad_()
    sm = topk(xg, k, apply_softmax=apply_softmax)
    assert_equal(indx, sm.indx.to(torch.int32), "indx")
    (sm.vals.float() * dy.to(device).float()).sum().backward()
    full = ort.topk_backward(x, indx, dy, apply_softmax)
    assert torch.allclose(xg.grad.cpu().float(), full.float(), **tol)
