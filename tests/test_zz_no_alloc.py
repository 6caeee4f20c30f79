"""`tk_route_static`, the routing entry point that allocates nothing (its scratch memory is a device array inside the
library), against `tk_route` with a caller workspace: bit-equal outputs on two calls in a row, the second with a
smaller input (the array keeps the first call's contents), and on the multi-launch path as well as the
single-launch one.  Sizes beyond the built-in buffer are refused with a message.  Through the C ABI (ctypes)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _route_both(device, T, E, k, seed):
    from triton_amd.tensor_details.bitmatrix import _route
    from triton_amd.tensor_details.ragged_tensor import _alloc
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn((T, E), generator=g).to(device)
    outs = []
    for static in (False, True):
        vals = torch.empty((T, k), dtype=torch.float32, device=device)
        indx = torch.empty((T, k), dtype=torch.int16, device=device)
        words = (E + 31) // 32
        bm = torch.zeros((words, (T + 31) // 32 * 32), dtype=torch.int32, device=device)
        bm_t = bm.transpose(0, 1)[:T]
        ragged = _alloc(E, T * k, device)
        r = _route(logits, indx, None, E, k, apply_softmax=True, use_provided_indx=False, vals=vals, bitmatrix_data=bm_t,
                   want_meta=True, want_extras=True, ragged=ragged, static_scratch=static)
        torch.cuda.synchronize()
        width = ragged[3]
        outs.append(dict(vals=vals, indx=indx, bitmatrix=bm, col_sum=r["col_sum"], col_sorted=r["col_sorted_indx"],
                         row_sorted=r["row_sorted_indx"], gather=r["gather_indx"], gammas=r["gammas"],
                         slice_offs=ragged[0], block_offs=ragged[1], schedule=ragged[2][:, :width]))
    return outs


def _assert_same(a, b, what):
    for name in a:
        assert torch.equal(a[name], b[name]), f"{what}: {name} differs between tk_route and tk_route_static"


# (first call, second smaller call): the single-launch router (T*k <= 1024) and the three-launch one
@pytest.mark.parametrize("first,second", [((4096, 128, 4), (300, 128, 4)), ((64, 128, 4), (16, 128, 4)),
                                          ((1500, 200, 8), (129, 13, 1))])
def test_route_static_matches_route_twice_in_a_row(device, first, second):
    for i, (T, E, k) in enumerate((first, second)):
        ref, got = _route_both(device, T, E, k, seed=10 * T + E + i)
        _assert_same(ref, got, f"T={T} E={E} k={k}")
        assert int(got["col_sum"].sum()) == T * k


def test_route_static_refuses_sizes_beyond_its_buffer(device):
    from triton_amd import _native as nt
    T, E = 65536, 2048  # tk_route_workspace_bytes is 8 MiB here, the built-in array holds 2 MiB
    assert nt.lib().tk_route_workspace_bytes(T, E) > 2 * 1024 * 1024
    d = nt.RouteDesc()
    dummy = torch.zeros(16, dtype=torch.int32, device=device)
    d.logits = dummy.data_ptr()
    d.logits_dtype = nt.TK_F32
    d.n_tokens, d.n_rows, d.n_experts, d.k = T, -1, E, 2
    d.indx = dummy.data_ptr()
    d.indx_dtype = nt.TK_I16
    d.col_sum = d.col_sorted_indx = d.row_sorted_indx = dummy.data_ptr()
    rc = nt.lib().tk_route_static(d, None)  # refused before anything is launched
    assert rc == nt.TK_ERR_UNSUPPORTED
    assert "scratch" in nt.last_error()


def test_route_static_in_a_hip_graph_after_one_eager_call(device):
    """The address of the built-in scratch array is looked up on the first call on a device (or by
    `tk_route_static_prepare`), which must happen outside graph capture; afterwards the entry point can be captured.
    The graph is replayed twice with eager routing work in between and compared with `tk_route` each time."""
    from triton_amd import _native as nt
    from triton_amd.tensor_details.bitmatrix import _route
    from triton_amd.tensor_details.ragged_tensor import _alloc
    assert nt.lib().tk_route_static_prepare() == nt.TK_OK
    T, E, k = 64, 128, 4
    g = torch.Generator().manual_seed(77)
    logits = torch.randn((T, E), generator=g).to(device)

    def run(static, lg):
        vals = torch.empty((T, k), dtype=torch.float32, device=device)
        indx = torch.empty((T, k), dtype=torch.int16, device=device)
        bm = torch.zeros(((E + 31) // 32, (T + 31) // 32 * 32), dtype=torch.int32, device=device)
        ragged = _alloc(E, T * k, device)
        r = _route(lg, indx, None, E, k, apply_softmax=True, use_provided_indx=False, vals=vals, bitmatrix_data=bm.transpose(0, 1)[:T],
                   want_meta=True, want_extras=True, ragged=ragged, static_scratch=static)
        return dict(vals=vals, indx=indx, bitmatrix=bm, col_sum=r["col_sum"], col_sorted=r["col_sorted_indx"],
                    row_sorted=r["row_sorted_indx"], gather=r["gather_indx"], gammas=r["gammas"], slice_offs=ragged[0],
                    block_offs=ragged[1])

    run(True, logits)  # eager call: allocations of the Python helpers are warmed up outside the capture as well
    torch.cuda.synchronize()
    lg = logits.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(True, lg)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        got = run(True, lg)
    for rep in range(2):
        lg.copy_(torch.randn((T, E), generator=g).to(device))  # new inputs for every replay
        graph.replay()
        torch.cuda.synchronize()
        ref = run(False, lg)
        torch.cuda.synchronize()
        _assert_same(ref, got, f"graph replay {rep}")
