"""dmoe_route_noalloc (the entry point that allocates nothing: its scratch is a buffer built into the library) gives
the bits of dmoe_route, through the C ABI, on calls in a row that share the built-in buffer."""
import ctypes

import pytest
import torch

from disagmoe_amd import _lib
from helpers import announce, dev

pytestmark = pytest.mark.gpu


def _route(ids: torch.Tensor, E: int, order: int, noalloc: bool):
    R = ids.numel()
    mappings = torch.full((R,), -7, dtype=torch.int64, device=ids.device)
    batch_sizes = torch.full((E,), -7, dtype=torch.int64, device=ids.device)
    offsets = torch.full((E + 1,), -7, dtype=torch.int64, device=ids.device)
    stream = torch.cuda.current_stream(ids.device).cuda_stream
    if noalloc:
        _lib.call("dmoe_route_noalloc", ids.data_ptr(), _lib.I32, R, E, order, mappings.data_ptr(), _lib.I64,
                  batch_sizes.data_ptr(), offsets.data_ptr(), stream)
    else:
        need = ctypes.c_size_t(0)
        _lib.call("dmoe_route_scratch_bytes", R, E, ctypes.byref(need))
        scratch = torch.empty(max(need.value, 1), dtype=torch.uint8, device=ids.device)
        _lib.call("dmoe_route", ids.data_ptr(), _lib.I32, R, E, order, mappings.data_ptr(), _lib.I64,
                  batch_sizes.data_ptr(), offsets.data_ptr(), scratch.data_ptr(), scratch.numel(), stream)
    torch.cuda.synchronize()
    return mappings, batch_sizes, offsets


def test_noalloc_route_matches_route_on_consecutive_calls():
    from oracle import routing
    g = torch.Generator().manual_seed(77)
    # sizes beyond one workgroup's 12 chunks, so that the histograms go through the scratch buffer: a large call with
    # the scanning launch (96 chunks x 64 experts), then a smaller one that finds the first call's contents there,
    # then a tiny one that needs no scratch at all
    for R, E, order in [(49152, 64, _lib.ORDER_REFERENCE), (9000, 8, _lib.ORDER_REFERENCE), (20000, 300, _lib.ORDER_STABLE),
                        (700, 8, _lib.ORDER_REFERENCE)]:
        announce(test="route_noalloc", R=R, E=E, order=order)
        ids = torch.randint(0, E, (R,), generator=g, dtype=torch.int32)
        if E > 2:
            ids[ids == 1] = 2                                        # an expert without rows
        got = _route(ids.to(dev()), E, order, noalloc=True)
        want = _route(ids.to(dev()), E, order, noalloc=False)
        for a, b in zip(got, want):
            assert torch.equal(a, b)
        if order == _lib.ORDER_REFERENCE:
            m_ref, cnt_ref = routing.get_mappings_from_exp_ids(ids, E)
            assert got[0].cpu().tolist() == m_ref and got[1].cpu().tolist() == cnt_ref


def test_noalloc_route_recorded_into_a_graph():
    """The caller the entry point is for: recorded once into a graph (after a first eager call, which looks up the
    built-in buffer's address), replayed with new ids after eager calls of other sizes have used the same buffer."""
    from oracle import routing
    R, E = 20000, 16                                                  # 40 chunks: the histograms go through the buffer
    g = torch.Generator().manual_seed(5)
    ids = torch.randint(0, E, (R,), generator=g, dtype=torch.int32).to(dev())
    mappings = torch.full((R,), -7, dtype=torch.int64, device=dev())
    batch_sizes = torch.full((E,), -7, dtype=torch.int64, device=dev())
    offsets = torch.full((E + 1,), -7, dtype=torch.int64, device=dev())
    _route(ids, E, _lib.ORDER_REFERENCE, noalloc=True)
    announce(test="route_noalloc_graph", R=R, E=E)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        _lib.call("dmoe_route_noalloc", ids.data_ptr(), _lib.I32, R, E, _lib.ORDER_REFERENCE, mappings.data_ptr(), _lib.I64,
                  batch_sizes.data_ptr(), offsets.data_ptr(), torch.cuda.current_stream().cuda_stream)
    for rep in range(3):
        new_ids = torch.randint(0, E, (R,), generator=g, dtype=torch.int32)
        new_ids[new_ids == 3] = 4
        ids.copy_(new_ids)
        other = torch.randint(0, 64, (49152 if rep % 2 == 0 else 9000,), generator=g, dtype=torch.int32).to(dev())
        _route(other, 64, _lib.ORDER_STABLE, noalloc=True)            # an eager call of another size in between
        graph.replay()
        torch.cuda.synchronize()
        m_ref, cnt_ref = routing.get_mappings_from_exp_ids(new_ids, E)
        assert mappings.cpu().tolist() == m_ref and batch_sizes.cpu().tolist() == cnt_ref, rep
        assert offsets.cpu().tolist() == [0] + torch.tensor(cnt_ref).cumsum(0).tolist()


def test_noalloc_route_refuses_what_does_not_fit():
    limit = ctypes.c_size_t(0)
    _lib.call("dmoe_route_noalloc_max_bytes", ctypes.byref(limit))
    assert limit.value == 4 << 20
    R, E = 600000, 4096                                              # (1172 + 1) chunks x 4096 experts x 4 bytes = 19 MB
    ids = torch.zeros(R, dtype=torch.int32, device=dev())
    out = torch.empty(R, dtype=torch.int64, device=dev())
    rc = _lib.load().dmoe_route_noalloc(ids.data_ptr(), _lib.I32, R, E, _lib.ORDER_REFERENCE, out.data_ptr(), _lib.I64,
                                        None, None, torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.ERR_WORKSPACE
    assert b"built-in buffer" in _lib.load().dmoe_last_error()
