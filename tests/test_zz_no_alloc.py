"""`smoe_route_static` - the routing prep for callers that cannot allocate - through the C ABI, against `smoe_route`
(the existing entry point it is a variant of) and against the oracle: bit-exact, on two calls in a row of which the
second is smaller (the built-in histogram buffer then still holds the first call's contents)."""
import ctypes

import pytest
import torch

import oracle
from scattermoe_amd import _C

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _ids(L, E, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, E, (L,), generator=g)


def _route(lib, entry, ids, E):
    L = ids.numel()
    eid = torch.empty(L, dtype=torch.int64, device=DEV)
    idx = torch.empty(L, dtype=torch.int64, device=DEV)
    off = torch.empty(E, dtype=torch.int64, device=DEV)
    stream = _C.stream_ptr(ids.device)
    if entry == "static":
        rc = lib.smoe_route_static(_C.ptr(ids), _C.index_code(ids.dtype), L, E, _C.ptr(eid), _C.ptr(idx), _C.ptr(off),
                                   stream)
    else:
        need = lib.smoe_route_workspace_bytes(L, E)
        ws = torch.empty(max(need, 1), dtype=torch.uint8, device=DEV)
        rc = lib.smoe_route(_C.ptr(ids), _C.index_code(ids.dtype), L, E, _C.ptr(eid), _C.ptr(idx), _C.ptr(off),
                            _C.ptr(ws), need, stream)
    assert rc == 0, lib.smoe_last_error()
    torch.cuda.synchronize()
    return eid.cpu(), idx.cpu(), off.cpu()


def test_route_static_matches_route_on_two_calls_in_a_row():
    lib = _C.load()
    with torch.cuda.device(0):
        assert lib.smoe_route_static_init() == 0, lib.smoe_last_error()
        # large first (64 chunks x 128 experts of histograms), then smaller inputs that reuse the same buffer
        # ((32768, 8) still takes the three launches and the buffer; the last two are sorted by one workgroup,
        # without it)
        for L, E, dtype in [(262144, 128, torch.int64), (100000, 600, torch.int64), (40000, 33, torch.int32),
                            (32768, 8, torch.int64), (4097, 5, torch.int64), (300, 8, torch.int64)]:
            ids = _ids(L, E, seed=L + E).to(dtype)
            got = _route(lib, "static", ids.to(DEV), E)
            want = _route(lib, "workspace", ids.to(DEV), E)
            ref = oracle.route_ref(ids, E)
            for a, b, c in zip(got, want, ref):
                assert torch.equal(a, b) and torch.equal(a, c), "L=%d E=%d" % (L, E)


def test_route_static_allocates_nothing_and_replays_from_a_graph():
    """What the entry point is for: after smoe_route_static_init() a call changes neither torch's nor the device's
    memory accounting, and it can be captured into a HIP graph (capture forbids allocation) and replayed on fresh
    ids - with eager work between the replays - bit-exact against the oracle every time."""
    lib = _C.load()
    L, E = 100000, 64                                    # three launches, histograms in the built-in buffer
    with torch.cuda.device(0):
        assert lib.smoe_route_static_init() == 0, lib.smoe_last_error()
        ids = _ids(L, E, seed=1).to(DEV)
        eid = torch.empty(L, dtype=torch.int64, device=DEV)
        idx = torch.empty(L, dtype=torch.int64, device=DEV)
        off = torch.empty(E, dtype=torch.int64, device=DEV)

        def call():
            rc = lib.smoe_route_static(_C.ptr(ids), _C.index_code(ids.dtype), L, E, _C.ptr(eid), _C.ptr(idx),
                                       _C.ptr(off), _C.stream_ptr(ids.device))
            assert rc == 0, lib.smoe_last_error()

        call()
        torch.cuda.synchronize()
        before = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0])
        call()
        torch.cuda.synchronize()
        assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0]) == before

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            call()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            call()
        for r in range(3):
            fresh = _ids(L, E, seed=10 + r)
            ids.copy_(fresh.to(DEV))
            eid.fill_(-1); idx.fill_(-1); off.fill_(-1)                  # eager work between the replays
            graph.replay()
            torch.cuda.synchronize()
            for got, want in zip((eid, idx, off), oracle.route_ref(fresh, E)):
                assert torch.equal(got.cpu(), want), "replay %d" % r


def test_route_static_rejects_what_does_not_fit():
    lib = _C.load()
    one = ctypes.c_void_p(256)
    # 2^20 bytes hold 262144 chunk-by-expert counters: 4096 chunks x 128 experts is twice that
    assert lib.smoe_route_static(one, 0, 4096 * 4096, 128, one, one, one, None) == -4      # SMOE_ERR_WORKSPACE
    assert b"built-in buffer" in lib.smoe_last_error()
    assert lib.smoe_route_static(None, 0, 16, 8, None, None, None, None) == -1             # SMOE_ERR_NULL
