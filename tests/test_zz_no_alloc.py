"""The entry point that allocates nothing (tango_edge_softmax_fwd_static) against the
workspace form of the same operation (tango_edge_softmax_fwd), through the C ABI.

Both run the same kernels, so the outputs must agree bit for bit.  Two calls in a row share
the library's fixed device array; the second, smaller one must not be disturbed by what the
first left there."""
import numpy as np
import pytest
import torch

from gpu_util import dev, host, powerlaw_graph

pytestmark = pytest.mark.gpu


def _dst_major(src, dst, n):
    order = np.argsort(dst, kind="stable")
    indptr = np.zeros(n + 1, np.int64)
    np.cumsum(np.bincount(dst, minlength=n), out=indptr[1:])
    return indptr, order.astype(np.int64)


def _both(L, e, indptr, eids, rows, slope):
    from tango_amd._lib import check
    E, H = e.shape
    stream = torch.cuda.current_stream().cuda_stream
    ws_bytes = L.tango_edge_softmax_workspace(E, H)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")
    want = torch.full_like(e, float("nan"))
    check(L.tango_edge_softmax_fwd(want.data_ptr(), e.data_ptr(), indptr.data_ptr(), eids.data_ptr(), rows, E, H,
                                   slope, ws.data_ptr(), ws_bytes, stream), "edge_softmax_fwd")
    got = torch.full_like(e, float("nan"))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    check(L.tango_edge_softmax_fwd_static(got.data_ptr(), e.data_ptr(), indptr.data_ptr(), eids.data_ptr(), rows,
                                          E, H, slope, stream), "edge_softmax_fwd_static")
    torch.cuda.synchronize()
    assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == before
    return host(got), host(want)


def test_static_scratch_matches_workspace_form_twice(orc):
    from tango_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(71)
    # first call: hubs with thousands of in-edges (rows cut by many span boundaries), H = 8
    # second call: a smaller graph and another head count, over the scratch the first call left behind
    for n, E, H, slope in ((6000, 400000, 8, 0.2), (900, 7001, 3, 1.0)):
        src, dst = powerlaw_graph(rng, n, E)
        indptr, eids = _dst_major(src, dst, n)
        e = rng.standard_normal((E, H)).astype(np.float32) * 3
        got, want = _both(L, dev(e), dev(indptr), dev(eids), n, slope)
        assert np.isfinite(got).all()
        assert np.array_equal(got, want)
        ref = orc.edge_softmax_fwd(e, indptr, eids, slope)
        np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-6)


def test_static_scratch_calls_on_two_streams_are_ordered(orc):
    """Two calls that share the device array, issued back to back on different streams without any host-side
    ordering: the second waits for the first on the GPU, so both results are right."""
    from tango_amd import _lib
    from tango_amd._lib import check
    L = _lib.lib()
    rng = np.random.default_rng(72)
    cases = []
    for n, E, H in ((5000, 300000, 8), (4000, 250000, 4)):
        src, dst = powerlaw_graph(rng, n, E)
        indptr, eids = _dst_major(src, dst, n)
        e = rng.standard_normal((E, H)).astype(np.float32) * 3
        cases.append((n, E, H, e, indptr, eids, dev(e), dev(indptr), dev(eids), torch.full((E, H), float("nan"), device="cuda")))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for rep in range(3):
        for (n, E, H, _, _, _, e_d, ip_d, id_d, out), st in zip(cases, streams):
            check(L.tango_edge_softmax_fwd_static(out.data_ptr(), e_d.data_ptr(), ip_d.data_ptr(), id_d.data_ptr(), n, E, H,
                                                  0.2, st.cuda_stream), "edge_softmax_fwd_static")
    torch.cuda.synchronize()
    for n, E, H, e, indptr, eids, _, _, _, out in cases:
        np.testing.assert_allclose(host(out), orc.edge_softmax_fwd(e, indptr, eids, 0.2), rtol=1e-5, atol=1e-6)
