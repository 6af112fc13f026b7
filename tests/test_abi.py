"""CPU-side checks of the drop-in boundary: the library loads without a GPU
and exports every symbol that include/tango_hip.h declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "tango_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tango_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    from tango_amd import _lib
    handle = ctypes.CDLL(_lib.LIB_PATH)
    names = declared_symbols()
    assert len(names) >= 20
    for n in names:
        assert hasattr(handle, n), "library lacks %s" % n
        assert n in _lib.SIGNATURES, "ctypes binding lacks %s" % n
    assert set(_lib.SIGNATURES) == set(names)


def test_status_strings_and_version():
    from tango_amd import _lib
    L = _lib.lib()
    assert L.tango_abi_version() >= 1
    assert L.tango_status_string(0) == b"ok"
    for code in (-1, -2, -3, -4):
        assert L.tango_status_string(code) not in (b"ok", b"unknown status")
    assert L.tango_status_string(-99) == b"unknown status"


def test_argument_validation_needs_no_gpu():
    # every entry point validates on the host before touching the device
    from tango_amd import _lib
    L = _lib.lib()
    assert L.tango_absmax_f32(None, 10, None, None) == -1
    assert L.tango_quantize_f32_i8(None, -1, None, None, 0, None, 0, 0, None, None) == -1
    assert L.tango_spmm_csr_u_mul_e(1, 1, 1, None, 1, 1, 1, 4, 4, 2, 8, 3, 10, None) == -2  # D not in {1, F}
    assert L.tango_sddmm_ewise_i8(7, 1, None, 1, 1, 1, 1, 1, 1, 4, 4, None) == -2  # unknown op
    assert L.tango_spmm_csr_copy_u(1, 1, 1, 1, 8, 1, 4, 1 << 31, 10, 8, None) == -2  # node ids must fit 31 bits
    # the dense-block aggregation: a plan is required, and features wider than 256 columns have no workspace size
    assert L.tango_spmm_csr_copy_u_dense(1, None, 1, 64, 1, None, None, 0, None, 64, None, None, None, 0, None) == -1
    plan = _lib.DensePlan()
    plan.rows, plan.num_src, plan.row_blocks, plan.dense_rows, plan.dense_cols = 512, 512, 1, 256, 256
    assert L.tango_spmm_dense_workspace(ctypes.byref(plan), 300) == 0
    assert L.tango_spmm_dense_workspace(ctypes.byref(plan), 41) >= 256 * 64 + 256 * 64 * 4
    assert L.tango_spmm_dense_mask_build(None, None, 32, 4, None, None, None, None, 0, None, None, None, None) == -1


def test_static_scratch_rejects_oversized_input():
    from tango_amd import _lib
    L = _lib.lib()
    E, H = 40_000_000, 8
    assert L.tango_edge_softmax_workspace(E, H) > (4 << 20)
    # rejected on the host before any launch: the pointers are never dereferenced
    assert L.tango_edge_softmax_fwd_static(16, 16, 16, None, 10, E, H, 0.2, None) == -5
    assert b"scratch" in L.tango_status_string(-5)


def test_infer_broadcast_shape():
    from tango_amd.kernels import infer_broadcast_shape as ibs
    assert ibs("add", (8, 1), (8, 1)) == (8, 1)
    assert ibs("mul", (4, 16), (4, 1)) == (4, 16)
    assert ibs("dot", (8, 16), (8, 16)) == (8, 1)
    assert ibs("add", (3,), (2, 3)) == (2, 3)
    import pytest
    with pytest.raises(ValueError):
        ibs("add", (3,), (4,))


def test_backward_passes_refuse_graph_capture(monkeypatch):
    """Capturing a whole training step into a HIP graph once ended the process with a segmentation fault whose
    cause is not established; until it is, every backward pass of the package raises when its stream is being
    captured.  Checked on the host: the capture state is stubbed, no GPU work is involved (the capture itself is
    deliberately never attempted on a GPU, not even to see the error)."""
    import pytest
    import torch
    from tango_amd import kernels
    from tango_amd.QLinear import Qlinear_func, Qlinear_shared_func
    from tango_amd.SDDMM import sddmm_u_add_v, sddmm_u_dot_v
    from tango_amd.SPMM import spmm_copy_u, spmm_u_mul_e
    from tango_amd.edge_softmax import _EdgeSoftmax
    from tango_amd.gat import attn_scores
    from tango_amd.loss import _SoftmaxXent
    kernels.refuse_capture("eager")  # not capturing: passes
    monkeypatch.setattr(torch.cuda, "is_initialized", lambda: True)
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: True)
    with pytest.raises(RuntimeError, match="HIP graph"):
        kernels.refuse_capture("x")
    for fn, nargs in ((Qlinear_func, 1), (Qlinear_shared_func, 2), (sddmm_u_add_v, 1), (sddmm_u_dot_v, 1),
                      (spmm_copy_u, 1), (spmm_u_mul_e, 1), (_EdgeSoftmax, 1), (attn_scores, 2), (_SoftmaxXent, 1)):
        with pytest.raises(RuntimeError, match="HIP graph"):
            fn.backward(object(), *([None] * nargs))  # refuses before it looks at its context


def test_bipartite_graph_formats():
    """A bipartite Graph (sources and destinations numbered in spaces of their own): its compressed formats are
    those of the square graph on max(n_src, n_dst) nodes cut to their own row counts, and the relation parts of
    a heterogeneous graph put every edge in exactly one part with endpoints inside the part's node types.
    Host tensors only."""
    import numpy as np
    import torch
    from tango_amd.graph import Graph, hetero_power_law
    rng = np.random.default_rng(4)
    ns, nd, E = 7, 19, 60
    src, dst = rng.integers(0, ns, E), rng.integers(0, nd, E)
    g = Graph(torch.from_numpy(src), torch.from_numpy(dst), ns, nd)
    sq = Graph(torch.from_numpy(src), torch.from_numpy(dst), nd)
    assert (g.num_src_nodes(), g.num_dst_nodes(), g.num_edges()) == (ns, nd, E)
    import pytest
    with pytest.raises(ValueError):
        g.num_nodes()
    ip, ix, eid = g.adj_sparse("csr")
    sip, six, seid = sq.adj_sparse("csr")
    assert ip.numel() == ns + 1 and torch.equal(ip, sip[:ns + 1]) and torch.equal(ix, six) and torch.equal(eid, seid)
    ip, ix, eid = g.adj_sparse("csc")
    assert ip.numel() == nd + 1 and all(torch.equal(a, b) for a, b in zip((ip, ix, eid), sq.adj_sparse("csc")))
    assert torch.equal(g.in_degrees(), torch.bincount(torch.from_numpy(dst), minlength=nd))
    assert torch.equal(g.out_degrees(), torch.bincount(torch.from_numpy(src), minlength=ns))
    g2 = g.reorder_edges_by_dst()
    assert g2.num_dst_nodes() == nd and bool((g2.edges()[1][1:] >= g2.edges()[1][:-1]).all())
    # the generator's heterogeneous graph, cut into parts the way relation_graphs does (that function itself
    # builds the device-side formats and needs the library)
    sizes, rels = (30, 20, 10), ((0, 1), (1, 0), (1, 2), (2, 0))
    hg, node_type, edge_type = hetero_power_law(type_sizes=sizes, relations=rels, edges_per_relation=100)
    bounds = np.cumsum((0,) + sizes)
    s, d = (t.numpy() for t in hg.edges())
    for r, (a, b) in enumerate(rels):
        m = edge_type.numpy() == r
        assert (node_type.numpy()[s[m]] == a).all() and (node_type.numpy()[d[m]] == b).all()
        assert s[m].min() >= bounds[a] and s[m].max() < bounds[a + 1] and d[m].max() < bounds[b + 1]


def test_label_reuse_input_and_warm_up_schedule():
    """evaluation/arxiv_gat.py:534-543 on host tensors: one-hot label columns for the chosen nodes only, and a
    learning rate that climbs linearly over the first 50 epochs and is left alone afterwards."""
    import torch
    from tango_amd.evaluation import add_labels, warm_up_lr
    feat = torch.arange(12.0).reshape(4, 3)
    labels = torch.tensor([2, 0, 1, 2])
    out = add_labels(feat, labels, torch.tensor([0, 2]), 3)
    assert out.shape == (4, 6) and torch.equal(out[:, :3], feat)
    assert torch.equal(out[:, 3:], torch.tensor([[0.0, 0, 1], [0, 0, 0], [0, 1, 0], [0, 0, 0]]))
    opt = torch.optim.SGD([torch.zeros(1, requires_grad=True)], lr=0.5)
    seen = []
    for epoch in (1, 25, 50, 51):
        warm_up_lr(opt, 0.2, epoch)
        seen.append(opt.param_groups[0]["lr"])
    assert seen == [0.2 / 50, 0.1, 0.2, 0.2]


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asking for more exits with a message before anything touches a device."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode != 0 and "one GPU" in (res.stderr + res.stdout)


def test_stochastic_windows_are_never_handed_out_twice(monkeypatch):
    """Eager stochastic quantize calls interleaved with the capture and replays of a graph: replaying the
    (host offset, advance) pairs against a stand-in for the device counter, no window of the random stream is used
    twice, and captured calls draw from a part of the stream of their own.  Host only: the capture state is stubbed."""
    import torch
    from tango_amd import config
    capturing = [False]
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: capturing[0])
    key = object()
    monkeypatch.setattr(config, "device_offset", lambda device: key)
    monkeypatch.setattr(config, "_pending", {})
    counter = [0]
    used = []

    def run(args):  # what the kernels do: draw at counter + offset, then the one-thread kernel moves the counter
        used.append(counter[0] + args["offset"][0])
        counter[0] += args["advance"]

    def eager(k):
        for _ in range(k):
            run(config.stochastic_args(None))

    eager(5)
    capturing[0] = True
    graph = [config.stochastic_args(None) for _ in range(3)]  # recorded, not run: the counter stays put
    capturing[0] = False
    eager(4)                      # after the capture, before any replay
    for _ in range(2):
        for args in graph:        # a replay
            run(args)
        eager(70)                 # crosses a batch boundary of the eager calls
    assert len(set(used)) == len(used)
    assert all(a["offset"][0] == config.CAPTURE_BASE and a["advance"] == config.WINDOW for a in graph)
    assert all(u % config.WINDOW == 0 for u in used)
