#!/usr/bin/env python3
"""Benchmark of the quantized-GNN primitive layer on one MI355X.

A "step" is one training epoch (forward + loss + backward + Adam step) of the
quantized 2-layer GCN 602 -> 256 -> 41 on the synthetic 232,965-node /
~114.6M-edge power-law graph: int8 GEMMs with cached quantized operands, the
GEMM epilogue's scale handed to the int8 aggregation, stochastic rounding on
gradients.  Inputs are resident in HBM before the timed region.  Prints one
JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# Counter figures of the dominant kernel on the default benchmark graph live in one place, the committed
# rocprofv3 summary below (a line `bench-constants: {json}`): bytes that cross the L2 <-> fabric boundary per
# launch (FETCH_SIZE + WRITE_SIZE, each scaled by what the same counter reads for a 1 GiB device copy) and the
# launch time with every gather hitting the L2.  Counters cannot be read from inside a timed run.
SPMM_COUNTER_SUMMARY = os.path.join(ROOT, "profiles", "spmm_copy_u_F256_counters.md")


def counter_constants(path=SPMM_COUNTER_SUMMARY):
    try:
        with open(path) as f:
            for line in f:
                if line.startswith("bench-constants:"):
                    return json.loads(line.split(":", 1)[1])
    except (OSError, ValueError):
        pass
    return {}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--nodes", type=int, default=232965)
    ap.add_argument("--edges", type=int, default=114_600_000)
    ap.add_argument("--cpu-fraction", type=float, default=1.0, help="share of rows the CPU baseline runs")
    ap.add_argument("--cpu-reps", type=int, default=7, help="repetitions of the CPU baseline (median reported)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-primitives", action="store_true")
    ap.add_argument("--emit", default=None, metavar="JSON_FILE",
                    help="also store the result under the key 'measured_mi355x' of this JSON file")
    ap.add_argument("--feat", type=int, default=256, help="feature width of --profile-mode spmm")
    ap.add_argument("--permute-ids", action="store_true",
                    help="--profile-mode spmm on the benchmark graph with its node ids randomly permuted")
    ap.add_argument("--no-dense", action="store_true",
                    help="--profile-mode spmm without the dense bit blocks: the gather kernel on the whole adjacency")
    ap.add_argument("--l2-window", action="store_true",
                    help="--profile-mode spmm --no-dense with every column index folded into the first 16,384 rows "
                         "(4 MB of 256-byte rows): all gathers hit the L2, the launch time is the request-rate floor")
    ap.add_argument("--gemm-shape", default="256,41", metavar="K,N",
                    help="layer shape of --profile-mode gradx / gradw (dY [nodes, N] int8, X [nodes, K])")
    ap.add_argument("--attn-graph", choices=["gat", "hgt"], default="gat",
                    help="graph of --profile-mode umule / sddmm-dot: the 169,343-node GAT graph (8 heads x 16) or the "
                         "170,000-node / 8.17 M-edge homogenised heterogeneous graph (4 heads x 64)")
    ap.add_argument("--profile-mode", default=None,
                    choices=["spmm", "copy", "mfma", "qlinear", "gradx", "gradw", "sddmm", "quantize", "softmax", "umule",
                             "gat", "arxiv", "arxiv-gcn", "hgt", "hetero"],
                    help="run only the dominant kernel (spmm: copy_u F=256 on the benchmark graph) or a "
                         "1 GiB device copy (counter calibration), for rocprofv3 --pmc passes")
    return ap.parse_args()


class KernelTimer:
    """HIP-event timing of selected launches on torch's current stream (the stream the library launches on)."""

    def __init__(self):
        self.spans = {}

    def wrap(self, fn, key_of):
        import torch

        def timed(*a, **kw):
            key = key_of(*a, **kw)
            if key is None:
                return fn(*a, **kw)
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            r = fn(*a, **kw)
            e.record()
            self.spans.setdefault(key, []).append((s, e))
            return r
        return timed

    def mean_ms(self, key):
        v = [s.elapsed_time(e) for s, e in self.spans.get(key, [])]
        return sum(v) / len(v) if v else None

    def clear(self):
        self.spans = {}


def time_op(fn, iters=20, warm=3):
    import torch
    for _ in range(warm):
        fn()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) / iters


# Bytes per column index the aggregation kernels read: graph_preprocess makes one-time int32 copies
# of the int64 index arrays (conversion: two elementwise casts per graph, outside every timed region).
IDX_BYTES = 4


def spmm_bytes(nnz, rows, F, idx=IDX_BYTES):
    """Gather-traffic model: every gathered row counted once per edge.  Most of these bytes are served by the
    caches, so the rate it gives is an effective (cache-inclusive) bandwidth, not a fraction of HBM."""
    return nnz * (F + idx) + rows * (4 * F + 8)


def spmm_compulsory_bytes(nnz, rows, num_src, F, idx=IDX_BYTES):
    """What must cross HBM at least once: the index stream, the int8 features, the fp32 output."""
    return nnz * idx + rows * 8 + num_src * F + rows * 4 * F


def mfma_probe(torch, iters=4000):
    """Sustained rate of the int8 matrix instructions (register-resident chains, 32 wavefronts per CU)."""
    from tango_amd import _lib
    L = _lib.lib()
    sink = torch.zeros(64 + 65536, dtype=torch.int32, device="cuda")  # the result word, then a source for the staged probe
    st = torch.cuda.current_stream().cuda_stream
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    blocks = cus * 8
    out = {}
    shapes = ((0, "16x16x64", 2 * 16 * 16 * 64), (1, "32x32x32", 2 * 32 * 32 * 32),
              # the same instruction with its first operand expanded from bits in front of every 1, 2, 4 of them
              (2, "32x32x32_8valu", 2 * 32 * 32 * 32), (3, "32x32x32_4valu", 2 * 32 * 32 * 32),
              (4, "32x32x32_2valu", 2 * 32 * 32 * 32),
              # the bit-block kernel's inner loop without global loads (64 instructions per round), without / with
              # the LDS writes and the barrier that end a unit; two workgroups per CU
              (5, "32x32x32_loop", 2 * 32 * 32 * 32), (6, "32x32x32_loop_write_barrier", 2 * 32 * 32 * 32),
              (7, "32x32x32_loop_barrier", 2 * 32 * 32 * 32),
              # ... and with the next chunk staged by global-to-LDS loads from a cached buffer (sink: 256 B + 256 KB)
              (8, "32x32x32_loop_lds_loads_barrier", 2 * 32 * 32 * 32))
    for shape, name, ops in shapes:
        nb, it, per = (blocks, iters, 8) if shape < 5 else (cus * 2, iters // 8, 64)
        ms = time_op(lambda: _lib.check(L.tango_probe_mfma_i8(shape, it, nb, sink.data_ptr(), st), "probe"),
                     iters=5, warm=2)
        out["i8_%s_TOPS" % name] = round(nb * 4 * it * per * ops / ms / 1e9, 1)
    return out


def folded_spmm_ms(g, K, torch, F=256, window=16384, iters=10):
    """The gather kernel on the whole adjacency with every column index folded into the first `window` rows:
    every gather hits the L2, so the time is what the L2 request rate alone allows for this many slots."""
    ip, ix = g.adj_csc[0], g.adj_csc32[0]
    folded = torch.remainder(ix, window).to(torch.int32)
    feat = torch.randint(-127, 128, (g.num_nodes(), F), dtype=torch.int8, device="cuda")
    out = torch.empty((g.num_nodes(), F), dtype=torch.float32, device="cuda")
    one = torch.full((1,), 0.01, device="cuda")
    ms = time_op(lambda: K.cuda_kernels.csr_SPMM(out, ip, folded, feat, one, max_row=g.max_in_degree), iters=iters)
    return ms


def dense_part_ms(plan, K, torch, F, ld=None, iters=10):
    """The dense half of the aggregation alone (staging + zeroing + matrix product of the bit blocks)."""
    from tango_amd import _lib
    L = _lib.lib()
    ld = F if ld is None else ld
    feat = torch.randint(-127, 128, (plan.num_src, ld), dtype=torch.int8, device="cuda")
    nbytes = L.tango_spmm_dense_workspace(plan.ref, F)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    return time_op(lambda: _lib.check(L.tango_spmm_dense_partial(plan.ref, feat.data_ptr(), ld, F, ws.data_ptr(), nbytes, st),
                                      "dense_partial"), iters=iters)


def rest_launch_ms(plan, K, torch, F, ld=None, iters=20):
    """The gather kernel on the rest alone, bracketed by HIP events on its own stream: the dense half runs once
    (its partial sums stay in the workspace), then only tango_spmm_dense_rest is launched and timed."""
    from tango_amd import _lib
    L = _lib.lib()
    ld = F if ld is None else ld
    feat = torch.randint(-127, 128, (plan.num_src, ld), dtype=torch.int8, device="cuda")
    out = torch.empty((plan.rows, F), dtype=torch.float32, device="cuda")
    scale = torch.full((1,), 0.01, device="cuda")
    nbytes = L.tango_spmm_dense_workspace(plan.ref, F)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    _lib.check(L.tango_spmm_dense_partial(plan.ref, feat.data_ptr(), ld, F, ws.data_ptr(), nbytes, st), "dense_partial")
    return time_op(lambda: _lib.check(L.tango_spmm_dense_rest(out.data_ptr(), plan.ref, feat.data_ptr(), ld, scale.data_ptr(),
                                                              None, None, 0, None, F, ws.data_ptr(), nbytes, st),
                                      "dense_rest"), iters=iters)


def permuted_graph(g, torch, seed=11):
    """The same graph with its node ids randomly permuted (the generator numbers nodes by falling degree)."""
    from tango_amd.graph import Graph
    from tango_amd.util import graph_preprocess
    gen = torch.Generator(device="cuda").manual_seed(seed)
    perm = torch.randperm(g.num_nodes(), generator=gen, device="cuda")
    src, dst = g.coo
    return graph_preprocess(Graph(perm[src], perm[dst], g.num_nodes()))


def gather_entry(ms, model_bytes, compulsory_bytes):
    return {"ms": round(ms, 4), "gather_model_GBps": round(model_bytes / ms / 1e6, 1),
            "frac_hbm_compulsory": round(compulsory_bytes / ms / 1e6 / HBM_PEAK_GBPS, 4)}


def primitives(g, K, torch):
    """Per-primitive throughput at the sizes the metric quotes (outside the timed epoch)."""
    out = {}
    n, nnz = g.num_nodes(), g.num_edges()
    one = torch.ones(1, device="cuda") * 0.01
    for F in (16, 64, 128, 256):
        feat = torch.randint(-127, 128, (n, F), dtype=torch.int8, device="cuda")
        ms = time_op(lambda: K.csr_SPMM(g, feat, one), iters=10)
        out["spmm_copy_u_F%d" % F] = gather_entry(ms, spmm_bytes(nnz, n, F), spmm_compulsory_bytes(nnz, n, n, F))
        del feat
    # u_mul_e, broadcast edge value, at the four sizes of evaluation/SPMM_broadcast.py:67-75
    for H, F in ((2, 128), (4, 128), (2, 256), (4, 256)):
        feat = torch.randint(-127, 128, (n, H, F), dtype=torch.int8, device="cuda")
        ev = torch.randint(-127, 128, (H, 1, nnz), dtype=torch.int8, device="cuda")
        ms = time_op(lambda: K.multi_cusparse_SPMM(g, feat, ev, one), iters=5)
        out["spmm_u_mul_e_H%d_F%d" % (H, F)] = gather_entry(ms, nnz * (H * F + H + 2 * IDX_BYTES) + n * (4 * H * F + 8),
                                                            nnz * (H + 2 * IDX_BYTES) + n * (5 * H * F + 8))
        del feat, ev
    # u_mul_e without broadcast: every head has one feature column and its own edge value
    # (evaluation/SPMM_nobroadcast.py:27-29: N [n, H, 1], E [nnz, H, 1]); and the incidence form (copy_e)
    H = 8
    feat = torch.randint(-127, 128, (n, H, 1), dtype=torch.int8, device="cuda")
    ev = torch.randint(-127, 128, (nnz, H, 1), dtype=torch.int8, device="cuda")
    ms = time_op(lambda: K.multi_cusparse_SPMM(g, feat, ev, one, edge_major=True), iters=5)
    out["spmm_u_mul_e_nobroadcast_H8"] = gather_entry(ms, nnz * (H + H + 2 * IDX_BYTES) + n * (4 * H + 8),
                                                      nnz * (H + 2 * IDX_BYTES) + n * (5 * H + 8))
    del feat, ev
    # the incidence form (copy_e) at the widths of evaluation/test_incidence.py:85-86
    for Fw in range(4, 33, 4):
        ev = torch.randint(-127, 128, (nnz, Fw), dtype=torch.int8, device="cuda")
        ms = time_op(lambda: K.incidence_SPMM(g, ev, one), iters=5)
        out["spmm_incidence_F%d" % Fw] = gather_entry(ms, nnz * (Fw + IDX_BYTES) + n * (4 * Fw + 8),
                                                      nnz * (Fw + IDX_BYTES) + n * (4 * Fw + 8))
        del ev
    # SDDMM on this graph at the two sizes of evaluation/SDDMM_test.py:57: add with (1, 16), dot with (4, 64)
    U = torch.randint(-127, 128, (n, 1, 16), dtype=torch.int8, device="cuda")
    ms = time_op(lambda: K.mySDDMM_int8(g, "add", U, U, one, one, False), iters=5)
    out["sddmm_add_H1_F16_114.8Me"] = gather_entry(ms, nnz * (16 + 2 * 16 + 4 * 16), nnz * 16 + 2 * n * 16 + 4 * nnz * 16)
    U = torch.randint(-127, 128, (n, 4, 64), dtype=torch.int8, device="cuda")
    ms = time_op(lambda: K.mySDDMM_int8(g, "dot", U, U, one, one, False), iters=5)
    out["sddmm_dot_H4_D64_114.8Me"] = gather_entry(ms, nnz * (16 + 2 * 4 * 64 + 4 * 4), nnz * 16 + 2 * n * 256 + 4 * nnz * 4)
    del U
    # ten stacked bias-free QLinear layers, forward + backward per layer (evaluation/linear_test.py:11-37)
    import torch.nn as nn
    from tango_amd.QLinear import QLinear
    for width in (256, 512):
        Xs = torch.randn(n, width, device="cuda", requires_grad=True)
        model = nn.Sequential(*[QLinear(width, width, bias=False) for _ in range(10)]).cuda()

        def fwd_bwd():
            model(Xs)[0][0].backward()
        ms = time_op(fwd_bwd, iters=5, warm=2)
        ops = 3 * 2.0 * n * width * width  # forward, gradX, gradW
        out["qlinear_stack10_%dx%d_fwd_bwd_per_layer" % (n, width)] = {"ms": round(ms / 10, 4),
                                                                        "TOPS": round(ops / (ms / 10) / 1e9, 1)}
        del Xs, model
    # QLinear forward / backward at (M, K, N) = (232965, 602, 256) and (232965, 256, 41)
    for (M, Kd, N) in ((n, 602, 256), (n, 256, 41), (n, 128, 16)):
        X = torch.randn(M, Kd, device="cuda")
        W = torch.randn(N, Kd, device="cuda") * 0.05
        sX, sW = K.cuda_kernels.get_scale(X), K.cuda_kernels.get_scale(W)
        ld = (Kd + 15) // 16 * 16
        Xq = torch.empty((M, ld), dtype=torch.int8, device="cuda")[:, :Kd]
        Wq = torch.empty((N, Kd), dtype=torch.int8, device="cuda")
        ms = time_op(lambda: K.QGEMM_forward(X, Xq, sX, W, Wq, sW, None, True), iters=10)
        ops = 2.0 * M * N * Kd
        byt = 5 * (M * Kd + N * Kd) + 4 * M * N
        tag = "qlinear_fwd_%dx%dx%d" % (M, Kd, N)
        out[tag] = {"ms": round(ms, 4), "TOPS": round(ops / ms / 1e9, 2), "GBps": round(byt / ms / 1e6, 1),
                    "frac_hbm": round(byt / ms / 1e6 / HBM_PEAK_GBPS, 4),
                    "frac_i8_mfma": round(ops / ms / 1e9 / 5000.0, 4)}
        dY, s_dY = K.quantize_padded(torch.randn(M, N, device="cuda"))
        ms = time_op(lambda: K.QGEMM_backward(dY, Xq, Wq, s_dY, sX, sW, True, False), iters=10)
        byt = M * N + N * Kd + 4 * M * Kd
        out[tag.replace("fwd", "gradX")] = {"ms": round(ms, 4), "TOPS": round(ops / ms / 1e9, 2),
                                            "GBps": round(byt / ms / 1e6, 1),
                                            "frac_hbm": round(byt / ms / 1e6 / HBM_PEAK_GBPS, 4)}
        ms = time_op(lambda: K.QGEMM_backward(dY, Xq, Wq, s_dY, sX, sW, False, True), iters=10)
        byt = M * (N + Kd) + 4 * N * Kd
        out[tag.replace("fwd", "gradW")] = {"ms": round(ms, 4), "TOPS": round(ops / ms / 1e9, 2),
                                            "GBps": round(byt / ms / 1e6, 1),
                                            "frac_hbm": round(byt / ms / 1e6 / HBM_PEAK_GBPS, 4),
                                            "frac_i8_mfma": round(ops / ms / 1e9 / 5000.0, 4)}
        del X, W, Xq, dY
    # the two call patterns of evaluation/test_cache_GEMM.py and evaluation/test_fuse.py at the first layer's shape:
    # the forward on an input that was quantized once before (several consumers share it), and the output scale
    # from the GEMM's epilogue against a separate absmax pass over Y
    M, Kd, N = n, 256, 256
    X = torch.randn(M, Kd, device="cuda")
    W = torch.randn(N, Kd, device="cuda") * 0.05
    sX, sW = K.cuda_kernels.get_scale(X), K.cuda_kernels.get_scale(W)
    Xq = torch.empty((M, Kd), dtype=torch.int8, device="cuda")
    Wq = torch.empty((N, Kd), dtype=torch.int8, device="cuda")
    t_fused = time_op(lambda: K.QGEMM_forward(X, Xq, sX, W, Wq, sW, None, True), iters=10)
    t_cached = time_op(lambda: K.QGEMM_forward(None, Xq, sX, W, Wq, sW, None, True), iters=10)
    t_plain = time_op(lambda: K.cuda_kernels.get_scale(K.QGEMM_forward(X, Xq, sX, W, Wq, sW, None, False)), iters=10)
    out["qlinear_fwd_%dx%dx%d" % (M, Kd, N)] = {"ms": round(t_fused, 4), "ms_input_already_int8": round(t_cached, 4),
                                                 "ms_with_separate_output_absmax": round(t_plain, 4)}
    del X, W, Xq, Wq
    # quantize / absmax streaming
    X = torch.randn(n, 602, device="cuda")
    ms = time_op(lambda: K.cuda_kernels.get_scale(X))
    out["absmax_140M"] = {"ms": round(ms, 4), "GBps": round(4 * X.numel() / ms / 1e6, 1)}
    s = K.cuda_kernels.get_scale(X)
    q = torch.empty(X.shape, dtype=torch.int8, device="cuda")
    ms = time_op(lambda: K.cuda_kernels.quantize(q, X, s))
    out["quantize_140M"] = {"ms": round(ms, 4), "GBps": round(5 * X.numel() / ms / 1e6, 1)}
    del X, q
    return out


def sddmm_primitives(K, torch):
    """GAT-shaped SDDMM on the 169,343-node / 1.17M-edge graph (8 heads x 16)."""
    from tango_amd.graph import chung_lu
    from tango_amd.util import graph_preprocess
    g = graph_preprocess(chung_lu(169343, 1166243, 2.2, seed=4, device="cuda"))
    n, E, H, D = g.num_nodes(), g.num_edges(), 8, 16
    U = torch.randint(-127, 128, (n, H, D), dtype=torch.int8, device="cuda")
    V = torch.randint(-127, 128, (n, H, D), dtype=torch.int8, device="cuda")
    one = torch.ones(1, device="cuda") * 0.01
    out = {"graph": {"nodes": n, "edges": E}}
    ms = time_op(lambda: K.mySDDMM_int8(g, "dot", U, V, one, one, False))
    out["sddmm_dot_H8_D16"] = gather_entry(ms, E * (16 + 2 * H * D + 4 * H), E * 16 + 2 * n * H * D + 4 * E * H)
    el = torch.randint(-127, 128, (n, H, 1), dtype=torch.int8, device="cuda")
    ms = time_op(lambda: K.mySDDMM_int8(g, "add", el, el, one, one, False))
    out["sddmm_add_H8"] = gather_entry(ms, E * (16 + 2 * H + 4 * H), E * 16 + 2 * n * H + 4 * E * H)
    e = torch.randn(E, H, 1, device="cuda")
    ip, _, eid = g.adj_csc
    ms = time_op(lambda: K.cuda_kernels.edge_softmax_forward(e, ip, eid, 0.2))
    b = E * (8 * H + 8)  # a stream: e read once, a written once, row pointers / edge ids
    out["edge_softmax_H8"] = {"ms": round(ms, 4), "GBps": round(b / ms / 1e6, 1),
                              "frac_hbm": round(b / ms / 1e6 / HBM_PEAK_GBPS, 4)}
    return out


def step_ms(fn, iters, warm):
    """ms per training step: the median of three timed runs of ``iters`` steps (a step of a thousand launches is
    close to host-bound, and one host hiccup in a single run of ten moves its mean by a third)."""
    time_op(fn, iters=1, warm=warm)
    runs = sorted(time_op(fn, iters=iters, warm=0) for _ in range(3))
    return runs[1]


def model_steps(K, torch, which=("gat", "arxiv", "arxiv-gcn", "hgt", "hetero"), iters=10, warm=3):
    """The other model configurations, one training step each (forward + loss + backward + Adam):
    the 3-layer GAT (hidden 16 x 8 heads, evaluation/test_gat.py:170-214) on the 169,343-node graph
    and two HGT layers (256-d, 4 heads) on the homogenised 3-type / 4-relation graph."""
    from tango_amd import config
    config.grad_round_mode = "stochastic"  # as in the epoch: gradients are rounded stochastically (Philox on the device)
    out = {}
    torch.manual_seed(4)
    for name, fn in (("gat", _gat_step), ("arxiv", _arxiv_step), ("arxiv-gcn", _arxiv_gcn_step), ("hgt", _hgt_step),
                     ("hetero", _hetero_step)):
        if name in which:
            out.update(fn(K, torch, iters, warm))
    return out


def _gat_graph(torch):
    from tango_amd.graph import chung_lu
    from tango_amd.util import graph_preprocess
    # edges numbered in destination-major order: the [E, H] tensors of the attention layers are then
    # walked front to back (node outputs do not depend on the numbering)
    g = graph_preprocess(chung_lu(169343, 1166243, 2.2, seed=4, device="cuda").reorder_edges_by_dst())
    return g, torch.randn(g.num_nodes(), 128, device="cuda")


def _gat_step(K, torch, iters, warm):
    from tango_amd.gat import GAT
    from tango_amd.loss import cross_entropy
    g, x = _gat_graph(torch)
    n = g.num_nodes()
    model = GAT(g, 3, 128, 16, 40, [8, 8, 1], torch.nn.functional.elu).cuda()
    labels = torch.randint(0, 16, (n,), device="cuda")
    opt = torch.optim.Adam(model.parameters(), lr=1e-3, fused=True)

    def gat_step():
        opt.zero_grad(set_to_none=True)
        cross_entropy(model(x), labels).backward()
        opt.step()
    return {"gat3_step_169343n_1.34Me_ms": round(step_ms(gat_step, iters, warm), 3)}


def _arxiv_step(K, torch, iters, warm):
    # the stack the reference trains on this graph (evaluation/arxiv_gat.py:376-448): a residual projection in
    # every layer, batch norm between layers, a one-head output layer, the smoothed loss; dropout off
    from tango_amd.evaluation import arxiv_loss
    from tango_amd.gat import ArxivGAT
    g, x = _gat_graph(torch)
    n = g.num_nodes()
    am = ArxivGAT(128, 40, 16, 3, 8, torch.nn.functional.relu).cuda()
    al = torch.randint(0, 40, (n,), device="cuda")
    aopt = torch.optim.RMSprop(am.parameters(), lr=2e-3)

    def arxiv_step():
        aopt.zero_grad(set_to_none=True)
        arxiv_loss(am(g, x), al).backward()
        aopt.step()
    return {"arxiv_gat3_step_169343n_1.34Me_ms": round(step_ms(arxiv_step, iters, warm), 3)}


def _arxiv_gcn_step(K, torch, iters, warm):
    # evaluation/arxiv_gcn.py:156-209 on the same graph: three graph convolutions (hidden 256) with a quantized linear
    # skip branch each, batch norm + ReLU between them; dropout off
    from tango_amd.evaluation import arxiv_loss
    from tango_amd.gcn import ArxivGCN
    g, x = _gat_graph(torch)
    n = g.num_nodes()
    gm = ArxivGCN(128, 256, 40, 3, torch.relu, 0.0, True).cuda()
    gl = torch.randint(0, 40, (n,), device="cuda")
    gopt = torch.optim.Adam(gm.parameters(), lr=5e-3, fused=True)

    def arxiv_gcn_step():
        gopt.zero_grad(set_to_none=True)
        arxiv_loss(gm(g, x), gl).backward()
        gopt.step()
    return {"arxiv_gcn3_step_169343n_1.34Me_ms": round(step_ms(arxiv_gcn_step, iters, warm), 3)}


def _hgt_step(K, torch, iters, warm):
    from tango_amd.gat import HGTStack
    from tango_amd.graph import hetero_power_law
    from tango_amd.loss import cross_entropy
    from tango_amd.util import graph_preprocess
    g, _, _ = hetero_power_law(device="cuda")
    g = graph_preprocess(g.reorder_edges_by_dst())
    n = g.num_nodes()
    hgt = HGTStack(256, 256, 16, 4, n_layers=2).cuda()
    xh = torch.randn(n, 256, device="cuda")
    lh = torch.randint(0, 16, (n,), device="cuda")
    opth = torch.optim.Adam(hgt.parameters(), lr=1e-3, fused=True)

    def hgt_step():
        opth.zero_grad(set_to_none=True)
        cross_entropy(hgt(g, xh), lh).backward()
        opth.step()
    return {"hgt2_step_170000n_8.17Me_ms": round(step_ms(hgt_step, iters, warm), 3)}


def _hetero_step(K, torch, iters, warm):
    # the same graph as a heterogeneous one: weights per node type and per relation, one SDDMM and one aggregation
    # per relation, one softmax over all in-edges
    from tango_amd.gat import HeteroHGTLayer, relation_graphs, relation_major
    from tango_amd.graph import hetero_power_law
    from tango_amd.loss import cross_entropy
    from tango_amd.util import graph_preprocess
    sizes, rels = (100_000, 50_000, 20_000), ((0, 1), (1, 0), (1, 2), (2, 0))
    g2, _, etype = hetero_power_law(type_sizes=sizes, relations=rels, device="cuda")
    g2, etype = relation_major(g2, etype)
    g2 = graph_preprocess(g2)
    rg = relation_graphs(g2, etype, rels, sizes)
    n = g2.num_nodes()
    xh = torch.randn(n, 256, device="cuda")
    lh = torch.randint(0, 16, (n,), device="cuda")
    layers = torch.nn.ModuleList([HeteroHGTLayer(256, 256, 4, sizes, rg) for _ in range(2)]).cuda()
    proj = torch.nn.Linear(256, 16).cuda()
    opt2 = torch.optim.Adam(list(layers.parameters()) + list(proj.parameters()), lr=1e-3, fused=True)

    def hetero_step():
        opt2.zero_grad(set_to_none=True)
        h = xh
        for layer in layers:
            h = layer(g2, h)
        cross_entropy(proj(h), lh).backward()
        opt2.step()
    return {"hetero_hgt2_step_170000n_8.17Me_ms": round(step_ms(hetero_step, iters, warm), 3)}


def cpu_baseline(g, X, W1, W2, frac, reps=3):
    """The CPU oracle (a port of the reference's semantics, OpenMP over the host
    cores) on every k-th destination row / node of the same workload:
    forward GEMM+aggregation of both layers and the backward aggregations and
    GEMMs, i.e. the primitives of one epoch.  Returns (epoch-equivalent ms, note)."""
    import numpy as np
    from oracle import oracle as orc
    n = g.num_nodes()
    stride = max(1, int(round(1.0 / frac)))
    rows = np.arange(0, n, stride)
    threads = len(os.sched_getaffinity(0))
    orc.set_num_threads(threads)

    def sub_csr(fmt):
        ip, ix, _ = fmt
        ip, ix = ip.cpu().numpy(), ix.cpu().numpy()
        starts, ends = ip[rows], ip[rows + 1]
        lens = ends - starts
        sip = np.zeros(rows.size + 1, np.int64)
        np.cumsum(lens, out=sip[1:])
        take = np.repeat(starts - sip[:-1], lens) + np.arange(sip[-1])
        return sip, ix[take]

    csc, csr = sub_csr(g.adj_csc), sub_csr(g.adj_csr)
    Xs = X[rows].cpu().numpy()
    W1n, W2n = W1.cpu().numpy(), W2.cpu().numpy()
    rng = np.random.default_rng(0)
    # int8 node features to gather from: the quantized layer outputs themselves when every row is run (set inside
    # the loop below), stand-ins of the same shape when only a sample of the rows is
    f1 = rng.integers(-127, 128, (n, 256)).astype(np.int8)
    f2 = rng.integers(-127, 128, (n, 41)).astype(np.int8)
    dY1 = rng.standard_normal((rows.size, 256)).astype(np.float32)  # upstream gradients (inputs, not timed)
    dY2 = rng.standard_normal((rows.size, 41)).astype(np.float32)
    times = []
    for _ in range(max(1, reps)):
        t0 = time.perf_counter()
        # layer 1 forward: GEMM (quantize fused) then aggregation of 256-wide rows
        Y1, Xq, W1q, sX, sW1, sY1 = orc.qgemm_fwd(Xs, W1n, reduce=True)
        Y1q = orc.quantize(Y1, sY1)
        agg1 = orc.spmm_csr_copy_u(csc[0], csc[1], Y1q if stride == 1 else f1, sY1)
        # layer 2 forward
        H1 = np.maximum(agg1, 0)
        Y2, Hq, W2q, sH, sW2, sY2 = orc.qgemm_fwd(H1, W2n, reduce=True)
        Y2q = orc.quantize(Y2, sY2)
        orc.spmm_csr_copy_u(csc[0], csc[1], Y2q if stride == 1 else f2, sY2)
        # backward: aggregation of dZ on the reverse graph, then gradX / gradW, both layers
        orc.spmm_csr_copy_u(csr[0], csr[1], f2, 0.01)
        s2 = orc.absmax_scale(dY2)
        dY2q = orc.quantize(dY2, s2)
        orc.qgemm_bwd_dx(dY2q, W2q, s2, sW2)
        orc.qgemm_bwd_dw(dY2q, Hq, s2, sH)
        orc.spmm_csr_copy_u(csr[0], csr[1], f1, 0.01)
        s1 = orc.absmax_scale(dY1)
        dY1q = orc.quantize(dY1, s1)
        orc.qgemm_bwd_dw(dY1q, Xq, s1, sX)
        times.append(time.perf_counter() - t0)
    dt = sorted(times)[len(times) // 2]
    note = ("oracle port, OpenMP x%d, primitives of one epoch on every %dth node/destination row "
            "(%d rows, %d edges), median of %d runs, %.1f s each, scaled by %d"
            % (threads, stride, rows.size, int(csc[0][-1]), len(times), dt, stride))
    return dt * 1000.0 * stride, threads, note


def cpu_fp32_torch(g, X, W1, W2, labels, frac, reps=5):
    """What the reference's scripts compare against, on the host cores, in fp32: the aggregation (sparse CSR @ dense,
    256 wide) and nn.functional.linear (602 -> 256), one warm-up and the median of ``reps`` runs each, and one epoch
    of the same 2-layer GCN math (evaluation/test_gcn.py:67-139: forward, cross-entropy, backward written out with
    the reverse aggregation as a second CSR) as the median of three runs after a warm-up.  On every k-th
    destination row, scaled to the full size, when ``frac`` < 1."""
    import torch
    n = g.num_nodes()
    stride = max(1, int(round(1.0 / frac)))
    rows = torch.arange(0, n, stride)

    def sub_csr(fmt):
        ip, ix = fmt[0].cpu(), fmt[1].cpu()
        starts, ends = ip[rows], ip[rows + 1]
        lens = ends - starts
        sip = torch.zeros(rows.numel() + 1, dtype=torch.int64)
        torch.cumsum(lens, 0, out=sip[1:])
        take = torch.repeat_interleave(starts - sip[:-1], lens) + torch.arange(int(sip[-1]))
        return torch.sparse_csr_tensor(sip, ix[take], torch.ones(int(sip[-1])), size=(rows.numel(), n))

    def median_ms(fn, k):
        fn()
        t = []
        for _ in range(k):
            t0 = time.perf_counter()
            fn()
            t.append(time.perf_counter() - t0)
        return sorted(t)[len(t) // 2] * 1e3 * stride

    A, At = sub_csr(g.adj_csc), sub_csr(g.adj_csr)
    dense = torch.randn(n, 256)
    Xc, W1c, W2c, lab = X.cpu(), W1.cpu(), W2.cpu(), labels.cpu()
    Xs = Xc[rows]
    out = {"spmm_F256_ms": round(median_ms(lambda: A @ dense, reps), 1),
           "linear_602x256_ms": round(median_ms(lambda: torch.nn.functional.linear(Xs, W1c), reps), 1)}
    ns = g.out_degrees().float().clamp(min=1).pow(-0.5).cpu().unsqueeze(1)
    nd = g.in_degrees().float().clamp(min=1).pow(-0.5).cpu().unsqueeze(1)

    def epoch():
        if stride != 1:  # the sampled rows cannot feed a second layer: run the two layers' primitives on stand-ins
            y1 = A @ dense
            A @ dense[:, :41]
            At @ dense[:, :41]
            At @ dense
            torch.nn.functional.linear(Xs, W1c)
            return y1
        y1 = torch.nn.functional.linear(Xc * ns, W1c)
        h1 = torch.relu((A @ y1) * nd)
        y2 = torch.nn.functional.linear(h1 * ns, W2c)
        logits = (A @ y2) * nd
        p = torch.softmax(logits, 1)
        p[torch.arange(n), lab] -= 1.0
        dz2 = (p / n) * nd
        dy2 = At @ dz2
        dW2 = dy2.t() @ (h1 * ns)
        dh1 = (dy2 @ W2c) * ns
        dz1 = (dh1 * (h1 > 0)) * nd
        dy1 = At @ dz1
        dW1 = dy1.t() @ (Xc * ns)
        return dW1, dW2

    out["gcn_epoch_ms"] = round(median_ms(epoch, 3), 1)
    out["threads"] = torch.get_num_threads()
    out["cores"] = len(os.sched_getaffinity(0))
    out["sample"] = ("one warm-up, median of %d (primitives) / 3 (epoch) runs; every %dth row, scaled by %d"
                     % (reps, stride, stride))
    return out


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    import torch
    from tango_amd import config, kernels as K
    from tango_amd.gcn import GCN
    from tango_amd.graph import chung_lu
    from tango_amd.loss import cross_entropy
    from tango_amd.util import graph_preprocess

    torch.cuda.set_device(0)
    if args.profile_mode == "copy":
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"profile_mode": "copy", "bytes_read": src.numel() * 4, "bytes_written": src.numel() * 4}))
        return
    if args.profile_mode == "mfma":
        print(json.dumps(dict(mfma_probe(torch), profile_mode="mfma")))
        return
    if args.profile_mode in ("gat", "arxiv", "arxiv-gcn", "hgt", "hetero"):  # one training step of the attention models, for kernel traces
        out = model_steps(K, torch, which=(args.profile_mode,), iters=args.steps, warm=args.warmup)
        print(json.dumps(dict(out, profile_mode=args.profile_mode)))
        return
    if args.profile_mode == "qlinear":  # the forward GEMM of layer 1, fp32 in, Xq cached, fp32 out + scale
        M, Kd, N = args.nodes, 602, 256
        X = torch.randn(M, Kd, device="cuda")
        W = torch.randn(N, Kd, device="cuda") * 0.05
        sX, sW = K.cuda_kernels.get_scale(X), K.cuda_kernels.get_scale(W)
        Xq = torch.empty((M, 608), dtype=torch.int8, device="cuda")[:, :Kd]
        Wq = torch.empty((N, Kd), dtype=torch.int8, device="cuda")
        ms = time_op(lambda: K.QGEMM_forward(X, Xq, sX, W, Wq, sW, None, True), iters=args.steps, warm=args.warmup)
        print(json.dumps({"profile_mode": "qlinear", "M": M, "K": Kd, "N": N, "avg_ms": round(ms, 4),
                          "ops": 2 * M * N * Kd, "algorithmic_bytes": 5 * (M * Kd + N * Kd) + 4 * M * N + 4 * N}))
        return
    if args.profile_mode in ("gradx", "gradw"):
        # gradX: int8 dY [M, N] -> fp32 dX [M, K] (default shape: the epoch's second layer);
        # gradW: int8 dY [M, N] and int8 X [M, K] -> fp32 dW [N, K]
        Kd, N = (int(v) for v in args.gemm_shape.split(","))
        M = args.nodes
        dY, s_dY = K.quantize_padded(torch.randn(M, N, device="cuda"))
        Wq, sW = K.quantize(torch.randn(N, Kd, device="cuda") * 0.05)
        ld = (Kd + 15) // 16 * 16
        Xq = torch.randint(-127, 128, (M, ld), dtype=torch.int8, device="cuda")[:, :Kd]
        sX = torch.ones(1, device="cuda")
        dx = args.profile_mode == "gradx"
        ms = time_op(lambda: K.QGEMM_backward(dY, Xq, Wq, s_dY, sX, sW, dx, not dx), iters=args.steps, warm=args.warmup)
        byt = M * N + N * Kd + 4 * M * Kd if dx else M * (N + Kd) + 4 * N * Kd
        print(json.dumps({"profile_mode": args.profile_mode, "M": M, "K": Kd, "N": N, "avg_ms": round(ms, 4),
                          "ops": 2 * M * N * Kd, "algorithmic_bytes": byt}))
        return
    if args.profile_mode == "umule":  # the attention layers' aggregation (u_mul_e, edge-major int8 edge values) and SDDMM dot
        from tango_amd.graph import hetero_power_law
        if args.attn_graph == "gat":
            g4, H, D = chung_lu(169343, 1166243, 2.2, seed=4, device="cuda"), 8, 16
        else:
            g4, H, D = hetero_power_law(device="cuda")[0], 4, 64
        g4 = graph_preprocess(g4.reorder_edges_by_dst())
        n4, E = g4.num_nodes(), g4.num_edges()
        feat = torch.randint(-127, 128, (n4, H, D), dtype=torch.int8, device="cuda")
        ev = torch.randint(-127, 128, (E, H, 1), dtype=torch.int8, device="cuda")
        one = torch.full((1,), 0.01, device="cuda")
        ms = time_op(lambda: K.multi_cusparse_SPMM(g4, feat, ev, one, edge_major=True), iters=args.steps, warm=args.warmup)
        ms_d = time_op(lambda: K.mySDDMM_int8(g4, "dot", feat, feat, one, one, False), iters=args.steps, warm=args.warmup)
        print(json.dumps({"profile_mode": "umule", "graph": args.attn_graph, "nodes": n4, "edges": E, "H": H, "D": D,
                          "u_mul_e_ms": round(ms, 4), "sddmm_dot_ms": round(ms_d, 4),
                          "u_mul_e_gather_model_bytes": E * (H * D + H + 2 * IDX_BYTES) + n4 * (4 * H * D + 8),
                          "u_mul_e_compulsory_bytes": E * (H + 2 * IDX_BYTES) + n4 * (5 * H * D + 8),
                          "sddmm_gather_model_bytes": E * (16 + 2 * H * D + 4 * H),
                          "sddmm_compulsory_bytes": E * 16 + 2 * n4 * H * D + 4 * E * H}))
        return
    if args.profile_mode == "softmax":  # edge softmax forward / backward, 8 heads, on the 169,343-node graph
        g4 = graph_preprocess(chung_lu(169343, 1166243, 2.2, seed=4, device="cuda").reorder_edges_by_dst())
        E, H = g4.num_edges(), 8
        e = torch.randn(E, H, 1, device="cuda")
        ip, _, eid = g4.adj_csc
        ms_f = time_op(lambda: K.cuda_kernels.edge_softmax_forward(e, ip, eid, 0.2), iters=args.steps, warm=args.warmup)
        a = K.cuda_kernels.edge_softmax_forward(e, ip, eid, 0.2)
        da = torch.randn_like(a)
        ms_b = time_op(lambda: K.cuda_kernels.edge_softmax_backward(a, da, e, ip, eid, 0.2), iters=args.steps, warm=args.warmup)
        print(json.dumps({"profile_mode": "softmax", "edges": E, "H": H, "fwd_ms": round(ms_f, 4), "bwd_ms": round(ms_b, 4),
                          "fwd_bytes": E * (8 * H + 8), "bwd_bytes": E * (16 * H + 8)}))
        return
    if args.profile_mode == "quantize":
        X = torch.randn(args.nodes, 602, device="cuda")
        s = K.cuda_kernels.get_scale(X)
        q = torch.empty(X.shape, dtype=torch.int8, device="cuda")
        ms = time_op(lambda: K.cuda_kernels.quantize(q, X, s), iters=args.steps, warm=args.warmup)
        ms_a = time_op(lambda: K.cuda_kernels.get_scale(X), iters=args.steps, warm=args.warmup)
        print(json.dumps({"profile_mode": "quantize", "elements": X.numel(), "quantize_ms": round(ms, 4),
                          "absmax_ms": round(ms_a, 4), "quantize_bytes": 5 * X.numel(), "absmax_bytes": 4 * X.numel()}))
        return
    if args.profile_mode == "sddmm":
        g4 = graph_preprocess(chung_lu(169343, 1166243, 2.2, seed=4, device="cuda"))
        n4, E, H, D = g4.num_nodes(), g4.num_edges(), 8, 16
        U = torch.randint(-127, 128, (n4, H, D), dtype=torch.int8, device="cuda")
        V = torch.randint(-127, 128, (n4, H, D), dtype=torch.int8, device="cuda")
        one = torch.full((1,), 0.01, device="cuda")
        ms = time_op(lambda: K.mySDDMM_int8(g4, "dot", U, V, one, one, False), iters=args.steps, warm=args.warmup)
        print(json.dumps({"profile_mode": "sddmm", "nodes": n4, "edges": E, "H": H, "D": D, "avg_ms": round(ms, 4),
                          "algorithmic_bytes": E * (16 + 2 * H * D + 4 * H),
                          "compulsory_bytes": E * 16 + 2 * n4 * H * D + 4 * E * H}))
        return
    t0 = time.perf_counter()
    g = graph_preprocess(chung_lu(args.nodes, args.edges, 2.0, seed=3, max_degree=21000, symmetric=True,
                                  device="cuda"), dense_blocks=not (args.no_dense or args.l2_window))
    torch.cuda.synchronize()
    n, nnz = g.num_nodes(), g.num_edges()
    max_deg = int(g.in_degrees().max().item())
    sys.stderr.write("graph: %d nodes, %d directed edges, max in-degree %d (%.1f s)\n"
                     % (n, nnz, max_deg, time.perf_counter() - t0))

    if args.profile_mode == "spmm":
        if args.l2_window:
            ms = folded_spmm_ms(g, K, torch, F=args.feat, iters=args.steps)
            print(json.dumps({"profile_mode": "spmm", "l2_window": True, "F": args.feat, "nodes": n, "edges": nnz,
                              "avg_ms": round(ms, 4), "requests": nnz * ((args.feat + 127) // 128)}))
            return
        if args.permute_ids:
            g = permuted_graph(g, torch) if not args.no_dense else graph_preprocess(
                permuted_graph(g, torch), dense_blocks=False)
        ld = (args.feat + 63) // 64 * 64 if args.feat % 16 else args.feat
        feat = torch.randint(-127, 128, (n, ld), dtype=torch.int8, device="cuda")[:, :args.feat]
        one = torch.full((1,), 0.01, device="cuda")
        ms = time_op(lambda: K.csr_SPMM(g, feat, one), iters=args.steps, warm=args.warmup)
        plan = g.dense_csc
        info = {"profile_mode": "spmm", "F": args.feat, "nodes": n, "edges": nnz, "avg_ms": round(ms, 4),
                "permuted_ids": bool(args.permute_ids), "gather_model_bytes": spmm_bytes(nnz, n, args.feat),
                "compulsory_bytes": spmm_compulsory_bytes(nnz, n, n, args.feat), "dense_blocks": plan is not None}
        if plan is not None:
            info.update({"dense_cells": plan.cells, "rest_edges": plan.res_indices.numel(),
                         "dense_part_ms": round(dense_part_ms(plan, K, torch, args.feat, ld), 4)})
        print(json.dumps(info))
        return

    gen = torch.Generator().manual_seed(5)
    X = torch.randn(n, 602, generator=gen).cuda()
    labels = torch.randint(0, 41, (n,), generator=gen).cuda()
    torch.manual_seed(5)
    model = GCN(g, 602, 256, 41, 1, torch.relu, 0.0).cuda()
    opt = torch.optim.Adam(model.parameters(), lr=1e-2, weight_decay=5e-4, fused=True)  # one kernel for all parameters
    config.grad_round_mode = "stochastic"

    timer = KernelTimer()
    raw_spmm = K.cuda_kernels.csr_SPMM
    K.cuda_kernels.csr_SPMM = staticmethod(timer.wrap(
        raw_spmm, lambda out, *a, **kw: "spmm_F%d" % (out.size(1))))
    raw_dense = K.cuda_kernels.csr_SPMM_dense
    K.cuda_kernels.csr_SPMM_dense = staticmethod(timer.wrap(
        raw_dense, lambda out, *a, **kw: "spmm_F%d" % (out.size(1))))

    def step():
        loss = cross_entropy(model(X), labels)
        opt.zero_grad(set_to_none=True)
        loss.backward()
        opt.step()
        return loss

    for _ in range(args.warmup):
        step()
    timer.clear()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t1) * 1000.0 / args.steps
    K.cuda_kernels.csr_SPMM = staticmethod(raw_spmm)
    K.cuda_kernels.csr_SPMM_dense = staticmethod(raw_dense)

    # Dominant kernel: the gather kernel of the 256-wide copy_u aggregation (forward and reverse launches), which
    # walks what is left of the adjacency after its dense bit blocks went to the matrix cores
    # (tango_spmm_csr_copy_u_dense = staging + dense_block_kernel + this kernel).  The whole call is timed with
    # HIP events inside the epochs; the dense part is timed alone right after them (same shapes), and the
    # difference is the gather kernel's launch time (profiles/gcn_epoch_kernel_trace.md has rocprofv3's figure
    # for the same kernel).  What binds it is not HBM: the int8 features stay in the Infinity Cache, a gathered
    # 128-byte row piece is one L2 -> L1 line, and the misses of the 4 MB L2s are refilled over the fabric, which
    # is the limit it sits at.  `achieved` is therefore the traffic measured beyond the L2s (rocprofv3 FETCH_SIZE
    # + WRITE_SIZE of this kernel, committed summary) over the launch time, priced against the 8 TB/s memory-side
    # peak the contract names; the gather-traffic model (every gathered byte counted per edge) is reported beside
    # it as an effective rate without a fraction, since the caches serve most of it.
    op_ms = timer.mean_ms("spmm_F256")
    plan = g.dense_csc
    consts = counter_constants() if (args.nodes, args.edges) == (232965, 114_600_000) else {}
    dense_ms = dense_part_ms(plan, K, torch, 256) if plan is not None else 0.0
    # the kernel's own launches between HIP events; the call minus the dense part timed alone is kept beside it
    # (it comes out a few per cent lower: the dense part runs faster inside the epoch than in a loop of its own)
    k_ms = rest_launch_ms(plan, K, torch, 256) if plan is not None else op_ms
    derived_ms = op_ms - dense_ms
    rest = plan.res_indices.numel() if plan is not None else nnz
    alg = spmm_bytes(rest, n, 256)
    comp = spmm_compulsory_bytes(rest, n, n, 256)
    traffic = consts.get("traffic_bytes_per_launch")
    folded_ms = folded_spmm_ms(g, K, torch) if not args.no_primitives else None
    floor_ms = folded_ms * rest / nnz if folded_ms else None
    achieved = traffic / k_ms / 1e6 if traffic else None
    probe = mfma_probe(torch)
    roofline = {"kernel": consts.get("kernel", "spmm_quad_kernel<4> on the rest of the adjacency, F=256"),
                "bound": "hbm", "served_from": "infinity cache (the L2 misses are refilled over the fabric, not from HBM)",
                "achieved": round(achieved, 1) if achieved else None, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBPS, 4) if achieved else None, "traffic": traffic,
                "achieved_basis": "measured bytes beyond L2 per launch (FETCH_SIZE + WRITE_SIZE of the gather kernel, "
                                  "profiles/spmm_copy_u_F256_counters.md) / avg_launch_ms",
                "binding_limit": "refills of the L2 misses over the fabric (half of the gathers hit the 4 MB L2s); "
                                 "with every gather hitting, the L2 request rate (one 128-byte line per gathered row piece)",
                "avg_launch_ms": round(k_ms, 4), "launches_timed": 20 if plan is not None else len(timer.spans.get("spmm_F256", [])),
                "avg_launch_basis": "HIP events around tango_spmm_dense_rest (this kernel alone, the blocks' sums already in the workspace)",
                "aggregation_call_ms": round(op_ms, 4), "aggregation_calls_timed": len(timer.spans.get("spmm_F256", [])),
                "dense_part_ms": round(dense_ms, 4), "call_minus_dense_part_ms": round(derived_ms, 4),
                "rest_edges": rest, "rest_share": round(rest / nnz, 4),
                "l2_all_hit_launch_ms": round(floor_ms, 4) if floor_ms else None,
                "l2_all_hit_basis": "the gather kernel on the whole adjacency with all column indices folded into a 4 MB "
                                    "window, measured in this run, scaled by the rest's share of the slots",
                "frac_l2_floor": round(floor_ms / k_ms, 4) if floor_ms else None,
                "compulsory_bytes": comp, "frac_hbm_compulsory": round(comp / k_ms / 1e6 / HBM_PEAK_GBPS, 4),
                "model": {"name": "gather traffic of the rest (cache-served)", "bytes": alg, "index_bytes": IDX_BYTES,
                          "effective_GBps": round(alg / k_ms / 1e6, 1)}}
    if plan is not None:
        ops = 2.0 * plan.cells * 256
        block_ms = consts.get("dense_block_ms")  # rocprofv3 kernel trace; dense_part_ms also holds staging and zeroing
        roofline["dense_blocks"] = {
            "kernel": "dense_block_kernel<4,2,4> (v_mfma_i32_32x32x32_i8, bits expanded to 0/1 bytes)", "bound": "mfma",
            "cells": plan.cells, "ops": ops, "part_ms": round(dense_ms, 4),
            "TOPS": round(ops / dense_ms / 1e9, 1), "peak_TOPS": 5000.0, "frac": round(ops / dense_ms / 1e9 / 5000.0, 4),
            "kernel_trace_ms": block_ms,
            "probe_TOPS": probe["i8_32x32x32_TOPS"], "frac_of_probe": round(ops / dense_ms / 1e9 / probe["i8_32x32x32_TOPS"], 4)}
    roofline["mfma_i8_probe"] = probe

    result = {
        "metric": "quant GCN epoch ms @233K nodes/114.6M edges; SpMM/SDDMM GB/s; QLinear TOPS",
        "value": round(ms_per_step, 3), "unit": "ms/epoch", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 3), "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "int8",
        "data": "synthetic",
        "config": {"workload": "2-layer quantized GCN 602->256->41 training epoch (fwd+loss+bwd+Adam), "
                               "Chung-Lu graph gamma=2.0 seed=3 symmetric + self loops",
                   "nodes": n, "edges": nnz, "max_in_degree": max_deg, "grad_rounding": "stochastic",
                   "loss": round(float(loss.item()), 4)},
        "roofline": roofline,
    }
    result["spmm_F41_ms"] = timer.mean_ms("spmm_F41")

    if not args.no_primitives:
        prims = primitives(g, K, torch)
        prims.update(sddmm_primitives(K, torch))
        prims.update(model_steps(K, torch))
        result["primitives"] = prims
        # sensitivity: the same aggregation with the node ids randomly permuted (hub rows scattered over the
        # feature matrix instead of contiguous at its top)
        gp = permuted_graph(g, torch)
        feat = torch.randint(-127, 128, (n, 256), dtype=torch.int8, device="cuda")
        one = torch.full((1,), 0.01, device="cuda")
        prims["spmm_copy_u_F256_permuted_ids"] = {"ms": round(time_op(lambda: K.csr_SPMM(gp, feat, one), iters=10), 4)}
        del gp, feat
        result["spmm_gather_model_GBps"] = prims["spmm_copy_u_F256"]["gather_model_GBps"]
        result["sddmm_gather_model_GBps"] = prims["sddmm_dot_H8_D16"]["gather_model_GBps"]
        result["qlinear_TOPS"] = prims["qlinear_fwd_%dx602x256" % n]["TOPS"]

    if not args.no_cpu:
        W1 = model.layers[0].weight.detach()
        W2 = model.layers[1].weight.detach()
        ms, cores, note = cpu_baseline(g, X, W1, W2, args.cpu_fraction, args.cpu_reps)
        result["cpu_baseline"] = {"value": round(ms, 1), "unit": "ms/epoch", "cores": cores, "kind": "port",
                                  "sample": note}
        result["cpu_fp32_torch"] = cpu_fp32_torch(g, X, W1, W2, labels, args.cpu_fraction)
    print(json.dumps(result))
    if args.emit:
        try:
            with open(args.emit) as f:
                doc = json.load(f)
        except (OSError, ValueError):
            doc = {}
        doc["measured_mi355x"] = result
        with open(args.emit, "w") as f:
            json.dump(doc, f, indent=2)
            f.write("\n")


if __name__ == "__main__":
    main()
