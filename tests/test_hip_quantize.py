"""GPU parity: absmax / quantize / transpose_quant kernels vs the CPU oracle (bit-exact)."""
import numpy as np
import pytest
import torch

from gpu_util import dev, host, sc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    from tango_amd import kernels
    return kernels


@pytest.mark.parametrize("n", [1, 3, 4, 5, 1023, 65536, 65537, 1000003, 4 * 1048576 + 2])
def test_get_scale(K, orc, n):
    rng = np.random.default_rng(n)
    x = rng.standard_normal(n).astype(np.float32)
    x[-1] = 9.5 if n % 2 else -9.5  # maximum in the tail element
    assert host(K.cuda_kernels.get_scale(dev(x)))[0] == orc.absmax_scale(x)


def test_get_scale_misaligned_view_and_zero(K, orc):
    rng = np.random.default_rng(0)
    x = rng.standard_normal(300001).astype(np.float32)
    t = dev(x)
    for off in (1, 2, 3):
        assert host(K.cuda_kernels.get_scale(t[off:]))[0] == orc.absmax_scale(x[off:])
    assert host(K.cuda_kernels.get_scale(torch.zeros(100000, device="cuda")))[0] == 0.0
    # stale contents of the output slot must not leak: call twice on shrinking data
    big = K.cuda_kernels.get_scale(dev(x * 100))
    small = K.cuda_kernels.get_scale(dev(x))
    assert host(small)[0] == orc.absmax_scale(x) and host(big)[0] > host(small)[0]


def test_get_scale_rows(K, orc):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((1000, 41)).astype(np.float32)
    assert np.array_equal(host(K.cuda_kernels.get_scale_rows(dev(x))), orc.absmax_rows(x))
    wide = rng.standard_normal((50, 700)).astype(np.float32)
    view = dev(wide)[:, :602]
    assert np.array_equal(host(K.cuda_kernels.get_scale_rows(view)), orc.absmax_rows(wide[:, :602]))


@pytest.mark.parametrize("mode", ["rne", "trunc"])
@pytest.mark.parametrize("n", [1, 2, 3, 7, 4096, 100003, 232965 * 41])
def test_quantize_deterministic(K, orc, mode, n):
    rng = np.random.default_rng(n + 5)
    x = rng.standard_normal(n).astype(np.float32)
    s = orc.absmax_scale(x)
    q, s_dev = K.quantize(dev(x), round_mode=mode)
    assert host(s_dev)[0] == s
    assert np.array_equal(host(q), orc.quantize(x, s, orc.RNE if mode == "rne" else orc.TRUNC))


def test_quantize_ties_clamp_and_zero_scale(K, orc):
    x = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.5, 300.0, -300.0, 0.0, 0.49999997,
                  np.inf, -np.inf, np.nan, 1e-30], np.float32)
    for mode, om in (("rne", orc.RNE), ("trunc", orc.TRUNC)):
        q, _ = K.quantize(dev(x), sc(1.0), round_mode=mode)
        assert np.array_equal(host(q), orc.quantize(x, 1.0, om))
    q, _ = K.quantize(torch.zeros(37, device="cuda"))
    assert not host(q).any()
    # misaligned views take the scalar kernel
    y = np.random.default_rng(3).standard_normal(5003).astype(np.float32)
    q, s = K.quantize(dev(y)[1:])
    assert np.array_equal(host(q), orc.quantize(y[1:], host(s)[0]))


@pytest.mark.parametrize("n,offset", [(5, 0), (100003, 0), (100003, 4096), (100003, 3), (1 << 20, (1 << 34) + 1)])
def test_quantize_stochastic(K, orc, n, offset):
    rng = np.random.default_rng(n)
    x = rng.standard_normal(n).astype(np.float32)
    s = orc.absmax_scale(x)
    u = rng.random(n, dtype=np.float32)
    q, _ = K.quantize(dev(x), sc(s), round_mode="stochastic", noise=dev(u))
    assert np.array_equal(host(q), orc.quantize(x, s, orc.STOCHASTIC, noise=u))
    q, _ = K.quantize(dev(x), sc(s), round_mode="stochastic", seed=0xDEADBEEFCAFE, offset=offset)
    assert np.array_equal(host(q), orc.quantize(x, s, orc.STOCHASTIC, seed=0xDEADBEEFCAFE, offset=offset))


def test_stochastic_unbiased_native_rng(K):
    x = torch.randn(1 << 22, device="cuda", generator=torch.Generator("cuda").manual_seed(1))
    q, s = K.quantize(x, round_mode="stochastic", seed=99)
    err = (q.double() * s.double() - x.double()).mean().item()
    assert abs(err) < 1e-3
    q2, _ = K.quantize(x, round_mode="stochastic", seed=100)
    assert not torch.equal(q, q2)


def test_quantize_rows_padded(K, orc):
    rng = np.random.default_rng(4)
    for rows, cols, ld in ((1000, 41, 48), (333, 41, 41), (64, 602, 608), (17, 3, 16)):
        x = rng.standard_normal((rows, cols)).astype(np.float32)
        s = orc.absmax_scale(x)
        out = torch.full((rows, ld), 77, dtype=torch.int8, device="cuda")
        K.cuda_kernels.quantize_rows(out, dev(x), sc(s))
        assert np.array_equal(host(out), orc.quantize_rows(x, s, False, ldq=ld))
        sr = orc.absmax_rows(x)
        K.cuda_kernels.quantize_rows(out, dev(x), dev(sr), per_row=True, round_mode="trunc")
        assert np.array_equal(host(out), orc.quantize_rows(x, sr, True, ldq=ld, mode=orc.TRUNC))
        K.cuda_kernels.quantize_rows(out, dev(x), sc(s), round_mode="stochastic", seed=5, offset=8)
        assert np.array_equal(host(out), orc.quantize_rows(x, s, False, ldq=ld, mode=orc.STOCHASTIC, seed=5, offset=8))


@pytest.mark.parametrize("rows,cols", [(3001, 41), (2000, 602), (70001, 3), (1601, 41)])
@pytest.mark.parametrize("rowmul", [False, True])
def test_quantize_dense_rows_of_odd_width(K, orc, rows, cols, rowmul):
    """Dense inputs whose rows do not hold a multiple of four columns, quantized into padded rows: the flat walk
    (16-byte loads, a lane's four elements in up to two rows, one Philox block per lane) for inputs of at least
    65,536 elements, the row-strided kernel below that; every rounding mode, the random stream at an aligned and
    at an unaligned offset, injected noise, the row multiplier; the padding must come back as zeros."""
    rng = np.random.default_rng(rows + cols)
    x = (rng.standard_normal((rows, cols)) * 3).astype(np.float32)
    rm = (rng.random(rows).astype(np.float32) + 0.5) if rowmul else None
    s = orc.absmax_ex(x, row_mul=rm)[0] if rowmul else orc.absmax_scale(x)
    ld = (cols + 15) // 16 * 16
    noise = rng.random((rows, cols)).astype(np.float32)
    cases = [("rne", {}, dict(mode=orc.RNE)), ("trunc", {}, dict(mode=orc.TRUNC)),
             ("stochastic", dict(seed=7, offset=0), dict(mode=orc.STOCHASTIC, seed=7, offset=0)),
             ("stochastic", dict(seed=7, offset=4 * 10 ** 6 + 5), dict(mode=orc.STOCHASTIC, seed=7, offset=4 * 10 ** 6 + 5)),
             ("stochastic", dict(noise=dev(noise)), dict(mode=orc.STOCHASTIC, noise=noise))]
    for mode, kw, okw in cases:
        q, _ = K.quantize_padded(dev(x), sc(s), round_mode=mode, row_mul=None if rm is None else dev(rm), **kw)
        want = orc.quantize_rows_ex(x, s, row_mul=rm, ldq=ld, **okw)
        full = host(q._base) if q._base is not None else host(q)
        assert np.array_equal(full[:, :cols], want[:, :cols]), (mode, kw.keys())
        assert not full[:, cols:].any()


@pytest.mark.parametrize("shape", [(1335586, 8, 1), (1001, 4, 1), (77, 2, 3), (4096, 1, 1), (5, 64, 4)])
def test_transpose_quant(K, orc, shape):
    rng = np.random.default_rng(6)
    e = rng.random(shape, dtype=np.float32)
    s = orc.absmax_scale(e)
    got = K.transpose_quant(dev(e), sc(s))
    assert tuple(got.shape) == (shape[1], shape[2], shape[0])
    assert np.array_equal(host(got).reshape(shape[1] * shape[2], shape[0]), orc.transpose_quant(e, s))


def test_absmax_accumulating_form(K, orc):
    """tango_absmax_acc_f32 maxes into a slot that holds 0 or a partial result; the Python layer hands it
    pre-zeroed pool slots, which must never be handed out twice."""
    from tango_amd._lib import lib, check
    L = lib()
    rng = np.random.default_rng(11)
    a = rng.standard_normal(300001).astype(np.float32)
    b = (rng.standard_normal(77) * 9).astype(np.float32)
    slot = torch.zeros(1, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    for t in (dev(a), dev(b), dev(a[:3])):
        check(L.tango_absmax_acc_f32(t.data_ptr(), t.numel(), slot.data_ptr(), st), "acc")
    assert host(slot)[0] == max(orc.absmax_scale(a), orc.absmax_scale(b))
    x = dev(a)
    s1, s2 = K.cuda_kernels.get_scale(x), K.cuda_kernels.get_scale(x * 2)
    assert s1.data_ptr() != s2.data_ptr()
    assert host(s1)[0] == orc.absmax_scale(a) and host(s2)[0] == orc.absmax_scale(a * 2)
    s3, _ = K.cuda_kernels.absmax_ex(x.view(-1, 1)[:300000].view(3000, 100))
    assert host(s3)[0] == orc.absmax_scale(a[:300000])


def test_device_resident_stream_position_advances_on_graph_replay(K, orc):
    """Stochastic rounding whose position in the random stream lives in device memory: the kernel adds the word
    to its offset and a one-thread kernel advances it afterwards, so every replay of a captured quantize draws
    the next window (a host-side offset would be frozen into the captured launch).  Each replay equals the oracle
    with the window the counter stood at."""
    from tango_amd import config
    n = 100003
    x = torch.randn(n, device="cuda")
    s = K.cuda_kernels.get_scale(x)
    counter = torch.zeros(1, dtype=torch.int64, device="cuda")
    out = torch.empty(n, dtype=torch.int8, device="cuda")

    def step():
        K.cuda_kernels.quantize(out, x, s, round_mode="stochastic", seed=9, offset=counter, advance=config.WINDOW)

    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        step()  # warm-up outside capture: the counter now stands at one window
    torch.cuda.current_stream().wait_stream(stream)
    assert int(counter) == config.WINDOW
    assert np.array_equal(host(out), orc.quantize(host(x), host(s)[0], orc.STOCHASTIC, seed=9, offset=0))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    seen = []
    for k in range(1, 4):
        x.mul_(1.0)  # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert int(counter) == (k + 1) * config.WINDOW
        got = host(out)
        assert np.array_equal(got, orc.quantize(host(x), host(s)[0], orc.STOCHASTIC, seed=9, offset=k * config.WINDOW))
        seen.append(got)
    assert not np.array_equal(seen[0], seen[1]) and not np.array_equal(seen[1], seen[2])
    # a host offset and the device word add up
    counter.fill_(8)
    K.cuda_kernels.quantize(out, x, s, round_mode="stochastic", seed=9, offset=counter)
    out2 = torch.empty_like(out)
    K.cuda_kernels.quantize(out2, x, s, round_mode="stochastic", seed=9, offset=8)
    assert torch.equal(out, out2) and int(counter) == 8


def test_stochastic_positions_with_batched_counter_moves(K, orc):
    """config.stochastic_args outside a capture: call k of a device draws window k of the stream whether the
    position is carried by the device counter or by the pending count passed by value, and the counter moves once
    per config.BATCH calls."""
    from tango_amd import config
    old_seed = config.seed
    config.seed = 77
    config.reset_offsets()
    try:
        n = 4099
        x = torch.randn(n, device="cuda")
        s = K.cuda_kernels.get_scale(x)
        counter = config.device_offset(x.device)
        for k in range(config.BATCH + 3):
            q, _ = K.quantize(x, s, round_mode="stochastic", **config.stochastic_args(x.device))
            if k in (0, 1, config.BATCH - 2, config.BATCH - 1, config.BATCH, config.BATCH + 2):
                want = orc.quantize(host(x), host(s)[0], orc.STOCHASTIC, seed=77, offset=k * config.WINDOW)
                assert np.array_equal(host(q), want), k
            moved = (k + 1) // config.BATCH * config.BATCH
            assert int(counter) == moved * config.WINDOW, k
    finally:
        config.seed = old_seed
        config.reset_offsets()
