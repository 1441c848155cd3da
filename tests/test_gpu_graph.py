"""The compute entry points inside a captured HIP graph: every replay must give the bits of the
eager call, also after the inputs changed between replays and with eager work and
synchronisations in between (a decode loop replays one graph per token)."""
import ctypes as C

import numpy as np
import pytest

import oracle
from camelid_amd import binding as B
from camelid_amd.binding import DeviceBuffer, Weight, check, lib
from tests import gpu_util as G

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _init():
    assert lib().cml_available() == 1
    B.init(0)
    yield


@pytest.fixture()
def stream():
    s = C.c_void_p()
    check(lib().cml_stream_create(C.byref(s)), "cml_stream_create")
    yield s
    check(lib().cml_stream_sync(s))
    check(lib().cml_stream_destroy(s))


def capture(stream, fn):
    L = lib()
    check(L.cml_graph_begin_capture(stream), "begin capture")
    fn(stream)
    g = C.c_void_p()
    check(L.cml_graph_end_capture(stream, C.byref(g)), "end capture")
    return g


def h2d(buf: DeviceBuffer, a: np.ndarray) -> None:
    a = np.ascontiguousarray(a)
    check(lib().cml_memcpy_h2d(buf.ptr, a.ctypes.data, a.nbytes, None), "cml_memcpy_h2d")


def replay_and_compare(stream, call, inputs, set_input, read_output, replays=3):
    """`call(stream)` enqueues the work; inputs[i] is installed by set_input before replay i.
    Each replay is compared with an eager run of the same call on the same input."""
    L = lib()
    set_input(inputs[0])
    graph = capture(stream, call)
    try:
        for i in range(replays):
            set_input(inputs[i % len(inputs)])
            call(stream)                                   # eager, on the same stream
            check(L.cml_stream_sync(stream))
            want = read_output()
            check(L.cml_memset_dev(OUT_SCRUB[0].ptr, 0xFF, OUT_SCRUB[0].nbytes, None))
            check(L.cml_stream_sync(None))
            check(L.cml_graph_launch(graph, stream), "cml_graph_launch")
            check(L.cml_stream_sync(stream))
            got = read_output()
            assert G.same_bits(got, want), f"replay {i}"
            assert np.all(np.isfinite(got))
    finally:
        check(L.cml_graph_destroy(graph))


OUT_SCRUB = [None]   # the output buffer of the case at hand, scrubbed between the eager run and the replay


@pytest.mark.parametrize("name,fmt", [("Q8_0", oracle.Q8_0), ("Q4_0", oracle.Q4_0), ("Q4_K", oracle.Q4_K), ("Q6_K", oracle.Q6_K)])
@pytest.mark.parametrize("n", [1, 3, 16])
def test_matmul_f32_replays_are_the_eager_bits(stream, name, fmt, n):
    rows, cols = 300, 2048
    w = Weight.upload(fmt, rows, cols, G.synth_weight(fmt, rows, cols, seed=500 + fmt))
    rng = np.random.default_rng(501 + n)
    xs = [rng.standard_normal((n, cols)).astype(np.float32) for _ in range(3)]
    xd, od = DeviceBuffer(n * cols * 4), DeviceBuffer(n * rows * 4)
    ws_bytes = lib().cml_matmul_workspace_bytes(fmt, cols, n)
    ws = DeviceBuffer(max(ws_bytes, 16))
    OUT_SCRUB[0] = od
    G.say(f"graph matmul_f32 {name} n={n}")
    replay_and_compare(
        stream,
        lambda st: check(lib().cml_matmul_f32(w.handle, xd.ptr, n, od.ptr, ws.ptr, ws_bytes, st), "cml_matmul_f32"),
        xs, lambda x: (h2d(xd, x), check(lib().cml_stream_sync(None))),
        lambda: od.to_numpy(np.float32, (n, rows)))
    # and the last replay is the oracle's result
    want = oracle.matmul(fmt, w.download(), cols, xs[2], order=oracle.ORDER_PRIMARY, threads=4)
    assert G.max_rel(od.to_numpy(np.float32, (n, rows)), want) <= 1e-5


@pytest.mark.parametrize("T", [1, 6])
@pytest.mark.parametrize("fmt,hidden,ff", [(B.CML_Q4_K, 512, 256), (B.CML_Q4_0, 512, 96)])
def test_moe_layer_replays_are_the_eager_bits(stream, fmt, hidden, ff, T):
    """Routing + the whole expert lane captured together: the grouping pass, the fused prologues
    and the weighted sum use no memset nodes and no host round trip."""
    E, k = 16, 4
    L = lib()
    gate_up = G.synth_weight(fmt, E * 2 * ff, hidden, 510)
    down = G.synth_weight(fmt, E * hidden, ff, 511)
    wgu = Weight.upload(fmt, E * 2 * ff, hidden, gate_up)
    wd = Weight.upload(fmt, E * hidden, ff, down)
    rng = np.random.default_rng(512 + T)
    cases = [(rng.standard_normal((T, hidden)).astype(np.float32), rng.standard_normal((T, E)).astype(np.float32)) for _ in range(3)]
    xd, ld = DeviceBuffer(T * hidden * 4), DeviceBuffer(T * E * 4)
    idx, wts, od = DeviceBuffer(T * k * 4), DeviceBuffer(T * k * 4), DeviceBuffer(T * hidden * 4)
    ws_bytes = L.cml_moe_workspace_bytes(fmt, hidden, ff, T, k, E)
    ws = DeviceBuffer(ws_bytes)
    OUT_SCRUB[0] = od

    def call(st):
        check(L.cml_moe_route_softmax_top_k(ld.ptr, T, E, k, None, idx.ptr, wts.ptr, st), "route")
        check(L.cml_moe_ffn_ex(wgu.handle, None, wd.handle, E, k, idx.ptr, wts.ptr, xd.ptr, T, od.ptr, ws.ptr, ws_bytes, 1, st), "moe")

    def set_input(c):
        h2d(xd, c[0])
        h2d(ld, c[1])
        check(L.cml_stream_sync(None))

    G.say(f"graph moe fmt={fmt} T={T}")
    replay_and_compare(stream, call, cases, set_input, lambda: od.to_numpy(np.float32, (T, hidden)))
    want = oracle.moe_ffn_ex(fmt, gate_up, None, down, E, k, hidden, ff, cases[2][1], cases[2][0], variant=1, threads=4)
    assert G.max_rel(od.to_numpy(np.float32, (T, hidden)), want) <= 1e-5


def test_producers_and_lm_head_neighbours_replay(stream):
    """rms_norm -> Q8_K, gelu_tanh*up -> Q8_0, embedding gather and argmax in one captured graph."""
    L = lib()
    cols, n, rows = 1024, 2, 77
    rng = np.random.default_rng(520)
    table = G.synth_weight(B.CML_Q4_K, rows, cols, 521)
    wt = Weight.upload(B.CML_Q4_K, rows, cols, table)
    xs = [rng.standard_normal((n, cols)).astype(np.float32) * (1 + i) for i in range(3)]
    gamma = DeviceBuffer.from_numpy((rng.standard_normal(cols) * 0.1 + 1).astype(np.float32))
    ids = DeviceBuffer.from_numpy(np.array([5, 76], np.uint32))
    xd = DeviceBuffer(n * cols * 4)
    normed, q, sc = DeviceBuffer(n * cols * 4), DeviceBuffer(n * cols), DeviceBuffer(n * (cols // 256) * 4)
    hq, hs = DeviceBuffer(n * cols), DeviceBuffer(n * (cols // 32) * 4)
    emb, am = DeviceBuffer(n * cols * 4), DeviceBuffer(n * 4)
    OUT_SCRUB[0] = q

    def call(st):
        check(L.cml_rms_norm_quantize(2, xd.ptr, gamma.ptr, C.c_float(1e-5), n, cols, normed.ptr, q.ptr, sc.ptr, st), "rms_norm")
        check(L.cml_glu_quantize(1, 1, xd.ptr, normed.ptr, n, cols, hq.ptr, hs.ptr, st), "glu")
        check(L.cml_embed_gather(wt.handle, ids.ptr, n, emb.ptr, st), "gather")
        check(L.cml_argmax_f32(normed.ptr, n, cols, am.ptr, st), "argmax")

    def read():
        return np.concatenate([normed.to_numpy(np.float32, (n * cols,)), q.to_numpy(np.int8, (n * cols,)).astype(np.float32),
                               sc.to_numpy(np.float32, (n * (cols // 256),)), hq.to_numpy(np.int8, (n * cols,)).astype(np.float32),
                               hs.to_numpy(np.float32, (n * (cols // 32),)), emb.to_numpy(np.float32, (n * cols,)),
                               am.to_numpy(np.uint32, (n,)).astype(np.float32)])

    G.say("graph producers + gather + argmax")
    replay_and_compare(stream, call, xs, lambda x: (h2d(xd, x), check(L.cml_stream_sync(None))), read)
    want = oracle.rms_norm(xs[2], gamma.to_numpy(np.float32, (cols,)), 1e-5)
    assert G.same_bits(normed.to_numpy(np.float32, (n, cols)), want)
    assert list(am.to_numpy(np.uint32, (n,))) == [int(np.argmax(want[i])) for i in range(n)]
