"""GPU parity of the mixture-of-experts path (BASELINE config 5, Mixtral-shaped):
routing bit-exact in the selected experts, mixing weights and outputs within
tolerance of the oracle's composition (route -> gate/up band matvec -> silu_mul
-> down band matvec -> weighted sum in routed order)."""
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


def gpu_route(logits, k):
    logits = np.ascontiguousarray(logits, np.float32)
    T, E = logits.shape
    ld = DeviceBuffer.from_numpy(logits)
    idx = DeviceBuffer(T * k * 4)
    w = DeviceBuffer(T * k * 4)
    check(lib().cml_moe_route_top_k(ld.ptr, T, E, k, idx.ptr, w.ptr, None), "cml_moe_route_top_k")
    check(lib().cml_stream_sync(None))
    return idx, w, idx.to_numpy(np.int32, (T, k)), w.to_numpy(np.float32, (T, k))


def gpu_route_softmax(logits, k, down_scale=None):
    logits = np.ascontiguousarray(logits, np.float32)
    T, E = logits.shape
    ld = DeviceBuffer.from_numpy(logits)
    ds = None if down_scale is None else DeviceBuffer.from_numpy(np.ascontiguousarray(down_scale, np.float32))
    idx = DeviceBuffer(T * k * 4)
    w = DeviceBuffer(T * k * 4)
    check(lib().cml_moe_route_softmax_top_k(ld.ptr, T, E, k, None if ds is None else ds.ptr, idx.ptr, w.ptr, None),
          "cml_moe_route_softmax_top_k")
    check(lib().cml_stream_sync(None))
    return idx, w, idx.to_numpy(np.int32, (T, k)), w.to_numpy(np.float32, (T, k))


def gpu_moe(gate, up, down, E, k, idx_dev, w_dev, x, glu=None):
    """glu None: cml_moe_ffn; else cml_moe_ffn_ex with that activation (up may be None: fused gate|up)."""
    T, hidden = x.shape
    ff = down.cols
    xd = DeviceBuffer.from_numpy(x)
    out = DeviceBuffer(T * hidden * 4)
    out.fill(0xFF)
    ws_bytes = lib().cml_moe_workspace_bytes(gate.fmt, hidden, ff, T, k, E)
    assert ws_bytes > 0
    ws = DeviceBuffer(ws_bytes)
    if glu is None:
        check(lib().cml_moe_ffn(gate.handle, up.handle, down.handle, E, k, idx_dev.ptr, w_dev.ptr, xd.ptr, T, out.ptr,
                                ws.ptr, ws_bytes, None), "cml_moe_ffn")
    else:
        check(lib().cml_moe_ffn_ex(gate.handle, None if up is None else up.handle, down.handle, E, k, idx_dev.ptr, w_dev.ptr,
                                   xd.ptr, T, out.ptr, ws.ptr, ws_bytes, glu, None), "cml_moe_ffn_ex")
    check(lib().cml_stream_sync(None))
    return out.to_numpy(np.float32, (T, hidden))


def gpu_moe_logits(gate, up, down, E, k, logits, x):
    """cml_moe_ffn_logits: routing and expert lane in one call; the workspace is poisoned first."""
    T, hidden = x.shape
    ff = down.cols
    xd = DeviceBuffer.from_numpy(x)
    ld = DeviceBuffer.from_numpy(np.ascontiguousarray(logits, np.float32))
    out = DeviceBuffer(T * hidden * 4)
    out.fill(0xFF)
    ws_bytes = lib().cml_moe_workspace_bytes(gate.fmt, hidden, ff, T, k, E)
    ws = DeviceBuffer(ws_bytes)
    ws.fill(0xFF)
    check(lib().cml_moe_ffn_logits(gate.handle, up.handle, down.handle, E, k, ld.ptr, xd.ptr, T, out.ptr, ws.ptr, ws_bytes, None),
          "cml_moe_ffn_logits")
    check(lib().cml_stream_sync(None))
    return out.to_numpy(np.float32, (T, hidden))


def test_route_top_k_matches_oracle():
    rng = np.random.default_rng(300)
    logits = rng.standard_normal((257, 8)).astype(np.float32)
    logits[0] = 0.0                       # all tied: lowest indices win
    logits[1, 3] = logits[1, 5] = 2.0     # tie for first place
    logits[2] = [-np.inf] * 7 + [1.0]     # a non-finite logit gets weight 0
    logits[3] = -np.inf                   # nothing finite: uniform
    G.say("moe route 257x8 top-2")
    _, _, idx, w = gpu_route(logits, 2)
    for t in range(logits.shape[0]):
        oi, ow = oracle.softmax_top_k(logits[t], 2)
        assert list(idx[t]) == list(oi), t
        assert np.allclose(w[t], ow, rtol=3e-7, atol=1e-9), t   # expf may differ in the last bit
    G.say("moe route 64x16 top-4")
    logits = rng.standard_normal((64, 16)).astype(np.float32)
    _, _, idx, w = gpu_route(logits, 4)
    for t in range(64):
        oi, ow = oracle.softmax_top_k(logits[t], 4)
        assert list(idx[t]) == list(oi) and np.allclose(w[t], ow, rtol=3e-7)


def test_route_top_k_many_experts_both_kernels():
    """128 experts: k <= 64 takes the wave-per-token kernel, larger k the thread-per-token one."""
    rng = np.random.default_rng(302)
    logits = (rng.standard_normal((9, 128)) * 2).astype(np.float32)
    logits[0] = 1.5                         # all tied
    logits[1, 100] = np.inf                 # an infinite logit is selected first and gets weight 0
    logits[2, 5] = np.nan
    for k in (1, 8, 64, 70, 128):
        G.say(f"moe route 9x128 top-{k}")
        _, _, idx, w = gpu_route(logits, k)
        for t in range(logits.shape[0]):
            oi, ow = oracle.softmax_top_k(logits[t], k)
            assert list(idx[t]) == list(oi), (k, t)
            assert np.allclose(w[t], ow, rtol=1e-6, atol=1e-12, equal_nan=True), (k, t)


def _experts(E, hidden, ff, seed):
    gate = G.synth_weight(B.CML_Q4_K, E * ff, hidden, seed)
    up = G.synth_weight(B.CML_Q4_K, E * ff, hidden, seed + 1)
    down = G.synth_weight(B.CML_Q4_K, E * hidden, ff, seed + 2)
    return gate, up, down


@pytest.mark.parametrize("T", [1, 2, 5, 32])
def test_moe_ffn_small_matches_oracle(T):
    E, k, hidden, ff = 8, 2, 512, 1024
    gate, up, down = _experts(E, hidden, ff, 310)
    rng = np.random.default_rng(311 + T)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    if T >= 5:
        logits[:, 3] += 4.0   # crowd one expert: more than 8 assignments in one group at T = 32
    G.say(f"moe ffn small T={T}")
    wg = Weight.upload(B.CML_Q4_K, E * ff, hidden, gate)
    wu = Weight.upload(B.CML_Q4_K, E * ff, hidden, up)
    wd = Weight.upload(B.CML_Q4_K, E * hidden, ff, down)
    idx_dev, w_dev, idx, w = gpu_route(logits, k)
    with G.env(CAMELID_HIP_EXACT_ORDER="1"):
        got = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    want = oracle.moe_ffn(B.CML_Q4_K, gate, up, down, E, k, hidden, ff, logits, x, threads=8)
    assert G.max_rel(got, want) <= 1e-5
    got2 = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)   # default K-split policy
    assert G.max_rel(got2, want) <= 1e-5


@pytest.mark.parametrize("T", [1, 3, 9])
@pytest.mark.parametrize("E,k,hidden,ff", [(8, 2, 512, 1024), (16, 4, 1024, 512), (5, 5, 256, 256)])
def test_moe_ffn_logits_is_route_then_ffn(E, k, hidden, ff, T):
    """cml_moe_ffn_logits on shapes its gate|up launch does not route itself: a routing launch into the
    workspace, then the expert lane -- the bits of cml_moe_route_top_k followed by cml_moe_ffn; infinite
    and NaN logits included."""
    gate, up, down = _experts(E, hidden, ff, 340 + E)
    rng = np.random.default_rng(341 + T)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[0, 1] = np.inf
    if T > 1:
        logits[1, 0] = np.nan
        logits[T - 1, :] = 0.25   # every expert ties
    wg = Weight.upload(B.CML_Q4_K, E * ff, hidden, gate)
    wu = Weight.upload(B.CML_Q4_K, E * ff, hidden, up)
    wd = Weight.upload(B.CML_Q4_K, E * hidden, ff, down)
    G.say(f"moe ffn from logits E={E} k={k} {hidden}x{ff} T={T}")
    want = gpu_moe(wg, wu, wd, E, k, *gpu_route(logits, k)[:2], x)
    assert G.same_bits(gpu_moe_logits(wg, wu, wd, E, k, logits, x), want)


def _stacked_from_one(base, E, block_bytes, scale0):
    """E experts from one expert's wire bytes, made distinct cheaply: expert e carries its own f16 super-block
    scale d in every block (the first two bytes of a Q4_K block), so which expert served a slot shows in every output."""
    out = np.tile(base, E).reshape(E, -1, block_bytes)
    for e in range(E):
        out[e, :, 0:2] = np.frombuffer(np.float16(scale0 * (1.0 + 0.03 * e)).tobytes(), np.uint8)
    return out.reshape(-1)


# The gate|up launch routes the token itself where it runs 8-row waves, which the launch policy picks while the routed slots
# of both projections stay below about 4.5 sixteen-row waves per SIMD quarter (top-2 and top-3 at these sizes); with top-4
# and top-8 it runs 16-row waves, whose launch has no routing variant, and a routing launch goes first.
@pytest.mark.parametrize("E,k,ff,in_launch", [(72, 3, 12288, True), (100, 2, 14336, True), (8, 3, 12288, True), (72, 4, 12288, False),
                                              (100, 8, 12800, False)])
def test_moe_ffn_logits_routes_inside_the_launch_like_the_routing_launch(E, k, ff, in_launch):
    """One token on Q4_K experts whose gate / up bands take no K cut (12288 rows of 4096 values): the gate|up
    launch routes the token itself (every wave, from the logits).  More than 64 experts (both halves of a lane's
    pair), top-3 / 4 / 8, logits that tie, infinities and NaNs: the bits of the routing launch followed by the
    expert lane (CAMELID_HIP_MOE_FOLD_ROUTE=0), and the counters say which ran."""
    hidden = 4096
    g1, u1, d1 = _experts(1, hidden, ff, 360 + E + k)
    gate, up, down = (_stacked_from_one(t, E, 144, 0.004) for t in (g1, u1, d1))
    wg = Weight.upload(B.CML_Q4_K, E * ff, hidden, gate)
    wu = Weight.upload(B.CML_Q4_K, E * ff, hidden, up)
    wd = Weight.upload(B.CML_Q4_K, E * hidden, ff, down)
    del gate, up, down
    rng = np.random.default_rng(361 + E)
    x = rng.standard_normal((1, hidden)).astype(np.float32)
    base = rng.standard_normal((1, E)).astype(np.float32)
    tied = base.copy()
    tied[0, E // 2:] = tied[0, 1]            # many experts tie, across lane 64 where there are that many
    tied[0, 3] = tied[0, 1]
    odd = base.copy()
    odd[0, 0], odd[0, E - 1], odd[0, E // 2] = np.nan, np.inf, -np.inf
    outs = []
    for i, logits in enumerate((base, tied, odd, np.full((1, E), 0.25, np.float32))):
        G.say(f"moe ffn routed in the launch E={E} k={k} case={i}")
        proof = (G.engaged(r"^q4k\.dot\.direct\.ring\.route$", none=(r"^moe\.route",)) if in_launch else
                 G.engaged(r"^moe\.route", r"^q4k\.dot\.direct", none=(r"\.route$",)))
        with proof:
            got = gpu_moe_logits(wg, wu, wd, E, k, logits, x)
        with G.env(CAMELID_HIP_MOE_FOLD_ROUTE="0"), G.engaged(r"^moe\.route", r"^q4k\.dot\.direct", none=(r"\.route$",)):
            want = gpu_moe_logits(wg, wu, wd, E, k, logits, x)
        assert G.same_bits(got, want), (E, k, i)
        assert G.same_bits(got, gpu_moe(wg, wu, wd, E, k, *gpu_route(logits, k)[:2], x)), (E, k, i)
        outs.append(got)
    assert not G.same_bits(outs[0], outs[3])   # the routing does change the result: the experts differ


def test_moe_ffn_logits_rejects_bad_arguments():
    E, k, hidden, ff = 4, 2, 256, 256
    gate, up, down = _experts(E, hidden, ff, 350)
    wg = Weight.upload(B.CML_Q4_K, E * ff, hidden, gate)
    wu = Weight.upload(B.CML_Q4_K, E * ff, hidden, up)
    wd = Weight.upload(B.CML_Q4_K, E * hidden, ff, down)
    x = DeviceBuffer.from_numpy(np.zeros((1, hidden), np.float32))
    lg = DeviceBuffer.from_numpy(np.zeros((1, E), np.float32))
    out = DeviceBuffer(hidden * 4)
    ws_bytes = lib().cml_moe_workspace_bytes(B.CML_Q4_K, hidden, ff, 1, k, E)
    ws = DeviceBuffer(ws_bytes)
    L = lib()
    assert L.cml_moe_ffn_logits(wg.handle, wu.handle, wd.handle, E, k, None, x.ptr, 1, out.ptr, ws.ptr, ws_bytes, None) == 2
    assert L.cml_moe_ffn_logits(wg.handle, None, wd.handle, E, k, lg.ptr, x.ptr, 1, out.ptr, ws.ptr, ws_bytes, None) == 2
    assert L.cml_moe_ffn_logits(wg.handle, wu.handle, wd.handle, E, E + 1, lg.ptr, x.ptr, 1, out.ptr, ws.ptr, ws_bytes, None) == 3
    assert L.cml_moe_ffn_logits(wg.handle, wu.handle, wd.handle, E, k, lg.ptr, x.ptr, 1, out.ptr, ws.ptr, ws_bytes - 256, None) == 3
    assert L.cml_moe_ffn_logits(wg.handle, wu.handle, wd.handle, E, k, lg.ptr, x.ptr, 0, out.ptr, ws.ptr, ws_bytes, None) == 0


@pytest.mark.parametrize("T", [1, 2, 5, 32])
def test_moe_ffn_mixtral_with_q6k_down_matches_oracle(T):
    """Q4_K_M-style files keep some expert down projections in Q6_K: gate / up Q4_K, down Q6_K."""
    E, k, hidden, ff = 8, 2, 512, 1024
    gate = G.synth_weight(B.CML_Q4_K, E * ff, hidden, 312)
    up = G.synth_weight(B.CML_Q4_K, E * ff, hidden, 313)
    down = G.synth_weight(B.CML_Q6_K, E * hidden, ff, 314)
    rng = np.random.default_rng(315 + T)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    if T >= 5:
        logits[:, 3] += 4.0
    G.say(f"moe ffn Q4_K gate/up + Q6_K down T={T}")
    wg = Weight.upload(B.CML_Q4_K, E * ff, hidden, gate)
    wu = Weight.upload(B.CML_Q4_K, E * ff, hidden, up)
    wd = Weight.upload(B.CML_Q6_K, E * hidden, ff, down)
    idx_dev, w_dev, idx, w = gpu_route(logits, k)
    want = oracle.moe_ffn_ex(B.CML_Q4_K, gate, up, down, E, k, hidden, ff, logits, x, threads=8, fmt_down=B.CML_Q6_K)
    with G.env(CAMELID_HIP_EXACT_ORDER="1"):
        got = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    assert G.max_rel(got, want) <= 1e-5
    got2 = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)   # default K-split policy
    assert G.max_rel(got2, want) <= 1e-5


def test_moe_ffn_is_the_sum_of_single_expert_calls():
    """Grouping must not change any (token, expert) cell: compare with per-token, per-expert
    matvecs through the plain entry points, mixed on the host in routed order."""
    E, k, hidden, ff, T = 4, 2, 256, 512, 6
    gate, up, down = _experts(E, hidden, ff, 320)
    rng = np.random.default_rng(321)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    wg = Weight.upload(B.CML_Q4_K, E * ff, hidden, gate)
    wu = Weight.upload(B.CML_Q4_K, E * ff, hidden, up)
    wd = Weight.upload(B.CML_Q4_K, E * hidden, ff, down)
    idx_dev, w_dev, idx, w = gpu_route(logits, k)
    G.say("moe ffn vs single-expert calls")
    with G.env(CAMELID_HIP_EXACT_ORDER="1"):
        got = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
        want = np.zeros((T, hidden), np.float32)
        for t in range(T):
            for s in range(k):
                e = int(idx[t, s])
                g = G.gpu_matmul_f32(wg.slice(e * ff, ff), x[t])
                u = G.gpu_matmul_f32(wu.slice(e * ff, ff), x[t])
                h = oracle.silu_mul(g, u)
                y = G.gpu_matmul_f32(wd.slice(e * hidden, hidden), h)
                want[t] = (want[t] + (y * w[t, s]).astype(np.float32)).astype(np.float32)
    assert G.max_rel(got, want) <= 2e-6   # silu's expf is the only difference


@pytest.mark.parametrize("fmt,fmt_down,hidden,ff", [(B.CML_Q4_K, B.CML_Q4_K, 512, 1024), (B.CML_Q4_0, B.CML_Q8_0, 352, 96)])
@pytest.mark.parametrize("T", [1, 3])
def test_moe_ffn_skips_slots_with_expert_ids_out_of_range(fmt, fmt_down, hidden, ff, T):
    """A routed slot whose expert id is outside [0, n_experts) is served by nobody and adds nothing:
    the same bits as the call with that slot left out (decode and batched paths; the workspace
    starts poisoned so that a slot's stale output would show)."""
    E, k = 8, 3
    gate_up, down = _experts_fused(fmt, fmt_down, E, hidden, ff, 700)
    wgu = Weight.upload(fmt, E * 2 * ff, hidden, gate_up)
    wd = Weight.upload(fmt_down, E * hidden, ff, down)
    rng = np.random.default_rng(701 + T)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    idx = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    w = rng.random((T, k)).astype(np.float32)
    for bad in (E + 5, -1):
        idx_bad = idx.copy()
        idx_bad[:, 1] = bad
        G.say(f"moe ffn with expert id {bad} in slot 1, fmt={fmt}/{fmt_down} T={T}")
        got = _moe_poisoned(wgu, wd, E, k, idx_bad, w, x)
        want = _moe_poisoned(wgu, wd, E, k - 1, np.ascontiguousarray(idx[:, [0, 2]]), np.ascontiguousarray(w[:, [0, 2]]), x)
        assert np.isfinite(got).all()
        assert G.same_bits(got, want)


@pytest.mark.parametrize("E,k,hidden,ff", [(8, 2, 512, 1024), (8, 3, 4096, 14336 // 4), (16, 4, 1024, 2048), (4, 1, 256, 768)])
def test_moe_decode_down_projection_with_the_weighted_sum_folded_in(E, k, hidden, ff):
    """One token, Q4_K experts: the down projections of the routed experts and the weighted sum run as
    one launch (a workgroup owns a row tile for all slots) -- bit for bit the separate launches
    (CAMELID_HIP_MOE_FOLD_SUM=0), under the default K cut and with it forbidden, also when a slot's
    expert id is out of range."""
    gate_up, down = _experts_fused(B.CML_Q4_K, B.CML_Q4_K, E, hidden, ff, 800 + E)
    wgu = Weight.upload(B.CML_Q4_K, E * 2 * ff, hidden, gate_up)
    wd = Weight.upload(B.CML_Q4_K, E * hidden, ff, down)
    rng = np.random.default_rng(801 + hidden)
    x = rng.standard_normal((1, hidden)).astype(np.float32)
    idx = rng.permutation(E)[:k].astype(np.int32).reshape(1, k)
    w = rng.random((1, k)).astype(np.float32)
    for exact in ("0", "1"):
        for bad in (False, True):
            if bad and k < 2:
                continue
            ids = idx.copy()
            if bad:
                ids[0, k - 1] = E + 3
            G.say(f"moe decode, folded sum, E={E} k={k} {hidden}x{ff} exact={exact} bad={bad}")
            with G.env(CAMELID_HIP_EXACT_ORDER=exact):
                folded = _moe_poisoned(wgu, wd, E, k, ids, w, x)
                with G.env(CAMELID_HIP_EXACT_ORDER=exact, CAMELID_HIP_MOE_FOLD_SUM=0):
                    separate = _moe_poisoned(wgu, wd, E, k, ids, w, x)
            assert np.isfinite(folded).all()
            assert G.same_bits(folded, separate)


def _moe_poisoned(wgu, wd, E, k, idx, w, x):
    T, hidden = x.shape
    ff = wd.cols
    xd = DeviceBuffer.from_numpy(x)
    out = DeviceBuffer(T * hidden * 4)
    out.fill(0xFF)
    ws_bytes = lib().cml_moe_workspace_bytes(wgu.fmt, hidden, ff, T, k, E)
    ws = DeviceBuffer(ws_bytes)
    ws.fill(0xFF)    # NaN patterns wherever a float is read without having been written
    idx_dev = DeviceBuffer.from_numpy(np.ascontiguousarray(idx, np.int32))
    w_dev = DeviceBuffer.from_numpy(np.ascontiguousarray(w, np.float32))
    check(lib().cml_moe_ffn_ex(wgu.handle, None, wd.handle, E, k, idx_dev.ptr, w_dev.ptr, xd.ptr, T, out.ptr, ws.ptr, ws_bytes,
                               GLU_GELU_TANH, None), "cml_moe_ffn_ex")
    check(lib().cml_stream_sync(None))
    return out.to_numpy(np.float32, (T, hidden))


@pytest.mark.parametrize("E,k,hidden,ff,T", [(8, 2, 512, 1024, 7), (8, 2, 1024, 2048, 40), (4, 3, 256, 768, 16), (16, 4, 512, 512, 33)])
def test_moe_gate_and_up_in_one_launch_give_the_bits_of_two(E, k, hidden, ff, T):
    """Batches on Q4_K experts with gate and up as separate tensors: both projections run as one
    matrix-core launch (twice the workgroups in one grid) -- bit for bit the two launches
    (CAMELID_HIP_MOE_PAIR_LAUNCH=0)."""
    gate, up, down = _experts(E, hidden, ff, 970 + E)
    wg = Weight.upload(B.CML_Q4_K, E * ff, hidden, gate)
    wu = Weight.upload(B.CML_Q4_K, E * ff, hidden, up)
    wd = Weight.upload(B.CML_Q4_K, E * hidden, ff, down)
    rng = np.random.default_rng(971 + T)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[:, 1] -= 50.0    # an expert nobody routes to
    idx_dev, w_dev, _, _ = gpu_route(logits, k)
    G.say(f"moe gate|up pair launch, E={E} k={k} {hidden}x{ff} T={T}")
    one = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    with G.env(CAMELID_HIP_MOE_PAIR_LAUNCH=0):
        two = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    assert np.isfinite(one).all()
    assert G.same_bits(one, two)


@pytest.mark.parametrize("E,k,hidden,ff,T", [(8, 2, 4096, 1024, 40), (8, 2, 2048, 2048, 16), (8, 3, 3072, 2048, 30), (8, 2, 4096, 2048, 9)])
def test_moe_staged_once_walks_of_several_units_give_the_bits_of_one_unit_each(E, k, hidden, ff, T):
    """The expert-grouped matrix-core launch on rows of up to 16 super-blocks stages the activation once per
    workgroup and walks several groups of row tiles against it (gate and up in one list, the ring refilled
    across the group boundaries); rows of 2048 and 4096 values take the walk with the row length known at
    compile time.  Every shape of that launch -- one unit per workgroup, three, the launcher's own choice, the
    general walk, the phased staging -- gives the same bits, and so do gate and up as two launches."""
    gate, up, down = _experts(E, hidden, ff, 1170 + E)
    wg = Weight.upload(B.CML_Q4_K, E * ff, hidden, gate)
    wu = Weight.upload(B.CML_Q4_K, E * ff, hidden, up)
    wd = Weight.upload(B.CML_Q4_K, E * hidden, ff, down)
    rng = np.random.default_rng(1171 + T)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[:, 1] -= 50.0    # an expert nobody routes to
    idx_dev, w_dev, _, _ = gpu_route(logits, k)
    fixed = {4096: r"\.k16", 2048: r"\.k8"}.get(hidden)
    G.say(f"moe staged-once unit walk, E={E} k={k} {hidden}x{ff} T={T}")
    with G.env(CAMELID_HIP_TUNING=1, CAMELID_HIP_Q4K_MFMA_UNITS=1), G.engaged(r"^q4k\.mfma\.(tile|serial_split)\.g1t1\.grouped\.once", none=(r"\.units$",)):
        one = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    assert np.isfinite(one).all()
    with G.env(CAMELID_HIP_TUNING=1, CAMELID_HIP_Q4K_MFMA_UNITS=3), G.engaged(r"^q4k\.mfma\.(tile|serial_split)\.g1t1\.grouped\.once.*\.units$"):
        three = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    assert G.same_bits(one, three)
    with G.engaged(r"^q4k\.mfma\.(tile|serial_split)\.g1t1\.grouped\.once" + (fixed or "")):
        auto = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    assert G.same_bits(one, auto)
    with G.env(CAMELID_HIP_TUNING=1, CAMELID_HIP_Q4K_MFMA_FIXED_ROWS=0, CAMELID_HIP_Q4K_MFMA_UNITS=5), \
            G.engaged(r"^q4k\.mfma\.(tile|serial_split)\.g1t1\.grouped\.once\.units$"):
        general = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    assert G.same_bits(one, general)
    with G.env(CAMELID_HIP_MOE_PAIR_LAUNCH=0):
        two = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    assert G.same_bits(one, two)
    with G.env(CAMELID_HIP_TUNING=1, CAMELID_HIP_Q4K_MFMA_STAGE_ONCE=0), G.engaged(r"^q4k\.mfma\.(tile|serial_split)\.g1t1\.grouped$"):
        phased = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    assert G.same_bits(one, phased)


@pytest.mark.parametrize("E,k,hidden,ff,T", [(8, 2, 4096, 1024, 64), (4, 2, 2048, 2048, 70), (8, 3, 3072, 2048, 40)])
def test_moe_experts_with_more_than_16_assignments_take_two_token_groups_per_wave(E, k, hidden, ff, T):
    """Once the experts of a batch hold more than 16 assignments on average, the staged-once launch gives a wave
    two 16-token groups (one pass over an expert's weights serves 32 assignments; one workgroup per compute unit):
    the same bits as one group per wave with a second token column, and as gate and up in two launches."""
    gate, up, down = _experts(E, hidden, ff, 1270 + E)
    wg = Weight.upload(B.CML_Q4_K, E * ff, hidden, gate)
    wu = Weight.upload(B.CML_Q4_K, E * ff, hidden, up)
    wd = Weight.upload(B.CML_Q4_K, E * hidden, ff, down)
    rng = np.random.default_rng(1271 + T)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[:, 0] += 1.5     # a crowded expert (more than 32 assignments at the larger T), an idle one
    logits[:, 1] -= 50.0
    idx_dev, w_dev, _, _ = gpu_route(logits, k)
    G.say(f"moe two token groups per wave, E={E} k={k} {hidden}x{ff} T={T}")
    with G.engaged(r"^q4k\.mfma\.(tile|serial_split)\.g2t1\.grouped\.once"):
        two_groups = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    assert np.isfinite(two_groups).all()
    with G.env(CAMELID_HIP_TUNING=1, CAMELID_HIP_Q4K_MFMA_ONCE_TWO_GROUPS=0), \
            G.engaged(r"^q4k\.mfma\.(tile|serial_split)\.g1t1\.grouped\.once", none=(r"\.g2t1",)):
        one_group = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    assert G.same_bits(two_groups, one_group)
    with G.env(CAMELID_HIP_TUNING=1, CAMELID_HIP_Q4K_MFMA_UNITS=3, CAMELID_HIP_Q4K_MFMA_FIXED_ROWS=0):
        general = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    assert G.same_bits(two_groups, general)
    with G.env(CAMELID_HIP_MOE_PAIR_LAUNCH=0):
        two_launches = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    assert G.same_bits(two_groups, two_launches)


@pytest.mark.parametrize("E,k,hidden,ff,T", [(8, 2, 6144, 1024, 24), (8, 2, 5120, 1024, 9), (8, 2, 8192, 1024, 40)])
def test_moe_experts_with_long_rows_take_the_staged_once_walk(E, k, hidden, ff, T):
    """Expert groups whose gate / up rows are 5120, 6144 or 8192 values (a Mixtral-8x22B-shaped layer has 6144):
    the staged-once launch with 32 slabs of LDS, one workgroup per compute unit -- the bits of the phased
    launch, with one or three groups of row tiles per workgroup."""
    gate, up, down = _experts(E, hidden, ff, 1370 + E)
    wg = Weight.upload(B.CML_Q4_K, E * ff, hidden, gate)
    wu = Weight.upload(B.CML_Q4_K, E * ff, hidden, up)
    wd = Weight.upload(B.CML_Q4_K, E * hidden, ff, down)
    rng = np.random.default_rng(1371 + T)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[:, 1] -= 50.0    # an expert nobody routes to
    idx_dev, w_dev, _, _ = gpu_route(logits, k)
    G.say(f"moe long rows, E={E} k={k} {hidden}x{ff} T={T}")
    with G.engaged(rf"^q4k\.mfma\.(tile|serial_split)\.g1t1\.grouped\.once\.k{hidden // 256}"):
        walk = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    assert np.isfinite(walk).all()
    with G.env(CAMELID_HIP_TUNING=1, CAMELID_HIP_Q4K_MFMA_ONCE_LONG_ROWS=0), G.engaged(r"^q4k\.mfma\.(tile|serial_split)\.g1t1\.grouped$"):
        phased = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    assert G.same_bits(walk, phased)
    with G.env(CAMELID_HIP_TUNING=1, CAMELID_HIP_Q4K_MFMA_UNITS=3), G.engaged(rf"\.once\.k{hidden // 256}\.units$"):
        three = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    assert G.same_bits(walk, three)


@pytest.mark.parametrize("T", [1, 32])
def test_c5_mixtral_shaped_moe(T):
    """8 experts, gate/up 14336x4096 and down 4096x14336 in Q4_K, top-2 routing."""
    E, k, hidden, ff = 8, 2, 4096, 14336
    G.say(f"C5 Mixtral-shaped MoE T={T}: building 8 experts")
    gate, up, down = _experts(E, hidden, ff, 330)
    rng = np.random.default_rng(331 + T)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    wg = Weight.upload(B.CML_Q4_K, E * ff, hidden, gate)
    wu = Weight.upload(B.CML_Q4_K, E * ff, hidden, up)
    wd = Weight.upload(B.CML_Q4_K, E * hidden, ff, down)
    idx_dev, w_dev, idx, w = gpu_route(logits, k)
    G.say(f"C5 Mixtral-shaped MoE T={T}: device run")
    proof = (G.engaged(r"^q4k\.dot\.direct", r"^q4k\.down_sum", none=(r"^q4k\.mfma\.", r"^moe\.weighted_sum")) if T == 1 else
             G.engaged(r"^moe\.plan", r"^q4k\.mfma\..*grouped", r"^moe\.weighted_sum", none=(r"^q4k\.dot\.",)))
    with proof:
        got = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    # routing and expert lane as one call (one token: routed inside the gate|up launch): the same bits,
    # also with the routing as a launch of its own and on logits that tie
    G.say(f"C5 Mixtral-shaped MoE T={T}: the entry that takes logits")
    assert G.same_bits(gpu_moe_logits(wg, wu, wd, E, k, logits, x), got)
    with G.env(CAMELID_HIP_MOE_FOLD_ROUTE="0"):
        assert G.same_bits(gpu_moe_logits(wg, wu, wd, E, k, logits, x), got)
    tied = logits.copy()
    tied[:, 5] = tied[:, 2]
    tied[:, 7] = tied[:, 2]
    assert G.same_bits(gpu_moe_logits(wg, wu, wd, E, k, tied, x), gpu_moe(wg, wu, wd, E, k, *gpu_route(tied, k)[:2], x))
    odd = logits.copy()
    odd[:, 1] = np.inf
    odd[:, 6] = np.nan
    odd[:, 0] = -np.inf
    assert G.same_bits(gpu_moe_logits(wg, wu, wd, E, k, odd, x), gpu_moe(wg, wu, wd, E, k, *gpu_route(odd, k)[:2], x))
    tt = min(T, 8)   # the oracle walks 3 full expert matvecs per (token, expert): bound the CPU work
    want = oracle.moe_ffn(B.CML_Q4_K, gate, up, down, E, k, hidden, ff, logits[:tt], x[:tt], threads=16)
    assert G.max_rel(got[:tt], want) <= 1e-5
    assert np.all(np.isfinite(got))
    if T > 1:
        # every token of the batch: the bits of a single-token call of the same entry point (the batch runs the
        # grouped matrix-core kernels and a weighted-sum launch, the single token the packed-dot decode launches with
        # the sum folded into the down projection -- different kernels, one association)
        for t in range(T):
            G.say(f"C5 Mixtral-shaped MoE T={T}: token {t} alone")
            with G.engaged(r"^q4k\.dot\.direct", r"^q4k\.down_sum", none=(r"^q4k\.mfma\.",)):
                one = gpu_moe(wg, wu, wd, E, k, *gpu_route(logits[t:t + 1], k)[:2], x[t:t + 1])
            assert G.same_bits(got[t:t + 1], one), t


# ---------------------------------------------------------------- Gemma-4 variant ----

GLU_SILU, GLU_GELU_TANH = 0, 1
ACT_Q8_0, ACT_Q8_K = 1, 2


def test_route_softmax_top_k_matches_oracle():
    """Softmax over all experts, top-k by probability, scales renormalised over the selection and
    multiplied by down_scale (reference src/gemma4_runtime.rs:5567-5610): indices exact, scales
    within the last bits expf may differ in."""
    rng = np.random.default_rng(340)
    logits = (rng.standard_normal((130, 128)) * 3).astype(np.float32)
    logits[0] = 0.0                                   # all tied: the lowest indices, scale 1/k each
    logits[1, 7] = logits[1, 99] = logits[1].max() + 1  # tie for first place: 7 before 99
    logits[2] = [((e * 37 + 11) % 17) / 17.0 for e in range(128)]   # the reference's own tie vector
    ds = rng.uniform(0.5, 2.0, 128).astype(np.float32)
    for k, scale in ((8, ds), (1, None), (128, ds)):
        G.say(f"moe route softmax 130x128 top-{k}")
        # full ranking (k = 128) on a few rows only: two random logits a few ulps apart would rank
        # by the last bit of expf, which the device and the host libm need not share
        lg = logits[:4] if k == 128 else logits
        _, _, idx, w = gpu_route_softmax(lg, k, scale)
        for t in range(lg.shape[0]):
            oi, ow = oracle.router_softmax_top_k(lg[t], k, down_scale=scale)
            assert list(idx[t]) == list(oi), (k, t)
            assert np.allclose(w[t], ow, rtol=1e-6, atol=1e-12), (k, t)
    _, _, idx, w = gpu_route_softmax(logits[:1], 8)
    assert list(idx[0]) == list(range(8)) and list(w[0]) == [0.125] * 8
    G.say("moe route softmax 5x16 top-3")
    logits = rng.standard_normal((5, 16)).astype(np.float32)
    _, _, idx, w = gpu_route_softmax(logits, 3)
    for t in range(5):
        oi, ow = oracle.router_softmax_top_k(logits[t], 3)
        assert list(idx[t]) == list(oi) and np.allclose(w[t], ow, rtol=1e-6)


def test_route_softmax_rejects_bad_shapes():
    d = DeviceBuffer(4096)
    L = lib()
    assert L.cml_moe_route_softmax_top_k(d.ptr, 1, 129, 2, None, d.ptr, d.ptr, None) == 6   # more than 128 experts
    assert L.cml_moe_route_softmax_top_k(d.ptr, 1, 8, 9, None, d.ptr, d.ptr, None) == 3     # k > experts
    assert L.cml_moe_route_softmax_top_k(None, 1, 8, 2, None, d.ptr, d.ptr, None) == 2
    assert L.cml_moe_route_softmax_top_k(None, 0, 8, 2, None, None, None, None) == 0        # empty batch


def _experts_fused(fmt, fmt_down, E, hidden, ff, seed):
    gate_up = G.synth_weight(fmt, E * 2 * ff, hidden, seed)
    down = G.synth_weight(fmt_down, E * hidden, ff, seed + 2)
    return gate_up, down


def _split_gate_up(gate_up, fmt, E, hidden, ff):
    rb = oracle.row_bytes(fmt, hidden)
    gu = np.asarray(gate_up, np.uint8).reshape(E, 2, ff * rb)
    return np.ascontiguousarray(gu[:, 0]).reshape(-1), np.ascontiguousarray(gu[:, 1]).reshape(-1)


GEMMA_SMALL = [
    # (gate/up format, down format, hidden, ff): whole blocks of each format; 352 = 11 and 96 = 3
    # blocks of 32, so rows end inside a 16-lane step
    (B.CML_Q4_K, B.CML_Q4_K, 512, 256),
    (B.CML_Q4_0, B.CML_Q4_0, 352, 96),
    (B.CML_Q8_0, B.CML_Q8_0, 352, 96),
    (B.CML_Q4_0, B.CML_Q8_0, 512, 704),
    (B.CML_Q4_K, B.CML_Q4_0, 256, 96),
    (B.CML_Q4_K, B.CML_Q6_K, 256, 512),
    (B.CML_Q6_K, B.CML_Q6_K, 512, 256),
    (B.CML_Q8_0, B.CML_Q6_K, 96, 256),
]


@pytest.mark.parametrize("T", [1, 2, 5, 40])
@pytest.mark.parametrize("fmt,fmt_down,hidden,ff", GEMMA_SMALL)
def test_moe_ffn_ex_gemma4_small_matches_oracle(fmt, fmt_down, hidden, ff, T):
    E, k = 16, 4
    gate_up, down = _experts_fused(fmt, fmt_down, E, hidden, ff, 350)
    gate, up = _split_gate_up(gate_up, fmt, E, hidden, ff)
    rng = np.random.default_rng(351 + T)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    if T >= 5:
        logits[:, 3] += 4.0   # crowd one expert: more than 8 assignments in one group at T = 40
    ds = rng.uniform(0.5, 2.0, E).astype(np.float32)
    G.say(f"moe ffn_ex gemma4 small fmt={fmt}/{fmt_down} {hidden}x{ff} T={T}")
    wgu = Weight.upload(fmt, E * 2 * ff, hidden, gate_up)
    wg = Weight.upload(fmt, E * ff, hidden, gate)
    wu = Weight.upload(fmt, E * ff, hidden, up)
    wd = Weight.upload(fmt_down, E * hidden, ff, down)
    idx_dev, w_dev, idx, w = gpu_route_softmax(logits, k, ds)
    want = oracle.moe_ffn_ex(fmt, gate_up, None, down, E, k, hidden, ff, logits, x, variant=1, down_scale=ds, threads=8,
                             fmt_down=fmt_down)
    with G.env(CAMELID_HIP_EXACT_ORDER="1"):
        fused = gpu_moe(wgu, None, wd, E, k, idx_dev, w_dev, x, glu=GLU_GELU_TANH)
        split = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x, glu=GLU_GELU_TANH)
    assert G.max_rel(fused, want) <= 1e-5
    assert G.same_bits(fused, split)      # one projection over gate|up or two: the same cells
    got2 = gpu_moe(wgu, None, wd, E, k, idx_dev, w_dev, x, glu=GLU_GELU_TANH)   # default K-split policy
    assert G.max_rel(got2, want) <= 1e-5


@pytest.mark.parametrize("fmt,fmt_down", [(B.CML_Q4_0, B.CML_Q4_0), (B.CML_Q8_0, B.CML_Q4_0), (B.CML_Q4_0, B.CML_Q4_K),
                                          (B.CML_Q4_K, B.CML_Q6_K), (B.CML_Q6_K, B.CML_Q8_0)])
def test_moe_ffn_ex_is_the_sum_of_single_expert_calls(fmt, fmt_down):
    """Grouping must not change any (token, expert) cell, for the 32-value formats too: compare
    with per-token, per-expert matvecs through the plain entry points, mixed on the host."""
    E, k, hidden, ff, T = 6, 3, 256, 256, 7
    gate_up, down = _experts_fused(fmt, fmt_down, E, hidden, ff, 360)
    rng = np.random.default_rng(361)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    wgu = Weight.upload(fmt, E * 2 * ff, hidden, gate_up)
    wd = Weight.upload(fmt_down, E * hidden, ff, down)
    idx_dev, w_dev, idx, w = gpu_route_softmax(logits, k)
    G.say(f"moe ffn_ex vs single-expert calls fmt={fmt}/{fmt_down}")
    with G.env(CAMELID_HIP_EXACT_ORDER="1"):
        got = gpu_moe(wgu, None, wd, E, k, idx_dev, w_dev, x, glu=GLU_GELU_TANH)
        want = np.zeros((T, hidden), np.float32)
        for t in range(T):
            for s in range(k):
                e = int(idx[t, s])
                gu = G.gpu_matmul_f32(wgu.slice(e * 2 * ff, 2 * ff), x[t]).reshape(-1)
                h = oracle.gelu_tanh_mul(gu[:ff], gu[ff:])
                y = G.gpu_matmul_f32(wd.slice(e * hidden, hidden), h).reshape(-1)
                want[t] = (want[t] + (y * w[t, s]).astype(np.float32)).astype(np.float32)
    assert G.max_rel(got, want) <= 2e-6   # gelu's tanhf is the only difference


def test_moe_ffn_ex_rejects_bad_arguments():
    E, k, hidden, ff = 4, 2, 256, 256
    gate_up, down = _experts_fused(B.CML_Q4_0, B.CML_Q4_0, E, hidden, ff, 370)
    wgu = Weight.upload(B.CML_Q4_0, E * 2 * ff, hidden, gate_up)
    wd = Weight.upload(B.CML_Q4_0, E * hidden, ff, down)
    w6 = Weight.upload(B.CML_Q6_K, 256, 256, G.synth_weight(B.CML_Q6_K, 256, 256, 371))
    d = DeviceBuffer(1 << 20)
    L = lib()
    args = (E, k, d.ptr, d.ptr, d.ptr, 1, d.ptr, d.ptr, 1 << 20)
    assert L.cml_moe_ffn_ex(wgu.handle, None, wd.handle, *args, 7, None) == 2        # unknown activation
    assert L.cml_moe_ffn_ex(w6.handle, None, wd.handle, *args, 1, None) == 3         # a 256-row Q6_K tensor is not 4 x 512 rows
    assert L.cml_moe_ffn_ex(wgu.handle, wd.handle, wd.handle, *args, 1, None) == 3   # up of another shape
    assert L.cml_moe_ffn_ex(wgu.handle, None, wd.handle, E, k, d.ptr, d.ptr, d.ptr, 1, d.ptr, d.ptr, 16, 1, None) == 3  # workspace
    assert L.cml_moe_ffn(wgu.handle, None, wd.handle, *args, None) == 2              # the plain entry needs up


@pytest.mark.parametrize("T", [1, 32])
def test_gemma4_26b_shaped_moe(T):
    """The geometry the reference admits for its Gemma-4 26B expert lane (src/gemma4_runtime.rs:
    3389-3397, 4068-4079): 128 experts, top-8, hidden 2816, expert width 704, Q4_0, fused gate|up."""
    E, k, hidden, ff = 128, 8, 2816, 704
    G.say(f"Gemma-4 26B-shaped MoE T={T}: building 128 experts")
    gate_up, down = _experts_fused(B.CML_Q4_0, B.CML_Q4_0, E, hidden, ff, 380)
    rng = np.random.default_rng(381 + T)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    logits = (rng.standard_normal((T, E)) * 2).astype(np.float32)
    ds = rng.uniform(0.5, 2.0, E).astype(np.float32)
    wgu = Weight.upload(B.CML_Q4_0, E * 2 * ff, hidden, gate_up)
    wd = Weight.upload(B.CML_Q4_0, E * hidden, ff, down)
    idx_dev, w_dev, idx, w = gpu_route_softmax(logits, k, ds)
    G.say(f"Gemma-4 26B-shaped MoE T={T}: device run")
    got = gpu_moe(wgu, None, wd, E, k, idx_dev, w_dev, x, glu=GLU_GELU_TANH)
    tt = min(T, 4)
    want = oracle.moe_ffn_ex(B.CML_Q4_0, gate_up, None, down, E, k, hidden, ff, logits[:tt], x[:tt], variant=1,
                             down_scale=ds, threads=16)
    assert G.max_rel(got[:tt], want) <= 1e-5
    assert np.all(np.isfinite(got))
    if T > tt:   # the rest of the batch: the same cells as a single-token call (bit for bit: one chain per cell)
        one = gpu_moe(wgu, None, wd, E, k, *gpu_route_softmax(logits[T - 1:T], k, ds)[:2], x[T - 1:T], glu=GLU_GELU_TANH)
        assert G.same_bits(got[T - 1:T], one)


# ---------------------------------------------------------------- the pieces ----

def gpu_plan(idx, E):
    idx = np.ascontiguousarray(idx, np.int32)
    T, k = idx.shape
    d_idx = DeviceBuffer.from_numpy(idx)
    off, tok = DeviceBuffer((E + 1) * 4), DeviceBuffer(max(1, T * k) * 4)
    r2a, uni = DeviceBuffer(max(1, T * k) * 4), DeviceBuffer(E * 4)
    for b in (off, tok, r2a, uni):
        b.fill(0x7F)
    check(lib().cml_moe_plan(d_idx.ptr, T, k, E, off.ptr, tok.ptr, r2a.ptr, uni.ptr, None), "cml_moe_plan")
    check(lib().cml_stream_sync(None))
    return (off, tok, r2a, uni), (off.to_numpy(np.int32, (E + 1,)), tok.to_numpy(np.int32, (T * k,)),
                                  r2a.to_numpy(np.int32, (T * k,)), uni.to_numpy(np.int32, (E,)))


@pytest.mark.parametrize("T,k,E", [(1, 2, 8), (7, 3, 6), (32, 8, 128), (100, 8, 128), (600, 8, 128), (300, 1, 5)])
def test_moe_plan_is_a_stable_grouping(T, k, E):
    """The route-union plan (reference gemma4_plan_route_union, src/gemma4_runtime.rs:12309-12424):
    a stable sort of the routed slots by expert, checked against numpy's stable argsort."""
    rng = np.random.default_rng(390 + T)
    idx = np.stack([rng.permutation(E)[:k] for _ in range(T)]).astype(np.int32)
    if T >= 7:
        idx[:, 0] = 3 % E          # crowd one expert across waves and passes
        idx[2, k - 1] = E + 5      # ids out of range are dropped
        idx[5, k - 1] = -1
    G.say(f"moe plan T={T} k={k} E={E}")
    _, (off, tok, r2a, uni) = gpu_plan(idx, E)
    flat = idx.reshape(-1)
    valid = (flat >= 0) & (flat < E)
    order = np.flatnonzero(valid)[np.argsort(flat[valid], kind="stable")]
    counts = np.bincount(flat[valid], minlength=E)
    assert list(off) == [0] + list(np.cumsum(counts))
    assert list(tok[:order.size]) == list(order // k)
    want_r2a = np.full(T * k, -1, np.int32)
    want_r2a[order] = np.arange(order.size)
    assert list(r2a) == list(want_r2a)
    used = np.flatnonzero(counts)
    assert list(uni) == list(used) + [-1] * (E - used.size)


@pytest.mark.parametrize("fmt,fmt_down,hidden,ff", [(B.CML_Q4_K, B.CML_Q4_K, 512, 256), (B.CML_Q4_0, B.CML_Q8_0, 352, 96)])
@pytest.mark.parametrize("T", [1, 9])
def test_moe_pieces_compose_to_the_whole(fmt, fmt_down, hidden, ff, T):
    """plan + quantize + routed matvec (gate|up) + gated activation + routed matvec (down) +
    weighted sum through the separate entry points = cml_moe_ffn_ex, bit for bit."""
    E, k = 16, 4
    L = lib()
    gate_up, down = _experts_fused(fmt, fmt_down, E, hidden, ff, 400)
    rng = np.random.default_rng(401 + T)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[:, 2] += 3.0
    wgu = Weight.upload(fmt, E * 2 * ff, hidden, gate_up)
    wd = Weight.upload(fmt_down, E * hidden, ff, down)
    idx_dev, w_dev, idx, w = gpu_route_softmax(logits, k)
    G.say(f"moe pieces vs whole fmt={fmt}/{fmt_down} T={T}")
    with G.env(CAMELID_HIP_EXACT_ORDER="1"):
        whole = gpu_moe(wgu, None, wd, E, k, idx_dev, w_dev, x, glu=GLU_GELU_TANH)
        (off, tok, r2a, uni), _ = gpu_plan(idx, E)
        A = T * k
        act_in = ACT_Q8_K if fmt == B.CML_Q4_K else ACT_Q8_0
        act_mid = ACT_Q8_K if fmt_down == B.CML_Q4_K else ACT_Q8_0
        per_in, per_mid = (256 if act_in == ACT_Q8_K else 32), (256 if act_mid == ACT_Q8_K else 32)
        xd = DeviceBuffer.from_numpy(x)
        xq, xs = DeviceBuffer(T * hidden), DeviceBuffer(T * (hidden // per_in) * 4)
        quant = L.cml_quantize_q8_k if act_in == ACT_Q8_K else L.cml_quantize_q8_0
        check(quant(xd.ptr, T, hidden, xq.ptr, xs.ptr, None))
        gu = DeviceBuffer(A * 2 * ff * 4)
        check(L.cml_moe_gemv_routed(wgu.handle, E, xq.ptr, xs.ptr, off.ptr, tok.ptr, uni.ptr, min(E, A), T, gu.ptr, None),
              "cml_moe_gemv_routed gate|up")
        check(L.cml_stream_sync(None))
        g_u = gu.to_numpy(np.float32, (A, 2, ff))
        gd = DeviceBuffer.from_numpy(np.ascontiguousarray(g_u[:, 0]))
        ud = DeviceBuffer.from_numpy(np.ascontiguousarray(g_u[:, 1]))
        hq, hs = DeviceBuffer(A * ff), DeviceBuffer(A * (ff // per_mid) * 4)
        check(L.cml_glu_quantize(GLU_GELU_TANH, act_mid, gd.ptr, ud.ptr, A, ff, hq.ptr, hs.ptr, None), "cml_glu_quantize")
        y = DeviceBuffer(A * hidden * 4)
        check(L.cml_moe_gemv_routed(wd.handle, E, hq.ptr, hs.ptr, off.ptr, None, None, 0, T, y.ptr, None), "cml_moe_gemv_routed down")
        out = DeviceBuffer(T * hidden * 4)
        check(L.cml_moe_weighted_sum(y.ptr, r2a.ptr, w_dev.ptr, T, k, hidden, out.ptr, None), "cml_moe_weighted_sum")
        check(L.cml_stream_sync(None))
    assert G.same_bits(out.to_numpy(np.float32, (T, hidden)), whole)


def test_moe_pieces_reject_bad_arguments():
    L = lib()
    d = DeviceBuffer(1 << 16)
    w6 = Weight.upload(B.CML_Q6_K, 256, 256, G.synth_weight(B.CML_Q6_K, 256, 256, 410))
    w4 = Weight.upload(B.CML_Q4_0, 96, 64, G.synth_weight(B.CML_Q4_0, 96, 64, 411))
    assert L.cml_moe_plan(d.ptr, 4, 2, 129, d.ptr, d.ptr, d.ptr, d.ptr, None) == 6
    assert L.cml_moe_plan(d.ptr, 4, 0, 8, d.ptr, d.ptr, d.ptr, d.ptr, None) == 3
    assert L.cml_moe_plan(None, 4, 2, 8, d.ptr, d.ptr, d.ptr, d.ptr, None) == 2
    assert L.cml_moe_gemv_routed(w6.handle, 3, d.ptr, d.ptr, d.ptr, None, None, 0, 1, d.ptr, None) == 3   # 256 rows, 3 experts
    assert L.cml_moe_gemv_routed(w4.handle, 5, d.ptr, d.ptr, d.ptr, None, None, 0, 1, d.ptr, None) == 3   # 96 rows, 5 experts
    assert L.cml_moe_gemv_routed(w4.handle, 4, None, d.ptr, d.ptr, None, None, 0, 1, d.ptr, None) == 2
    assert L.cml_moe_gemv_routed(w4.handle, 4, d.ptr, d.ptr, d.ptr, None, None, 0, 0, d.ptr, None) == 0   # nothing routed
    assert L.cml_moe_weighted_sum(None, None, d.ptr, 1, 2, 64, d.ptr, None) == 2
    assert L.cml_moe_weighted_sum(d.ptr, None, d.ptr, 0, 2, 64, d.ptr, None) == 0


def test_weighted_sum_maps_grouped_assignments_in_router_order_bitwise():
    """The reference's own fixture for the routed weighted sum (moe_weighted_sum_batched_maps_csr_
    assignments_in_router_order_bitwise, src/cuda_resident/tests.rs:12603-12735): 15 tokens x 8
    routes over 32 experts, expert of (token, route) = (7*route + 3*token) % 32, experts reused
    across tokens, so the grouped order is not router order.  The plan built on the device must be
    the expert-major map the fixture constructs, and the sum must walk ranks 0..7 with a separately
    rounded multiply and add."""
    T, R, E, hidden = 15, 8, 32, 2816
    experts = np.array([[(r * 7 + t * 3) % E for r in range(R)] for t in range(T)], np.int32)
    assert all(len(set(row)) == R for row in experts)
    want_map = np.full(T * R, -1, np.int32)
    n = 0
    for e in range(E):
        for t in range(T):
            for r in range(R):
                if experts[t, r] == e:
                    want_map[t * R + r] = n
                    n += 1
    assert n == T * R and list(want_map) != list(range(T * R))
    G.say("moe weighted sum: reference fixture 15x8 over 32 experts")
    (off, tok, r2a, uni), (_, _, got_map, _) = gpu_plan(experts, E)
    assert list(got_map) == list(want_map)
    rng = np.random.default_rng(420)
    y = (rng.standard_normal((T * R, hidden)) * (1 + np.arange(T * R)[:, None] / 64.0)).astype(np.float32)
    scales = (0.0125 + (np.arange(T * R) % R) * 0.017 + rng.uniform(0, 0.01, T * R)).astype(np.float32)
    yd, sd = DeviceBuffer.from_numpy(y), DeviceBuffer.from_numpy(scales)
    out = DeviceBuffer(T * hidden * 4)
    check(lib().cml_moe_weighted_sum(yd.ptr, r2a.ptr, sd.ptr, T, R, hidden, out.ptr, None), "cml_moe_weighted_sum")
    check(lib().cml_stream_sync(None))
    got = out.to_numpy(np.float32, (T, hidden))
    want = np.zeros((T, hidden), np.float32)
    for t in range(T):
        for r in range(R):
            want[t] = want[t] + (y[want_map[t * R + r]] * scales[t * R + r]).astype(np.float32)
    assert G.same_bits(got, want) and np.any(got != 0)
    # a malformed map entry is skipped, not read
    bad = want_map.copy()
    bad[5] = T * R + 7
    bd = DeviceBuffer.from_numpy(bad)
    check(lib().cml_moe_weighted_sum(yd.ptr, bd.ptr, sd.ptr, T, R, hidden, out.ptr, None))
    check(lib().cml_stream_sync(None))
    got = out.to_numpy(np.float32, (T, hidden))
    want0 = np.zeros(hidden, np.float32)
    for r in range(R):
        if r != 5:
            want0 = want0 + (y[want_map[r]] * scales[r]).astype(np.float32)
    assert G.same_bits(got[0], want0)


@pytest.mark.parametrize("fmt", [B.CML_Q4_0, B.CML_Q8_0])
def test_moe_batches_on_the_matrix_cores_are_bitwise_the_packed_dot_path(fmt):
    """Enough assignments per expert send the Q8_0 / Q4_0 expert projections to the matrix-core
    kernel (grouped mode): the same cells as the packed-dot grouped kernel, bit for bit."""
    E, k, hidden, ff, T = 8, 2, 512, 256, 70
    gate_up, down = _experts_fused(fmt, fmt, E, hidden, ff, 430)
    rng = np.random.default_rng(431)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[:, 5] += 2.0       # one crowded expert: several 16-token blocks in its group
    logits[:, 1] -= 50.0      # and one that nobody picks
    wgu = Weight.upload(fmt, E * 2 * ff, hidden, gate_up)
    wd = Weight.upload(fmt, E * hidden, ff, down)
    idx_dev, w_dev, idx, w = gpu_route_softmax(logits, k)
    assert 1 not in idx
    G.say(f"moe matrix-core grouped fmt={fmt} T={T}")
    with G.env(CAMELID_HIP_B32_MFMA_MIN_GROUP=1 << 30):
        packed = gpu_moe(wgu, None, wd, E, k, idx_dev, w_dev, x, glu=GLU_GELU_TANH)
    for min_group in (1, 6):
        with G.env(CAMELID_HIP_B32_MFMA_MIN_GROUP=min_group):
            got = gpu_moe(wgu, None, wd, E, k, idx_dev, w_dev, x, glu=GLU_GELU_TANH)
        assert G.same_bits(got, packed)
    want = oracle.moe_ffn_ex(fmt, gate_up, None, down, E, k, hidden, ff, logits[:6], x[:6], variant=1, threads=8)
    assert G.max_rel(packed[:6], want) <= 1e-5
