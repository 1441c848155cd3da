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


def gpu_moe(gate, up, down, E, k, idx_dev, w_dev, x):
    T, hidden = x.shape
    ff = down.cols
    xd = DeviceBuffer.from_numpy(x)
    out = DeviceBuffer(T * hidden * 4)
    out.fill(0xFF)
    ws_bytes = lib().cml_moe_workspace_bytes(B.CML_Q4_K, hidden, ff, T, k, E)
    assert ws_bytes > 0
    ws = DeviceBuffer(ws_bytes)
    check(lib().cml_moe_ffn(gate.handle, up.handle, down.handle, E, k, idx_dev.ptr, w_dev.ptr, xd.ptr, T, out.ptr,
                            ws.ptr, ws_bytes, None), "cml_moe_ffn")
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
    got = gpu_moe(wg, wu, wd, E, k, idx_dev, w_dev, x)
    tt = min(T, 4)   # the oracle walks 3 full expert matvecs per (token, expert): bound the CPU work
    want = oracle.moe_ffn(B.CML_Q4_K, gate, up, down, E, k, hidden, ff, logits[:tt], x[:tt], threads=16)
    assert G.max_rel(got[:tt], want) <= 1e-5
    assert np.all(np.isfinite(got))
    if T > tt:   # the rest of the batch: same cells as single-token calls of the same entry point
        one = gpu_moe(wg, wu, wd, E, k, *gpu_route(logits[T - 1:T], k)[:2], x[T - 1:T])
        assert G.max_rel(got[T - 1:T], one) <= 1e-6
