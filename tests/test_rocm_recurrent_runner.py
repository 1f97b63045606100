"""Rollout with a sequential (recurrent) policy through the C ABI: the policy's kept state, evaluate_step, and the off-policy runner step on the Pendulum,
against the CPU checker and the reference's own run (fixture).

Tolerance: 1e-5 relative to the largest magnitude of the reference tensor for floating point; counters, flags and ring cursors exactly."""
import ctypes as C

import numpy as np
import pytest

import helpers
from helpers import rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-5
EXACT = ("episode_step", "truncated", "steps", "position", "current_episode_start")
CLOSE = ("states", "episode_return", "hidden", "rows", "previous_truncated")


def test_recurrent_runner_step_against_reference_vectors(oracle, rocm):
    """Every fixture step on the device from the checker's state (which itself must land on the fixture bit for bit)."""
    g = helpers.recurrent_runner_golden()
    cpu, steps = helpers.recurrent_runner_from_golden(oracle, g)
    gpu, _ = helpers.recurrent_runner_from_golden(rocm, g)
    for i in range(steps):
        print("step", i, flush=True)
        before = cpu.numpy()
        gpu.load(dict(before, hidden=before["hidden"], steps=before["steps"]),
                 [(before["data"].reshape(cpu.n, -1, 10)[e], before["position"][e], before["full"][e], before["current_episode_start"][e],
                   before["episode_start"].reshape(cpu.n, -1)[e]) for e in range(cpu.n)])
        want = helpers.recurrent_runner_golden_step(cpu, g, i)
        got = helpers.recurrent_runner_golden_step(gpu, g, i)
        for k in EXACT:
            assert np.array_equal(got[k], want[k]), (i, k, got[k], want[k])
            assert np.array_equal(want[k], g[f"s{i}_{k}"]), (i, k)
        for k in CLOSE:
            assert rel_err(got[k], want[k]) <= TOL, (i, k, rel_err(got[k], want[k]))


@pytest.mark.parametrize("case", [(4096, 64, 2, True, 5), (1000, 32, 1, False, 0), (65536, 16, 1, True, 100)])
def test_recurrent_runner_step_many_environments(oracle, rocm, case):
    """Many environments, wider and deeper policies, three steps each from the checker's state; episodes of 2 steps so that resets occur, an auto-reset
    period inside the run (or none)."""
    print("case", case, flush=True)
    N, H, n_gru, fast, period = case
    rng = np.random.default_rng(N + H)
    specs = [(0, 3, H, "relu")] + [(1, H, H, "identity")] * n_gru + [(0, H, 2, "identity")]
    params = helpers.random_seq_params(rng, specs)
    runs = [helpers.RecurrentRunnerOnBackend(be, specs, params, N, 8, 2, period) for be in (oracle, rocm)]
    for r in runs:
        for l in r.state.hidden:
            r.policy.layers[l].gru.fast_tanh = int(fast)
    for i in range(3):
        noise, ini = rng.standard_normal(N).astype(np.float32), np.stack([rng.uniform(-np.pi, np.pi, N), rng.uniform(-1, 1, N)], 1).astype(np.float32)
        before = runs[0].numpy()
        r = runs[1]
        r.states.upload(before["states"]); r.ep_step.upload(before["episode_step"]); r.ep_ret.upload(before["episode_return"]); r.trunc.upload(before["truncated"])
        r.state.set(before["hidden"], before["steps"])
        r.rb.data.upload(before["data"]); r.rb.position.upload(before["position"]); r.rb.full.upload(before["full"])
        r.rb.current_episode_start.upload(before["current_episode_start"]); r.rb.episode_start.upload(before["episode_start"])
        for r in runs:
            r.step(noise, ini)
        want, got = runs[0].numpy(), runs[1].numpy()
        for k in ("episode_step", "truncated", "position", "full", "current_episode_start", "episode_start"):
            assert np.array_equal(got[k], want[k]), (i, k)
        for l in range(n_gru):
            assert np.array_equal(got["steps"][l], want["steps"][l]), (i, l)
            assert rel_err(got["hidden"][l], want["hidden"][l]) <= TOL, (i, l, rel_err(got["hidden"][l], want["hidden"][l]))
        for k in ("states", "episode_return", "data"):
            assert rel_err(got[k], want[k]) <= TOL, (i, k, rel_err(got[k], want[k]))
    assert want["truncated"].any() or (want["episode_step"] < 2).any()


@pytest.mark.parametrize("H", [16, 64, 24])
def test_evaluate_step_chain_equals_sequence_forward_on_device(rocm, H):
    """S single steps on the kept state against one forward pass over the sequence with the same resets (two different sets of kernels of the library)."""
    rng = np.random.default_rng(H)
    S, B, I, O = 9, 37, 5, 3
    specs = [(0, I, H, "tanh"), (1, H, H, "identity"), (0, H, O, "identity")]
    params = helpers.random_seq_params(rng, specs)
    x = rng.standard_normal((S, B, I)).astype(np.float32)
    reset = (rng.uniform(size=(S, B)) < 0.15).astype(np.uint8)
    net = helpers.SeqNet(rocm, specs, params, S, B)
    ws, wsn = net.workspace()
    xd, rd = rocm.array(x), rocm.array(reset)
    rocm.call("seq_forward", net.layers, net.n, xd.ptr, I, rd.ptr, S, B, ws, wsn)
    rocm.sync()
    want = net.output().reshape(S, B, O)
    state = helpers.SeqStateOnBackend(rocm, specs, B)
    rocm.call("seq_reset_state", net.layers, net.n, C.byref(state.c), None, B)
    n = int(rocm.device.lib.rlt_rocm_seq_evaluate_step_workspace_bytes(net.layers, net.n, B))
    sws = rocm.device.empty((n,), np.uint8)
    y = rocm.zeros((B, O))
    for t in range(S):
        m = rocm.array(reset[t])
        if t:
            rocm.call("seq_reset_state", net.layers, net.n, C.byref(state.c), m.ptr, B)
        xt = rocm.array(x[t])
        rocm.call("seq_evaluate_step", net.layers, net.n, xt.ptr, I, C.byref(state.c), 0, y.ptr, O, B, sws.ptr, n)
        rocm.sync()
        assert rel_err(y.numpy(), want[t]) <= TOL, (t, rel_err(y.numpy(), want[t]))
    assert rocm.device.lib.rlt_rocm_seq_evaluate_step(rocm.device.handle, net.layers, net.n, xd.ptr, I, C.byref(state.c), 0, y.ptr, O, B, sws.ptr, 16) == helpers.capi.RLT_E_INVALID_ARGUMENT
