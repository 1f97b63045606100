"""Evaluation episodes on the device (rlt_rocm_pendulum_evaluate) against the CPU checker and the reference's own results, through the C ABI.

Tolerance: fp32 rollouts of a closed loop amplify rounding differences step by step, so returns are compared at 1e-5 relative over short horizons
(20 steps) and at 2e-3 over the reference's 200 steps; episode lengths and the terminated counts are integers and must be equal."""
import os

import numpy as np
import pytest

import helpers
from helpers import rel_err

pytestmark = pytest.mark.gpu


def test_evaluation_against_reference_vectors(rocm):
    """The SAC actor after 0, 150, 400 and 6,000 loop steps, 10 episodes x 200 steps from the initial states the reference drew: the reference's returns
    and statistics (tests/golden/evaluation_pendulum_seed0.npz)."""
    g = np.load(os.path.join(helpers.GOLDEN, "evaluation_pendulum_seed0.npz"))
    for k in range(len(g["stops"])):
        ret, length, summary = helpers.evaluate_on_backend(rocm, [3, 64, 64, 2], g[f"e{k}_actor"], "relu", "identity", 2, g[f"e{k}_initial_states"], 200)
        assert np.array_equal(length, g[f"e{k}_episode_length"])
        assert rel_err(ret, g[f"e{k}_returns"]) <= 2e-3, (k, ret, g[f"e{k}_returns"])
        assert rel_err(summary[:2], g[f"e{k}_summary"][:2]) <= 2e-3 and np.array_equal(summary[2:], g[f"e{k}_summary"][2:])


# (hidden width, layers, policy kind, hidden activation, output activation, episodes): one launch for three layers of width <= 64, else step by step
CASES = [(64, 3, 2, "relu", "identity", 10), (64, 3, 1, "tanh", "tanh", 100), (32, 3, 1, "relu", "tanh", 7), (17, 3, 2, "fast_tanh", "identity", 64),
         (256, 3, 2, "relu", "identity", 33), (64, 2, 1, "tanh", "tanh", 10), (48, 4, 2, "relu", "identity", 300)]


@pytest.mark.parametrize("case", CASES)
def test_evaluation_matches_checker(oracle, rocm, case):
    print("case", case, flush=True)
    H, layers, kind, ha, oa, n = case
    dims = [3] + [H] * (layers - 1) + [kind]
    rng = np.random.default_rng(H + n)
    params = helpers.random_params(rng, dims)
    ini = np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-1, 1, n)], 1).astype(np.float32)
    for steps, tol in ((20, 1e-5), (200, 2e-3)):
        want = helpers.evaluate_on_backend(oracle, dims, params, ha, oa, kind, ini, steps)
        got = helpers.evaluate_on_backend(rocm, dims, params, ha, oa, kind, ini, steps)
        assert np.array_equal(got[1], want[1]) and np.all(got[1] == steps)
        assert rel_err(got[0], want[0]) <= tol, (steps, rel_err(got[0], want[0]))
        assert rel_err(got[2][:2], want[2][:2]) <= tol and np.array_equal(got[2][2:], want[2][2:])


@pytest.mark.parametrize("case", [(32, 3, 1, "fast_tanh", "identity", 100), (64, 3, 1, "tanh", "identity", 10), (128, 3, 1, "tanh", "identity", 16), (16, 3, 2, "relu", "identity", 5)])
def test_evaluation_with_a_standardize_layer_matches_checker(oracle, rocm, case):
    """PPO's actors: (observation - mean) * precision in front of the first layer (one launch for widths <= 64, step by step above)."""
    print("case", case, flush=True)
    H, layers, kind, ha, oa, n = case
    dims = [3] + [H] * (layers - 1) + [kind]
    rng = np.random.default_rng(3 * H + n)
    params = helpers.random_params(rng, dims)
    ini = np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-1, 1, n)], 1).astype(np.float32)
    standardize = (rng.normal(0, 0.5, 3).astype(np.float32), rng.uniform(0.3, 3, 3).astype(np.float32))
    plain = helpers.evaluate_on_backend(rocm, dims, params, ha, oa, kind, ini, 20)
    for steps, tol in ((20, 1e-5), (200, 2e-3)):
        want = helpers.evaluate_on_backend(oracle, dims, params, ha, oa, kind, ini, steps, standardize)
        got = helpers.evaluate_on_backend(rocm, dims, params, ha, oa, kind, ini, steps, standardize)
        assert np.array_equal(got[1], want[1]) and np.all(got[1] == steps)
        assert rel_err(got[0], want[0]) <= tol, (steps, rel_err(got[0], want[0]))
        assert rel_err(got[2][:2], want[2][:2]) <= tol and np.array_equal(got[2][2:], want[2][2:])
        if steps == 20:
            assert rel_err(got[0], plain[0]) > 1e-3      # the layer is not ignored


def test_evaluation_rejects_bad_arguments(rocm):
    capi = helpers.capi
    import ctypes as C
    dims = [3, 64, 64, 2]
    actor = helpers.Mlp(rocm, dims, helpers.random_params(np.random.default_rng(0), dims), 4, trainable=False)
    ini, ret, length, summary = rocm.zeros((4, 2)), rocm.zeros((4,)), rocm.zeros((4,), np.uint32), rocm.zeros((6,))
    env = capi.pendulum_parameters()
    lib, h = rocm.device.lib, rocm.device.handle
    bad = capi.RLT_E_INVALID_ARGUMENT if hasattr(capi, "RLT_E_INVALID_ARGUMENT") else -1
    assert lib.rlt_rocm_pendulum_evaluate(h, C.byref(env), 1, actor.layers, 3, ini.ptr, 4, 10, ret.ptr, length.ptr, summary.ptr) != 0      # kind 1 needs one output
    assert lib.rlt_rocm_pendulum_evaluate(h, C.byref(env), 2, actor.layers, 3, ini.ptr, 0, 10, ret.ptr, length.ptr, summary.ptr) != 0
    assert lib.rlt_rocm_pendulum_evaluate(h, C.byref(env), 2, actor.layers, 3, None, 4, 10, ret.ptr, length.ptr, summary.ptr) != 0
    assert lib.rlt_rocm_pendulum_evaluate(h, C.byref(env), 2, actor.layers, 3, ini.ptr, 4, 10, ret.ptr, length.ptr, summary.ptr) == 0
    rocm.sync()


def test_evaluation_of_a_trained_actor_on_both_device_paths(oracle, rocm, monkeypatch):
    """A trained actor holds the pendulum at its unstable equilibrium for most of the 200 steps: 100 episodes on the one-launch kernel, on the per-step
    kernels of the same library and on the checker must agree episode by episode. (A wavefront of the one-launch kernel keeps a copy of the episode's
    state in every lane; copies that differ in the last bit feed the network a state no pendulum is in, and the balanced pendulum is lost within 100
    steps -- returns then differ by hundreds.)"""
    g = np.load(os.path.join(helpers.GOLDEN, "evaluation_pendulum_seed0.npz"))
    params = g["e3_actor"]
    rng = np.random.default_rng(11)
    ini = np.stack([rng.uniform(-np.pi, np.pi, 100), rng.uniform(-1, 1, 100)], 1).astype(np.float32)
    want = helpers.evaluate_on_backend(oracle, [3, 64, 64, 2], params, "relu", "identity", 2, ini, 200)
    one_launch = helpers.evaluate_on_backend(rocm, [3, 64, 64, 2], params, "relu", "identity", 2, ini, 200)
    monkeypatch.setenv("RLT_EVALUATE_ONE_LAUNCH", "0")
    per_step = helpers.evaluate_on_backend(rocm, [3, 64, 64, 2], params, "relu", "identity", 2, ini, 200)
    assert want[2][0] > -250 and (want[0] > -20).sum() >= 5          # trained: several episodes are balanced from the start
    for got in (one_launch, per_step):
        assert np.abs(got[0] - want[0]).max() <= 0.05, np.abs(got[0] - want[0]).max()
        assert abs(got[2][0] - want[2][0]) <= 0.01


def test_evaluation_with_recurrent_policy_against_reference_vectors(oracle, rocm):
    """The reference's recurrent SAC actor (one and two GRU layers, hidden state restarting every 6 steps), 5 episodes x 40 steps from the initial states the
    reference drew: the reference's returns and statistics (tests/golden/evaluation_recurrent_pendulum.npz), and the policy state the run leaves."""
    n = 0
    for label, specs, params, period, ini, step_limit, ret, length, summary in helpers.evaluation_recurrent_golden_cases(helpers.evaluation_recurrent_golden()):
        print("case", label, flush=True)
        got, want = (helpers.evaluate_recurrent(be, specs, params, period, ini, step_limit) for be in (rocm, oracle))
        assert np.array_equal(got["length"], length) and rel_err(got["returns"], ret) <= 1e-4, (label, got["returns"], ret)
        assert rel_err(got["summary"][:2], summary[:2]) <= 1e-4 and np.array_equal(got["summary"][2:], summary[2:])
        for a, b in zip(got["steps"], want["steps"]):
            assert np.array_equal(a, b)
        for a, b in zip(got["hidden"], want["hidden"]):
            assert rel_err(a, b) <= 1e-4
        n += 1
    assert n == 6


@pytest.mark.parametrize("case", [(16, 1, True, 6, 2, 10), (64, 2, False, 50, 2, 300), (32, 1, True, 0, 1, 4096), (24, 2, True, 7, 2, 33)])
def test_evaluation_with_recurrent_policy_matches_checker(oracle, rocm, case):
    """Other widths (register-resident and generic GRU step kernels), depths, exact and fast gates, restart periods (0: never), both policy kinds, many episodes."""
    print("case", case, flush=True)
    H, n_gru, fast, period, kind, n = case
    rng = np.random.default_rng(H + n)
    specs = [(0, 3, H, "relu")] + [(1, H, H, "identity")] * n_gru + [(0, H, kind, "identity" if kind == 2 else "tanh")]
    params = helpers.random_seq_params(rng, specs)
    ini = np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-1, 1, n)], 1).astype(np.float32)
    for steps, tol in ((20, 1e-5), (200, 2e-3)):
        want, got = (helpers.evaluate_recurrent(be, specs, params, period, ini, steps, kind, fast) for be in (oracle, rocm))
        assert np.array_equal(got["length"], want["length"]) and np.all(got["length"] == steps)
        assert rel_err(got["returns"], want["returns"]) <= tol, (steps, rel_err(got["returns"], want["returns"]))
        assert rel_err(got["summary"][:2], want["summary"][:2]) <= tol and np.array_equal(got["summary"][2:], want["summary"][2:])
        for a, b in zip(got["steps"], want["steps"]):
            assert np.array_equal(a, b)


def test_evaluation_with_recurrent_policy_rejects_bad_arguments(rocm):
    import ctypes as C
    capi = helpers.capi
    specs = [(0, 3, 16, "relu"), (1, 16, 16, "identity"), (0, 16, 2, "identity")]
    N = 4
    policy = helpers.SeqNet(rocm, specs, helpers.random_seq_params(np.random.default_rng(0), specs), 1, N, trainable=False)
    state = helpers.SeqStateOnBackend(rocm, specs, N)
    ini, ret, length, summary = rocm.zeros((N, 2)), rocm.zeros((N,)), rocm.zeros((N,), np.uint32), rocm.zeros((6,))
    env = capi.pendulum_parameters()
    lib, h = rocm.device.lib, rocm.device.handle
    wsn = int(lib.rlt_rocm_pendulum_evaluate_recurrent_workspace_bytes(policy.layers, policy.n, N))
    ws = rocm.device.empty((wsn,), np.uint8)
    call = lambda kind, n, period, w, wn: lib.rlt_rocm_pendulum_evaluate_recurrent(h, C.byref(env), kind, policy.layers, policy.n, C.byref(state.c), period, ini.ptr, n, 10,
                                                                                    ret.ptr, length.ptr, summary.ptr, w, wn)
    assert call(1, N, 6, ws.ptr, wsn) != 0           # kind 1 needs one output
    assert call(2, 0, 6, ws.ptr, wsn) != 0
    assert call(2, N, -1, ws.ptr, wsn) != 0
    assert call(2, N, 6, ws.ptr, wsn // 2) != 0      # workspace too small
    assert call(2, N, 6, None, 0) != 0
    assert call(2, N, 6, ws.ptr, wsn) == 0
    rocm.sync()

