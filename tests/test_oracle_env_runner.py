"""The checker's runner step over any environment (oracle/rlt_oracle.cpp, rlt_oracle_env_runner_step) against what pins it without a GPU:
on the Pendulum it must leave exactly what the checker's Pendulum runner step leaves (which the seeded SAC loop pins against the reference,
tests/test_oracle_vs_reference.py); on the other environments its per-step buffers must be the environment functions' own outputs and its
bookkeeping must follow operations_generic_per_env.h:88-104 (truncated = terminated or step limit, counters, ring rows)."""
import ctypes as C

import numpy as np
import pytest

import helpers
from helpers import capi


@pytest.fixture(scope="module")
def oracle():
    return helpers.HostBackend()


def test_generic_step_on_the_pendulum_equals_the_pendulum_runner_step(oracle):
    n, cap, limit, steps = 23, 17, 9, 60
    rng = np.random.default_rng(0)
    params = helpers.random_params(rng, [3, 16, 16, 2])
    draws = [(np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-1, 1, n)], 1).astype(np.float32), rng.standard_normal((n, 1)).astype(np.float32)) for _ in range(steps)]
    sas = capi.SasParameters(-20.0, 2.0, 1e-6, -1.0)
    # generic
    runner = helpers.EnvRunnerOnBackend(oracle, capi.ENV_PENDULUM, n, limit)
    rb = helpers.ReplayOnBackend(oracle, n, cap)
    actor = helpers.Mlp(oracle, [3, 16, 16, 2], params, n, trainable=False)
    # Pendulum-specific
    z = oracle.zeros
    states, ep_step, ep_ret, trunc = z((n, 2)), z((n,), np.uint32), z((n,)), oracle.array(np.ones(n, np.uint8))
    prunner = capi.PendulumRunner(states.ptr, ep_step.ptr, ep_ret.ptr, trunc.ptr, n, limit, capi.pendulum_parameters())
    prb = helpers.ReplayOnBackend(oracle, n, cap)
    for ini, noise in draws:
        oracle.call("env_runner_step", C.byref(runner.c), C.byref(rb.c), 2, actor.layers, actor.n, C.byref(sas), None, noise.ctypes.data, ini.ctypes.data, None, 0)
        assert oracle.lib.rlt_oracle_pendulum_runner_step(C.byref(prunner), C.byref(prb.c), 2, actor.layers, actor.n, C.byref(sas), None, noise.ctypes.data, ini.ctypes.data) == 0
        for a, b in ((runner.states, states), (runner.ep_step, ep_step), (runner.ep_ret, ep_ret), (runner.trunc, trunc)):
            assert np.array_equal(a.numpy(), b.numpy())
    for a, b in ((rb.data, prb.data), (rb.episode_start, prb.episode_start), (rb.position, prb.position), (rb.current_episode_start, prb.current_episode_start), (rb.full, prb.full)):
        assert np.array_equal(a.numpy(), b.numpy())
    assert rb.full.numpy().all()


@pytest.mark.parametrize("kind", [capi.ENV_ACROBOT, capi.ENV_CAR])
def test_bookkeeping_around_the_environments_own_step(oracle, kind):
    sd, od, ad = capi.ENV_DIMS[kind]
    n, cap, limit, steps = 40, 12, 15, 50
    rng = np.random.default_rng(kind)
    runner = helpers.EnvRunnerOnBackend(oracle, kind, n, limit)
    rb = helpers.ReplayOnBackend(oracle, n, cap, od, ad)
    R = 2 * od + ad + 3
    expected_step = np.zeros(n, np.uint32); expected_return = np.zeros(n, np.float32); truncated = np.ones(n, bool)
    position = np.zeros(n, np.int64)
    seen_termination = False
    for _ in range(steps):
        ini = (np.zeros((n, sd)) if kind == capi.ENV_CAR else rng.uniform(-0.1, 0.1, (n, sd))).astype(np.float32)
        if kind == capi.ENV_ACROBOT:
            ini[::5, 0] += 2.2      # some episodes start with the first link raised: their tip crosses the line within a few steps
        else:
            ini[::4, 0] = 0.97; ini[::4, 3] = 3.0      # some cars start at the edge of the unit square, heading out
        actions = rng.uniform(-1, 1, (n, ad)).astype(np.float32)
        before = runner.states.numpy()
        oracle.call("env_runner_step", C.byref(runner.c), C.byref(rb.c), 0, None, 0, None, actions.ctypes.data, None, ini.ctypes.data, None, 0)
        # the environment's own function on the state the step started from
        start = np.where(truncated[:, None], ini, before).astype(np.float32)
        s = start.copy(); o = np.zeros((n, od), np.float32); no = np.zeros((n, od), np.float32); r = np.zeros(n, np.float32); t = np.zeros(n, np.uint8)
        if kind == capi.ENV_CAR:
            p = capi.car_parameters(); oracle.call("car_step", C.byref(p), s.ctypes.data, actions.ctypes.data, o.ctypes.data, no.ctypes.data, r.ctypes.data, t.ctypes.data, n)
        else:
            p = capi.acrobot_parameters(); oracle.call("acrobot_step", C.byref(p), 0, s.ctypes.data, actions.ctypes.data, o.ctypes.data, no.ctypes.data, r.ctypes.data, t.ctypes.data, n)
        for got, want in ((runner.states, s), (runner.obs, o), (runner.next_obs, no), (runner.rew, r), (runner.term, t), (runner.act, actions)):
            assert np.array_equal(got.numpy(), want)
        expected_step = np.where(truncated, 0, expected_step) + 1
        expected_return = (np.where(truncated, np.float32(0), expected_return) + r).astype(np.float32)
        truncated = (t != 0) | (expected_step == limit)
        seen_termination |= bool(t.any())
        assert np.array_equal(runner.ep_step.numpy(), expected_step) and np.array_equal(runner.ep_ret.numpy(), expected_return)
        assert np.array_equal(runner.trunc.numpy() != 0, truncated)
        rows = rb.data.numpy().reshape(n, cap, R)[np.arange(n), position]
        assert np.array_equal(rows, np.concatenate([o, actions, r[:, None], no, t[:, None].astype(np.float32), truncated[:, None].astype(np.float32)], 1))
        position = (position + 1) % cap
    assert seen_termination


@pytest.mark.parametrize("standardize,truncate", [(False, 0), (True, 1)])
def test_generic_collect_on_the_pendulum_equals_the_pendulum_collect(oracle, standardize, truncate):
    """rlt_oracle_env_on_policy_collect with a policy of dense layers on the Pendulum leaves the dataset and runner state that
    rlt_oracle_on_policy_collect leaves, which the reference's PPO loop pins (tests/test_oracle_vs_reference.py)."""
    n, steps, limit, ld = 19, 23, 7, 14
    col = dict(observations=0, actions_mean=3, actions=4, action_log_probs=5, rewards=6, terminated=7, truncated=8, all_reset=9)
    rng = np.random.default_rng(3)
    dims = [3, 16, 16, 1]
    params = helpers.random_params(rng, dims)
    specs = [(0, 3, 16, "relu"), (0, 16, 16, "relu"), (0, 16, 1, "identity")]
    log_std = np.array([-0.5], np.float32)
    st = (rng.uniform(-0.2, 0.2, 3).astype(np.float32), rng.uniform(0.5, 2.0, 3).astype(np.float32)) if standardize else None
    specific = helpers.OnPolicyOnBackend(oracle, n, steps, ld, col, limit)
    actor = helpers.Mlp(oracle, dims, params, n, trainable=False)
    runner = helpers.EnvRunnerOnBackend(oracle, capi.ENV_PENDULUM, n, limit)
    policy = helpers.SeqNet(oracle, specs, params, 1, n, trainable=False)
    for _ in range(3):
        noise = rng.standard_normal((steps, n, 1)).astype(np.float32)
        ini = np.stack([rng.uniform(-np.pi, np.pi, (steps, n)), rng.uniform(-1, 1, (steps, n))], 2).astype(np.float32)
        specific.data.upload(np.zeros_like(specific.data.numpy()))
        specific.collect(actor, log_std, noise, ini, st, truncate)
        data = oracle.zeros(((steps + 1) * n, ld))
        o = data.offset
        d = capi.OnPolicyDataset(o(0), o(3), o(4), o(5), o(6), o(7), o(8), o(9), ld, steps)
        oracle.call("env_on_policy_collect", C.byref(runner.c), C.byref(d), policy.layers, policy.n, None, 0, log_std.ctypes.data, st[0].ctypes.data if st else None,
                    st[1].ctypes.data if st else None, noise.ctypes.data, ini.ctypes.data, truncate, None, 0)
        assert np.array_equal(data.numpy(), specific.data.numpy())
        for a, b in zip(runner.snapshot()[:4], (specific.states, specific.ep_step, specific.ep_ret, specific.trunc)):
            assert np.array_equal(a, b.numpy())
    assert data.numpy()[:, 9].sum() > n


def test_sequential_step_on_the_pendulum_equals_the_recurrent_pendulum_runner_step(oracle):
    """head_kind 2 (sample_and_squash) with a dense-GRU-dense policy: the generic step leaves what rlt_oracle_pendulum_runner_step_recurrent leaves, which
    the reference's recurrent SAC loop pins (tests/test_oracle_vs_reference.py, recurrent runner golden vectors)."""
    n, cap, limit, period, steps = 11, 9, 6, 4, 40
    specs = [(0, 3, 8, "relu"), (1, 8, 8, "identity"), (0, 8, 2, "identity")]
    rng = np.random.default_rng(2)
    params = helpers.random_seq_params(rng, specs)
    specific = helpers.RecurrentRunnerOnBackend(oracle, specs, params, n, cap, limit, period)
    runner = helpers.EnvRunnerOnBackend(oracle, capi.ENV_PENDULUM, n, limit)
    rb = helpers.ReplayOnBackend(oracle, n, cap)
    policy = helpers.SeqNet(oracle, specs, params, 1, n, trainable=False)
    state = helpers.SeqStateOnBackend(oracle, specs, n)
    sas = capi.SasParameters(-20.0, 2.0, 1e-6, -1.0)
    for _ in range(steps):
        noise = rng.standard_normal((n, 1)).astype(np.float32)
        ini = np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-1, 1, n)], 1).astype(np.float32)
        specific.step(noise, ini)
        oracle.call("env_runner_step_sequential", C.byref(runner.c), C.byref(rb.c), policy.layers, policy.n, C.byref(state.c), period, 2, C.byref(sas), 0.0, noise.ctypes.data,
                    ini.ctypes.data, None, 0)
        want = specific.numpy()
        for a, b in ((runner.states, want["states"]), (runner.ep_step, want["episode_step"]), (runner.ep_ret, want["episode_return"]), (runner.trunc, want["truncated"]),
                     (rb.data, want["data"]), (rb.position, want["position"]), (rb.episode_start, want["episode_start"])):
            assert np.array_equal(a.numpy(), b)
        hidden, counters = state.numpy()
        assert all(np.array_equal(a, b) for a, b in zip(hidden, want["hidden"])) and all(np.array_equal(a, b) for a, b in zip(counters, want["steps"]))
    assert rb.full.numpy().all()
