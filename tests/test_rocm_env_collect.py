"""On-policy collection over every batched environment with MLP and recurrent policies (rl/components/on_policy_runner/operations_generic.h:105-146,
operations_generic_per_env.h:8-74): the HIP path against the CPU checker on the same draws. Flags and counters bit-exact; floats to 1e-5 of each
column's largest magnitude (1e-4 on the Acrobot, whose double-precision sub-expressions the kernel computes in float)."""
import ctypes as C

import numpy as np
import pytest

import helpers
from helpers import capi, rel_err
from test_rocm_env_runner import initial_states

pytestmark = pytest.mark.gpu


def columns(od, ad):
    col, o = {}, 0
    for name, width in (("observations", od), ("actions_mean", ad), ("actions", ad), ("action_log_probs", 1), ("rewards", 1), ("terminated", 1), ("truncated", 1), ("all_reset", 1)):
        col[name] = o; o += width
    return col, o + 3      # a few unused columns: the row stride is not the sum of the widths


def collect(backend, kind, specs, params, n, steps, limit, log_std, noise, ini, standardize, truncate, iterations):
    sd, od, ad = capi.ENV_DIMS[kind]
    col, ld = columns(od, ad)
    runner = helpers.EnvRunnerOnBackend(backend, kind, n, limit)
    policy = helpers.SeqNet(backend, specs, params, 1, n, trainable=False)
    state = helpers.SeqStateOnBackend(backend, specs, n)
    recurrent = any(k for k, *_ in specs)
    out = []
    for it in range(iterations):
        data = backend.zeros(((steps + 1) * n, ld))
        o = data.offset
        d = capi.OnPolicyDataset(o(col["observations"]), o(col["actions_mean"]), o(col["actions"]), o(col["action_log_probs"]), o(col["rewards"]), o(col["terminated"]),
                                 o(col["truncated"]), o(col["all_reset"]), ld, steps)
        ls, nz, ii = backend.array(log_std), backend.array(noise[it]), backend.array(ini[it])
        sm = backend.array(standardize[0]) if standardize else None; sp = backend.array(standardize[1]) if standardize else None
        ws, wsn = (None, 0)
        if backend.name == "rocm":
            ws, wsn = backend.workspace(backend.device.lib.rlt_rocm_env_on_policy_collect_workspace_bytes(C.byref(runner.c), policy.layers, policy.n))
        backend.call("env_on_policy_collect", C.byref(runner.c), C.byref(d), policy.layers, policy.n, C.byref(state.c) if recurrent else None, 8, ls.ptr,
                     sm.ptr if sm else None, sp.ptr if sp else None, nz.ptr, ii.ptr, truncate, ws, wsn)
        backend.sync()
        out.append((data.numpy(), runner.snapshot()[:4], state.numpy()))
    return out, col


CASES = [  # environment, policy layers (kind, in, out, activation), n_envs, steps, step limit, standardize, truncate_on_each_iteration
    (capi.ENV_PENDULUM, [(0, 3, 16, "relu"), (1, 16, 16, "identity"), (0, 16, 1, "identity")], 33, 24, 10, False, 0),      # recurrent policy: state reset at episode ends
    (capi.ENV_ACROBOT, [(0, 6, 32, "tanh"), (0, 32, 32, "tanh"), (0, 32, 1, "identity")], 64, 20, 15, True, 0),
    (capi.ENV_ACROBOT_SWINGUP, [(0, 6, 16, "relu"), (1, 16, 16, "identity"), (1, 16, 16, "identity"), (0, 16, 1, "identity")], 20, 16, 0, False, 1),
    (capi.ENV_CAR, [(0, 6, 32, "relu"), (0, 32, 2, "tanh")], 50, 30, 12, False, 0),
]


@pytest.mark.parametrize("kind,specs,n,steps,limit,standardize,truncate", CASES)
def test_collect_matches_the_checker(oracle, rocm, kind, specs, n, steps, limit, standardize, truncate):
    sd, od, ad = capi.ENV_DIMS[kind]
    rng = np.random.default_rng(kind + 7)
    params = helpers.random_seq_params(rng, specs)
    iterations = 3
    noise = [rng.standard_normal((steps, n, ad)).astype(np.float32) for _ in range(iterations)]
    ini = [np.stack([initial_states(rng, kind, n) for _ in range(steps)]) for _ in range(iterations)]
    log_std = rng.uniform(-1.0, -0.3, ad).astype(np.float32)
    st = (rng.uniform(-0.2, 0.2, od).astype(np.float32), rng.uniform(0.5, 2.0, od).astype(np.float32)) if standardize else None
    ref, col = collect(oracle, kind, specs, params, n, steps, limit, log_std, noise, ini, st, truncate, iterations)
    got, _ = collect(rocm, kind, specs, params, n, steps, limit, log_std, noise, ini, st, truncate, iterations)
    tol = 1e-4 if kind in (capi.ENV_ACROBOT, capi.ENV_ACROBOT_SWINGUP) else 1e-5
    widths = dict(observations=od, actions_mean=ad, actions=ad, action_log_probs=1, rewards=1, terminated=1, truncated=1, all_reset=1)
    resets = 0
    for (rd, rr, rs), (gd, gr, gs) in zip(ref, got):
        for name, w in widths.items():
            a, b = gd[:, col[name]:col[name] + w], rd[:, col[name]:col[name] + w]
            if name in ("terminated", "truncated", "all_reset"):
                assert np.array_equal(a, b), name
            else:
                assert rel_err(a, b) <= tol, (name, rel_err(a, b))
        assert np.array_equal(gd[:, col["all_reset"] + 1:], rd[:, col["all_reset"] + 1:])      # the unused columns stay untouched
        assert rel_err(gr[0], rr[0]) <= tol and np.array_equal(gr[1], rr[1]) and rel_err(gr[2], rr[2]) <= tol and np.array_equal(gr[3], rr[3])
        for a, b in zip(gs[0], rs[0]):
            assert rel_err(a, b) <= tol
        for a, b in zip(gs[1], rs[1]):
            assert np.array_equal(a, b)
        resets += int(rd[:, col["all_reset"]].sum())
    assert resets > n      # episodes ended and started again inside the collected steps
