"""Evaluation episodes over every batched environment (rlt_rocm_env_evaluate; rl/utils/evaluation/operations_generic.h:113-233) against the CPU checker,
through the C ABI: dense and recurrent policies, both heads, a standardize layer, episodes that terminate.

Tolerance: episode lengths and the terminated count are integers and must be equal; returns to 1e-5 of their largest magnitude over short horizons (the
Acrobot's to 1e-4: the kernel computes in float what the reference's dynamics compute partly in double), 2e-3 over long ones, where a closed loop amplifies
rounding differences step by step (and separates some of the Acrobot's episodes altogether: the share that stays together is checked)."""
import numpy as np
import pytest

import helpers
from helpers import capi, rel_err

pytestmark = pytest.mark.gpu


def initial_states(rng, kind, n):
    if kind == capi.ENV_PENDULUM:
        return np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-1, 1, n)], 1).astype(np.float32)
    if kind == capi.ENV_PENDULUM_POSITION:
        return np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-1, 1, n), np.zeros(n)], 1).astype(np.float32)
    if kind == capi.ENV_CAR:
        s = np.zeros((n, 6), np.float32)
        s[:, :2] = rng.uniform(-0.5, 0.5, (n, 2))
        s[::3, 0] = 0.9; s[::3, 3] = 2.0 + rng.uniform(0, 1, len(s[::3]))      # some cars start near the edge of the unit square, heading out
        return s
    if kind == capi.ENV_ACROBOT_SWINGUP:
        s = np.zeros((n, 4), np.float32)
        s[:, :2] = rng.uniform(-np.pi, np.pi, (n, 2))
        return s
    s = rng.uniform(-0.1, 0.1, (n, 4)).astype(np.float32)
    s[::4, 0] += 2.0 + rng.uniform(0, 0.3, len(s[::4]))      # some episodes start with the first link raised: the tip crosses the line within a few steps
    return s


def dense(od, width, out, hidden="relu", last="identity"):
    return [(0, od, width, hidden), (0, width, width, hidden), (0, width, out, last)]


CASES = [
    # environment, policy kind, episodes, layers of the policy (None: dense 32-32), auto-reset period, standardize
    (capi.ENV_ACROBOT, 2, 40, None, 0, False),
    (capi.ENV_ACROBOT, 1, 9, None, 0, True),
    (capi.ENV_ACROBOT_SWINGUP, 2, 100, None, 0, False),
    (capi.ENV_CAR, 2, 30, None, 0, False),
    (capi.ENV_CAR, 1, 64, None, 0, True),
    (capi.ENV_PENDULUM, 2, 17, None, 0, False),
    (capi.ENV_ACROBOT_SWINGUP, 2, 12, "gru", 8, False),
    (capi.ENV_ACROBOT, 1, 20, "gru", 0, False),
    (capi.ENV_PENDULUM_POSITION, 2, 50, "gru", 100, False),      # the reference's recurrent configuration of the Pendulum: position only, restart of the hidden state every 100 steps
]


@pytest.mark.parametrize("case", CASES)
def test_env_evaluate_matches_the_checker(oracle, rocm, case):
    print("case", case, flush=True)
    kind, policy_kind, n, layers, period, with_standardize = case
    sd, od, ad = capi.ENV_DIMS[kind]
    out = policy_kind * ad
    last = "tanh" if policy_kind == 1 else "identity"
    specs = dense(od, 32, out, last=last) if layers is None else [(0, od, 24, "relu"), (1, 24, 16, "identity"), (0, 16, out, last)]
    rng = np.random.default_rng(100 * kind + 10 * policy_kind + n)
    params = helpers.random_seq_params(rng, specs)
    ini = initial_states(rng, kind, n)
    standardize = (rng.normal(0, 0.3, od).astype(np.float32), rng.uniform(0.5, 2, od).astype(np.float32)) if with_standardize else None
    acrobot = kind in (capi.ENV_ACROBOT, capi.ENV_ACROBOT_SWINGUP)
    terminated_somewhere = False
    for steps, tol in ((12, 1e-4 if acrobot else 1e-5), (150, 2e-3)):
        want = helpers.env_evaluate_on_backend(oracle, kind, specs, params, policy_kind, ini, steps, period, standardize)
        got = helpers.env_evaluate_on_backend(rocm, kind, specs, params, policy_kind, ini, steps, period, standardize)
        if steps == 12:      # over long horizons an episode near the line can terminate a step apart in the two arithmetics
            assert np.array_equal(got[1], want[1]), (got[1], want[1])
            assert rel_err(got[0], want[0]) <= tol, (steps, rel_err(got[0], want[0]))
            assert rel_err(got[2][:2], want[2][:2]) <= tol and np.array_equal(got[2][[2, 4, 5]], want[2][[2, 4, 5]]) and abs(got[2][3] - want[2][3]) <= 1e-5 * steps, (got[2], want[2])
        else:
            same = got[1] == want[1]
            assert same.mean() >= 0.8, (got[1], want[1])
            close = np.abs(got[0][same] - want[0][same]) <= tol * np.abs(want[0][same]).max()
            # the Acrobot is a double pendulum: over 150 steps a few episodes separate from a last-bit difference; the others stay together
            assert close.mean() >= (0.6 if acrobot else 1.0), (steps, close.mean(), got[0], want[0])
        assert got[1].max() <= steps and got[1].min() >= 1
        assert got[2][4] >= np.sum(got[1] < steps)      # every episode that stopped early terminated (one may also terminate on its last step)
        terminated_somewhere = terminated_somewhere or want[2][4] > 0
        assert abs(got[2][5] - got[2][4] / n) <= 1e-6
        assert abs(got[2][2] - got[1].mean()) <= 1e-3 * steps
    assert terminated_somewhere == (kind in (capi.ENV_ACROBOT, capi.ENV_CAR)), want[2]      # the cases exercise what they are for


def test_env_evaluate_of_the_pendulum_is_the_pendulum_evaluation(rocm):
    """The same episodes through the Pendulum's own entry point (one launch) and through the entry point for any environment (step by step)."""
    rng = np.random.default_rng(5)
    dims = [3, 64, 64, 2]
    params = helpers.random_params(rng, dims)
    ini = initial_states(rng, capi.ENV_PENDULUM, 25)
    own = helpers.evaluate_on_backend(rocm, dims, params, "relu", "identity", 2, ini, 40)
    specs = dense(3, 64, 2)
    general = helpers.env_evaluate_on_backend(rocm, capi.ENV_PENDULUM, specs, params, 2, ini, 40)
    assert np.array_equal(general[1], own[1])
    assert rel_err(general[0], own[0]) <= 1e-4 and rel_err(general[2][:4], own[2][:4]) <= 1e-4


def test_env_evaluate_rejects_what_it_cannot_run(rocm):
    specs = dense(6, 32, 1, last="tanh")
    params = helpers.random_seq_params(np.random.default_rng(0), specs)
    ini = np.zeros((4, 4), np.float32)
    with pytest.raises(RuntimeError):      # a policy whose output is not [mean | log_std]
        helpers.env_evaluate_on_backend(rocm, capi.ENV_ACROBOT, specs, params, 2, ini, 5)
    with pytest.raises(RuntimeError):      # an unknown environment
        helpers.env_evaluate_on_backend(rocm, 9, specs, params, 1, ini, 5)
