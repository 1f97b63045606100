"""Car step kernel (the variant without a track) against the CPU checker and the reference's own outputs, through the C ABI.

Tolerance: 1e-5 relative to the largest magnitude per tensor for one step (fp32 against the reference's float with a few double sub-expressions); the
terminated flag may differ only where the next position is within 1e-5 of the bound; the tire forces switch on at vx > vt or vy > vt, a comparison of
inputs, so it cannot flip."""
import ctypes as C
import os

import numpy as np
import pytest

import helpers
from helpers import rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-5


def compare(got, want):
    for name, g, w in zip(("next_states", "observations", "next_observations", "rewards"), got[:4], want[:4]):
        for c in range(g.shape[1] if g.ndim == 2 else 1):
            gc, wc = (g[:, c], w[:, c]) if g.ndim == 2 else (g, w)
            assert rel_err(gc, wc) <= TOL, (name, c, rel_err(gc, wc))
    differ = np.nonzero(got[4] != want[4])[0]
    if len(differ):
        margin = np.abs(np.abs(want[0][differ, :2]) - 1.0).min(1)
        assert margin.max() <= 1e-5, (differ, margin)


def random_states(rng, n):
    s = np.stack([rng.uniform(-1.2, 1.2, n), rng.uniform(-1.2, 1.2, n), rng.uniform(-4, 4, n), rng.uniform(-0.5, 3, n), rng.uniform(-1, 1, n), rng.uniform(-8, 8, n)], 1).astype(np.float32)
    s[: n // 50, 3:] = 0
    return s, rng.uniform(-1.3, 1.3, (n, 2)).astype(np.float32)


def test_car_against_reference_vectors(rocm):
    g = np.load(os.path.join(helpers.GOLDEN, "car_steps.npz"))
    compare(helpers.car_on_backend(rocm, g["states"], g["actions"]), tuple(g[k] for k in ("next_states", "observations", "next_observations", "rewards", "terminated")))
    traj = g["trajectory"]
    s, _, _, r, t = helpers.car_on_backend(rocm, traj[:60], g["trajectory_actions"][:60])      # every step restarted from the reference's state
    for c in range(6):
        assert rel_err(s[:, c], traj[1:61, c]) <= TOL, c
    assert rel_err(r, g["trajectory_rewards"][:60]) <= TOL and np.array_equal(t, g["trajectory_terminated"][:60])


@pytest.mark.parametrize("n", [1, 4099, 200000])
def test_car_matches_checker(oracle, rocm, n):
    print("case", n, flush=True)
    states, actions = random_states(np.random.default_rng(n), n)
    compare(helpers.car_on_backend(rocm, states, actions), helpers.car_on_backend(oracle, states, actions))


def test_car_closed_loop_and_optional_outputs(oracle, rocm):
    """200 steps in a closed loop from rest under gentle inputs (differences grow along the chain: 1e-3), and NULL outputs are skipped."""
    rng = np.random.default_rng(1)
    n = 256
    sg = so = np.zeros((n, 6), np.float32)
    for k in range(200):
        a = np.stack([rng.uniform(0.2, 0.8, n), rng.uniform(-0.2, 0.2, n)], 1).astype(np.float32)
        sg, so = helpers.car_on_backend(rocm, sg, a)[0], helpers.car_on_backend(oracle, so, a)[0]
    assert np.abs(so[:, 3]).max() > 0.5
    for c in range(6):
        assert np.abs(sg[:, c] - so[:, c]).max() <= 1e-3 * max(np.abs(so[:, c]).max(), 1.0), c
    p = helpers.capi.car_parameters()
    s, a = rocm.array(so), rocm.array(np.zeros((n, 2), np.float32))
    rocm.call("car_step", C.byref(p), s.ptr, a.ptr, None, None, None, None, n)
    rocm.sync()
    want = helpers.car_on_backend(oracle, so, np.zeros((n, 2), np.float32))[0]
    for c in range(6):
        assert rel_err(s.numpy()[:, c], want[:, c]) <= TOL
    assert rocm.device.lib.rlt_rocm_car_step(rocm.device.handle, C.byref(p), None, a.ptr, None, None, None, None, n) != 0
