"""Acrobot / AcrobotSwingup step kernel against the CPU checker and the reference's own outputs, through the C ABI.

Tolerance: the kernel computes in fp32 where the reference evaluates parts of dsdt in double: 1e-5 relative to the largest magnitude per tensor for
one step at the joint velocities the task moves in (|w1| <= 6, |w2| <= 10 rad/s) and for at least 99% of states drawn up to the velocity clamps; the
rest get a slack proportional to the step's own measured amplification of input perturbations (see allowance()). The terminated flag may differ
only where the checker's own criterion is within 1e-4 of its threshold."""
import os

import numpy as np
import pytest

import helpers
from helpers import rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-5


def circle_distance(a, b):
    d = np.abs(a - b)
    d[:, :2] = np.minimum(d[:, :2], 2 * np.pi - d[:, :2])        # an angle next to +-pi may wrap to the other end on one side only
    return d


def allowance(oracle, kind, states, actions, want_next):
    """Per-row slack for the states: at high joint velocities one Runge-Kutta step of 0.2 s amplifies a perturbation of the input thousands of times
    (the integrator is past its stability range there), and fp32 rounding inside the step is amplified the same way. The gain is measured on the
    checker itself with finite differences; the slack is gain x fp32 epsilon x the state's magnitude, with a factor 16."""
    rng = np.random.default_rng(0)
    gain = np.zeros(states.shape[0])
    for _ in range(6):
        delta = (1e-4 * np.sign(rng.standard_normal(states.shape))).astype(np.float32)
        moved = helpers.acrobot_on_backend(oracle, kind, states + delta, actions)[0]
        gain = np.maximum(gain, circle_distance(moved, want_next).max(1) / 1e-4)
    return 16 * gain * 6e-8 * 30.0


def compare(got, want, states_before, slack=None):
    scale = np.abs(want[0]).max()
    err = circle_distance(got[0], want[0]).max(1)
    moderate = (np.abs(states_before[:, 2]) <= 6) & (np.abs(states_before[:, 3]) <= 10)
    assert err[moderate].max(initial=0.0) <= TOL * scale, err[moderate].max()
    if slack is None:
        slack = np.zeros_like(err)
    assert np.all(err <= TOL * scale + slack), (np.nonzero(err > TOL * scale + slack)[0][:5], err.max())
    assert (err <= TOL * scale).mean() >= 0.99
    assert rel_err(got[1], want[1]) <= TOL and rel_err(got[3], want[3]) <= TOL + (slack.max() > 0) * 1e-4
    # next observations follow the next states: compare them where the states agree
    fine = err <= TOL * scale
    assert np.abs(got[2][fine] - want[2][fine]).max() <= 2 * TOL * scale
    differ = np.nonzero((got[4] != want[4]) & fine)[0]
    if len(differ):
        ns = want[0][differ].astype(np.float64)
        margin = np.abs(-np.cos(ns[:, 0]) - np.cos(ns[:, 1] + ns[:, 0]) - 1.0)
        assert margin.max() <= 1e-4, (differ, margin)


@pytest.mark.parametrize("kind", [0, 1, 2])
def test_acrobot_against_reference_vectors(oracle, rocm, kind):
    g = np.load(os.path.join(helpers.GOLDEN, "acrobot_steps.npz"))
    got = helpers.acrobot_on_backend(rocm, kind, g["states"], g["actions"])
    want = tuple(g[f"k{kind}_{name}"] for name in ("next_states", "observations", "next_observations", "rewards", "terminated"))
    compare(got, want, g["states"], allowance(oracle, kind, g["states"], g["actions"], want[0]))
    # the first 25 steps of the reference's trajectory, every step restarted from the reference's state
    traj = g[f"k{kind}_trajectory"]
    s, _, _, r, t = helpers.acrobot_on_backend(rocm, kind, traj[:25], g["trajectory_actions"][:25])
    assert np.abs(s - traj[1:26]).max() <= TOL * np.abs(traj[1:26]).max() and rel_err(r, g[f"k{kind}_trajectory_rewards"][:25]) <= TOL


@pytest.mark.parametrize("kind,n", [(0, 1), (0, 100000), (1, 4099), (2, 65536)])
def test_acrobot_matches_checker(oracle, rocm, kind, n):
    print("case", kind, n, flush=True)
    rng = np.random.default_rng(n)
    states = np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-np.pi, np.pi, n), rng.uniform(-13, 13, n), rng.uniform(-29, 29, n)], 1).astype(np.float32)
    actions = rng.uniform(-1.3, 1.3, n).astype(np.float32)
    want = helpers.acrobot_on_backend(oracle, kind, states, actions)
    compare(helpers.acrobot_on_backend(rocm, kind, states, actions), want, states, allowance(oracle, kind, states, actions, want[0]))


def test_acrobot_closed_loop_and_optional_outputs(oracle, rocm):
    """40 steps in a closed loop from small states (rounding differences grow with the chain: 1e-3), and NULL outputs are skipped."""
    import ctypes as C
    rng = np.random.default_rng(1)
    n = 512
    sg = so = (rng.uniform(-0.1, 0.1, (n, 4))).astype(np.float32)
    for k in range(40):
        a = rng.uniform(-1, 1, n).astype(np.float32)
        sg, so = helpers.acrobot_on_backend(rocm, 1, sg, a)[0], helpers.acrobot_on_backend(oracle, 1, so, a)[0]
    d = np.abs(sg - so); d[:, :2] = np.minimum(d[:, :2], 2 * np.pi - d[:, :2])
    assert d.max() <= 1e-3 * np.abs(so).max()
    p = helpers.capi.acrobot_parameters()
    s, a = rocm.array(so), rocm.array(np.zeros(n, np.float32))
    rocm.call("acrobot_step", C.byref(p), 0, s.ptr, a.ptr, None, None, None, None, n)
    rocm.sync()
    want = helpers.acrobot_on_backend(oracle, 0, so, np.zeros(n, np.float32))[0]
    assert np.abs(s.numpy() - want).max() <= TOL * np.abs(want).max()
    assert rocm.device.lib.rlt_rocm_acrobot_step(rocm.device.handle, C.byref(p), 0, None, a.ptr, None, None, None, None, n) != 0
