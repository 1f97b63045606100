"""Writes tests/golden/acrobot_steps.npz from the REAL reference (oracle/_ref/librlt_ref_envs_generic.so, built by oracle/Makefile from
/root/reference). Runs only where the reference is mounted; the committed .npz is data, not source.

For the Acrobot, the AcrobotSwingup and the AcrobotSwingup with EasyParameters (kinds 0, 1, 2): 256 random states (angles over the full circle,
velocities up to the clamps, a few exactly at rest) with actions in [-1.3, 1.3] (so that the clamp to [-1, 1] is exercised), and what the
reference's observe / step / reward / terminated give for them; plus a 200-step trajectory per kind from a state near rest under a fixed action
sequence, each step fed with the reference's own previous next state."""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import helpers  # noqa: E402

ref = C.CDLL(os.path.join(helpers.ORACLE_DIR, "_ref", "librlt_ref_envs_generic.so"))
P = C.c_void_p
ref.rlt_ref_acrobot_steps.argtypes = [C.c_int, P, P, P, P, P, P, P, C.c_int]


def steps(kind, states, actions):
    n = states.shape[0]
    ns, o, no, r, t = np.zeros((n, 4), np.float32), np.zeros((n, 6), np.float32), np.zeros((n, 6), np.float32), np.zeros(n, np.float32), np.zeros(n, np.uint8)
    assert ref.rlt_ref_acrobot_steps(kind, states.ctypes.data, actions.ctypes.data, ns.ctypes.data, o.ctypes.data, no.ctypes.data, r.ctypes.data, t.ctypes.data, n) == 0
    return ns, o, no, r, t


rng = np.random.default_rng(4)
n = 256
states = np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-np.pi, np.pi, n), rng.uniform(-4 * np.pi, 4 * np.pi, n), rng.uniform(-9 * np.pi, 9 * np.pi, n)], 1).astype(np.float32)
states[:4] = 0
states[4] = [np.pi, 0, 0, 0]
actions = rng.uniform(-1.3, 1.3, n).astype(np.float32)
out = {"states": states, "actions": actions}
T = 200
traj_actions = np.clip(np.cumsum(rng.normal(0, 0.3, T)), -1, 1).astype(np.float32)
out["trajectory_actions"] = traj_actions
for kind in range(3):
    ns, o, no, r, t = steps(kind, states, actions)
    out[f"k{kind}_next_states"], out[f"k{kind}_observations"], out[f"k{kind}_next_observations"], out[f"k{kind}_rewards"], out[f"k{kind}_terminated"] = ns, o, no, r, t
    s = np.array([[0.05, -0.03, 0.02, 0.01]], np.float32)
    traj, rew, term = [s[0].copy()], [], []
    for k in range(T):
        s, _, _, r1, t1 = steps(kind, s, traj_actions[k:k + 1])
        traj.append(s[0].copy()); rew.append(r1[0]); term.append(t1[0])
    out[f"k{kind}_trajectory"], out[f"k{kind}_trajectory_rewards"], out[f"k{kind}_trajectory_terminated"] = np.array(traj), np.array(rew, np.float32), np.array(term, np.uint8)
np.savez_compressed(os.path.join(HERE, "acrobot_steps.npz"), **out)
print("wrote acrobot_steps.npz", int(out["k0_terminated"].sum()), "terminal next states of", n, "; trajectory terminals", [int(out[f"k{k}_trajectory_terminated"].sum()) for k in range(3)])
