"""Writes tests/golden/car_steps.npz from the REAL reference (oracle/_ref/librlt_ref_envs_generic.so, built by oracle/Makefile from
/root/reference). Runs only where the reference is mounted; the committed .npz is data, not source.

The Car without a track: 512 random states (positions around the termination bounds, all headings, forward and backward speeds on both sides of the
tire-force threshold vt, some at rest) with actions in [-1.3, 1.3]^2, and what the reference's observe / step / reward / terminated give for them;
plus a 300-step trajectory from rest under a fixed action sequence, each step fed with the reference's own previous next state."""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import helpers  # noqa: E402

ref = C.CDLL(os.path.join(helpers.ORACLE_DIR, "_ref", "librlt_ref_envs_generic.so"))
P = C.c_void_p
ref.rlt_ref_car_steps.argtypes = [P, P, P, P, P, P, P, C.c_int]


def steps(states, actions):
    n = states.shape[0]
    ns, o, no, r, t = np.zeros((n, 6), np.float32), np.zeros((n, 6), np.float32), np.zeros((n, 6), np.float32), np.zeros(n, np.float32), np.zeros(n, np.uint8)
    assert ref.rlt_ref_car_steps(states.ctypes.data, actions.ctypes.data, ns.ctypes.data, o.ctypes.data, no.ctypes.data, r.ctypes.data, t.ctypes.data, n) == 0
    return ns, o, no, r, t


rng = np.random.default_rng(6)
n = 512
states = np.stack([rng.uniform(-1.2, 1.2, n), rng.uniform(-1.2, 1.2, n), rng.uniform(-4, 4, n), rng.uniform(-0.5, 3, n), rng.uniform(-1, 1, n), rng.uniform(-8, 8, n)], 1).astype(np.float32)
states[:16, 3:] = 0
states[16:32, 3] = rng.uniform(0.005, 0.015, 16)       # around vt = 0.01
actions = rng.uniform(-1.3, 1.3, (n, 2)).astype(np.float32)
out = {"states": states, "actions": actions}
for name, v in zip(("next_states", "observations", "next_observations", "rewards", "terminated"), steps(states, actions)):
    out[name] = v
T = 300
traj_actions = np.stack([np.clip(0.6 + 0.3 * np.sin(np.arange(T) / 20.0), -1, 1), np.clip(np.cumsum(rng.normal(0, 0.05, T)), -1, 1)], 1).astype(np.float32)
s = np.zeros((1, 6), np.float32)
traj, rew, term = [s[0].copy()], [], []
for k in range(T):
    s, _, _, r1, t1 = steps(s, traj_actions[k:k + 1])
    traj.append(s[0].copy()); rew.append(r1[0]); term.append(t1[0])
out["trajectory_actions"], out["trajectory"], out["trajectory_rewards"], out["trajectory_terminated"] = traj_actions, np.array(traj), np.array(rew, np.float32), np.array(term, np.uint8)
np.savez_compressed(os.path.join(HERE, "car_steps.npz"), **out)
print("wrote car_steps.npz", int(out["terminated"].sum()), "terminal of", n, "; trajectory ends at", out["trajectory"][-1], "terminal steps", int(out["trajectory_terminated"].sum()))
