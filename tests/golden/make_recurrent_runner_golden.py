"""Writes tests/golden/recurrent_runner_pendulum.npz from the REAL reference (oracle/_ref/librlt_ref_sac_gru3_generic.so, built by oracle/Makefile from
/root/reference). Runs only where the reference is mounted; the committed .npz is data (inputs/expected outputs), not source.

The reference's SAC loop with its recurrent approximators (actor dense 3-16, GRU 16, dense 16-2, sample_and_squash; three environments, 30-step
episodes, 260-row rings, auto-reset of the policy state every 6 steps; seed 4) is warmed up and advanced 24 loop steps with the runner step's
draws written out. Kept: the runner, the policy state and the replay rings before the first of these steps, and per step the actor's parameters
the step ran with, the initial states and noise it drew, which environments started a new episode, and afterwards the runner, the policy state,
the ring cursors and the rows the step wrote."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import helpers  # noqa: E402

STEPS = 24
ref = helpers.RefSacGru(3, 4)
for _ in range(ref.n_warmup):
    ref.step()
n, cap, limit, period, n_gru = ref.runner_dims()
out = {"dims": np.array([n, cap, limit, period, n_gru, STEPS], np.int32), "actor_layers": np.array([[k, i, o, helpers.capi.ACT[a]] for k, i, o, a in ref.actor_specs], np.int32)}
before, rings = ref.runner(), ref.rings()
for k in ("states", "episode_step", "episode_return", "truncated"):
    out["before_" + k] = before[k]
out["before_hidden"], out["before_steps"] = np.stack(before["hidden"]), np.stack(before["steps"])
out["before_data"] = np.concatenate([r[0] for r in rings]); out["before_position"] = np.array([r[1] for r in rings], np.uint32)
out["before_full"] = np.array([r[2] for r in rings], np.uint8); out["before_current_episode_start"] = np.array([r[3] for r in rings], np.uint32)
out["before_episode_start"] = np.concatenate([r[4] for r in rings])
for i in range(STEPS):
    out[f"s{i}_actor"] = ref.actor_parameters()
    positions = [r[1] for r in ref.rings()]
    out[f"s{i}_initial_states"], out[f"s{i}_noise"], out[f"s{i}_reset"] = ref.manual_step()
    after, rings = ref.runner(), ref.rings()
    for k in ("states", "episode_step", "episode_return", "truncated"):
        out[f"s{i}_{k}"] = after[k]
    out[f"s{i}_hidden"], out[f"s{i}_steps"] = np.stack(after["hidden"]), np.stack(after["steps"])
    out[f"s{i}_position"] = np.array([r[1] for r in rings], np.uint32)
    out[f"s{i}_current_episode_start"] = np.array([r[3] for r in rings], np.uint32)
    out[f"s{i}_rows"] = np.stack([rings[e][0][positions[e]] for e in range(n)])                     # the row every ring received
    out[f"s{i}_previous_truncated"] = np.array([rings[e][0][(positions[e] - 1) % cap][9] for e in range(n)], np.float32)   # the flag the prologue sets on the row before
ref.close()
np.savez_compressed(os.path.join(HERE, "recurrent_runner_pendulum.npz"), **out)
print("wrote recurrent_runner_pendulum.npz", len(out), "arrays")
