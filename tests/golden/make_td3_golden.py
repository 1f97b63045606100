"""Writes tests/golden/td3_pendulum_seed7.npz from the REAL reference (oracle/_ref/librlt_ref_td3_generic.so, built by oracle/Makefile
from /root/reference). Runs only where the reference is mounted; the committed .npz is data (inputs/expected outputs), not source.

The reference's TD3-on-Pendulum loop (seed 7) is warmed up (100 steps of uniform exploration, no training) and then advanced 36 loop
steps. Kept: the hyperparameters, all parameters before the first training step, and for every step the batch it trained on, the
clamped target-action noise together with the N(0,1) draws behind it, the N(0,1) draws of the actor's sampling layer in both critic
updates and the actor update, which of the four operations ran, the float64 sum and sum of squares of every network's parameters
afterwards, and -- after steps 1 and 35 -- all parameters."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import helpers  # noqa: E402

STEPS = 36
ref = helpers.RefTd3(7)
for _ in range(ref.n_warmup):
    ref.step()
out = {"dims": np.array([ref.batch, ref.hidden, STEPS]), "hyperparameters": ref.hp.copy(), "parameters_before": ref.parameters()}
for i in range(STEPS):
    z, c0, c1, na, flags = ref.manual_step()
    oab, r, t, fm, nfm = ref.batch_data()
    assert fm.all() and nfm[ref.batch:].all()
    out[f"s{i}_flags"] = np.array(flags, np.int32)
    out[f"s{i}_oab"], out[f"s{i}_rewards"], out[f"s{i}_terminated"] = oab, r, t
    out[f"s{i}_target_noise_z"], out[f"s{i}_target_noise"] = z, ref.target_noise()
    out[f"s{i}_noise_critic_0"], out[f"s{i}_noise_critic_1"], out[f"s{i}_noise_actor"] = c0, c1, na
    p = ref.parameters()
    out[f"s{i}_digest"] = helpers.td3_digest(p, ref.hidden)
    if i in (1, STEPS - 1):
        out[f"s{i}_after"] = p
out["ages_after"] = ref.ages()
ref.close()
np.savez_compressed(os.path.join(HERE, "td3_pendulum_seed7.npz"), **out)
print("wrote td3_pendulum_seed7.npz", len(out), "arrays")
