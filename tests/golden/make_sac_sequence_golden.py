"""Writes tests/golden/sac_sequence_pendulum.npz from the REAL reference (oracle/_ref/librlt_ref_sac_gru{3,5}_generic.so, built by oracle/Makefile
from /root/reference). Runs only where the reference is mounted; the committed .npz is data (inputs/expected outputs), not source.

The reference's SAC loop with its recurrent approximators (dense -> GRU -> dense, and dense -> GRU -> GRU -> dense -> dense; hidden 16, FAST_TANH
gates) on the Pendulum with three environments, 30-step episodes, 260-row rings, batches of 16 sequences of 6 steps with the first step
included in the targets (seed 4) is warmed up (100 steps of uniform exploration, no training) and then advanced 20 (8) loop steps. Kept per
depth: the layer lists, the hyperparameters, all parameters before the first training step, and for every step the batch it trained on (all
seven tensors, as gather_batch left them, stale entries included), both noise tensors, the float64 sum and sum of squares of every network's
parameters afterwards, and -- after the steps named in `snapshots` -- all parameters."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import helpers  # noqa: E402

out = {}
for n_layers, steps, snapshots in ((3, 20, (1, 19)), (5, 8, (7,))):
    ref = helpers.RefSacGru(n_layers, 4)
    for _ in range(ref.n_warmup):
        ref.step()
    p = f"l{n_layers}_"
    out[p + "dims"] = np.array([ref.batch, ref.seq, ref.obs_dim, ref.act_dim, ref.include_first, steps], np.int32)
    for name, specs in (("actor", ref.actor_specs), ("critic", ref.critic_specs)):
        out[p + name + "_layers"] = np.array([[k, i, o, helpers.capi.ACT[a]] for k, i, o, a in specs], np.int32)
    out[p + "hyperparameters"] = ref.hp.copy()
    out[p + "parameters_before"] = ref.parameters()
    out[p + "snapshots"] = np.array(snapshots, np.int32)
    for i in range(steps):
        ref.step()
        for k, v in ref.batch_data().items():
            out[f"{p}s{i}_{k}"] = v
        out[f"{p}s{i}_noise_critic"], out[f"{p}s{i}_noise_actor"] = ref.noise()
        params = ref.parameters()
        out[f"{p}s{i}_digest"] = helpers.sac_sequence_digest(params, ref.actor_specs, ref.critic_specs)
        if i in snapshots:
            out[f"{p}s{i}_after"] = params
    out[p + "ages_after"] = np.array(ref.ages(), np.uint32)
    ref.close()
np.savez_compressed(os.path.join(HERE, "sac_sequence_pendulum.npz"), **out)
print("wrote sac_sequence_pendulum.npz", len(out), "arrays")
