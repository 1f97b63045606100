"""Writes tests/golden/evaluation_recurrent_pendulum.npz from the REAL reference (oracle/_ref/librlt_ref_sac_gru{3,5}_generic.so, built by oracle/Makefile from
/root/reference). Runs only where the reference is mounted; the committed .npz is data (inputs/expected outputs), not source.

The reference's SAC loop with its recurrent approximators (actor dense 3-16, one or two GRU 16 layers, [dense,] dense 16-2, sample_and_squash; seed 9) is evaluated
with rl::utils::evaluation::evaluate (5 episodes x 40 steps, Evaluation mode, the hidden state restarting every 6 steps) before training and after 40 and 150
training steps. Kept per run: the actor's parameters, the initial states the call drew, the returns, episode lengths and the summary."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import helpers  # noqa: E402

out = {}
for n_layers in (3, 5):
    ref = helpers.RefSacGru(n_layers, 9)
    stops = [0, ref.n_warmup + 40, ref.n_warmup + 150]
    out["dims"] = np.array([ref.runner_dims()[3], 40, len(stops)], np.int32)
    out[f"l{n_layers}_actor_layers"] = np.array([[k, i, o, helpers.capi.ACT[a]] for k, i, o, a in ref.actor_specs], np.int32)
    done = 0
    for k, stop in enumerate(stops):
        while done < stop:
            ref.step(); done += 1
        p = f"l{n_layers}_e{k}_"
        out[p + "actor"] = ref.actor_parameters()
        out[p + "initial_states"], out[p + "returns"], out[p + "length"], out[p + "summary"] = ref.evaluate(100 + k)
    ref.close()
np.savez_compressed(os.path.join(HERE, "evaluation_recurrent_pendulum.npz"), **out)
print("wrote evaluation_recurrent_pendulum.npz", len(out), "arrays")
