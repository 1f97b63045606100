"""Writes tests/golden/evaluation_pendulum_seed0.npz from the REAL reference (oracle/_ref/librlt_ref_generic.so, built by oracle/Makefile from
/root/reference). Runs only where the reference is mounted; the committed .npz is data, not source.

The reference's SAC-on-Pendulum loop (seed 0, batch 100) is stopped after 0, 150, 400 and 6,000 steps (the last one a trained actor that swings
the pendulum up and balances it: a closed loop in which a policy evaluated inconsistently loses the pendulum again); at each stop the reference's
rl::utils::evaluation::evaluate runs 10 episodes of 200 steps with the current actor in Evaluation mode from initial states it samples
(engine seeds 5, 6, 7, 8). Kept per stop: the actor's parameters (flat, per layer [weights | biases]), the sampled initial states, and the
reference's result (returns, episode lengths, the six summary values)."""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import helpers  # noqa: E402

ref = C.CDLL(helpers.REF_GENERIC)
P = C.c_void_p
ref.rlt_ref_sac_create.restype = P
ref.rlt_ref_sac_step.argtypes = [P]; ref.rlt_ref_sac_step_count.argtypes = [P]; ref.rlt_ref_sac_get_parameters.argtypes = [P, P]
ref.rlt_ref_sac_parameter_count.argtypes = [P]; ref.rlt_ref_sac_parameter_count.restype = C.c_size_t
ref.rlt_ref_sac_evaluate.argtypes = [P, C.c_uint32, P, P, P, P]
h = P(ref.rlt_ref_sac_create(0, 100))
params = np.zeros(ref.rlt_ref_sac_parameter_count(h), np.float32)
n_actor = helpers.mlp_param_count([3, 64, 64, 2])
out = {"stops": np.array([0, 150, 400, 6000]), "seeds": np.array([5, 6, 7, 8])}
for k, (stop, seed) in enumerate(zip(out["stops"], out["seeds"])):
    while ref.rlt_ref_sac_step_count(h) < stop:
        ref.rlt_ref_sac_step(h)
    ref.rlt_ref_sac_get_parameters(h, params.ctypes.data)
    ini, ret, length, summary = np.zeros((10, 2), np.float32), np.zeros(10, np.float32), np.zeros(10, np.uint32), np.zeros(6, np.float32)
    ref.rlt_ref_sac_evaluate(h, int(seed), ini.ctypes.data, ret.ctypes.data, length.ctypes.data, summary.ctypes.data)
    out[f"e{k}_actor"], out[f"e{k}_initial_states"], out[f"e{k}_returns"], out[f"e{k}_episode_length"], out[f"e{k}_summary"] = params[:n_actor].copy(), ini, ret, length, summary
np.savez_compressed(os.path.join(HERE, "evaluation_pendulum_seed0.npz"), **out)
print("wrote evaluation_pendulum_seed0.npz", {k: v.shape for k, v in out.items()})
