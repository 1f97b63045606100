"""Writes tests/golden/ppo_pendulum_seed0.npz from the REAL reference (oracle/_ref/librlt_ref_ppo_generic.so, built by oracle/Makefile
from /root/reference). Runs only where the reference is mounted; the committed .npz is data (inputs/expected outputs), not source.

Two loop steps of the reference's seeded PPO-on-Pendulum loop (8 environments x 40 steps, episode limit 25, minibatch 64, 3 epochs).
Per loop step: the collected dataset after the reference's generalized advantage estimation (all columns), every parameter (actor,
log_std, critic) before and after the reference's train(), and the row permutation of every epoch (the reference shuffles the dataset
in place; the permutation is that shuffle replayed on a row-index array from the loop's RNG state)."""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import helpers  # noqa: E402

ref = helpers.RefPpo(0)
oracle = helpers.HostBackend()
out = {"dims": np.array([ref.n_envs, ref.steps, ref.data_dim, ref.rows, ref.obs_dim, ref.action_dim, ref.batch, ref.epochs, ref.actor_hidden, ref.critic_hidden]),
       "columns": np.array([ref.col[c] for c in helpers.PPO_COLUMNS]), "hyper": np.array([ref.hyper[k] for k in sorted(ref.hyper)], np.float64),
       "hyper_names": np.array(sorted(ref.hyper))}
n = ref.n_envs * ref.steps
for step in range(2):
    ref.lib.rlt_ref_ppo_collect_and_gae(ref.h)
    out[f"s{step}_dataset"] = ref.dataset()
    out[f"s{step}_before"] = ref.parameters()
    state = ref.rng_state()
    perms = np.zeros((ref.epochs, n), np.uint32)
    assert oracle.lib.rlt_oracle_ppo_shuffle(state, 16384, n, ref.epochs, perms.ctypes.data) == 0
    ref.lib.rlt_ref_ppo_train(ref.h)
    assert ref.rng_state().value == state.value
    out[f"s{step}_permutations"] = perms
    out[f"s{step}_after"] = ref.parameters()
np.savez_compressed(os.path.join(HERE, "ppo_pendulum_seed0.npz"), **out)
print("wrote", os.path.join(HERE, "ppo_pendulum_seed0.npz"), {k: v.shape for k, v in out.items()})
