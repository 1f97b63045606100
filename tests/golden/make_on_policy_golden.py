"""Writes tests/golden/on_policy_pendulum_seed3.npz from the REAL reference (oracle/_ref/librlt_ref_ppo_normalize_generic.so, built by
oracle/Makefile from /root/reference). Runs only where the reference is mounted; the committed .npz is data, not source.

The reference's PPO-on-Pendulum loop with running observation normalisation (seed 3, 8 environments x 40 steps, episodes truncated
after 25 steps) is advanced through its first loop step (normaliser warm-up collect, re-initialised runner, second collect) and a
second one. Kept for each of the three collect() calls: runner state before and after, actor parameters, log_std and standardize
statistics, the dataset the reference wrote, and the draws behind it (the N(0,1) value of every sampled action, the initial state of
every reset) as recovered by the restated collection running on the reference's RNG state; and the running normalisers and standardize
statistics after each update()."""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import helpers  # noqa: E402

oracle = helpers.HostBackend()
b = helpers.RefPpo(3, normalize=True)
n, S, ld, c = b.n_envs, b.steps, b.data_dim, b.col
out = {"dims": np.array([n, S, ld, b.actor_hidden, b.episode_step_limit]), "columns": np.array([c[k] for k in helpers.PPO_COLUMNS])}
k = 0


def collect():
    global k
    p = b.parameters()
    na = helpers.mlp_param_count([3, b.actor_hidden, b.actor_hidden, 1])
    actor = helpers.Mlp(oracle, [3, b.actor_hidden, b.actor_hidden, 1], p[:na], n, "tanh", "identity", trainable=False)
    st, before, rng = b.standardize(), b.runner(), b.rng_state()
    b.lib.rlt_ref_ppo_collect(b.h)
    o = helpers.OnPolicyOnBackend(oracle, n, S, ld, c, b.episode_step_limit, before)
    noise, ini = np.zeros((S, n, 1), np.float32), np.zeros((S, n, 2), np.float32)
    ls, sm, sp = oracle.array(p[na:na + 1]), oracle.array(st["actor_mean"]), oracle.array(st["actor_precision"])
    assert oracle.lib.rlt_oracle_on_policy_collect_with_rng(C.byref(o.c), C.byref(o.d), actor.layers, actor.n, ls.ptr, sm.ptr, sp.ptr, noise.ctypes.data, ini.ctypes.data,
                                                            0, rng, 16384) == 0
    assert rng.value == b.rng_state().value
    want = b.dataset()
    assert np.array_equal(o.data.numpy()[:, :c["all_values"]], want[:, :c["all_values"]])
    out[f"c{k}_actor"], out[f"c{k}_log_std"] = p[:na], p[na:na + 1]
    out[f"c{k}_standardize_mean"], out[f"c{k}_standardize_precision"] = st["actor_mean"], st["actor_precision"]
    for name, v in before.items():
        out[f"c{k}_before_{name}"] = v
    for name, v in b.runner().items():
        out[f"c{k}_after_{name}"] = v
    out[f"c{k}_noise"], out[f"c{k}_initial_states"], out[f"c{k}_dataset"] = noise, ini, want[:, :c["all_values"]]
    k += 1


def update():
    b.lib.rlt_ref_ppo_update_normalizers(b.h)
    for name, v in {**b.normalizers(), **b.standardize()}.items():
        out[f"u{k - 1}_{name}"] = v


collect(); update(); b.lib.rlt_ref_ppo_reinit_runner(b.h)
collect(); update(); b.lib.rlt_ref_ppo_values_and_gae(b.h); b.lib.rlt_ref_ppo_train(b.h)
collect(); update()
b.close()
np.savez_compressed(os.path.join(HERE, "on_policy_pendulum_seed3.npz"), **out)
print("wrote on_policy_pendulum_seed3.npz", len(out), "arrays")
