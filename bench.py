#!/usr/bin/env python3
"""Benchmark of the dense-network training hot path on one MI355X.

Prints ONE JSON line. `value` is SAC loop steps per second at batch 256 on the Pendulum-shaped configuration (one loop step =
1 environment step + replay add + gather of 256 transitions + 2 critic updates + target update + 1 actor update, i.e. 3 network
updates), everything resident on the device, synthetic data. The same line carries the fused MLP forward+backward TFLOP/s at
batch 65,536 (17->256->256->6) with its roofline fraction, and the reference CPU path timed on this host.
"""
import argparse
import ctypes as C
import importlib.util
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
FP32_PEAK_TFLOPS = 157.3
HBM_PEAK_GBPS = 8000.0
# one SAC loop step at batch 256 with 3-64-64-2 / 4-64-64-1 networks: per sample 52,480 flop per critic update (actor and both target critics forward on the next
# observations, critic forward + backward) and 61,440 per actor update (actor forward, both critics forward + backward_input, actor backward)
SAC_STEP_FLOP = 256 * (2 * 52480 + 61440)
MLP_FLOP_PER_SAMPLE_FWD = 2 * (17 * 256 + 256 * 256 + 256 * 6)                       # 142,848
MLP_FLOP_PER_SAMPLE_BWD = 2 * (17 * 256 + 256 * 256 + 256 * 6) + 2 * (256 * 256 + 256 * 6)   # weight grads + d_input of layers 2,3: 276,992


def package():
    path = os.path.join(ROOT, "rl-tools_amd")
    spec = importlib.util.spec_from_file_location("rl_tools_amd", os.path.join(path, "__init__.py"), submodule_search_locations=[path])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["rl_tools_amd"] = mod
    spec.loader.exec_module(mod)
    return mod


class HipEvents:
    """hipEvent timing on the library's own stream (the kernels are not launched on any framework's current stream)."""

    def __init__(self, stream):
        self.hip = C.CDLL("libamdhip64.so")
        self.stream = C.c_void_p(stream)

    def record(self):
        e = C.c_void_p()
        assert self.hip.hipEventCreate(C.byref(e)) == 0
        assert self.hip.hipEventRecord(e, self.stream) == 0
        return e

    def elapsed_ms(self, a, b):
        assert self.hip.hipEventSynchronize(b) == 0
        ms = C.c_float()
        assert self.hip.hipEventElapsedTime(C.byref(ms), a, b) == 0
        return ms.value


# HBM bytes of one mlp_forward_backward call at batch 65,536, from two counter runs (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0 KiB per dispatch,
# the factors being what the same counters read for a 256 MiB copy): fused kernel 15.0 + 75.8, reduce kernel 70.6 + 0.3, prepare 1.2 + 0.5 MiB
MLP_CALL_HBM_BYTES = int((15392 + 77617 + 72292 + 281 + 1228 + 544) * 1024)
# the same for one PPO minibatch update of 8,192 rows: mlp3s_kernel 16.9 + 12.0, adam_pair_kernel 1.3 + 0.3 MiB
PPO_UPDATE_HBM_BYTES = int((17308 + 12270 + 1355 + 357) * 1024)


def checker():
    """tests/helpers.py: the loader of the CPU checker (oracle/), used by the CPU legs only."""
    tests = os.path.join(ROOT, "tests")
    if tests not in sys.path:
        sys.path.insert(0, tests)
    import helpers as tests_helpers
    return tests_helpers


def bench_mlp(helpers, rocm, batch, iters, warmup):
    capi = helpers.capi
    dims = [17, 256, 256, 6]
    rng = np.random.default_rng(0)
    net = helpers.Mlp(rocm, dims, helpers.xavier_params(rng, dims), batch)
    x = rocm.array(rng.standard_normal((batch, 17)).astype(np.float32))
    dy = rocm.array(rng.standard_normal((batch, 6)).astype(np.float32))
    y = rocm.zeros((batch, 6))
    ws, wsn = net.workspace()
    adam = capi.adam_parameters(epsilon=1e-8)
    ev = HipEvents(rocm.device.lib.rlt_rocm_get_stream(rocm.device.handle))

    def fwd_bwd():
        rocm.call("mlp_forward_backward", net.layers, net.n, x.ptr, 17, y.ptr, 6, dy.ptr, 6, None, 0, 0.0, batch, ws, wsn)

    def fwd():
        rocm.call("mlp_forward", net.layers, net.n, x.ptr, 17, batch)

    def bwd():      # after a forward(): the reference's call pattern (the gradient buffer becomes d_pre of the last layer in place, the identity here)
        rocm.call("mlp_backward", net.layers, net.n, x.ptr, 17, dy.ptr, 6, None, 0, batch, 1, ws, wsn)

    def step():
        rocm.call("adam_step", net.adam, net.n_adam, C.byref(adam), net.age.ptr, 0.0, None)

    out = {}
    for name, fn in (("forward_backward", fwd_bwd), ("forward", fwd), ("backward", bwd), ("adam", step)):
        rocm.call("mlp_zero_gradient", net.layers, net.n)
        for _ in range(warmup):
            fn()
        rocm.sync()
        a = ev.record()
        for _ in range(iters):
            fn()
        b = ev.record()
        out[name + "_ms"] = ev.elapsed_ms(a, b) / iters
    flop = (MLP_FLOP_PER_SAMPLE_FWD + MLP_FLOP_PER_SAMPLE_BWD) * batch
    out["tflops"] = flop / (out["forward_backward_ms"] * 1e-3) / 1e12
    out["batch"] = batch
    return out


def bench_env(helpers, rocm, n_envs=65536, capacity=16, steps=200, batch=4096):
    """Environment-step pipeline: Pendulum step of every environment with a deterministic 3-64-64-1 actor + replay add, then a gather."""
    capi = helpers.capi
    rng = np.random.default_rng(1)
    dims = [3, 64, 64, 1]
    actor = helpers.Mlp(rocm, dims, helpers.xavier_params(rng, dims), n_envs, "relu", "tanh", trainable=False)
    rb = helpers.ReplayOnBackend(rocm, n_envs, capacity)
    states, ep_step, ep_ret = rocm.zeros((n_envs, 2)), rocm.zeros((n_envs,), np.uint32), rocm.zeros((n_envs,))
    trunc = rocm.array(np.ones(n_envs, np.uint8))
    ini = rocm.array(np.stack([rng.uniform(-np.pi, np.pi, n_envs), rng.uniform(-1, 1, n_envs)], 1).astype(np.float32))
    runner = capi.PendulumRunner(states.ptr, ep_step.ptr, ep_ret.ptr, trunc.ptr, n_envs, 200, capi.pendulum_parameters())
    ev = HipEvents(rocm.device.lib.rlt_rocm_get_stream(rocm.device.handle))

    def step():
        rocm.call("pendulum_runner_step", C.byref(runner), C.byref(rb.c), 1, actor.layers, actor.n, None, None, None, ini.ptr, 0, 0)
    for _ in range(5):
        step()
    rocm.sync()
    a = ev.record()
    for _ in range(steps):
        step()
    e = ev.record()
    ms = ev.elapsed_ms(a, e)
    envs = rocm.array(rng.integers(0, n_envs, batch).astype(np.uint32)); offs = rocm.array(rng.integers(0, capacity, batch).astype(np.uint32))
    oab, rew, term = rocm.zeros((2, batch, 4)), rocm.zeros((batch,)), rocm.zeros((batch,), np.uint8)

    def gather():
        rocm.call("gather_batch", C.byref(rb.c), envs.ptr, offs.ptr, 0, 200, batch, oab.ptr, rew.ptr, term.ptr, None, None, None, None)
    for _ in range(5):
        gather()
    rocm.sync()
    a = ev.record()
    for _ in range(100):
        gather()
    e = ev.record()
    gather_us = ev.elapsed_ms(a, e) * 10.0
    env_steps = n_envs * steps
    # evaluation step of the training loop: 10 episodes x 200 steps with the deterministic actor, one launch
    env_p = capi.pendulum_parameters()
    e_ini, e_ret, e_len, e_sum = rocm.array(ini.numpy()[:10].copy()), rocm.zeros((10,)), rocm.zeros((10,), np.uint32), rocm.zeros((6,))

    def evaluate():
        rocm.call("pendulum_evaluate", C.byref(env_p), 1, actor.layers, actor.n, e_ini.ptr, 10, 200, e_ret.ptr, e_len.ptr, e_sum.ptr)
    for _ in range(3):
        evaluate()
    rocm.sync()
    a = ev.record()
    for _ in range(20):
        evaluate()
    e = ev.record()
    evaluate_us = ev.elapsed_ms(a, e) * 1e3 / 20
    # AcrobotSwingup: one Runge-Kutta step of a million environments with all outputs (state 16 B in and out, action 4, observations 2 x 24, reward 4, flag 1 = 89 B each)
    n_acro = 1 << 20
    acro_p = capi.acrobot_parameters()
    a_states = rocm.array(rng.uniform(-1, 1, (n_acro, 4)).astype(np.float32)); a_actions = rocm.array(rng.uniform(-1, 1, n_acro).astype(np.float32))
    a_obs, a_next, a_rew, a_term = rocm.zeros((n_acro, 6)), rocm.zeros((n_acro, 6)), rocm.zeros((n_acro,)), rocm.zeros((n_acro,), np.uint8)

    def acrobot():
        rocm.call("acrobot_step", C.byref(acro_p), 1, a_states.ptr, a_actions.ptr, a_obs.ptr, a_next.ptr, a_rew.ptr, a_term.ptr, n_acro)
    for _ in range(3):
        acrobot()
    rocm.sync()
    a = ev.record()
    for _ in range(50):
        acrobot()
    e = ev.record()
    acrobot_us = ev.elapsed_ms(a, e) * 1e3 / 50
    return {"n_envs": n_envs, "replay_rows": n_envs * capacity, "steps": steps, "us_per_step": ms * 1e3 / steps, "env_steps_per_s": env_steps / (ms * 1e-3),
            "algorithmic_GBps": env_steps * 68 / (ms * 1e-3) / 1e9, "policy_tflops": env_steps * 8704.0 / (ms * 1e-3) / 1e12, "gather_batch": batch, "gather_us": gather_us, "gather_algorithmic_GBps": batch * 85 / (gather_us * 1e-6) / 1e9,
            "evaluation_10_episodes_x_200_steps_us": evaluate_us,
            "acrobot": {"n_envs": n_acro, "us_per_step": acrobot_us, "env_steps_per_s": n_acro / (acrobot_us * 1e-6), "algorithmic_GBps": n_acro * 89 / (acrobot_us * 1e-6) / 1e9}}


def bench_ppo(helpers, rocm, n_envs=4096, steps=128, epochs=4, minibatch=8192):
    """Synthetic PPO iteration: GAE over a (steps+1) x n_envs dataset, then epochs x (rows / minibatch) minibatch updates of an actor
    105-64-64-8 (tanh, learned log_std) and a critic 105-64-64-1 (tanh) on host-drawn row permutations."""
    capi = helpers.capi
    O, A, H = 105, 8, 64
    rows = n_envs * steps
    rng = np.random.default_rng(3)
    col = dict(observations=0, actions=O, action_log_probs=O + A, rewards=O + A + 1, terminated=O + A + 2, truncated=O + A + 3, all_values=O + A + 4,
               advantages=O + A + 5, target_values=O + A + 6)
    ld = O + A + 7
    data = rng.standard_normal((rows + n_envs, ld)).astype(np.float32)
    done = (rng.random(rows + n_envs) < 0.01).astype(np.float32)
    data[:, col["terminated"]] = done; data[:, col["truncated"]] = done
    data[:, col["action_log_probs"]] = (-0.9189385 - np.log(0.5) - 0.5 * (data[:, O:O + A] / 0.5) ** 2).sum(1)
    params = np.concatenate([helpers.random_params(rng, [O, H, H, A]) * 0.1, np.log(np.full(A, 0.5, np.float32)), helpers.random_params(rng, [O, H, H, 1])]).astype(np.float32)
    agent = helpers.PpoOnBackend(rocm, O, A, H, H, minibatch, params, "tanh", "tanh", capi.adam_parameters(3e-4, epsilon=1e-8))
    pp = capi.ppo_parameters()
    dd = rocm.array(data)
    perms = [rocm.array(rng.permutation(rows).astype(np.uint32)) for _ in range(epochs)]
    ev = HipEvents(rocm.device.lib.rlt_rocm_get_stream(rocm.device.handle))

    def gae():
        rocm.call("ppo_gae", dd.offset(col["rewards"]), dd.offset(col["terminated"]), dd.offset(col["truncated"]), dd.offset(col["all_values"]),
                  dd.offset(col["advantages"]), dd.offset(col["target_values"]), ld, n_envs, steps, 0.99, 0.95, 0)

    def iteration():
        for perm in perms:      # one call per epoch: the reference's batch loop over the epoch's shuffled rows
            rocm.call("ppo_train_epoch", C.byref(agent.c), C.byref(pp), dd.offset(col["observations"]), dd.offset(col["observations"]), dd.offset(col["actions"]),
                      dd.offset(col["action_log_probs"]), dd.offset(col["advantages"]), dd.offset(col["target_values"]), ld, perm.ptr, rows // minibatch, None)
    for _ in range(3):
        gae()
    rocm.sync()
    a = ev.record()
    for _ in range(20):
        gae()
    e = ev.record()
    gae_us = ev.elapsed_ms(a, e) * 1e3 / 20
    iteration(); rocm.sync()
    a = ev.record(); iteration(); e = ev.record()
    ms = ev.elapsed_ms(a, e)
    n_updates = epochs * (rows // minibatch)
    flop = 106368.0 * rows * epochs
    # on-policy collection with the Pendulum: 4,096 environments x 128 steps (actor 3-64-64-1, standardized observations), one launch for all steps
    pn, ps = 4096, 128
    pcol = dict(observations=0, actions_mean=3, actions=4, action_log_probs=5, rewards=6, terminated=7, truncated=8, all_reset=9, all_values=10)
    runner = helpers.OnPolicyOnBackend(rocm, pn, ps, 13, pcol, 200)
    pdims = [3, 64, 64, 1]
    pactor = helpers.Mlp(rocm, pdims, helpers.random_params(rng, pdims), pn, "relu", "tanh", trainable=False)
    ls, nz = rocm.array(np.array([-0.5], np.float32)), rocm.array(rng.standard_normal((ps, pn, 1)).astype(np.float32))
    ini = rocm.array(np.stack([rng.uniform(-np.pi, np.pi, (ps, pn)), rng.uniform(-1, 1, (ps, pn))], 2).astype(np.float32))
    sm, sp = rocm.array(np.zeros(3, np.float32)), rocm.array(np.ones(3, np.float32))
    wsn = rocm.device.lib.rlt_rocm_on_policy_collect_workspace_bytes(C.byref(runner.c), pactor.layers, pactor.n)
    ws, wsn = rocm.workspace(wsn)

    def collect():
        rocm.call("on_policy_collect", C.byref(runner.c), C.byref(runner.d), pactor.layers, pactor.n, ls.ptr, sm.ptr, sp.ptr, nz.ptr, ini.ptr, 0, ws, wsn)
    collect(); rocm.sync()
    a = ev.record()
    for _ in range(5):
        collect()
    e = ev.record()
    collect_ms = ev.elapsed_ms(a, e) / 5
    return {"rows": rows, "minibatch": minibatch, "epochs": epochs, "gae_us": gae_us, "gae_algorithmic_GBps": rows * 24 / (gae_us * 1e-6) / 1e9,
            "iteration_ms": ms, "us_per_minibatch_update": ms * 1e3 / n_updates, "samples_per_s": rows * epochs / (ms * 1e-3), "tflops": flop / (ms * 1e-3) / 1e12,
            "pendulum_collect": {"n_envs": pn, "steps": ps, "ms": collect_ms, "env_steps_per_s": pn * ps / (collect_ms * 1e-3)}}


def bench_gru(helpers, rocm, batch, S=64, I=146, H=64, iters=10):
    """Sequence model step: GRU 146->64 over 64 steps, head 64->64 (tanh) ->4, MSE loss, backward through time, Adam on everything."""
    capi = helpers.capi
    rng = np.random.default_rng(4)
    params, x, _, _ = helpers.gru_random_case(rng, S, batch, I, H, False)
    params["h0"] = np.zeros(H, np.float32)
    gru = helpers.GruOnBackend(rocm, S, batch, I, H, params)
    rows = S * batch
    head = helpers.Mlp(rocm, [H, 64, 4], helpers.xavier_params(rng, [H, 64, 4]), rows, "tanh", "identity")
    target = rocm.array(rng.standard_normal((rows, 4)).astype(np.float32))
    y_head, d_h = rocm.zeros((rows, 4)), rocm.zeros((S, batch, H))
    xd = rocm.array(x)
    moments = [rocm.zeros(a.shape) for a in (gru.W_i, gru.b_i, gru.W_h, gru.b_h) for _ in range(2)]
    tensors = []
    for k, (p, g, flag) in enumerate(((gru.W_i, gru.dW_i, 1), (gru.b_i, gru.db_i, 2), (gru.W_h, gru.dW_h, 1), (gru.b_h, gru.db_h, 2))):
        tensors.append(capi.AdamTensor(p.ptr, g.ptr, moments[2 * k].ptr, moments[2 * k + 1].ptr, None, int(np.prod(p.shape)), flag))
    # one optimiser for the whole model: the GRU's four tensors and the head's four in one Adam launch
    tensors += [head.adam[i] for i in range(head.n_adam)]
    model_adam = (capi.AdamTensor * len(tensors))(*tensors)
    age = rocm.array(np.array([1], np.uint32))
    adam = capi.adam_parameters(epsilon=1e-8)
    ws, wsn = head.workspace()
    ev = HipEvents(rocm.device.lib.rlt_rocm_get_stream(rocm.device.handle))
    n_gru_gradients = int(np.prod(gru.grads.shape))

    def step():
        rocm.call("fill_f32", gru.grads.ptr, 1, n_gru_gradients, n_gru_gradients, 0.0)      # the GRU's gradient tensors are one flat array
        rocm.call("mlp_zero_gradient", head.layers, head.n)
        rocm.call("gru_forward", C.byref(gru.c), xd.ptr, None, S, batch, gru.ws, gru.wsn)
        # the head's forward, MSE gradient (2 / (rows * 4) * (y - target), loss weight 1) and backward_full with the gradient for the GRU's output
        rocm.call("mlp_forward_backward_input", head.layers, head.n, gru.out.ptr, H, y_head.ptr, 4, None, 0, target.ptr, 4, 2.0 / (rows * 4), d_h.ptr, H, rows, ws, wsn)
        rocm.call("gru_backward", C.byref(gru.c), xd.ptr, d_h.ptr, None, None, S, batch, 1, gru.ws, gru.wsn)
        rocm.call("adam_step", model_adam, len(tensors), C.byref(adam), age.ptr, 0.0, None)
    for _ in range(3):
        step()
    rocm.sync()
    a = ev.record()
    for _ in range(iters):
        step()
    e = ev.record()
    ms = ev.elapsed_ms(a, e) / iters
    return {"batch": batch, "sequence_length": S, "ms_per_step": ms, "sequences_per_s": batch / (ms * 1e-3), "tflops": 211968.0 * rows / (ms * 1e-3) / 1e12}


def bench_sac_sequence(helpers, rocm, S=100, B=100, iters=10, cpu_seconds=1.5):
    """The training part of one SAC loop step on a sequence batch with the reference's recurrent approximators at the sizes of its Pendulum
    configuration with memory (100 sequences of 100 steps; actor dense-GRU-GRU-dense at width 16, critics at width 32): 2 critic updates,
    target update, actor update. The same calls on the CPU checker (one thread, plain loops) are timed next to it on a bounded sample."""
    rng = np.random.default_rng(6)
    OBS, ACT = 3, 1
    actor_specs = [(0, OBS, 16, "relu"), (1, 16, 16, "identity"), (1, 16, 16, "identity"), (0, 16, 2 * ACT, "identity")]
    critic_specs = [(0, OBS + ACT, 32, "relu"), (1, 32, 32, "identity"), (1, 32, 32, "identity"), (0, 32, 1, "identity")]
    critics = [helpers.random_seq_params(rng, critic_specs) for _ in range(2)]
    params = np.concatenate([helpers.random_seq_params(rng, actor_specs)] + critics + [c.copy() for c in critics] + [np.array([0.0], np.float32)])
    final = (rng.uniform(size=(S, B)) < 0.05).astype(np.uint8); final[-1] = 1
    reset = np.zeros((S, B), np.uint8); reset[0] = 1; reset[1:] = final[:-1]
    next_reset = np.zeros((S + 1, B), np.uint8); next_reset[0] = 1; next_reset[1:] = final
    next_final = np.zeros((S + 1, B), np.uint8); next_final[1:] = final
    data = dict(observations_actions_base=rng.standard_normal((S + 1, B, OBS + ACT)).astype(np.float32), rewards=rng.standard_normal((S, B)).astype(np.float32),
                terminated=np.zeros((S, B), np.uint8), reset=reset, next_reset_base=next_reset, final_step_mask=final, next_final_step_mask_base=next_final)
    nc, na = rng.standard_normal((S + 1, B, ACT)).astype(np.float32), rng.standard_normal((S, B, ACT)).astype(np.float32)
    out = {"sequence_length": S, "batch": B, "actor": "3-16-GRU16-GRU16-2", "critic": "4-32-GRU32-GRU32-1"}
    for be in (rocm, checker().HostBackend()):      # the CPU leg: the same calls on the checker
        agent = helpers.SacSequenceOnBackend(be, actor_specs, critic_specs, params, S, B, OBS, ACT, True)
        agent.set_batch(data)
        ncd, nad = be.array(nc), be.array(na)

        def step(together=False):
            if together:      # both critics in one call: the loop's shared batch (what the devices::ROCM loop step issues)
                be.call("sac_sequence_train_critics", C.byref(agent.c), ncd.ptr)
            for k in range(0 if together else 2):
                be.call("sac_sequence_train_critic", C.byref(agent.c), k, ncd.ptr)
            be.call("sac_sequence_update_critic_targets", C.byref(agent.c))
            be.call("sac_sequence_train_actor", C.byref(agent.c), nad.ptr)
        if be.name == "rocm":
            ev = HipEvents(rocm.device.lib.rlt_rocm_get_stream(rocm.device.handle))
            for _ in range(3):
                step(True)
            rocm.sync()
            a = ev.record()
            for _ in range(iters):
                step(True)
            e = ev.record()
            out["ms_per_training_step_both_critics_in_one_call"] = ev.elapsed_ms(a, e) / iters
            for _ in range(3):
                step()
            rocm.sync()
            a = ev.record()
            t0 = time.perf_counter()
            for _ in range(iters):
                step()
            host_ms = (time.perf_counter() - t0) * 1e3 / iters      # what the host needs to issue a step's launches (it does not wait for them)
            e = ev.record()
            ms = ev.elapsed_ms(a, e) / iters
            out["ms_per_training_step"] = ms
            out["host_ms_to_issue_a_training_step"] = host_ms
            out["sequences_per_s"] = 3 * B / (ms * 1e-3)
        else:
            step()
            t0 = time.perf_counter(); n = 0
            while time.perf_counter() - t0 < cpu_seconds:
                step(); n += 1
            out["cpu_checker_ms_per_training_step"] = (time.perf_counter() - t0) / n * 1e3
            out["cpu_sample"] = f"{n} training steps of the CPU restatement, one thread"
    # the runner step with the recurrent actor over 4,096 environments (prologue, policy state reset, one evaluate_step, action draw, epilogue + replay add)
    N = 4096
    run = helpers.RecurrentRunnerOnBackend(rocm, actor_specs, params[:helpers.seq_param_count(actor_specs)], N, 16, 200, S)
    noise = rocm.array(rng.standard_normal(N).astype(np.float32))
    ini = rocm.array(np.stack([rng.uniform(-np.pi, np.pi, N), rng.uniform(-1, 1, N)], 1).astype(np.float32))

    def runner_step():
        rocm.call("pendulum_runner_step_recurrent", C.byref(run.c), C.byref(run.rb.c), run.policy.layers, run.policy.n, C.byref(run.state.c), run.period, C.byref(run.sas),
                  noise.ptr, ini.ptr, run.ws, run.wsn)
    for _ in range(3):
        runner_step()
    rocm.sync()
    ev = HipEvents(rocm.device.lib.rlt_rocm_get_stream(rocm.device.handle))
    a = ev.record()
    for _ in range(50):
        runner_step()
    e = ev.record()
    us = ev.elapsed_ms(a, e) / 50 * 1e3
    out["recurrent_runner_step"] = {"n_envs": N, "us_per_step": us, "env_steps_per_s": N / (us * 1e-6)}
    # the evaluation step of the loop with the recurrent actor: 10 episodes of 200 steps (state reset, then observe, evaluate_step and environment step per step)
    E, L = 10, 200
    policy = helpers.SeqNet(rocm, actor_specs, params[:helpers.seq_param_count(actor_specs)], 1, E, trainable=False)
    state = helpers.SeqStateOnBackend(rocm, actor_specs, E)
    env = helpers.capi.pendulum_parameters()
    ini_e = rocm.array(np.stack([rng.uniform(-np.pi, np.pi, E), rng.uniform(-1, 1, E)], 1).astype(np.float32))
    ret, length, summary = rocm.zeros((E,)), rocm.zeros((E,), np.uint32), rocm.zeros((6,))
    wsn = int(rocm.device.lib.rlt_rocm_pendulum_evaluate_recurrent_workspace_bytes(policy.layers, policy.n, E))
    ws = rocm.device.empty((wsn,), np.uint8)

    def evaluation():
        rocm.call("pendulum_evaluate_recurrent", C.byref(env), 2, policy.layers, policy.n, C.byref(state.c), S, ini_e.ptr, E, L, ret.ptr, length.ptr, summary.ptr, ws.ptr, wsn)
    evaluation()
    rocm.sync()
    a = ev.record()
    for _ in range(3):
        evaluation()
    e = ev.record()
    out["recurrent_evaluation"] = {"episodes": E, "steps": L, "ms": ev.elapsed_ms(a, e) / 3}
    return out


def pmc_probe(helpers, rocm, batch):
    n = 64 * 1024 * 1024      # floats: 256 MiB read + 256 MiB written per copy
    src, dst = rocm.zeros((n,)), rocm.zeros((n,))
    for _ in range(3):
        rocm.call("memcpy_d2d", dst.ptr, src.ptr, n * 4)
    rocm.sync()
    dims = [17, 256, 256, 6]
    rng = np.random.default_rng(0)
    net = helpers.Mlp(rocm, dims, helpers.xavier_params(rng, dims), batch)
    x = rocm.array(rng.standard_normal((batch, 17)).astype(np.float32)); dy = rocm.array(rng.standard_normal((batch, 6)).astype(np.float32)); y = rocm.zeros((batch, 6))
    ws, wsn = net.workspace()
    for _ in range(3):
        rocm.call("mlp_forward_backward", net.layers, net.n, x.ptr, 17, y.ptr, 6, dy.ptr, 6, None, 0, 0.0, batch, ws, wsn)
    rocm.sync()


def bench_sac(helpers, rocm, steps, warmup, batch=256, capacity=10000, per_operation=False, phase_profile=False):
    """SAC loop steps entirely on the device: runner step with the actor, device-side gather draws and noise, training."""
    capi = helpers.capi
    lib, h = rocm.device.lib, rocm.device.handle
    rng = np.random.default_rng(1)
    na, nc = helpers.mlp_param_count([3, 64, 64, 2]), helpers.mlp_param_count([4, 64, 64, 1])
    critics = [helpers.random_params(rng, [4, 64, 64, 1]) for _ in range(2)]
    params = np.concatenate([helpers.random_params(rng, [3, 64, 64, 2])] + critics + critics + [np.array([np.log(0.5)], np.float32)])
    agent = helpers.SacOnBackend(rocm, batch, 64, params, masks=False)
    rb = helpers.ReplayOnBackend(rocm, 1, capacity)
    states, ep_step, ep_ret, trunc = rocm.zeros((1, 2)), rocm.zeros((1,), np.uint32), rocm.zeros((1,)), rocm.array(np.ones(1, np.uint8))
    runner = capi.PendulumRunner(states.ptr, ep_step.ptr, ep_ret.ptr, trunc.ptr, 1, 200, capi.pendulum_parameters())
    rollout_noise, warm_action = rocm.zeros((1, 1)), rocm.zeros((1, 1))
    noise_c, noise_a = rocm.zeros((batch, 1)), rocm.zeros((batch, 1))
    env_idx, offs = rocm.zeros((batch,), np.uint32), rocm.zeros((batch,), np.uint32)
    seed = 1234
    counter = [0]

    def env_step(policy):
        counter[0] += 1
        c = counter[0]
        if policy == 0:
            rocm.check(lib.rlt_rocm_rand_f32(h, warm_action.ptr, 1, -1.0, 1.0, seed, 8 * c))
        else:
            rocm.check(lib.rlt_rocm_randn_f32(h, rollout_noise.ptr, 1, seed, 8 * c))
        rocm.check(lib.rlt_rocm_pendulum_runner_step(h, C.byref(runner), C.byref(rb.c), 2 if policy else 0, agent.actor.layers, 3, C.byref(agent.c.sas),
                                                     warm_action.ptr, rollout_noise.ptr, None, seed, 8 * c + 1))

    rocm.check = rocm.device.check

    for _ in range(batch):        # fill the replay buffer with the warm-up policy
        env_step(0)
    if per_operation:             # one launch per reference operation, driven by the library's host loop over its own entry points
        scratch = capi.SacLoopScratch(rollout_noise.ptr, noise_c.ptr, noise_a.ptr, env_idx.ptr, offs.ptr)
        rocm.call("sac_set_per_operation", 1)
        try:
            rocm.call("sac_pendulum_loop_by_calls", C.byref(agent.c), C.byref(runner), C.byref(rb.c), warmup, seed, 1 << 20, C.byref(scratch))
            rocm.sync()
            t0 = time.perf_counter()
            rocm.call("sac_pendulum_loop_by_calls", C.byref(agent.c), C.byref(runner), C.byref(rb.c), steps, seed, (1 << 20) + warmup, C.byref(scratch))
            rocm.sync()
            dt = time.perf_counter() - t0
        finally:
            rocm.call("sac_set_per_operation", 0)
    else:                         # the persistent kernel: all `steps` loop steps in one launch
        ticks, stage_ticks = rocm.zeros((16,), np.uint64), rocm.zeros((48,), np.uint64)
        outputs = capi.SacLoopOutputs(None, None, None, None, None, ticks.ptr if phase_profile else None)
        if phase_profile == "stages":
            outputs.stage_ticks = stage_ticks.ptr
        ev = HipEvents(lib.rlt_rocm_get_stream(h))
        done = [0]

        def run(n):
            rocm.check(lib.rlt_rocm_sac_pendulum_loop(h, C.byref(agent.c), C.byref(runner), C.byref(rb.c), n, seed, done[0], None, C.byref(outputs)))
            done[0] += n
        run(max(warmup, 1))
        rocm.sync()
        ticks.upload(np.zeros(16, np.uint64)); stage_ticks.upload(np.zeros(48, np.uint64))
        # HIP events on the library's stream around launches of `steps` loop steps each, repeated until at least 5 ms are timed (a single
        # short launch would mostly measure the launch itself); everything the loop reads and writes is resident on the device
        launches = 0
        a = ev.record()
        while True:
            run(steps)
            launches += 1
            if launches * steps * 20e-6 >= 5e-3:       # about 20 us per loop step: enqueue enough work before the first look at the clock
                b = ev.record()
                dt = ev.elapsed_ms(a, b) * 1e-3
                if dt >= 5e-3 or launches >= 4096:
                    break
        total_steps = launches * steps
        long_run = None
        if steps < 20000:         # the same measurement with one launch of 20,000 steps, for reference
            a = ev.record(); run(20000); b = ev.record()
            long_run = 20000 / (ev.elapsed_ms(a, b) * 1e-3)
        if phase_profile:
            names = ["env step", "critic phase: TD error + both backward passes", "announce critic gradients", "wait + critic Adam", "announce + wait for critic parameters", "critic weight refresh",
                     "actor phase", "announce + wait for actor gradients", "actor Adam", "announce + wait for actor parameters", "actor weight refresh"]
            names += ["critic phase: batch rows into LDS", "critic phase: actor on next obs | critic 1 forward", "critic phase: target critics", "critic phase: critic 0 forward", "unused"]
            tk = ticks.numpy()[:16].astype(np.float64) / 100.0 / (total_steps + (20000 if long_run else 0))      # 100 MHz constant clock -> microseconds per step
            shader_cycles = tk[15] * 100.0; tk = tk[:15]; names = names[:15]
            print("phase profile (us per loop step, workgroup 0):", {f"{i}:{n}": round(float(v), 2) for i, (n, v) in enumerate(zip(names, tk))}, "sum", round(float(tk.sum()), 2),
                  "shader clock MHz", round(shader_cycles / tk.sum(), 1), file=sys.stderr, flush=True)
            if phase_profile == "stages":
                mhz = shader_cycles / tk.sum()
                st = stage_ticks.numpy().astype(np.float64) / 100.0 / (total_steps + (20000 if long_run else 0)) * mhz      # shader cycles per loop step
                stage_names = {0: "A layer 1 (actor on next obs | critic 1)", 2: "A layers 2+3", 4: "next action + log-probability (one wavefront)", 6: "B layer 1 (target critics)",
                               8: "B layers 2+3", 10: "TD target + D layer 1 (critic 0 | actor on obs)", 12: "D layers 2+3", 14: "d_output, actor sample (one wavefront each)",
                               16: "critics backward: layer 3, gate of layer 2", 18: "critics backward: dW2, layer 1",
                               20: "critics on new action: layer 1", 22: "layers 2+3", 24: "backward layer 3, gate", 26: "backward layer 1 -> d action",
                               28: "min-Q routing, sample_and_squash backward (one wavefront)", 30: "actor backward: layer 3, gate", 32: "actor backward: dW2 | layer 1, target polyak in LDS"}
                print("stage profile (shader cycles per loop step, thread 0 of workgroup 0): stage's own instructions / wait at the barrier behind it", file=sys.stderr)
                for i in sorted(stage_names):
                    print("  %2d %-70s %7.0f  / %5.0f" % (i, stage_names[i], st[i], st[i + 1] if i + 1 < 48 and i not in (18, 32) else 0.0), file=sys.stderr)
                print("  critic phase stages sum %.0f cycles, actor phase stages sum %.0f cycles" % (st[:19].sum(), st[20:33].sum()), file=sys.stderr, flush=True)
    p = agent.parameters()
    assert np.all(np.isfinite(p)), "SAC parameters went non-finite"
    # what the run has learned (untimed): 100 evaluation episodes of 200 steps with the actor as it stands after warmup + steps loop steps from random weights
    ini = rocm.array(np.stack([rng.uniform(-np.pi, np.pi, 100), rng.uniform(-1, 1, 100)], 1).astype(np.float32))
    ret, length, summary = rocm.zeros((100,)), rocm.zeros((100,), np.uint32), rocm.zeros((6,))
    env = capi.pendulum_parameters()
    rocm.call("pendulum_evaluate", C.byref(env), 2, agent.actor.layers, agent.actor.n, ini.ptr, 100, 200, ret.ptr, length.ptr, summary.ptr)
    rocm.sync()
    if per_operation:
        total_steps, launches, long_run = steps, None, None
    return {"steps_per_s": total_steps / dt, "ms_per_step": dt / total_steps * 1e3, "launches_per_step": (1.0 / steps) if not per_operation else None,
            "timed_loop_steps": total_steps, "timed_launches": launches, "steps_per_s_one_launch_of_20000_steps": long_run,
            "evaluation_return_after_run": float(summary.numpy()[0])}


def bench_sac_api(helpers, rocm, steps=2000, warmup=200, batch=256, capacity=10000, graph_replay=True):
    """The API path: the reference's loop step composed of the library's own entry points by its host loop (no Python between the calls),
    with the fused three-launch updates; and the four update calls alone on synthetic batches for a wider agent (observation 27, action 8)."""
    capi = helpers.capi
    lib, h = rocm.device.lib, rocm.device.handle
    rng = np.random.default_rng(1)
    out = {}

    def parameters(obs, act, hidden=64):
        critics = [helpers.random_params(rng, [obs + act, hidden, hidden, 1]) for _ in range(2)]
        return np.concatenate([helpers.random_params(rng, [obs, hidden, hidden, 2 * act])] + critics + critics + [np.array([np.log(0.5)], np.float32)])

    agent = helpers.SacOnBackend(rocm, batch, 64, parameters(3, 1), masks=False)
    rb = helpers.ReplayOnBackend(rocm, 1, capacity)
    states, ep_step, ep_ret, trunc = rocm.zeros((1, 2)), rocm.zeros((1,), np.uint32), rocm.zeros((1,)), rocm.array(np.ones(1, np.uint8))
    runner = capi.PendulumRunner(states.ptr, ep_step.ptr, ep_ret.ptr, trunc.ptr, 1, 200, capi.pendulum_parameters())
    rollout_noise, warm_action = rocm.zeros((1, 1)), rocm.zeros((1, 1))
    noise_c, noise_a = rocm.zeros((batch, 1)), rocm.zeros((batch, 1))
    env_idx, offs = rocm.zeros((batch,), np.uint32), rocm.zeros((batch,), np.uint32)
    seed = 99
    for c in range(1, batch + 1):      # fill the replay buffer with the uniform warm-up policy
        rocm.device.check(lib.rlt_rocm_rand_f32(h, warm_action.ptr, 1, -1.0, 1.0, seed, 8 * c))
        rocm.device.check(lib.rlt_rocm_pendulum_runner_step(h, C.byref(runner), C.byref(rb.c), 0, agent.actor.layers, 3, C.byref(agent.c.sas), warm_action.ptr, None, None, seed, 8 * c + 1))
    scratch = capi.SacLoopScratch(rollout_noise.ptr, noise_c.ptr, noise_a.ptr, env_idx.ptr, offs.ptr)
    ev = HipEvents(lib.rlt_rocm_get_stream(h))
    # how the update kernels finish and where their workgroups run (rlt_rocm_set_update_options); the library's default comes last and is the figure reported
    variants = {}
    offset = 1 << 20
    for name, tail, one_xcd in (("optimiser_as_own_launch", 0, 1), ("optimiser_in_kernel_spread_over_xcds", 1, 0), ("optimiser_in_kernel_one_xcd", 1, 1)):
        rocm.call("set_update_options", tail, one_xcd)
        rocm.call("sac_pendulum_loop_by_calls", C.byref(agent.c), C.byref(runner), C.byref(rb.c), warmup, seed, offset, C.byref(scratch))
        rocm.sync()
        t0 = time.perf_counter(); a = ev.record()
        rocm.call("sac_pendulum_loop_by_calls", C.byref(agent.c), C.byref(runner), C.byref(rb.c), steps, seed, offset + warmup, C.byref(scratch))
        b = ev.record()
        device_s = ev.elapsed_ms(a, b) * 1e-3       # waits for the second event
        wall_s = time.perf_counter() - t0
        offset += warmup + steps
        variants[name] = {"steps_per_s": steps / wall_s, "steps_per_s_by_device_clock": steps / device_s, "launches_per_step": 4 if tail else 7}
    # the same loop step recorded into a HIP graph (rlt_rocm_graph_*; what rl/environments/pendulum/sac/cuda/sac.cu:122-164 does with its step) and replayed
    graph = C.c_void_p()
    if graph_replay:
        rocm.call("graph_begin_capture")
        try:
            rocm.call("sac_pendulum_loop_by_calls", C.byref(agent.c), C.byref(runner), C.byref(rb.c), 1, seed, offset, C.byref(scratch))
            rocm.call("advance_streams", 8)
        finally:
            rocm.call("graph_end_capture", C.byref(graph))
    try:
        for _ in range(warmup if graph_replay else 0):
            rocm.call("graph_launch", graph)
        rocm.sync()
        t0 = time.perf_counter(); a = ev.record()
        for _ in range(steps if graph_replay else 0):
            rocm.call("graph_launch", graph)
        b = ev.record()
        graph_device_s = ev.elapsed_ms(a, b) * 1e-3
        if graph_replay:
            variants["recorded_graph_replayed"] = {"steps_per_s": steps / (time.perf_counter() - t0), "steps_per_s_by_device_clock": steps / graph_device_s, "launches_per_step": 4}
    finally:
        rocm.call("set_stream_offset", 0)
        if graph_replay:
            rocm.call("graph_destroy", graph)
    assert np.all(np.isfinite(agent.parameters())), "SAC parameters went non-finite"
    out.update(steps_per_s=steps / wall_s, steps_per_s_by_device_clock=steps / device_s, steps=steps, launches_per_step=4, variants=variants)
    # a wider agent: the update calls alone
    obs, act = 27, 8
    wide = helpers.SacOnBackend(rocm, batch, 64, parameters(obs, act), masks=False, obs=obs, act=act)
    oab = rng.standard_normal((2, batch, obs + act)).astype(np.float32); oab[:, :, obs:] = np.tanh(oab[:, :, obs:])
    wide.set_batch(oab, rng.standard_normal(batch).astype(np.float32), (rng.random(batch) < 0.05).astype(np.uint8))
    noise = rocm.array(rng.standard_normal((batch, act)).astype(np.float32))

    def updates(n):
        for _ in range(n):
            rocm.device.check(lib.rlt_rocm_sac_train_critics(h, C.byref(wide.c), noise.ptr, 1))
            rocm.device.check(lib.rlt_rocm_sac_train_actor(h, C.byref(wide.c), noise.ptr))
    updates(20)
    rocm.sync()
    a = ev.record(); updates(300); b = ev.record()
    out["wide_agent_obs27_act8_update_sets_per_s_by_device_clock"] = 300 / (ev.elapsed_ms(a, b) * 1e-3)
    # hidden width 256 (the zoo's AcrobotSwingup agent: observation 6, action 1): the per-operation path, about 60 launches per set of updates
    obs, act = 6, 1
    wide = helpers.SacOnBackend(rocm, batch, 256, parameters(obs, act, 256), masks=False, obs=obs, act=act)
    oab = rng.standard_normal((2, batch, obs + act)).astype(np.float32); oab[:, :, obs:] = np.tanh(oab[:, :, obs:])
    wide.set_batch(oab, rng.standard_normal(batch).astype(np.float32), (rng.random(batch) < 0.05).astype(np.uint8))
    noise = rocm.array(rng.standard_normal((batch, act)).astype(np.float32))
    updates(20)
    rocm.sync()
    a = ev.record(); updates(300); b = ev.record()
    out["width256_agent_obs6_act1_update_sets_per_s_by_device_clock"] = 300 / (ev.elapsed_ms(a, b) * 1e-3)
    # TD3 at the shapes of the zoo's Ant agent (src/rl/zoo/ant-v4/td3.h: observation 27, action 8, hidden width 256, ReLU, batch 256): both critics, the actor, the three
    # target updates per set
    obs, act = 27, 8
    adims, cdims = [obs, 256, 256, act], [obs + act, 256, 256, 1]
    nets = [helpers.random_params(rng, adims)] * 2 + [helpers.random_params(rng, cdims) for _ in range(2)]
    td3 = helpers.Td3OnBackend(rocm, batch, 256, np.concatenate(nets + [nets[2], nets[3]]).astype(np.float32), masks=False, obs=obs, act=act)
    oab = rng.standard_normal((2, batch, obs + act)).astype(np.float32); oab[:, :, obs:] = np.tanh(oab[:, :, obs:])
    td3.set_batch(oab, rng.standard_normal(batch).astype(np.float32), (rng.random(batch) < 0.05).astype(np.uint8), np.clip(rng.standard_normal((batch, act)) * 0.2, -0.5, 0.5).astype(np.float32))
    noise = rocm.array(rng.standard_normal((batch, act)).astype(np.float32))

    draws = helpers.capi.Td3CriticDraws(1, 4, (C.c_uint64 * 2)(5, 6), 0.2, 0.5)

    def td3_updates(n, one_call=True):
        for _ in range(n):
            if one_call:        # the loop's shared-batch case: the smoothing noise, both critics and their targets by one call with the draws made inside
                rocm.device.check(lib.rlt_rocm_td3_train_critics_drawn(h, C.byref(td3.c), C.byref(draws), None, 1))
                rocm.device.check(lib.rlt_rocm_td3_train_actor_drawn(h, C.byref(td3.c), 1, 7, None))
            else:               # a call per operation on noise tensors that are given
                for k in (0, 1):
                    rocm.device.check(lib.rlt_rocm_td3_train_critic(h, C.byref(td3.c), k, noise.ptr))
                rocm.device.check(lib.rlt_rocm_td3_update_critic_targets(h, C.byref(td3.c)))
                rocm.device.check(lib.rlt_rocm_td3_train_actor(h, C.byref(td3.c), noise.ptr))
            rocm.device.check(lib.rlt_rocm_td3_update_actor_target(h, C.byref(td3.c)))
    td3_updates(20)
    rocm.sync()
    a = ev.record(); td3_updates(300); b = ev.record()
    out["td3_width256_agent_obs27_act8_update_sets_per_s_by_device_clock"] = 300 / (ev.elapsed_ms(a, b) * 1e-3)
    td3_updates(20, False)
    rocm.sync()
    a = ev.record(); td3_updates(300, False); b = ev.record()
    out["td3_width256_agent_obs27_act8_update_sets_per_s_a_call_per_critic"] = 300 / (ev.elapsed_ms(a, b) * 1e-3)
    # TD3 at the shapes of the zoo's Pendulum agent (src/rl/zoo/pendulum-v1/td3.h: observation 3, action 1, hidden width 64, batch 100): the same two ways
    obs, act, td3_batch = 3, 1, 100
    nets = [helpers.random_params(rng, [obs, 64, 64, act])] * 2 + [helpers.random_params(rng, [obs + act, 64, 64, 1]) for _ in range(2)]
    td3 = helpers.Td3OnBackend(rocm, td3_batch, 64, np.concatenate(nets + [nets[2], nets[3]]).astype(np.float32), masks=False, obs=obs, act=act)
    oab = rng.standard_normal((2, td3_batch, obs + act)).astype(np.float32); oab[:, :, obs:] = np.tanh(oab[:, :, obs:])
    td3.set_batch(oab, rng.standard_normal(td3_batch).astype(np.float32), (rng.random(td3_batch) < 0.05).astype(np.uint8),
                  np.clip(rng.standard_normal((td3_batch, act)) * 0.2, -0.5, 0.5).astype(np.float32))
    noise = rocm.array(rng.standard_normal((td3_batch, act)).astype(np.float32))
    for one_call, key in ((True, "td3_width64_agent_obs3_act1_b100_update_sets_per_s_by_device_clock"), (False, "td3_width64_agent_obs3_act1_b100_update_sets_per_s_a_call_per_critic")):
        td3_updates(20, one_call)
        rocm.sync()
        a = ev.record(); td3_updates(300, one_call); b = ev.record()
        out[key] = 300 / (ev.elapsed_ms(a, b) * 1e-3)
    return out


def cpu_baseline(batch=256, seconds=12.0):
    """The reference's own SAC loop (compiled from the reference, CBLAS backend, one thread) on this host; falls back to the
    CPU restatement when that build is not present."""
    ref = os.path.join(ROOT, "oracle", "_ref", "librlt_ref_blas.so")
    cores = 1
    if os.path.exists(ref):
        lib = C.CDLL(ref)
        lib.rlt_ref_sac_create.restype = C.c_void_p
        lib.rlt_ref_sac_time_steps.restype = C.c_double
        lib.rlt_ref_sac_time_steps.argtypes = [C.c_void_p, C.c_int]
        lib.rlt_ref_cblas_name.restype = C.c_char_p
        lib.rlt_ref_sac_destroy.argtypes = [C.c_void_p]
        n, total, seed = 0, 0.0, 0
        while total < seconds:                                  # the reference's loop stops at its STEP_LIMIT of 10,000 steps
            hdl = C.c_void_p(lib.rlt_ref_sac_create(seed, batch)); seed += 1
            lib.rlt_ref_sac_time_steps(hdl, batch + 50)         # warm-up policy phase + first training steps (untimed)
            for _ in range(9):
                total += lib.rlt_ref_sac_time_steps(hdl, 1000); n += 1000
                if total >= seconds:
                    break
            lib.rlt_ref_sac_destroy(hdl)
        return {"value": n / total, "unit": "loop steps/s", "cores": cores, "kind": "reference", "cblas_path": lib.rlt_ref_cblas_name(),
                "sample": f"{n} post-warm-up loop steps of the reference's Pendulum SAC loop at batch {batch}, CBLAS = {os.path.basename(lib.rlt_ref_cblas_name().decode())}, 1 thread"}
    o = checker().HostBackend()
    cfg = checker().LoopConfig(0, batch, 64, 10000, batch, 200, 1e-7)
    loop = C.c_void_p(o.lib.rlt_oracle_sac_loop_create(C.byref(cfg)))
    for _ in range(batch + 10):
        o.lib.rlt_oracle_sac_loop_step(loop)
    n, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(50):
            o.lib.rlt_oracle_sac_loop_step(loop)
        n += 50
    dt = time.perf_counter() - t0
    return {"value": n / dt, "unit": "loop steps/s", "cores": cores, "kind": "port", "sample": f"{n} loop steps of the CPU restatement (plain loops) at batch {batch}"}


def cpu_other_configurations(helpers, cblas_path):
    """The other configurations on this host's CPU, one thread, bounded samples (a few seconds in all): the CPU restatement with its three GEMMs per dense
    layer routed through the same CBLAS the reference's CPU build uses (what its CPU_BLAS device does), or plain loops where no CBLAS was found."""
    o = checker().HostBackend()
    capi = helpers.capi
    blas = bool(cblas_path) and o.lib.rlt_oracle_use_cblas(cblas_path) == 0
    out = {"kind": "port", "cores": 1, "gemm": os.path.basename(cblas_path.decode()) if blas else "plain loops"}
    rng = np.random.default_rng(0)
    try:
        # configuration 1: MLP 17-256-256-6 forward + backward on a 4,096-row sample
        B, dims = 4096, [17, 256, 256, 6]
        net = helpers.Mlp(o, dims, helpers.xavier_params(rng, dims), B)
        x, dy, y = o.array(rng.standard_normal((B, 17)).astype(np.float32)), o.array(rng.standard_normal((B, 6)).astype(np.float32)), o.zeros((B, 6))

        def fwd_bwd():
            o.call("mlp_forward_backward", net.layers, net.n, x.ptr, 17, y.ptr, 6, dy.ptr, 6, None, 0, 0.0, B, None, 0)
        fwd_bwd()
        t0 = time.perf_counter(); n = 0
        while time.perf_counter() - t0 < 2.0:
            fwd_bwd(); n += 1
        dt = (time.perf_counter() - t0) / n
        out["mlp_forward_backward"] = {"sample_rows": B, "ms": dt * 1e3, "tflops": (MLP_FLOP_PER_SAMPLE_FWD + MLP_FLOP_PER_SAMPLE_BWD) * B / dt / 1e12}
        # configuration 3: one PPO minibatch update of 8,192 rows (observation 105, 8 actions, hidden 64, tanh)
        O, A, H, B = 105, 8, 64, 8192
        params = np.concatenate([helpers.random_params(rng, [O, H, H, A]) * 0.1, np.log(np.full(A, 0.5, np.float32)), helpers.random_params(rng, [O, H, H, 1])]).astype(np.float32)
        agent = helpers.PpoOnBackend(o, O, A, H, H, B, params, "tanh", "tanh", capi.adam_parameters(3e-4, epsilon=1e-8))
        ld = O + A + 7
        data = rng.standard_normal((B, ld)).astype(np.float32)
        data[:, O + A] = (-0.9189385 - np.log(0.5) - 0.5 * (data[:, O:O + A] / 0.5) ** 2).sum(1)
        dd, pp = o.array(data), capi.ppo_parameters()

        def update():
            o.call("ppo_train_minibatch", C.byref(agent.c), C.byref(pp), dd.offset(0), dd.offset(0), dd.offset(O), dd.offset(O + A), dd.offset(O + A + 5), dd.offset(O + A + 6), ld, None, None)
        update()
        t0 = time.perf_counter(); n = 0
        while time.perf_counter() - t0 < 2.0:
            update(); n += 1
        out["ppo_minibatch_update"] = {"rows": B, "us": (time.perf_counter() - t0) / n * 1e6}
        # configuration 2: one runner step of 65,536 Pendulum environments (actor 3-64-64-1, replay add)
        N = 65536
        dims = [3, 64, 64, 1]
        actor = helpers.Mlp(o, dims, helpers.xavier_params(rng, dims), N, "relu", "tanh", trainable=False)
        rb = helpers.ReplayOnBackend(o, N, 16)
        states, ep_step, ep_ret, trunc = o.zeros((N, 2)), o.zeros((N,), np.uint32), o.zeros((N,)), o.array(np.ones(N, np.uint8))
        ini = o.array(np.stack([rng.uniform(-np.pi, np.pi, N), rng.uniform(-1, 1, N)], 1).astype(np.float32))
        runner = capi.PendulumRunner(states.ptr, ep_step.ptr, ep_ret.ptr, trunc.ptr, N, 200, capi.pendulum_parameters())

        def step():
            assert o.lib.rlt_oracle_pendulum_runner_step(C.byref(runner), C.byref(rb.c), 1, actor.layers, actor.n, None, None, None, ini.ptr) == 0
        step()
        t0 = time.perf_counter(); n = 0
        while time.perf_counter() - t0 < 2.0:
            step(); n += 1
        out["runner_step"] = {"n_envs": N, "us": (time.perf_counter() - t0) / n * 1e6}
    finally:
        o.lib.rlt_oracle_use_cblas(None)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20000)
    ap.add_argument("--warmup", type=int, default=1000)
    ap.add_argument("--mlp-batch", type=int, default=65536)
    ap.add_argument("--mlp-iters", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--only", choices=["all", "mlp", "sac", "env", "ppo", "gru", "seq", "api"], default="all")
    ap.add_argument("--sac-phase-profile", nargs="?", const="phases", default=None, choices=["phases", "stages"],
                    help="print the persistent kernel's per-phase time (stderr); 'stages' adds the clock between the barrier-separated stages of the critic and actor phases")
    ap.add_argument("--pmc-probe", action="store_true", help="for counter runs under rocprofv3 --pmc: three 256 MiB device copies (a kernel of known traffic, to scale the counters by) "
                    "three MLP forward+backward calls, then the environment-pipeline and PPO workloads (their figures discarded)")
    ap.add_argument("--no-graph-replay", action="store_true", help="leave out the replay of a recorded loop step (for runs under rocprofv3, whose kernel tracing does not survive hipGraphLaunch here)")
    ap.add_argument("--no-mlp-by-batch", action="store_true", help="leave out configuration 1's other two batch sizes (for a kernel trace of the batch named by --mlp-batch alone)")
    ap.add_argument("--sac-per-operation", action="store_true", help="time the one-launch-per-operation SAC path instead of the persistent kernel")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the hot path has no cross-GPU part); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    helpers = package().builders      # networks, agents, runners on a backend (rl-tools_amd/builders.py)
    rocm = helpers.RocmBackend()
    info = rocm.device.info()
    if args.pmc_probe:
        pmc_probe(helpers, rocm, args.mlp_batch)
        bench_env(helpers, rocm)       # runner_fused_kernel, gather_kernel, acrobot_step_kernel
        bench_ppo(helpers, rocm)       # gae_kernel, the minibatch update's kernels
        rocm.close()
        return
    mlp = bench_mlp(helpers, rocm, args.mlp_batch, args.mlp_iters, 3) if args.only in ("all", "mlp") else None
    sac = bench_sac(helpers, rocm, args.steps, args.warmup, per_operation=args.sac_per_operation, phase_profile=args.sac_phase_profile) if args.only in ("all", "sac") else {"steps_per_s": 0.0, "ms_per_step": 0.0}
    mlp_other = {str(b): bench_mlp(helpers, rocm, b, 100, 10) for b in (256, 4096)} if args.only in ("all", "mlp") and not args.no_mlp_by_batch else None      # configuration 1's other two batch sizes
    api = bench_sac_api(helpers, rocm, graph_replay=not args.no_graph_replay) if args.only in ("all", "sac", "api") else None
    env = bench_env(helpers, rocm) if args.only in ("all", "env") else None
    ppo = bench_ppo(helpers, rocm) if args.only in ("all", "ppo") else None
    gru = [bench_gru(helpers, rocm, b) for b in (64, 1024)] if args.only in ("all", "gru") else None
    seq = bench_sac_sequence(helpers, rocm) if args.only in ("all", "seq") else None
    cpu = None if (args.no_cpu_baseline or args.only in ("mlp", "env", "ppo", "gru", "seq", "api")) else cpu_baseline()
    line = {
        "metric": "SAC updates/sec (critic+actor) at batch 256; fused MLP fwd+bwd TFLOP/s",
        "value": sac["steps_per_s"], "unit": "SAC loop steps/s (each = 2 critic + 1 actor update)",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": sac["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "SAC Pendulum loop step, batch 256, actor 3-64-64-2, critics 4-64-64-1, replay 10000; plus MLP 17-256-256-6 fwd+bwd at batch %d" % args.mlp_batch,
                   "device": info["name"], "compute_units": info["compute_units"]},
        "timed": {"loop_steps": sac.get("timed_loop_steps"), "launches_of_steps_each": sac.get("timed_launches"), "clock": "HIP events on the library's stream"},
        "steps_per_s_one_launch_of_20000_steps": sac.get("steps_per_s_one_launch_of_20000_steps"),
        "network_updates_per_s": 3 * sac["steps_per_s"], "mean_return_of_100_evaluation_episodes_after_the_run": sac.get("evaluation_return_after_run"), "sac_path": "per-operation launches" if args.sac_per_operation else "persistent kernel, one launch for all steps",
    }
    if api:
        line["sac_api_path_steps_per_s"] = api["steps_per_s"]
        line["sac_api_path"] = api
    if mlp:
        line["mlp_fwd_bwd_tflops"] = mlp["tflops"]
        line["mlp"] = mlp
        flop = (MLP_FLOP_PER_SAMPLE_FWD + MLP_FLOP_PER_SAMPLE_BWD) * mlp["batch"]
        line["roofline"] = {"bound": "mfma", "achieved": mlp["tflops"], "peak": FP32_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": mlp["tflops"] / FP32_PEAK_TFLOPS,
                            "traffic": MLP_CALL_HBM_BYTES if mlp["batch"] == 65536 else None, "traffic_unit": "bytes per call, from rocprofv3 FETCH_SIZE / WRITE_SIZE",
                            "kernel": "mlp_forward_backward call = mlp3_prepare_kernel + mlp3_fused_kernel + mlp3_reduce_kernel", "flop_per_launch": flop}
    if mlp_other:
        line["mlp_by_batch"] = mlp_other
    # one roofline object per configuration (the dominant kernel of each; `roofline` above stays the benchmark's own): algorithmic bytes or flop over the measured
    # time against MI355X's published peaks; traffic = HBM bytes per launch from the counter runs summarised under profiles/ (null where none was made)
    def hbm(kernel, gbps, traffic, note):
        return {"kernel": kernel, "bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS, "traffic": traffic, "algorithmic": note}

    def mfma(kernel, tflops, traffic, note):
        return {"kernel": kernel, "bound": "mfma", "achieved": tflops, "peak": FP32_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": tflops / FP32_PEAK_TFLOPS, "traffic": traffic, "algorithmic": note}
    rooflines = {}
    if sac.get("steps_per_s"):
        rooflines["sac_loop_step_b256"] = mfma("sac_pendulum_loop_kernel", SAC_STEP_FLOP * sac["steps_per_s"] / 1e12, None, "%.1f MFLOP per loop step (2 critic + 1 actor update at batch 256, widths 64)" % (SAC_STEP_FLOP / 1e6))
    if mlp_other:
        for b, m in mlp_other.items():
            rooflines["mlp_forward_backward_b" + b] = mfma("mlp_forward_backward call", m["tflops"], None, "%d flop per sample" % (MLP_FLOP_PER_SAMPLE_FWD + MLP_FLOP_PER_SAMPLE_BWD))
    if env:
        # the step's 68 bytes per environment would take 0.56 us at the memory's rate, the 3-64-64-1 actor's 8,704 flop per environment 3.6 us at the matrix pipeline's:
        # the kernel's bound is the latter; both fractions are given
        rooflines["env_step_65536"] = mfma("runner_fused_kernel", env["policy_tflops"], 9.98e6, "8,704 flop per environment step (the actor 3-64-64-1 on every environment)")
        rooflines["env_step_65536_bytes"] = hbm("runner_fused_kernel", env["algorithmic_GBps"], 9.98e6, "68 B per environment step")
        rooflines["gather_batch_4096"] = hbm("gather_kernel", env["gather_algorithmic_GBps"], 1.72e6, "85 B per row")
        rooflines["acrobot_step_1048576"] = hbm("acrobot_step_kernel", env["acrobot"]["algorithmic_GBps"], 93.6e6, "89 B per environment step")
    if ppo:
        rooflines["ppo_gae_4096x128"] = hbm("gae_kernel", ppo["gae_algorithmic_GBps"], 91.9e6, "24 B per dataset row")
        rooflines["ppo_minibatch_update_8192"] = mfma("mlp3s_kernel + adam_pair_kernel", ppo["tflops"], PPO_UPDATE_HBM_BYTES, "106,368 flop per row and epoch (actor 105-64-64-8 and critic 105-64-64-1, forward + backward)")
    if gru:
        for g in gru:
            rooflines["gru_training_step_b%d" % g["batch"]] = mfma("gru_forward_mfma_kernel + gru_backward_mfma_kernel + projections", g["tflops"], None, "forward + backward through time, 64 steps, input 146, hidden 64")
    if rooflines:
        line["rooflines"] = rooflines
    if env:
        line["env_pipeline"] = env
    if ppo:
        line["ppo_iteration"] = ppo
    if gru:
        line["gru_training_step"] = gru
    if seq:
        line["sac_sequence_training_step"] = seq
    if cpu:
        line["cpu_baseline"] = cpu
        line["speedup_vs_cpu_baseline"] = sac["steps_per_s"] / cpu["value"] if cpu["value"] else None
        line["cpu_other_configurations"] = cpu_other_configurations(helpers, cpu.get("cblas_path"))
    if cpu:
        cpu.pop("cblas_path", None)
    print(json.dumps(line), flush=True)
    rocm.close()


if __name__ == "__main__":
    main()
