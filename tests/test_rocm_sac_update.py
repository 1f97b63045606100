"""The fused SAC updates (two launches per train_critic / train_actor, one for update_critic_targets) for actors obs -> 64 -> 64 -> 2 act and
critics obs + act -> 64 -> 64 -> 1 of any width: against the CPU checker's train_critic / train_actor / update_critic_targets
(rl/algorithms/sac/operations_generic.h:243-337, 395-468, 488-527) and against the library's own one-launch-per-operation path, from
identical parameters, batches and noise. Tolerance: 1e-5 relative to each tensor's largest magnitude (fp32, different summation orders)."""
import ctypes as C
import os

import numpy as np
import pytest

import helpers
from helpers import rel_err

pytestmark = pytest.mark.gpu

TOL = 1e-5


def agent_parameters(rng, obs, act, hidden=64):
    d = obs + act
    critics = [helpers.random_params(rng, [d, hidden, hidden, 1]) for _ in range(2)]
    targets = [c + rng.uniform(-0.01, 0.01, c.size).astype(np.float32) for c in critics]
    return np.concatenate([helpers.random_params(rng, [obs, hidden, hidden, 2 * act])] + critics + targets + [np.array([np.log(0.5)], np.float32)])


def batch_of(rng, batch, obs, act):
    oab = rng.standard_normal((2, batch, obs + act)).astype(np.float32)
    oab[:, :, obs:] = np.tanh(oab[:, :, obs:])
    return oab, rng.standard_normal(batch).astype(np.float32), (rng.random(batch) < 0.1).astype(np.uint8)


def snapshot(agent):
    return dict(parameters=agent.parameters(), actor_gradient=agent.actor.grads.numpy(), critic0_gradient=agent.critics[0].grads.numpy(),
                critic1_gradient=agent.critics[1].grads.numpy(), log_alpha_gradient=agent.log_alpha.numpy()[1:2],
                actor_first_moment=agent.actor.m.numpy(), critic1_second_moment=agent.critics[1].v.numpy(),
                target_action_value=agent.target_q.numpy(), next_log_probabilities=agent.next_lp.numpy(), actor_log_probabilities=agent.a_lp.numpy(),
                actor_actions=agent.a_act.numpy(), actor_pre_squashing=agent.a_pre.numpy(),
                next_state_action_value_input=agent.nsavi.numpy(),
                ages=np.array([agent.actor.age.numpy()[0], agent.critics[0].age.numpy()[0], agent.critics[1].age.numpy()[0], agent.alpha_age.numpy()[0]], np.float64))


def run_updates(agent, batches, noises):
    """`len(batches)` loop steps' worth of updates: critic 0, critic 1, actor, targets, each critic and the actor on its own batch and noise"""
    b = agent.backend
    for (oab, rew, term), (n0, n1, na) in zip(batches, noises):
        for k, noise in ((0, n0), (1, n1)):
            agent.set_batch(oab[k], rew[k], term[k])
            noise_on_backend = b.array(noise)
            b.call("sac_train_critic", C.byref(agent.c), k, noise_on_backend.ptr)
            b.sync()       # the batch buffers are rewritten for the next update
        agent.set_batch(oab[2], rew[2], term[2])
        noise_on_backend = b.array(na)
        b.call("sac_train_actor", C.byref(agent.c), noise_on_backend.ptr)
        b.call("sac_update_critic_targets", C.byref(agent.c))
        b.sync()
    return snapshot(agent)


def make_inputs(seed, batch, obs, act, steps, hidden=64):
    rng = np.random.default_rng(seed)
    params = agent_parameters(rng, obs, act, hidden)
    batches, noises = [], []
    for _ in range(steps):
        three = [batch_of(rng, batch, obs, act) for _ in range(3)]
        batches.append(([t[0] for t in three], [t[1] for t in three], [t[2] for t in three]))
        noises.append(tuple(rng.standard_normal((batch, act)).astype(np.float32) for _ in range(3)))
    return params, batches, noises


SHAPES = [  # batch, obs, act, hidden activation
    (256, 3, 1, "relu"),        # Pendulum
    (256, 27, 8, "relu"),       # Ant-sized: two input tiles, the widest head
    (100, 17, 6, "tanh"),       # batch that is no multiple of 64 or 16
    (64, 11, 3, "fast_tanh"),
    (1, 5, 2, "relu"),
    (300, 111, 8, "relu"),      # wide observations: the 128-input variant of the kernel
    (130, 120, 8, "sigmoid"),   # the input limit exactly
]


@pytest.mark.parametrize("batch,obs,act,hidden_act", SHAPES)
def test_fused_updates_match_the_checker_and_the_per_operation_path(oracle, rocm, batch, obs, act, hidden_act):
    steps = 3
    params, batches, noises = make_inputs(batch * 131 + obs, batch, obs, act, steps)
    results = {}
    for name, backend, per_operation in (("checker", oracle, None), ("fused", rocm, 0), ("per_operation", rocm, 1)):
        agent = helpers.SacOnBackend(backend, batch, 64, params, masks=False, obs=obs, act=act, hidden_act=hidden_act)
        if per_operation is not None:
            rocm.call("sac_set_per_operation", per_operation)
        try:
            results[name] = run_updates(agent, batches, noises)
        finally:
            if per_operation is not None:
                rocm.call("sac_set_per_operation", 0)
    # which path ran: only the per-operation launches fill the critics' next-input buffer
    assert not results["fused"].pop("next_state_action_value_input").any()
    assert results["per_operation"].pop("next_state_action_value_input").any() and results["checker"].pop("next_state_action_value_input").any()
    for other in ("checker", "per_operation"):
        for key, ref in results[other].items():
            err = rel_err(results["fused"][key], ref)
            assert err <= TOL, (other, key, err)
    # the update did something: three Adam steps moved every network
    moved = np.abs(results["fused"]["parameters"] - params)
    assert moved.max() > 1e-4 and results["fused"]["ages"].tolist() == [1 + steps] * 4


@pytest.mark.parametrize("batch,obs,act,hidden,hidden_act", [(256, 6, 1, 256, "fast_tanh"), (100, 17, 6, 128, "relu"), (48, 3, 1, 200, "relu"), (256, 27, 8, 256, "relu"),
                                                             (30, 111, 8, 72, "tanh"), (512, 5, 2, 16, "sigmoid")])
def test_wider_agents_match_the_checker_on_both_paths(oracle, rocm, batch, obs, act, hidden, hidden_act):
    """Hidden widths other than 64 (the zoo's AcrobotSwingup agent: 6-256-256-2 and 7-256-256-1 at batch 256; Ant-sized: 27 / 8): one launch per update on the
    kernel for widths up to 256 (every network pass of the update by sixteen wavefronts per 16 rows, the optimiser as its last step), and one launch per
    operation (the few-rows forward kernel, a wavefront per 16 x 16 tile in the backward contractions; also with one launch per layer, RLT_MLP_ROWS=0).
    Three loop steps' worth of updates against the CPU checker."""
    steps = 3
    params, batches, noises = make_inputs(batch * 7 + hidden, batch, obs, act, steps, hidden)
    results = {}
    for name, backend, per_operation, rows in (("checker", oracle, None, None), ("one_launch", rocm, 0, None), ("per_operation", rocm, 1, "1"), ("per_layer", rocm, 1, "0")):
        if rows is not None:
            os.environ["RLT_MLP_ROWS"] = rows
        if per_operation is not None:
            rocm.call("sac_set_per_operation", per_operation)
        try:
            agent = helpers.SacOnBackend(backend, batch, hidden, params, masks=False, obs=obs, act=act, hidden_act=hidden_act)
            results[name] = run_updates(agent, batches, noises)
        finally:
            os.environ.pop("RLT_MLP_ROWS", None)
            rocm.call("sac_set_per_operation", 0)
    # which path ran: only the per-operation launches fill the critics' next-input buffer
    assert not results["one_launch"].pop("next_state_action_value_input").any()
    assert results["per_operation"].pop("next_state_action_value_input").any() and results["per_layer"].pop("next_state_action_value_input").any()
    results["checker"].pop("next_state_action_value_input")
    for other in ("checker", "per_operation", "per_layer"):
        for key, ref in results[other].items():
            err = rel_err(results["one_launch"][key], ref)
            # log(1 - a^2 + 1e-6) moves by 1e-4 per ulp of tanh for actions within 1e-3 of +-1: the log-probabilities get that much
            assert err <= (1e-4 if "log_probabilities" in key else TOL), (other, key, err)
    moved = np.abs(results["one_launch"]["parameters"] - params)
    assert moved.max() > 1e-4 and results["one_launch"]["ages"].tolist() == [1 + steps] * 4


def test_agents_outside_the_fused_shapes_take_the_per_operation_path(oracle, rocm):
    """an agent with sequence masks: same entry points, same results as the checker"""
    batch, obs, act = 64, 3, 1
    out = []
    for backend in (oracle, rocm):
        loop, cfg = helpers.make_loop(oracle, batch)
        params = helpers.loop_parameters(oracle, loop)
        oracle.lib.rlt_oracle_sac_loop_destroy(loop)
        agent = helpers.SacOnBackend(backend, batch, 64, params, masks=True)
        oab, rew, term = batch_of(np.random.default_rng(1), batch, obs, act)
        noise = np.random.default_rng(2).standard_normal((batch, act)).astype(np.float32)
        agent.set_batch(oab, rew, term)
        noise_on_backend = backend.array(noise)
        backend.call("sac_train_critic", C.byref(agent.c), 0, noise_on_backend.ptr)
        backend.call("sac_train_actor", C.byref(agent.c), noise_on_backend.ptr)
        backend.call("sac_update_critic_targets", C.byref(agent.c))
        backend.sync()
        out.append((agent.parameters(), agent.nsavi.numpy(), agent.d_ci[0].numpy()))      # the per-operation path fills every training buffer
    for got, ref in zip(out[1], out[0]):
        assert rel_err(got, ref) <= TOL
    assert np.abs(out[1][1]).max() > 0


def test_loop_by_calls_equals_the_same_calls_issued_one_by_one(rocm):
    """rlt_rocm_sac_pendulum_loop_by_calls is a host loop over public entry points with documented Philox sequences per step: issuing those
    calls from here with the same sequence numbers leaves bit-identical parameters, replay rows and runner state."""
    capi = helpers.capi
    batch, capacity, steps, seed, first = 64, 500, 40, 11, 1000
    rng = np.random.default_rng(0)
    params = agent_parameters(rng, 3, 1)
    final = []
    for by_calls in (True, False):
        agent = helpers.SacOnBackend(rocm, batch, 64, params, masks=False)
        rb = helpers.ReplayOnBackend(rocm, 1, capacity)
        states, ep_step, ep_ret, trunc = rocm.zeros((1, 2)), rocm.zeros((1,), np.uint32), rocm.zeros((1,)), rocm.array(np.ones(1, np.uint8))
        runner = capi.PendulumRunner(states.ptr, ep_step.ptr, ep_ret.ptr, trunc.ptr, 1, 200, capi.pendulum_parameters())
        rollout_noise, warm_action = rocm.zeros((1, 1)), rocm.zeros((1, 1))
        noise_c, noise_a = rocm.zeros((batch, 1)), rocm.zeros((batch, 1))
        env_idx, offs = rocm.zeros((batch,), np.uint32), rocm.zeros((batch,), np.uint32)
        for c in range(batch + 10):      # uniform warm-up policy
            rocm.call("rand_f32", warm_action.ptr, 1, -1.0, 1.0, seed, 8 * c + 1)
            rocm.call("pendulum_runner_step", C.byref(runner), C.byref(rb.c), 0, agent.actor.layers, 3, C.byref(agent.c.sas), warm_action.ptr, None, None, seed, 8 * c + 2)
        if by_calls:
            scratch = capi.SacLoopScratch(rollout_noise.ptr, noise_c.ptr, noise_a.ptr, env_idx.ptr, offs.ptr)
            rocm.call("sac_pendulum_loop_by_calls", C.byref(agent.c), C.byref(runner), C.byref(rb.c), steps, seed, first, C.byref(scratch))
        else:
            for i in range(steps):
                g = 8 * (first + i)
                rocm.call("randn_f32", rollout_noise.ptr, 1, seed, g + 1)
                rocm.call("pendulum_runner_step", C.byref(runner), C.byref(rb.c), 2, agent.actor.layers, 3, C.byref(agent.c.sas), None, rollout_noise.ptr, None, seed, g + 2)
                rocm.call("gather_draw", C.byref(rb.c), batch, seed, g + 3, env_idx.ptr, offs.ptr)
                rocm.call("gather_batch", C.byref(rb.c), env_idx.ptr, offs.ptr, 0, 200, batch, agent.oab.ptr, agent.rewards.ptr, agent.terminated.ptr, None, None, None, None)
                rocm.call("randn_f32", noise_c.ptr, batch, seed, g + 4)
                for k in range(2):
                    rocm.call("sac_train_critic", C.byref(agent.c), k, noise_c.ptr)
                rocm.call("sac_update_critic_targets", C.byref(agent.c))
                rocm.call("randn_f32", noise_a.ptr, batch, seed, g + 5)
                rocm.call("sac_train_actor", C.byref(agent.c), noise_a.ptr)
        rocm.sync()
        final.append((agent.parameters(), rb.data.numpy(), states.numpy(), ep_ret.numpy()))
    for a, b in zip(*final):
        assert np.array_equal(a, b)
    assert np.abs(final[0][0] - params).max() > 1e-3 and np.all(np.isfinite(final[0][0]))


@pytest.mark.parametrize("batch,obs,act,hidden_act", [(256, 3, 1, "relu"), (100, 17, 6, "tanh"), (300, 111, 8, "relu"), (1, 5, 2, "relu")])
def test_optimiser_in_the_kernel_and_placement_leave_the_same_bits(rocm, batch, obs, act, hidden_act):
    """The update kernel's own last step (its last workgroup adds up the partial gradients and applies Adam) against the optimiser as a launch
    of its own, and the workgroups on one XCD against spread over all: the same sums in the same order, so every tensor is bit-identical."""
    params, batches, noises = make_inputs(batch * 17 + act, batch, obs, act, 3)
    results = []
    try:
        for tail, one_xcd in ((1, 1), (1, 0), (0, 1), (0, 0)):
            rocm.call("set_update_options", tail, one_xcd)
            agent = helpers.SacOnBackend(rocm, batch, 64, params, masks=False, obs=obs, act=act, hidden_act=hidden_act)
            results.append(run_updates(agent, batches, noises))
    finally:
        rocm.call("set_update_options", 1, 1)
    for other in results[1:]:
        for key, ref in results[0].items():
            assert np.array_equal(other[key], ref), key
    assert results[0]["ages"].tolist() == [4] * 4


@pytest.mark.parametrize("batch,obs,act,hidden", [(256, 3, 1, 64), (64, 11, 3, 64), (300, 27, 8, 64), (256, 6, 1, 256), (96, 17, 6, 200)])
def test_both_critics_in_one_launch_equal_the_separate_calls(oracle, rocm, batch, obs, act, hidden):
    """rlt_rocm_sac_train_critics (both critics on the shared batch and the soft update of the targets in one launch; the noise an array or
    drawn by the kernel from its Philox stream) against train_critic(0), train_critic(1), update_critic_targets: bit for bit, and against the
    CPU checker's three calls to 1e-5; then train_actor with its noise drawn by the kernel against randn + train_actor."""
    rng = np.random.default_rng(batch + obs)
    params = agent_parameters(rng, obs, act, hidden)
    oab, rew, term = batch_of(rng, batch, obs, act)
    seed, stream = 77, 123
    noise_dev = rocm.zeros((batch, act))
    rocm.call("randn_f32", noise_dev.ptr, batch * act, seed, stream)
    rocm.sync()
    noise = noise_dev.numpy()
    runs = {}
    for name, backend in (("checker", oracle), ("separate", rocm), ("together", rocm), ("together_drawn", rocm)):
        agent = helpers.SacOnBackend(backend, batch, hidden, params, masks=False, obs=obs, act=act)
        agent.set_batch(oab, rew, term)
        n = backend.array(noise)
        drawn = backend.zeros((batch, act))
        for step in range(2):
            if name in ("checker", "separate"):
                for k in range(2):
                    backend.call("sac_train_critic", C.byref(agent.c), k, n.ptr)
                backend.call("sac_update_critic_targets", C.byref(agent.c))
                backend.call("sac_train_actor", C.byref(agent.c), n.ptr)
            elif name == "together":
                backend.call("sac_train_critics", C.byref(agent.c), n.ptr, 1)
                backend.call("sac_train_actor", C.byref(agent.c), n.ptr)
            else:
                backend.call("sac_train_critics_drawn", C.byref(agent.c), drawn.ptr, seed, stream, 1)
                backend.call("sac_train_actor_drawn", C.byref(agent.c), drawn.ptr, seed, stream)
        backend.sync()
        runs[name] = snapshot(agent)
        if name == "together_drawn":
            assert np.array_equal(drawn.numpy(), noise)
    for name in ("together", "together_drawn"):
        for key, ref in runs["separate"].items():
            assert np.array_equal(runs[name][key], ref), (name, key)
    runs["checker"].pop("next_state_action_value_input"); runs["separate"].pop("next_state_action_value_input")
    for key, ref in runs["checker"].items():
        assert rel_err(runs["separate"][key], ref) <= TOL, key
    assert runs["together"]["ages"].tolist() == [3] * 4
