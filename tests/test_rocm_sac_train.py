"""SAC train_critic / train_actor / update_critic_targets on the HIP path, in lock step with the CPU checker's seeded
reference loop: the checker draws the batch indices and the noise (as the reference's RNG would), both sides consume
the same batch and noise, and parameters are compared as training proceeds
(pattern: tests/src/rl/algorithms/sac/cuda/sac.cu:77-299, tests/src/rl/cuda/rl.cu:230-376)."""
import ctypes as C

import numpy as np
import pytest

import helpers
from helpers import capi, rel_err

pytestmark = pytest.mark.gpu


def make_loop(oracle, batch, seed=0):
    cfg = helpers.LoopConfig(seed, batch, 64, 10000, max(batch, 100), 200, 1e-7)
    return C.c_void_p(oracle.lib.rlt_oracle_sac_loop_create(C.byref(cfg))), cfg


def loop_parameters(oracle, loop):
    n = oracle.lib.rlt_oracle_sac_loop_parameter_count(loop)
    out = np.zeros(n, np.float32)
    oracle.lib.rlt_oracle_sac_loop_get_parameters(loop, out.ctypes.data)
    return out


def np_from(ptr, shape, dtype=np.float32):
    n = int(np.prod(shape))
    return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(np.ctypeslib.as_ctypes_type(dtype))), (n,)).reshape(shape).copy()


@pytest.mark.parametrize("batch", [256, 100])
def test_train_steps_in_lock_step_with_seeded_loop(oracle, rocm, batch):
    loop, cfg = make_loop(oracle, batch)
    lib = oracle.lib
    for _ in range(cfg.n_warmup_steps):
        assert lib.rlt_oracle_sac_loop_step(loop) == 0
    agent = helpers.SacOnBackend(rocm, batch, 64, loop_parameters(oracle, loop))
    A = lib.rlt_oracle_sac_loop_agent(loop).contents
    worst = 0.0
    n_updates = 300
    for step in range(n_updates):
        assert lib.rlt_oracle_sac_loop_step(loop) == 0
        # the checker's batch and noise of this step
        oab = np_from(A.observations_actions_base, (2, batch, 4)); rew = np_from(A.rewards, (batch,)); term = np_from(A.terminated, (batch,), np.uint8)
        nc = np_from(lib.rlt_oracle_sac_loop_noise_critic(loop), (batch, 1)); na = np_from(lib.rlt_oracle_sac_loop_noise_actor(loop), (batch, 1))
        agent.set_batch(oab, rew, term)
        ncd, nad = rocm.array(nc), rocm.array(na)
        for k in range(2):
            rocm.call("sac_train_critic", C.byref(agent.c), k, ncd.ptr)
        rocm.call("sac_update_critic_targets", C.byref(agent.c))
        rocm.call("sac_train_actor", C.byref(agent.c), nad.ptr)
        if step % 25 == 0 or step == n_updates - 1:
            rocm.sync()
            ref, got = loop_parameters(oracle, loop), agent.parameters()
            err = rel_err(got, ref)
            worst = max(worst, err)
            print(f"step {step}: parameter rel err {err:.3e}", flush=True)
            # intermediate buffers of this step (same inputs on both sides up to the drift so far)
            assert rel_err(agent.target_q.numpy(), np_from(A.target_action_value, (batch,))) <= 5e-4
    # trajectories drift apart through ReLU/min(Q1,Q2) switches; after 300 lock-step updates (900 network updates) on identical
    # batches and noise the parameter vectors must still agree to 1e-3 of the largest weight
    assert worst <= 1e-3, worst
    lib.rlt_oracle_sac_loop_destroy(loop)


def test_single_update_from_identical_state(oracle, rocm):
    """One critic + target + actor update from bit-identical parameters: 1e-5 relative on every parameter tensor and on the
    intermediate buffers (target values, critic input gradients, actor head gradient)."""
    batch = 256
    loop, cfg = make_loop(oracle, batch, seed=3)
    lib = oracle.lib
    for _ in range(cfg.n_warmup_steps + 20):
        lib.rlt_oracle_sac_loop_step(loop)
    params = loop_parameters(oracle, loop)
    A = lib.rlt_oracle_sac_loop_agent(loop).contents
    agents = [helpers.SacOnBackend(b, batch, 64, params) for b in (oracle, rocm)]
    # Adam moments and ages of the running loop are not copied: both sides start the optimiser state afresh
    oab = np_from(A.observations_actions_base, (2, batch, 4)); rew = np_from(A.rewards, (batch,)); term = np_from(A.terminated, (batch,), np.uint8)
    rng = np.random.default_rng(0)
    nc, na = rng.standard_normal((batch, 1)).astype(np.float32), rng.standard_normal((batch, 1)).astype(np.float32)
    out = []
    for ag in agents:
        b = ag.backend
        ag.set_batch(oab, rew, term)
        ncd, nad = b.array(nc), b.array(na)
        for k in range(2):
            b.call("sac_train_critic", C.byref(ag.c), k, ncd.ptr)
        b.call("sac_update_critic_targets", C.byref(ag.c))
        b.call("sac_train_actor", C.byref(ag.c), nad.ptr)
        b.sync()
        out.append(dict(params=ag.parameters(), target=ag.target_q.numpy(), nsavi=ag.nsavi.numpy(), dci0=ag.d_ci[0].numpy(), dci1=ag.d_ci[1].numpy(),
                        daos=ag.d_aos.numpy(), dao=ag.d_ao.numpy(), critic_grads=ag.critics[1].grads.numpy(), actor_grads=ag.actor.grads.numpy(),
                        log_alpha=ag.log_alpha.numpy(), savi=ag.savi.numpy()))
    for key in out[0]:
        assert rel_err(out[1][key], out[0][key]) <= 1e-5, (key, rel_err(out[1][key], out[0][key]))
    lib.rlt_oracle_sac_loop_destroy(loop)
