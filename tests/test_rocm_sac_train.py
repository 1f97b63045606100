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


make_loop, loop_parameters, np_from, loop_state, push_state = helpers.make_loop, helpers.loop_parameters, helpers.np_from, helpers.loop_state, helpers.push_state


def run_update(rocm, agent, A, lib, loop, batch, loss_ptr=None):
    oab = np_from(A.observations_actions_base, (2, batch, 4)); rew = np_from(A.rewards, (batch,)); term = np_from(A.terminated, (batch,), np.uint8)
    nc = np_from(lib.rlt_oracle_sac_loop_noise_critic(loop), (batch, 1)); na = np_from(lib.rlt_oracle_sac_loop_noise_actor(loop), (batch, 1))
    agent.set_batch(oab, rew, term)
    ncd, nad = rocm.array(nc), rocm.array(na)
    for k in range(2):
        rocm.call("sac_train_critic", C.byref(agent.c), k, ncd.ptr)
    if loss_ptr is not None:    # critic 1's loss on its training forward pass (train_actor re-runs the critics on other inputs)
        rocm.call("mse_evaluate", agent.critics[1].out[2].ptr, 1, agent.target_q.ptr, 1, batch, 1, 0.5, loss_ptr)
    rocm.call("sac_update_critic_targets", C.byref(agent.c))
    rocm.call("sac_train_actor", C.byref(agent.c), nad.ptr)
    return ncd, nad


def test_1000_updates_from_the_checkers_state(oracle, rocm):
    """1,000 seeded loop steps (3,000 network updates). Before each step the HIP side is given the checker's exact state, both run
    the step on the same batch and noise, and gradients, updated parameters and the critic loss are compared. A ReLU
    pre-activation or a min(Q1,Q2) that sits within rounding of its switch point can flip on one side; such a step moves one
    sample's contribution (1/256 of a gradient). The critic gradient is driven by the TD error Q - y, a small difference of large
    values: fp32 rounding of Q (1e-7 relative) is amplified by kappa = max|y| / max|Q - y| (about 100 late in training), for
    ANY fp32 implementation including the reference's own BLAS path. Stated tolerance: updated parameters agree to 1e-5 (relative
    to the largest parameter) on every step; gradients to 1e-5 * kappa on 99% of the steps and 1e-2 on every step; the critic
    loss (itself a mean of squared TD errors) to 1e-5 * kappa."""
    batch = 256
    loop, cfg = make_loop(oracle, batch)
    lib = oracle.lib
    for _ in range(cfg.n_warmup_steps):
        assert lib.rlt_oracle_sac_loop_step(loop) == 0
    agent = helpers.SacOnBackend(rocm, batch, 64, loop_parameters(oracle, loop))
    A = lib.rlt_oracle_sac_loop_agent(loop).contents
    loss_dev = rocm.zeros((1,))
    grad_err, param_err, loss_err, kappa = [], [], [], []
    for step in range(1000):
        push_state(agent, loop_state(oracle, loop, batch))
        assert lib.rlt_oracle_sac_loop_step(loop) == 0
        run_update(rocm, agent, A, lib, loop, batch, loss_dev.ptr)
        rocm.sync()
        st = loop_state(oracle, loop, batch)
        y = np_from(A.target_action_value, (batch,))
        kappa.append(max(1.0, np.abs(y).max() / max(np.abs(np_from(A.d_output_critic[1], (batch,))).max() * batch, 1e-30)))
        ge = max(rel_err(agent.actor.grads.numpy(), st["actor"]["grads"]), rel_err(agent.critics[0].grads.numpy(), st["critic0"]["grads"]),
                 rel_err(agent.critics[1].grads.numpy(), st["critic1"]["grads"]))
        pe = rel_err(agent.parameters(), loop_parameters(oracle, loop))
        le = abs(float(loss_dev.numpy()[0]) - lib.rlt_oracle_sac_loop_critic_loss(loop, 1)) / max(abs(lib.rlt_oracle_sac_loop_critic_loss(loop, 1)), 1e-30)
        grad_err.append(ge); param_err.append(pe); loss_err.append(le)
        if step % 100 == 0:
            print(f"step {step}: grad {ge:.2e} param {pe:.2e} loss {le:.2e}", flush=True)
    grad_err, param_err, loss_err, kappa = map(np.array, (grad_err, param_err, loss_err, kappa))
    print("kappa: median %.1f max %.1f" % (np.median(kappa), kappa.max()))
    print("gradient rel err: median %.2e p99 %.2e max %.2e" % (np.median(grad_err), np.percentile(grad_err, 99), grad_err.max()))
    print("parameter rel err: median %.2e p99 %.2e max %.2e" % (np.median(param_err), np.percentile(param_err, 99), param_err.max()))
    print("critic loss rel err: median %.2e max %.2e" % (np.median(loss_err), loss_err.max()))
    assert np.percentile(grad_err / kappa, 99) <= 1e-5 and grad_err.max() <= 1e-2
    assert param_err.max() <= 1e-5
    assert (loss_err / kappa).max() <= 1e-5
    lib.rlt_oracle_sac_loop_destroy(loop)


@pytest.mark.parametrize("batch", [256, 100])
def test_free_running_trajectory(oracle, rocm, batch):
    """Both sides train freely on the same batches and noise for 1,000 loop steps with no re-synchronisation. fp32 SAC training is
    chaotic (a single flipped ReLU/min is amplified), so the trajectories are required to coincide to 1e-5 while no flip has
    happened (first 100 steps) and afterwards to stay statistically the same: the critic loss averaged over 100-step windows
    agrees to 10%, and the two parameter vectors end no further apart than the distance travelled from the initial parameters.
    Yardstick: the reference's own two CPU backends (generic loops vs OpenBLAS, both compiled from the reference) started from
    the same seed are 0.02 apart after 100 such steps and 0.91 apart after 1,000 (distance travelled 0.94)."""
    loop, cfg = make_loop(oracle, batch)
    lib = oracle.lib
    for _ in range(cfg.n_warmup_steps):
        assert lib.rlt_oracle_sac_loop_step(loop) == 0
    p0 = loop_parameters(oracle, loop)
    agent = helpers.SacOnBackend(rocm, batch, 64, p0)
    A = lib.rlt_oracle_sac_loop_agent(loop).contents
    loss_dev = rocm.zeros((1000,))
    ref_loss = []
    early = 0.0
    for step in range(1000):
        assert lib.rlt_oracle_sac_loop_step(loop) == 0
        ref_loss.append(lib.rlt_oracle_sac_loop_critic_loss(loop, 1))
        run_update(rocm, agent, A, lib, loop, batch, loss_dev.offset(step))
        if step % 20 == 0 and step < 100:
            rocm.sync()
            early = max(early, rel_err(agent.parameters(), loop_parameters(oracle, loop)))
    rocm.sync()
    got_loss, ref_loss = loss_dev.numpy().astype(np.float64), np.array(ref_loss)
    ref_p, got_p = loop_parameters(oracle, loop), agent.parameters()
    travelled = np.abs(ref_p - p0).max()
    apart = np.abs(ref_p - got_p).max()
    win = lambda x: x.reshape(10, 100).mean(1)
    print("early parameter rel err %.2e; windowed loss ref %s got %s; apart %.3e travelled %.3e" % (early, win(ref_loss), win(got_loss), apart, travelled), flush=True)
    assert early <= 1e-5
    assert np.all(np.abs(win(got_loss) - win(ref_loss)) <= 0.10 * np.abs(win(ref_loss)))
    assert apart <= travelled
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
