"""The persistent SAC loop kernel (rlt_rocm_sac_pendulum_loop: N reference loop steps in one launch) against the CPU checker's
seeded loop. The checker's state after its warm-up is copied to the device, the checker then runs N steps while its random
draws (reset states, exploration noise, gather offsets, critic/actor noise) are recorded, and the kernel replays the same N
steps from those draws."""
import ctypes as C

import numpy as np
import pytest

import helpers
from helpers import capi, rel_err, np_from

pytestmark = pytest.mark.gpu


def run_fused(rocm, agent, runner, draws, n_steps, with_outputs=True):
    dev = {k: rocm.array(draws[k]) for k in ("rollout_noise", "initial_states", "sample_offsets", "noise_critic", "noise_actor")}
    inputs = capi.SacLoopInputs(dev["rollout_noise"].ptr, dev["initial_states"].ptr, dev["sample_offsets"].ptr, dev["noise_critic"].ptr, dev["noise_actor"].ptr)
    B = agent.batch
    loss = rocm.zeros((n_steps, 2)); oab = rocm.zeros((2, B, 4)); rew = rocm.zeros((B,)); term = rocm.zeros((B,), np.uint8); y = rocm.zeros((B,))
    outputs = capi.SacLoopOutputs(loss.ptr, oab.ptr, rew.ptr, term.ptr, y.ptr, None)
    lib, h = rocm.device.lib, rocm.device.handle
    rc = lib.rlt_rocm_sac_pendulum_loop(h, C.byref(agent.c), C.byref(runner.c), C.byref(runner.rb.c), n_steps, 0, 0, C.byref(inputs), C.byref(outputs) if with_outputs else None)
    assert rc == 0, lib.rlt_rocm_error_string(rc)
    rocm.sync()
    return dict(loss=loss.numpy(), oab=oab.numpy(), rewards=rew.numpy(), terminated=term.numpy(), target=y.numpy())


@pytest.mark.parametrize("batch,n_steps,placement", [(256, 1, None), (256, 100, None), (64, 250, None), (256, 100, "spread"), (640, 30, None)])
def test_fused_loop_replays_the_checkers_steps(oracle, rocm, batch, n_steps, placement, monkeypatch):
    """placement: up to 32 workgroups (batch 512) run on one XCD and exchange through its L2; "spread" forces the layout that larger
    batches (here 640 = 40 workgroups) take, spread over the XCDs with stores written through to memory."""
    print("case", batch, n_steps, placement, flush=True)
    if placement:
        monkeypatch.setenv("RLT_SAC_LOOP_PLACEMENT", placement)
    lib = oracle.lib
    loop, cfg = helpers.make_loop(oracle, batch)
    for _ in range(cfg.n_warmup_steps + 3):        # a few trained steps so that Adam moments and ages are non-trivial
        assert lib.rlt_oracle_sac_loop_step(loop) == 0
    agent = helpers.SacOnBackend(rocm, batch, 64, helpers.loop_parameters(oracle, loop), masks=False)
    helpers.push_state(agent, helpers.loop_state(oracle, loop, batch))
    runner = helpers.RunnerOnBackend(rocm, 10000, oracle, loop)
    draws = helpers.collect_loop_draws(oracle, loop, batch, n_steps)
    out = run_fused(rocm, agent, runner, draws, n_steps)
    A = lib.rlt_oracle_sac_loop_agent(loop).contents
    st = helpers.loop_state(oracle, loop, batch)
    # environment / replay side: the same transitions were generated and stored (fp32 dynamics: 1e-5), cursors exact
    rb = lib.rlt_oracle_sac_loop_replay(loop).contents
    rn = lib.rlt_oracle_sac_loop_runner(loop).contents
    pos = int(np_from(rb.position, (1,), np.uint32)[0])
    assert int(runner.rb.position.numpy()[0]) == pos and int(runner.ep_step.numpy()[0]) == int(np_from(rn.episode_step, (1,), np.uint32)[0])
    assert np.array_equal(runner.rb.episode_start.numpy()[:pos], np_from(rb.episode_start, (10000,), np.uint32)[:pos])
    tol_env = 1e-5 if n_steps <= 100 else 2e-3      # the policy drifts with the parameters over a long free run
    assert rel_err(runner.rb.data.numpy()[:pos], np_from(rb.data, (10000, 10))[:pos]) <= tol_env
    assert rel_err(runner.states.numpy(), np_from(rn.states, (1, 2))) <= tol_env
    # last batch: gathered rows are copies (exact when the rows themselves are exact, i.e. always for rows from before the run)
    ref_oab = np_from(A.observations_actions_base, (2, batch, 4))
    assert rel_err(out["oab"], ref_oab) <= tol_env and np.array_equal(out["terminated"], np_from(A.terminated, (batch,), np.uint8))
    # training side
    errs = {name: rel_err(getattr(agent, attr).params.numpy() if not isinstance(attr, tuple) else attr[0][attr[1]].params.numpy(), st[name]["params"])
            for name, attr in (("actor", "actor"), ("critic0", (agent.critics, 0)), ("critic1", (agent.critics, 1)), ("target0", (agent.targets, 0)), ("target1", (agent.targets, 1)))}
    print("parameter rel err", errs, "loss rel err first/last", abs(out["loss"][0] - draws["critic_loss"][0]) / draws["critic_loss"][0],
          abs(out["loss"][-1] - draws["critic_loss"][-1]) / draws["critic_loss"][-1], flush=True)
    if n_steps == 1:
        for name, e in errs.items():
            assert e <= 1e-5, (name, e)
        assert rel_err(out["target"], np_from(A.target_action_value, (batch,))) <= 1e-5
        assert rel_err(agent.critics[0].grads.numpy(), st["critic0"]["grads"]) <= 1e-4      # TD-error conditioning, see test_rocm_sac_train
        assert rel_err(agent.critics[1].grads.numpy(), st["critic1"]["grads"]) <= 1e-4
        assert rel_err(agent.actor.grads.numpy(), st["actor"]["grads"]) <= 1e-4
        assert rel_err(agent.log_alpha.numpy(), st["log_alpha"]) <= 1e-5
        for k in range(2):
            assert abs(out["loss"][0, k] - draws["critic_loss"][0, k]) <= 1e-4 * draws["critic_loss"][0, k]
    else:
        # free-running for n_steps with no re-synchronisation (see test_rocm_sac_train.py for the yardstick): identical while no
        # ReLU/min flips, statistically the same afterwards
        for name, e in errs.items():
            assert e <= (1e-4 if n_steps <= 100 else 5e-2), (name, e)
        w = min(50, n_steps)
        assert np.all(np.abs(out["loss"][-w:].mean(0) - draws["critic_loss"][-w:].mean(0)) <= 0.1 * draws["critic_loss"][-w:].mean(0))
    assert int(agent.actor.age.numpy()[0]) == int(st["actor"]["age"][0]) and int(agent.critics[1].age.numpy()[0]) == int(st["critic1"]["age"][0])
    lib.rlt_oracle_sac_loop_destroy(loop)


def test_fused_loop_device_rng_trains_and_rejects_unsupported_shapes(oracle, rocm):
    """Without host draws the kernel uses its own generator: parameters stay finite, the replay cursor advances by n_steps, and the
    critic loss decreases over 1,500 steps from a fresh agent. Shapes outside what the kernel is built for are refused."""
    batch = 256
    lib = oracle.lib
    loop, cfg = helpers.make_loop(oracle, batch)
    for _ in range(cfg.n_warmup_steps):
        assert lib.rlt_oracle_sac_loop_step(loop) == 0
    agent = helpers.SacOnBackend(rocm, batch, 64, helpers.loop_parameters(oracle, loop), masks=False)
    runner = helpers.RunnerOnBackend(rocm, 10000, oracle, loop)
    pos0 = int(runner.rb.position.numpy()[0])
    n = 1500
    loss = rocm.zeros((n, 2))
    outputs = capi.SacLoopOutputs(loss.ptr, None, None, None, None, None)
    rlib, h = rocm.device.lib, rocm.device.handle
    assert rlib.rlt_rocm_sac_pendulum_loop(h, C.byref(agent.c), C.byref(runner.c), C.byref(runner.rb.c), n, 7, 0, None, C.byref(outputs)) == 0
    rocm.sync()
    p = agent.parameters()
    assert np.all(np.isfinite(p)) and int(runner.rb.position.numpy()[0]) == pos0 + n
    l = loss.numpy()
    assert np.all(np.isfinite(l)) and l[-200:].mean() < 0.5 * l[:50].mean()
    data = runner.rb.data.numpy()[pos0:pos0 + n]
    assert np.all(np.abs(data[:, 3]) <= 1) and np.all(data[:, 4] <= 0) and np.allclose(data[:, 0] ** 2 + data[:, 1] ** 2, 1, atol=1e-5)
    assert data[:, 9].sum() >= n // 200 - 1          # episodes of 200 steps are truncated and restarted
    masked = helpers.SacOnBackend(rocm, batch, 64, helpers.loop_parameters(oracle, loop), masks=True)
    assert rlib.rlt_rocm_sac_pendulum_loop(h, C.byref(masked.c), C.byref(runner.c), C.byref(runner.rb.c), 1, 7, 0, None, None) == -2
    odd = helpers.SacOnBackend(rocm, 40, 64, helpers.loop_parameters(oracle, loop), masks=False)
    assert rlib.rlt_rocm_sac_pendulum_loop(h, C.byref(odd.c), C.byref(runner.c), C.byref(runner.rb.c), 1, 7, 0, None, None) == -2
    lib.rlt_oracle_sac_loop_destroy(loop)


def test_sac_learns_the_pendulum_to_the_reference_acceptance_bar(oracle, rocm):
    """The reference's own acceptance test for this loop (tests/src/rl/algorithms/sac/cpu/test.cpp:9-43): 10,000 loop steps from a fresh agent, the mean return
    of the evaluation episodes taken every 1,000 steps, and the 80th percentile of those ten means must exceed -200. Here: 100 warm-up steps on the checker,
    9,900 loop steps in the persistent kernel with the device's own generator, 10 evaluation episodes of 200 steps on the device from sampled initial states
    (an untrained actor scores below -1,000). For comparison, the CPU checker's loop (bit-identical to the reference) at this batch size gives the means
    -1783, -1110, -707, -226, -176, -196, -156, -131, -316, -441 (80th percentile -156): late dips below the bar belong to the algorithm at batch 256."""
    batch = 256
    lib = oracle.lib
    loop, cfg = helpers.make_loop(oracle, batch)
    for _ in range(cfg.n_warmup_steps):
        assert lib.rlt_oracle_sac_loop_step(loop) == 0
    agent = helpers.SacOnBackend(rocm, batch, 64, helpers.loop_parameters(oracle, loop), masks=False)
    runner = helpers.RunnerOnBackend(rocm, 10000, oracle, loop)
    rlib, h = rocm.device.lib, rocm.device.handle
    rng = np.random.default_rng(11)
    env = capi.pendulum_parameters()
    ret, length, summary = rocm.zeros((10,)), rocm.zeros((10,), np.uint32), rocm.zeros((6,))

    def evaluate():
        ini = rocm.array(np.stack([rng.uniform(-np.pi, np.pi, 10), rng.uniform(-1, 1, 10)], 1).astype(np.float32))
        rocm.call("pendulum_evaluate", C.byref(env), 2, agent.actor.layers, agent.actor.n, ini.ptr, 10, 200, ret.ptr, length.ptr, summary.ptr)
        rocm.sync()
        return float(summary.numpy()[0])
    untrained = evaluate()
    returns = []
    done = 0
    for chunk in [900] + [1000] * 9:
        assert rlib.rlt_rocm_sac_pendulum_loop(h, C.byref(agent.c), C.byref(runner.c), C.byref(runner.rb.c), chunk, 7, done, None, None) == 0
        rocm.sync()
        done += chunk
        returns.append(evaluate())
    print("mean evaluation returns", round(untrained), [round(r) for r in returns], flush=True)
    assert untrained < -600 and len(returns) == 10
    assert sorted(returns)[int(len(returns) * 0.8)] > -200, returns
    lib.rlt_oracle_sac_loop_destroy(loop)
