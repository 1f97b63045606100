"""The CPU checker against golden vectors written by the real reference (tests/golden/make_sac_golden.py): the seeded
SAC-on-Pendulum loop must reproduce the reference's parameters, replay rows, gathered batches, masks and noise BIT-EXACTLY.
Runs without /root/reference (the fixture is data)."""
import ctypes as C
import os

import numpy as np
import pytest

import helpers

GOLD = np.load(os.path.join(helpers.GOLDEN, "sac_pendulum_seed0.npz"))


def np_from(ptr, shape, dtype=np.float32):
    n = int(np.prod(shape))
    return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(np.ctypeslib.as_ctypes_type(dtype))), (n,)).reshape(shape).copy()


@pytest.mark.parametrize("batch,checkpoints", [(100, [0, 100, 101, 150, 300]), (256, [256, 257, 300, 500])])
def test_seeded_loop_reproduces_reference_vectors(oracle, batch, checkpoints):
    lib = oracle.lib
    cfg = helpers.LoopConfig(0, batch, 64, 10000, max(batch, 100), 200, 1e-7)
    loop = C.c_void_p(lib.rlt_oracle_sac_loop_create(C.byref(cfg)))
    n = lib.rlt_oracle_sac_loop_parameter_count(loop)
    p = np.zeros(n, np.float32)
    A = lib.rlt_oracle_sac_loop_agent(loop).contents
    rb = lib.rlt_oracle_sac_loop_replay(loop).contents
    done = 0
    for cp in checkpoints:
        while done < cp:
            assert lib.rlt_oracle_sac_loop_step(loop) == 0
            done += 1
        key = f"b{batch}_s{cp}"
        lib.rlt_oracle_sac_loop_get_parameters(loop, p.ctypes.data)
        assert np.array_equal(p[::16], GOLD[key + "_params16"]), key
        assert p.astype(np.float64).sum() == GOLD[key + "_sum"][0] and (p.astype(np.float64) ** 2).sum() == GOLD[key + "_sum"][1]
        pos, full = int(np_from(rb.position, (1,), np.uint32)[0]), int(np_from(rb.full, (1,), np.uint8)[0])
        assert [pos, full] == list(GOLD[key + "_replay_pos"])
        data = np_from(rb.data, (10000, 10))
        assert np.array_equal(data[max(0, pos - 8):pos], GOLD[key + "_replay_tail"])
        if cp > max(batch, 100):
            assert np.array_equal(np_from(A.observations_actions_base, (2, batch, 4)), GOLD[key + "_oab"])
            assert np.array_equal(np_from(A.rewards, (batch,)), GOLD[key + "_rewards"])
            assert np.array_equal(np_from(A.terminated, (batch,), np.uint8), GOLD[key + "_terminated"])
            assert np.array_equal(np_from(lib.rlt_oracle_sac_loop_noise_critic(loop), (batch,)), GOLD[key + "_noise_critic"])
            assert np.array_equal(np_from(lib.rlt_oracle_sac_loop_noise_actor(loop), (batch,)), GOLD[key + "_noise_actor"])
            # masks: final_step_mask / reset are the agent's views; next_final_step_mask is padded step 1 of its base tensor
            assert np.array_equal(np_from(A.final_step_mask, (batch,), np.uint8), GOLD[key + "_final_step_mask"])
            assert np.array_equal(np_from(A.reset, (batch,), np.uint8), GOLD[key + "_reset"])
            assert np.array_equal(np_from(A.next_final_step_mask, (batch,), np.uint8), GOLD[key + "_next_final_step_mask_base"][batch:])
            assert np.all(GOLD[key + "_next_final_step_mask_base"][:batch] == 0) and np.all(GOLD[key + "_next_reset_base"] == 1)
    lib.rlt_oracle_sac_loop_destroy(loop)


def ppo_golden_setup(backend):
    """Agent, parameters and per-loop-step records from tests/golden/ppo_pendulum_seed0.npz (written by the real reference)."""
    capi = helpers.capi
    g = np.load(os.path.join(helpers.GOLDEN, "ppo_pendulum_seed0.npz"))
    n_envs, steps, data_dim, rows, obs_dim, action_dim, batch, epochs, actor_hidden, critic_hidden = [int(x) for x in g["dims"]]
    hy = dict(zip([str(k) for k in g["hyper_names"]], [float(v) for v in g["hyper"]]))
    col = dict(zip(helpers.PPO_COLUMNS, [int(c) for c in g["columns"]]))
    adam = capi.adam_parameters(hy["alpha"], hy["beta_1"], hy["beta_2"], hy["epsilon"], hy["epsilon_sqrt"])
    pp = capi.ppo_parameters(hy["epsilon_clip"], hy["action_entropy_coefficient"], hy["advantage_epsilon"], int(hy["normalize_advantage"]), int(hy["learn_action_std"]))
    agent = helpers.PpoOnBackend(backend, obs_dim, action_dim, actor_hidden, critic_hidden, batch, g["s0_before"], "tanh", "relu", adam)
    return g, agent, pp, hy, col, dict(n_envs=n_envs, steps=steps, data_dim=data_dim, rows=rows, batch=batch, n=n_envs * steps)


def test_ppo_gae_and_update_reproduce_reference_vectors(oracle):
    """GAE and two loop steps' worth of PPO updates (30 minibatch updates) against what the reference itself produced: bit-exact."""
    g, agent, pp, hy, col, d = ppo_golden_setup(oracle)
    for step in range(2):
        data = g[f"s{step}_dataset"]
        dd = oracle.array(data)
        adv, tgt = oracle.zeros(data.shape), oracle.zeros(data.shape)
        oracle.call("ppo_gae", dd.offset(col["rewards"]), dd.offset(col["terminated"]), dd.offset(col["truncated"]), dd.offset(col["all_values"]), adv.ptr, tgt.ptr,
                    d["data_dim"], d["n_envs"], d["steps"], hy["gamma"], hy["lambda"], 0)
        assert np.array_equal(adv.numpy()[:d["n"], 0], data[:d["n"], col["advantages"]]) and np.array_equal(tgt.numpy()[:d["n"], 0], data[:d["n"], col["target_values"]])
        assert np.array_equal(agent.parameters(), g[f"s{step}_before"])
        helpers.ppo_train_like_reference(oracle, agent, pp, dd, d["data_dim"], col, d["n"], g[f"s{step}_permutations"], d["batch"])
        assert np.array_equal(agent.parameters(), g[f"s{step}_after"]), step


def gru_golden_case(case):
    g = np.load(os.path.join(helpers.GOLDEN, "gru_seed.npz"))
    S, B, I, H = [int(v) for v in g["dims"]]
    params = {k: g[f"{case}_param_{k}"] for k in ("W_i", "b_i", "W_h", "b_h", "h0")}
    reset = g[f"{case}_reset"] if f"{case}_reset" in g else None
    want = {k: g[f"{case}_want_{k}"] for k in ("output", "post", "npp", "dx", "dy", "dW_i", "db_i", "dW_h", "db_h")}
    return (S, B, I, H), params, g[f"{case}_x"], g[f"{case}_d_output"], reset, want


@pytest.mark.parametrize("case", ["plain", "reset"])
def test_gru_reproduces_reference_vectors(oracle, case):
    """Forward and backward through time of the restated GRU against what the reference's own layer produced: bit-exact."""
    (S, B, I, H), params, x, dy, reset, want = gru_golden_case(case)
    g = helpers.GruOnBackend(oracle, S, B, I, H, params)
    g.forward(x, reset)
    g.backward(dy)
    got = g.results()
    for k in want:
        assert np.array_equal(got[k], want[k]), k


def test_td3_reproduces_reference_vectors(oracle):
    """36 loop steps of the reference's TD3-on-Pendulum run (both critic updates every step; critic targets, the delayed actor update and
    the actor target every second step), from the reference's parameters, batches and noise draws: bit-exact digests of all six
    networks after every step, all parameters after steps 1 and 35, the Adam ages at the end; the smoothing noise from its N(0,1) draws."""
    (batch, hidden, steps), hyper, g = helpers.td3_golden()
    agent = helpers.Td3OnBackend(oracle, batch, hidden, g["parameters_before"], hyper=hyper)
    blocked = 0
    for i in range(steps):
        z, out = oracle.array(g[f"s{i}_target_noise_z"]), oracle.zeros((batch, 1))
        oracle.call("td3_target_action_noise", z.ptr, float(g["hyperparameters"][3]), float(g["hyperparameters"][4]), out.ptr, batch)
        assert np.array_equal(out.numpy(), g[f"s{i}_target_noise"])
        helpers.td3_golden_step(agent, g, i)
        assert np.array_equal(helpers.td3_digest(agent.parameters(), hidden), g[f"s{i}_digest"]), i
        if f"s{i}_after" in g:
            assert np.array_equal(agent.parameters(), g[f"s{i}_after"]), i
        if g[f"s{i}_flags"][2]:
            blocked += int((np.abs(agent.pre_clip.numpy()) > 1).sum())
    assert np.array_equal(agent.ages(), g["ages_after"])
    assert blocked >= 1           # the sampling layer's backward pass blocked at least one gradient on the way


def test_td3_operations_closed_forms(oracle):
    """Each elementwise TD3 operation against its definition written independently in numpy (float32 arithmetic)."""
    rng = np.random.default_rng(3)
    B, A = 37, 3
    f32 = np.float32
    mean = rng.uniform(-1.2, 1.2, (B, A)).astype(f32); noise = rng.standard_normal((B, A)).astype(f32); std = f32(0.3)
    m, n, pc, out = oracle.array(mean), oracle.array(noise), oracle.zeros((B, A)), oracle.zeros((B, A))
    oracle.call("td3_sampling_forward", m.ptr, A, n.ptr, A, float(std), pc.ptr, A, out.ptr, A, B, A)
    sample = mean + noise * std
    assert np.array_equal(pc.numpy(), sample) and np.array_equal(out.numpy(), np.clip(sample, -1, 1))
    assert (np.abs(sample) > 1).sum() > 5
    oracle.call("td3_sampling_forward", m.ptr, A, None, 0, float(std), None, 0, out.ptr, A, B, A)     # evaluation mode: no noise
    assert np.array_equal(out.numpy(), np.clip(mean, -1, 1))
    # backward: derivative of clip(x, -1, 1), by central differences of the forward pass on samples away from the kinks
    dy = rng.standard_normal((B, A)).astype(f32)
    d, dx = oracle.array(dy), oracle.zeros((B, A))
    oracle.call("td3_sampling_backward", pc.ptr, A, d.ptr, A, dx.ptr, A, B, A)
    h = 1e-3
    numeric = (np.clip(sample.astype(np.float64) + h, -1, 1) - np.clip(sample.astype(np.float64) - h, -1, 1)) / (2 * h) * dy
    away = np.abs(np.abs(sample) - 1) > 2 * h
    assert np.allclose(dx.numpy()[away], numeric[away], atol=1e-6) and away.sum() > B * A - 6
    # noisy next actions, target values
    a = rng.uniform(-1, 1, (B, A)).astype(f32); tn = np.clip(rng.standard_normal((B, A)) * 0.2, -0.5, 0.5).astype(f32)
    aa, tt = oracle.array(a), oracle.array(tn)
    oracle.call("td3_noisy_next_actions", aa.ptr, A, tt.ptr, A, B, A)
    assert np.array_equal(aa.numpy(), np.clip(a + tn, -1, 1))
    q1, q2, r = (rng.standard_normal(B).astype(f32) for _ in range(3)); term = (rng.random(B) < 0.4).astype(np.uint8)
    gamma = f32(0.97)
    for ignore in (0, 1):
        a1, a2, ar, at, y = oracle.array(q1), oracle.array(q2), oracle.array(r), oracle.array(term), oracle.zeros((B,))
        oracle.call("td3_target_action_values", a1.ptr, a2.ptr, ar.ptr, at.ptr, float(gamma), ignore, y.ptr, B)
        keep = np.ones(B, bool) if ignore else term == 0
        assert np.array_equal(y.numpy(), r + np.where(keep, gamma * np.minimum(q1, q2), f32(0)))


def test_td3_masks_equal_training_on_the_unmasked_rows(oracle):
    """With a final-step mask, the critic and actor updates must equal (to rounding) the same updates on a batch that holds only the
    unmasked rows: the loss weight batch/n turns the mean over the batch into the mean over the n final steps."""
    (batch, hidden, _), hyper, g = helpers.td3_golden()
    rng = np.random.default_rng(5)
    keep = rng.random(batch) < 0.6; keep[:2] = [True, False]
    idx = np.nonzero(keep)[0]; n = idx.size
    noises = [rng.standard_normal((batch, 1)).astype(np.float32) for _ in range(3)]
    full = helpers.Td3OnBackend(oracle, batch, hidden, g["parameters_before"], hyper=hyper, masks=True)
    full.m_final.upload(keep.astype(np.uint8))
    full.set_batch(g["s0_oab"], g["s0_rewards"], g["s0_terminated"], g["s0_target_noise"])
    full.loop_step([1, 1, 1, 1], *noises)
    sub = helpers.Td3OnBackend(oracle, n, hidden, g["parameters_before"], hyper=hyper)
    sub.set_batch(g["s0_oab"][:, idx], g["s0_rewards"][idx], g["s0_terminated"][idx], g["s0_target_noise"][idx])
    sub.loop_step([1, 1, 1, 1], *[z[idx] for z in noises])
    assert helpers.rel_err(full.parameters(), sub.parameters()) < 2e-6
    # a clear next-step mask keeps the stored next action in the target critics' input
    full.m_next_final.upload(np.zeros(batch, np.uint8))
    noise = oracle.array(noises[0])
    oracle.call("td3_train_critic", C.byref(full.c), 0, noise.ptr)
    assert np.array_equal(full.nsavi.numpy(), g["s0_oab"][1])


def test_on_policy_collect_and_normalisers_reproduce_reference_vectors(oracle):
    """Three collect() calls of the reference's PPO loop with observation normalisation (the warm-up one, one after the runner was
    re-initialised, one that continues running episodes): the restated collection, from the reference's runner state, actor, standardize
    statistics and draws, reproduces every column and the runner state afterwards bit for bit; the running normalisers and the standardize
    statistics after each update likewise."""
    dims, col, g = helpers.on_policy_golden()
    n, S, ld, hidden, limit = dims
    rows = n * S
    mean, std, age = oracle.zeros((3,)), oracle.array(np.ones(3, np.float32)), oracle.array(np.zeros(1, np.uint32))
    mean_p, std_p, age_p = oracle.zeros((3,)), oracle.array(np.ones(3, np.float32)), oracle.array(np.zeros(1, np.uint32))
    lm, lp = oracle.zeros((3,)), oracle.zeros((3,))
    for k in range(3):
        o = helpers.on_policy_golden_collect(oracle, g, k, dims, col)
        got, want = o.data.numpy()[:, :col["all_values"]], g[f"c{k}_dataset"]
        assert np.array_equal(got, want), k
        for name, v in o.runner_state().items():
            assert np.array_equal(v, g[f"c{k}_after_{name}"]), (k, name)
        if k > 0:
            assert g[f"c{k}_standardize_precision"].max() > 1.2        # the statistics in use are not the trivial ones
        dd = oracle.array(np.concatenate([want, np.zeros((want.shape[0], ld - want.shape[1]), np.float32)], 1))
        oracle.call("running_normalizer_update", dd.offset(col["observations"]), ld, rows, 3, mean.ptr, std.ptr, age.ptr)
        oracle.call("running_normalizer_update", dd.offset(col["observations"]), ld, rows + n, 3, mean_p.ptr, std_p.ptr, age_p.ptr)
        assert np.array_equal(mean.numpy(), g[f"u{k}_mean"]) and np.array_equal(std.numpy(), g[f"u{k}_std"])
        assert np.array_equal(mean_p.numpy(), g[f"u{k}_mean_privileged"]) and np.array_equal(std_p.numpy(), g[f"u{k}_std_privileged"])
        assert [int(age.numpy()[0]), int(age_p.numpy()[0])] == list(g[f"u{k}_ages"])
        oracle.call("standardize_set_statistics", mean.ptr, std.ptr, lm.ptr, lp.ptr, 3)
        assert np.array_equal(lm.numpy(), g[f"u{k}_actor_mean"]) and np.array_equal(lp.numpy(), g[f"u{k}_actor_precision"])
    assert g["c2_before_episode_step"].max() > 0 and g["c2_dataset"][n:rows, col["all_reset"]].sum() >= n    # episodes carried over, truncations inside


def test_standardize_and_running_normaliser_closed_forms(oracle):
    """The standardize layer and the running normaliser against their definitions written independently in numpy."""
    rng = np.random.default_rng(8)
    f32 = np.float32
    B, D, ld = 57, 5, 9
    x = rng.standard_normal((B, ld)).astype(f32) * 3 + 1
    x[:, 2] = 0.25                                  # a constant column: its deviation is reported as exactly 0
    mean = rng.standard_normal(D).astype(f32); std = np.abs(rng.standard_normal(D)).astype(f32) + 0.1; std[3] = 0
    lm, lp = oracle.zeros((D,)), oracle.zeros((D,))
    m, s = oracle.array(mean), oracle.array(std)
    oracle.call("standardize_set_statistics", m.ptr, s.ptr, lm.ptr, lp.ptr, D)
    precision = np.where(std == 0, f32(0), f32(1) / np.where(std == 0, f32(1), std)).astype(f32)
    assert np.array_equal(lm.numpy(), mean) and np.array_equal(lp.numpy(), precision) and precision[3] == 0
    xd, y = oracle.array(x), oracle.zeros((B, D))
    oracle.call("standardize_forward", lm.ptr, lp.ptr, xd.ptr, ld, y.ptr, D, B, D)
    want = (x[:, :D] - mean) * np.where(precision == 0, f32(1), precision)       # a zero precision leaves the centred value unscaled
    assert np.array_equal(y.numpy(), want)
    dy = rng.standard_normal((B, D)).astype(f32)
    d, dx = oracle.array(dy), oracle.zeros((B, D))
    oracle.call("standardize_backward_input", lp.ptr, d.ptr, D, dx.ptr, D, B, D)
    assert np.array_equal(dx.numpy(), dy * precision)
    # running normaliser: after k updates the mean is the average of the k batch means, likewise for the deviations (sample deviation, n - 1)
    rm, rs, age = oracle.zeros((D,)), oracle.array(np.ones(D, f32)), oracle.array(np.zeros(1, np.uint32))
    means, stds = [], []
    for k in range(4):
        batch = (rng.standard_normal((B, ld)) * (k + 1) + k).astype(f32); batch[:, 2] = 0.25
        bd = oracle.array(batch)
        oracle.call("running_normalizer_update", bd.ptr, ld, B, D, rm.ptr, rs.ptr, age.ptr)
        means.append(batch[:, :D].astype(np.float64).mean(0)); stds.append(batch[:, :D].astype(np.float64).std(0, ddof=1))
        assert int(age.numpy()[0]) == k + 1
        assert np.allclose(rm.numpy(), np.mean(means, 0), rtol=2e-6, atol=2e-6)
        want_std = np.mean(stds, 0); want_std[2] = 0 if k == 0 else want_std[2]
        assert np.allclose(np.delete(rs.numpy(), 2), np.delete(np.mean(stds, 0), 2), rtol=1e-5)
    assert rs.numpy()[2] == 0                      # first update: 1 + (0 - 1) / 1, then 0 + (0 - 0) / k


def test_evaluation_reproduces_reference_vectors(oracle):
    """rl::utils::evaluation::evaluate (10 episodes x 200 steps, Evaluation mode) of the SAC actor after 0, 150 and 400 loop steps: returns, episode
    lengths and summary statistics equal the reference's bit for bit (tests/golden/make_evaluation_golden.py). A deterministic actor with a tanh
    output layer whose single output row is the mean row of the same network must give the same episodes: that pins policy kind 1."""
    g = np.load(os.path.join(helpers.GOLDEN, "evaluation_pendulum_seed0.npz"))
    assert list(g["stops"]) == [0, 150, 400, 6000] and g["e3_summary"][0] > -250 > g["e0_summary"][0]      # the last actor is a trained one
    for k in range(len(g["stops"])):
        params, ini = g[f"e{k}_actor"], g[f"e{k}_initial_states"]
        ret, length, summary = helpers.evaluate_on_backend(oracle, [3, 64, 64, 2], params, "relu", "identity", 2, ini, 200)
        assert np.array_equal(ret, g[f"e{k}_returns"]) and np.array_equal(length, g[f"e{k}_episode_length"]) and np.array_equal(summary, g[f"e{k}_summary"])
        # statistics as the definition has them (population standard deviation), in float64
        assert abs(summary[0] - ret.astype(np.float64).mean()) <= 1e-3 and abs(summary[1] - ret.astype(np.float64).std()) <= 1e-2
        assert summary[2] == 200 and summary[3] == 0 and summary[4] == 0 and summary[5] == 0
        head = 3 * 64 + 64 + 64 * 64 + 64
        mean_only = np.concatenate([params[:head], params[head:head + 64], params[head + 128:head + 129]])     # first row of W3, first bias
        ret1, length1, summary1 = helpers.evaluate_on_backend(oracle, [3, 64, 64, 1], mean_only, "relu", "tanh", 1, ini, 200)
        assert np.array_equal(ret1, ret) and np.array_equal(summary1, summary)
    # shorter horizon: the return is a prefix sum of the same rewards, so it is larger (rewards are negative) and the lengths follow the limit
    ret50, length50, _ = helpers.evaluate_on_backend(oracle, [3, 64, 64, 2], g["e2_actor"], "relu", "identity", 2, g["e2_initial_states"], 50)
    assert np.all(length50 == 50) and np.all(ret50 > g["e2_returns"]) and np.all(ret50 < 0)


def test_evaluation_with_recurrent_policy_reproduces_reference_vectors(oracle):
    """rl::utils::evaluation::evaluate with the reference's recurrent SAC actor (one and two GRU layers; 5 episodes x 40 steps, the hidden state restarting every
    6 steps), untrained and after 40 and 150 training steps: returns, lengths and summary equal the reference's bit for bit
    (tests/golden/make_evaluation_recurrent_golden.py). Independently of the reference: the call resets the policy state itself (the helper hands it a state
    filled with other values), the state it leaves is that of 40 steps (40 mod 6 = 4 steps after the last restart), a horizon that ends on a restart leaves the
    initial hidden state, and a sequential policy of dense layers only gives the episodes of the same network evaluated as an MLP."""
    g = helpers.evaluation_recurrent_golden()
    n = 0
    for label, specs, params, period, ini, step_limit, ret, length, summary in helpers.evaluation_recurrent_golden_cases(g):
        got = helpers.evaluate_recurrent(oracle, specs, params, period, ini, step_limit)
        assert np.array_equal(got["returns"], ret) and np.array_equal(got["length"], length) and np.array_equal(got["summary"], summary), label
        assert all(np.all(s == step_limit % period) for s in got["steps"])
        ends_on_restart = helpers.evaluate_recurrent(oracle, specs, params, period, ini, 3 * period)
        off = 0
        for k, (kind, i, o, _) in enumerate(specs):
            if kind == 1:
                h0 = params[off + 3 * o * i + 3 * o + 3 * o * o + 3 * o:off + 3 * o * i + 3 * o + 3 * o * o + 3 * o + o]
                layer = [l for l, sp in enumerate(specs) if sp[0] == 1].index(k)
                assert np.array_equal(ends_on_restart["hidden"][layer], np.tile(h0, (len(ini), 1))) and np.all(ends_on_restart["steps"][layer] == 0)
                off += 3 * o * i + 3 * o + 3 * o * o + 3 * o + o
            else:
                off += i * o + o
        never = helpers.evaluate_recurrent(oracle, specs, params, 0, ini, step_limit)          # without the restarts the episodes differ
        assert not np.array_equal(never["returns"], ret) and all(np.all(s == step_limit) for s in never["steps"])
        n += 1
    assert n == 6
    rng = np.random.default_rng(5)
    dims = [3, 24, 24, 2]
    params = helpers.random_params(rng, dims)
    ini = np.stack([rng.uniform(-np.pi, np.pi, 9), rng.uniform(-1, 1, 9)], 1).astype(np.float32)
    want = helpers.evaluate_on_backend(oracle, dims, params, "tanh", "identity", 2, ini, 60)
    got = helpers.evaluate_recurrent(oracle, [(0, 3, 24, "tanh"), (0, 24, 24, "tanh"), (0, 24, 2, "identity")], params, 7, ini, 60)
    assert np.array_equal(got["returns"], want[0]) and np.array_equal(got["length"], want[1]) and np.array_equal(got["summary"], want[2])


def test_acrobot_reproduces_reference_vectors_and_conserves_energy(oracle):
    """Acrobot / AcrobotSwingup / EasyParameters steps against the reference's own outputs (tests/golden/make_acrobot_golden.py), bit for bit, random
    states and 200-step trajectories. Then what the mechanics fix: without torque the equations of motion conserve
    E = 1/2 dq^T M(q) dq - (m1 lc1 + m2 l1) g cos(q1) - m2 lc2 g cos(q1 + q2) with M = [[d1, d2], [d2, m2 lc2^2 + I2]], so E drifts only by the
    integration error, and that error falls about 16-fold (32-fold per unit time) when the classic Runge-Kutta step is halved."""
    g = np.load(os.path.join(helpers.GOLDEN, "acrobot_steps.npz"))
    for kind in range(3):
        got = helpers.acrobot_on_backend(oracle, kind, g["states"], g["actions"])
        for name, v in zip(("next_states", "observations", "next_observations", "rewards", "terminated"), got):
            assert np.array_equal(v, g[f"k{kind}_{name}"]), (kind, name)
        s = g[f"k{kind}_trajectory"][:1].copy()
        for k in range(200):
            s, _, _, r, t = helpers.acrobot_on_backend(oracle, kind, s, g["trajectory_actions"][k:k + 1])
            assert np.array_equal(s[0], g[f"k{kind}_trajectory"][k + 1]) and r[0] == g[f"k{kind}_trajectory_rewards"][k] and t[0] == g[f"k{kind}_trajectory_terminated"][k], (kind, k)

    def energy(s):
        q1, q2, w1, w2 = (s[:, i].astype(np.float64) for i in range(4))
        m1 = m2 = l1 = 1.0; lc1 = lc2 = 0.5; I1 = I2 = 1.0; grav = float(np.float32(9.8))
        d1 = m1 * lc1 ** 2 + m2 * (l1 ** 2 + lc2 ** 2 + 2 * l1 * lc2 * np.cos(q2)) + I1 + I2
        d2 = m2 * (lc2 ** 2 + l1 * lc2 * np.cos(q2)) + I2
        kinetic = 0.5 * (d1 * w1 ** 2 + 2 * d2 * w1 * w2 + (m2 * lc2 ** 2 + I2) * w2 ** 2)
        return kinetic - (m1 * lc1 + m2 * l1) * grav * np.cos(q1) - m2 * lc2 * grav * np.cos(q1 + q2)
    rng = np.random.default_rng(0)
    start = np.stack([rng.uniform(-1.5, 1.5, 32), rng.uniform(-1.5, 1.5, 32), rng.uniform(-1, 1, 32), rng.uniform(-1, 1, 32)], 1).astype(np.float32)
    zero = np.zeros(32, np.float32)         # action 0 is torque 0 for the symmetric torque range
    drift = {}
    for dt, steps in ((0.1, 10), (0.05, 20)):       # one second of motion either way
        p = helpers.capi.acrobot_parameters(); p.dt = dt
        s = start.copy()
        for _ in range(steps):
            s = helpers.acrobot_on_backend(oracle, 0, s, zero, params=p)[0]
        drift[dt] = np.abs(energy(s) - energy(start)).max()
    scale = np.abs(energy(start)).max()
    assert drift[0.1] <= 2e-4 * scale and drift[0.05] <= 1.5e-5 * scale, drift
    assert drift[0.1] / max(drift[0.05], 1e-9) >= 6.0, drift        # fourth-order method, float32 round-off included
    # a torque does work on the second joint: E changes by about torque * angle swept there
    p = helpers.capi.acrobot_parameters(); p.dt = 0.01
    s = np.zeros((1, 4), np.float32)
    swept = 0.0
    for _ in range(20):
        before = s[0, 1]
        s = helpers.acrobot_on_backend(oracle, 0, s, np.array([0.4], np.float32), params=p)[0]
        swept += float(s[0, 1] - before)
    assert abs((energy(s) - energy(np.zeros((1, 4), np.float32)))[0] - 2.0 * swept) <= 0.02 * abs(2.0 * swept)      # action 0.4 -> torque 2


def test_car_reproduces_reference_vectors_and_kinematics(oracle):
    """Car steps against the reference's own outputs (tests/golden/make_car_golden.py), bit for bit, random states and a 300-step trajectory. Then what
    the model fixes by itself: (1) a car rolling straight (no lateral speed, no yaw rate, no steering) has no slip angles, hence no lateral forces: it
    keeps its heading and obeys x' = x + dt cos(mu) vx, vx' = vx + dt (cm u - cr0 - cr2 vx^2) / m; (2) the dynamics do not depend on where the car is or
    which way it points: shifting and rotating the pose shifts and rotates the next pose and leaves the body-frame velocities alone; (3) below the
    speed threshold the tires transmit no lateral force, so yaw rate and lateral speed change only by the omega x v terms."""
    g = np.load(os.path.join(helpers.GOLDEN, "car_steps.npz"))
    got = helpers.car_on_backend(oracle, g["states"], g["actions"])
    for name, v in zip(("next_states", "observations", "next_observations", "rewards", "terminated"), got):
        assert np.array_equal(v, g[name]), name
    s = g["trajectory"][:1].copy()
    for k in range(300):
        s, _, _, r, t = helpers.car_on_backend(oracle, s, g["trajectory_actions"][k:k + 1])
        assert np.array_equal(s[0], g["trajectory"][k + 1]) and r[0] == g["trajectory_rewards"][k] and t[0] == g["trajectory_terminated"][k], k
    p = helpers.capi.car_parameters()
    rng = np.random.default_rng(0)
    n = 64
    # (1) straight rolling
    mu, vx, u = rng.uniform(-3, 3, n), rng.uniform(0.1, 2.5, n), rng.uniform(-1, 1, n)
    st = np.stack([rng.uniform(-0.5, 0.5, n), rng.uniform(-0.5, 0.5, n), mu, vx, np.zeros(n), np.zeros(n)], 1).astype(np.float32)
    nx = helpers.car_on_backend(oracle, st, np.stack([u, np.zeros(n)], 1))[0].astype(np.float64)
    s64 = st.astype(np.float64); u32 = u.astype(np.float32).astype(np.float64)
    assert np.abs(nx[:, 0] - (s64[:, 0] + p.dt * np.cos(s64[:, 2]) * s64[:, 3])).max() <= 1e-6
    assert np.abs(nx[:, 1] - (s64[:, 1] + p.dt * np.sin(s64[:, 2]) * s64[:, 3])).max() <= 1e-6
    assert np.abs(nx[:, 3] - (s64[:, 3] + p.dt * (p.cm * u32 - p.cr0 - p.cr2 * s64[:, 3] ** 2) / p.m)).max() <= 1e-5
    assert np.array_equal(nx[:, 2], s64[:, 2]) and np.all(nx[:, 4] == 0) and np.all(nx[:, 5] == 0)
    # (2) pose equivariance
    st = np.stack([rng.uniform(-0.3, 0.3, n), rng.uniform(-0.3, 0.3, n), rng.uniform(-1, 1, n), rng.uniform(0.2, 2, n), rng.uniform(-0.5, 0.5, n), rng.uniform(-4, 4, n)], 1).astype(np.float32)
    act = rng.uniform(-1, 1, (n, 2)).astype(np.float32)
    base = helpers.car_on_backend(oracle, st, act)[0].astype(np.float64)
    phi, shift = 0.7, np.array([0.2, -0.1])
    rot = np.array([[np.cos(phi), -np.sin(phi)], [np.sin(phi), np.cos(phi)]])
    moved = st.astype(np.float64).copy()
    moved[:, :2] = moved[:, :2] @ rot.T + shift; moved[:, 2] += phi
    nm = helpers.car_on_backend(oracle, moved.astype(np.float32), act)[0].astype(np.float64)
    assert np.abs(nm[:, :2] - (base[:, :2] @ rot.T + shift)).max() <= 2e-6 and np.abs(nm[:, 2] - (base[:, 2] + phi)).max() <= 1e-6
    assert np.abs(nm[:, 3:] - base[:, 3:]).max() <= 1e-6 * np.abs(base[:, 3:]).max()
    # (3) below the threshold: no tire forces
    st = np.stack([np.zeros(n), np.zeros(n), rng.uniform(-1, 1, n), rng.uniform(-0.01, 0.009, n), rng.uniform(-0.01, 0.009, n), rng.uniform(-2, 2, n)], 1).astype(np.float32)
    nx = helpers.car_on_backend(oracle, st, np.stack([np.zeros(n), rng.uniform(-1, 1, n)], 1))[0].astype(np.float64)
    s64 = st.astype(np.float64)
    assert np.array_equal(nx[:, 5], s64[:, 5])
    assert np.abs(nx[:, 4] - (s64[:, 4] - p.dt * s64[:, 5] * s64[:, 3])).max() <= 1e-8


def test_sequence_gather_reproduces_reference_vectors_and_invariants(oracle):
    """gather_batch for sequence batches against the reference's own batches (tests/golden/make_sequence_gather_golden.py), every tensor entry for entry,
    from the stored draws. Then on synthetic rings what the construction guarantees whatever the draws: observation/action rows of the batch are rows of
    the chosen ring or the step after a sequence end (next observation + zero action); sequences never run across an episode end or the ring's cursor;
    every sample's masks are consistent (the step after a final step carries the next observation and a zero action, and a new sequence starts
    behind it; the last unpadded step ends a sequence or is such a padding step)."""
    for rings, sampling, draws, max_len, batch, seq, want in helpers.sequence_gather_golden():
        got = helpers.gather_sequence_on_backend(oracle, rings, sampling, draws, max_len, batch, seq)
        for k in helpers.SEQUENCE_BATCH_FIELDS:
            assert np.array_equal(got[k], want[k]), k
    rng = np.random.default_rng(0)
    for (always, random_len, steps) in ((1, 1, 700), (0, 0, 700), (1, 1, 100), (0, 1, 180)):
        obs, cap, max_len, batch, seq = 5, 300, 40, 128, 12
        rings = helpers.synthetic_rings(rng, 4, cap, obs, steps, max_len)
        sampling = helpers.capi.SequenceSampling(always, random_len, 1, 0.5, 1)
        env, off, nom, length = helpers.random_sequence_draws(rng, rings, sampling, max_len, batch, seq)
        got = helpers.gather_sequence_on_backend(oracle, rings, sampling, (env, off, nom, length), max_len, batch, seq)
        oab, final, reset, nfinal = got["observations_actions_base"], got["final_step_mask"], got["reset"], got["next_final_step_mask_base"]
        assert np.all((final[-1] == 1) | (final[-2] == 1)) and np.all(reset[0] == 1) and np.all(nfinal[0] == 0)      # the last step ends a sequence or pads after one
        for b in range(batch):
            data, position, full, es = rings[env[b]]
            valid = np.arange(cap) if full else np.arange(position)
            s = 0
            while s <= seq:
                # a sequence starts at s: find the ring row it starts from
                rows = np.nonzero((data[valid][:, :obs + 1] == oab[s, b]).all(1))[0]
                assert len(rows) >= 1 and reset[min(s, seq - 1), b] == 1 or s == seq, (b, s)
                if s == seq:
                    break
                r = valid[rows[0]]
                if always:
                    assert es[r] == r
                while True:
                    assert np.array_equal(oab[s, b], data[r, :obs + 1]) and got["rewards"][s, b] == data[r, obs + 1]
                    if final[s, b]:
                        assert np.array_equal(oab[s + 1, b, :obs], data[r, obs + 2:2 * obs + 2]) and oab[s + 1, b, obs] == 0 and nfinal[s + 1, b] == 1
                        s += 2      # the step after a final step holds the next observation; a new sequence starts after it
                        break
                    assert data[r, -1] == 0 and (r + 1) % cap != position       # not the end of an episode, not the cursor
                    r = (r + 1) % cap
                    s += 1


def test_car_on_track_rays_and_flags_on_a_synthetic_track(oracle):
    """CarTrack without the reference: on a straight corridor the three ray distances have closed forms (the ray leaves the corridor through a wall at
    a known distance, in steps of half a cell), terminated says whether the next position is in a drivable cell, the reward is the forward speed, and
    the step is the Car's. Cells beyond the bitmap count as not drivable."""
    H, W, scale = 60, 200, 0.02
    track = np.zeros((H, W), np.uint8)
    track[20:40, :] = 1                                  # a corridor along x, 20 cells = 0.4 m wide, centred on y = 0
    rng = np.random.default_rng(0)
    n = 200
    x = rng.uniform(-1.0, 1.0, n); y = rng.uniform(-0.15, 0.15, n)
    states = np.stack([x, y, np.zeros(n), rng.uniform(0.1, 1, n), np.zeros(n), np.zeros(n)], 1).astype(np.float32)      # heading along +x
    ns, o, no, r, t = helpers.car_track_on_backend(oracle, track, scale, states, np.zeros((n, 2), np.float32))
    assert np.array_equal(r, states[:, 3]) and np.array_equal(o[:, :6], states)
    assert np.array_equal(ns, helpers.car_on_backend(oracle, states, np.zeros((n, 2), np.float32))[0])
    half = scale / 2
    # straight ahead: the corridor runs to the end of the bitmap at x = +2.0, farther than the ray (50 half-cells = 0.5 m) unless the car is near it
    free = np.minimum(np.floor((2.0 - states[:, 0].astype(np.float64)) / half - 1e-9) + 1, 50)
    assert np.abs(o[:, 7] * 50 - free).max() <= 1
    # 20 degrees to the left (+y): the wall at y = +0.2 is (0.2 - y) / sin(20 deg) away along the ray
    ang = 20 / 180 * np.pi
    left = np.minimum((0.2 - states[:, 1].astype(np.float64)) / np.sin(ang) / half, 50)
    right = np.minimum((0.2 + states[:, 1].astype(np.float64)) / np.sin(ang) / half, 50)
    assert np.abs(o[:, 8] * 50 - left).max() <= 1.5 and np.abs(o[:, 6] * 50 - right).max() <= 1.5
    # terminated: the next position's cell
    cx = np.floor((ns[:, 0].astype(np.float64) + scale * W / 2) / scale).astype(int); cy = np.floor((-ns[:, 1].astype(np.float64) + scale * H / 2) / scale).astype(int)
    inside = (cx >= 0) & (cx < W) & (cy >= 0) & (cy < H)
    want = np.ones(n, np.uint8); want[inside] = 1 - track[cy[inside], cx[inside]]
    assert np.array_equal(t, want)
    # off the bitmap: everything reads as not drivable
    far = np.array([[5.0, 0.0, 0.0, 1.0, 0.0, 0.0], [0.0, -3.0, 1.0, 1.0, 0.0, 0.0]], np.float32)
    _, o2, _, _, t2 = helpers.car_track_on_backend(oracle, track, scale, far, np.zeros((2, 2), np.float32))
    assert np.all(o2[:, 6:] == 0) and np.all(t2 == 1)


@pytest.mark.parametrize("n_layers", [3, 5])
def test_sac_on_sequence_batches_reproduces_reference_vectors(oracle, n_layers):
    """SAC with the reference's recurrent approximators on sequence batches: from the fixture's parameters, batches and noise the restatement
    reproduces the parameter digests after every loop step and the full parameter snapshots, bit for bit."""
    g = helpers.sac_sequence_golden()
    actor_specs, critic_specs, (B, S, obs, act, first, steps), hyper = helpers.sac_sequence_golden_case(g, n_layers)
    p = f"l{n_layers}_"
    agent = helpers.SacSequenceOnBackend(oracle, actor_specs, critic_specs, g[p + "parameters_before"], S, B, obs, act, bool(first), hyper)
    resets_inside = 0
    for i in range(steps):
        helpers.sac_sequence_golden_step(agent, g, n_layers, i)
        resets_inside += int(g[f"{p}s{i}_reset"][1:].sum())
        params = agent.parameters()
        assert np.array_equal(helpers.sac_sequence_digest(params, actor_specs, critic_specs), g[f"{p}s{i}_digest"]), i
        if i in g[p + "snapshots"]:
            assert np.array_equal(params, g[f"{p}s{i}_after"]), i
    assert agent.ages() == [int(a) for a in g[p + "ages_after"]]
    assert resets_inside > 20       # sequences that restart inside the batch are what the reset modes are about


def test_sac_sequence_of_length_one_equals_the_single_step_update(oracle):
    """Independent of the sequence fixture: with sequence length 1, dense layers only, every step final and the `next` views starting at padded
    step 1, the sequence update must give what the single-step SAC update (pinned against the reference's default loop) gives."""
    rng = np.random.default_rng(3)
    B, H, OBS, ACT = 64, 16, 3, 1
    actor_specs = [(0, OBS, H, "relu"), (0, H, H, "relu"), (0, H, 2 * ACT, "identity")]
    critic_specs = [(0, OBS + ACT, H, "relu"), (0, H, H, "relu"), (0, H, 1, "identity")]
    na, nc = helpers.seq_param_count(actor_specs), helpers.seq_param_count(critic_specs)
    critics = [helpers.random_seq_params(rng, critic_specs) for _ in range(2)]
    params = np.concatenate([helpers.random_seq_params(rng, actor_specs)] + critics + [c.copy() for c in critics] + [np.array([np.log(0.5)], np.float32)])
    assert params.size == na + 4 * nc + 1
    oab = rng.standard_normal((2, B, OBS + ACT)).astype(np.float32)
    rewards, terminated = rng.standard_normal((1, B)).astype(np.float32), (rng.uniform(size=(1, B)) < 0.2).astype(np.uint8)
    ones = np.ones((1, B), np.uint8)
    seq = helpers.SacSequenceOnBackend(oracle, actor_specs, critic_specs, params, 1, B, OBS, ACT, include_first=False)
    seq.set_batch(dict(observations_actions_base=oab, rewards=rewards, terminated=terminated, reset=ones, next_reset_base=np.ones((2, B), np.uint8), final_step_mask=ones,
                       next_final_step_mask_base=np.ones((2, B), np.uint8)))
    one = helpers.SacOnBackend(oracle, B, H, params)
    one.set_batch(oab, rewards[0], terminated[0])
    for _ in range(3):
        nc_, na_ = rng.standard_normal((1, B, ACT)).astype(np.float32), rng.standard_normal((1, B, ACT)).astype(np.float32)
        seq.train(nc_, na_)
        n1, n2 = oracle.array(nc_), oracle.array(na_)
        for k in range(2):
            oracle.call("sac_train_critic", C.byref(one.c), k, n1.ptr)
        oracle.call("sac_update_critic_targets", C.byref(one.c))
        oracle.call("sac_train_actor", C.byref(one.c), n2.ptr)
        assert np.array_equal(seq.parameters(), one.parameters())


@pytest.mark.parametrize("with_reset", [False, True])
def test_sequential_model_gradients_against_finite_differences(oracle, with_reset):
    """dense -> GRU -> GRU -> dense with exact gate functions: the gradients of sum(output * g) with respect to the input and to a sample of
    every layer's parameters, by central differences in float64-accumulated outputs, with and without resets inside the sequence."""
    rng = np.random.default_rng(17 + with_reset)
    S, B, I, H, O = 5, 3, 4, 6, 2
    specs = [(0, I, H, "tanh"), (1, H, H, "identity"), (1, H, H, "identity"), (0, H, O, "identity")]
    params = helpers.random_seq_params(rng, specs)
    x, g = rng.standard_normal((S, B, I)).astype(np.float32), rng.standard_normal((S, B, O)).astype(np.float32)
    reset = np.zeros((S, B), np.uint8)
    if with_reset:
        reset[2, 0] = reset[3, 2] = reset[1, 1] = 1

    def loss(p, xx):
        net = helpers.SeqNet(oracle, specs, p, S, B, fast_tanh=False)
        xd, rd = oracle.array(xx), oracle.array(reset)
        oracle.call("seq_forward", net.layers, net.n, xd.ptr, I, rd.ptr if with_reset else None, S, B, None, 0)
        return float((net.output().astype(np.float64).reshape(g.shape) * g).sum())
    net = helpers.SeqNet(oracle, specs, params, S, B, fast_tanh=False)
    xd, rd, gd, dx = oracle.array(x), oracle.array(reset), oracle.array(g), oracle.zeros((S, B, I))
    oracle.call("seq_zero_gradient", net.layers, net.n)
    oracle.call("seq_forward", net.layers, net.n, xd.ptr, I, rd.ptr if with_reset else None, S, B, None, 0)
    oracle.call("seq_backward", net.layers, net.n, xd.ptr, I, gd.ptr, dx.ptr, rd.ptr if with_reset else None, S, B, 1, 0, None, 0)
    grads, dxn = net.grads.numpy(), dx.numpy()
    eps = 2e-3
    checked = 0
    for idx in rng.choice(params.size, 60, replace=False):
        hi, lo = params.copy(), params.copy(); hi[idx] += eps; lo[idx] -= eps
        fd = (loss(hi, x) - loss(lo, x)) / (2 * eps)
        assert abs(fd - grads[idx]) <= 2e-2 * max(1.0, abs(fd)), (idx, fd, grads[idx])
        checked += grads[idx] != 0
    assert checked > 40       # the initial hidden state is not learned: its gradient stays zero
    for idx in [(0, 0, 0), (2, 0, 1), (4, 2, 3), (1, 1, 2)]:
        hi, lo = x.copy(), x.copy(); hi[idx] += eps; lo[idx] -= eps
        fd = (loss(params, hi) - loss(params, lo)) / (2 * eps)
        assert abs(fd - dxn[idx]) <= 2e-2 * max(1.0, abs(fd)), (idx, fd, dxn[idx])
    # the switch of backward_input: without the resets the input gradient of a multi-layer model differs where a reset cut the sequence
    if with_reset:
        out = []
        for flag in (0, 1):
            gd2, dx2 = oracle.array(g), oracle.zeros((S, B, I))
            oracle.call("seq_backward", net.layers, net.n, None, 0, gd2.ptr, dx2.ptr, rd.ptr, S, B, 0, flag, None, 0)
            out.append(dx2.numpy())
        assert np.allclose(out[1], dxn, rtol=1e-5, atol=1e-6) and not np.allclose(out[0], out[1], rtol=1e-3, atol=1e-5)


def test_recurrent_runner_step_reproduces_reference_vectors(oracle):
    """The off-policy runner step with the reference's recurrent actor (fixture written by its SAC loop): states, counters, truncation flags, the policy's
    hidden state and step counters (with their automatic restart every 6 steps and the reset where an episode starts), ring cursors and the rows written,
    bit for bit over 24 loop steps."""
    g = helpers.recurrent_runner_golden()
    run, steps = helpers.recurrent_runner_from_golden(oracle, g)
    restarts = new_episodes = 0
    for i in range(steps):
        got = helpers.recurrent_runner_golden_step(run, g, i)
        for k in ("states", "episode_step", "episode_return", "truncated", "hidden", "steps", "position", "current_episode_start", "rows", "previous_truncated"):
            assert np.array_equal(got[k], g[f"s{i}_{k}"]), (i, k)
        restarts += int((g[f"s{i}_steps"] == 0).sum()); new_episodes += int(g[f"s{i}_reset"].sum())
    assert restarts >= 9 and new_episodes >= 3


@pytest.mark.parametrize("fast_tanh", [False, True])
def test_evaluate_step_chain_equals_the_sequence_forward_pass(oracle, fast_tanh):
    """Independent of the reference: S single steps on the kept state give what one forward pass over the S-step sequence gives (same arithmetic, bit for
    bit), a reset mask in the middle equals a reset flag of the sequence, and with an auto-reset period the state restarts after that many steps."""
    rng = np.random.default_rng(31 + fast_tanh)
    S, B, I, H, O = 7, 5, 3, 8, 2
    specs = [(0, I, H, "relu"), (1, H, H, "identity"), (1, H, H, "identity"), (0, H, O, "identity")]
    params = helpers.random_seq_params(rng, specs)
    # a non-zero initial hidden state, so that a restart is visible
    off = helpers.seq_param_count(specs[:1]) + 3 * H * H + 3 * H + 3 * H * H + 3 * H
    params[off:off + H] = rng.uniform(-0.5, 0.5, H)
    x = rng.standard_normal((S, B, I)).astype(np.float32)
    reset = np.zeros((S, B), np.uint8); reset[3, 1] = reset[5, 4] = 1
    net = helpers.SeqNet(oracle, specs, params, S, B, fast_tanh=fast_tanh)
    xd, rd = oracle.array(x), oracle.array(reset)
    oracle.call("seq_forward", net.layers, net.n, xd.ptr, I, rd.ptr, S, B, None, 0)
    want = net.output().reshape(S, B, O)
    state = helpers.SeqStateOnBackend(oracle, specs, B)
    oracle.call("seq_reset_state", net.layers, net.n, C.byref(state.c), None, B)
    y = oracle.zeros((B, O))
    for t in range(S):
        if reset[t].any():
            m = oracle.array(reset[t])
            oracle.call("seq_reset_state", net.layers, net.n, C.byref(state.c), m.ptr, B)
        xt = oracle.array(x[t])
        oracle.call("seq_evaluate_step", net.layers, net.n, xt.ptr, I, C.byref(state.c), 0, y.ptr, O, B, None, 0)
        assert np.array_equal(y.numpy(), want[t]), t
    assert all(list(s) == [S, S - 3, S, S, S - 5] for s in state.numpy()[1])      # steps since each row's last reset
    # auto-reset every 3 steps == a sequence with reset flags at steps 3 and 6
    reset3 = np.zeros((S, B), np.uint8); reset3[3] = reset3[6] = 1
    rd3 = oracle.array(reset3)
    oracle.call("seq_forward", net.layers, net.n, xd.ptr, I, rd3.ptr, S, B, None, 0)
    want3 = net.output().reshape(S, B, O)
    oracle.call("seq_reset_state", net.layers, net.n, C.byref(state.c), None, B)
    for t in range(S):
        xt = oracle.array(x[t])
        oracle.call("seq_evaluate_step", net.layers, net.n, xt.ptr, I, C.byref(state.c), 3, y.ptr, O, B, None, 0)
        assert np.array_equal(y.numpy(), want3[t]), t
    assert not np.array_equal(want3[3:], want[3:])


def test_env_evaluate_reproduces_reference_vectors_and_counts_terminations(oracle):
    """The evaluation over any environment: with the Pendulum it gives the reference's own episodes bit for bit (the vectors above); with the Acrobot, whose
    episodes terminate, every episode equals that episode run alone, one step at a time, until its first terminated flag -- the terminating step's
    reward counted, nothing after it (rl/utils/evaluation/operations_generic.h:166-197)."""
    g = np.load(os.path.join(helpers.GOLDEN, "evaluation_pendulum_seed0.npz"))
    specs = [(0, 3, 64, "relu"), (0, 64, 64, "relu"), (0, 64, 2, "identity")]
    for k in range(len(g["stops"])):
        ret, length, summary = helpers.env_evaluate_on_backend(oracle, helpers.capi.ENV_PENDULUM, specs, g[f"e{k}_actor"], 2, g[f"e{k}_initial_states"], 200)
        assert np.array_equal(ret, g[f"e{k}_returns"]) and np.array_equal(length, g[f"e{k}_episode_length"]) and np.array_equal(summary, g[f"e{k}_summary"])
    rng = np.random.default_rng(11)
    n, limit = 12, 60
    specs = [(0, 6, 16, "tanh"), (0, 16, 1, "tanh")]
    params = helpers.random_seq_params(rng, specs)
    ini = rng.uniform(-0.1, 0.1, (n, 4)).astype(np.float32)
    ini[::2, 0] += 2.0 + rng.uniform(0, 0.4, n // 2).astype(np.float32)      # every other episode starts with the first link raised
    ret, length, summary = helpers.env_evaluate_on_backend(oracle, helpers.capi.ENV_ACROBOT, specs, params, 1, ini, limit)
    W1, b1, W2, b2 = params[:96].reshape(16, 6), params[96:112], params[112:128].reshape(1, 16), params[128:129]
    n_terminated = 0
    for e in range(n):
        state, total, steps = ini[e:e + 1].copy(), np.float32(0), 0
        for _ in range(limit):
            _, obs, _, _, _ = helpers.acrobot_on_backend(oracle, 0, state, np.zeros(1, np.float32))
            action = np.tanh(np.tanh(obs.astype(np.float64) @ W1.T.astype(np.float64) + b1) @ W2.T.astype(np.float64) + b2).astype(np.float32).reshape(1)
            state, _, _, r, t = helpers.acrobot_on_backend(oracle, 0, state, action)
            total = np.float32(total + r[0]); steps += 1
            if t[0]:
                n_terminated += 1
                break
        assert length[e] == steps and abs(ret[e] - total) <= 1e-6 * steps, (e, length[e], steps, ret[e], total)
    assert 0 < n_terminated < n and summary[4] == n_terminated and summary[5] == np.float32(n_terminated) / np.float32(n)
    assert abs(summary[2] - length.mean()) <= 1e-4 and abs(summary[3] - length.std()) <= 1e-3
