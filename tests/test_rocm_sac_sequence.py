"""Sequential models with GRU layers and SAC's train_critic / train_actor on sequence batches, through the C ABI, against the CPU checker.

Tolerance: 1e-5 relative to the largest magnitude of the reference tensor (fp32); the device agent starts every loop step from the checker's
state (parameters, Adam moments and ages), so that differences do not accumulate through Adam's sign-like first steps."""
import ctypes as C

import numpy as np
import pytest

import helpers
from helpers import rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-5


def copy_net(src, dst):
    for name in ("params", "grads", "m", "v", "age"):
        a = getattr(src, name)
        if a is not None:
            getattr(dst, name).upload(a.numpy())


def copy_agent(src, dst):
    copy_net(src.actor, dst.actor)
    for k in range(2):
        copy_net(src.critics[k], dst.critics[k]); copy_net(src.targets[k], dst.targets[k])
    dst.log_alpha.upload(src.log_alpha.numpy()); dst.alpha_age.upload(src.alpha_age.numpy())


def compare_agents(got, want, where, tol=TOL):
    for name, a, b in [("actor", got.actor, want.actor)] + [(f"critic{k}", got.critics[k], want.critics[k]) for k in range(2)]:
        assert rel_err(a.grads.numpy(), b.grads.numpy()) <= tol, (where, name, "gradients", rel_err(a.grads.numpy(), b.grads.numpy()))
        assert rel_err(a.params.numpy(), b.params.numpy()) <= tol, (where, name, "parameters", rel_err(a.params.numpy(), b.params.numpy()))
    for k in range(2):
        assert rel_err(got.targets[k].params.numpy(), want.targets[k].params.numpy()) <= tol, (where, "target", k)
    assert rel_err(got.log_alpha.numpy(), want.log_alpha.numpy()) <= tol, (where, "log_alpha", got.log_alpha.numpy(), want.log_alpha.numpy())
    for key in ("target", "next_lp", "next_q0", "next_q1", "d_ci0", "d_ci1", "d_ao", "a_lp"):
        # the log-probabilities hold log(1 - a^2 + 1e-6): for an action within 1e-3 of +-1 one ulp of tanh moves that term by 1e-4 (the
        # reference's own formula, equally sensitive on the CPU); what is formed from them (targets, log_alpha) is held to the tolerance
        t = 10 * tol if key.endswith("_lp") else tol
        assert rel_err(got.buf[key].numpy(), want.buf[key].numpy()) <= t, (where, key, rel_err(got.buf[key].numpy(), want.buf[key].numpy()))
    assert got.ages() == want.ages()


# (steps, batch, in, hidden, out, GRU layers, fast_tanh, resets)
MODEL_CASES = [(6, 16, 4, 16, 1, 1, True, True), (7, 5, 3, 8, 2, 2, False, True), (5, 33, 17, 64, 6, 1, True, True), (9, 64, 11, 64, 3, 2, True, False),
               (1, 7, 4, 16, 1, 1, True, False), (12, 130, 6, 32, 2, 1, False, True)]


@pytest.mark.parametrize("case", MODEL_CASES)
def test_sequential_model_forward_and_backward_match_checker(oracle, rocm, case):
    print("case", case, flush=True)
    S, B, I, H, O, n_gru, fast, with_reset = case
    rng = np.random.default_rng(S * 100 + B)
    specs = [(0, I, H, "relu")] + [(1, H, H, "identity")] * n_gru + [(0, H, H, "tanh"), (0, H, O, "identity")]
    params = helpers.random_seq_params(rng, specs)
    x, g = rng.standard_normal((S, B, I + 2)).astype(np.float32), rng.standard_normal((S, B, O)).astype(np.float32)      # the input has a leading dimension of I + 2
    reset = (rng.uniform(size=(S, B)) < 0.2).astype(np.uint8)
    res = {}
    for be in (oracle, rocm):
        net = helpers.SeqNet(be, specs, params, S, B, fast_tanh=fast)
        ws, wsn = net.workspace()
        xd, rd = be.array(x), be.array(reset)
        r = rd.ptr if with_reset else None
        be.call("seq_zero_gradient", net.layers, net.n)
        be.call("seq_forward", net.layers, net.n, xd.ptr, I + 2, r, S, B, ws, wsn)
        out = {"y": net.output()}
        gd, dx = be.array(g), be.zeros((S, B, I))
        be.call("seq_backward", net.layers, net.n, xd.ptr, I + 2, gd.ptr, dx.ptr, r, S, B, 1, 0, ws, wsn)
        be.sync()
        out["grads"], out["dx"], out["d_output_after"] = net.grads.numpy(), dx.numpy(), gd.numpy()
        for flag in (0, 1):       # backward_input with and without the resets handed to the inner layers
            gd2, dx2 = be.array(g), be.zeros((S, B, I))
            be.call("seq_backward", net.layers, net.n, None, 0, gd2.ptr, dx2.ptr, r, S, B, 0, flag, ws, wsn)
            be.sync()
            out[f"dx_input_only_{flag}"] = dx2.numpy()
        res[be.name] = out
    for k, want in res["oracle"].items():
        assert rel_err(res["rocm"][k], want) <= TOL, (k, rel_err(res["rocm"][k], want))
    if with_reset and reset[1:].any() and S > 1:
        assert rel_err(res["oracle"]["dx_input_only_0"], res["oracle"]["dx_input_only_1"]) > 1e-3
        assert rel_err(res["oracle"]["dx_input_only_1"], res["oracle"]["dx"]) <= 1e-6


@pytest.mark.parametrize("n_layers", [3, 5])
def test_sac_sequence_updates_against_reference_vectors(oracle, rocm, n_layers):
    """The reference's own run (fixture): every loop step on the device from the checker's state, compared after the step in gradients,
    parameters, target networks, log_alpha and the training buffers; the checker itself must land on the fixture's snapshots bit for bit."""
    g = helpers.sac_sequence_golden()
    actor_specs, critic_specs, (B, S, obs, act, first, steps), hyper = helpers.sac_sequence_golden_case(g, n_layers)
    p = f"l{n_layers}_"
    agents = [helpers.SacSequenceOnBackend(be, actor_specs, critic_specs, g[p + "parameters_before"], S, B, obs, act, bool(first), hyper) for be in (oracle, rocm)]
    for i in range(steps):
        print("step", i, flush=True)
        copy_agent(agents[0], agents[1])
        for a in agents:
            helpers.sac_sequence_golden_step(a, g, n_layers, i)
        compare_agents(agents[1], agents[0], (n_layers, i))
        if i in g[p + "snapshots"]:
            assert np.array_equal(agents[0].parameters(), g[f"{p}s{i}_after"])


def synthetic_sequence_batch(rng, S, B, D):
    """A batch with the structure gather_batch produces: sequences end at random steps (final-step mask), the step after an end is a reset
    and carries the next observation; the `next` flags are the same ones shifted by a step."""
    final = (rng.uniform(size=(S, B)) < 0.3).astype(np.uint8); final[-1] = 1
    reset = np.zeros((S, B), np.uint8); reset[0] = 1; reset[1:] = final[:-1]
    next_reset = np.zeros((S + 1, B), np.uint8); next_reset[0] = 1; next_reset[1:] = final
    next_final = np.zeros((S + 1, B), np.uint8); next_final[1:] = final
    return dict(observations_actions_base=rng.standard_normal((S + 1, B, D)).astype(np.float32), rewards=rng.standard_normal((S, B)).astype(np.float32),
                terminated=(rng.uniform(size=(S, B)) < 0.1).astype(np.uint8), reset=reset, next_reset_base=next_reset, final_step_mask=final, next_final_step_mask_base=next_final)


@pytest.mark.parametrize("case", [(32, 128, 11, 3, 64, True), (10, 100, 5, 2, 32, False), (100, 100, 3, 1, 32, True)])
def test_sac_sequence_updates_at_larger_shapes(oracle, rocm, case):
    """Wider networks (hidden 64 takes the register-resident GRU kernels), several action dimensions, longer sequences -- up to the sequence
    length and batch size of the reference's recurrent Pendulum configuration (100 x 100) -- on synthetic batches, two loop steps each."""
    print("case", case, flush=True)
    S, B, OBS, ACT, H, first = case
    rng = np.random.default_rng(S + B)
    actor_specs = [(0, OBS, H, "relu"), (1, H, H, "identity"), (0, H, 2 * ACT, "identity")]
    critic_specs = [(0, OBS + ACT, H, "relu"), (1, H, H, "identity"), (1, H, H, "identity"), (0, H, 1, "identity")]
    critics = [helpers.random_seq_params(rng, critic_specs) for _ in range(2)]
    params = np.concatenate([helpers.random_seq_params(rng, actor_specs)] + critics + [c.copy() for c in critics] + [np.array([np.log(0.5)], np.float32)])
    hyper = dict(sas=helpers.capi.SasParameters(-20.0, 2.0, 1e-6, -float(ACT)))
    agents = [helpers.SacSequenceOnBackend(be, actor_specs, critic_specs, params, S, B, OBS, ACT, first, hyper) for be in (oracle, rocm)]
    T = S + 1 if first else S
    for i in range(2):
        data = synthetic_sequence_batch(rng, S, B, OBS + ACT)
        nc, na = rng.standard_normal((T, B, ACT)).astype(np.float32), rng.standard_normal((S, B, ACT)).astype(np.float32)
        copy_agent(agents[0], agents[1])
        for a in agents:
            a.set_batch(data); a.train(nc, na)
        compare_agents(agents[1], agents[0], (case, i), tol=2e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("case", [(100, 100, 3, 1, 32, True), (10, 100, 5, 2, 32, False), (48, 64, 11, 3, 64, True)])
def test_both_critics_in_one_call_leave_the_bits_of_the_two_calls(rocm, case):
    """rlt_rocm_sac_sequence_train_critics (the target part once, the two critics' passes side by side on the handle's two streams from 48 steps up) against
    rlt_rocm_sac_sequence_train_critic for critic 0 and then for critic 1: three loop steps each from the same parameters, batches and noise; every parameter and the
    training buffers that both leave behind, bit for bit."""
    S, B, OBS, ACT, H, first = case
    rng = np.random.default_rng(S * 3 + B)
    actor_specs = [(0, OBS, H, "relu"), (1, H, H, "identity"), (0, H, 2 * ACT, "identity")]
    critic_specs = [(0, OBS + ACT, H, "relu"), (1, H, H, "identity"), (1, H, H, "identity"), (0, H, 1, "identity")]
    critics = [helpers.random_seq_params(rng, critic_specs) for _ in range(2)]
    params = np.concatenate([helpers.random_seq_params(rng, actor_specs)] + critics + [c.copy() * 0.9 for c in critics] + [np.array([np.log(0.5)], np.float32)])
    hyper = dict(sas=helpers.capi.SasParameters(-20.0, 2.0, 1e-6, -float(ACT)))
    agents = [helpers.SacSequenceOnBackend(rocm, actor_specs, critic_specs, params, S, B, OBS, ACT, first, hyper) for _ in range(2)]
    T = S + 1 if first else S
    for i in range(3):
        data = synthetic_sequence_batch(rng, S, B, OBS + ACT)
        nc, na = rng.standard_normal((T, B, ACT)).astype(np.float32), rng.standard_normal((S, B, ACT)).astype(np.float32)
        for a, together in zip(agents, (False, True)):
            a.set_batch(data); a.train(nc, na, both_critics_in_one_call=together)
        assert np.array_equal(agents[0].parameters(), agents[1].parameters()), (case, i)
        for key in ("target", "d_output", "next_q0", "next_q1", "next_lp", "nsavi"):
            if key in agents[0].buf:
                assert np.array_equal(agents[0].buf[key].numpy(), agents[1].buf[key].numpy()), (case, i, key)
        assert agents[0].ages() == agents[1].ages()
    assert np.abs(agents[1].parameters() - params).max() > 1e-4


def test_sac_sequence_of_length_one_equals_single_step_update_on_device(rocm):
    """Sequence length 1, dense layers only, every step final: the sequence entry points and the single-step entry points of the same library."""
    rng = np.random.default_rng(5)
    B, H, OBS, ACT = 256, 64, 3, 1
    actor_specs = [(0, OBS, H, "relu"), (0, H, H, "relu"), (0, H, 2 * ACT, "identity")]
    critic_specs = [(0, OBS + ACT, H, "relu"), (0, H, H, "relu"), (0, H, 1, "identity")]
    critics = [helpers.random_seq_params(rng, critic_specs) for _ in range(2)]
    params = np.concatenate([helpers.random_seq_params(rng, actor_specs)] + critics + [c.copy() for c in critics] + [np.array([np.log(0.5)], np.float32)])
    oab = rng.standard_normal((2, B, OBS + ACT)).astype(np.float32)
    rewards, terminated = rng.standard_normal((1, B)).astype(np.float32), (rng.uniform(size=(1, B)) < 0.2).astype(np.uint8)
    ones = np.ones((1, B), np.uint8)
    seq = helpers.SacSequenceOnBackend(rocm, actor_specs, critic_specs, params, 1, B, OBS, ACT, include_first=False)
    seq.set_batch(dict(observations_actions_base=oab, rewards=rewards, terminated=terminated, reset=ones, next_reset_base=np.ones((2, B), np.uint8), final_step_mask=ones,
                       next_final_step_mask_base=np.ones((2, B), np.uint8)))
    one = helpers.SacOnBackend(rocm, B, H, params)
    one.set_batch(oab, rewards[0], terminated[0])
    nc, na = rng.standard_normal((1, B, ACT)).astype(np.float32), rng.standard_normal((1, B, ACT)).astype(np.float32)
    seq.train(nc, na)
    n1, n2 = rocm.array(nc), rocm.array(na)
    for k in range(2):
        rocm.call("sac_train_critic", C.byref(one.c), k, n1.ptr)
    rocm.call("sac_update_critic_targets", C.byref(one.c))
    rocm.call("sac_train_actor", C.byref(one.c), n2.ptr)
    rocm.sync()
    assert rel_err(seq.parameters(), one.parameters()) <= TOL


def test_sac_sequence_rejects_inconsistent_arguments(rocm):
    rng = np.random.default_rng(0)
    specs_a, specs_c = [(0, 3, 16, "relu"), (1, 16, 16, "identity"), (0, 16, 2, "identity")], [(0, 4, 16, "relu"), (1, 16, 16, "identity"), (0, 16, 1, "identity")]
    critics = [helpers.random_seq_params(rng, specs_c) for _ in range(4)]
    params = np.concatenate([helpers.random_seq_params(rng, specs_a)] + critics + [np.zeros(1, np.float32)])
    agent = helpers.SacSequenceOnBackend(rocm, specs_a, specs_c, params, 4, 8, 3, 1)
    noise = rocm.zeros((5, 8, 1))
    lib, h = rocm.device.lib, rocm.device.handle
    assert lib.rlt_rocm_sac_sequence_train_critic(h, C.byref(agent.c), 2, noise.ptr) == helpers.capi.RLT_E_INVALID_ARGUMENT
    assert lib.rlt_rocm_sac_sequence_train_actor(h, C.byref(agent.c), None) == helpers.capi.RLT_E_INVALID_ARGUMENT
    agent.c.workspace_bytes = 16
    assert lib.rlt_rocm_sac_sequence_train_critic(h, C.byref(agent.c), 0, noise.ptr) == helpers.capi.RLT_E_INVALID_ARGUMENT
    agent.c.workspace_bytes = agent.ws.nbytes
    agent.c.action_dim = 2        # the actor's last layer has 2 outputs = 2 * 1
    assert lib.rlt_rocm_sac_sequence_update_critic_targets(h, C.byref(agent.c)) == helpers.capi.RLT_E_INVALID_ARGUMENT
    assert lib.rlt_rocm_seq_forward(h, agent.actor.layers, 3, noise.ptr, 2, None, 4, 8, None, 0) == helpers.capi.RLT_E_INVALID_ARGUMENT      # leading dimension below the input width
