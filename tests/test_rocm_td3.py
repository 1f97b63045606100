"""TD3 on the HIP path through the C ABI against the CPU checker: the elementwise operations bit for bit, the critic / delayed actor /
target updates in lock step with the checker on the batches and noise draws of the reference's own run (tests/golden), and one update
at a wider shape with masks. fp32 tolerance of the updates: 1e-5 relative to the largest parameter (the contraction order differs)."""
import ctypes as C

import numpy as np
import pytest

import helpers
from helpers import rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-5


@pytest.mark.parametrize("B,A", [(1, 1), (100, 1), (4099, 6), (65537, 3)])
def test_elementwise_operations_bit_exact(oracle, rocm, B, A):
    print("case", B, A, flush=True)
    rng = np.random.default_rng(B + A)
    f32 = np.float32
    mean = rng.uniform(-1.2, 1.2, (B, A)).astype(f32); noise = rng.standard_normal((B, A)).astype(f32); dy = rng.standard_normal((B, A)).astype(f32)
    z = rng.standard_normal((B, A)).astype(f32); act = rng.uniform(-1, 1, (B, A)).astype(f32)
    q1, q2, r = (rng.standard_normal(B).astype(f32) for _ in range(3)); term = (rng.random(B) < 0.4).astype(np.uint8)
    res = {}
    for b in (oracle, rocm):
        m, n, d = b.array(mean), b.array(noise), b.array(dy)
        pc, out, out_eval, dx = b.zeros((B, A)), b.zeros((B, A)), b.zeros((B, A)), b.zeros((B, A))
        b.call("td3_sampling_forward", m.ptr, A, n.ptr, A, 0.3, pc.ptr, A, out.ptr, A, B, A)
        b.call("td3_sampling_forward", m.ptr, A, None, 0, 0.3, None, 0, out_eval.ptr, A, B, A)
        b.call("td3_sampling_backward", pc.ptr, A, d.ptr, A, dx.ptr, A, B, A)
        zz, tn = b.array(z), b.zeros((B, A))
        b.call("td3_target_action_noise", zz.ptr, 0.2, 0.5, tn.ptr, B * A)
        aa = b.array(act)
        b.call("td3_noisy_next_actions", aa.ptr, A, tn.ptr, A, B, A)
        a1, a2, ar, at, y, y_ignore = b.array(q1), b.array(q2), b.array(r), b.array(term), b.zeros((B,)), b.zeros((B,))
        b.call("td3_target_action_values", a1.ptr, a2.ptr, ar.ptr, at.ptr, 0.99, 0, y.ptr, B)
        b.call("td3_target_action_values", a1.ptr, a2.ptr, ar.ptr, at.ptr, 0.99, 1, y_ignore.ptr, B)
        b.sync()
        res[b.name] = dict(pre_clip=pc.numpy(), out=out.numpy(), out_eval=out_eval.numpy(), dx=dx.numpy(), target_noise=tn.numpy(), noisy=aa.numpy(),
                           y=y.numpy(), y_ignore=y_ignore.numpy())
    for k, want in res["oracle"].items():
        assert np.array_equal(res["rocm"][k], want), k


@pytest.mark.parametrize("per_operation", [1, 0])
def test_lock_step_with_the_checker_on_the_references_run(oracle, rocm, per_operation):
    """Both implementations of the updates: one launch per reference operation, and (the default for these shapes) the kernel that runs all
    network passes of an update in one launch, which fills only target_action_value and the sampling layer's pre_clip of the training buffers.
    The 36 loop steps of the committed reference run (72 critic updates, 18 delayed actor updates, 18 target updates of each kind).
    Before every step the HIP side gets the checker's exact state; both run the step on the reference's batch and draws; updated
    parameters of all six networks agree to 1e-5 of the largest parameter, gradients to 1e-5 of the largest gradient component times
    kappa = max|y| / max|Q - y| (rounding of Q is amplified by that factor in the TD error for any fp32 implementation)."""
    (batch, hidden, steps), hyper, g = helpers.td3_golden()
    ref = helpers.Td3OnBackend(oracle, batch, hidden, g["parameters_before"], hyper=hyper)
    dev = helpers.Td3OnBackend(rocm, batch, hidden, g["parameters_before"], hyper=hyper)
    worst_p = worst_g = 0.0
    rocm.call("sac_set_per_operation", per_operation)
    for i in range(steps):
        dev.push(ref.state())
        helpers.td3_golden_step(ref, g, i)
        try:
            helpers.td3_golden_step(dev, g, i)
        finally:
            rocm.call("sac_set_per_operation", 0)
        rocm.call("sac_set_per_operation", per_operation)
        pe = rel_err(dev.parameters(), ref.parameters())
        y, td = ref.target_q.numpy(), ref.d_out_c.numpy() * batch / 2
        kappa = max(1.0, np.abs(y).max() / max(np.abs(td).max(), 1e-30))
        ge = rel_err(dev.gradients(), ref.gradients()) / kappa
        assert np.array_equal(dev.ages(), ref.ages())
        assert rel_err(dev.target_q.numpy(), y) <= TOL and (not per_operation or rel_err(dev.nsavi.numpy(), ref.nsavi.numpy()) <= TOL)
        worst_p, worst_g = max(worst_p, pe), max(worst_g, ge)
        if i % 6 == 0:
            print(f"step {i}: parameters {pe:.2e} gradients/kappa {ge:.2e} kappa {kappa:.1f}", flush=True)
        assert pe <= TOL and ge <= TOL, (i, pe, ge)
    rocm.call("sac_set_per_operation", 0)
    # the checker itself reproduced the reference's parameters bit for bit on the way (the CPU suite asserts the same)
    assert np.array_equal(ref.parameters(), g[f"s{steps - 1}_after"])
    print("worst: parameters %.2e gradients %.2e" % (worst_p, worst_g))


def test_free_running_first_updates_match_the_reference_vectors(rocm):
    """No checker in the loop: the HIP side alone, from the reference's initial parameters, over the first two loop steps (4 critic
    updates, 1 actor update, both target updates) against the parameters the reference itself had after them."""
    (batch, hidden, _), hyper, g = helpers.td3_golden()
    dev = helpers.Td3OnBackend(rocm, batch, hidden, g["parameters_before"], hyper=hyper)
    for i in range(2):
        helpers.td3_golden_step(dev, g, i)
    assert rel_err(dev.parameters(), g["s1_after"]) <= TOL
    assert np.array_equal(helpers.td3_digest(dev.parameters(), hidden) != 0, np.ones((6, 2), bool))


@pytest.mark.parametrize("batch,hidden,obs,act,masks", [(256, 64, 3, 1, True), (1000, 256, 17, 6, True), (4096, 256, 17, 6, False)])
def test_one_update_at_other_shapes_with_masks(oracle, rocm, batch, hidden, obs, act, masks):
    """A full loop step (both critics, targets, actor, actor target) on random data at shapes beyond the Pendulum example, with final-step
    and next-final-step masks that clear a third of the rows, terminated flags, and samples outside [-1, 1]."""
    print("case", batch, hidden, obs, act, masks, flush=True)
    rng = np.random.default_rng(batch + act)
    D = obs + act
    adims, cdims = [obs, hidden, hidden, act], [D, hidden, hidden, 1]
    nets = [helpers.random_params(rng, adims)] * 2 + [helpers.random_params(rng, cdims) for _ in range(2)]
    params = np.concatenate(nets + [nets[2] * 0.9, nets[3] * 1.1]).astype(np.float32)
    oab = rng.standard_normal((2, batch, D)).astype(np.float32); oab[:, :, obs:] = np.clip(oab[:, :, obs:], -1, 1)
    rewards = rng.standard_normal(batch).astype(np.float32); term = (rng.random(batch) < 0.2).astype(np.uint8)
    tn = np.clip(rng.standard_normal((batch, act)) * 0.2, -0.5, 0.5).astype(np.float32)
    noises = [rng.standard_normal((batch, act)).astype(np.float32) for _ in range(3)]
    hyper = dict(gamma=0.99, actor_polyak=0.995, critic_polyak=0.99, sampling_std=0.5, adam=helpers.capi.adam_parameters(epsilon=1e-7))
    out = {}
    for b in (oracle, rocm):
        ag = helpers.Td3OnBackend(b, batch, hidden, params, hyper=hyper, masks=masks, obs=obs, act=act)
        if masks:
            ag.m_final.upload((rng.random(batch) < 0.67).astype(np.uint8) if b is oracle else out["oracle"]["m_final"])
            ag.m_next_final.upload((rng.random(batch) < 0.67).astype(np.uint8) if b is oracle else out["oracle"]["m_next"])
        ag.set_batch(oab, rewards, term, tn)
        ag.loop_step([1, 1, 1, 1], *noises)
        out[b.name] = dict(params=ag.parameters(), grads=ag.gradients(), nsavi=ag.nsavi.numpy(), savi=ag.savi.numpy(), y=ag.target_q.numpy(), d_c=ag.d_out_c.numpy(),
                           d_a=ag.d_out_a.numpy(), d_ci=ag.d_ci.numpy(), d_ao=ag.d_ao.numpy(), pre_clip=ag.pre_clip.numpy(), m_final=ag.m_final.numpy(), m_next=ag.m_next_final.numpy(),
                           critic_pre=np.concatenate([ag.critics[0].pre[0].numpy(), ag.critics[0].pre[1].numpy()], axis=1))
    want, got = out["oracle"], out["rocm"]
    assert (np.abs(want["pre_clip"]) > 1).sum() > batch * act // 20
    for k in ("nsavi", "savi", "y", "d_c", "d_a", "pre_clip"):
        e = rel_err(got[k], want[k])
        print(k, "%.2e" % e, flush=True)
        assert e <= TOL, (k, e)
    # The gradient that reaches the actor passes through critic 0's ReLUs. A pre-activation within rounding of zero may switch on one
    # side only, which changes that row's input gradient by O(1): such rows are allowed if the checker's pre-activation shows the
    # near-zero unit, and the quantities summed over the batch are then compared with that many rows' worth of slack.
    scale = np.abs(want["d_ci"]).max()
    row_err = np.abs(got["d_ci"] - want["d_ci"]).max(axis=1) / scale
    bad = np.nonzero(row_err > TOL)[0]
    print("rows of d_critic_input beyond tolerance:", bad.size, flush=True)
    assert bad.size <= 3
    for r in bad:
        assert np.abs(want["critic_pre"][r]).min() <= 1e-5 * np.abs(want["critic_pre"]).max(), (r, row_err[r])
    ok = np.ones(batch, bool); ok[bad] = False
    assert rel_err(got["d_ci"][ok], want["d_ci"][ok]) <= TOL and rel_err(got["d_ao"][ok], want["d_ao"][ok]) <= TOL
    slack = TOL + 2.0 * bad.size / batch
    for k in ("grads", "params"):
        e = rel_err(got[k], want[k])
        print(k, "%.2e" % e, flush=True)
        assert e <= slack, (k, e)


FUSED_SHAPES = [  # batch, obs, act, hidden activation
    (256, 3, 1, "relu"),        # Pendulum
    (256, 27, 8, "relu"),       # two input tiles, the widest action
    (100, 17, 6, "tanh"),       # batch that is no multiple of 16
    (1, 5, 2, "relu"),
    (300, 111, 8, "fast_tanh"), # wide observations: the 128-input variant of the kernel
]


@pytest.mark.parametrize("batch,obs,act,hidden_act", FUSED_SHAPES)
def test_fused_updates_match_the_checker_and_the_per_operation_path(oracle, rocm, batch, obs, act, hidden_act):
    """The one-launch updates (rl/algorithms/td3/operations_generic.h:170-281 for actors obs -> 64 -> 64 -> act with tanh output and critics
    obs + act -> 64 -> 64 -> 1): three loop steps (both critics, targets, actor, actor target each) from identical parameters, batches and noise
    against the checker and against the one-launch-per-operation path; samples beyond [-1, 1] and terminated rows included. 1e-5 relative to
    each tensor's largest magnitude."""
    fused_against_checker_and_per_operation(oracle, rocm, batch, obs, act, hidden_act, 64)


@pytest.mark.parametrize("batch,obs,act,hidden,hidden_act", [(256, 6, 1, 256, "fast_tanh"), (100, 17, 6, 128, "relu"), (48, 3, 1, 200, "relu"), (256, 27, 8, 256, "relu"),
                                                             (30, 111, 8, 72, "tanh"), (512, 5, 2, 16, "sigmoid")])
def test_wider_agents_match_the_checker_on_both_paths(oracle, rocm, batch, obs, act, hidden, hidden_act):
    """The same at hidden widths other than 64 (up to 256; the kernel that takes 16 rows per workgroup of sixteen wavefronts through every pass, with the
    optimiser's launch adding up the workgroups' partial sums): the shapes that the SAC updates are tested at."""
    fused_against_checker_and_per_operation(oracle, rocm, batch, obs, act, hidden_act, hidden)


def fused_against_checker_and_per_operation(oracle, rocm, batch, obs, act, hidden_act, hidden):
    rng = np.random.default_rng(batch * 7 + obs)
    D = obs + act
    adims, cdims = [obs, hidden, hidden, act], [D, hidden, hidden, 1]
    nets = [helpers.random_params(rng, adims)] * 2 + [helpers.random_params(rng, cdims) for _ in range(2)]
    params = np.concatenate(nets + [nets[2] * 0.9, nets[3] * 1.1]).astype(np.float32)
    hyper = dict(gamma=0.99, actor_polyak=0.995, critic_polyak=0.99, sampling_std=0.5, adam=helpers.capi.adam_parameters(epsilon=1e-7))
    steps = []
    for _ in range(3):
        oab = rng.standard_normal((2, batch, D)).astype(np.float32); oab[:, :, obs:] = np.clip(oab[:, :, obs:], -1, 1)
        steps.append((oab, rng.standard_normal(batch).astype(np.float32), (rng.random(batch) < 0.2).astype(np.uint8),
                      np.clip(rng.standard_normal((batch, act)) * 0.2, -0.5, 0.5).astype(np.float32), [rng.standard_normal((batch, act)).astype(np.float32) for _ in range(3)]))
    out = {}
    for name, b, per_operation in (("checker", oracle, None), ("fused", rocm, 0), ("per_operation", rocm, 1)):
        ag = helpers.Td3OnBackend(b, batch, hidden, params, hyper=hyper, masks=False, obs=obs, act=act, hidden_act=hidden_act)
        if per_operation is not None:
            rocm.call("sac_set_per_operation", per_operation)
        try:
            for oab, rewards, term, tn, noises in steps:
                ag.set_batch(oab, rewards, term, tn)
                ag.loop_step([1, 1, 1, 1], *noises)
        finally:
            rocm.call("sac_set_per_operation", 0)
        out[name] = dict(params=ag.parameters(), grads=ag.gradients(), y=ag.target_q.numpy(), pre_clip=ag.pre_clip.numpy(), ages=ag.ages(), nsavi=ag.nsavi.numpy())
    # which path ran: only the per-operation launches fill the critics' next-input buffer
    assert not out["fused"].pop("nsavi").any() and out["per_operation"].pop("nsavi").any() and out["checker"].pop("nsavi").any()
    assert (np.abs(out["checker"]["pre_clip"]) > 1).sum() >= batch * act // 50
    for other in ("checker", "per_operation"):
        for key, ref in out[other].items():
            err = rel_err(out["fused"][key], ref)
            assert err <= TOL, (other, key, err)
    assert np.abs(out["fused"]["params"] - params).max() > 1e-4


@pytest.mark.parametrize("batch,obs,act,hidden,hidden_act", [(256, 27, 8, 256, "relu"), (100, 6, 1, 256, "relu"), (48, 3, 1, 200, "tanh"), (256, 3, 1, 64, "relu")])
def test_both_critics_in_one_call_leave_the_bits_of_the_two_calls(rocm, batch, obs, act, hidden, hidden_act):
    """rlt_rocm_td3_train_critics against rlt_rocm_td3_train_critic for critic 0 and then critic 1 on the same batch and target noise, each critic with its own sampling
    noise: three loop steps from the same parameters; every parameter, the gradients, the optimisers' ages and the target values (the second critic's), bit for bit.
    Both updates run as one launch (at width 64 in the update kernel for that width, beyond it in the one for widths up to 256)."""
    rng = np.random.default_rng(batch + hidden)
    D = obs + act
    adims, cdims = [obs, hidden, hidden, act], [D, hidden, hidden, 1]
    nets = [helpers.random_params(rng, adims)] * 2 + [helpers.random_params(rng, cdims) for _ in range(2)]
    params = np.concatenate(nets + [nets[2] * 0.9, nets[3] * 1.1]).astype(np.float32)
    hyper = dict(gamma=0.99, actor_polyak=0.995, critic_polyak=0.99, sampling_std=0.5, adam=helpers.capi.adam_parameters(epsilon=1e-7))
    agents = [helpers.Td3OnBackend(rocm, batch, hidden, params, hyper=hyper, masks=False, obs=obs, act=act, hidden_act=hidden_act) for _ in range(2)]
    for step in range(3):
        oab = rng.standard_normal((2, batch, D)).astype(np.float32); oab[:, :, obs:] = np.clip(oab[:, :, obs:], -1, 1)
        rewards, term = rng.standard_normal(batch).astype(np.float32), (rng.random(batch) < 0.2).astype(np.uint8)
        tn = np.clip(rng.standard_normal((batch, act)) * 0.2, -0.5, 0.5).astype(np.float32)
        noises = [rng.standard_normal((batch, act)).astype(np.float32) for _ in range(3)]
        for ag, together in zip(agents, (False, True)):
            ag.set_batch(oab, rewards, term, tn)
            ag.loop_step([1, 1, 1, 1], *noises, both_critics_in_one_call=together)
        for what in ("parameters", "gradients", "ages"):
            a, b = (getattr(ag, what)() for ag in agents)
            assert np.array_equal(a, b), (step, what)
        assert np.array_equal(agents[0].target_q.numpy(), agents[1].target_q.numpy()), step
    assert np.abs(agents[1].parameters() - params).max() > 1e-4



@pytest.mark.parametrize("batch,obs,act,hidden,hidden_act", [(256, 27, 8, 256, "relu"), (100, 6, 1, 256, "relu"), (48, 3, 2, 200, "tanh"), (256, 3, 1, 64, "relu")])
def test_updates_with_their_draws_leave_the_bits_of_the_separate_calls(rocm, batch, obs, act, hidden, hidden_act):
    """rlt_rocm_td3_train_critics_drawn and rlt_rocm_td3_train_actor_drawn (the smoothing noise and the sampling noises drawn by the library, inside the update's launch
    at hidden widths beyond 64) against rlt_rocm_randn_f32 on the same streams, rlt_rocm_td3_target_action_noise, rlt_rocm_td3_train_critics and _train_actor: three
    loop steps from the same parameters (in the second the drawn call also makes update_critic_targets); the smoothing noise left in the agent's buffer, every parameter, the gradients, the optimisers' ages and the target values,
    bit for bit."""
    rng = np.random.default_rng(7 * batch + hidden)
    D, count = obs + act, batch * act
    adims, cdims = [obs, hidden, hidden, act], [D, hidden, hidden, 1]
    nets = [helpers.random_params(rng, adims)] * 2 + [helpers.random_params(rng, cdims) for _ in range(2)]
    params = np.concatenate(nets + [nets[2] * 0.9, nets[3] * 1.1]).astype(np.float32)
    hyper = dict(gamma=0.99, actor_polyak=0.995, critic_polyak=0.99, sampling_std=0.5, adam=helpers.capi.adam_parameters(epsilon=1e-7))
    agents = [helpers.Td3OnBackend(rocm, batch, hidden, params, hyper=hyper, masks=False, obs=obs, act=act, hidden_act=hidden_act) for _ in range(2)]
    seed, std, clip = 1234, 0.2, 0.25         # the clamp reaches one draw in five
    for step in range(3):
        oab = rng.standard_normal((2, batch, D)).astype(np.float32); oab[:, :, obs:] = np.clip(oab[:, :, obs:], -1, 1)
        rewards, term = rng.standard_normal(batch).astype(np.float32), (rng.random(batch) < 0.2).astype(np.uint8)
        streams = [10 * step + k for k in range(4)]
        for ag, drawn in zip(agents, (False, True)):
            ag.set_batch(oab, rewards, term, np.zeros((batch, act), np.float32))
            noise = rocm.zeros((3, batch, act))
            if drawn:
                draws = helpers.capi.Td3CriticDraws(seed, streams[0], (C.c_uint64 * 2)(streams[1], streams[2]), std, clip)
                rocm.call("td3_train_critics_drawn", C.byref(ag.c), C.byref(draws), noise.ptr, step % 2)
                if step % 2 == 0:
                    rocm.call("td3_update_critic_targets", C.byref(ag.c))
                rocm.call("td3_train_actor_drawn", C.byref(ag.c), seed, streams[3], noise.ptr)
            else:
                rocm.call("randn_f32", ag.target_noise.ptr, count, seed, streams[0])
                rocm.call("td3_target_action_noise", ag.target_noise.ptr, std, clip, ag.target_noise.ptr, count)
                for k in range(3):
                    rocm.call("randn_f32", noise.ptr + 4 * count * k, count, seed, streams[1 + k])
                rocm.call("td3_train_critics", C.byref(ag.c), noise.ptr, noise.ptr + 4 * count)
                rocm.call("td3_update_critic_targets", C.byref(ag.c))
                rocm.call("td3_train_actor", C.byref(ag.c), noise.ptr + 8 * count)
            rocm.call("td3_update_actor_target", C.byref(ag.c))
            rocm.sync()
        assert np.array_equal(agents[0].target_noise.numpy(), agents[1].target_noise.numpy()), step
        assert np.abs(agents[1].target_noise.numpy()).max() == np.float32(clip)
        for what in ("parameters", "gradients", "ages"):
            a, b = (getattr(ag, what)() for ag in agents)
            assert np.array_equal(a, b), (step, what)
        assert np.array_equal(agents[0].target_q.numpy(), agents[1].target_q.numpy()), step
    assert np.abs(agents[1].parameters() - params).max() > 1e-4
