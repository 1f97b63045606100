"""PPO on the GPU through the C ABI against the CPU checker and against vectors written by the real reference.

fp32 tolerance: 1e-5 relative to the largest magnitude of the tensor compared, for single operations; after a sequence of Adam
updates the parameters are compared to 2e-4 of their largest magnitude (Adam divides by sqrt(v): a rounding-level difference in a
near-zero gradient moves that parameter by up to the learning rate)."""
import ctypes as C

import numpy as np
import pytest

import helpers
from helpers import rel_err
from test_oracle_golden import ppo_golden_setup

pytestmark = pytest.mark.gpu
TOL = 1e-5


@pytest.mark.parametrize("batch,action_dim", [(64, 1), (1000, 8), (8192, 8), (300, 33)])
@pytest.mark.parametrize("normalize,learn_std", [(1, 1), (0, 1), (1, 0)])
def test_surrogate_gradient_matches_checker(oracle, rocm, batch, action_dim, normalize, learn_std):
    print("case", batch, action_dim, normalize, learn_std, flush=True)
    capi = helpers.capi
    rng = np.random.default_rng(batch + action_dim)
    means = rng.standard_normal((batch, action_dim)).astype(np.float32)
    log_std = (0.3 * rng.standard_normal(action_dim)).astype(np.float32)
    actions = (means + np.exp(log_std) * rng.standard_normal((batch, action_dim))).astype(np.float32)
    # rollout log-probabilities near the current ones, so that ratios straddle the clipping range on both sides
    z = (actions - means) / np.exp(log_std)
    lp_now = (-0.9189385332046727 - log_std - 0.5 * z * z).sum(1)
    log_probs = (lp_now + 0.3 * rng.standard_normal(batch)).astype(np.float32)
    advantages = (3.0 * rng.standard_normal(batch) + 0.5).astype(np.float32)
    pp = capi.ppo_parameters(0.2, 0.01, 1e-8, normalize, learn_std)
    res = []
    for b in (oracle, rocm):
        d_means, d_ls = b.zeros((batch, action_dim)), b.array(np.full(action_dim, 0.25 if not learn_std else 0.0, np.float32))
        m_, ls_, a_, lp_, adv_ = (b.array(x) for x in (means, log_std, actions, log_probs, advantages))     # named: the arrays must outlive the call
        b.call("ppo_surrogate_gradient", m_.ptr, action_dim, ls_.ptr, a_.ptr, action_dim, lp_.ptr, 1, adv_.ptr, 1, C.byref(pp), d_means.ptr, action_dim,
               d_ls.ptr if learn_std else None, batch, action_dim)
        b.sync()
        res.append((d_means.numpy(), d_ls.numpy()))
    ratio = np.exp(lp_now - log_probs)
    assert (ratio > 1.2).any() and (ratio < 0.8).any() and ((ratio > 0.8) & (ratio < 1.2)).any()     # all three branches occur
    assert rel_err(res[1][0], res[0][0]) <= TOL
    if learn_std:
        # The reference (and the checker, bit for bit) adds 2 * batch terms one by one into a single fp32 accumulator per action dimension,
        # which carries a rounding error of up to batch * 2^-24 of the running magnitude; the kernel sums in a tree. The bound is that error.
        scale = max(np.abs(res[0][1]).max(), np.abs(advantages).max() / batch * 4)
        assert np.abs(res[1][1] - res[0][1]).max() <= batch * 2.0 ** -24 * scale, (np.abs(res[1][1] - res[0][1]).max(), batch * 2.0 ** -24 * scale)
    else:
        assert np.array_equal(res[1][1], np.full(action_dim, 0.25, np.float32))


@pytest.mark.parametrize("B,N,updates", [(512, 4096, 8), (8192, 32768, 3)])
def test_train_minibatch_matches_checker_on_synthetic_dataset(oracle, rocm, B, N, updates):
    """The shape of the synthetic PPO benchmark (observation 105, action 8, hidden 64, tanh) at minibatch 512 and at the benchmark's own 8,192:
    one update compared tensor by tensor, then several updates on shuffled rows compared at the end."""
    capi = helpers.capi
    O, A, H = 105, 8, 64
    rng = np.random.default_rng(2)
    na, nc = helpers.mlp_param_count([O, H, H, A]), helpers.mlp_param_count([O, H, H, 1])
    params = np.concatenate([helpers.random_params(rng, [O, H, H, A]), np.log(np.full(A, 0.5, np.float32)), helpers.random_params(rng, [O, H, H, 1])])
    ld = O + 2 * A + 8
    data = rng.standard_normal((N, ld)).astype(np.float32)
    col = dict(observations=0, actions=O + A, action_log_probs=O + 2 * A, advantages=O + 2 * A + 6, target_values=O + 2 * A + 7)
    pp = capi.ppo_parameters()
    perm = rng.permutation(N).astype(np.uint32)
    # rollout log-probabilities consistent with the dataset's actions under the initial policy (plus noise), so that ratios sit around 1
    net = helpers.Mlp(oracle, [O, H, H, A], params[:na], N, "tanh", trainable=False)
    out = oracle.zeros((N, A))
    data0 = oracle.array(data)
    oracle.call("mlp_evaluate", net.layers, net.n, data0.offset(0), ld, out.ptr, A, N, None, 0)
    z = (data[:, col["actions"]:col["actions"] + A] - out.numpy()) / 0.5
    data[:, col["action_log_probs"]] = (-0.9189385332046727 - np.log(0.5) - 0.5 * z * z).sum(1) + 0.2 * rng.standard_normal(N).astype(np.float32)
    results = []
    for b in (oracle, rocm):
        agent = helpers.PpoOnBackend(b, O, A, H, H, B, params, "tanh", "tanh", capi.adam_parameters(3e-4, epsilon=1e-8))
        dd, idx, loss = b.array(data), b.array(perm), b.zeros((1,))
        args = (dd.offset(col["observations"]), dd.offset(col["observations"]), dd.offset(col["actions"]), dd.offset(col["action_log_probs"]),
                dd.offset(col["advantages"]), dd.offset(col["target_values"]), ld)
        b.call("ppo_train_minibatch", C.byref(agent.c), C.byref(pp), *args, None, loss.ptr)
        b.sync()
        first = dict(actor_grads=agent.actor.grads.numpy(), critic_grads=agent.critic.grads.numpy(), d_log_std=agent.d_log_std.numpy(), loss=loss.numpy(),
                     params=agent.parameters())
        for k in range(updates):
            b.call("ppo_train_minibatch", C.byref(agent.c), C.byref(pp), *args, idx.offset(k * B), loss.ptr)
        b.sync()
        results.append((first, agent.parameters(), loss.numpy()))
    (f0, p0, l0), (f1, p1, l1) = results
    for key in f0:
        # d_log_std: the reference (and the checker, bit for bit) adds 2 * batch terms one by one into a single fp32 accumulator per action dimension,
        # which carries a rounding error of up to batch * 2^-24 of the running magnitude; the kernel sums in a tree
        bound = max(TOL, B * 2.0 ** -24) if key == "d_log_std" else TOL
        assert rel_err(f1[key], f0[key]) <= bound, (key, rel_err(f1[key], f0[key]))
    assert rel_err(p1, p0) <= 2e-4 and rel_err(l1, l0) <= 1e-4


def test_sums_per_xcd_and_sums_by_the_optimiser_agree(rocm):
    """At 8,192 rows the minibatch kernel's 256 workgroups add their partial gradient sums up per XCD inside the launch (eight blocks per network
    are left for the optimiser's launch); with that switched off (rlt_rocm_set_update_options) the optimiser's launch adds up all 128 blocks per
    network. The two orders of summation differ in the last bits only."""
    capi = helpers.capi
    O, A, H, B = 105, 8, 64, 8192
    rng = np.random.default_rng(6)
    params = np.concatenate([helpers.random_params(rng, [O, H, H, A]), np.log(np.full(A, 0.5, np.float32)), helpers.random_params(rng, [O, H, H, 1])])
    ld = O + A + 3
    data = rng.standard_normal((B, ld)).astype(np.float32)
    data[:, O + A] = -A * 1.5 + 0.3 * rng.standard_normal(B).astype(np.float32)
    pp = capi.ppo_parameters()
    results = []
    for in_kernel in (1, 0):
        rocm.call("set_update_options", in_kernel, 1)
        try:
            agent = helpers.PpoOnBackend(rocm, O, A, H, H, B, params, "tanh", "tanh", capi.adam_parameters(3e-4, epsilon=1e-8))
            dd, loss = rocm.array(data), rocm.zeros((1,))
            for _ in range(3):
                rocm.call("ppo_train_minibatch", C.byref(agent.c), C.byref(pp), dd.offset(0), dd.offset(0), dd.offset(O), dd.offset(O + A), dd.offset(O + A + 1),
                          dd.offset(O + A + 2), ld, None, loss.ptr)
            rocm.sync()
            results.append((agent.actor.grads.numpy(), agent.critic.grads.numpy(), agent.d_log_std.numpy(), agent.parameters(), loss.numpy()))
        finally:
            rocm.call("set_update_options", 1, 1)
    for a, b in zip(*results):
        assert rel_err(a, b) <= 2e-5, rel_err(a, b)
    assert int(agent.actor.age.numpy()[0]) == 4 and int(agent.critic.age.numpy()[0]) == 4


@pytest.mark.parametrize("O,A,H,B,act", [(105, 8, 64, 512, "tanh"), (3, 1, 64, 200, "tanh"), (17, 6, 256, 300, "tanh"), (3, 1, 32, 256, "fast_tanh"), (11, 2, 16, 128, "tanh"),
                                         (5, 3, 48, 96, "relu")])
def test_train_minibatch_with_standardize_layers_matches_checker(oracle, rocm, O, A, H, B, act):
    """Standardize layers in front of actor and critic (the loop's approximators, rl/algorithms/ppo/loop/core/config.h:51-83): the networks
    read (x - mean) * precision, the factor only where it is not 0 (nn/layers/standardize/operations_generic.h:68-86). Hidden width 64 takes
    the kernel that reads the dataset rows itself, widths below 64 the same kernel on zero-padded copies of the parameters (the zoo's PPO configuration of
    the Pendulum is width 32 with fast_tanh), 256 the packed minibatch; four updates on shuffled rows, compared tensor by tensor after the first and at
    the end. The third observation column has precision 0."""
    capi = helpers.capi
    N = 4 * B
    rng = np.random.default_rng(O * 7 + A)
    params = np.concatenate([helpers.random_params(rng, [O, H, H, A]), np.log(np.full(A, 0.5, np.float32)), helpers.random_params(rng, [O, H, H, 1])])
    ld = O + 2 * A + 8
    data = (rng.standard_normal((N, ld)) * 3 + 1.5).astype(np.float32)
    col = dict(observations=0, actions=O + A, action_log_probs=O + 2 * A, advantages=O + 2 * A + 6, target_values=O + 2 * A + 7)
    data[:, col["action_log_probs"]] = -A * 1.5 + 0.3 * rng.standard_normal(N).astype(np.float32)
    data[:, col["actions"]:col["actions"] + A] = rng.standard_normal((N, A)).astype(np.float32)
    standardize = [rng.standard_normal(O) * 0.5 + 1.5, 1.0 / (2.0 + rng.random(O)), rng.standard_normal(O) * 0.5 + 1.5, 1.0 / (2.0 + rng.random(O))]
    standardize[1][2 % O] = 0.0
    perm = rng.permutation(N).astype(np.uint32)
    pp = capi.ppo_parameters()
    results = []
    for b in (oracle, rocm):
        agent = helpers.PpoOnBackend(b, O, A, H, H, B, params, act, act, capi.adam_parameters(3e-4, epsilon=1e-8), standardize=standardize)
        dd, idx, loss = b.array(data), b.array(perm), b.zeros((1,))
        args = (dd.offset(col["observations"]), dd.offset(col["observations"]), dd.offset(col["actions"]), dd.offset(col["action_log_probs"]),
                dd.offset(col["advantages"]), dd.offset(col["target_values"]), ld)
        b.call("ppo_train_minibatch", C.byref(agent.c), C.byref(pp), *args, None, loss.ptr)
        b.sync()
        first = dict(actor_grads=agent.actor.grads.numpy(), critic_grads=agent.critic.grads.numpy(), d_log_std=agent.d_log_std.numpy(), loss=loss.numpy())
        for k in range(4):
            b.call("ppo_train_minibatch", C.byref(agent.c), C.byref(pp), *args, idx.offset(k * B), loss.ptr)
        b.sync()
        results.append((first, agent.parameters(), loss.numpy()))
    (f0, p0, l0), (f1, p1, l1) = results
    for key in f0:
        assert rel_err(f1[key], f0[key]) <= TOL, (key, rel_err(f1[key], f0[key]))
    assert rel_err(p1, p0) <= 2e-4 and rel_err(l1, l0) <= 1e-4
    # the layers matter: without them the first update's gradients differ
    plain = helpers.PpoOnBackend(rocm, O, A, H, H, B, params, act, act, capi.adam_parameters(3e-4, epsilon=1e-8))
    dd, loss = rocm.array(data), rocm.zeros((1,))
    rocm.call("ppo_train_minibatch", C.byref(plain.c), C.byref(pp), dd.offset(0), dd.offset(0), dd.offset(col["actions"]), dd.offset(col["action_log_probs"]),
              dd.offset(col["advantages"]), dd.offset(col["target_values"]), ld, None, loss.ptr)
    rocm.sync()
    assert rel_err(plain.critic.grads.numpy(), f0["critic_grads"]) > 1e-2


@pytest.mark.parametrize("normalize", [1, 0])
def test_train_epoch_matches_checker_and_minibatch_calls(oracle, rocm, normalize):
    """One epoch call (advantage statistics of all minibatches formed up front, 40 minibatches = two chunks of that) against the checker's batch
    loop and against the same minibatches issued one call at a time; ragged minibatch size, losses per minibatch."""
    capi = helpers.capi
    O, A, H, B, NMB = 105, 8, 64, 200, 40
    N = B * NMB
    rng = np.random.default_rng(9)
    na = helpers.mlp_param_count([O, H, H, A])
    params = np.concatenate([helpers.random_params(rng, [O, H, H, A]), np.log(np.full(A, 0.5, np.float32)), helpers.random_params(rng, [O, H, H, 1])])
    ld = O + 2 * A + 8
    data = rng.standard_normal((N, ld)).astype(np.float32)
    col = dict(observations=0, actions=O + A, action_log_probs=O + 2 * A, advantages=O + 2 * A + 6, target_values=O + 2 * A + 7)
    net = helpers.Mlp(oracle, [O, H, H, A], params[:na], N, "tanh", trainable=False)
    out, data0 = oracle.zeros((N, A)), oracle.array(data)
    oracle.call("mlp_evaluate", net.layers, net.n, data0.offset(0), ld, out.ptr, A, N, None, 0)
    z = (data[:, col["actions"]:col["actions"] + A] - out.numpy()) / 0.5
    data[:, col["action_log_probs"]] = (-0.9189385332046727 - np.log(0.5) - 0.5 * z * z).sum(1) + 0.2 * rng.standard_normal(N).astype(np.float32)
    perm = rng.permutation(N).astype(np.uint32)
    pp = capi.ppo_parameters()
    pp.normalize_advantage = normalize
    results = []
    for b, epoch_call in ((oracle, True), (rocm, True), (rocm, False)):
        agent = helpers.PpoOnBackend(b, O, A, H, H, B, params, "tanh", "tanh", capi.adam_parameters(3e-4, epsilon=1e-8))
        dd, idx, losses = b.array(data), b.array(perm), b.zeros((NMB,))
        args = (dd.offset(col["observations"]), dd.offset(col["observations"]), dd.offset(col["actions"]), dd.offset(col["action_log_probs"]),
                dd.offset(col["advantages"]), dd.offset(col["target_values"]), ld)
        if epoch_call:
            b.call("ppo_train_epoch", C.byref(agent.c), C.byref(pp), *args, idx.ptr, NMB, losses.ptr)
        else:
            for k in range(NMB):
                b.call("ppo_train_minibatch", C.byref(agent.c), C.byref(pp), *args, idx.offset(k * B), losses.offset(k))
        b.sync()
        results.append((agent.parameters(), losses.numpy(), agent.d_log_std.numpy()))
    want, got, single = results
    assert np.array_equal(got[0], single[0]) and np.array_equal(got[1], single[1])        # the same kernels on the same statistics: bitwise
    assert rel_err(got[0], want[0]) <= 2e-4 and rel_err(got[1], want[1]) <= 1e-4 and rel_err(got[2], want[2]) <= 1e-3


def test_ppo_against_reference_vectors(rocm):
    """GAE bit-exact structure aside (fp32, same operation order per environment), the 30 minibatch updates of two loop steps reproduce the
    reference's parameters; the dataset, permutations and parameters come from the reference's own run (tests/golden/ppo_pendulum_seed0.npz)."""
    g, agent, pp, hy, col, d = ppo_golden_setup(rocm)
    for step in range(2):
        data = g[f"s{step}_dataset"]
        dd = rocm.array(data)
        adv, tgt = rocm.zeros(data.shape), rocm.zeros(data.shape)
        rocm.call("ppo_gae", dd.offset(col["rewards"]), dd.offset(col["terminated"]), dd.offset(col["truncated"]), dd.offset(col["all_values"]), adv.ptr, tgt.ptr,
                  d["data_dim"], d["n_envs"], d["steps"], hy["gamma"], hy["lambda"], 0)
        rocm.sync()
        assert rel_err(adv.numpy()[:d["n"], 0], data[:d["n"], col["advantages"]]) <= TOL and rel_err(tgt.numpy()[:d["n"], 0], data[:d["n"], col["target_values"]]) <= TOL
        # each loop step starts from the reference's own parameters (the optimiser moments carry over inside the agent)
        losses = helpers.ppo_train_like_reference(rocm, agent, pp, dd, d["data_dim"], col, d["n"], g[f"s{step}_permutations"], d["batch"])
        assert np.all(np.isfinite(losses))
        got, want = agent.parameters(), g[f"s{step}_after"]
        assert rel_err(got, want) <= 2e-4, (step, rel_err(got, want))


def test_ppo_learns_the_pendulum_end_to_end_on_the_device(rocm):
    """Collection, critic values, GAE and the epoch of minibatch updates chained on the device for 400 iterations (3.3 M environment steps) with the
    hyperparameters of the reference's Pendulum configuration: the mean return of 100 evaluation episodes must rise from below -900 to above -300
    The CPU checker driven by the same draws (160 s for 300 iterations) follows the same curve: -1050, -970, -948, -968, -823, -570, -411, -433,
    -343, -252, -183, -257 every 25 iterations, against -1124, -1056, -981, -980, -760, -609, -429, -415, -332, -231, -222, -215 on the device."""
    returns = helpers.ppo_pendulum_loop(rocm, 400, seed=0, log=False)
    print("mean evaluation returns every 25 iterations", [round(r) for r in returns], flush=True)
    assert returns[0] < -900 and max(returns[-4:]) > -300, returns
