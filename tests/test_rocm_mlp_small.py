"""Single-pass forward + backward kernel for in -> 64 -> 64 -> out networks (one 16-row tile per wavefront), through the C ABI.

Checked against the CPU checker at sizes it finishes in seconds (all three loss epilogues: given gradient, MSE target, PPO's
clipped surrogate via the minibatch update), against the per-layer kernels of the same library at the benchmark size, and through
properties that hold at any size (accumulation with beta = 1, linearity of the gradients in the upstream gradient).

Tolerance: 1e-5 relative to the largest magnitude of the reference tensor (fp32)."""
import ctypes as C

import numpy as np
import pytest

import helpers
from helpers import Mlp, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-5


def run(backend, dims, params, x, dy, ha, oa, use_target, scale, repeat=1, want_y=True):
    B = x.shape[0]
    net = Mlp(backend, dims, params, B, ha, oa)
    xd, yd, dyd = backend.array(x), backend.zeros((B, dims[-1])), backend.array(dy)
    ws, wsn = net.workspace()
    backend.call("mlp_zero_gradient", net.layers, net.n)
    for _ in range(repeat):
        if use_target:
            backend.call("mlp_forward_backward", net.layers, net.n, xd.ptr, dims[0], yd.ptr if want_y else None, dims[-1], None, 0, dyd.ptr, dims[-1], scale, B, ws, wsn)
        else:
            backend.call("mlp_forward_backward", net.layers, net.n, xd.ptr, dims[0], yd.ptr if want_y else None, dims[-1], dyd.ptr, dims[-1], None, 0, 0.0, B, ws, wsn)
    backend.sync()
    return yd.numpy(), net.grads.numpy(), net.offsets


# (batch, in, out, hidden activation, output activation, MSE target instead of a given gradient)
CASES = [(512, 105, 8, "tanh", "identity", False), (512, 105, 1, "tanh", "identity", True), (256, 3, 1, "relu", "identity", False),
         (256, 4, 1, "relu", "identity", True), (1000, 3, 2, "relu", "tanh", False), (37, 128, 16, "fast_tanh", "sigmoid", False),
         (1, 17, 6, "relu", "identity", False), (16, 16, 4, "tanh", "tanh", True), (17, 65, 5, "relu", "relu", False), (4100, 33, 9, "relu", "identity", True)]


@pytest.mark.parametrize("case", CASES)
def test_narrow_forward_backward_matches_checker(oracle, rocm, case):
    print("case", case, flush=True)
    B, I, O, ha, oa, use_target = case
    dims = [I, 64, 64, O]
    rng = np.random.default_rng(B * 131 + I)
    params = helpers.random_params(rng, dims)
    x = rng.standard_normal((B, I)).astype(np.float32); dy = rng.standard_normal((B, O)).astype(np.float32)
    scale = 1.0 / B
    want, got = run(oracle, dims, params, x, dy, ha, oa, use_target, scale), run(rocm, dims, params, x, dy, ha, oa, use_target, scale)
    assert rel_err(got[0], want[0]) <= TOL
    if ha == "relu" and rel_err(got[1], want[1]) > TOL:
        # a hidden unit whose pre-activation rounds to the other side of zero switches a whole row's contribution; accept only if the
        # checker's own pre-activations come that close to zero
        net = Mlp(oracle, dims, params, B, ha, oa)
        xd = oracle.array(x)
        oracle.call("mlp_forward", net.layers, net.n, xd.ptr, I, B)
        near = min(np.abs(net.pre[0].numpy()).min(), np.abs(net.pre[1].numpy()).min())
        assert near <= 1e-6, (near, rel_err(got[1], want[1]))
        return
    for (off, nw, nb) in want[2]:
        ew = rel_err(got[1][off:off + nw], want[1][off:off + nw]); eb = rel_err(got[1][off + nw:off + nw + nb], want[1][off + nw:off + nw + nb])
        assert ew <= TOL and eb <= TOL, (off, ew, eb)


def test_narrow_accumulates_and_skips_null_output(rocm):
    dims = [105, 64, 64, 8]
    rng = np.random.default_rng(5)
    params = helpers.random_params(rng, dims)
    x = rng.standard_normal((300, 105)).astype(np.float32); dy = rng.standard_normal((300, 8)).astype(np.float32)
    once = run(rocm, dims, params, x, dy, "tanh", "identity", False, 0.0, repeat=1)
    twice = run(rocm, dims, params, x, dy, "tanh", "identity", False, 0.0, repeat=2, want_y=False)
    assert rel_err(twice[1], 2.0 * once[1]) <= 1e-6          # beta = 1: a second call adds the same gradient again
    assert np.all(twice[0] == 0.0)                            # y == NULL: nothing written


@pytest.mark.parametrize("case", [(8192, 105, 8, "tanh"), (65536, 3, 1, "relu"), (50000, 105, 1, "fast_tanh")])
def test_narrow_full_size_against_per_layer_kernels_and_linearity(rocm, monkeypatch, case):
    """Benchmark-sized minibatches: against the per-layer kernels of the same library (checked against the checker at small sizes), bitwise
    repeatability (fixed summation order), and linearity of the gradients in the upstream gradient."""
    print("case", case, flush=True)
    B, I, O, ha = case
    dims = [I, 64, 64, O]
    rng = np.random.default_rng(B + I)
    params = helpers.random_params(rng, dims)
    x = rng.standard_normal((B, I)).astype(np.float32); dy = (rng.standard_normal((B, O)) / B).astype(np.float32)
    y, g, offsets = run(rocm, dims, params, x, dy, ha, "identity", False, 0.0)
    y_again, g_again, _ = run(rocm, dims, params, x, dy, ha, "identity", False, 0.0)
    assert np.array_equal(g, g_again) and np.array_equal(y, y_again)
    _, g3, _ = run(rocm, dims, params, x, 3.0 * dy, ha, "identity", False, 0.0)
    assert rel_err(g3, 3.0 * g) <= 1e-6
    monkeypatch.setenv("RLT_MLP_SINGLE_PASS", "0")
    y2, g2, _ = run(rocm, dims, params, x, dy, ha, "identity", False, 0.0)
    assert rel_err(y, y2) <= TOL
    slack = 20 * TOL if ha == "relu" else TOL     # relu: a few of the 65,536 rows may sit on a switch point of a hidden unit
    for (off, nw, nb) in offsets:
        ew = rel_err(g[off:off + nw], g2[off:off + nw]); eb = rel_err(g[off + nw:off + nw + nb], g2[off + nw:off + nw + nb])
        assert ew <= slack and eb <= slack, (off, ew, eb)


@pytest.mark.parametrize("sizes", [(8192, 16384), (1000, 3000)])
def test_ppo_update_narrow_networks_against_per_layer_kernels(rocm, monkeypatch, sizes):
    """The PPO minibatch update at the benchmark's minibatch size (8,192 rows, observation 105, 8 actions) and at a ragged one, with actor and critic
    in one launch reading shuffled rows straight out of the dataset, against the same update on the per-layer kernels (which gather the rows
    first); at 512 rows the checker covers the same path."""
    capi = helpers.capi
    O, A, H = 105, 8, 64
    B, N = sizes
    rng = np.random.default_rng(21)
    na = helpers.mlp_param_count([O, H, H, A])
    params = np.concatenate([helpers.random_params(rng, [O, H, H, A]), np.log(np.full(A, 0.5, np.float32)), helpers.random_params(rng, [O, H, H, 1])])
    ld = O + 2 * A + 8
    data = rng.standard_normal((N, ld)).astype(np.float32)
    col = dict(observations=0, actions=O + A, action_log_probs=O + 2 * A, advantages=O + 2 * A + 6, target_values=O + 2 * A + 7)
    net = Mlp(rocm, [O, H, H, A], params[:na], N, "tanh", trainable=False)
    out, data0 = rocm.zeros((N, A)), rocm.array(data)
    ws, wsn = net.workspace()
    rocm.call("mlp_evaluate", net.layers, net.n, data0.offset(0), ld, out.ptr, A, N, ws, wsn)
    rocm.sync()
    z = (data[:, col["actions"]:col["actions"] + A] - out.numpy()) / 0.5
    data[:, col["action_log_probs"]] = (-0.9189385332046727 - np.log(0.5) - 0.5 * z * z).sum(1) + 0.2 * rng.standard_normal(N).astype(np.float32)
    perm = rng.permutation(N).astype(np.uint32)
    pp = capi.ppo_parameters()
    results = []
    for single in ("1", "0"):
        monkeypatch.setenv("RLT_MLP_SINGLE_PASS", single)
        agent = helpers.PpoOnBackend(rocm, O, A, H, H, B, params, "tanh", "tanh", capi.adam_parameters(3e-4, epsilon=1e-8))
        dd, idx, loss = rocm.array(data), rocm.array(perm), rocm.zeros((1,))
        args = (dd.offset(col["observations"]), dd.offset(col["observations"]), dd.offset(col["actions"]), dd.offset(col["action_log_probs"]),
                dd.offset(col["advantages"]), dd.offset(col["target_values"]), ld)
        rocm.call("ppo_train_minibatch", C.byref(agent.c), C.byref(pp), *args, idx.ptr, loss.ptr)
        rocm.sync()
        results.append(dict(actor_grads=agent.actor.grads.numpy(), critic_grads=agent.critic.grads.numpy(), d_log_std=agent.d_log_std.numpy(), loss=loss.numpy(),
                            means=agent.actor.out[-1].numpy(), params=agent.parameters()))
    got, want = results
    for key in want:
        assert rel_err(got[key], want[key]) <= TOL, (key, rel_err(got[key], want[key]))


# (batch, layer widths, hidden activation, output activation, MSE target instead of a given gradient)
INPUT_GRADIENT_CASES = [(4096, [64, 64, 4], "tanh", "identity", True),        # the head of the sequence-model benchmark on a recurrent layer's output
                        (300, [17, 64, 6], "relu", "identity", False), (70, [128, 64, 16], "fast_tanh", "tanh", False), (1, [3, 64, 1], "relu", "identity", True),
                        (513, [33, 64, 64, 9], "relu", "identity", False), (256, [4, 64, 64, 1], "tanh", "identity", True),
                        (200, [20, 48, 5], "relu", "identity", True)]          # hidden width 48: the per-layer kernels with the same contract


@pytest.mark.parametrize("case", INPUT_GRADIENT_CASES)
def test_forward_backward_with_input_gradient(oracle, rocm, case):
    """rlt_rocm_mlp_forward_backward_input on two- and three-layer networks: output, weight gradients (accumulated twice) and the gradient with
    respect to the input against the checker's forward / backward_full."""
    B, dims, ha, oa, use_target = case
    rng = np.random.default_rng(B + len(dims))
    params = helpers.random_params(rng, dims)
    x = rng.standard_normal((B, dims[0])).astype(np.float32); dy = rng.standard_normal((B, dims[-1])).astype(np.float32)
    results = []
    for backend in (oracle, rocm):
        net = Mlp(backend, dims, params, B, ha, oa)
        xd, yd, dyd = backend.array(x), backend.zeros((B, dims[-1])), backend.array(dy)
        dx = backend.array(np.full((B, dims[0] + 3), 7.0, np.float32))      # a pitch: the three extra columns must stay untouched
        ws, wsn = net.workspace()
        backend.call("mlp_zero_gradient", net.layers, net.n)
        for _ in range(2):
            if use_target:
                backend.call("mlp_forward_backward_input", net.layers, net.n, xd.ptr, dims[0], yd.ptr, dims[-1], None, 0, dyd.ptr, dims[-1], 2.0 / B, dx.ptr, dims[0] + 3, B, ws, wsn)
            else:
                backend.call("mlp_forward_backward_input", net.layers, net.n, xd.ptr, dims[0], yd.ptr, dims[-1], dyd.ptr, dims[-1], None, 0, 0.0, dx.ptr, dims[0] + 3, B, ws, wsn)
        backend.sync()
        results.append((yd.numpy(), net.grads.numpy(), dx.numpy()))
    (wy, wg, wdx), (gy, gg, gdx) = results
    assert rel_err(gy, wy) <= TOL
    assert np.all(gdx[:, dims[0]:] == 7.0)
    if ha == "relu" and max(rel_err(gg, wg), rel_err(gdx[:, :dims[0]], wdx[:, :dims[0]])) > TOL:
        net = Mlp(oracle, dims, params, B, ha, oa)
        xd = oracle.array(x)
        oracle.call("mlp_forward", net.layers, net.n, xd.ptr, dims[0], B)
        near = min(np.abs(p.numpy()).min() for p in net.pre[:-1])
        assert near <= 1e-6, (near, rel_err(gg, wg))      # a pre-activation within rounding of zero switched sides
        return
    assert rel_err(gg, wg) <= TOL
    assert rel_err(gdx[:, :dims[0]], wdx[:, :dims[0]]) <= TOL
