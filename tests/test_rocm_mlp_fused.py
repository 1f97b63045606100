"""Parity of the single-pass forward+backward kernel (in -> 256 -> 256 -> out) with the CPU checker, through the C ABI.

fp32 tolerance: 1e-5 relative to the largest magnitude of the tensor compared (the contraction order differs from the checker's)."""
import numpy as np
import pytest

import helpers
from helpers import Mlp, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-5


def run(backend, dims, params, x, dy, hidden_act, out_act, use_target, mse_scale, repeat=1, want_y=True):
    B = x.shape[0]
    net = Mlp(backend, dims, params, B, hidden_act, out_act)
    xd, yd, dyd = backend.array(x), backend.zeros((B, dims[-1])), backend.array(dy)
    ws, wsn = net.workspace()
    backend.call("mlp_zero_gradient", net.layers, net.n)
    for _ in range(repeat):
        if use_target:
            backend.call("mlp_forward_backward", net.layers, net.n, xd.ptr, dims[0], yd.ptr if want_y else None, dims[-1], None, 0, dyd.ptr, dims[-1], mse_scale, B, ws, wsn)
        else:
            backend.call("mlp_forward_backward", net.layers, net.n, xd.ptr, dims[0], yd.ptr if want_y else None, dims[-1], dyd.ptr, dims[-1], None, 0, 0.0, B, ws, wsn)
    backend.sync()
    return yd.numpy(), net.grads.numpy(), net.offsets


CASES = [
    # batch, in, out, hidden act, out act, target?
    (64, 17, 6, "relu", "identity", False),       # exactly one tile
    (1000, 17, 6, "relu", "identity", False),     # ragged last tile (1000 = 15 * 64 + 40)
    (37, 17, 6, "relu", "identity", False),       # less than one tile
    (4096 + 3, 17, 6, "tanh", "identity", True),  # mse gradient formed from a target inside the kernel
    (640, 32, 16, "sigmoid", "tanh", False),      # widest input / output the kernel takes, non-identity output
    (200, 1, 1, "fast_tanh", "sigmoid", True),    # narrowest
    (20000, 11, 3, "relu", "identity", False),    # more tiles than workgroups: accumulators carry over tiles
]


@pytest.mark.parametrize("case", CASES)
def test_fused_matches_checker(oracle, rocm, case, monkeypatch):
    print("case", case, flush=True)
    monkeypatch.setenv("RLT_MLP_WIDE", "0")      # batches of at most 4,096 rows would take the sixteen-row tiles (tests/test_rocm_mlp_wide.py); this file is about the 64-row tiles
    B, I, O, ha, oa, use_target = case
    dims = [I, 256, 256, O]
    rng = np.random.default_rng(B * 31 + I)
    params = helpers.random_params(rng, dims)
    x = rng.standard_normal((B, I)).astype(np.float32)
    dy = rng.standard_normal((B, O)).astype(np.float32)
    ref = run(oracle, dims, params, x, dy, ha, oa, use_target, 1.0 / B)
    got = run(rocm, dims, params, x, dy, ha, oa, use_target, 1.0 / B)
    assert rel_err(got[0], ref[0]) <= TOL, ("y", rel_err(got[0], ref[0]))
    # per-layer weight and bias gradients individually (a small layer must not hide behind a large one)
    for (off, nw, nb) in ref[2]:
        ew = rel_err(got[1][off:off + nw], ref[1][off:off + nw]); eb = rel_err(got[1][off + nw:off + nw + nb], ref[1][off + nw:off + nw + nb])
        assert ew <= TOL and eb <= TOL, (off, ew, eb)


def test_fused_accumulates_and_tolerates_null_output(oracle, rocm, monkeypatch):
    monkeypatch.setenv("RLT_MLP_WIDE", "0")
    dims = [17, 256, 256, 6]
    rng = np.random.default_rng(5)
    params = helpers.random_params(rng, dims)
    x = rng.standard_normal((300, 17)).astype(np.float32); dy = rng.standard_normal((300, 6)).astype(np.float32)
    once = run(rocm, dims, params, x, dy, "relu", "identity", False, 0.0, repeat=1)
    twice = run(rocm, dims, params, x, dy, "relu", "identity", False, 0.0, repeat=2, want_y=False)
    assert rel_err(twice[1], 2.0 * once[1]) <= 1e-6          # beta = 1: a second call adds the same gradient again
    assert np.all(twice[0] == 0.0)                            # y == NULL: nothing written


def forward_then_backward(backend, dims, params, x, dy, ha, oa):
    """The reference's call pattern: forward() (keeps every layer's pre-activations and outputs), then backward() of a given gradient."""
    B = x.shape[0]
    net = Mlp(backend, dims, params, B, ha, oa)
    xd, dyd = backend.array(x), backend.array(dy)
    ws, wsn = net.workspace()
    backend.call("mlp_zero_gradient", net.layers, net.n)
    backend.call("mlp_forward", net.layers, net.n, xd.ptr, dims[0], B)
    backend.call("mlp_backward", net.layers, net.n, xd.ptr, dims[0], dyd.ptr, dims[-1], None, 0, B, 1, ws, wsn)
    backend.sync()
    return dict(pre=[p.numpy() for p in net.pre], out=[o.numpy() for o in net.out], grads=net.grads.numpy(), d_output=dyd.numpy(), offsets=net.offsets)


@pytest.mark.parametrize("case", [(1024, 17, 6, "relu", "identity"), (4099, 17, 6, "tanh", "tanh"), (1100, 32, 16, "sigmoid", "sigmoid"), (2048, 1, 1, "fast_tanh", "identity")])
def test_forward_then_backward_single_pass_modes_match_checker(oracle, rocm, case):
    """forward() and backward() as separate calls at batch >= 1,024 run the single-pass kernel in its forward-only and backward-only modes:
    every layer's pre-activations and outputs, the in-place d_pre of the last layer, and all gradients against the checker."""
    print("case", case, flush=True)
    B, I, O, ha, oa = case
    dims = [I, 256, 256, O]
    rng = np.random.default_rng(B + I)
    params = helpers.random_params(rng, dims)
    x = rng.standard_normal((B, I)).astype(np.float32); dy = rng.standard_normal((B, O)).astype(np.float32)
    want, got = forward_then_backward(oracle, dims, params, x, dy, ha, oa), forward_then_backward(rocm, dims, params, x, dy, ha, oa)
    for l in range(3):
        assert rel_err(got["pre"][l], want["pre"][l]) <= TOL and rel_err(got["out"][l], want["out"][l]) <= TOL, l
    assert rel_err(got["d_output"], want["d_output"]) <= TOL          # backward leaves the gradient at the last pre-activations there
    for (off, nw, nb) in want["offsets"]:
        ew = rel_err(got["grads"][off:off + nw], want["grads"][off:off + nw]); eb = rel_err(got["grads"][off + nw:off + nw + nb], want["grads"][off + nw:off + nw + nb])
        assert ew <= TOL and eb <= TOL, (off, ew, eb)


def test_single_pass_modes_full_size_against_per_layer_kernels(rocm, monkeypatch):
    """Batch 65,536: forward() + backward() through the single-pass modes against the same calls kept on the per-layer kernels."""
    B, dims = 65536, [17, 256, 256, 6]
    rng = np.random.default_rng(12)
    params = helpers.random_params(rng, dims)
    x = rng.standard_normal((B, 17)).astype(np.float32); dy = (rng.standard_normal((B, 6)) / B).astype(np.float32)
    got = forward_then_backward(rocm, dims, params, x, dy, "relu", "identity")
    monkeypatch.setenv("RLT_MLP_SINGLE_PASS", "0")
    want = forward_then_backward(rocm, dims, params, x, dy, "relu", "identity")
    for l in range(3):
        assert rel_err(got["pre"][l], want["pre"][l]) <= TOL and rel_err(got["out"][l], want["out"][l]) <= TOL, l
    for (off, nw, nb) in want["offsets"]:
        assert rel_err(got["grads"][off:off + nw], want["grads"][off:off + nw]) <= TOL and rel_err(got["grads"][off + nw:off + nw + nb], want["grads"][off + nw:off + nw + nb]) <= TOL


def test_fused_full_size_against_per_layer_path_and_linearity(rocm, monkeypatch):
    """Batch 65,536 (the benchmark shape): the checker would take minutes, so compare with the per-layer kernels of the same
    library (themselves checked against the checker at small sizes) and use linearity of the gradients in d_output."""
    B, dims = 65536, [17, 256, 256, 6]
    rng = np.random.default_rng(11)
    params = helpers.random_params(rng, dims)
    x = rng.standard_normal((B, 17)).astype(np.float32); dy = (rng.standard_normal((B, 6)) / B).astype(np.float32)
    y, g, offsets = run(rocm, dims, params, x, dy, "relu", "identity", False, 0.0)
    # per-layer path: forward (stores activations), backward
    monkeypatch.setenv("RLT_MLP_SINGLE_PASS", "0")
    net = Mlp(rocm, dims, params, B)
    xd, dyd = rocm.array(x), rocm.array(dy)
    ws, wsn = net.workspace()
    rocm.call("mlp_zero_gradient", net.layers, net.n)
    rocm.call("mlp_forward", net.layers, net.n, xd.ptr, 17, B)
    rocm.call("mlp_backward", net.layers, net.n, xd.ptr, 17, dyd.ptr, 6, None, 0, B, 1, ws, wsn)
    rocm.sync()
    assert rel_err(y, net.out[-1].numpy()) <= TOL
    g2 = net.grads.numpy()
    for (off, nw, nb) in offsets:
        assert rel_err(g[off:off + nw], g2[off:off + nw]) <= TOL and rel_err(g[off + nw:off + nw + nb], g2[off + nw:off + nw + nb]) <= TOL
    # gradients are linear in the upstream gradient
    _, g3, _ = run(rocm, dims, params, x, (-3.0 * dy).astype(np.float32), "relu", "identity", False, 0.0)
    assert rel_err(g3, -3.0 * g) <= 2e-6
