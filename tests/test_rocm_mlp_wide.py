"""Parity of the forward + backward call on sixteen-row tiles (three-layer networks of hidden width up to 256 over at most 4,096 rows: mlp_wide_kernel, a workgroup of
sixteen wavefronts per tile, the workgroups' partial gradient sums added up by a second launch) with the CPU checker and with the library's other paths for the same
call (RLT_MLP_WIDE=0), through the C ABI.

fp32 tolerance: 1e-5 relative to the largest magnitude of the tensor compared (the contraction order differs from the checker's)."""
import numpy as np
import pytest

import helpers
from helpers import Mlp, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-5


def run(backend, dims, params, x, dy, hidden_act, use_target, mse_scale, repeat=1, want_y=True):
    B = x.shape[0]
    net = Mlp(backend, dims, params, B, hidden_act, "identity")
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
    # batch, in, hidden, out, hidden activation, target?
    (256, 17, 256, 6, "relu", False),        # the benchmark's network at its small batch
    (4096, 17, 256, 6, "relu", True),        # ... and at its middle one: 256 workgroups
    (37, 17, 256, 6, "tanh", False),         # a ragged last tile
    (1, 3, 64, 1, "relu", True),             # one row
    (300, 35, 256, 1, "relu", True),         # a critic of the Ant's width (27 + 8 inputs): the first layer in more than two chunks
    (100, 128, 200, 16, "fast_tanh", False), # the widest input and output, a hidden width that is no multiple of 16
    (2048, 1, 16, 2, "sigmoid", False),      # the narrowest
]


@pytest.mark.parametrize("case", CASES)
def test_sixteen_row_tiles_match_the_checker_and_the_other_paths(oracle, rocm, case, monkeypatch):
    print("case", case, flush=True)
    B, I, H, O, ha, use_target = case
    dims = [I, H, H, O]
    rng = np.random.default_rng(B * 31 + I + H)
    params = helpers.random_params(rng, dims)
    x = rng.standard_normal((B, I)).astype(np.float32)
    dy = rng.standard_normal((B, O)).astype(np.float32)
    ref = run(oracle, dims, params, x, dy, ha, use_target, 1.0 / B)
    got = run(rocm, dims, params, x, dy, ha, use_target, 1.0 / B)
    monkeypatch.setenv("RLT_MLP_WIDE", "0")
    other = run(rocm, dims, params, x, dy, ha, use_target, 1.0 / B)
    monkeypatch.delenv("RLT_MLP_WIDE")
    for name, want in (("checker", ref), ("other path", other)):
        assert rel_err(got[0], want[0]) <= TOL, (name, "y", rel_err(got[0], want[0]))
        for (off, nw, nb) in ref[2]:      # per-layer weight and bias gradients individually (a small layer must not hide behind a large one)
            ew = rel_err(got[1][off:off + nw], want[1][off:off + nw]); eb = rel_err(got[1][off + nw:off + nw + nb], want[1][off + nw:off + nw + nb])
            assert ew <= TOL and eb <= TOL, (name, off, ew, eb)
    assert np.abs(got[1]).max() > 0


def test_gradients_accumulate_and_the_output_may_be_null(oracle, rocm):
    """Two calls add up (the reduction adds onto the layers' gradients, as backward() does); y = NULL is allowed."""
    dims = [17, 256, 256, 6]
    rng = np.random.default_rng(3)
    params = helpers.random_params(rng, dims)
    x, dy = rng.standard_normal((500, 17)).astype(np.float32), rng.standard_normal((500, 6)).astype(np.float32)
    once = run(rocm, dims, params, x, dy, "relu", False, 0.0)
    twice = run(rocm, dims, params, x, dy, "relu", False, 0.0, repeat=2, want_y=False)
    assert rel_err(twice[1], 2.0 * once[1]) <= 1e-6 and not twice[0].any()
    ref = run(oracle, dims, params, x, dy, "relu", False, 0.0, repeat=2)
    assert rel_err(twice[1], ref[1]) <= TOL


def test_the_call_takes_the_sixteen_row_tiles_where_this_file_says_so(rocm, monkeypatch):
    """Which path ran: the sixteen-row tiles and the path the call takes without them (RLT_MLP_WIDE=0) agree to tolerance but not bit for bit."""
    dims = [17, 256, 256, 6]
    rng = np.random.default_rng(4)
    params = helpers.random_params(rng, dims)
    x, dy = rng.standard_normal((256, 17)).astype(np.float32), rng.standard_normal((256, 6)).astype(np.float32)
    wide = run(rocm, dims, params, x, dy, "relu", False, 0.0)
    monkeypatch.setenv("RLT_MLP_WIDE", "0")
    other = run(rocm, dims, params, x, dy, "relu", False, 0.0)
    assert rel_err(wide[1], other[1]) <= TOL and not np.array_equal(wide[1], other[1])


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
    return dict(grads=net.grads.numpy(), d_output=dyd.numpy(), offsets=net.offsets, pre=[p.numpy() for p in net.pre], out=[o.numpy() for o in net.out])


@pytest.mark.parametrize("case", [(256, 17, 256, 6, "relu", "identity"), (4096, 17, 256, 6, "relu", "tanh"), (37, 35, 200, 1, "tanh", "identity"), (100, 128, 72, 16, "fast_tanh", "sigmoid"),
                                  (1000, 3, 64, 2, "sigmoid", "identity")])
def test_backward_alone_on_sixteen_row_tiles_matches_the_checker_and_the_other_paths(oracle, rocm, case, monkeypatch):
    """backward() after forward(): the tiles read the hidden layers' outputs back from memory; the last layer may have any activation (its derivative is applied to the
    given gradient before the kernel runs, in place as in the reference)."""
    print("case", case, flush=True)
    B, I, H, O, ha, oa = case
    dims = [I, H, H, O]
    rng = np.random.default_rng(B + 7 * I + H)
    params = helpers.random_params(rng, dims)
    x, dy = rng.standard_normal((B, I)).astype(np.float32), rng.standard_normal((B, O)).astype(np.float32)
    ref = forward_then_backward(oracle, dims, params, x, dy, ha, oa)
    got = forward_then_backward(rocm, dims, params, x, dy, ha, oa)
    monkeypatch.setenv("RLT_MLP_WIDE", "0")
    other = forward_then_backward(rocm, dims, params, x, dy, ha, oa)
    monkeypatch.delenv("RLT_MLP_WIDE")
    for name, want in (("checker", ref), ("other path", other)):
        assert rel_err(got["d_output"], want["d_output"]) <= TOL, name
        for l in range(3):      # what forward() keeps: every layer's pre-activations and outputs (hidden widths beyond 64 take the tiles in forward() as well)
            assert rel_err(got["pre"][l], want["pre"][l]) <= TOL and rel_err(got["out"][l], want["out"][l]) <= TOL, (name, l)
        for (off, nw, nb) in ref["offsets"]:
            ew = rel_err(got["grads"][off:off + nw], want["grads"][off:off + nw]); eb = rel_err(got["grads"][off + nw:off + nw + nb], want["grads"][off + nw:off + nw + nb])
            assert ew <= TOL and eb <= TOL, (name, off, ew, eb)
    assert not np.array_equal(got["grads"], other["grads"])      # two different kernels ran

