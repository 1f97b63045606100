"""HIP dense / MLP / Adam kernels against the CPU checker on the same seeded inputs (through the C ABI).

Tolerance: 1e-5 relative to the largest magnitude of the reference tensor (fp32 forward/backward/Adam, as the target
states); the reference's own device-parity tests use an absolute 1e-6 on O(1) quantities
(tests/src/nn/cuda/cuda_basics.cu:629-827), shapes below include theirs (:814-827)."""
import ctypes as C
import os

import numpy as np
import pytest

import helpers
from helpers import Mlp, capi, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-5

# (batch, in, hidden, out) -- cuda_basics.cu:814-827 plus the benchmark shapes and ragged sizes
SHAPES = [(1, 1, 1, 1), (1, 256, 10, 100), (2, 256, 10, 100), (32, 256, 10, 100), (1024, 256, 10, 100), (10, 256, 200, 100),
          (9, 256, 60, 100), (200, 256, 11, 100), (64, 256, 50, 101), (256, 256, 256, 256), (256, 4, 64, 1), (256, 3, 64, 2),
          (300, 17, 256, 6), (4096, 17, 256, 6), (77, 5, 33, 3), (513, 130, 129, 37),
          (250, 70, 200, 5), (100, 6, 256, 1), (1024, 7, 256, 2), (2048, 65, 96, 3), (128, 64, 64, 64)]      # the last rows: grids of a few workgroups, reductions of 64 and more


def build_pair(oracle, rocm, shape, seed, hidden_act="relu", out_act="identity"):
    B, I, H, O = shape
    rng = np.random.default_rng(seed)
    dims = [I, H, H, O]
    params = helpers.random_params(rng, dims)
    x = rng.standard_normal((B, I)).astype(np.float32)
    dy = rng.standard_normal((B, O)).astype(np.float32)
    nets = [Mlp(b, dims, params, B, hidden_act, out_act) for b in (oracle, rocm)]
    return nets, x, dy


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("acts", [("relu", "identity"), ("tanh", "tanh")])
def test_mlp_forward_backward_matches_oracle(oracle, rocm, shape, acts):
    check_forward_backward(oracle, rocm, shape, acts)


# GELU (with the reference's constant, nn/activation_functions.h:33-36), FAST_TANH and SIGMOID as hidden and as output activation, on a
# ragged shape (per-layer kernels), the 256-wide shapes below and above the single-pass threshold, and a 64-wide one
@pytest.mark.parametrize("shape", [(77, 5, 33, 3), (300, 17, 256, 6), (4096, 17, 256, 6), (2048, 105, 64, 8)])
@pytest.mark.parametrize("acts", [("gelu", "identity"), ("gelu", "gelu"), ("fast_tanh", "sigmoid"), ("sigmoid", "fast_tanh")])
def test_every_activation_function(oracle, rocm, shape, acts):
    check_forward_backward(oracle, rocm, shape, acts)


def check_forward_backward(oracle, rocm, shape, acts):
    print("case", shape, acts, flush=True)
    nets, x, dy = build_pair(oracle, rocm, shape, seed=hash(shape) % 1000, hidden_act=acts[0], out_act=acts[1])
    B, I, H, O = shape
    results = []
    for net in nets:
        b = net.backend
        xd, dyd, dxd, yd = b.array(x), b.array(dy), b.zeros((B, I)), b.zeros((B, O))
        ws, wsn = net.workspace()
        b.call("mlp_zero_gradient", net.layers, net.n)
        b.call("mlp_evaluate", net.layers, net.n, xd.ptr, I, yd.ptr, O, B, ws, wsn)
        b.call("mlp_forward", net.layers, net.n, xd.ptr, I, B)
        b.call("mlp_backward", net.layers, net.n, xd.ptr, I, dyd.ptr, O, dxd.ptr, I, B, 1, ws, wsn)
        b.sync()
        results.append(dict(y=yd.numpy(), out=net.out[-1].numpy(), pre0=net.pre[0].numpy(), grads=net.grads.numpy(), dx=dxd.numpy(), dy=dyd.numpy()))
    ref, got = results
    for key in ref:
        assert rel_err(got[key], ref[key]) <= TOL, (key, rel_err(got[key], ref[key]))
    # per-layer weight/bias gradients individually (a small layer must not hide behind a large one)
    for (off, nw, nb) in nets[0].offsets:
        assert rel_err(got["grads"][off:off + nw], ref["grads"][off:off + nw]) <= TOL
        assert rel_err(got["grads"][off + nw:off + nw + nb], ref["grads"][off + nw:off + nw + nb]) <= TOL


def test_mlp_backward_input_only_and_accumulation(oracle, rocm):
    shape = (256, 4, 64, 1)
    nets, x, dy = build_pair(oracle, rocm, shape, seed=3)
    B, I, H, O = shape
    res = []
    for net in nets:
        b = net.backend
        xd, dxd = b.array(x), b.zeros((B, I))
        ws, wsn = net.workspace()
        b.call("mlp_zero_gradient", net.layers, net.n)
        b.call("mlp_forward", net.layers, net.n, xd.ptr, I, B)
        dyd = b.array(dy)
        b.call("mlp_backward", net.layers, net.n, None, 0, dyd.ptr, O, dxd.ptr, I, B, 0, ws, wsn)   # backward_input: no weight gradients
        g0 = net.grads.numpy().copy()
        for _ in range(2):      # gradients accumulate (beta = 1) until zero_gradient
            dyd = b.array(dy)
            b.call("mlp_backward", net.layers, net.n, xd.ptr, I, dyd.ptr, O, None, 0, B, 1, ws, wsn)
        b.sync()
        res.append((dxd.numpy(), g0, net.grads.numpy()))
    assert rel_err(res[1][0], res[0][0]) <= TOL
    assert np.all(res[1][1] == 0) and np.all(res[0][1] == 0)
    assert rel_err(res[1][2], res[0][2]) <= TOL


@pytest.mark.parametrize("shape", [(1, 3, 8, 2), (256, 17, 256, 6), (1000, 4, 64, 1)])
def test_dense_layer_entry_points(oracle, rocm, shape):
    nets, x, dy = build_pair(oracle, rocm, shape, seed=11, hidden_act="tanh")
    B, I, H, O = shape
    res = []
    for net in nets:
        b = net.backend
        L = C.pointer(net.layers[0])
        xd, yd, dd, did = b.array(x), b.zeros((B, H)), b.array(np.random.default_rng(5).standard_normal((B, H)).astype(np.float32)), b.zeros((B, I))
        b.call("mlp_zero_gradient", net.layers, net.n)
        b.call("dense_evaluate", L, xd.ptr, I, yd.ptr, H, B)
        y0 = yd.numpy()
        b.call("dense_forward", L, xd.ptr, I, yd.ptr, H, B)
        b.call("dense_backward_full", L, xd.ptr, I, dd.ptr, H, did.ptr, I, B)
        b.sync()
        off, nw, nb = net.offsets[0]
        res.append((y0, yd.numpy(), net.pre[0].numpy(), dd.numpy(), did.numpy(), net.grads.numpy()[off:off + nw + nb]))
    for g, r in zip(res[1], res[0]):
        assert rel_err(g, r) <= TOL


@pytest.mark.parametrize("eps", [1e-7, 1e-8])
def test_adam_steps_match_oracle(oracle, rocm, eps):
    shape = (64, 17, 256, 6)
    nets, x, dy = build_pair(oracle, rocm, shape, seed=21)
    rng = np.random.default_rng(4)
    total = nets[0].params.shape[0]
    p = capi.adam_parameters(epsilon=eps)
    out = []
    for net in nets:
        b = net.backend
        norm = b.zeros((1,))
        for step in range(5):
            g = np.random.default_rng(100 + step).standard_normal(total).astype(np.float32) * (10.0 ** (step - 3))
            net.grads.upload(g)
            b.call("adam_step", net.adam, net.n_adam, C.byref(p), net.age.ptr, 0.0, norm.ptr)
        b.sync()
        out.append((net.params.numpy(), net.m.numpy(), net.v.numpy(), net.age.numpy(), norm.numpy()))
    for g, r in zip(out[1][:3], out[0][:3]):
        assert rel_err(g, r) <= TOL
    assert out[1][3][0] == out[0][3][0] == 6
    assert rel_err(out[1][4], out[0][4]) <= TOL
    # first-step closed form: |delta p| = alpha * |g| / (|g| + eps) up to rounding, checked on the oracle side in test_oracle_closed_forms


def test_adam_fused_polyak_and_polyak_update(oracle, rocm):
    rng = np.random.default_rng(9)
    n = 5000
    vals = [rng.standard_normal(n).astype(np.float32) for _ in range(5)]
    res = []
    for b in (oracle, rocm):
        p, g, m, v, t = (b.array(a) for a in vals)
        age = b.array(np.array([1], np.uint32))
        tensors = (capi.AdamTensor * 1)(capi.AdamTensor(p.ptr, g.ptr, m.ptr, v.ptr, t.ptr, n, 1))
        par = capi.adam_parameters()
        b.call("adam_step", tensors, 1, C.byref(par), age.ptr, 0.995, None)
        src, dst = b.array(vals[0]), b.array(vals[1])
        b.call("polyak_update", src.ptr, dst.ptr, n, 0.9, 0)
        b.call("polyak_update", src.ptr, dst.ptr, n, 0.9, 1)
        b.sync()
        res.append((p.numpy(), t.numpy(), dst.numpy()))
    for g, r in zip(res[1], res[0]):
        assert rel_err(g, r) <= TOL


def test_forward_backward_fused_entry(oracle, rocm):
    for shape, use_target in (((512, 17, 256, 6), False), ((300, 105, 64, 1), True)):
        nets, x, dy = build_pair(oracle, rocm, shape, seed=8, hidden_act="relu" if not use_target else "tanh")
        B, I, H, O = shape
        res = []
        for net in nets:
            b = net.backend
            xd, yd, dyd = b.array(x), b.zeros((B, O)), b.array(dy)
            ws, wsn = net.workspace()
            b.call("mlp_zero_gradient", net.layers, net.n)
            if use_target:
                b.call("mlp_forward_backward", net.layers, net.n, xd.ptr, I, yd.ptr, O, None, 0, dyd.ptr, O, 1.0 / B, B, ws, wsn)
            else:
                b.call("mlp_forward_backward", net.layers, net.n, xd.ptr, I, yd.ptr, O, dyd.ptr, O, None, 0, 0.0, B, ws, wsn)
            b.sync()
            res.append((yd.numpy(), net.grads.numpy(), dyd.numpy()))
        assert rel_err(res[1][0], res[0][0]) <= TOL
        assert rel_err(res[1][1], res[0][1]) <= TOL
        assert np.array_equal(res[1][2], dy)      # the caller's upstream gradient / target is left untouched


def test_rejects_bad_arguments(rocm):
    net = Mlp(rocm, [4, 8, 8, 1], helpers.random_params(np.random.default_rng(0), [4, 8, 8, 1]), 16)
    lib, h = rocm.device.lib, rocm.device.handle
    x = rocm.zeros((16, 4))
    assert lib.rlt_rocm_mlp_forward(h, net.layers, net.n, None, 4, 16) == -1
    assert lib.rlt_rocm_mlp_forward(h, net.layers, net.n, x.ptr, 3, 16) == -1      # leading dimension too small
    assert lib.rlt_rocm_mlp_forward(h, net.layers, net.n, x.ptr, 4, 0) == -1
    assert lib.rlt_rocm_mlp_evaluate(h, net.layers, net.n, x.ptr, 4, x.ptr, 1, 16, None, 0) == -1   # missing workspace
    assert lib.rlt_rocm_check_status(h) == 0


@pytest.mark.parametrize("dims,batch", [([33, 256, 40, 7, 256, 3], 300), ([7, 256, 256, 1], 256), ([6, 256], 17), ([256, 255, 254, 253, 252, 251, 250, 249, 2], 2048),
                                        ([5, 16, 17, 15, 1], 1)])
def test_all_layers_in_one_launch_match_the_checker_and_the_per_layer_kernels(oracle, rocm, dims, batch):
    """Batches of up to 2,048 rows through layers at most 256 wide take one launch for all layers (evaluate, and forward with every layer's pre-activations and
    outputs kept): networks of one to eight layers, widths that are no multiples of 4 or 16, batches that are no multiple of 16. Against the CPU checker to 1e-5 and
    against the per-layer kernels (RLT_MLP_ROWS=0; another order of summation) to the same bound."""
    print("case", dims, batch, flush=True)
    rng = np.random.default_rng(sum(dims) + batch)
    params = helpers.random_params(rng, dims)
    x = rng.standard_normal((batch, dims[0])).astype(np.float32)
    results = []
    for backend, rows in ((oracle, None), (rocm, "1"), (rocm, "0")):
        if rows is not None:
            os.environ["RLT_MLP_ROWS"] = rows
            os.environ["RLT_MLP_WIDE"] = rows      # three layers wider than 64 take the sixteen-row tiles (tests/test_rocm_mlp_wide.py): off with the few-rows kernel
        try:
            net = Mlp(backend, dims, params, batch, "tanh", "identity")
            xd, yd = backend.array(x), backend.zeros((batch, dims[-1]))
            ws, wsn = net.workspace()
            backend.call("mlp_evaluate", net.layers, net.n, xd.ptr, dims[0], yd.ptr, dims[-1], batch, ws, wsn)
            backend.call("mlp_forward", net.layers, net.n, xd.ptr, dims[0], batch)
            backend.sync()
            results.append([yd.numpy()] + [p.numpy() for p in net.pre] + [o.numpy() for o in net.out])
        finally:
            os.environ.pop("RLT_MLP_ROWS", None); os.environ.pop("RLT_MLP_WIDE", None)
    ref, one_launch, per_layer = results
    for k in range(len(ref)):
        assert rel_err(one_launch[k], ref[k]) <= TOL and rel_err(per_layer[k], ref[k]) <= TOL and rel_err(one_launch[k], per_layer[k]) <= TOL, k
    if batch < 1024:      # from 1,024 rows forward() takes the per-layer or the single-pass kernels
        assert np.array_equal(one_launch[0], one_launch[-1])      # evaluate and forward: the same kernel, the same bits


@pytest.mark.parametrize("n_layers", [1, 3, 10])
def test_zero_gradient_of_tensors_that_lie_apart(rocm, n_layers):
    """Gradient tensors that are allocations of their own (as the reference's containers are), here ranges of one buffer with gaps between them: cleared by
    one launch per 16 runs, nothing outside them touched; two tensors that happen to lie back to back count as one run."""
    rng = np.random.default_rng(n_layers)
    dims = [int(d) for d in rng.integers(1, 40, n_layers + 1)]
    sizes = []
    for l in range(n_layers):
        sizes += [dims[l] * dims[l + 1], dims[l + 1]]
    gaps = [int(g) for g in rng.integers(0, 9, len(sizes) + 1)]      # a gap of zero makes two tensors adjacent
    total = sum(sizes) + sum(gaps)
    buffer = rocm.array(np.full(total, 7.0, np.float32))
    params = rocm.array(np.ones(sum(sizes), np.float32))
    layers = (capi.DenseLayer * n_layers)()
    offsets, at, p_at = [], gaps[0], 0
    for k, size in enumerate(sizes):
        offsets.append((at, size)); at += size + gaps[k + 1]
    for l in range(n_layers):
        L = layers[l]
        L.in_dim, L.out_dim, L.activation = dims[l], dims[l + 1], capi.ACT["relu"]
        L.weights, L.biases = params.offset(p_at), params.offset(p_at + sizes[2 * l]); p_at += sizes[2 * l] + sizes[2 * l + 1]
        L.d_weights, L.d_biases = buffer.offset(offsets[2 * l][0]), buffer.offset(offsets[2 * l + 1][0])
    rocm.call("mlp_zero_gradient", layers, n_layers)
    rocm.sync()
    want = np.full(total, 7.0, np.float32)
    for at, size in offsets:
        want[at:at + size] = 0.0
    assert np.array_equal(buffer.numpy(), want)
