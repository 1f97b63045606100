"""rlt_rocm_dense_backward_static -- the entry point that allocates nothing -- against rlt_rocm_dense_backward, through the C ABI.
Both run the same launches (act'(pre) * d_output in place, split-batch contraction, fixed-order reduction) and differ only in where the
partial sums live, so the results are compared bit for bit (stricter than the 1e-5 the fp32 kernels are held to against the CPU checker,
which the allocating entry point is checked against elsewhere)."""
import ctypes as C

import numpy as np
import pytest

import helpers
from helpers import capi

pytestmark = pytest.mark.gpu


def run_backward(rocm, static, batch, in_dim, out_dim, act, seed, ldx=None, ldd=None):
    ldx, ldd = ldx or in_dim, ldd or out_dim
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((batch, ldx)).astype(np.float32)
    d_out = rng.standard_normal((batch, ldd)).astype(np.float32)
    pre = rng.standard_normal((batch, out_dim)).astype(np.float32)
    w, b = rng.standard_normal((out_dim, in_dim)).astype(np.float32), rng.standard_normal(out_dim).astype(np.float32)
    dw0, db0 = rng.standard_normal((out_dim, in_dim)).astype(np.float32), rng.standard_normal(out_dim).astype(np.float32)     # gradients accumulate onto what is there
    xd, dd, pd, wd, bd, dwd, dbd = (rocm.array(a) for a in (x, d_out, pre, w, b, dw0, db0))
    L = capi.DenseLayer()
    L.weights, L.biases, L.d_weights, L.d_biases, L.pre_activations = wd.ptr, bd.ptr, dwd.ptr, dbd.ptr, pd.ptr
    L.in_dim, L.out_dim, L.activation = in_dim, out_dim, capi.ACT[act]
    rocm.call("dense_backward_static" if static else "dense_backward", C.byref(L), xd.ptr, ldx, dd.ptr, ldd, batch)
    rocm.sync()
    out = dwd.numpy(), dbd.numpy(), dd.numpy()
    for a in (xd, dd, pd, wd, bd, dwd, dbd):
        a.free()
    return out, (x, d_out, pre, dw0, db0)


def test_two_calls_in_a_row_match_the_allocating_entry_point(rocm):
    """The second call is smaller than the first: it must not see what the first left in the shared array."""
    for (batch, i, o, act) in [(8192, 105, 64, "tanh"), (1000, 17, 64, "relu")]:
        got, _ = run_backward(rocm, True, batch, i, o, act, seed=batch)
        want, inputs = run_backward(rocm, False, batch, i, o, act, seed=batch)
        for g, w in zip(got, want):
            assert np.array_equal(g, w), (batch, i, o)
        # and against numpy in double, to the fp32 bar of the other kernels
        x, d_out, pre, dw0, db0 = inputs
        dact = 1 - np.tanh(pre.astype(np.float64)) ** 2 if act == "tanh" else (pre > 0).astype(np.float64)
        d_pre = dact * d_out
        assert helpers.rel_err(got[0], dw0 + d_pre.T @ x.astype(np.float64)) <= 1e-5
        assert helpers.rel_err(got[1], db0 + d_pre.sum(0)) <= 1e-5
        assert helpers.rel_err(got[2], d_pre) <= 1e-6


@pytest.mark.parametrize("batch,i,o,act,ldx,ldd", [(256, 4, 64, "relu", None, None), (300, 64, 1, "identity", None, None), (4096, 64, 64, "relu", 70, 66), (16128, 256, 256, "relu", None, None),
                                                    (1, 3, 2, "sigmoid", None, None), (32768, 146, 192, "identity", None, None)])
def test_shapes_with_and_without_a_split(rocm, batch, i, o, act, ldx, ldd):
    got, _ = run_backward(rocm, True, batch, i, o, act, seed=7, ldx=ldx, ldd=ldd)
    want, _ = run_backward(rocm, False, batch, i, o, act, seed=7, ldx=ldx, ldd=ldd)
    for g, w in zip(got, want):
        assert np.array_equal(g, w)


def test_sizes_beyond_the_fixed_array_are_rejected(rocm):
    batch, i, o = 65536, 256, 256          # 128 splits x 65,792 floats = 33.7 MB of partial sums
    lib, h = rocm.device.lib, rocm.device.handle
    x, d, pre = rocm.zeros((batch, i)), rocm.zeros((batch, o)), rocm.zeros((batch, o))
    w, b, dw, db = rocm.zeros((o, i)), rocm.zeros((o,)), rocm.zeros((o, i)), rocm.zeros((o,))
    L = capi.DenseLayer()
    L.weights, L.biases, L.d_weights, L.d_biases, L.pre_activations = w.ptr, b.ptr, dw.ptr, db.ptr, pre.ptr
    L.in_dim, L.out_dim, L.activation = i, o, capi.ACT["relu"]
    rc = lib.rlt_rocm_dense_backward_static(h, C.byref(L), x.ptr, i, d.ptr, o, batch)
    assert rc == capi.RLT_E_WORKSPACE_TOO_SMALL
    assert b"fixed array" in lib.rlt_rocm_error_string(rc)
    rocm.sync()
    assert not dw.numpy().any()            # nothing was launched
    assert lib.rlt_rocm_dense_backward_static(h, None, x.ptr, i, d.ptr, o, batch) == capi.RLT_E_INVALID_ARGUMENT
    assert lib.rlt_rocm_dense_backward(h, C.byref(L), x.ptr, i, d.ptr, o, batch) == 0     # the allocating entry point takes the size
    rocm.sync()
    for a in (x, d, pre, w, b, dw, db):
        a.free()
