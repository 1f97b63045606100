"""The Tensor elementwise operations (containers/tensor/operations_generic.h:365-481, 573-760): the CPU checker against numpy's textbook functions
(no GPU), and the HIP entries against the checker on views with pitches, in place and out of place."""
import ctypes as C

import numpy as np
import pytest

import helpers
from helpers import capi, rel_err


def fast_tanh(x):
    x = np.clip(x, -3, 3)
    return x * (27 + x * x) / (27 + 9 * x * x)


UNARY_REFERENCE = dict(negate=lambda a, p: -a, abs=lambda a, p: np.abs(a), constant=lambda a, p: np.full_like(a, p),
                       sigmoid=lambda a, p: np.where(a < -20, 0.0, np.where(a > 20, 1.0, 1 / (1 + np.exp(-a)))), fast_sigmoid=lambda a, p: 0.5 * fast_tanh(0.5 * a) + 0.5,
                       exp=lambda a, p: np.exp(a), tanh=lambda a, p: np.tanh(a), fast_tanh=lambda a, p: fast_tanh(a), one_minus=lambda a, p: 1 - a,
                       scale=lambda a, p: a * p, scale_reciprocal=lambda a, p: 1 / a * p)
BINARY_REFERENCE = dict(add=np.add, subtract=np.subtract, multiply=np.multiply, divide=np.divide)


def inputs(seed, rows, cols, ld):
    rng = np.random.default_rng(seed)
    a = rng.uniform(-4, 4, (rows, ld)).astype(np.float32)
    a[0, 0], a[-1, cols - 1] = -25.0, 25.0        # beyond the sigmoid's saturation points
    b = rng.uniform(0.5, 3, (rows, ld)).astype(np.float32) * rng.choice([-1, 1], (rows, ld)).astype(np.float32)
    return a, b


def test_checker_against_textbook_functions():
    oracle = helpers.HostBackend()
    rows, cols, ld = 7, 13, 16
    a, b = inputs(0, rows, cols, ld)
    for name, op in capi.UNARY.items():
        dst = np.full((rows, ld), 99.0, np.float32)
        oracle.call("unary_f32", op, 0.37, a.ctypes.data, ld, dst.ctypes.data, ld, rows, cols)
        want = UNARY_REFERENCE[name](a[:, :cols].astype(np.float64), 0.37)
        assert np.allclose(dst[:, :cols], want, rtol=2e-6, atol=1e-7), name
        assert np.all(dst[:, cols:] == 99.0)       # the pitch gap is untouched
    assert dst is not None
    sig = np.zeros((rows, ld), np.float32)
    oracle.call("unary_f32", capi.UNARY["sigmoid"], 0.0, a.ctypes.data, ld, sig.ctypes.data, ld, rows, cols)
    assert sig[0, 0] == 0.0 and sig[-1, cols - 1] == 1.0
    for name, op in capi.BINARY.items():
        dst = np.zeros((rows, ld), np.float32)
        oracle.call("binary_f32", op, a.ctypes.data, ld, b.ctypes.data, ld, dst.ctypes.data, ld, rows, cols)
        assert np.array_equal(dst[:, :cols], BINARY_REFERENCE[name](a[:, :cols], b[:, :cols])), name      # one IEEE operation each: exact
    acc = np.random.default_rng(1).standard_normal((rows, ld)).astype(np.float32)
    dst = np.zeros((rows, ld), np.float32)
    oracle.call("multiply_accumulate_f32", a.ctypes.data, ld, b.ctypes.data, ld, acc.ctypes.data, ld, dst.ctypes.data, ld, rows, cols)
    assert np.array_equal(dst[:, :cols], acc[:, :cols] + (a[:, :cols] * b[:, :cols]))
    out = np.zeros(1, np.float32)
    oracle.call("reduce_abs_max_f32", a.ctypes.data, a.size, out.ctypes.data)
    assert out[0] == np.abs(a).max() == 25.0


@pytest.mark.gpu
@pytest.mark.parametrize("rows,cols,ld", [(1, 100_003, 100_003), (257, 64, 70), (3, 5, 5)])
def test_hip_entries_match_the_checker(oracle, rocm, rows, cols, ld):
    a, b = inputs(rows, rows, cols, ld)
    acc = np.random.default_rng(2).standard_normal((rows, ld)).astype(np.float32)
    ad, bd, cd = rocm.array(a), rocm.array(b), rocm.array(acc)
    for name, op in capi.UNARY.items():
        want = np.full((rows, ld), 99.0, np.float32)
        oracle.call("unary_f32", op, 0.37, a.ctypes.data, ld, want.ctypes.data, ld, rows, cols)
        dst = rocm.array(np.full((rows, ld), 99.0, np.float32))
        rocm.call("unary_f32", op, 0.37, ad.ptr, ld, dst.ptr, ld, rows, cols)
        got = dst.numpy()
        assert rel_err(got[:, :cols], want[:, :cols]) <= 1e-6, name
        assert np.all(got[:, cols:] == 99.0)
        in_place = rocm.array(a)
        rocm.call("unary_f32", op, 0.37, in_place.ptr, ld, in_place.ptr, ld, rows, cols)
        assert np.array_equal(in_place.numpy()[:, :cols], got[:, :cols]) and np.array_equal(in_place.numpy()[:, cols:], a[:, cols:])
    for name, op in capi.BINARY.items():
        want = np.zeros((rows, ld), np.float32)
        oracle.call("binary_f32", op, a.ctypes.data, ld, b.ctypes.data, ld, want.ctypes.data, ld, rows, cols)
        dst = rocm.zeros((rows, ld))
        rocm.call("binary_f32", op, ad.ptr, ld, bd.ptr, ld, dst.ptr, ld, rows, cols)
        assert np.array_equal(dst.numpy()[:, :cols], want[:, :cols]), name      # single IEEE operations: bit-exact
    want = np.zeros((rows, ld), np.float32)
    oracle.call("multiply_accumulate_f32", a.ctypes.data, ld, b.ctypes.data, ld, acc.ctypes.data, ld, want.ctypes.data, ld, rows, cols)
    rocm.call("multiply_accumulate_f32", ad.ptr, ld, bd.ptr, ld, cd.ptr, ld, cd.ptr, ld, rows, cols)      # into the accumulator, as the GRU's gate products do
    assert np.array_equal(cd.numpy()[:, :cols], want[:, :cols])
    out = rocm.zeros((1,))
    rocm.call("reduce_abs_max_f32", ad.ptr, a.size, out.ptr)
    assert out.numpy()[0] == np.abs(a).max()
    assert rocm.device.lib.rlt_rocm_unary_f32(rocm.device.handle, 99, 0.0, ad.ptr, ld, ad.ptr, ld, rows, cols) == capi.RLT_E_INVALID_ARGUMENT
