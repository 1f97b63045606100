"""GRU forward and backward through time on the GPU, through the C ABI, against the CPU checker and against vectors written by the reference.

fp32 tolerance: 1e-5 relative to the largest magnitude of the tensor compared (contraction orders differ from the checker's)."""
import numpy as np
import pytest

import helpers
from helpers import rel_err
from test_oracle_golden import gru_golden_case

pytestmark = pytest.mark.gpu
TOL = 1e-5
KEYS = ("output", "post", "npp", "dx", "dy", "dW_i", "db_i", "dW_h", "db_h")


def run_pair(oracle, rocm, S, B, I, H, seed, with_reset, **kw):
    rng = np.random.default_rng(seed)
    params, x, dy, reset = helpers.gru_random_case(rng, S, B, I, H, with_reset)
    res = []
    for b in (oracle, rocm):
        g = helpers.GruOnBackend(b, S, B, I, H, params)
        g.forward(x, reset)
        g.backward(dy, **kw)
        b.sync()
        res.append(g.results())
    return res


@pytest.mark.parametrize("shape", [(7, 5, 6, 8), (1, 3, 4, 16), (24, 40, 11, 32), (12, 37, 20, 48), (9, 130, 3, 64), (5, 2, 7, 100)])
@pytest.mark.parametrize("with_reset", [False, True])
def test_gru_matches_checker(oracle, rocm, shape, with_reset):
    print("case", shape, with_reset, flush=True)
    S, B, I, H = shape
    want, got = run_pair(oracle, rocm, S, B, I, H, sum(shape), with_reset)
    for k in KEYS:
        assert rel_err(got[k], want[k]) <= TOL, (k, rel_err(got[k], want[k]))


def test_gru_backward_input_only_and_gradient_accumulation(oracle, rocm):
    S, B, I, H = 6, 9, 5, 32
    want, got = run_pair(oracle, rocm, S, B, I, H, 3, True, want_w=0)
    for k in ("dx", "dy"):
        assert rel_err(got[k], want[k]) <= TOL
    for k in ("dW_i", "db_i", "dW_h", "db_h"):
        assert not got[k].any()                                   # backward_input leaves the gradients alone
    rng = np.random.default_rng(5)
    params, x, dy, reset = helpers.gru_random_case(rng, S, B, I, H, False)
    g = helpers.GruOnBackend(rocm, S, B, I, H, params)
    g.forward(x); g.backward(dy, want_d_input=False); rocm.sync()
    once = g.results()
    g.backward(dy, want_d_input=False); rocm.sync()
    twice = g.results()
    for k in ("dW_i", "db_i", "dW_h"):
        assert rel_err(twice[k], 2 * once[k]) <= 1e-6           # gradients accumulate
    assert rel_err(twice["db_h"][2 * H:], 2 * once["db_h"][2 * H:]) <= 1e-6 and np.array_equal(twice["db_h"][:2 * H], twice["db_i"][:2 * H])
    assert not once["dx"].any()


@pytest.mark.parametrize("case", ["plain", "reset"])
def test_gru_against_reference_vectors(rocm, case):
    (S, B, I, H), params, x, dy, reset, want = gru_golden_case(case)
    g = helpers.GruOnBackend(rocm, S, B, I, H, params)
    g.forward(x, reset); g.backward(dy); rocm.sync()
    got = g.results()
    for k in KEYS:
        assert rel_err(got[k], want[k]) <= TOL, (k, rel_err(got[k], want[k]))


def test_gru_benchmark_shape(oracle, rocm):
    """I = 146, H = 64, S = 64 (the sequence-model benchmark): batch 64 against the checker; batch 1,024 through properties that do not need
    it -- batch rows are independent, so its first 64 rows reproduce the batch-64 run, and the gradients are linear in the upstream gradient."""
    S, I, H = 64, 146, 64
    want, got = run_pair(oracle, rocm, S, 64, I, H, 21, False)
    for k in KEYS:
        assert rel_err(got[k], want[k]) <= 2e-5, (k, rel_err(got[k], want[k]))
    rng = np.random.default_rng(21)
    params, x64, dy64, _ = helpers.gru_random_case(rng, S, 64, I, H, False)
    x = rng.standard_normal((S, 1024, I)).astype(np.float32); dy = rng.standard_normal((S, 1024, H)).astype(np.float32)
    x[:, :64], dy[:, :64] = x64, dy64
    g = helpers.GruOnBackend(rocm, S, 1024, I, H, params)
    g.forward(x); g.backward(dy); rocm.sync()
    big = g.results()
    for k in ("output", "post", "npp", "dx", "dy"):
        assert rel_err(big[k][:, :64], got[k]) <= 2e-6, k
    g2 = helpers.GruOnBackend(rocm, S, 1024, I, H, params)
    g2.forward(x); g2.backward(-2.0 * dy); rocm.sync()
    lin = g2.results()
    for k in ("dW_i", "db_i", "dW_h", "db_h", "dx"):
        assert rel_err(lin[k], -2.0 * big[k]) <= 2e-6, k


def test_gru_weight_gradients_over_a_long_batch(oracle, rocm):
    """16,384 (step, row) pairs and more take the weight-gradient kernel that keeps the whole 192 x 146 / 192 x 64 gradient in one workgroup's accumulators:
    batch 256 against the checker; batch 1,024 as the sum of its four quarters run separately (the gradients add over batch rows)."""
    S, I, H = 64, 146, 64
    print("batch 256 against the checker", flush=True)
    want, got = run_pair(oracle, rocm, S, 256, I, H, 33, True)
    for k in KEYS:
        assert rel_err(got[k], want[k]) <= 2e-5, (k, rel_err(got[k], want[k]))
    print("batch 1,024 against its quarters", flush=True)
    rng = np.random.default_rng(34)
    params, x, dy, reset = helpers.gru_random_case(rng, S, 1024, I, H, True)
    g = helpers.GruOnBackend(rocm, S, 1024, I, H, params)
    g.forward(x, reset); g.backward(dy); rocm.sync()
    whole = g.results()
    parts = []
    for q in range(4):
        sl = slice(256 * q, 256 * (q + 1))
        gq = helpers.GruOnBackend(rocm, S, 256, I, H, params)
        gq.forward(np.ascontiguousarray(x[:, sl]), None if reset is None else np.ascontiguousarray(reset[:, sl])); gq.backward(np.ascontiguousarray(dy[:, sl])); rocm.sync()
        parts.append(gq.results())
    for k in ("dW_i", "db_i", "dW_h", "db_h"):
        assert rel_err(whole[k], sum(p[k] for p in parts)) <= 1e-5, k
    for k in ("output", "dx"):
        assert rel_err(whole[k][:, 256:512], parts[1][k]) <= 2e-6, k
