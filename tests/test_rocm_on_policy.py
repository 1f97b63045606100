"""On-policy collection, the standardize layer and the running normaliser on the HIP path, through the C ABI.

Reference: rl/components/on_policy_runner/operations_generic.h:105-146 (+ operations_generic_per_env.h:8-74),
nn/layers/standardize/operations_generic.h:54-120, rl/components/running_normalizer/operations_generic.h:18-45.
Tolerances: flags, counters and copies bit-exact; fp32 arithmetic 1e-5 relative to the largest magnitude of the column compared (the
reference evaluates a few sub-expressions of the Pendulum and of the log-probability in double)."""
import ctypes as C

import numpy as np
import pytest

import helpers
from helpers import rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-5


def compare_datasets(got, want, col, n, S, tol=TOL):
    rows = n * S
    for name in ("terminated", "truncated"):
        assert np.array_equal(got[:rows, col[name]], want[:rows, col[name]]), name
    assert np.array_equal(got[:rows + n, col["all_reset"]], want[:rows + n, col["all_reset"]])
    for name, nrows, w in (("observations", rows + n, 3), ("actions_mean", rows, 1), ("actions", rows, 1), ("action_log_probs", rows, 1), ("rewards", rows, 1)):
        e = rel_err(got[:nrows, col[name]:col[name] + w], want[:nrows, col[name]:col[name] + w])
        assert e <= tol, (name, e)


def test_collect_matches_the_references_vectors(rocm):
    """The three collect() calls of the committed reference run (warm-up, re-initialised runner, continued episodes; standardize statistics
    in use from the second on), from the reference's runner state and draws: the dataset the reference wrote and the runner state after."""
    dims, col, g = helpers.on_policy_golden()
    n, S, ld, hidden, limit = dims
    for k in range(3):
        print("collect", k, flush=True)
        o = helpers.on_policy_golden_collect(rocm, g, k, dims, col)
        compare_datasets(o.data.numpy(), g[f"c{k}_dataset"], col, n, S)
        rs = o.runner_state()
        assert np.array_equal(rs["episode_step"], g[f"c{k}_after_episode_step"]) and np.array_equal(rs["truncated"], g[f"c{k}_after_truncated"])
        assert rel_err(rs["states"], g[f"c{k}_after_states"]) <= TOL and rel_err(rs["episode_return"], g[f"c{k}_after_episode_return"]) <= TOL


@pytest.mark.parametrize("n,S,hidden,limit,standardize,force", [(4096, 16, 64, 7, True, 0), (1000, 5, 32, 0, False, 1), (3, 30, 16, 4, True, 0), (1000, 40, 64, 0, False, 1),
                                                                (17, 64, 64, 9, True, 0)])
def test_collect_matches_checker_at_other_sizes(oracle, rocm, n, S, hidden, limit, standardize, force):
    """Wider cases against the checker: 4,096 environments, no step limit, truncate-on-each-iteration, tiny batches; environments start
    from a mixed state (some mid-episode, some flagged for reset)."""
    print("case", n, S, hidden, limit, standardize, force, flush=True)
    rng = np.random.default_rng(n + S)
    col = dict(observations=0, actions_mean=3, actions=4, action_log_probs=5, rewards=6, terminated=7, truncated=8, all_reset=9, all_values=10)
    ld = 13
    dims = [3, hidden, hidden, 1]
    params = helpers.random_params(rng, dims)
    log_std = np.array([-0.3], np.float32)
    st = (rng.standard_normal(3).astype(np.float32) * 0.2, (1.0 / (0.5 + rng.random(3))).astype(np.float32)) if standardize else None
    before = dict(states=np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-1, 1, n)], 1).astype(np.float32),
                  episode_step=rng.integers(0, max(limit, 1), n).astype(np.uint32), episode_return=rng.standard_normal(n).astype(np.float32),
                  truncated=(rng.random(n) < 0.3).astype(np.uint8))
    noise = rng.standard_normal((S, n, 1)).astype(np.float32)
    ini = np.stack([rng.uniform(-np.pi, np.pi, (S, n)), rng.uniform(-1, 1, (S, n))], 2).astype(np.float32)
    out = {}
    for b in (oracle, rocm):
        o = helpers.OnPolicyOnBackend(b, n, S, ld, col, limit, before)
        actor = helpers.Mlp(b, dims, params, n, "tanh", "identity", trainable=False)
        o.collect(actor, log_std, noise, ini, standardize=st, truncate_on_each_iteration=force)
        out[b.name] = (o.data.numpy(), o.runner_state())
    (got, grs), (want, wrs) = out["rocm"], out["oracle"]
    # episodes that run for 40 steps without a reset let rounding differences grow along the closed loop: 5e-5 there
    tol = 5e-5 if (limit == 0 and S >= 40) else TOL
    compare_datasets(got, want, col, n, S, tol)
    assert np.array_equal(grs["episode_step"], wrs["episode_step"]) and np.array_equal(grs["truncated"], wrs["truncated"])
    assert rel_err(grs["states"], wrs["states"]) <= tol and rel_err(grs["episode_return"], wrs["episode_return"]) <= tol
    if force:
        assert want[:n, col["all_reset"]].all()


@pytest.mark.parametrize("rows,dim,ld", [(328, 3, 13), (65536, 105, 120), (2, 1, 1)])
def test_running_normaliser_and_standardize_match_checker(oracle, rocm, rows, dim, ld):
    print("case", rows, dim, ld, flush=True)
    rng = np.random.default_rng(rows + dim)
    batches = [(rng.standard_normal((rows, ld)) * (k + 1) + 0.5 * k).astype(np.float32) for k in range(3)]
    for x in batches:
        x[:, 0] = 0.75               # a constant column
    dy = rng.standard_normal((rows, dim)).astype(np.float32)
    res = {}
    for b in (oracle, rocm):
        mean, std, age = b.zeros((dim,)), b.array(np.ones(dim, np.float32)), b.array(np.zeros(1, np.uint32))
        for x in batches:
            xd = b.array(x)
            b.call("running_normalizer_update", xd.ptr, ld, rows, dim, mean.ptr, std.ptr, age.ptr)
        lm, lp, y, d, dx = b.zeros((dim,)), b.zeros((dim,)), b.zeros((rows, dim)), b.array(dy), b.zeros((rows, dim))
        b.call("standardize_set_statistics", mean.ptr, std.ptr, lm.ptr, lp.ptr, dim)
        xd = b.array(batches[-1])
        b.call("standardize_forward", lm.ptr, lp.ptr, xd.ptr, ld, y.ptr, dim, rows, dim)
        b.call("standardize_backward_input", lp.ptr, d.ptr, dim, dx.ptr, dim, rows, dim)
        b.sync()
        res[b.name] = dict(mean=mean.numpy(), std=std.numpy(), age=age.numpy(), lm=lm.numpy(), lp=lp.numpy(), y=y.numpy(), dx=dx.numpy())
    want, got = res["oracle"], res["rocm"]
    assert np.array_equal(got["age"], want["age"]) and int(want["age"][0]) == 3
    assert want["std"][0] == 0 and got["std"][0] == 0 and got["lp"][0] == 0          # the constant column: deviation exactly 0, precision 0
    for k in ("mean", "std", "lm", "lp", "y", "dx"):
        # the checker sums the column in row order in fp32; the kernel sums in a tree: compare with the fp32 summation error bound in mind
        tol = max(TOL, rows * 2.0 ** -24) if k in ("mean", "std", "lm", "lp", "y", "dx") else TOL
        e = rel_err(got[k], want[k])
        assert e <= tol, (k, e)


def test_one_launch_collection_against_per_step_kernels(rocm, monkeypatch):
    """3 -> 64 -> 64 -> 1 actors are collected in one launch for all steps; the same collection kept on the per-step kernels (the path of other actor
    shapes, checked against the checker above) must give the same dataset: 4,096 environments x 128 steps, episodes of 25 steps."""
    n, S, limit = 4096, 128, 25
    rng = np.random.default_rng(5)
    col = dict(observations=0, actions_mean=3, actions=4, action_log_probs=5, rewards=6, terminated=7, truncated=8, all_reset=9, all_values=10)
    ld = 13
    dims = [3, 64, 64, 1]
    params = helpers.random_params(rng, dims)
    log_std = np.array([-0.5], np.float32)
    st = (rng.standard_normal(3).astype(np.float32) * 0.2, (1.0 / (0.5 + rng.random(3))).astype(np.float32))
    before = dict(states=np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-1, 1, n)], 1).astype(np.float32), episode_step=rng.integers(0, limit, n).astype(np.uint32),
                  episode_return=rng.standard_normal(n).astype(np.float32), truncated=(rng.random(n) < 0.3).astype(np.uint8))
    noise = rng.standard_normal((S, n, 1)).astype(np.float32)
    ini = np.stack([rng.uniform(-np.pi, np.pi, (S, n)), rng.uniform(-1, 1, (S, n))], 2).astype(np.float32)
    out = []
    for flag in ("1", "0"):
        monkeypatch.setenv("RLT_COLLECT_ONE_LAUNCH", flag)
        o = helpers.OnPolicyOnBackend(rocm, n, S, ld, col, limit, before)
        actor = helpers.Mlp(rocm, dims, params, n, "relu", "tanh", trainable=False)
        o.collect(actor, log_std, noise, ini, standardize=st)
        out.append((o.data.numpy(), o.runner_state()))
    (got, grs), (want, wrs) = out
    compare_datasets(got, want, col, n, S)
    assert np.array_equal(grs["episode_step"], wrs["episode_step"]) and np.array_equal(grs["truncated"], wrs["truncated"])
    assert rel_err(grs["states"], wrs["states"]) <= TOL and rel_err(grs["episode_return"], wrs["episode_return"]) <= TOL
