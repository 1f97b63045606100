"""Batched off-policy runner step (environment step of every environment + replay add) and gather on the GPU, through the C ABI.

Reference: rl/components/off_policy_runner/operations_generic.h:183-238, operations_generic_per_env.h:8-108, gather_batch :240-430.
Tolerances: environment arithmetic 1e-5 relative (the reference evaluates a few sub-expressions in double); cursors, flags, episode
bookkeeping and every copy (replay add of given values, gather) bit-exact."""
import ctypes as C

import numpy as np
import pytest

import helpers
from helpers import rel_err

pytestmark = pytest.mark.gpu


class Runner:
    def __init__(self, b, n_envs, capacity, limit):
        capi = helpers.capi
        self.b, self.n, self.cap = b, n_envs, capacity
        self.rb = helpers.ReplayOnBackend(b, n_envs, capacity)
        self.states = b.zeros((n_envs, 2)); self.ep_step = b.zeros((n_envs,), np.uint32); self.ep_ret = b.zeros((n_envs,))
        self.trunc = b.array(np.ones(n_envs, np.uint8))
        self.c = capi.PendulumRunner(self.states.ptr, self.ep_step.ptr, self.ep_ret.ptr, self.trunc.ptr, n_envs, limit, capi.pendulum_parameters())

    def step(self, actor, initial_states, kind=1, actions=None, noise=None):
        """kind 0: given actions; 1: the actor's output is the action; 2: actor [mean | log_std] + tanh-Gaussian head with the given noise"""
        ini = self.b.array(initial_states)
        self._keep = [self.b.array(x) for x in (actions, noise) if x is not None]
        sas = helpers.capi.SasParameters(-20.0, 2.0, 1e-6, -1.0)
        args = (C.byref(self.c), C.byref(self.rb.c), kind, actor.layers if actor else None, actor.n if actor else 0, C.byref(sas) if kind == 2 else None,
                self._keep[0].ptr if kind == 0 else None, self._keep[0].ptr if kind == 2 else None, ini.ptr)
        if self.b.name == "oracle":
            assert self.b.lib.rlt_oracle_pendulum_runner_step(*args) == 0
        else:
            self.b.call("pendulum_runner_step", *args, 0, 0)

    def snapshot(self):
        return dict(states=self.states.numpy(), ep_step=self.ep_step.numpy(), ep_ret=self.ep_ret.numpy(), trunc=self.trunc.numpy(), data=self.rb.data.numpy(),
                    episode_start=self.rb.episode_start.numpy(), position=self.rb.position.numpy(), ces=self.rb.current_episode_start.numpy(), full=self.rb.full.numpy())

    def load(self, s):
        self.states.upload(s["states"]); self.ep_step.upload(s["ep_step"]); self.ep_ret.upload(s["ep_ret"]); self.trunc.upload(s["trunc"]); self.rb.data.upload(s["data"])
        self.rb.episode_start.upload(s["episode_start"]); self.rb.position.upload(s["position"]); self.rb.current_episode_start.upload(s["ces"]); self.rb.full.upload(s["full"])


def compare(got, want, tol=1e-5):
    for k in ("ep_step", "trunc", "episode_start", "position", "ces", "full"):
        assert np.array_equal(got[k], want[k]), k
    for k in ("states", "ep_ret"):
        assert rel_err(got[k], want[k]) <= tol, (k, rel_err(got[k], want[k]))
    assert np.array_equal(got["data"][:, 8:], want["data"][:, 8:])           # terminated / truncated columns
    assert rel_err(got["data"], want["data"]) <= tol, rel_err(got["data"], want["data"])


def test_runner_steps_with_truncation_and_ring_wrap(oracle, rocm):
    """37 environments, rings of 16 rows, episodes of 5 steps, 40 steps: every ring wraps twice and every episode boundary (reset from
    host-drawn initial states, truncated flag written back into the previous row, current_episode_start) is crossed several times. The GPU
    state is re-seeded from the checker's each step, so one step's rounding does not feed the next."""
    n, cap, limit = 37, 16, 5
    rng = np.random.default_rng(4)
    dims = [3, 64, 64, 1]
    params = helpers.random_params(rng, dims)
    a_o, a_r = (helpers.Mlp(b, dims, params, n, "relu", "tanh", trainable=False) for b in (oracle, rocm))
    r_o, r_r = Runner(oracle, n, cap, limit), Runner(rocm, n, cap, limit)
    for t in range(40):
        print("step", t, flush=True)
        ini = np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-1, 1, n)], 1).astype(np.float32)
        r_r.load(r_o.snapshot())
        r_o.step(a_o, ini); r_r.step(a_r, ini)
        rocm.sync()
        compare(r_r.snapshot(), r_o.snapshot())
    s = r_o.snapshot()
    assert s["full"].all() and (s["position"] == 40 % cap).all() and s["data"][:, 9].sum() >= n * 2


def test_runner_and_gather_at_benchmark_size(oracle, rocm):
    """65,536 environments with 16 replay rows each (1,048,576 rows), then a batch of 4,096 gathered from host-drawn (environment, offset)
    pairs. Two steps against the checker; after 20 steps the size-independent properties: every cursor at 20 mod 16 with the ring full,
    every gathered row bit-identical to the replay row it names."""
    n, cap, limit, B = 65536, 16, 200, 4096
    rng = np.random.default_rng(6)
    dims = [3, 64, 64, 1]
    params = helpers.random_params(rng, dims)
    a_o, a_r = (helpers.Mlp(b, dims, params, n, "relu", "tanh", trainable=False) for b in (oracle, rocm))
    r_o, r_r = Runner(oracle, n, cap, limit), Runner(rocm, n, cap, limit)
    ini = np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-1, 1, n)], 1).astype(np.float32)
    for t in range(2):
        r_o.step(a_o, ini); r_r.step(a_r, ini)
    rocm.sync()
    compare(r_r.snapshot(), r_o.snapshot(), tol=2e-5)
    for t in range(18):
        r_r.step(a_r, ini)
    rocm.sync()
    s = r_r.snapshot()
    assert (s["position"] == 20 % cap).all() and s["full"].all() and (s["ep_step"] == 20).all() and np.isfinite(s["data"]).all()
    envs = rng.integers(0, n, B).astype(np.uint32); offs = rng.integers(0, cap, B).astype(np.uint32)
    ed, od = rocm.array(envs), rocm.array(offs)
    oab, rew, term = rocm.zeros((2, B, 4)), rocm.zeros((B,)), rocm.zeros((B,), np.uint8)
    rocm.call("gather_batch", C.byref(r_r.rb.c), ed.ptr, od.ptr, 0, limit, B, oab.ptr, rew.ptr, term.ptr, None, None, None, None)
    rocm.sync()
    data = s["data"].reshape(n, cap, 10)
    index = (s["position"][envs] + limit + offs) % cap            # full ring: rl/components/off_policy_runner/operations_generic.h:305-308
    rows = data[envs, index]
    got = oab.numpy()
    assert np.array_equal(got[0], rows[:, 0:4]) and np.array_equal(got[1, :, :3], rows[:, 5:8]) and np.array_equal(rew.numpy(), rows[:, 4])
    assert np.array_equal(term.numpy(), (rows[:, 8] != 0).astype(np.uint8))


@pytest.mark.parametrize("kind,hidden,hidden_act,n", [(2, 64, "relu", 1000), (2, 64, "tanh", 70), (1, 64, "tanh", 33), (1, 32, "relu", 100), (2, 48, "relu", 100), (0, 0, "", 100)])
def test_runner_policy_kinds_and_shapes(oracle, rocm, kind, hidden, hidden_act, n):
    """The three policy kinds; hidden width 64 takes the one-launch kernel (ragged last tile, every hidden activation class), other widths
    and given actions the per-operation path. Ten steps with short episodes, GPU state re-seeded from the checker's each step."""
    print("case", kind, hidden, hidden_act, n, flush=True)
    cap, limit = 8, 4
    rng = np.random.default_rng(kind * 100 + hidden + n)
    actors = (None, None)
    if kind:
        dims = [3, hidden, hidden, kind]
        params = helpers.random_params(rng, dims)
        actors = [helpers.Mlp(b, dims, params, n, hidden_act, "tanh" if kind == 1 else "identity", trainable=False) for b in (oracle, rocm)]
    r_o, r_r = Runner(oracle, n, cap, limit), Runner(rocm, n, cap, limit)
    for t in range(10):
        ini = np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-1, 1, n)], 1).astype(np.float32)
        actions = rng.uniform(-1.5, 1.5, (n, 1)).astype(np.float32) if kind == 0 else None
        noise = rng.standard_normal((n, 1)).astype(np.float32) if kind == 2 else None
        r_r.load(r_o.snapshot())
        r_o.step(actors[0], ini, kind, actions, noise); r_r.step(actors[1], ini, kind, actions, noise)
        rocm.sync()
        compare(r_r.snapshot(), r_o.snapshot())
