"""HIP SAC / replay / Pendulum / GAE kernels against the CPU checker (through the C ABI).
Bit-exact where the work is copies and integer index arithmetic (replay add, gather_batch, masks); 1e-5 relative
(per-tensor scale) for fp32 arithmetic."""
import ctypes as C

import numpy as np
import pytest

import helpers
from helpers import capi, rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-5


def both(oracle, rocm):
    return (oracle, rocm)


@pytest.mark.parametrize("batch,dim", [(256, 1), (100, 3), (1, 1), (1500, 2)])
def test_sample_and_squash_forward_backward(oracle, rocm, batch, dim):
    rng = np.random.default_rng(batch + dim)
    inp = rng.standard_normal((batch, 2 * dim)).astype(np.float32) * 1.5
    inp[::7, dim:] = 3.0          # beyond the upper clamp: gradient gated to zero
    inp[1::11, dim:] = -25.0      # below the lower clamp
    noise = rng.standard_normal((batch, dim)).astype(np.float32)
    dout = rng.standard_normal((batch, dim)).astype(np.float32) / batch
    p = capi.SasParameters(-20.0, 2.0, 1e-6, -float(dim))
    res = []
    for b in both(oracle, rocm):
        i_, n_, do_ = b.array(inp), b.array(noise), b.array(dout)
        act, pre, lp, din = b.zeros((batch, dim)), b.zeros((batch, dim)), b.zeros((batch,)), b.zeros((batch, 2 * dim))
        la, dla = b.array(np.array([np.log(0.5)], np.float32)), b.array(np.array([0.25], np.float32))
        b.call("sas_forward", C.byref(p), i_.ptr, 2 * dim, n_.ptr, dim, act.ptr, dim, pre.ptr, dim, lp.ptr, batch, dim)
        b.call("sas_backward", C.byref(p), i_.ptr, 2 * dim, n_.ptr, dim, act.ptr, dim, pre.ptr, dim, do_.ptr, dim, din.ptr, 2 * dim, la.ptr, dla.ptr, batch, dim)
        act2, lp2 = b.zeros((batch, dim)), b.zeros((batch,))
        b.call("sas_forward", C.byref(p), i_.ptr, 2 * dim, None, 0, act2.ptr, dim, None, 0, lp2.ptr, batch, dim)   # evaluation mode
        b.sync()
        res.append((act.numpy(), pre.numpy(), lp.numpy(), din.numpy(), dla.numpy(), act2.numpy(), lp2.numpy()))
    for g, r in zip(res[1], res[0]):
        assert rel_err(g, r) <= TOL
    assert np.all(res[1][3][::7, dim:] == 0)


def test_target_values_min_q_masks_mse(oracle, rocm):
    B, D, A = 333, 6, 2
    rng = np.random.default_rng(1)
    q1, q2, r, lp = (rng.standard_normal(B).astype(np.float32) for _ in range(4))
    term = (rng.random(B) < 0.2).astype(np.uint8)
    d1, d2 = rng.standard_normal((B, D)).astype(np.float32), rng.standard_normal((B, D)).astype(np.float32)
    mask = (rng.random(B) < 0.5).astype(np.uint8)
    src, dst = rng.standard_normal((B, A)).astype(np.float32), rng.standard_normal((B, A)).astype(np.float32)
    res = []
    for b in both(oracle, rocm):
        a = {k: b.array(v) for k, v in dict(q1=q1, q2=q2, r=r, lp=lp, term=term, d1=d1, d2=d2, mask=mask, src=src, dst=dst).items()}
        la = b.array(np.array([-0.3], np.float32))
        y, dao, dmse, loss = b.zeros((B,)), b.zeros((B, A)), b.zeros((B,)), b.zeros((1,))
        w = b.array(np.array([0.37], np.float32)); cnt = b.zeros((1,))
        b.call("sac_target_action_values", a["q1"].ptr, a["q2"].ptr, a["r"].ptr, a["term"].ptr, a["lp"].ptr, la.ptr, 0.99, 0, y.ptr, B)
        b.call("sac_min_value_d_output", a["q1"].ptr, a["q2"].ptr, a["d1"].ptr, a["d2"].ptr, D, D, A, dao.ptr, A, B)
        b.call("mask_copy", a["src"].ptr, A, a["dst"].ptr, A, a["mask"].ptr, 1, B, A)
        g = b.array(d1)
        b.call("mask_zero", g.ptr, D, a["mask"].ptr, 0, B, D)
        b.call("mse_gradient", a["q1"].ptr, 1, y.ptr, 1, dmse.ptr, 1, B, 1, 0.0, w.ptr)
        b.call("mse_evaluate", a["q1"].ptr, 1, y.ptr, 1, B, 1, 0.5, loss.ptr)
        b.call("cast_reduce_sum_u8", a["mask"].ptr, B, cnt.ptr)
        s = b.array(np.array([4.0, 0.5], np.float32)); b.call("scale_f32", s.ptr, 2, 3.0, 1)
        b.sync()
        res.append((y.numpy(), dao.numpy(), a["dst"].numpy(), g.numpy(), dmse.numpy(), loss.numpy(), cnt.numpy(), s.numpy()))
    assert rel_err(res[1][0], res[0][0]) <= TOL
    for i in (1, 2, 3, 6):                       # pure copies / selections / counts: exact
        assert np.array_equal(res[1][i], res[0][i]), i
    for i in (4, 5, 7):
        assert rel_err(res[1][i], res[0][i]) <= TOL


def fill_replay(b, rb, rng_seed, n_envs, capacity, n_steps):
    rng = np.random.default_rng(rng_seed)
    for step in range(n_steps):
        obs, nobs = rng.standard_normal((n_envs, 3)).astype(np.float32), rng.standard_normal((n_envs, 3)).astype(np.float32)
        act, rew = rng.standard_normal((n_envs, 1)).astype(np.float32), rng.standard_normal(n_envs).astype(np.float32)
        term, trunc = (rng.random(n_envs) < 0.05).astype(np.uint8), (rng.random(n_envs) < 0.1).astype(np.uint8)
        args = [b.array(v) for v in (obs, act, rew, nobs, term, trunc)]
        b.call("replay_add", C.byref(rb.c), *[a.ptr for a in args])


@pytest.mark.parametrize("n_envs,capacity,steps", [(1, 50, 37), (1, 16, 40), (7, 16, 16), (64, 8, 29)])
def test_replay_add_and_gather_bit_exact(oracle, rocm, n_envs, capacity, steps):
    """Ring wrap (steps > capacity), a ring exactly full (steps == capacity) and a partially filled ring; gather in the
    reference's DETERMINISTIC mode (index = sample number, tests/src/rl/cuda/rl.cu:201-228) and with host-drawn
    (env, offset) pairs."""
    B = min(steps, capacity) if n_envs == 1 else 48
    rng = np.random.default_rng(5)
    out = []
    for b in both(oracle, rocm):
        rb = helpers.ReplayOnBackend(b, n_envs, capacity)
        fill_replay(b, rb, 77, n_envs, capacity, steps)
        b.sync()
        state = [x.numpy() for x in (rb.data, rb.episode_start, rb.position, rb.current_episode_start, rb.full)]
        eligible = capacity if steps >= capacity else steps
        envs = np.random.default_rng(6).integers(0, n_envs, B).astype(np.uint32)
        offs = np.random.default_rng(7).integers(0, eligible, B).astype(np.uint32)
        got = []
        for deterministic in ((1, 0) if n_envs == 1 else (0,)):
            oab, rew, term = b.array(np.full((2, B, 4), 7.0, np.float32)), b.zeros((B,)), b.zeros((B,), np.uint8)
            masks = [b.array(np.full(n, 9, np.uint8)) for n in (B, 2 * B, B, 2 * B)]
            ed, od = b.array(envs), b.array(offs)
            b.call("gather_batch", C.byref(rb.c), ed.ptr, od.ptr, deterministic, 5, B, oab.ptr, rew.ptr, term.ptr, *[m.ptr for m in masks])
            b.sync()
            got.append([oab.numpy(), rew.numpy(), term.numpy()] + [m.numpy() for m in masks])
        out.append((state, got))
    for s_ref, s_got in zip(out[0][0], out[1][0]):
        assert np.array_equal(s_ref, s_got)
    for g_ref, g_got in zip(out[0][1], out[1][1]):
        for r, g in zip(g_ref, g_got):
            assert np.array_equal(r, g)


def test_gather_draw_in_range(rocm):
    rb = helpers.ReplayOnBackend(rocm, 5, 32)
    fill_replay(rocm, rb, 1, 5, 32, 11)
    B = 4096
    e, o = rocm.zeros((B,), np.uint32), rocm.zeros((B,), np.uint32)
    rocm.device.check(rocm.device.lib.rlt_rocm_gather_draw(rocm.device.handle, C.byref(rb.c), B, 123, 0, e.ptr, o.ptr))
    rocm.sync()
    e, o = e.numpy(), o.numpy()
    assert e.max() < 5 and o.max() < 11 and len(np.unique(e)) == 5 and len(np.unique(o)) == 11


def test_pendulum_step_matches_oracle(oracle, rocm):
    N = 5000
    rng = np.random.default_rng(2)
    states = np.stack([rng.uniform(-np.pi, np.pi, N), rng.uniform(-8, 8, N)], 1).astype(np.float32)
    states[:10, 0] *= 10          # angles far outside [-pi, pi] exercise angle_normalize
    actions = rng.uniform(-2, 2, N).astype(np.float32)   # beyond [-1,1]: clamped in the dynamics, not in the reward
    p = capi.pendulum_parameters()
    res = []
    for b in both(oracle, rocm):
        s, a = b.array(states), b.array(actions)
        o, no, r = b.zeros((N, 3)), b.zeros((N, 3)), b.zeros((N,))
        for _ in range(3):
            b.call("pendulum_step", C.byref(p), s.ptr, a.ptr, o.ptr, no.ptr, r.ptr, N)
        b.sync()
        res.append((s.numpy(), o.numpy(), no.numpy(), r.numpy()))
    # the reference evaluates some sub-expressions in double (double literals); the fp32 kernel differs in the last ulp
    for g, r in zip(res[1], res[0]):
        assert rel_err(g, r) <= TOL


# chunked scan: whole chunks (16, 128), ragged last chunk (7, 17, 33), more chunks than a wavefront (2000), one environment per workgroup (2000),
# the serial kernel beyond 4,096 steps (5000), a single sample
@pytest.mark.parametrize("n_envs,steps,ld,ignore_termination", [(64, 16, 1, 0), (4096, 128, 9, 0), (100, 7, 3, 0), (3, 2000, 2, 0), (2, 5000, 1, 0), (33, 17, 4, 1),
                                                                  (1, 1, 1, 0), (700, 33, 2, 1), (129, 4096, 1, 0)])
def test_gae_matches_oracle(oracle, rocm, n_envs, steps, ld, ignore_termination):
    rng = np.random.default_rng(n_envs)
    rows = (steps + 1) * n_envs
    data = rng.standard_normal((rows, 6 * ld)).astype(np.float32)
    term = (rng.random(rows) < 0.01)
    trunc = term | (rng.random(rows) < 0.02)
    res = []
    for b in both(oracle, rocm):
        cols = [b.array(np.ascontiguousarray(np.repeat(v[:, None], ld, 1))) for v in
                (data[:, 0], term.astype(np.float32), trunc.astype(np.float32), data[:, 1])]
        adv, tv = b.zeros((rows, ld)), b.zeros((rows, ld))
        b.call("ppo_gae", cols[0].ptr, cols[1].ptr, cols[2].ptr, cols[3].ptr, adv.ptr, tv.ptr, ld, n_envs, steps, 0.99, 0.95, ignore_termination)
        b.sync()
        res.append((adv.numpy()[:steps * n_envs, 0], tv.numpy()[:steps * n_envs, 0]))
    for g, r in zip(res[1], res[0]):
        assert rel_err(g, r) <= TOL
