"""Car-on-a-track step kernel against the CPU checker on synthetic tracks, through the C ABI (the reference's own track is part of its source and stays
with it; the checker is pinned against the compiled reference on that track where the reference is mounted).

Tolerance: states 1e-5 relative per column (fp32 against the reference's float with a few double sub-expressions). The three ray distances come in
steps of 1/50: they must be equal wherever the states are, up to 0.5% of the rays, which may stop one step earlier or later where a ray grazes a cell
corner; terminated may differ only where the next position is within 1e-5 of a cell edge."""
import numpy as np
import pytest

import helpers
from helpers import rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-5


@pytest.mark.parametrize("n,shape", [(1, (80, 120)), (4099, (80, 120)), (200000, (100, 100)), (5000, (33, 257))])
def test_car_track_matches_checker(oracle, rocm, n, shape):
    print("case", n, shape, flush=True)
    H, W = shape
    scale = 0.02
    track = helpers.ring_track(H, W)
    rng = np.random.default_rng(n)
    hx, hy = scale * W / 2, scale * H / 2
    states = np.stack([rng.uniform(-1.1 * hx, 1.1 * hx, n), rng.uniform(-1.1 * hy, 1.1 * hy, n), rng.uniform(-4, 4, n), rng.uniform(-0.5, 3, n), rng.uniform(-1, 1, n), rng.uniform(-8, 8, n)], 1).astype(np.float32)
    actions = rng.uniform(-1.3, 1.3, (n, 2)).astype(np.float32)
    want = helpers.car_track_on_backend(oracle, track, scale, states, actions)
    got = helpers.car_track_on_backend(rocm, track, scale, states, actions)
    for c in range(6):
        assert rel_err(got[0][:, c], want[0][:, c]) <= TOL and rel_err(got[2][:, c], want[2][:, c]) <= TOL, c
    assert np.array_equal(got[1][:, :6], states) and np.array_equal(got[3], want[3])
    for k in (1, 2):      # ray distances before and after the step
        d = np.abs(got[k][:, 6:] - want[k][:, 6:])
        assert d.max() <= 1.0 / 50 + 1e-6 and (d > 0).mean() <= 0.005, (k, d.max(), (d > 0).mean())
    differ = np.nonzero(got[4] != want[4])[0]
    if len(differ):
        cx = (want[0][differ, 0].astype(np.float64) + hx) / scale; cy = (-want[0][differ, 1].astype(np.float64) + hy) / scale
        edge = np.minimum(np.abs(cx - np.round(cx)), np.abs(cy - np.round(cy)))
        assert edge.max() <= 1e-4, (differ, edge)
    assert 0 < want[4].sum() < n or n == 1


def test_car_track_drives_a_lap_segment_like_the_checker(oracle, rocm):
    """300 closed-loop steps along the ring under a simple steering rule computed from the observations (keep the left and right rays equal): the cars stay
    on the track on both sides, and positions agree to 2e-3 m on a 2 m track."""
    H, W, scale, n = 100, 100, 0.02, 64
    track = helpers.ring_track(H, W)
    rng = np.random.default_rng(5)
    phi = rng.uniform(0, 2 * np.pi, n)
    rad = 0.65
    start = np.stack([rad * np.cos(phi), rad * np.sin(phi), phi + np.pi / 2, np.full(n, 0.3), np.zeros(n), np.zeros(n)], 1).astype(np.float32)
    sg = so = start
    obs_g = obs_o = None
    for k in range(300):
        def rule(state, obs):       # hold 0.5 m/s, steer towards the longer of the two side rays
            return np.zeros((n, 2), np.float32) if obs is None else np.stack([np.clip(2 * (0.5 - state[:, 3]), -1, 1), np.clip(2.0 * (obs[:, 8] - obs[:, 6]), -1, 1)], 1).astype(np.float32)
        sg, _, obs_g, _, tg = helpers.car_track_on_backend(rocm, track, scale, sg, rule(sg, obs_g))
        so, _, obs_o, _, to = helpers.car_track_on_backend(oracle, track, scale, so, rule(so, obs_o))
        assert to.sum() == 0 and tg.sum() == 0, k
    assert np.abs(sg[:, :2] - so[:, :2]).max() <= 2e-3 and np.hypot(so[:, 0] - start[:, 0], so[:, 1] - start[:, 1]).max() > 0.3


def test_car_track_rejects_bad_arguments(rocm):
    import ctypes as C
    p = helpers.capi.car_parameters()
    track = rocm.array(helpers.ring_track(20, 20))
    s, a = rocm.zeros((4, 6)), rocm.zeros((4, 2))
    lib, h = rocm.device.lib, rocm.device.handle
    bad = helpers.capi.RLT_E_INVALID_ARGUMENT
    assert lib.rlt_rocm_car_track_step(h, C.byref(p), None, 20, 20, C.c_float(0.02), s.ptr, a.ptr, None, None, None, None, 4) == bad
    assert lib.rlt_rocm_car_track_step(h, C.byref(p), track.ptr, 20, 0, C.c_float(0.02), s.ptr, a.ptr, None, None, None, None, 4) == bad
    assert lib.rlt_rocm_car_track_step(h, C.byref(p), track.ptr, 20, 20, C.c_float(0.0), s.ptr, a.ptr, None, None, None, None, 4) == bad
    assert lib.rlt_rocm_car_track_step(h, C.byref(p), track.ptr, 20, 20, C.c_float(0.02), s.ptr, a.ptr, None, None, None, None, 4) == 0
    rocm.sync()
