"""The off-policy runner step over every batched environment (rl/components/off_policy_runner/operations_generic.h:183-238,
operations_generic_per_env.h:8-108): the HIP path against the CPU checker over several hundred steps with resets, terminations, ring wrap and
all three policy kinds. Index work, flags and copies bit-exact; floats to 1e-5 of each tensor's largest magnitude (1e-4 for the Acrobot's
states after many Runge-Kutta steps, whose double-precision sub-expressions the kernel computes in float)."""
import ctypes as C

import numpy as np
import pytest

import helpers
from helpers import capi, rel_err

pytestmark = pytest.mark.gpu


def initial_states(rng, kind, n):
    if kind == capi.ENV_PENDULUM:
        return np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-1, 1, n)], 1).astype(np.float32)
    if kind == capi.ENV_PENDULUM_POSITION:      # (theta, theta_dot, last action = 0)
        return np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-1, 1, n), np.zeros(n)], 1).astype(np.float32)
    if kind == capi.ENV_CAR:
        s = np.zeros((n, 6), np.float32)
        s[::4, 0] = 0.97; s[::4, 3] = 3.0      # some cars start at the edge of the unit square, heading out
        return s
    s = rng.uniform(-0.1, 0.1, (n, 4)).astype(np.float32)
    if kind == capi.ENV_ACROBOT:
        s[::5, 0] += 2.2      # some episodes start with the first link raised: their tip crosses the line within a few steps
    return s


@pytest.mark.parametrize("kind,policy_kind,n_envs,capacity,limit,steps", [
    (capi.ENV_PENDULUM, 2, 37, 50, 20, 120),
    (capi.ENV_PENDULUM_POSITION, 2, 41, 30, 15, 90),   # the velocity is hidden from the observation, the state remembers the last action
    (capi.ENV_PENDULUM_POSITION, 0, 300, 8, 6, 40),
    (capi.ENV_ACROBOT, 0, 64, 40, 30, 100),            # terminates when the tip swings above the bar
    (capi.ENV_ACROBOT_SWINGUP, 2, 130, 25, 12, 60),
    (capi.ENV_CAR, 1, 50, 30, 25, 80),                 # terminates when the car leaves the unit square
    (capi.ENV_CAR, 2, 1, 7, 5, 30),
    # sixteen environments or fewer: the whole step is one launch
    (capi.ENV_PENDULUM, 2, 5, 12, 9, 50),
    (capi.ENV_ACROBOT, 0, 16, 10, 30, 45),
    (capi.ENV_ACROBOT, 1, 9, 20, 30, 80),
    (capi.ENV_ACROBOT_SWINGUP, 2, 3, 25, 11, 60),
    (capi.ENV_CAR, 1, 7, 15, 8, 40),
    (capi.ENV_PENDULUM_POSITION, 2, 1, 30, 10, 70),
])
def test_env_runner_step_matches_the_checker(oracle, rocm, kind, policy_kind, n_envs, capacity, limit, steps):
    sd, od, ad = capi.ENV_DIMS[kind]
    rng = np.random.default_rng(kind * 10 + policy_kind)
    out = ad * (2 if policy_kind == 2 else 1)
    params = helpers.random_params(rng, [od, 32, 32, out])
    draws = [(initial_states(rng, kind, n_envs), rng.uniform(-1, 1, (n_envs, ad)).astype(np.float32), rng.standard_normal((n_envs, ad)).astype(np.float32)) for _ in range(steps)]
    results = []
    for backend in (oracle, rocm):
        runner = helpers.EnvRunnerOnBackend(backend, kind, n_envs, limit)
        rb = helpers.ReplayOnBackend(backend, n_envs, capacity, od, ad)
        actor = helpers.Mlp(backend, [od, 32, 32, out], params, n_envs, "relu", "tanh" if policy_kind == 1 else "identity", trainable=False) if policy_kind else None
        sas = capi.SasParameters(-20.0, 2.0, 1e-6, -float(ad))
        ws, wsn = runner.workspace(policy_kind, actor)
        trace = []
        for ini, given, noise in draws:
            i_d, g_d, n_d = backend.array(ini), backend.array(given), backend.array(noise)
            backend.call("env_runner_step", C.byref(runner.c), C.byref(rb.c), policy_kind, actor.layers if actor else None, actor.n if actor else 0, C.byref(sas),
                         g_d.ptr, n_d.ptr, i_d.ptr, ws, wsn)
            backend.sync()
            trace.append(runner.snapshot())
        results.append((trace, [a.numpy() for a in (rb.data, rb.episode_start, rb.position, rb.current_episode_start, rb.full)]))
    (ref_trace, ref_rb), (got_trace, got_rb) = results
    tol = 1e-4 if kind in (capi.ENV_ACROBOT, capi.ENV_ACROBOT_SWINGUP) else 1e-5
    n_term = n_reset = 0
    for step, (ref, got) in enumerate(zip(ref_trace, got_trace)):
        for k in (1, 3, 8):      # episode_step, truncated, terminated: exact
            assert np.array_equal(got[k], ref[k]), (step, k)
        for k in (0, 2, 4, 5, 6, 7):
            assert rel_err(got[k], ref[k]) <= tol, (step, k, rel_err(got[k], ref[k]))
        n_term += int(ref[8].sum()); n_reset += int(ref[3].sum())
    assert n_reset > 0 and (kind in (capi.ENV_PENDULUM, capi.ENV_PENDULUM_POSITION, capi.ENV_ACROBOT_SWINGUP) or n_term > 0)      # the cases exercise what they are for
    assert rel_err(got_rb[0], ref_rb[0]) <= tol
    for k in range(1, 5):
        assert np.array_equal(got_rb[k], ref_rb[k])
    assert ref_rb[4].all() or steps < capacity      # the rings wrapped


def test_env_dims(rocm):
    lib = rocm.device.lib
    for kind, dims in capi.ENV_DIMS.items():
        s, o, a = C.c_int(), C.c_int(), C.c_int()
        assert lib.rlt_rocm_env_dims(kind, C.byref(s), C.byref(o), C.byref(a)) == 0 and (s.value, o.value, a.value) == dims
    assert lib.rlt_rocm_env_dims(9, None, None, None) == capi.RLT_E_INVALID_ARGUMENT


@pytest.mark.parametrize("kind,specs,head_kind,n_envs,capacity,limit,period,steps", [
    (capi.ENV_PENDULUM, [(0, 3, 16, "relu"), (1, 16, 16, "identity"), (0, 16, 1, "tanh")], 3, 40, 30, 12, 5, 70),        # TD3's exploration head on a recurrent policy
    (capi.ENV_ACROBOT, [(0, 6, 16, "relu"), (1, 16, 16, "identity"), (1, 16, 16, "identity"), (0, 16, 2, "identity")], 2, 33, 20, 10, 0, 50),
    (capi.ENV_PENDULUM_POSITION, [(0, 2, 16, "relu"), (1, 16, 16, "identity"), (1, 16, 16, "identity"), (0, 16, 2, "identity")], 2, 32, 40, 20, 8, 60),     # the reference's recurrent SAC actor on the Pendulum without velocity
    (capi.ENV_CAR, [(0, 6, 32, "relu"), (0, 32, 2, "tanh")], 1, 50, 25, 9, 0, 40),                                   # a policy of dense layers, deterministic
    # sixteen environments or fewer and dense layers: the whole step is one launch
    (capi.ENV_ACROBOT_SWINGUP, [(0, 6, 256, "fast_tanh"), (0, 256, 256, "fast_tanh"), (0, 256, 2, "identity")], 2, 1, 40, 15, 0, 90),        # the zoo's SAC actor of width 256, one environment
    (capi.ENV_ACROBOT, [(0, 6, 200, "relu"), (0, 200, 100, "relu"), (0, 100, 1, "tanh")], 3, 4, 20, 10, 0, 50),
    (capi.ENV_CAR, [(0, 6, 48, "tanh"), (0, 48, 2, "tanh")], 1, 9, 25, 9, 0, 40),
    (capi.ENV_PENDULUM_POSITION, [(0, 2, 64, "relu"), (0, 64, 64, "relu"), (0, 64, 64, "relu"), (0, 64, 2, "identity")], 2, 16, 12, 7, 0, 40),
])
def test_env_runner_step_with_a_sequential_policy(oracle, rocm, kind, specs, head_kind, n_envs, capacity, limit, period, steps):
    sd, od, ad = capi.ENV_DIMS[kind]
    rng = np.random.default_rng(kind + 40)
    params = helpers.random_seq_params(rng, specs)
    draws = [(initial_states(rng, kind, n_envs), rng.standard_normal((n_envs, ad)).astype(np.float32)) for _ in range(steps)]
    recurrent = any(k for k, *_ in specs)
    results = []
    for backend in (oracle, rocm):
        runner = helpers.EnvRunnerOnBackend(backend, kind, n_envs, limit)
        rb = helpers.ReplayOnBackend(backend, n_envs, capacity, od, ad)
        policy = helpers.SeqNet(backend, specs, params, 1, n_envs, trainable=False)
        state = helpers.SeqStateOnBackend(backend, specs, n_envs)
        sas = capi.SasParameters(-20.0, 2.0, 1e-6, -float(ad))
        ws, wsn = (None, 0)
        if backend.name == "rocm":
            ws, wsn = backend.workspace(backend.device.lib.rlt_rocm_env_runner_step_sequential_workspace_bytes(C.byref(runner.c), policy.layers, policy.n))
        trace = []
        for ini, noise in draws:
            i_d, n_d = backend.array(ini), backend.array(noise)
            backend.call("env_runner_step_sequential", C.byref(runner.c), C.byref(rb.c), policy.layers, policy.n, C.byref(state.c) if recurrent else None, period, head_kind,
                         C.byref(sas), 0.3, n_d.ptr, i_d.ptr, ws, wsn)
            backend.sync()
            trace.append(runner.snapshot() + list(state.numpy()[0]) + list(state.numpy()[1]))
        results.append((trace, [a.numpy() for a in (rb.data, rb.episode_start, rb.position, rb.current_episode_start, rb.full)]))
    (ref_trace, ref_rb), (got_trace, got_rb) = results
    tol = 1e-4 if kind in (capi.ENV_ACROBOT, capi.ENV_ACROBOT_SWINGUP) else 1e-5
    for step, (ref, got) in enumerate(zip(ref_trace, got_trace)):
        for k, (a, b) in enumerate(zip(got, ref)):
            if a.dtype in (np.uint8, np.uint32):
                assert np.array_equal(a, b), (step, k)
            else:
                # relative to the tensor's largest magnitude, which for one environment is one number that may be close to zero: not below 0.1
                assert np.abs(a - b).max() <= tol * max(0.1, np.abs(b).max()), (step, k, np.abs(a - b).max(), np.abs(b).max())
    assert rel_err(got_rb[0], ref_rb[0]) <= tol and all(np.array_equal(got_rb[k], ref_rb[k]) for k in range(1, 5))
    assert ref_rb[4].all()
    if head_kind == 3 and n_envs >= 32:      # the exploration head clipped some actions
        acts = np.concatenate([t[5] for t in ref_trace])
        assert np.abs(acts).max() <= 1.0 and (np.abs(acts) == 1.0).any()


INITIAL_RANGES = {      # the environments' sample_initial_state: each state component uniform in [low, high]
    capi.ENV_PENDULUM: ([-np.pi, -1.0], [np.pi, 1.0]),                                   # rl/environments/pendulum/operations_generic.h:40-45
    capi.ENV_PENDULUM_POSITION: ([-np.pi, -1.0, 0.0], [np.pi, 1.0, 0.0]),
    capi.ENV_ACROBOT: ([-0.1] * 4, [0.1] * 4),                                           # rl/environments/acrobot/operations_generic.h:39-52
    capi.ENV_ACROBOT_SWINGUP: ([-0.1] * 4, [0.1] * 4),
}


@pytest.mark.parametrize("kind,specs,head_kind,n_envs,capacity,limit,steps", [
    (capi.ENV_ACROBOT_SWINGUP, [(0, 6, 256, "fast_tanh"), (0, 256, 256, "fast_tanh"), (0, 256, 2, "identity")], 2, 1, 40, 15, 60),
    (capi.ENV_ACROBOT_SWINGUP, [], 0, 1, 40, 15, 40),                                    # the warm-up phase: uniform actions, no policy
    (capi.ENV_PENDULUM, [(0, 3, 64, "relu"), (0, 64, 64, "relu"), (0, 64, 1, "tanh")], 3, 16, 20, 9, 40),
    (capi.ENV_PENDULUM_POSITION, [(0, 2, 32, "relu"), (0, 32, 1, "tanh")], 1, 5, 20, 9, 30),
    (capi.ENV_ACROBOT, [], 0, 7, 20, 30, 50),
])
def test_env_runner_step_that_draws_inside_the_launch_matches_the_one_fed_with_arrays(rocm, kind, specs, head_kind, n_envs, capacity, limit, steps):
    """rlt_rocm_env_runner_step_drawn against the same step fed with arrays that rlt_rocm_rand_f32 / rlt_rocm_randn_f32 filled from the same seed and streams."""
    sd, od, ad = capi.ENV_DIMS[kind]
    rng = np.random.default_rng(kind + 70)
    params = helpers.random_seq_params(rng, specs) if specs else None
    low, high = (np.asarray(v, np.float32) for v in INITIAL_RANGES[kind])
    seed = 20240
    sas = capi.SasParameters(-20.0, 2.0, 1e-6, -float(ad))
    results = []
    for drawn in (False, True):
        runner = helpers.EnvRunnerOnBackend(rocm, kind, n_envs, limit)
        rb = helpers.ReplayOnBackend(rocm, n_envs, capacity, od, ad)
        policy = helpers.SeqNet(rocm, specs, params, 1, n_envs, trainable=False) if specs else None
        layers, n_layers = (policy.layers, policy.n) if policy else (None, 0)
        u, noise = rocm.zeros((n_envs, sd)), rocm.zeros((n_envs, ad))
        ws, wsn = rocm.workspace(rocm.device.lib.rlt_rocm_env_runner_step_sequential_workspace_bytes(C.byref(runner.c), layers, n_layers)) if specs else (None, 0)
        trace = []
        for step in range(steps):
            noise_stream, initial_stream = 100 + 2 * step, 101 + 2 * step
            if drawn:
                rocm.call("env_runner_step_drawn", C.byref(runner.c), C.byref(rb.c), layers, n_layers, head_kind, C.byref(sas), 0.3, low.ctypes.data, high.ctypes.data,
                          noise.ptr, seed, noise_stream, initial_stream)
            else:
                rocm.call("rand_f32", u.ptr, n_envs * sd, 0.0, 1.0, seed, initial_stream)
                rocm.sync()
                ini = rocm.array((low + (high - low) * u.numpy()).astype(np.float32))
                if head_kind == 0:
                    rocm.call("rand_f32", noise.ptr, n_envs * ad, -1.0, 1.0, seed, noise_stream)
                    rocm.call("env_runner_step", C.byref(runner.c), C.byref(rb.c), 0, None, 0, C.byref(sas), noise.ptr, None, ini.ptr, None, 0)
                else:
                    rocm.call("randn_f32", noise.ptr, n_envs * ad, seed, noise_stream)
                    rocm.call("env_runner_step_sequential", C.byref(runner.c), C.byref(rb.c), layers, n_layers, None, 0, head_kind, C.byref(sas), 0.3, noise.ptr, ini.ptr, ws, wsn)
            rocm.sync()
            trace.append(runner.snapshot() + [noise.numpy()])
        results.append((trace, [a.numpy() for a in (rb.data, rb.episode_start, rb.position, rb.current_episode_start, rb.full)]))
    (ref_trace, ref_rb), (got_trace, got_rb) = results
    n_reset = 0
    for step, (ref, got) in enumerate(zip(ref_trace, got_trace)):
        n_reset += int(ref[3].sum())
        for k, (a, b) in enumerate(zip(got, ref)):
            if a.dtype in (np.uint8, np.uint32):
                assert np.array_equal(a, b), (step, k)
            else:      # the initial states' low + (high - low) * u may round once or twice (fused or not)
                assert np.abs(a - b).max() <= 2e-6 * max(1.0, np.abs(b).max()), (step, k, np.abs(a - b).max())
    assert n_reset > 0           # episodes ended and the next step drew new initial states
    assert np.abs(got_rb[0] - ref_rb[0]).max() <= 2e-6 * max(1.0, np.abs(ref_rb[0]).max()) and all(np.array_equal(got_rb[k], ref_rb[k]) for k in range(1, 5))

    # a recurrent or wider policy, or more environments: the caller draws into arrays
    many = helpers.EnvRunnerOnBackend(rocm, kind, 17, limit)
    many_rb = helpers.ReplayOnBackend(rocm, 17, capacity, od, ad)
    lib, h = rocm.device.lib, rocm.device.handle
    assert lib.rlt_rocm_env_runner_step_drawn(h, C.byref(many.c), C.byref(many_rb.c), None, 0, 0, C.byref(sas), 0.3, low.ctypes.data, high.ctypes.data, None, seed, 1, 2) == capi.RLT_E_UNSUPPORTED
