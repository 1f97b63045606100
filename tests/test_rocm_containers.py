"""Container and generator entry points of the C ABI (the reference pins its CUDA containers the same way: copies there and back with
abs_diff == 0, views of wider matrices, tests/src/nn/cuda/cuda_basics.cu:25-351). Copies, fills and the generator's words are checked
bit for bit; float conversions of the generator to the last-bit differences of the device's log / sincos."""
import ctypes as C

import numpy as np
import pytest
from scipy import stats

import helpers
from helpers import capi

pytestmark = pytest.mark.gpu


def test_round_trip_is_exact(rocm):
    """COPY_CONTAINER: host -> device -> host returns the bytes; a changed element shows up as exactly that difference."""
    rng = np.random.default_rng(0)
    for shape in [(1, 1), (10, 10), (100, 100), (257, 33)]:
        m = rng.standard_normal(shape).astype(np.float32)
        d = rocm.array(m)
        assert np.array_equal(d.numpy(), m)
        m2 = m.copy(); m2[0, 0] += 17.0
        d.upload(m2)
        assert abs(float(np.abs(d.numpy().astype(np.float64) - m).sum()) - 17.0) < 1e-4
    for dtype in (np.uint8, np.uint32, np.float64):
        m = (rng.random(1000) * 200).astype(dtype)
        assert np.array_equal(rocm.array(m).numpy(), m)


def test_device_to_device_copy(rocm):
    rng = np.random.default_rng(1)
    m = rng.standard_normal((300, 70)).astype(np.float32)
    a, b = rocm.array(m), rocm.zeros(m.shape)
    rocm.call("memcpy_d2d", b.ptr, a.ptr, m.nbytes)
    rocm.sync()
    assert np.array_equal(b.numpy(), m)
    # a sub-range at an offset that is not a multiple of anything
    c = rocm.zeros((1000,))
    rocm.call("memcpy_d2d", c.offset(13), a.offset(7), 501 * 4)
    rocm.sync()
    expected = np.zeros(1000, np.float32); expected[13:13 + 501] = m.ravel()[7:7 + 501]
    assert np.array_equal(c.numpy(), expected)
    rocm.call("memcpy_d2d", c.ptr, a.ptr, 0)      # empty copy: accepted, nothing happens
    rocm.sync()
    assert np.array_equal(c.numpy(), expected)


@pytest.mark.parametrize("rows,cols,off_r,off_c,view_r,view_c", [(100, 100, 25, 25, 50, 50), (50, 10, 5, 5, 40, 5), (7, 129, 0, 1, 7, 127), (64, 64, 63, 0, 1, 64)])
def test_strided_views_all_three_kinds(rocm, rows, cols, off_r, off_c, view_r, view_c):
    """COPYING_VIEWS: a view of a wider matrix copied host -> device, device -> device into a view of another pitch, device -> host into a
    third pitch; everything outside the views stays what it was."""
    rng = np.random.default_rng(rows * cols)
    host = rng.standard_normal((rows, cols)).astype(np.float32)
    view = host[off_r:off_r + view_r, off_c:off_c + view_c]
    # host view -> view of a device matrix with another pitch
    d_rows, d_cols = view_r + 3, view_c + 9
    background = rng.standard_normal((d_rows, d_cols)).astype(np.float32)
    d = rocm.array(background)
    rocm.call("memcpy2d", d.offset(2 * d_cols + 4), d_cols * 4, host.ctypes.data + (off_r * cols + off_c) * 4, cols * 4, view_c * 4, view_r, 1)
    expected = background.copy(); expected[2:2 + view_r, 4:4 + view_c] = view
    assert np.array_equal(d.numpy(), expected)
    # device view -> device view (a third pitch)
    e_cols = view_c + 2
    background2 = rng.standard_normal((view_r + 1, e_cols)).astype(np.float32)
    e = rocm.array(background2)
    rocm.call("memcpy2d", e.offset(1 * e_cols + 1), e_cols * 4, d.offset(2 * d_cols + 4), d_cols * 4, view_c * 4, view_r, 0)
    rocm.sync()
    expected2 = background2.copy(); expected2[1:1 + view_r, 1:1 + view_c] = view
    assert np.array_equal(e.numpy(), expected2)
    # device view -> host view
    back = np.full((rows, cols), -7.0, np.float32)
    rocm.call("memcpy2d", back.ctypes.data + (off_r * cols + off_c) * 4, cols * 4, e.offset(1 * e_cols + 1), e_cols * 4, view_c * 4, view_r, 2)
    expected3 = np.full((rows, cols), -7.0, np.float32); expected3[off_r:off_r + view_r, off_c:off_c + view_c] = view
    assert np.array_equal(back, expected3)


def test_strided_copy_rejects_bad_arguments(rocm):
    d = rocm.zeros((4, 4))
    host = np.zeros((4, 4), np.float32)
    lib, h = rocm.device.lib, rocm.device.handle
    assert lib.rlt_rocm_memcpy2d(h, d.ptr, 8, host.ctypes.data, 16, 16, 4, 1) == capi.RLT_E_INVALID_ARGUMENT      # destination pitch below the width
    assert lib.rlt_rocm_memcpy2d(h, d.ptr, 16, host.ctypes.data, 16, 16, 4, 3) == capi.RLT_E_INVALID_ARGUMENT     # unknown kind
    assert lib.rlt_rocm_memcpy2d(h, None, 16, host.ctypes.data, 16, 16, 4, 1) == capi.RLT_E_INVALID_ARGUMENT
    assert lib.rlt_rocm_memcpy2d(h, d.ptr, 16, host.ctypes.data, 16, 0, 4, 1) == 0                            # empty: accepted


def test_set_all_on_a_view_leaves_the_pitch_gap_alone(rocm):
    rng = np.random.default_rng(3)
    for rows, cols, ld in [(13, 7, 11), (1, 1, 5), (300, 64, 64), (129, 3, 257)]:
        background = rng.standard_normal((rows, ld)).astype(np.float32)
        d = rocm.array(background)
        rocm.call("fill_f32", d.ptr, rows, cols, ld, 2.5)
        rocm.sync()
        expected = background.copy(); expected[:, :cols] = 2.5
        assert np.array_equal(d.numpy(), expected)
    b = rocm.array(np.arange(1000, dtype=np.uint8))
    rocm.call("fill_u8", b.offset(3), 990, 201)
    rocm.sync()
    expected = np.arange(1000, dtype=np.uint8); expected[3:993] = 201
    assert np.array_equal(b.numpy(), expected)


def test_sums_match_the_checker(oracle, rocm):
    rng = np.random.default_rng(4)
    for n in (1, 63, 4546, 71_942, 1_000_003):
        x = (rng.standard_normal(n) * (1 + 3 * rng.random(n))).astype(np.float32)
        for squared in (0, 1):
            res = []
            for b in (oracle, rocm):
                xd, out = b.array(x), b.zeros((1,))
                b.call("reduce_sum_f32", xd.ptr, n, squared, out.ptr)
                b.sync()
                res.append(float(out.numpy()[0]))
            scale = float(np.abs(x.astype(np.float64) ** (2 if squared else 1)).sum())
            assert abs(res[1] - res[0]) <= 1e-6 * scale, (n, squared, res)
    m = (rng.random(100_000) < 0.3).astype(np.uint8); m[m != 0] = rng.integers(1, 255, int(m.sum()))     # any non-zero byte counts as true
    out = rocm.zeros((1,))
    rocm.call("cast_reduce_sum_u8", rocm.array(m).ptr, len(m), out.ptr)
    rocm.sync()
    assert out.numpy()[0] == float((m != 0).sum())


def test_gradient_norm_of_a_network(oracle, rocm):
    """gradient_norm(mlp) = sum over the layers' weight and bias gradients of their squared sums (nn_models/mlp/operations_generic.h:367-377)."""
    rng = np.random.default_rng(5)
    dims = (17, 256, 256, 6)
    g = rng.standard_normal(helpers.mlp_param_count(dims)).astype(np.float32)
    gd, out = rocm.array(g), rocm.zeros((1,))
    rocm.call("reduce_sum_f32", gd.ptr, len(g), 1, out.ptr)
    rocm.sync()
    layerwise, off = 0.0, 0
    for i in range(3):
        for count in (dims[i] * dims[i + 1], dims[i + 1]):
            layerwise += float((g[off:off + count].astype(np.float64) ** 2).sum()); off += count
    assert abs(out.numpy()[0] - layerwise) <= 1e-6 * layerwise


def test_adam_reset_then_step_matches_the_checker(oracle, rocm):
    rng = np.random.default_rng(6)
    n = 4546
    p, g = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    m, v = rng.standard_normal(n).astype(np.float32), np.abs(rng.standard_normal(n)).astype(np.float32)
    params = capi.AdamParameters(1e-3, 0.9, 0.999, 1e-7, 1e-7, 0.0, 1.0, 0, 0, 0, 0.0)
    res = []
    for b in (oracle, rocm):
        pd, gd, md, vd = b.array(p), b.array(g), b.array(m), b.array(v)
        age = b.array(np.array([23], np.uint32))
        t = capi.AdamTensor()
        t.parameters, t.gradient, t.first_moment, t.second_moment, t.count, t.flags = pd.ptr, gd.ptr, md.ptr, vd.ptr, n, 1
        b.call("adam_reset", C.byref(t), 1, age.ptr)
        b.sync()
        after_reset = (md.numpy().copy(), vd.numpy().copy(), age.numpy().copy())
        for _ in range(2):
            b.call("adam_step", C.byref(t), 1, C.byref(params), age.ptr, 1.0, None)
        b.sync()
        res.append(after_reset + (pd.numpy(), md.numpy(), vd.numpy(), age.numpy()))
    for r in res:
        assert not r[0].any() and not r[1].any() and r[2][0] == 1 and r[6][0] == 3
    for i in (3, 4, 5):
        assert helpers.rel_err(res[1][i], res[0][i]) <= 1e-5


# ---------------------------------------------------------------- generator

def device_bits(rocm, n, seed, stream):
    d = rocm.zeros((n,), np.uint32)
    rocm.call("rand_bits_u32", d.ptr, n, seed, stream)
    rocm.sync()
    return d.numpy()


def oracle_bits(oracle, n, seed, stream):
    out = np.zeros(n, np.uint32)
    assert oracle.lib.rlt_oracle_rand_bits_u32(out.ctypes.data, n, seed, stream) == 0
    return out


# Random123's known-answer entries for philox4x32 with 10 rounds, read as (index, stream, seed) -> four words
KAT = [(0, 0, 0, (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
       (2**64 - 1, 2**64 - 1, 2**64 - 1, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
       (0x85a308d3243f6a88, 0x0370734413198a2e, 0x299f31d0a4093822, (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1))]


def test_generator_words_are_philox4x32_10(oracle, rocm):
    # the published vectors whose group index is small enough to ask for directly
    assert [hex(v) for v in device_bits(rocm, 4, 0, 0)] == [hex(v) for v in KAT[0][3]]
    # all three through the checker's block function = the device's stream words on the same (seed, stream), bit for bit
    for seed, stream, n in [(0, 0, 4099), (KAT[2][2], KAT[2][1], 1003), (2**64 - 1, 2**64 - 1, 64), (12345, 2**33 + 7, 1_000_001)]:
        assert np.array_equal(device_bits(rocm, n, seed, stream), oracle_bits(oracle, n, seed, stream)), (seed, stream)


def test_consecutive_streams_share_nothing(rocm):
    """Two calls that differ by one in `stream` draw from disjoint sequences (a caller passes a counter it increments per call)."""
    n = 256
    for k in (0, 1, 2, 1000, 2**32 - 1):
        a, b = rocm.zeros((n,)), rocm.zeros((n,))
        rocm.call("randn_f32", a.ptr, n, 99, k)
        rocm.call("randn_f32", b.ptr, n, 99, k + 1)
        rocm.sync()
        assert len(np.intersect1d(a.numpy(), b.numpy())) == 0
        ua, ub = device_bits(rocm, 4096, 99, k), device_bits(rocm, 4096, 99, k + 1)
        assert len(np.intersect1d(ua, ub)) <= 2
    # many short calls, as a training loop makes them: 2,000 calls x 256 values, no value twice except by 24-bit coincidence
    calls = np.stack([device_bits(rocm, 256, 5, s) for s in range(200)])
    assert len(np.unique(calls)) >= calls.size - 20          # 51,200^2 / 2^33 = 0.3 expected coincidences
    # a different seed is a different sequence too
    assert len(np.intersect1d(device_bits(rocm, 4096, 1, 7), device_bits(rocm, 4096, 2, 7))) <= 2


def test_uniform_and_normal_draws(oracle, rocm):
    n = 1_000_000
    u, z, v = rocm.zeros((n,)), rocm.zeros((n,)), rocm.zeros((n,))
    rocm.call("rand_f32", u.ptr, n, 0.0, 1.0, 11, 2)
    rocm.call("randn_f32", z.ptr, n, 5, 9)
    rocm.call("rand_f32", v.ptr, n, -3.0, 5.0, 11, 2)
    rocm.sync()
    u, z, v = u.numpy(), z.numpy(), v.numpy()
    ou, oz = np.zeros(n, np.float32), np.zeros(n, np.float32)
    oracle.lib.rlt_oracle_rand_f32(ou.ctypes.data, n, 0.0, 1.0, 11, 2)
    oracle.lib.rlt_oracle_randn_f32(oz.ctypes.data, n, 5, 9)
    assert np.array_equal(u, ou)                            # cell midpoints are exact in fp32
    assert np.max(np.abs(z - oz)) <= 2e-6 * max(1.0, np.max(np.abs(oz)))
    assert np.max(np.abs(v - (-3.0 + 8.0 * u.astype(np.float64)))) <= 1e-6
    assert u.min() > 0 and u.max() < 1 and v.min() >= -3 and v.max() <= 5
    zd = z.astype(np.float64)
    assert stats.kstest(u.astype(np.float64), "uniform").statistic < 1.95 / np.sqrt(n)
    assert stats.kstest(zd, "norm").statistic < 1.95 / np.sqrt(n)
    assert abs(zd.mean()) < 4 / np.sqrt(n) and abs(zd.var() - 1) < 4 * np.sqrt(2 / n)
    assert abs(stats.skew(zd)) < 4 * np.sqrt(6 / n) and abs(stats.kurtosis(zd)) < 4 * np.sqrt(24 / n)
    # a count that is no multiple of four, and a tiny one
    for count in (1, 2, 3, 5, 1023):
        d = rocm.array(np.full(count + 4, 7.0, np.float32))
        rocm.call("randn_f32", d.ptr, count, 5, 9)
        rocm.sync()
        got = d.numpy()
        assert np.max(np.abs(got[:count] - oz[:count])) <= 1e-5 and np.all(got[count:] == 7.0)


def test_gather_draw_matches_the_checker(oracle, rocm):
    n_envs, capacity, batch = 5, 1000, 100_000
    position = np.array([10, 999, 0, 500, 1], np.uint32)
    full = np.array([0, 0, 1, 1, 0], np.uint8)
    res = []
    for b in (oracle, rocm):
        pos, fl = b.array(position), b.array(full)
        rb = capi.ReplayBuffer()
        rb.data = b.zeros((n_envs * capacity * 10,)).ptr
        rb.episode_start = b.zeros((n_envs * capacity,), np.uint32).ptr
        rb.position, rb.full, rb.current_episode_start = pos.ptr, fl.ptr, b.zeros((n_envs,), np.uint32).ptr
        rb.n_envs, rb.capacity, rb.observation_dim, rb.action_dim = n_envs, capacity, 3, 1
        env, off = b.zeros((batch,), np.uint32), b.zeros((batch,), np.uint32)
        if b is oracle:
            assert oracle.lib.rlt_oracle_gather_draw(C.byref(rb), batch, 3, 77, env.ptr, off.ptr) == 0
        else:
            b.call("gather_draw", C.byref(rb), batch, 3, 77, env.ptr, off.ptr)
        b.sync()
        res.append((env.numpy(), off.numpy()))
    assert np.array_equal(res[1][0], res[0][0]) and np.array_equal(res[1][1], res[0][1])
    # two consecutive calls do not repeat each other's draws
    pos, fl = rocm.array(np.array([0], np.uint32)), rocm.array(np.array([1], np.uint8))
    rb = capi.ReplayBuffer()
    rb.data, rb.episode_start = rocm.zeros((10_000 * 10,)).ptr, rocm.zeros((10_000,), np.uint32).ptr
    rb.position, rb.full, rb.current_episode_start = pos.ptr, fl.ptr, rocm.zeros((1,), np.uint32).ptr
    rb.n_envs, rb.capacity, rb.observation_dim, rb.action_dim = 1, 10_000, 3, 1
    offs = []
    for k in (40, 41):
        env, off = rocm.zeros((256,), np.uint32), rocm.zeros((256,), np.uint32)
        rocm.call("gather_draw", C.byref(rb), 256, 3, k, env.ptr, off.ptr)
        rocm.sync()
        offs.append(off.numpy())
    assert not np.array_equal(offs[0][4:], offs[1][:-4]) and not np.array_equal(offs[0][1:], offs[1][:-1])
    assert (offs[0] == offs[1]).sum() <= 3


def test_runner_reset_draws_match_the_checker(oracle, rocm):
    """Environments that reset without given initial states draw theirs from the call's stream, on the one-launch path (an actor
    3 -> 64 -> 64 -> 1) and on the per-kernel path (given actions) alike."""
    n = 4096
    for fused in (True, False):
        rb = helpers.ReplayOnBackend(rocm, n, 8)
        states, ep_step, ep_ret = rocm.zeros((n, 2)), rocm.zeros((n,), np.uint32), rocm.zeros((n,))
        trunc = rocm.array(np.ones(n, np.uint8))
        rn = capi.PendulumRunner(states.ptr, ep_step.ptr, ep_ret.ptr, trunc.ptr, n, 200, capi.pendulum_parameters())
        stream = 1000 + int(fused)
        if fused:      # all-zero actor: the action is tanh(0) = 0
            actor = helpers.Mlp(rocm, (3, 64, 64, 1), np.zeros(helpers.mlp_param_count((3, 64, 64, 1)), np.float32), n, "relu", "tanh", trainable=False)
            rocm.call("pendulum_runner_step", C.byref(rn), C.byref(rb.c), 1, actor.layers, 3, None, None, None, None, 21, stream)
        else:
            actions = rocm.zeros((n, 1))
            rocm.call("pendulum_runner_step", C.byref(rn), C.byref(rb.c), 0, None, 0, None, actions.ptr, None, None, 21, stream)
        rocm.sync()
        expected = np.zeros((n, 2), np.float32)
        assert oracle.lib.rlt_oracle_pendulum_initial_states(expected.ctypes.data, n, 21, stream) == 0
        # the replay row holds the observation of the drawn state: (cos theta, sin theta, theta_dot)
        rows = rb.data.numpy().reshape(n, 8, 10)[:, 0, :]
        th, thd = expected[:, 0].astype(np.float64), expected[:, 1].astype(np.float64)
        assert np.max(np.abs(rows[:, 0] - np.cos(th))) <= 1e-6 and np.max(np.abs(rows[:, 1] - np.sin(th))) <= 1e-6
        assert np.array_equal(rows[:, 2], expected[:, 1])
        # and the state after the step with zero torque follows from it
        thd1 = np.clip(thd + 15.0 * np.sin(th) * 0.05, -8, 8)
        got = states.numpy()
        assert np.max(np.abs(got[:, 1] - thd1)) <= 1e-5 and np.max(np.abs(got[:, 0] - (th + thd1 * 0.05))) <= 1e-5


def test_set_stream_routes_work_to_the_callers_stream(rocm):
    """A caller-owned stream is adopted and released again (devices/cuda.h keeps one stream in the device object)."""
    hip = C.CDLL("libamdhip64.so")          # the HIP runtime the library itself is linked against
    s = C.c_void_p()
    assert hip.hipStreamCreate(C.byref(s)) == 0
    lib, h = rocm.device.lib, rocm.device.handle
    lib.rlt_rocm_get_stream.restype = C.c_void_p
    own = lib.rlt_rocm_get_stream(h)
    assert own and own != s.value
    assert lib.rlt_rocm_set_stream(h, s) == 0
    assert lib.rlt_rocm_get_stream(h) == s.value
    d = rocm.zeros((100_000,))
    rocm.call("fill_f32", d.ptr, 1, 100_000, 100_000, 3.0)
    assert hip.hipStreamSynchronize(s) == 0                # only the caller's stream is waited for
    assert lib.rlt_rocm_set_stream(h, None) == 0 and lib.rlt_rocm_get_stream(h) == own
    assert np.all(d.numpy() == 3.0)
    assert hip.hipStreamDestroy(s) == 0


@pytest.mark.parametrize("S,from_initial", [(1, 0), (7, 0), (16, 1)])
def test_gather_sequence_draw_matches_the_checker(oracle, rocm, S, from_initial):
    n_envs, capacity, batch, limit = 4, 2000, 20_000, 200
    padded = S + 1
    position = np.array([10, 1999, 0, 700], np.uint32)
    full = np.array([0, 0, 1, 1], np.uint8)
    res = []
    for b in (oracle, rocm):
        pos, fl = b.array(position), b.array(full)
        rb = capi.ReplayBuffer()
        rb.data = b.zeros((n_envs * capacity * 10,)).ptr
        rb.episode_start = b.zeros((n_envs * capacity,), np.uint32).ptr
        rb.position, rb.full, rb.current_episode_start = pos.ptr, fl.ptr, b.zeros((n_envs,), np.uint32).ptr
        rb.n_envs, rb.capacity, rb.observation_dim, rb.action_dim = n_envs, capacity, 3, 1
        P = capi.SequenceSampling()
        P.always_sample_from_initial_state, P.random_seq_length, P.enable_nominal_sequence_length_probability, P.nominal_sequence_length_probability = from_initial, 1, 1, 0.3
        env, off = b.zeros((batch,), np.uint32), b.zeros((batch, padded), np.uint32)
        nominal, lengths = b.zeros((batch, padded + 1), np.uint8), b.zeros((batch, padded + 1), np.uint32)
        if b is oracle:
            assert oracle.lib.rlt_oracle_gather_sequence_draw(C.byref(rb), C.byref(P), limit, batch, S, 5, 11, env.ptr, off.ptr, nominal.ptr, lengths.ptr) == 0
        else:
            b.call("gather_sequence_draw", C.byref(rb), C.byref(P), limit, batch, S, 5, 11, env.ptr, off.ptr, nominal.ptr, lengths.ptr)
        b.sync()
        res.append([a.numpy() for a in (env, off, nominal, lengths)])
    for want, got in zip(*res):
        assert np.array_equal(got, want)
