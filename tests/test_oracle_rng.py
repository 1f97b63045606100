"""The CPU restatement of the device's random draws (oracle/rlt_oracle_rng.cpp) against what fixes it from outside:
the published known-answer vectors of Philox4x32-10, and the distributions the conversions must produce."""
import ctypes as C

import numpy as np
import pytest
from scipy import stats

import helpers


@pytest.fixture(scope="module")
def lib():
    return helpers.load_oracle()


# Random123's known-answer file, entries "philox4x32 10": counter words, key words, expected output words
PHILOX4X32_10_KAT = [
    ((0x00000000, 0x00000000, 0x00000000, 0x00000000), (0x00000000, 0x00000000), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
    ((0xffffffff, 0xffffffff, 0xffffffff, 0xffffffff), (0xffffffff, 0xffffffff), (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
    ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0), (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
]


@pytest.mark.parametrize("counter,key,expected", PHILOX4X32_10_KAT)
def test_block_function_reproduces_the_published_vectors(lib, counter, key, expected):
    c, k, out = np.array(counter, np.uint32), np.array(key, np.uint32), np.zeros(4, np.uint32)
    assert lib.rlt_oracle_philox4x32_10(c.ctypes.data, k.ctypes.data, out.ctypes.data) == 0
    assert [hex(v) for v in out] == [hex(v) for v in expected]


def bits(lib, n, seed, stream):
    out = np.zeros(n, np.uint32)
    assert lib.rlt_oracle_rand_bits_u32(out.ctypes.data, n, seed, stream) == 0
    return out


def test_the_stream_words_are_the_block_function_on_the_documented_counter(lib):
    """element i = word i % 4 of the block at counter (index low, index high, stream low, stream high) under key (seed low, seed high)"""
    seed, stream = 0x299f31d0a4093822, 0x0370734413198a2e
    got = bits(lib, 4 * 5 + 3, seed, stream)
    for index in range(6):
        c = np.array([index, 0, stream & 0xffffffff, stream >> 32], np.uint32)
        k = np.array([seed & 0xffffffff, seed >> 32], np.uint32)
        out = np.zeros(4, np.uint32)
        lib.rlt_oracle_philox4x32_10(c.ctypes.data, k.ctypes.data, out.ctypes.data)
        n = min(4, len(got) - 4 * index)
        assert np.array_equal(got[4 * index:4 * index + n], out[:n])
    # the third published vector read through this mapping: index = its counter words 0, 1; stream = words 2, 3
    index = 0x85a308d3243f6a88
    c = np.array([index & 0xffffffff, index >> 32, stream & 0xffffffff, stream >> 32], np.uint32)
    out = np.zeros(4, np.uint32)
    lib.rlt_oracle_philox4x32_10(c.ctypes.data, np.array([seed & 0xffffffff, seed >> 32], np.uint32).ctypes.data, out.ctypes.data)
    assert [hex(v) for v in out] == [hex(v) for v in PHILOX4X32_10_KAT[2][2]]


def test_no_group_repeats_across_streams_seeds_and_indices(lib):
    """Philox is a bijection of the counter for a fixed key: 10^6 distinct (seed, stream, index) triples give 10^6 distinct groups.
    Consecutive stream numbers in particular share nothing (the defect of a generator whose second argument merely shifts the index)."""
    groups = []
    for seed in (0, 1, 2**63 + 5):
        for stream in (0, 1, 2, 3, 2**32, 2**40 + 1):
            groups.append(bits(lib, 4 * 55_556, seed, stream).reshape(-1, 4))
    g = np.concatenate(groups)
    assert len(g) >= 1_000_000
    packed = g.view([("a", np.uint32), ("b", np.uint32), ("c", np.uint32), ("d", np.uint32)]).ravel()
    assert len(np.unique(packed)) == len(packed)
    # and no single 32-bit word sequence of stream k reappears shifted in stream k + 1
    a, b = bits(lib, 4096, 7, 10), bits(lib, 4096, 7, 11)
    assert len(np.intersect1d(a, b)) <= 2      # 4096^2 / 2^32 = 0.004 expected coincidences


def test_bits_are_balanced(lib):
    w = bits(lib, 1 << 20, 42, 3)
    ones = np.array([((w >> b) & 1).mean() for b in range(32)])
    assert np.all(np.abs(ones - 0.5) < 4 * 0.5 / np.sqrt(len(w)))       # every bit position: 4 standard errors
    # serial correlation of consecutive words
    x = w.astype(np.float64) / 2**32 - 0.5
    assert abs(np.mean(x[:-1] * x[1:]) * 12) < 4 / np.sqrt(len(w))


def test_uniform_conversion(lib):
    n = 1_000_000
    u = np.zeros(n, np.float32)
    assert lib.rlt_oracle_rand_f32(u.ctypes.data, n, 0.0, 1.0, 11, 2) == 0
    w = bits(lib, n, 11, 2)
    assert np.array_equal(u, ((w >> 8).astype(np.float32) + np.float32(0.5)) * np.float32(2.0 ** -24))     # cell midpoints: exact in fp32
    assert u.min() > 0.0 and u.max() < 1.0
    assert stats.kstest(u.astype(np.float64), "uniform").statistic < 1.95 / np.sqrt(n)      # p > 0.001
    v = np.zeros(n, np.float32)
    lib.rlt_oracle_rand_f32(v.ctypes.data, n, -3.0, 5.0, 11, 2)
    assert np.allclose(v, -3.0 + 8.0 * u.astype(np.float64), atol=1e-6) and v.min() >= -3.0 and v.max() <= 5.0


def test_normal_conversion(lib):
    n = 1_000_000
    z = np.zeros(n, np.float32)
    assert lib.rlt_oracle_randn_f32(z.ctypes.data, n, 5, 9) == 0
    zd = z.astype(np.float64)
    assert abs(zd.mean()) < 4 / np.sqrt(n)
    assert abs(zd.var() - 1) < 4 * np.sqrt(2 / n)
    assert abs(stats.skew(zd)) < 4 * np.sqrt(6 / n) and abs(stats.kurtosis(zd)) < 4 * np.sqrt(24 / n)
    assert stats.kstest(zd, "norm").statistic < 1.95 / np.sqrt(n)
    # the Box-Muller pairing: elements (0, 1) of a group share a radius, as do (2, 3)
    w = bits(lib, 8, 5, 9).reshape(2, 4)
    unit = lambda x: ((x >> 8).astype(np.float64) + 0.5) * 2.0 ** -24
    for gi in range(2):
        for pair in range(2):
            r, a = np.sqrt(-2 * np.log(unit(w[gi, 2 * pair]))), 2 * np.pi * unit(w[gi, 2 * pair + 1])
            assert np.allclose(z[4 * gi + 2 * pair: 4 * gi + 2 * pair + 2], [r * np.cos(a), r * np.sin(a)], atol=2e-6)
    # the two elements of a pair are uncorrelated, and so are neighbouring groups
    assert abs(np.mean(zd[0::2] * zd[1::2])) < 4 / np.sqrt(n / 2)
    assert abs(np.mean(zd[:-4] * zd[4:])) < 4 / np.sqrt(n)


def test_gather_draw_is_uniform_over_the_eligible_rows(lib):
    capi = helpers.capi
    n_envs, capacity, batch = 5, 1000, 200_000
    position = np.array([10, 999, 0, 500, 1], np.uint32)
    full = np.array([0, 0, 1, 1, 0], np.uint8)
    rb = capi.ReplayBuffer()
    rb.position, rb.full, rb.n_envs, rb.capacity = position.ctypes.data, full.ctypes.data, n_envs, capacity
    env, off = np.zeros(batch, np.uint32), np.zeros(batch, np.uint32)
    assert lib.rlt_oracle_gather_draw(C.byref(rb), batch, 3, 77, env.ctypes.data, off.ctypes.data) == 0
    w = bits(lib, 4 * batch, 3, 77).reshape(-1, 4)
    eligible = np.where(full != 0, capacity, position).astype(np.uint64)
    assert np.array_equal(env, (w[:, 0].astype(np.uint64) * n_envs) >> 32)
    assert np.array_equal(off, (w[:, 1].astype(np.uint64) * eligible[env]) >> 32)
    assert np.all(off < eligible[env])
    counts = np.bincount(env, minlength=n_envs)
    assert stats.chisquare(counts).pvalue > 1e-3
    for e in (1, 2, 3):
        c = np.bincount(off[env == e] // 100, minlength=int(eligible[e] + 99) // 100)
        assert stats.chisquare(c[: int(eligible[e]) // 100]).pvalue > 1e-3


def test_initial_states_cover_the_pendulums_reset_ranges(lib):
    n = 100_000
    s = np.zeros((n, 2), np.float32)
    assert lib.rlt_oracle_pendulum_initial_states(s.ctypes.data, n, 1, 4) == 0
    assert np.all(np.abs(s[:, 0]) < np.pi) and np.all(np.abs(s[:, 1]) < 1)
    assert stats.kstest((s[:, 0].astype(np.float64) + np.pi) / (2 * np.pi), "uniform").pvalue > 1e-3
    assert stats.kstest((s[:, 1].astype(np.float64) + 1) / 2, "uniform").pvalue > 1e-3
    assert abs(np.corrcoef(s[:, 0], s[:, 1])[0, 1]) < 4 / np.sqrt(n)


def test_reduce_sum_and_adam_reset(lib):
    rng = np.random.default_rng(0)
    x = rng.standard_normal(100_003).astype(np.float32)
    out = np.zeros(1, np.float32)
    lib.rlt_oracle_reduce_sum_f32(x.ctypes.data, len(x), 0, out.ctypes.data)
    assert out[0] == np.float32(x.astype(np.float64).sum())
    lib.rlt_oracle_reduce_sum_f32(x.ctypes.data, len(x), 1, out.ctypes.data)
    assert out[0] == np.float32((x.astype(np.float64) ** 2).sum())
    # reset_optimizer_state: moments to zero, age to 1 (nn/optimizers/adam/instance/operations_generic.h:65-69, operations_generic.h:43-47),
    # and the first step after it is the closed form  p - alpha * sign-like g / (|g| + eps)
    capi = helpers.capi
    n = 257
    p, g = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    m, v = rng.standard_normal(n).astype(np.float32), np.abs(rng.standard_normal(n)).astype(np.float32)
    t = capi.AdamTensor()
    t.parameters, t.gradient, t.first_moment, t.second_moment, t.count = p.ctypes.data, g.ctypes.data, m.ctypes.data, v.ctypes.data, n
    age = np.array([17], np.uint32)
    assert lib.rlt_oracle_adam_reset(C.byref(t), 1, age.ctypes.data) == 0
    assert age[0] == 1 and not m.any() and not v.any()
    params = capi.AdamParameters()
    params.alpha, params.beta_1, params.beta_2, params.epsilon, params.epsilon_sqrt = 1e-3, 0.9, 0.999, 1e-7, 0.0
    p0 = p.copy()
    helpers.HostBackend().call("adam_step", C.byref(t), 1, C.byref(params), age.ctypes.data, 1.0, None)
    assert age[0] == 2
    gd = g.astype(np.float64)
    expected = p0 - 1e-3 * gd / (np.abs(gd) + 1e-7)
    assert np.allclose(p, expected, rtol=0, atol=2e-7)


def test_gather_sequence_draw_follows_the_documented_words(lib):
    """Every array against the raw words of the sample's groups (the documented order: environment, padded offsets, padded + 1 nominal
    decisions, padded + 1 lengths), ranges, and uniformity of lengths and nominal share."""
    capi = helpers.capi
    n_envs, capacity, batch, S, limit = 4, 2000, 50_000, 7, 200
    padded, words, groups = S + 1, 3 * (S + 1) + 3, (3 * (S + 1) + 3 + 3) // 4
    position = np.array([10, 1999, 0, 700], np.uint32)
    full = np.array([0, 0, 1, 1], np.uint8)
    rb = capi.ReplayBuffer()
    rb.position, rb.full, rb.n_envs, rb.capacity = position.ctypes.data, full.ctypes.data, n_envs, capacity
    for from_initial in (0, 1):
        P = capi.SequenceSampling()
        P.always_sample_from_initial_state, P.random_seq_length, P.enable_nominal_sequence_length_probability, P.nominal_sequence_length_probability = from_initial, 1, 1, 0.3
        env, off = np.zeros(batch, np.uint32), np.zeros((batch, padded), np.uint32)
        nominal, lengths = np.zeros((batch, padded + 1), np.uint8), np.zeros((batch, padded + 1), np.uint32)
        assert lib.rlt_oracle_gather_sequence_draw(C.byref(rb), C.byref(P), limit, batch, S, 9, 123, env.ctypes.data, off.ctypes.data, nominal.ctypes.data, lengths.ctypes.data) == 0
        w = bits(lib, 4 * groups * batch, 9, 123).reshape(batch, 4 * groups).astype(np.uint64)
        eligible = np.where(full != 0, capacity - limit if from_initial else capacity, position).astype(np.uint64)
        assert np.array_equal(env, (w[:, 0] * n_envs) >> 32)
        assert np.array_equal(off, (w[:, 1:1 + padded] * eligible[env][:, None]) >> 32) and np.all(off < eligible[env][:, None])
        unit = ((w[:, 1 + padded:2 * padded + 2] >> 8).astype(np.float64) + 0.5) * 2.0 ** -24
        assert np.array_equal(nominal, (unit.astype(np.float32) < np.float32(0.3)).astype(np.uint8))
        assert np.array_equal(lengths, 1 + ((w[:, 2 * padded + 2:3 * padded + 3] * (S - 1)) >> 32))
        assert lengths.min() == 1 and lengths.max() == S - 1
        assert stats.chisquare(np.bincount(lengths.reshape(-1))[1:]).pvalue > 1e-3
        assert abs(nominal.mean() - 0.3) < 4 * np.sqrt(0.21 / nominal.size)
    one = np.zeros((4, 3), np.uint32)
    assert lib.rlt_oracle_gather_sequence_draw(C.byref(rb), C.byref(P), limit, 4, 1, 9, 1, np.zeros(4, np.uint32).ctypes.data, np.zeros((4, 2), np.uint32).ctypes.data,
                                               np.zeros((4, 3), np.uint8).ctypes.data, one.ctypes.data) == 0
    assert np.all(one == 1)       # sequence length 1 leaves no choice
