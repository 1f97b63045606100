"""The CPU checker against the REAL reference compiled from /root/reference (oracle/_ref, built by oracle/Makefile): the whole
seeded SAC-on-Pendulum loop, bit for bit. Skipped where the reference build is absent (the GPU box still carries the built
library; a machine without it relies on tests/test_oracle_golden.py)."""
import ctypes as C
import os

import numpy as np
import pytest

import helpers

pytestmark = pytest.mark.skipif(not os.path.exists(helpers.REF_GENERIC), reason="oracle/_ref not built (needs /root/reference)")


def load_ref(path):
    ref = C.CDLL(path)
    ref.rlt_ref_sac_create.restype = C.c_void_p
    ref.rlt_ref_sac_parameter_count.restype = C.c_size_t
    ref.rlt_ref_sac_parameter_count.argtypes = [C.c_void_p]
    P = C.c_void_p
    for name, args in dict(step=[P], destroy=[P], get_parameters=[P, P], get_batch=[P, P, P, P], get_noise=[P, P, P], get_replay=[P, P, P, P, P],
                           get_critic_buffers=[P, C.c_int, P, P, P, P, P], get_actor_buffers=[P, P, P, P, P]).items():
        getattr(ref, "rlt_ref_sac_" + name).argtypes = args
    ref.rlt_ref_sac_evaluate.argtypes = [P, C.c_uint32, P, P, P, P]
    return ref


def reference_evaluation(ref, h, seed):
    """rl::utils::evaluation::evaluate of the loop's current actor by the reference: 10 episodes x 200 steps in Evaluation mode."""
    ini, ret, length, summary = np.zeros((10, 2), np.float32), np.zeros(10, np.float32), np.zeros(10, np.uint32), np.zeros(6, np.float32)
    ref.rlt_ref_sac_evaluate(h, seed, ini.ctypes.data, ret.ctypes.data, length.ctypes.data, summary.ctypes.data)
    return ini, ret, length, summary


def np_from(ptr, shape, dtype=np.float32):
    n = int(np.prod(shape))
    return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(np.ctypeslib.as_ctypes_type(dtype))), (n,)).reshape(shape).copy()


@pytest.mark.parametrize("batch,steps", [(100, 400), (256, 420)])
def test_loop_bit_exact_with_reference_generic_build(oracle, batch, steps):
    """Parameters after every step, the replay ring, the gathered batch, the noise and the training buffers
    (pattern: tests/src/rl/cuda/rl.cu:230-376 TRAIN_CRITIC_STEP_BY_STEP) are identical bit for bit."""
    ref, lib = load_ref(helpers.REF_GENERIC), oracle.lib
    cfg = helpers.LoopConfig(0, batch, 64, 10000, max(batch, 100), 200, 1e-7)
    loop = C.c_void_p(lib.rlt_oracle_sac_loop_create(C.byref(cfg)))
    h = C.c_void_p(ref.rlt_ref_sac_create(0, batch))
    n = lib.rlt_oracle_sac_loop_parameter_count(loop)
    assert n == ref.rlt_ref_sac_parameter_count(h)
    po, pr = np.zeros(n, np.float32), np.zeros(n, np.float32)
    A = lib.rlt_oracle_sac_loop_agent(loop).contents
    rb = lib.rlt_oracle_sac_loop_replay(loop).contents
    for step in range(steps):
        assert lib.rlt_oracle_sac_loop_step(loop) == 0
        ref.rlt_ref_sac_step(h)
        lib.rlt_oracle_sac_loop_get_parameters(loop, po.ctypes.data); ref.rlt_ref_sac_get_parameters(h, pr.ctypes.data)
        assert np.array_equal(po, pr), f"parameters differ after step {step}"
        if step > max(batch, 100) and step % 40 == 0:
            oab = np.zeros((2, batch, 4), np.float32); rew = np.zeros(batch, np.float32); term = np.zeros(batch, np.uint8)
            ref.rlt_ref_sac_get_batch(h, oab.ctypes.data, rew.ctypes.data, term.ctypes.data)
            assert np.array_equal(oab, np_from(A.observations_actions_base, (2, batch, 4)))
            assert np.array_equal(rew, np_from(A.rewards, (batch,))) and np.array_equal(term, np_from(A.terminated, (batch,), np.uint8))
            y, q1, q2, nin, dout = (np.zeros(s, np.float32) for s in (batch, batch, batch, (batch, 4), batch))
            ref.rlt_ref_sac_get_critic_buffers(h, 1, y.ctypes.data, q1.ctypes.data, q2.ctypes.data, nin.ctypes.data, dout.ctypes.data)
            assert np.array_equal(y, np_from(A.target_action_value, (batch,)))
            assert np.array_equal(q1, np_from(A.next_q[0], (batch,))) and np.array_equal(q2, np_from(A.next_q[1], (batch,)))
            assert np.array_equal(nin, np_from(A.next_state_action_value_input, (batch, 4)))
            sav, d1, d2, daos = (np.zeros(s, np.float32) for s in ((batch, 4), (batch, 4), (batch, 4), batch))
            ref.rlt_ref_sac_get_actor_buffers(h, sav.ctypes.data, d1.ctypes.data, d2.ctypes.data, daos.ctypes.data)
            assert np.array_equal(sav, np_from(A.state_action_value_input, (batch, 4)))
            assert np.array_equal(d1, np_from(A.d_critic_input[0], (batch, 4))) and np.array_equal(d2, np_from(A.d_critic_input[1], (batch, 4)))
            assert np.array_equal(daos, np_from(A.d_actor_output_squashing, (batch,)))
    data = np.zeros((10000, 10), np.float32); pos = C.c_uint32(); full = C.c_uint8(); es = np.zeros(10000, np.uint32)
    ref.rlt_ref_sac_get_replay(h, data.ctypes.data, C.byref(pos), C.byref(full), es.ctypes.data)
    assert pos.value == np_from(rb.position, (1,), np.uint32)[0] and not full.value
    assert np.array_equal(data[:pos.value], np_from(rb.data, (10000, 10))[:pos.value])      # rows beyond the cursor are uninitialised in the reference
    assert np.array_equal(es[:pos.value], np_from(rb.episode_start, (10000,), np.uint32)[:pos.value])
    lib.rlt_oracle_sac_loop_destroy(loop); ref.rlt_ref_sac_destroy(h)


def test_evaluation_bit_exact_with_reference(oracle):
    """rl::utils::evaluation::evaluate (10 episodes x 200 steps, Evaluation mode, sampled initial states) of the actor after 0, 150 and 400 loop
    steps: the reference's returns, episode lengths and statistics against the checker's, which is handed the same actor and the initial states
    the reference drew. Bit for bit: dynamics, observation, network and tanh are the same float operations in the same order."""
    ref, lib = load_ref(helpers.REF_GENERIC), oracle.lib
    batch = 100
    cfg = helpers.LoopConfig(0, batch, 64, 10000, 100, 200, 1e-7)
    loop = C.c_void_p(lib.rlt_oracle_sac_loop_create(C.byref(cfg)))
    h = C.c_void_p(ref.rlt_ref_sac_create(0, batch))
    A = lib.rlt_oracle_sac_loop_agent(loop).contents
    env = helpers.capi.pendulum_parameters()
    seen = []
    for stop, seed in ((0, 5), (150, 6), (400, 7)):
        while ref.rlt_ref_sac_step_count(h) < stop:
            assert lib.rlt_oracle_sac_loop_step(loop) == 0
            ref.rlt_ref_sac_step(h)
        ini, want_ret, want_len, want_sum = reference_evaluation(ref, h, seed)
        assert np.all(np.abs(ini[:, 0]) <= np.pi) and np.all(np.abs(ini[:, 1]) <= 1.0) and len(np.unique(ini[:, 0])) == 10
        ret, length, summary = np.zeros(10, np.float32), np.zeros(10, np.uint32), np.zeros(6, np.float32)
        assert lib.rlt_oracle_pendulum_evaluate(C.byref(env), 2, A.actor, 3, ini.ctypes.data, 10, 200, ret.ctypes.data, length.ctypes.data, summary.ctypes.data) == 0
        assert np.array_equal(ret, want_ret) and np.array_equal(length, want_len) and np.array_equal(summary, want_sum), (stop, ret, want_ret)
        assert np.all(length == 200) and summary[4] == 0 and np.all(ret < 0)
        seen.append(summary[0])
    assert len(set(seen)) == 3          # the actor changed between the evaluations
    lib.rlt_oracle_sac_loop_destroy(loop); ref.rlt_ref_sac_destroy(h)


@pytest.mark.skipif(not os.path.exists(helpers.REF_ENVS_GENERIC), reason="environment flavour of oracle/_ref not built")
@pytest.mark.parametrize("kind", [0, 1, 2])
def test_acrobot_bit_exact_with_reference(oracle, kind):
    """Acrobot (0), AcrobotSwingup (1) and AcrobotSwingup with EasyParameters (2): observe, step (Runge-Kutta over dsdt, angle wrap, velocity clamp),
    reward and terminated of the reference on 20,000 random states, and a 500-step closed chain where each side feeds on its own next state."""
    ref = C.CDLL(helpers.REF_ENVS_GENERIC)
    P = C.c_void_p
    ref.rlt_ref_acrobot_steps.argtypes = [C.c_int, P, P, P, P, P, P, P, C.c_int]

    def reference(states, actions):
        n = states.shape[0]
        ns, o, no, r, t = np.zeros((n, 4), np.float32), np.zeros((n, 6), np.float32), np.zeros((n, 6), np.float32), np.zeros(n, np.float32), np.zeros(n, np.uint8)
        assert ref.rlt_ref_acrobot_steps(kind, states.ctypes.data, actions.ctypes.data, ns.ctypes.data, o.ctypes.data, no.ctypes.data, r.ctypes.data, t.ctypes.data, n) == 0
        return ns, o, no, r, t
    rng = np.random.default_rng(kind)
    n = 20000
    states = np.stack([rng.uniform(-np.pi, np.pi, n), rng.uniform(-np.pi, np.pi, n), rng.uniform(-13, 13, n), rng.uniform(-29, 29, n)], 1).astype(np.float32)
    states[:10] = 0
    actions = rng.uniform(-1.3, 1.3, n).astype(np.float32)
    want, got = reference(states, actions), helpers.acrobot_on_backend(oracle, kind, states, actions)
    for w, g, name in zip(want, got, ("next_states", "observations", "next_observations", "rewards", "terminated")):
        assert np.array_equal(w, g), name
    if kind == 0:
        assert 0 < want[4].sum() < n and np.all(want[3] == -1)
    else:
        assert want[4].sum() == 0 and np.all(want[3] <= 0) and len(np.unique(want[3])) > n // 2
    assert (np.abs(want[0][:, 2]) == np.float32(4 * np.float32(np.pi))).sum() > 0        # the velocity clamp is reached
    sr = so = np.array([[0.05, -0.03, 0.02, 0.01]] * 4, np.float32) * np.arange(1, 5, dtype=np.float32)[:, None]
    for k in range(500):
        a = rng.uniform(-1, 1, 4).astype(np.float32)
        sr, so = reference(sr, a)[0], helpers.acrobot_on_backend(oracle, kind, so, a)[0]
        assert np.array_equal(sr, so), k


@pytest.mark.skipif(not os.path.exists(helpers.REF_ENVS_GENERIC), reason="environment flavour of oracle/_ref not built")
def test_car_bit_exact_with_reference(oracle):
    """The Car without a track: observe, step (tire forces on and off around the speed threshold, steering and throttle clamps), reward and terminated of
    the reference on 50,000 random states, and a 500-step closed chain."""
    ref = C.CDLL(helpers.REF_ENVS_GENERIC)
    P = C.c_void_p
    ref.rlt_ref_car_steps.argtypes = [P, P, P, P, P, P, P, C.c_int]

    def reference(states, actions):
        n = states.shape[0]
        ns, o, no, r, t = np.zeros((n, 6), np.float32), np.zeros((n, 6), np.float32), np.zeros((n, 6), np.float32), np.zeros(n, np.float32), np.zeros(n, np.uint8)
        assert ref.rlt_ref_car_steps(states.ctypes.data, actions.ctypes.data, ns.ctypes.data, o.ctypes.data, no.ctypes.data, r.ctypes.data, t.ctypes.data, n) == 0
        return ns, o, no, r, t
    rng = np.random.default_rng(2)
    n = 50000
    states = np.stack([rng.uniform(-1.2, 1.2, n), rng.uniform(-1.2, 1.2, n), rng.uniform(-4, 4, n), rng.uniform(-0.5, 3, n), rng.uniform(-1, 1, n), rng.uniform(-8, 8, n)], 1).astype(np.float32)
    states[:100, 3:] = 0
    states[100:1000, 3] = rng.uniform(0.005, 0.015, 900); states[100:1000, 4] = rng.uniform(0.005, 0.015, 900)
    actions = rng.uniform(-1.3, 1.3, (n, 2)).astype(np.float32)
    want, got = reference(states, actions), helpers.car_on_backend(oracle, states, actions)
    for w, g, name in zip(want, got, ("next_states", "observations", "next_observations", "rewards", "terminated")):
        assert np.array_equal(w, g), name
    assert 0 < want[4].sum() < n and np.all(want[3] > 0) and np.all(want[3] <= 1)
    sr = so = np.zeros((4, 6), np.float32)
    for k in range(500):
        a = np.stack([rng.uniform(0, 1, 4), rng.uniform(-0.3, 0.3, 4)], 1).astype(np.float32)
        sr, so = reference(sr, a)[0], helpers.car_on_backend(oracle, so, a)[0]
        assert np.array_equal(sr, so), k
    assert np.abs(sr[:, 3]).max() > 0.5          # the cars got going


class RefGatherSeq:
    """The reference's SAC loop with three environments, episodes of 30 steps and rings of 260 rows (oracle/ref_harness/ref_gather_seq.cpp)."""

    def __init__(self, seed):
        self.lib = C.CDLL(helpers.REF_GATHER_SEQ_GENERIC)
        P = C.c_void_p
        self.lib.rlt_ref_gather_seq_create.restype = P
        self.lib.rlt_ref_gather_seq_step.argtypes = [P]; self.lib.rlt_ref_gather_seq_destroy.argtypes = [P]
        self.lib.rlt_ref_gather_seq_get_replay.argtypes = [P, C.c_int, P, P, P, P]
        self.lib.rlt_ref_gather_seq_gather.argtypes = [P, C.c_int, C.c_uint32, C.c_char_p, C.c_int] + [P] * 7
        dims = (C.c_int * 6)()
        self.lib.rlt_ref_gather_seq_dims(dims)
        self.n_envs, self.capacity, self.max_episode_length, self.batch, self.sequence_length, self.row = list(dims)
        self.h = P(self.lib.rlt_ref_gather_seq_create(seed))

    def rings(self):
        out = []
        for e in range(self.n_envs):
            data, pos, full, es = np.zeros((self.capacity, self.row), np.float32), C.c_uint32(), C.c_uint8(), np.zeros(self.capacity, np.uint32)
            self.lib.rlt_ref_gather_seq_get_replay(self.h, e, data.ctypes.data, C.byref(pos), C.byref(full), es.ctypes.data)
            out.append((data, pos.value, full.value, es))
        return out

    def gather(self, variant, seed):
        S = 1 if variant == 2 else self.sequence_length
        PS, N, D = S + 1, self.batch, self.row // 2 - 1
        rng = C.create_string_buffer(16384)
        out = dict(observations_actions_base=np.zeros((PS, N, D), np.float32), rewards=np.zeros((S, N), np.float32), terminated=np.zeros((S, N), np.uint8),
                   reset=np.zeros((S, N), np.uint8), next_reset_base=np.zeros((PS, N), np.uint8), final_step_mask=np.zeros((S, N), np.uint8),
                   next_final_step_mask_base=np.zeros((PS, N), np.uint8))
        assert self.lib.rlt_ref_gather_seq_gather(self.h, variant, seed, rng, 16384, *[out[k].ctypes.data for k in helpers.SEQUENCE_BATCH_FIELDS]) == 0
        return S, rng, out


SEQUENCE_SAMPLING = {0: (1, 1, 1, 0.5, 1), 1: (0, 0, 1, 0.5, 1), 2: (0, 0, 1, 0.5, 0)}     # the harness's variants as SequentialBatchParameters


@pytest.mark.skipif(not os.path.exists(helpers.REF_GATHER_SEQ_GENERIC), reason="sequence-gather flavour of oracle/_ref not built")
def test_sequence_gather_bit_exact_with_reference(oracle):
    """gather_batch for SequentialBatch with SEQUENCE_LENGTH 8 (the reference's defaults: sequences start at their episode's first step and have random
    lengths; and both switched off) and 1, on the replay rings of the reference's own runner with three environments and 30-step episodes, before the
    rings are full (90 and 150 rows) and after they wrapped (600 loop steps into 260 rows, 60 of them eligible): every tensor of the batch equals the reference's, entry for
    entry including the entries gather_batch leaves untouched, with the draws made in the reference's order on its std::mt19937; and the draws the
    restatement hands back reproduce the same batch when fed in as arrays."""
    ref = RefGatherSeq(0)
    steps = 0
    seen_restart = seen_short = False
    for stop in (90, 150, 600):
        while steps < stop:
            ref.lib.rlt_ref_gather_seq_step(ref.h); steps += 1
        rings = ref.rings()
        assert all(r[1] == stop % ref.capacity for r in rings) and all(bool(r[2]) == (stop >= ref.capacity) for r in rings)
        for variant in (0, 1, 2):
            for seed in (1, 2, 3):
                S, rng, want = ref.gather(variant, seed)
                sampling = helpers.capi.SequenceSampling(*SEQUENCE_SAMPLING[variant])
                rb = helpers.replay_on_backend(oracle, rings)
                out = helpers.SequenceBatchOnBackend(oracle, ref.batch, S, ref.row // 2 - 1)
                env, off, nom, length = np.zeros(ref.batch, np.uint32), np.zeros((ref.batch, S + 1), np.uint32), np.zeros((ref.batch, S + 2), np.uint8), np.zeros((ref.batch, S + 2), np.uint32)
                assert oracle.lib.rlt_oracle_gather_sequence_batch_with_rng(C.byref(rb.c), C.byref(sampling), ref.max_episode_length, C.byref(out.c), rng, 16384,
                                                                            env.ctypes.data, off.ctypes.data, nom.ctypes.data, length.ctypes.data) == 0
                got = out.numpy()
                for k in helpers.SEQUENCE_BATCH_FIELDS:
                    assert np.array_equal(got[k], want[k]), (stop, variant, seed, k)
                fed = helpers.gather_sequence_on_backend(oracle, rings, sampling, (env, off, nom, length), ref.max_episode_length, ref.batch, S)
                for k in helpers.SEQUENCE_BATCH_FIELDS:
                    assert np.array_equal(fed[k], want[k]), ("fed", stop, variant, seed, k)
                assert len(np.unique(env)) == ref.n_envs
                if variant == 0:
                    seen_restart |= bool((want["reset"][1:].sum(0) > 0).any())            # a sequence ended early and another started inside the sample
                    seen_short |= bool((want["final_step_mask"][:-1].sum(0) > 0).any())
                if variant == 2:     # single steps: what rlt_*_gather_batch computes
                    oab, rew, term = oracle.zeros((2, ref.batch, 4)), oracle.zeros((ref.batch,)), oracle.zeros((ref.batch,), np.uint8)
                    e_, o_ = oracle.array(env), oracle.array(np.ascontiguousarray(off[:, 0]))
                    oracle.call("gather_batch", C.byref(rb.c), e_.ptr, o_.ptr, 0, ref.max_episode_length, ref.batch, oab.ptr, rew.ptr, term.ptr, None, None, None, None)
                    assert np.array_equal(oab.numpy(), want["observations_actions_base"]) and np.array_equal(rew.numpy(), want["rewards"][0])
    assert seen_restart and seen_short
    ref.lib.rlt_ref_gather_seq_destroy(ref.h)


@pytest.mark.skipif(not os.path.exists(helpers.REF_ENVS_GENERIC), reason="environment flavour of oracle/_ref not built")
def test_car_on_track_bit_exact_with_reference(oracle):
    """CarTrack on the reference's default track (100 x 100 cells of 20 mm, read from the compiled reference at run time): the nine observations with the
    three ray distances before and after the step, the step itself, reward = forward speed and terminated = off the track, on 50,000 random states
    inside the bitmap, on and off the track."""
    ref = C.CDLL(helpers.REF_ENVS_GENERIC)
    P = C.c_void_p
    ref.rlt_ref_car_track_steps.argtypes = [P, P, P, P, P, P, P, C.c_int]; ref.rlt_ref_car_track_bitmap.argtypes = [P]
    track = np.zeros((100, 100), np.uint8)
    ref.rlt_ref_car_track_bitmap(track.ctypes.data)
    assert 1000 < track.sum() < 5000
    rng = np.random.default_rng(3)
    n = 50000
    states = np.stack([rng.uniform(-0.95, 0.95, n), rng.uniform(-0.95, 0.95, n), rng.uniform(-4, 4, n), rng.uniform(-0.5, 3, n), rng.uniform(-1, 1, n), rng.uniform(-8, 8, n)], 1).astype(np.float32)
    actions = rng.uniform(-1.3, 1.3, (n, 2)).astype(np.float32)
    ns, o, no, r, t = np.zeros((n, 6), np.float32), np.zeros((n, 9), np.float32), np.zeros((n, 9), np.float32), np.zeros(n, np.float32), np.zeros(n, np.uint8)
    assert ref.rlt_ref_car_track_steps(states.ctypes.data, actions.ctypes.data, ns.ctypes.data, o.ctypes.data, no.ctypes.data, r.ctypes.data, t.ctypes.data, n) == 0
    got = helpers.car_track_on_backend(oracle, track, 20 / 1000.0, states, actions)
    for w, g, name in zip((ns, o, no, r, t), got, ("next_states", "observations", "next_observations", "rewards", "terminated")):
        assert np.array_equal(w, g), name
    on_track = o[:, 7] > 0
    assert 0.1 < on_track.mean() < 0.5 and 0 < t.sum() < n and np.array_equal(r, states[:, 3])
    assert len(np.unique(o[on_track, 6:])) > 20 and o[:, 6:].max() <= 1.0          # many different ray lengths, as fractions of the full ray


def test_small_ring_wraps_bit_exact_with_reference(oracle):
    """Replay capacity 250 (< 900 steps): the ring wraps three times, so `add` past the end, the prologue's wrap of the
    previous row, `full`, and gather's (position + MAX_EPISODE_LENGTH + offset) % CAPACITY index all run, and every
    parameter still matches the reference bit for bit after each step."""
    ref, lib = load_ref(helpers.REF_GENERIC), oracle.lib
    batch, cap = 32, 250
    cfg = helpers.LoopConfig(0, batch, 64, cap, 100, 200, 1e-7)
    loop = C.c_void_p(lib.rlt_oracle_sac_loop_create(C.byref(cfg)))
    h = C.c_void_p(ref.rlt_ref_sac_create(0, batch))
    n = lib.rlt_oracle_sac_loop_parameter_count(loop)
    po, pr = np.zeros(n, np.float32), np.zeros(n, np.float32)
    rb = lib.rlt_oracle_sac_loop_replay(loop).contents
    for step in range(900):
        assert lib.rlt_oracle_sac_loop_step(loop) == 0
        ref.rlt_ref_sac_step(h)
        lib.rlt_oracle_sac_loop_get_parameters(loop, po.ctypes.data); ref.rlt_ref_sac_get_parameters(h, pr.ctypes.data)
        assert np.array_equal(po, pr), f"parameters differ after step {step}"
    data = np.zeros((cap, 10), np.float32); pos = C.c_uint32(); full = C.c_uint8(); es = np.zeros(cap, np.uint32)
    ref.rlt_ref_sac_get_replay(h, data.ctypes.data, C.byref(pos), C.byref(full), es.ctypes.data)
    assert full.value == 1 == np_from(rb.full, (1,), np.uint8)[0] and pos.value == 900 % cap == np_from(rb.position, (1,), np.uint32)[0]
    assert np.array_equal(data, np_from(rb.data, (cap, 10)))
    assert np.array_equal(es, np_from(rb.episode_start, (cap,), np.uint32))
    lib.rlt_oracle_sac_loop_destroy(loop); ref.rlt_ref_sac_destroy(h)


@pytest.mark.skipif(not os.path.exists(helpers.REF_BLAS), reason="BLAS flavour of oracle/_ref not built")
def test_blas_flavour_of_reference_agrees_for_one_update(oracle):
    """The reference's CBLAS backend (its own -ffast-math build) after the first training step: same algorithm, different
    summation order, so 1e-5 relative rather than bit-exact."""
    ref, lib = load_ref(helpers.REF_BLAS), oracle.lib
    batch = 100
    cfg = helpers.LoopConfig(0, batch, 64, 10000, 100, 200, 1e-7)
    loop = C.c_void_p(lib.rlt_oracle_sac_loop_create(C.byref(cfg)))
    h = C.c_void_p(ref.rlt_ref_sac_create(0, batch))
    n = lib.rlt_oracle_sac_loop_parameter_count(loop)
    po, pr = np.zeros(n, np.float32), np.zeros(n, np.float32)
    for step in range(103):
        lib.rlt_oracle_sac_loop_step(loop); ref.rlt_ref_sac_step(h)
    lib.rlt_oracle_sac_loop_get_parameters(loop, po.ctypes.data); ref.rlt_ref_sac_get_parameters(h, pr.ctypes.data)
    assert helpers.rel_err(po, pr) <= 1e-5


@pytest.mark.skipif(not os.path.exists(helpers.REF_PPO_GENERIC), reason="oracle/_ref PPO harness not built (needs /root/reference)")
def test_ppo_gae_and_update_bit_exact_with_reference(oracle):
    """Three loop steps of the reference's PPO-on-Pendulum loop (8 envs x 40 steps, episodes truncated after 25 steps, 3 epochs of
    5 shuffled minibatches): the restated GAE reproduces the dataset's advantages and target values, and the restated update
    (surrogate gradient, log_std gradient, critic MSE, Adam) driven by the restated shuffle reproduces every parameter, bit for bit."""
    capi = helpers.capi
    ref = helpers.RefPpo(0)
    hy = ref.hyper
    adam = capi.adam_parameters(hy["alpha"], hy["beta_1"], hy["beta_2"], hy["epsilon"], hy["epsilon_sqrt"])
    pp = capi.ppo_parameters(hy["epsilon_clip"], hy["action_entropy_coefficient"], hy["advantage_epsilon"], int(hy["normalize_advantage"]), int(hy["learn_action_std"]))
    agent = helpers.PpoOnBackend(oracle, ref.obs_dim, ref.action_dim, ref.actor_hidden, ref.critic_hidden, ref.batch, ref.parameters(), "tanh", "relu", adam)
    n = ref.n_envs * ref.steps
    for loop_step in range(3):
        ref.lib.rlt_ref_ppo_collect_and_gae(ref.h)
        d = ref.dataset()
        c = ref.col
        assert d[:n, c["truncated"]].sum() >= ref.n_envs       # the case GAE treats specially does occur
        # GAE (rl/algorithms/ppo/operations_generic.h:60-95)
        dd = oracle.array(d)
        adv, tgt = oracle.zeros((ref.rows, ref.data_dim)), oracle.zeros((ref.rows, ref.data_dim))
        oracle.call("ppo_gae", dd.offset(c["rewards"]), dd.offset(c["terminated"]), dd.offset(c["truncated"]), dd.offset(c["all_values"]), adv.ptr, tgt.ptr,
                    ref.data_dim, ref.n_envs, ref.steps, hy["gamma"], hy["lambda"], 0)
        assert np.array_equal(adv.numpy()[:n, 0], d[:n, c["advantages"]]) and np.array_equal(tgt.numpy()[:n, 0], d[:n, c["target_values"]])
        # the update
        assert np.array_equal(agent.parameters(), ref.parameters())
        state = ref.rng_state()
        perms = np.zeros((ref.epochs, n), np.uint32)
        assert oracle.lib.rlt_oracle_ppo_shuffle(state, 16384, n, ref.epochs, perms.ctypes.data) == 0
        ref.lib.rlt_ref_ppo_train(ref.h)
        assert ref.rng_state().value == state.value             # the restated shuffle drew exactly what the reference drew
        helpers.ppo_train_like_reference(oracle, agent, pp, dd, ref.data_dim, c, n, perms, ref.batch)
        got, want = agent.parameters(), ref.parameters()
        assert np.array_equal(got, want), (loop_step, np.abs(got - want).max())
        assert ref.ages() == [int(agent.actor.age.numpy()[0]), int(agent.critic.age.numpy()[0])]
    ref.close()


@pytest.mark.skipif(not (os.path.exists(helpers.REF_GRU_GENERIC) and os.path.exists(helpers.REF_GRU_FAST_GENERIC)), reason="oracle/_ref GRU harness not built (needs /root/reference)")
@pytest.mark.parametrize("fast_tanh", [False, True])
@pytest.mark.parametrize("with_reset", [False, True])
def test_gru_forward_and_backward_through_time_bit_exact_with_reference(oracle, with_reset, fast_tanh):
    """The reference's own GRU layer (forward with kept intermediates, backward_full through 7 steps, optional per-sample resets) on random
    weights and inputs: outputs, intermediates, d_input, the in-place accumulated d_output and all four gradients, bit for bit; with the
    exact gate functions and with the FAST_TANH switch (a second build of the harness), whose inputs are scaled so that the clamp of the
    rational approximation at |x| = 3 is reached."""
    ref = C.CDLL(helpers.REF_GRU_FAST_GENERIC if fast_tanh else helpers.REF_GRU_GENERIC)
    dims = (C.c_int * 4)(); ref.rlt_ref_gru_dims(dims)
    S, B, I, H = list(dims)
    rng = np.random.default_rng(12 + with_reset)
    params, x, dy, reset = helpers.gru_random_case(rng, S, B, I, H, with_reset)
    if fast_tanh:
        x = (x * 6).astype(np.float32)
    want = dict(output=np.zeros((S, B, H), np.float32), post=np.zeros((S, B, 3 * H), np.float32), npp=np.zeros((S, B, H), np.float32), dx=np.zeros((S, B, I), np.float32),
                dW_i=np.zeros((3 * H, I), np.float32), db_i=np.zeros(3 * H, np.float32), dW_h=np.zeros((3 * H, H), np.float32), db_h=np.zeros(3 * H, np.float32),
                dy=np.zeros((S, B, H), np.float32))
    p = lambda a: a.ctypes.data_as(C.c_void_p)
    ref.rlt_ref_gru_forward_backward.argtypes = [C.c_void_p] * 17
    assert ref.rlt_ref_gru_forward_backward(p(params["W_i"]), p(params["b_i"]), p(params["W_h"]), p(params["b_h"]), p(params["h0"]), p(x), p(reset) if with_reset else None,
                                            p(dy), p(want["output"]), p(want["post"]), p(want["npp"]), p(want["dx"]), p(want["dW_i"]), p(want["db_i"]), p(want["dW_h"]),
                                            p(want["db_h"]), p(want["dy"])) == 0
    g = helpers.GruOnBackend(oracle, S, B, I, H, params, fast_tanh=fast_tanh)
    g.forward(x, reset)
    g.backward(dy)
    got = g.results()
    if with_reset:
        assert reset[1:].sum() > 3
    if fast_tanh:
        assert (want["post"][..., :2 * H] == 1.0).any() or (want["post"][..., 2 * H:] == 1.0).any() or (np.abs(want["post"][..., 2 * H:]) == 1.0).any()   # the clamp was reached
    for k in want:
        assert np.array_equal(got[k], want[k]), (k, np.abs(got[k] - want[k]).max())


@pytest.mark.skipif(not os.path.exists(helpers.REF_TD3_GENERIC), reason="oracle/_ref TD3 harness not built (needs /root/reference)")
def test_td3_updates_bit_exact_with_reference(oracle):
    """The reference's own TD3-on-Pendulum loop. Two copies with one seed: one advanced by the reference's step(), one by the same
    operations called one by one (so that the sampling-layer draws can be written out) -- they must agree, which ties what follows to
    step() itself. From the first training step on, the restatement gets the reference's batch, smoothing noise and sampling draws
    and must reproduce every parameter (actor, target actor, critics, target critics) and Adam age, bit for bit, over 100 loop steps
    (50 delayed actor updates, some with samples outside [-1, 1], where the sampling layer's backward pass blocks the gradient). The smoothing noise itself is restated from the N(0,1) draws behind it."""
    a, b = helpers.RefTd3(7), helpers.RefTd3(7)
    assert (b.batch, b.actor_interval, b.critic_target_interval, b.actor_target_interval) == (100, 2, 2, 2)
    for _ in range(b.n_warmup):
        a.step(); b.step()
    agent = helpers.Td3OnBackend(oracle, b.batch, b.hidden, b.parameters(), hyper=b.hyper())
    actor_updates = clipped = blocked = 0
    for i in range(100):
        a.step()
        z, c0, c1, na, flags = b.manual_step()
        assert np.array_equal(a.parameters(), b.parameters())
        assert flags[0] == 1 and flags[2] == flags[1] == flags[3] == (1 if i % 2 == 0 else 0)
        oab, r, t, fm, nfm = b.batch_data()
        assert fm.all() and nfm[b.batch:].all()          # SEQUENCE_LENGTH = 1: every step is a final step
        noise = b.target_noise()
        zd, out = oracle.array(z), oracle.zeros((b.batch, 1))
        oracle.call("td3_target_action_noise", zd.ptr, float(b.hp[3]), float(b.hp[4]), out.ptr, b.batch)
        assert np.array_equal(out.numpy(), noise)
        clipped += int((np.abs(noise) == np.float32(0.5)).sum())
        agent.set_batch(oab, r, t, noise)
        agent.loop_step(flags, c0, c1, na)
        actor_updates += flags[2]
        blocked += int((np.abs(agent.pre_clip.numpy()) > 1).sum()) if flags[2] else 0
        got, want = agent.parameters(), b.parameters()
        assert np.array_equal(got, want), (i, np.abs(got - want).max())
        assert np.array_equal(agent.ages(), b.ages())
    assert actor_updates == 50 and clipped >= 3 and blocked >= 3          # the clip at 2.5 standard deviations was exercised
    a.close(); b.close()


@pytest.mark.skipif(not os.path.exists(helpers.REF_PPO_NORMALIZE_GENERIC), reason="oracle/_ref PPO harness (normalising flavour) not built (needs /root/reference)")
def test_on_policy_collect_and_observation_normalisation_bit_exact_with_reference(oracle):
    """The reference's PPO loop with running observation normalisation on. One copy is advanced by the reference's step(), a second by
    the pieces step() is made of (collect, normaliser update, runner re-initialisation, critic values + GAE, train); they must stay
    identical, which ties the pieces to step(). Around every collect() of the second copy the restatement is given the runner state, the
    actor with its standardize statistics and the text form of the RNG, and must reproduce: every dataset column collect writes
    (observations incl. the final ones, action means, sampled actions, their log-probabilities, rewards, flags, delayed resets), the
    runner state and the RNG state afterwards, bit for bit; the same again from the returned draws instead of the RNG; and after
    update(): both running normalisers and the statistics set into the two standardize layers."""
    a, b = helpers.RefPpo(3, normalize=True), helpers.RefPpo(3, normalize=True)
    assert b.flags() == dict(normalize=True, continuously=True, truncate_on_each_iteration=False)
    n, S, ld, c = b.n_envs, b.steps, b.data_dim, b.col
    rows = n * S
    norm = dict(mean=oracle.zeros((3,)), std=oracle.array(np.ones(3, np.float32)), age=oracle.array(np.zeros(1, np.uint32)),
                mean_p=oracle.zeros((3,)), std_p=oracle.array(np.ones(3, np.float32)), age_p=oracle.array(np.zeros(1, np.uint32)))
    layer = {k: oracle.zeros((3,)) for k in ("actor_mean", "actor_precision", "critic_mean", "critic_precision")}
    n_collects = resets_inside = 0

    def collect_and_check():
        nonlocal n_collects, resets_inside
        p = b.parameters()
        na = helpers.mlp_param_count([3, b.actor_hidden, b.actor_hidden, 1])
        actor = helpers.Mlp(oracle, [3, b.actor_hidden, b.actor_hidden, 1], p[:na], n, "tanh", "identity", trainable=False)
        log_std = p[na:na + 1]
        st = b.standardize()
        before, rng = b.runner(), b.rng_state()
        b.lib.rlt_ref_ppo_collect(b.h)
        want = b.dataset()
        o = helpers.OnPolicyOnBackend(oracle, n, S, ld, c, b.episode_step_limit, before)
        noise, ini = np.zeros((S, n, 1), np.float32), np.full((S, n, 2), np.nan, np.float32)
        ls, sm, sp = oracle.array(log_std), oracle.array(st["actor_mean"]), oracle.array(st["actor_precision"])
        assert oracle.lib.rlt_oracle_on_policy_collect_with_rng(C.byref(o.c), C.byref(o.d), actor.layers, actor.n, ls.ptr, sm.ptr, sp.ptr, noise.ctypes.data, ini.ctypes.data,
                                                                0, rng, 16384) == 0
        got = o.data.numpy()
        for name, nrows in (("observations", rows + n), ("actions_mean", rows), ("actions", rows), ("action_log_probs", rows), ("rewards", rows), ("terminated", rows),
                            ("truncated", rows), ("all_reset", rows + n)):
            w = 3 if name == "observations" else 1
            assert np.array_equal(got[:nrows, c[name]:c[name] + w], want[:nrows, c[name]:c[name] + w]), (n_collects, name)
        assert rng.value == b.rng_state().value              # the restatement drew exactly what the reference drew
        after = b.runner()
        for k, v in o.runner_state().items():
            assert np.array_equal(v, after[k]), k
        # the same collection from the returned draws
        o2 = helpers.OnPolicyOnBackend(oracle, n, S, ld, c, b.episode_step_limit, before)
        o2.collect(actor, log_std, noise, np.nan_to_num(ini), standardize=(st["actor_mean"], st["actor_precision"]))
        assert np.array_equal(o2.data.numpy()[:, :c["all_values"]], got[:, :c["all_values"]])
        n_collects += 1
        resets_inside += int(want[n:rows, c["all_reset"]].sum())
        return want

    def update_and_check(d):
        b.lib.rlt_ref_ppo_update_normalizers(b.h)
        dd = oracle.array(d)
        oracle.call("running_normalizer_update", dd.offset(c["observations"]), ld, rows, 3, norm["mean"].ptr, norm["std"].ptr, norm["age"].ptr)
        oracle.call("running_normalizer_update", dd.offset(c["all_observations_privileged"]), ld, rows + n, 3, norm["mean_p"].ptr, norm["std_p"].ptr, norm["age_p"].ptr)
        oracle.call("standardize_set_statistics", norm["mean"].ptr, norm["std"].ptr, layer["actor_mean"].ptr, layer["actor_precision"].ptr, 3)
        oracle.call("standardize_set_statistics", norm["mean_p"].ptr, norm["std_p"].ptr, layer["critic_mean"].ptr, layer["critic_precision"].ptr, 3)
        wn, ws = b.normalizers(), b.standardize()
        assert np.array_equal(norm["mean"].numpy(), wn["mean"]) and np.array_equal(norm["std"].numpy(), wn["std"])
        assert np.array_equal(norm["mean_p"].numpy(), wn["mean_privileged"]) and np.array_equal(norm["std_p"].numpy(), wn["std_privileged"])
        assert [int(norm["age"].numpy()[0]), int(norm["age_p"].numpy()[0])] == list(wn["ages"])
        for k in layer:
            assert np.array_equal(layer[k].numpy(), ws[k]), k

    for loop_step in range(3):
        a.lib.rlt_ref_ppo_step(a.h)
        if loop_step == 0:            # warm-up of the normalisers (rl/algorithms/ppo/loop/core/operations_generic.h:104-114)
            update_and_check(collect_and_check())
            b.lib.rlt_ref_ppo_reinit_runner(b.h)
        update_and_check(collect_and_check())
        b.lib.rlt_ref_ppo_values_and_gae(b.h)
        b.lib.rlt_ref_ppo_train(b.h)
        assert np.array_equal(a.parameters(), b.parameters()) and a.rng_state().value == b.rng_state().value
    assert n_collects == 4 and resets_inside >= n           # truncations in the middle of a dataset did occur
    a.close(); b.close()


@pytest.mark.skipif(not (os.path.exists(helpers.ref_sac_gru_path(3)) and os.path.exists(helpers.ref_sac_gru_path(5))), reason="oracle/_ref recurrent SAC harness not built (needs /root/reference)")
@pytest.mark.parametrize("n_layers", [3, 5])
def test_sac_on_sequence_batches_bit_exact_with_reference(oracle, n_layers):
    """The reference's own SAC loop with its recurrent approximators (dense -> GRU -> dense, and dense -> GRU -> GRU -> dense -> dense, FAST_TANH
    gates) on sequence batches of 6 steps with the first step included in the targets. From the first training step on the restatement gets
    the batch the reference trained on (all seven tensors as its gather_batch left them) and both noise tensors, and must reproduce every
    parameter of the five networks, log_alpha and the four Adam ages bit for bit over 400 loop steps -- through the wrap of the 260-row rings,
    with sequences that restart inside the batch, shortened sequences and final-step counts that are no powers of two. What that fixes
    beyond the layers themselves: the `next` views starting at padded step 0, the target taking the value one step later but the
    log-probability at the same index, the loss weight formed as (1 / n) * s, backward_input of the critics running without the resets
    during the actor update, the log_alpha gradient divided by the number of set reset flags, polyak on the GRU tensors."""
    ref = helpers.RefSacGru(n_layers, 4)
    assert (ref.seq, ref.batch, ref.include_first) == (6, 16, 1)
    assert [k for k, _, _, _ in ref.critic_specs] == ([0, 1, 0] if n_layers == 3 else [0, 1, 1, 0, 0])
    for _ in range(ref.n_warmup):
        ref.step()
    agent = helpers.SacSequenceOnBackend(oracle, ref.actor_specs, ref.critic_specs, ref.parameters(), ref.seq, ref.batch, ref.obs_dim, ref.act_dim, True, ref.hyper())
    restarts = odd_counts = 0
    for i in range(400):
        ref.step()
        data = ref.batch_data()
        agent.set_batch(data)
        agent.train(*ref.noise())
        got, want = agent.parameters(), ref.parameters()
        assert np.array_equal(got, want), (i, np.abs(got - want).max())
        restarts += int(data["reset"][1:].sum())
        n = int(data["final_step_mask"].sum())
        odd_counts += (n & (n - 1)) != 0
    assert agent.ages() == ref.ages() == [401] * 4
    assert restarts > 1000 and odd_counts > 300
    ref.close()


@pytest.mark.skipif(not (os.path.exists(helpers.ref_sac_gru_path(3)) and os.path.exists(helpers.ref_sac_gru_path(5))), reason="oracle/_ref recurrent SAC harness not built (needs /root/reference)")
def test_sac_sequence_fixture_is_what_the_reference_gives():
    g = helpers.sac_sequence_golden()
    for n_layers in (3, 5):
        p = f"l{n_layers}_"
        ref = helpers.RefSacGru(n_layers, 4)
        for _ in range(ref.n_warmup):
            ref.step()
        assert np.array_equal(ref.parameters(), g[p + "parameters_before"])
        for i in range(int(g[p + "dims"][5])):
            ref.step()
            data = ref.batch_data()
            assert all(np.array_equal(data[k], g[f"{p}s{i}_{k}"]) for k in helpers.SEQUENCE_BATCH_FIELDS)
            if i in g[p + "snapshots"]:
                assert np.array_equal(ref.parameters(), g[f"{p}s{i}_after"])
        ref.close()


@pytest.mark.skipif(not (os.path.exists(helpers.ref_sac_gru_path(3)) and os.path.exists(helpers.ref_sac_gru_path(5))), reason="oracle/_ref recurrent SAC harness not built (needs /root/reference)")
@pytest.mark.parametrize("n_layers", [3, 5])
def test_recurrent_runner_step_bit_exact_with_reference(oracle, n_layers):
    """The runner step of the reference's SAC loop with its recurrent actor. Two copies with one seed: one advanced by the reference's step(), one by the same
    operations called one by one with the runner step's draws taken from a copy of the engine first (the harness checks that the engine then stands where the
    copy stands) -- they must agree in every parameter, which ties what follows to step() itself. Each step the restatement starts from the reference's runner,
    policy state and rings, gets the actor's parameters and the draws, and must reproduce environment states, counters, truncation flags, hidden states, step
    counters and the replay rings bit for bit over 300 loop steps (30 new episodes, the hidden state restarting every 6 steps, ring wrap at 260 rows)."""
    a, b = helpers.RefSacGru(n_layers, 4), helpers.RefSacGru(n_layers, 4)
    for _ in range(a.n_warmup):
        a.step(); b.step()
    n, cap, limit, period, n_gru = b.runner_dims()
    assert (n, cap, limit, period, n_gru) == (3, 260, 30, 6, 1 if n_layers == 3 else 2)
    run = helpers.RecurrentRunnerOnBackend(oracle, b.actor_specs, b.actor_parameters(), n, cap, limit, period)
    new_episodes = restarts = 0
    for i in range(300):
        run.load(b.runner(), b.rings())
        run.policy.params.upload(b.actor_parameters())
        a.step()
        ini, noise, flags = b.manual_step()
        assert np.array_equal(a.parameters(), b.parameters()), i
        if i == 0:
            assert flags.all()              # policy switch after the warm-up: every episode is truncated
            run.trunc.upload(flags)
        run.step(noise, ini)
        got, want, rings = run.numpy(), b.runner(), b.rings()
        for k in ("states", "episode_step", "episode_return", "truncated"):
            assert np.array_equal(got[k], want[k]), (i, k)
        for k in range(n_gru):
            assert np.array_equal(got["hidden"][k], want["hidden"][k]) and np.array_equal(got["steps"][k], want["steps"][k]), (i, k)
        assert np.array_equal(got["data"], np.concatenate([r[0] for r in rings])), i
        assert np.array_equal(got["position"], [r[1] for r in rings]) and np.array_equal(got["full"], [r[2] for r in rings])
        assert np.array_equal(got["current_episode_start"], [r[3] for r in rings]) and np.array_equal(got["episode_start"], np.concatenate([r[4] for r in rings]))
        new_episodes += int(flags.sum()); restarts += int(sum((s == 0).sum() for s in want["steps"]))
    assert new_episodes == 30 and restarts >= 150 and got["full"].all()
    a.close(); b.close()


@pytest.mark.parametrize("n_layers", [3, 5])
def test_evaluation_with_recurrent_policy_bit_exact_with_reference(oracle, n_layers):
    """rl::utils::evaluation::evaluate on the reference's recurrent SAC actor (one or two GRU layers, hidden state restarting every 6 steps), untrained and after
    40 and 150 training steps: the restatement reproduces every episode's return, the lengths and the summary bit for bit from the same initial states. The
    committed fixture (tests/golden/evaluation_recurrent_pendulum.npz) holds exactly these runs."""
    ref = helpers.RefSacGru(n_layers, 9)
    g = helpers.evaluation_recurrent_golden()
    period = ref.runner_dims()[3]
    done = 0
    for k, stop in enumerate([0, ref.n_warmup + 40, ref.n_warmup + 150]):
        while done < stop:
            ref.step(); done += 1
        ini, ret, length, summary = ref.evaluate(100 + k)
        got = helpers.evaluate_recurrent(oracle, ref.actor_specs, ref.actor_parameters(), period, ini, 40)
        assert np.array_equal(got["returns"], ret) and np.array_equal(got["length"], length) and np.array_equal(got["summary"], summary), (k, got["returns"], ret)
        assert np.all(length == 40) and np.all(ret < 0)
        if g is not None:
            p = f"l{n_layers}_e{k}_"
            assert np.array_equal(g[p + "actor"], ref.actor_parameters()) and np.array_equal(g[p + "initial_states"], ini) and np.array_equal(g[p + "returns"], ret)
            assert np.array_equal(g[p + "summary"], summary)
    ref.close()


@pytest.mark.parametrize("n_layers", [4, 5])
def test_td3_sequence_bit_exact_with_reference(oracle, n_layers):
    """The reference's TD3 loop with its recurrent approximators (actor GRU 16, GRU 16[, dense 16], dense 1; critics alike) on sequence batches of 16 x 6 steps:
    from the parameters after the warm-up, the restatement is given the batch and the clamped target-action noise of every loop step and must reproduce every
    parameter of the six networks (incl. the polyak-averaged targets, every second step) and the Adam ages bit for bit over 300 loop steps, free-running (its own
    parameters are never re-synchronised); the critic's target values and d_output of the last update are compared too."""
    ref = helpers.RefTd3Gru(n_layers, 5)
    for _ in range(ref.n_warmup):
        ref.step()
    assert ref.intervals == [1, 2, 2, 2] and ref.include_first == 1
    assert [k for k, _, _, _ in ref.actor_specs] == ([1, 1, 0] if n_layers == 4 else [1, 1, 0, 0])
    agent = helpers.Td3SequenceOnBackend(oracle, ref.actor_specs, ref.critic_specs, ref.parameters(), ref.seq, ref.batch, ref.obs_dim, ref.act_dim, True, ref.hyper())
    trained_actor = 0
    for i in range(300):
        flags = ref.flags(ref.step_count())
        ref.step()
        agent.set_batch(ref.batch_data())
        agent.train(ref.noise(), flags)
        trained_actor += flags[2]
        assert np.array_equal(agent.parameters(), ref.parameters()), (i, flags, float(np.abs(agent.parameters() - ref.parameters()).max()))
        assert agent.ages() == ref.ages()
        y, d = ref.critic_buffers()
        assert np.array_equal(agent.buf["target"].numpy(), y), i
        if not flags[2]:                        # the agent here has one d_output for critic and actor updates
            assert np.array_equal(agent.buf["d_output"].numpy(), d), i
    assert trained_actor == 150
    ref.close()

