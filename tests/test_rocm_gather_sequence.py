"""gather_batch for sequence batches on the device (rlt_rocm_gather_sequence_batch) through the C ABI: bit-exact against the reference's own batches and
against the CPU checker (copies and index arithmetic only)."""
import ctypes as C

import numpy as np
import pytest

import helpers

pytestmark = pytest.mark.gpu


def test_sequence_gather_against_reference_vectors(rocm):
    for rings, sampling, draws, max_len, batch, seq, want in helpers.sequence_gather_golden():
        got = helpers.gather_sequence_on_backend(rocm, rings, sampling, draws, max_len, batch, seq)
        for k in helpers.SEQUENCE_BATCH_FIELDS:
            assert np.array_equal(got[k], want[k]), (seq, k)


# (always_sample_from_initial_state, random_seq_length, include_first_step_in_targets, steps per ring, environments, capacity, observation width, batch, sequence length)
CASES = [(1, 1, 1, 700, 4, 300, 5, 128, 12), (0, 0, 1, 700, 4, 300, 5, 128, 12), (1, 1, 1, 100, 2, 300, 3, 1, 8), (0, 1, 0, 180, 3, 300, 17, 4099, 3), (0, 0, 0, 5000, 16, 1000, 105, 65536, 1),
         (1, 1, 1, 2500, 64, 1000, 33, 8192, 64)]


@pytest.mark.parametrize("case", CASES)
def test_sequence_gather_matches_checker(oracle, rocm, case):
    print("case", case, flush=True)
    always, random_len, include_first, steps, n_envs, cap, obs, batch, seq = case
    rng = np.random.default_rng(batch + seq)
    max_len = 40
    rings = helpers.synthetic_rings(rng, n_envs, cap, obs, steps, max_len)
    sampling = helpers.capi.SequenceSampling(always, random_len, 1, 0.5, include_first)
    draws = helpers.random_sequence_draws(rng, rings, sampling, max_len, batch, seq)
    want = helpers.gather_sequence_on_backend(oracle, rings, sampling, draws, max_len, batch, seq)
    got = helpers.gather_sequence_on_backend(rocm, rings, sampling, draws, max_len, batch, seq)
    for k in helpers.SEQUENCE_BATCH_FIELDS:
        assert np.array_equal(got[k], want[k]), k
    if seq == 1 and not always and not random_len:      # single steps: the same batch as rlt_rocm_gather_batch from the same draws
        rb = helpers.replay_on_backend(rocm, rings)
        oab, rew, term = rocm.zeros((2, batch, obs + 1)), rocm.zeros((batch,)), rocm.zeros((batch,), np.uint8)
        e_, o_ = rocm.array(draws[0]), rocm.array(np.ascontiguousarray(draws[1][:, 0]))
        rocm.call("gather_batch", C.byref(rb.c), e_.ptr, o_.ptr, 0, max_len, batch, oab.ptr, rew.ptr, term.ptr, None, None, None, None)
        rocm.sync()
        assert np.array_equal(oab.numpy(), got["observations_actions_base"]) and np.array_equal(rew.numpy(), got["rewards"][0]) and np.array_equal(term.numpy(), got["terminated"][0])


def test_sequence_gather_reports_bad_device_side_indices():
    """An environment index beyond the runner's environments is met on the device: that sample is skipped and the next rlt_rocm_check_status says so.
    On a device handle of its own, because the status is sticky."""
    backend = helpers.RocmBackend()
    try:
        rng = np.random.default_rng(0)
        rings = helpers.synthetic_rings(rng, 2, 100, 3, 60, 20)
        sampling = helpers.capi.SequenceSampling(0, 0, 1, 0.5, 1)
        env, off, nom, length = helpers.random_sequence_draws(rng, rings, sampling, 20, 8, 4)
        good = helpers.gather_sequence_on_backend(backend, rings, sampling, (env, off, nom, length), 20, 8, 4)
        assert backend.device.lib.rlt_rocm_check_status(backend.device.handle) == 0
        env_bad = env.copy(); env_bad[3] = 7
        rb = helpers.replay_on_backend(backend, rings)
        out = helpers.SequenceBatchOnBackend(backend, 8, 4, 4)
        d = [backend.array(np.ascontiguousarray(a)) for a in (env_bad, off, nom, length)]
        dc = helpers.capi.SequenceDraws(*[a.ptr for a in d])
        assert backend.device.lib.rlt_rocm_gather_sequence_batch(backend.device.handle, C.byref(rb.c), C.byref(sampling), C.byref(dc), 20, C.byref(out.c)) == 0
        assert backend.device.lib.rlt_rocm_check_status(backend.device.handle) == helpers.capi.RLT_E_INVALID_ARGUMENT
        got = {k: v.numpy() for k, v in out.arrays.items()}
        keep = np.arange(8) != 3
        for k in helpers.SEQUENCE_BATCH_FIELDS:
            assert np.array_equal(got[k][:, keep], good[k][:, keep]), k
        assert np.all(got["observations_actions_base"][:, 3] == -777.0)
        # host-side checks
        lib, h = backend.device.lib, backend.device.handle
        assert lib.rlt_rocm_gather_sequence_batch(h, C.byref(rb.c), C.byref(sampling), None, 20, C.byref(out.c)) == helpers.capi.RLT_E_INVALID_ARGUMENT
        always = helpers.capi.SequenceSampling(1, 1, 1, 0.5, 1)
        assert lib.rlt_rocm_gather_sequence_batch(h, C.byref(rb.c), C.byref(always), C.byref(dc), 100, C.byref(out.c)) == helpers.capi.RLT_E_INVALID_ARGUMENT    # no eligible rows
    finally:
        backend.close()
