"""Writes tests/golden/sequence_gather.npz from the REAL reference (oracle/_ref/librlt_ref_gather_seq_generic.so, built by oracle/Makefile from
/root/reference). Runs only where the reference is mounted; the committed .npz is data, not source.

The reference's SAC loop with three Pendulum environments, 30-step episodes and replay rings of 260 rows is stopped after 150 loop steps (rings not
full) and after 600 (wrapped twice). At each stop its gather_batch fills a SequentialBatch of 64 samples for three configurations: sequences of 8 with
the reference's defaults (start at the episode's first step, random lengths), sequences of 8 with both switched off, and single steps. Kept: the rings
(data, cursor, full flag, episode starts), every tensor of the reference's batch, and the draws behind it (environment, row offsets, length decisions)
as recovered by the restated gather running on the text form of the reference's std::mt19937 (it must reproduce the batch, or this script fails)."""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import helpers  # noqa: E402
from test_oracle_vs_reference import RefGatherSeq, SEQUENCE_SAMPLING  # noqa: E402

oracle = helpers.HostBackend()
ref = RefGatherSeq(0)
out = {"dims": np.array([ref.n_envs, ref.capacity, ref.max_episode_length, ref.batch, ref.sequence_length, ref.row]), "stops": np.array([150, 600]),
       "sampling": np.array([SEQUENCE_SAMPLING[v] for v in range(3)], np.float32)}
steps = 0
for si, stop in enumerate(out["stops"]):
    while steps < stop:
        ref.lib.rlt_ref_gather_seq_step(ref.h); steps += 1
    rings = ref.rings()
    out[f"s{si}_data"] = np.stack([r[0] for r in rings]); out[f"s{si}_position"] = np.array([r[1] for r in rings], np.uint32)
    out[f"s{si}_full"] = np.array([r[2] for r in rings], np.uint8); out[f"s{si}_episode_start"] = np.stack([r[3] for r in rings])
    for variant in range(3):
        S, rng, want = ref.gather(variant, 11 + variant)
        sampling = helpers.capi.SequenceSampling(*SEQUENCE_SAMPLING[variant])
        rb = helpers.replay_on_backend(oracle, rings)
        got = helpers.SequenceBatchOnBackend(oracle, ref.batch, S, ref.row // 2 - 1)
        env, off, nom, length = np.zeros(ref.batch, np.uint32), np.zeros((ref.batch, S + 1), np.uint32), np.zeros((ref.batch, S + 2), np.uint8), np.zeros((ref.batch, S + 2), np.uint32)
        assert oracle.lib.rlt_oracle_gather_sequence_batch_with_rng(C.byref(rb.c), C.byref(sampling), ref.max_episode_length, C.byref(got.c), rng, 16384, env.ctypes.data,
                                                                    off.ctypes.data, nom.ctypes.data, length.ctypes.data) == 0
        for k, v in got.numpy().items():
            assert np.array_equal(v, want[k]), (stop, variant, k)
            out[f"s{si}_v{variant}_{k}"] = want[k]
        out[f"s{si}_v{variant}_env_indices"], out[f"s{si}_v{variant}_sample_offsets"], out[f"s{si}_v{variant}_nominal"], out[f"s{si}_v{variant}_lengths"] = env, off, nom, length
np.savez_compressed(os.path.join(HERE, "sequence_gather.npz"), **out)
print("wrote sequence_gather.npz", len(out), "arrays")
