"""Writes tests/golden/sac_pendulum_seed0.npz from the REAL reference (oracle/_ref/librlt_ref_generic.so, built by oracle/Makefile
from /root/reference). Runs only where the reference is mounted; the committed .npz is data (inputs/expected outputs), not source.

Per batch size (100 and 256) the reference's seeded SAC-on-Pendulum loop is stepped and, at a few step counts, recorded:
every 16th parameter of the flat parameter vector (actor, critic 0/1, target 0/1, log_alpha), float64 sum and sum of squares of
the whole vector, the first rows of the replay ring, and the gathered batch / noise of that step."""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
ref = C.CDLL(os.path.join(ROOT, "oracle", "_ref", "librlt_ref_generic.so"))
ref.rlt_ref_sac_create.restype = C.c_void_p
ref.rlt_ref_sac_parameter_count.restype = C.c_size_t
ref.rlt_ref_sac_parameter_count.argtypes = [C.c_void_p]
P = C.c_void_p
for name, args in dict(step=[P], get_parameters=[P, P], get_batch=[P, P, P, P], get_masks=[P, P, P, P, P], get_noise=[P, P, P],
                       get_replay=[P, P, P, P, P]).items():
    getattr(ref, "rlt_ref_sac_" + name).argtypes = args

out = {}
for batch, checkpoints in ((100, [0, 100, 101, 150, 300]), (256, [256, 257, 300, 500])):
    h = C.c_void_p(ref.rlt_ref_sac_create(0, batch))
    n = ref.rlt_ref_sac_parameter_count(h)
    p = np.zeros(n, np.float32)
    done = 0
    for cp in checkpoints:
        while done < cp:
            ref.rlt_ref_sac_step(h); done += 1
        ref.rlt_ref_sac_get_parameters(h, p.ctypes.data)
        key = f"b{batch}_s{cp}"
        out[key + "_params16"] = p[::16].copy()
        out[key + "_sum"] = np.array([p.astype(np.float64).sum(), (p.astype(np.float64) ** 2).sum()])
        data = np.zeros((10000, 10), np.float32); pos = C.c_uint32(); full = C.c_uint8()
        ref.rlt_ref_sac_get_replay(h, data.ctypes.data, C.byref(pos), C.byref(full), None)
        out[key + "_replay_tail"] = data[max(0, pos.value - 8):pos.value].copy()
        out[key + "_replay_pos"] = np.array([pos.value, full.value])
        if cp > max(batch, 100):
            oab = np.zeros((2, batch, 4), np.float32); rew = np.zeros(batch, np.float32); term = np.zeros(batch, np.uint8)
            ref.rlt_ref_sac_get_batch(h, oab.ctypes.data, rew.ctypes.data, term.ctypes.data)
            nc, na = np.zeros(batch, np.float32), np.zeros(batch, np.float32)
            ref.rlt_ref_sac_get_noise(h, nc.ctypes.data, na.ctypes.data)
            masks = [np.zeros(batch, np.uint8), np.zeros(2 * batch, np.uint8), np.zeros(batch, np.uint8), np.zeros(2 * batch, np.uint8)]
            ref.rlt_ref_sac_get_masks(h, *[m.ctypes.data for m in masks])
            out[key + "_oab"] = oab; out[key + "_rewards"] = rew; out[key + "_terminated"] = term
            out[key + "_noise_critic"] = nc; out[key + "_noise_actor"] = na
            for name, m in zip(("reset", "next_reset_base", "final_step_mask", "next_final_step_mask_base"), masks):
                out[key + "_" + name] = m
np.savez_compressed(os.path.join(HERE, "sac_pendulum_seed0.npz"), **out)
print("wrote", len(out), "arrays")
