"""Writes tests/golden/gru_seed.npz from the REAL reference (oracle/_ref/librlt_ref_gru_generic.so, built by oracle/Makefile from
/root/reference). Runs only where the reference is mounted; the committed .npz is data (inputs/expected outputs), not source.

Two cases (without and with per-sample resets) of the reference's GRU layer at S=7, B=5, I=6, H=8: random weights, inputs and upstream
gradient, and what the reference's forward and backward_full produce from them (outputs, kept intermediates, d_input, the d_output it
accumulated into, the four gradients)."""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import helpers  # noqa: E402

ref = C.CDLL(helpers.REF_GRU_GENERIC)
dims = (C.c_int * 4)(); ref.rlt_ref_gru_dims(dims)
S, B, I, H = list(dims)
ref.rlt_ref_gru_forward_backward.argtypes = [C.c_void_p] * 17
out = {"dims": np.array([S, B, I, H])}
p = lambda a: a.ctypes.data_as(C.c_void_p)
for case, with_reset in (("plain", False), ("reset", True)):
    rng = np.random.default_rng(12 + with_reset)
    params, x, dy, reset = helpers.gru_random_case(rng, S, B, I, H, with_reset)
    want = dict(output=np.zeros((S, B, H), np.float32), post=np.zeros((S, B, 3 * H), np.float32), npp=np.zeros((S, B, H), np.float32), dx=np.zeros((S, B, I), np.float32),
                dW_i=np.zeros((3 * H, I), np.float32), db_i=np.zeros(3 * H, np.float32), dW_h=np.zeros((3 * H, H), np.float32), db_h=np.zeros(3 * H, np.float32),
                dy=np.zeros((S, B, H), np.float32))
    assert ref.rlt_ref_gru_forward_backward(p(params["W_i"]), p(params["b_i"]), p(params["W_h"]), p(params["b_h"]), p(params["h0"]), p(x), p(reset) if with_reset else None,
                                            p(dy), p(want["output"]), p(want["post"]), p(want["npp"]), p(want["dx"]), p(want["dW_i"]), p(want["db_i"]), p(want["dW_h"]),
                                            p(want["db_h"]), p(want["dy"])) == 0
    for k, v in params.items():
        out[f"{case}_param_{k}"] = v
    out[f"{case}_x"], out[f"{case}_d_output"] = x, dy
    if with_reset:
        out[f"{case}_reset"] = reset
    for k, v in want.items():
        out[f"{case}_want_{k}"] = v
np.savez_compressed(os.path.join(HERE, "gru_seed.npz"), **out)
print("wrote gru_seed.npz", len(out), "arrays")
