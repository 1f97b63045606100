"""Graph capture through the C ABI (rlt_rocm_graph_*; the reference's CUDA example records its loop step the same way,
src/rl/environments/pendulum/sac/cuda/sac.cu:122-164, devices/cuda.h:59,163): one SAC loop step recorded once and replayed must leave, bit
for bit, what the same number of unrecorded loop steps leaves -- parameters of all five networks, optimiser state, replay rows, runner state --
with fresh random numbers on every replay (the recorded graph ends by advancing the device's stream offset)."""
import ctypes as C

import numpy as np
import pytest

import helpers
from test_rocm_sac_update import agent_parameters

pytestmark = pytest.mark.gpu

RLT_E_CAPTURING = -6


class Loop:
    """agent, one Pendulum environment, its replay ring and the scratch arrays of rlt_rocm_sac_pendulum_loop_by_calls, warmed up with uniform actions"""

    def __init__(self, rocm, batch, hidden, capacity, seed):
        capi = helpers.capi
        self.rocm, self.seed = rocm, seed
        params = agent_parameters(np.random.default_rng(hidden), 3, 1, hidden)
        self.agent = helpers.SacOnBackend(rocm, batch, hidden, params, masks=False)
        self.rb = helpers.ReplayOnBackend(rocm, 1, capacity)
        self.states, self.ep_step, self.ep_ret, self.trunc = rocm.zeros((1, 2)), rocm.zeros((1,), np.uint32), rocm.zeros((1,)), rocm.array(np.ones(1, np.uint8))
        self.runner = capi.PendulumRunner(self.states.ptr, self.ep_step.ptr, self.ep_ret.ptr, self.trunc.ptr, 1, 200, capi.pendulum_parameters())
        self.buffers = [rocm.zeros((1, 1)), rocm.zeros((batch, 1)), rocm.zeros((batch, 1)), rocm.zeros((batch,), np.uint32), rocm.zeros((batch,), np.uint32)]
        self.scratch = capi.SacLoopScratch(*[b.ptr for b in self.buffers])
        warm_action = rocm.zeros((1, 1))
        for c in range(batch + 10):
            rocm.call("rand_f32", warm_action.ptr, 1, -1.0, 1.0, seed, 8 * c + 1)
            rocm.call("pendulum_runner_step", C.byref(self.runner), C.byref(self.rb.c), 0, self.agent.actor.layers, 3, C.byref(self.agent.c.sas), warm_action.ptr, None, None, seed, 8 * c + 2)

    def steps(self, n, first):
        self.rocm.call("sac_pendulum_loop_by_calls", C.byref(self.agent.c), C.byref(self.runner), C.byref(self.rb.c), n, self.seed, first, C.byref(self.scratch))

    def state(self):
        self.rocm.sync()
        return [self.agent.parameters(), self.agent.actor.m.numpy(), self.agent.critics[1].v.numpy(), self.rb.data.numpy(), self.states.numpy(), self.ep_ret.numpy(),
                self.agent.actor.age.numpy(), self.buffers[1].numpy(), self.buffers[3].numpy()]


def record_one_step(rocm, loop, first):
    graph = C.c_void_p()
    rocm.call("graph_begin_capture")
    try:
        loop.steps(1, first)
        rocm.call("advance_streams", 8)       # a loop step of the host loop uses the streams 8 g + 1 .. 8 g + 5
    finally:
        rocm.call("graph_end_capture", C.byref(graph))
    return graph


@pytest.mark.parametrize("hidden,batch,replays", [(64, 256, 1000), (256, 256, 1000)])
def test_replays_of_a_recorded_loop_step_equal_the_unrecorded_steps(rocm, hidden, batch, replays):
    """hidden 64: four launches per step (the fused kernels); hidden 256: the zoo's wider agents, one launch per operation (about sixty)"""
    first, chunk = 5000, replays // 5
    eager = Loop(rocm, batch, hidden, 1500, 21)
    eager.steps(3, first - 3)          # sizes every workspace the recorded calls will need
    checkpoints = []
    for k in range(5):
        eager.steps(chunk, first + k * chunk)
        checkpoints.append(eager.state())
    recorded = Loop(rocm, batch, hidden, 1500, 21)
    recorded.steps(3, first - 3)
    graph = record_one_step(rocm, recorded, first)
    try:
        for k in range(5):
            for _ in range(chunk):
                rocm.call("graph_launch", graph)
            # between the chunks the program reads everything back (waits, eager copies): every chunk of replays is checked, not only the last
            for got, ref in zip(recorded.state(), checkpoints[k]):
                assert np.array_equal(got, ref), k
    finally:
        rocm.call("set_stream_offset", 0)
        rocm.call("graph_destroy", graph)
    assert np.abs(checkpoints[-1][0] - checkpoints[0][0]).max() > 1e-4      # the steps trained


def test_what_a_recording_stream_cannot_do_is_refused(rocm):
    """allocation, host copies and a growing workspace return RLT_E_CAPTURING instead of breaking the recording; check_status does not wait"""
    lib, h = rocm.device.lib, rocm.device.handle
    x = rocm.zeros((16,))
    host = np.zeros(16, np.float32)
    ptr = C.c_void_p()
    graph = C.c_void_p()
    rocm.call("graph_begin_capture")
    try:
        assert lib.rlt_rocm_malloc(h, C.byref(ptr), 1024) == RLT_E_CAPTURING
        assert lib.rlt_rocm_memcpy_d2h(h, host.ctypes.data, x.ptr, 64) == RLT_E_CAPTURING
        assert lib.rlt_rocm_graph_begin_capture(h) == RLT_E_CAPTURING
        assert lib.rlt_rocm_check_status(h) == 0
        rocm.call("fill_f32", x.ptr, 1, 16, 16, 3.0)
    finally:
        rocm.call("graph_end_capture", C.byref(graph))
    assert not x.numpy().any()              # recorded, not run
    rocm.call("graph_launch", graph)
    assert np.all(x.numpy() == 3.0)
    rocm.call("graph_destroy", graph)
    assert lib.rlt_rocm_malloc(h, C.byref(ptr), 1024) == 0 and lib.rlt_rocm_free(h, ptr) == 0


def test_replays_of_recorded_td3_updates_with_their_draws_equal_the_unrecorded_calls(rocm):
    """TD3 at width 256 (batch 100, observation 6, action 1: the update kernel for hidden widths beyond 64): one update set -- the smoothing noise,
    both critics and their targets by rlt_rocm_td3_train_critics_drawn, the actor by rlt_rocm_td3_train_actor_drawn, the actor's target -- recorded once with the stream
    offset advanced at its end, replayed 200 times on one batch, against the same calls unrecorded with the stream numbers written out: every parameter, gradient and
    optimiser age and the smoothing noise of the last set, bit for bit, at four points on the way."""
    batch, obs, act, hidden, sets = 100, 6, 1, 256, 200
    rng = np.random.default_rng(11)
    D = obs + act
    nets = [helpers.random_params(rng, [obs, hidden, hidden, act])] * 2 + [helpers.random_params(rng, [D, hidden, hidden, 1]) for _ in range(2)]
    params = np.concatenate(nets + [nets[2], nets[3]]).astype(np.float32)
    hyper = dict(gamma=0.99, actor_polyak=0.995, critic_polyak=0.995, sampling_std=0.1, adam=helpers.capi.adam_parameters(epsilon=1e-7))
    oab = rng.standard_normal((2, batch, D)).astype(np.float32); oab[:, :, obs:] = np.clip(oab[:, :, obs:], -1, 1)
    rewards, term = rng.standard_normal(batch).astype(np.float32), (rng.random(batch) < 0.1).astype(np.uint8)
    agents = [helpers.Td3OnBackend(rocm, batch, hidden, params, hyper=hyper, masks=False, obs=obs, act=act) for _ in range(2)]
    for ag in agents:
        ag.set_batch(oab, rewards, term, np.zeros((batch, act), np.float32))
    seed, base = 77, 1000

    def update_set(ag, first_stream):
        draws = helpers.capi.Td3CriticDraws(seed, first_stream, (C.c_uint64 * 2)(first_stream + 1, first_stream + 2), 0.2, 0.5)
        rocm.call("td3_train_critics_drawn", C.byref(ag.c), C.byref(draws), None, 1)
        rocm.call("td3_train_actor_drawn", C.byref(ag.c), seed, first_stream + 3, None)
        rocm.call("td3_update_actor_target", C.byref(ag.c))

    def state(ag):
        rocm.sync()
        return [ag.parameters(), ag.gradients(), ag.ages(), ag.target_noise.numpy(), ag.target_q.numpy()]

    eager, recorded = agents
    for ag in agents:
        update_set(ag, base - 4)         # sizes every workspace the recorded calls will need
    checkpoints = []
    for g in range(sets):
        update_set(eager, base + 4 * g)
        if g % 50 == 49:
            checkpoints.append(state(eager))
    graph = C.c_void_p()
    rocm.call("graph_begin_capture")
    try:
        update_set(recorded, base)
        rocm.call("advance_streams", 4)
    finally:
        rocm.call("graph_end_capture", C.byref(graph))
    try:
        for k in range(4):
            for _ in range(50):
                rocm.call("graph_launch", graph)
            for got, ref in zip(state(recorded), checkpoints[k]):
                assert np.array_equal(got, ref), k
    finally:
        rocm.call("set_stream_offset", 0)
        rocm.call("graph_destroy", graph)
    assert np.abs(checkpoints[-1][0] - params).max() > 1e-4
