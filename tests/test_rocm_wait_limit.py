"""The bounded waits of the kernels whose workgroups wait for each other (the persistent SAC loop, rl/algorithms/sac/loop/core/operations_generic.h:110-155
in one launch; the update kernels that end with the optimiser's step): with the bound set to one poll from the host (rlt_rocm_set_wait_limit) the first
workgroups to arrive give up at once, every kernel still ends normally, and the next rlt_rocm_check_status reports RLT_E_DEVICE_TIMEOUT. The error is
sticky on that handle, so each case runs on a device handle of its own; the same calls on a fresh handle with the default bound succeed."""
import ctypes as C

import numpy as np
import pytest

import helpers
from test_rocm_sac_update import agent_parameters, batch_of

pytestmark = pytest.mark.gpu
capi = helpers.capi


def one_critic_update(backend, params, batch):
    rng = np.random.default_rng(5)
    agent = helpers.SacOnBackend(backend, batch, 64, params, masks=False)
    agent.set_batch(*batch_of(rng, batch, 3, 1))
    noise = backend.array(rng.standard_normal((batch, 1)).astype(np.float32))
    rc = backend.device.lib.rlt_rocm_sac_train_critic(backend.device.handle, C.byref(agent.c), 0, noise.ptr)
    return rc, agent


def test_update_kernel_gives_up_and_reports():
    params = agent_parameters(np.random.default_rng(1), 3, 1)
    impatient = helpers.RocmBackend()
    try:
        impatient.call("set_wait_limit", 1)
        rc, _ = one_critic_update(impatient, params, 256)
        assert rc == 0                                   # the launch itself succeeds
        lib, h = impatient.device.lib, impatient.device.handle
        assert lib.rlt_rocm_check_status(h) == capi.RLT_E_DEVICE_TIMEOUT
        assert b"gave up waiting" in lib.rlt_rocm_error_string(capi.RLT_E_DEVICE_TIMEOUT)
        assert lib.rlt_rocm_check_status(h) == capi.RLT_E_DEVICE_TIMEOUT      # sticky: the handle's results are void from here on
    finally:
        impatient.close()
    patient = helpers.RocmBackend()
    try:
        rc, agent = one_critic_update(patient, params, 256)
        assert rc == 0 and patient.device.lib.rlt_rocm_check_status(patient.device.handle) == 0
        assert np.abs(agent.parameters() - params).max() > 1e-5 and int(agent.critics[0].age.numpy()[0]) == 2
    finally:
        patient.close()


def test_persistent_loop_gives_up_and_reports(oracle):
    batch = 256
    loop, cfg = helpers.make_loop(oracle, batch)
    for _ in range(cfg.n_warmup_steps):
        assert oracle.lib.rlt_oracle_sac_loop_step(loop) == 0
    params = helpers.loop_parameters(oracle, loop)
    impatient = helpers.RocmBackend()
    try:
        impatient.call("set_wait_limit", 1)
        agent = helpers.SacOnBackend(impatient, batch, 64, params, masks=False)
        runner = helpers.RunnerOnBackend(impatient, 10000, oracle, loop)
        lib, h = impatient.device.lib, impatient.device.handle
        assert lib.rlt_rocm_sac_pendulum_loop(h, C.byref(agent.c), C.byref(runner.c), C.byref(runner.rb.c), 50, 7, 0, None, None) == 0
        assert lib.rlt_rocm_check_status(h) == capi.RLT_E_DEVICE_TIMEOUT      # the kernel left its step loop and ended
    finally:
        impatient.close()
        oracle.lib.rlt_oracle_sac_loop_destroy(loop)


def test_update_kernel_that_sums_per_xcd_gives_up_and_reports():
    """PPO's minibatch kernel at 8,192 rows (rl/algorithms/ppo/operations_generic.h:163-309): its 256 workgroups add their blocks of partial gradient sums up
    per XCD inside the launch, which makes the 16 workgroups of a network on one XCD wait for each other."""
    O, A, H, B = 105, 8, 64, 8192
    rng = np.random.default_rng(4)
    params = np.concatenate([helpers.random_params(rng, [O, H, H, A]), np.log(np.full(A, 0.5, np.float32)), helpers.random_params(rng, [O, H, H, 1])])
    ld = O + A + 3
    data = rng.standard_normal((B, ld)).astype(np.float32)
    pp = capi.ppo_parameters()

    def one_update(backend):
        agent = helpers.PpoOnBackend(backend, O, A, H, H, B, params, "tanh", "tanh", capi.adam_parameters(3e-4, epsilon=1e-8))
        dd = backend.array(data)
        rc = backend.device.lib.rlt_rocm_ppo_train_minibatch(backend.device.handle, C.byref(agent.c), C.byref(pp), dd.offset(0), dd.offset(0), dd.offset(O), dd.offset(O + A),
                                                             dd.offset(O + A + 1), dd.offset(O + A + 2), ld, None, None)
        return rc, agent

    impatient = helpers.RocmBackend()
    try:
        impatient.call("set_wait_limit", 1)
        rc, _ = one_update(impatient)
        assert rc == 0
        assert impatient.device.lib.rlt_rocm_check_status(impatient.device.handle) == capi.RLT_E_DEVICE_TIMEOUT
    finally:
        impatient.close()
    patient = helpers.RocmBackend()
    try:
        rc, agent = one_update(patient)
        assert rc == 0 and patient.device.lib.rlt_rocm_check_status(patient.device.handle) == 0
        assert np.abs(agent.parameters() - params).max() > 1e-5 and int(agent.actor.age.numpy()[0]) == 2
    finally:
        patient.close()
