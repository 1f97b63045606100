"""TD3 on sequence batches with sequential (recurrent) networks through the C ABI (rlt_rocm_td3_sequence_*) against the CPU checker, which reproduces the
reference's TD3 loop with its recurrent approximators bit for bit (tests/test_oracle_vs_reference.py).

Tolerance: 1e-5 relative to the largest magnitude of the checker's tensor for parameters and buffers after one training step from identical state (critic
gradients carry the TD-error conditioning and are compared at 1e-4); Adam ages exactly."""
import numpy as np
import pytest

import helpers
from helpers import rel_err
from test_rocm_sac_sequence import synthetic_sequence_batch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case", [(6, 16, 3, 1, 16, 1, True), (20, 64, 5, 2, 32, 2, True), (10, 100, 3, 1, 64, 1, False), (100, 100, 3, 1, 16, 2, True)])
def test_td3_sequence_updates_match_checker(oracle, rocm, case):
    """Three training steps (critics, critic targets, actor, actor target) from identical state; the device agent is re-synchronised to the checker's
    parameters before each step. Shapes: the reference's recurrent TD3 approximators (GRU, GRU[, dense], dense), also with an input dense layer."""
    print("case", case, flush=True)
    S, B, OBS, ACT, H, variant, include_first = case
    rng = np.random.default_rng(S * B + H)
    body = [(1, None, H, "identity"), (1, H, H, "identity")] + ([(0, H, H, "relu")] if variant == 2 else [])
    nets = []
    for in_dim, out_dim in ((OBS, ACT), (OBS + ACT, 1)):
        specs = [(k, in_dim if i is None else i, o, a) for k, i, o, a in body] + [(0, H, out_dim, "identity")]
        nets.append(specs)
    actor_specs, critic_specs = nets
    pa, pc = helpers.random_seq_params(rng, actor_specs), [helpers.random_seq_params(rng, critic_specs) for _ in range(2)]
    params = np.concatenate([pa, pc[0], pc[1], pa, pc[0], pc[1]])
    agents = [helpers.Td3SequenceOnBackend(be, actor_specs, critic_specs, params, S, B, OBS, ACT, include_first) for be in (oracle, rocm)]
    T = S + (1 if include_first else 0)
    for step in range(3):
        data = synthetic_sequence_batch(rng, S, B, OBS + ACT)
        noise = np.clip(rng.standard_normal((T, B, ACT)) * 0.2, -0.5, 0.5).astype(np.float32)
        cpu, gpu = agents
        for a, b in zip([cpu.actor, *cpu.critics, cpu.actor_target, *cpu.targets], [gpu.actor, *gpu.critics, gpu.actor_target, *gpu.targets]):
            b.params.upload(a.params.numpy())
            if a.grads is not None:
                b.m.upload(a.m.numpy()); b.v.upload(a.v.numpy()); b.age.upload(a.age.numpy())
        for ag in agents:
            ag.set_batch(data)
            ag.train(noise)
        assert gpu.ages() == cpu.ages()
        for name, a, b in [("actor", cpu.actor, gpu.actor), ("critic0", cpu.critics[0], gpu.critics[0]), ("critic1", cpu.critics[1], gpu.critics[1]),
                           ("actor_target", cpu.actor_target, gpu.actor_target), ("target0", cpu.targets[0], gpu.targets[0]), ("target1", cpu.targets[1], gpu.targets[1])]:
            assert rel_err(b.params.numpy(), a.params.numpy()) <= 1e-5, (step, name, rel_err(b.params.numpy(), a.params.numpy()))
            if a.grads is not None:
                assert rel_err(b.grads.numpy(), a.grads.numpy()) <= 1e-4, (step, name, "gradient", rel_err(b.grads.numpy(), a.grads.numpy()))
        for k in ("nsavi", "next_q0", "next_q1", "target", "savi", "d_ci", "d_ao", "d_output"):
            assert rel_err(gpu.buf[k].numpy(), cpu.buf[k].numpy()) <= 1e-5, (step, k, rel_err(gpu.buf[k].numpy(), cpu.buf[k].numpy()))


def test_td3_sequence_rejects_inconsistent_arguments(rocm):
    import ctypes as C
    rng = np.random.default_rng(0)
    actor_specs = [(1, 3, 16, "identity"), (0, 16, 1, "identity")]
    critic_specs = [(1, 4, 16, "identity"), (0, 16, 1, "identity")]
    pa, pc = helpers.random_seq_params(rng, actor_specs), helpers.random_seq_params(rng, critic_specs)
    agent = helpers.Td3SequenceOnBackend(rocm, actor_specs, critic_specs, np.concatenate([pa, pc, pc, pa, pc, pc]), 4, 8, 3, 1)
    agent.set_batch(synthetic_sequence_batch(rng, 4, 8, 4))
    lib, h = rocm.device.lib, rocm.device.handle
    assert lib.rlt_rocm_td3_sequence_train_critic(h, C.byref(agent.c), 2) != 0
    keep = agent.c.actor_input
    agent.c.actor_input = None
    assert lib.rlt_rocm_td3_sequence_train_actor(h, C.byref(agent.c)) != 0
    agent.c.actor_input = keep
    agent.c.workspace_bytes = 16
    assert lib.rlt_rocm_td3_sequence_train_critic(h, C.byref(agent.c), 0) != 0
    agent.c.workspace_bytes = int(lib.rlt_rocm_td3_sequence_workspace_bytes(C.byref(agent.c)))
    assert lib.rlt_rocm_td3_sequence_train_critic(h, C.byref(agent.c), 0) == 0 and lib.rlt_rocm_td3_sequence_train_actor(h, C.byref(agent.c)) == 0
    rocm.sync()


@pytest.mark.parametrize("case", [(100, 100, 3, 1, 16, 2, True), (10, 100, 3, 1, 64, 1, False), (48, 64, 5, 2, 32, 2, True)])
def test_both_critics_in_one_call_leave_the_bits_of_the_two_calls(rocm, case):
    """rlt_rocm_td3_sequence_train_critics (the target part once, the two critics' passes side by side on the handle's streams from 48 steps up) against
    rlt_rocm_td3_sequence_train_critic for critic 0 and then for critic 1: three training steps each from the same parameters, batches and noise; every parameter,
    gradient and optimiser age and the training buffers that both leave behind, bit for bit."""
    S, B, OBS, ACT, H, variant, include_first = case
    rng = np.random.default_rng(S * B + 7 * H)
    body = [(1, None, H, "identity"), (1, H, H, "identity")] + ([(0, H, H, "relu")] if variant == 2 else [])
    actor_specs, critic_specs = ([(k, in_dim if i is None else i, o, a) for k, i, o, a in body] + [(0, H, out_dim, "identity")] for in_dim, out_dim in ((OBS, ACT), (OBS + ACT, 1)))
    pa, pc = helpers.random_seq_params(rng, actor_specs), [helpers.random_seq_params(rng, critic_specs) for _ in range(2)]
    params = np.concatenate([pa, pc[0], pc[1], pa, pc[0] * 0.9, pc[1] * 1.1])
    agents = [helpers.Td3SequenceOnBackend(rocm, actor_specs, critic_specs, params, S, B, OBS, ACT, include_first) for _ in range(2)]
    T = S + (1 if include_first else 0)
    for step in range(3):
        data = synthetic_sequence_batch(rng, S, B, OBS + ACT)
        noise = np.clip(rng.standard_normal((T, B, ACT)) * 0.2, -0.5, 0.5).astype(np.float32)
        for ag, together in zip(agents, (False, True)):
            ag.set_batch(data)
            ag.train(noise, both_critics_in_one_call=together)
        assert np.array_equal(agents[0].parameters(), agents[1].parameters()), (case, step)
        assert agents[0].ages() == agents[1].ages()
        for a, b in zip([agents[0].actor, *agents[0].critics], [agents[1].actor, *agents[1].critics]):
            assert np.array_equal(a.grads.numpy(), b.grads.numpy()), (case, step)
        for k in ("nsavi", "next_q0", "next_q1", "target", "savi", "d_ci", "d_ao", "d_output"):
            assert np.array_equal(agents[0].buf[k].numpy(), agents[1].buf[k].numpy()), (case, step, k)
    assert np.abs(agents[1].parameters() - params).max() > 1e-4
