"""Builders of networks, agents, runners and batches on a backend, for the benchmark, the smoke run and the tests: each lays out device arrays
and fills the C ABI's descriptors (capi.py) the way the reference's objects hold the same state. A backend is anything with array / zeros / call /
sync (RocmBackend below: the HIP library through its C ABI); the tests hand the same builders a second backend of their own to check against."""
import ctypes as C

import numpy as np

from . import capi


class RocmBackend:
    """The HIP library through its C ABI."""
    name = "rocm"

    def __init__(self):
        self.device = capi.Device(0)
        self._ws = None

    def array(self, a):
        return self.device.array(np.ascontiguousarray(a))

    def zeros(self, shape, dtype=np.float32):
        return self.device.zeros(shape, dtype)

    def call(self, fn, *args):
        self.device.call(fn, *args)

    def workspace(self, nbytes):
        nbytes = int(nbytes)
        if self._ws is None or self._ws.nbytes < nbytes:
            self._ws = self.device.empty((nbytes,), np.uint8)
        return self._ws.ptr, self._ws.nbytes

    def sync(self):
        self.device.sync()

    def close(self):
        self.device.close()


def mlp_param_count(dims):
    return sum(dims[i] * dims[i + 1] + dims[i + 1] for i in range(len(dims) - 1))


def xavier_params(rng, dims):
    """Xavier-uniform weights, zero biases, flattened per layer as [weights, biases]."""
    parts = []
    for i in range(len(dims) - 1):
        bound = np.sqrt(6.0 / (dims[i] + dims[i + 1]))
        parts.append(rng.uniform(-bound, bound, size=dims[i + 1] * dims[i]).astype(np.float32))
        parts.append(np.zeros(dims[i + 1], np.float32))
    return np.concatenate(parts)


def random_params(rng, dims, bias_scale=0.1):
    parts = []
    for i in range(len(dims) - 1):
        bound = 1.0 / np.sqrt(dims[i])
        parts.append(rng.uniform(-bound, bound, size=dims[i + 1] * dims[i]).astype(np.float32))
        parts.append(rng.uniform(-bias_scale, bias_scale, size=dims[i + 1]).astype(np.float32))
    return np.concatenate(parts)


def fold_standardize_into_first_layer(dims, params, mean, precision):
    """The flat parameters of the network that computes W1 ((x - mean) * precision) + b1 as W1' x + b1' (in double, rounded once)."""
    out = params.astype(np.float32).copy()
    n_w = dims[1] * dims[0]
    w = params[:n_w].reshape(dims[1], dims[0]).astype(np.float64) * np.asarray(precision, np.float64)[None, :]
    b = params[n_w:n_w + dims[1]].astype(np.float64) - w @ np.asarray(mean, np.float64)
    out[:n_w] = w.reshape(-1).astype(np.float32)
    out[n_w:n_w + dims[1]] = b.astype(np.float32)
    return out


class Mlp:
    """A dense network laid out as flat arenas (parameters, gradients, Adam moments) on a backend, described to the C ABI
    by an array of rlt_dense_layer."""

    def __init__(self, backend, dims, params, batch, hidden_act="relu", out_act="identity", trainable=True):
        self.backend, self.dims, self.batch, self.trainable = backend, list(dims), batch, trainable
        self.n = len(dims) - 1
        total = mlp_param_count(dims)
        assert params.size == total
        self.params = backend.array(params.astype(np.float32))
        if trainable:
            self.grads = backend.zeros((total,)); self.m = backend.zeros((total,)); self.v = backend.zeros((total,))
            self.pre = [backend.zeros((batch, dims[i + 1])) for i in range(self.n)]
            self.out = [backend.zeros((batch, dims[i + 1])) for i in range(self.n)]
            self.age = backend.array(np.array([1], np.uint32))
        self.layers = (capi.DenseLayer * self.n)()
        adam = []
        off = 0
        self.offsets = []
        for i in range(self.n):
            nw, nb = dims[i] * dims[i + 1], dims[i + 1]
            L = self.layers[i]
            L.in_dim, L.out_dim = dims[i], dims[i + 1]
            L.activation = capi.ACT[out_act if i == self.n - 1 else hidden_act]
            L.weights, L.biases = self.params.offset(off), self.params.offset(off + nw)
            if trainable:
                L.d_weights, L.d_biases = self.grads.offset(off), self.grads.offset(off + nw)
                L.pre_activations, L.output = self.pre[i].ptr, self.out[i].ptr
                adam.append(capi.AdamTensor(L.weights, L.d_weights, self.m.offset(off), self.v.offset(off), None, nw, 1))
                adam.append(capi.AdamTensor(L.biases, L.d_biases, self.m.offset(off + nw), self.v.offset(off + nw), None, nb, 2))
            self.offsets.append((off, nw, nb))
            off += nw + nb
        self.adam = (capi.AdamTensor * len(adam))(*adam)
        self.n_adam = len(adam)

    def workspace(self):
        if self.backend.name != "rocm":
            return None, 0
        nbytes = self.backend.device.lib.rlt_rocm_mlp_workspace_bytes(self.layers, self.n, self.batch)
        return self.backend.workspace(nbytes)


class ArenaView:
    """A tensor inside a flat array of a backend: what the C ABI needs of it (`ptr`) and its contents."""

    def __init__(self, arena, start, shape):
        self.arena, self.start, self.shape = arena, start, tuple(shape)
        self.ptr = arena.offset(start)

    def numpy(self):
        n = int(np.prod(self.shape))
        return self.arena.numpy()[self.start:self.start + n].reshape(self.shape)


class GruOnBackend:
    """One GRU layer (parameters, gradients, kept intermediates) on a backend. params: dict W_i [3H x I], b_i, W_h [3H x H], b_h, h0.
    The four gradient tensors share one flat array (`grads`), so that one fill clears them."""

    def __init__(self, backend, S, B, I, H, params, fast_tanh=False):
        self.backend, self.S, self.B, self.I, self.H = backend, S, B, I, H
        f = lambda k: backend.array(np.asarray(params[k], np.float32))
        self.W_i, self.b_i, self.W_h, self.b_h, self.h0 = f("W_i"), f("b_i"), f("W_h"), f("b_h"), f("h0")
        self.grads = backend.zeros((3 * H * I + 3 * H + 3 * H * H + 3 * H,))
        self.dW_i, self.db_i = ArenaView(self.grads, 0, (3 * H, I)), ArenaView(self.grads, 3 * H * I, (3 * H,))
        self.dW_h, self.db_h = ArenaView(self.grads, 3 * H * I + 3 * H, (3 * H, H)), ArenaView(self.grads, 3 * H * I + 3 * H + 3 * H * H, (3 * H,))
        self.post, self.npp, self.out = backend.zeros((S, B, 3 * H)), backend.zeros((S, B, H)), backend.zeros((S, B, H))
        self.c = capi.GruLayer(self.W_i.ptr, self.b_i.ptr, self.W_h.ptr, self.b_h.ptr, self.h0.ptr, self.dW_i.ptr, self.db_i.ptr, self.dW_h.ptr, self.db_h.ptr,
                               self.post.ptr, self.npp.ptr, self.out.ptr, I, H, int(fast_tanh), 0)
        self.ws, self.wsn = (None, 0)
        if backend.name == "rocm":
            n = backend.device.lib.rlt_rocm_gru_workspace_bytes(C.byref(self.c), S, B)
            self._ws = backend.device.empty((max(int(n), 4),), np.uint8)
            self.ws, self.wsn = self._ws.ptr, int(n)

    def forward(self, x, reset=None):
        self.x = self.backend.array(np.asarray(x, np.float32))
        self.reset = self.backend.array(np.asarray(reset, np.uint8)) if reset is not None else None
        self.backend.call("gru_forward", C.byref(self.c), self.x.ptr, self.reset.ptr if self.reset else None, self.S, self.B, self.ws, self.wsn)

    def backward(self, d_output, want_d_input=True, want_w=1):
        self.dy = self.backend.array(np.asarray(d_output, np.float32))
        self.dx = self.backend.zeros((self.S, self.B, self.I))
        self.backend.call("gru_backward", C.byref(self.c), self.x.ptr, self.dy.ptr, self.dx.ptr if want_d_input else None, self.reset.ptr if self.reset else None,
                          self.S, self.B, want_w, self.ws, self.wsn)

    def results(self):
        return dict(output=self.out.numpy(), post=self.post.numpy(), npp=self.npp.numpy(), dx=self.dx.numpy(), dy=self.dy.numpy(), dW_i=self.dW_i.numpy(),
                    db_i=self.db_i.numpy(), dW_h=self.dW_h.numpy(), db_h=self.db_h.numpy())


def gru_random_case(rng, S, B, I, H, with_reset):
    params = dict(W_i=rng.uniform(-0.4, 0.4, (3 * H, I)), b_i=rng.uniform(-0.4, 0.4, 3 * H), W_h=rng.uniform(-0.4, 0.4, (3 * H, H)), b_h=rng.uniform(-0.4, 0.4, 3 * H),
                  h0=rng.uniform(-0.5, 0.5, H))
    params = {k: v.astype(np.float32) for k, v in params.items()}
    x = rng.standard_normal((S, B, I)).astype(np.float32); dy = rng.standard_normal((S, B, H)).astype(np.float32)
    reset = (rng.random((S, B)) < 0.25).astype(np.uint8) if with_reset else None
    return params, x, dy, reset


class PpoOnBackend:
    """PPO actor (MLP + action log_std), critic and their Adam state on one backend. Flat parameter order:
    actor [W|b per layer], log_std, critic [W|b per layer] (what the reference harness exports)."""

    def __init__(self, backend, obs_dim, action_dim, actor_hidden, critic_hidden, batch, params, actor_act="relu", critic_act="relu",
                 adam=None, obs_privileged_dim=None, standardize=None):
        self.backend, self.batch, self.action_dim = backend, batch, action_dim
        opd = obs_dim if obs_privileged_dim is None else obs_privileged_dim
        adims, cdims = [obs_dim, actor_hidden, actor_hidden, action_dim], [opd, critic_hidden, critic_hidden, 1]
        na, nc = mlp_param_count(adims), mlp_param_count(cdims)
        assert params.size == na + action_dim + nc
        self.actor = Mlp(backend, adims, params[:na], batch, actor_act, "identity")
        self.critic = Mlp(backend, cdims, params[na + action_dim:], batch, critic_act, "identity")
        self.log_std = backend.array(params[na:na + action_dim].astype(np.float32))
        self.d_log_std, self.m_log_std, self.v_log_std = (backend.zeros((action_dim,)) for _ in range(3))
        tensors = list(self.actor.adam) + [capi.AdamTensor(self.log_std.ptr, self.d_log_std.ptr, self.m_log_std.ptr, self.v_log_std.ptr, None, action_dim, 1)]
        self.actor_adam = (capi.AdamTensor * len(tensors))(*tensors)
        adam = adam or capi.adam_parameters(epsilon=1e-8)
        self.c = capi.PpoAgent(self.actor.layers, self.actor.n, self.critic.layers, self.critic.n, self.log_std.ptr, self.d_log_std.ptr,
                               self.actor_adam, len(tensors), self.critic.adam, self.critic.n_adam, adam, adam, self.actor.age.ptr, self.critic.age.ptr,
                               obs_dim, opd, action_dim, batch, None, 0)
        if standardize is not None:     # (actor mean, actor precision, critic mean, critic precision): standardize layers in front of the networks
            self.standardize = [backend.array(np.asarray(v, np.float32)) for v in standardize]
            (self.c.actor_standardize_mean, self.c.actor_standardize_precision, self.c.critic_standardize_mean,
             self.c.critic_standardize_precision) = [v.ptr for v in self.standardize]
        if backend.name == "rocm":
            n = backend.device.lib.rlt_rocm_ppo_workspace_bytes(C.byref(self.c))
            self.ws = backend.device.empty((int(n),), np.uint8)
            self.c.workspace, self.c.workspace_bytes = self.ws.ptr, n

    def parameters(self):
        return np.concatenate([self.actor.params.numpy(), self.log_std.numpy(), self.critic.params.numpy()])


class ReplayOnBackend:
    def __init__(self, backend, n_envs, capacity, obs_dim=3, act_dim=1):
        self.backend = backend
        self.row = 2 * obs_dim + act_dim + 3
        self.data = backend.zeros((n_envs * capacity, self.row))
        self.episode_start = backend.zeros((n_envs * capacity,), np.uint32)
        self.position = backend.zeros((n_envs,), np.uint32)
        self.current_episode_start = backend.zeros((n_envs,), np.uint32)
        self.full = backend.zeros((n_envs,), np.uint8)
        self.c = capi.ReplayBuffer(self.data.ptr, self.episode_start.ptr, self.position.ptr, self.current_episode_start.ptr, self.full.ptr,
                                   n_envs, capacity, obs_dim, act_dim)


class EnvRunnerOnBackend:
    """The off-policy runner's state and per-step buffers for any environment kind on one backend (all environments truncated at the start,
    as the reference initialises them)."""

    def __init__(self, backend, env_kind, n_envs, episode_step_limit):
        self.backend, self.kind, self.n = backend, env_kind, n_envs
        sd, od, ad = capi.ENV_DIMS[env_kind]
        z = backend.zeros
        self.states, self.ep_step, self.ep_ret = z((n_envs, sd)), z((n_envs,), np.uint32), z((n_envs,))
        self.trunc = backend.array(np.ones(n_envs, np.uint8))
        self.obs, self.act, self.next_obs, self.rew, self.term = z((n_envs, od)), z((n_envs, ad)), z((n_envs, od)), z((n_envs,)), z((n_envs,), np.uint8)
        c = capi.EnvRunner()
        c.env_kind, c.n_envs, c.episode_step_limit = env_kind, n_envs, episode_step_limit
        c.states, c.episode_step, c.episode_return, c.truncated = self.states.ptr, self.ep_step.ptr, self.ep_ret.ptr, self.trunc.ptr
        c.pendulum, c.acrobot, c.car = capi.pendulum_parameters(), capi.acrobot_parameters(), capi.car_parameters()
        c.observations, c.actions, c.next_observations, c.rewards, c.terminated = self.obs.ptr, self.act.ptr, self.next_obs.ptr, self.rew.ptr, self.term.ptr
        self.c = c

    def workspace(self, policy_kind, actor):
        if self.backend.name != "rocm" or policy_kind == 0:
            return None, 0
        lib = self.backend.device.lib
        return self.backend.workspace(lib.rlt_rocm_env_runner_step_workspace_bytes(C.byref(self.c), policy_kind, actor.layers if actor else None, actor.n if actor else 0))

    def snapshot(self):
        return [a.numpy() for a in (self.states, self.ep_step, self.ep_ret, self.trunc, self.obs, self.act, self.next_obs, self.rew, self.term)]


class SacOnBackend:
    """All SAC state on one backend (default: the Pendulum shapes, observation 3, action 1). params: actor, critic 0, critic 1, target 0, target 1, log_alpha."""

    def __init__(self, backend, batch, hidden, params, adam_eps=1e-7, masks=True, obs=3, act=1, hidden_act="relu"):
        OBS, ACT, D = obs, act, obs + act
        self.backend, self.batch = backend, batch
        n_actor = mlp_param_count([OBS, hidden, hidden, 2 * ACT]); n_critic = mlp_param_count([D, hidden, hidden, 1])
        o = 0
        self.actor = Mlp(backend, [OBS, hidden, hidden, 2 * ACT], params[o:o + n_actor], batch, hidden_act); o += n_actor
        self.critics = []
        for _ in range(2):
            self.critics.append(Mlp(backend, [D, hidden, hidden, 1], params[o:o + n_critic], batch, hidden_act)); o += n_critic
        self.targets = []
        for _ in range(2):
            self.targets.append(Mlp(backend, [D, hidden, hidden, 1], params[o:o + n_critic], batch, hidden_act, trainable=False)); o += n_critic
        self.log_alpha = backend.array(np.array([params[o], 0, 0, 0], np.float32))
        self.alpha_age = backend.array(np.array([1], np.uint32))
        z = backend.zeros
        self.oab = z((2, batch, D)); self.rewards = z((batch,)); self.terminated = z((batch,), np.uint8)
        self.m_final = backend.array(np.ones(batch, np.uint8)); self.m_next_final = backend.array(np.ones(batch, np.uint8))
        self.m_reset = backend.array(np.ones(batch, np.uint8))
        self.nsavi = z((batch, D)); self.next_q = [z((batch,)), z((batch,))]; self.next_lp = z((batch,)); self.target_q = z((batch,))
        self.d_out_c = [z((batch,)), z((batch,))]; self.savi = z((batch, D)); self.d_out_a = z((batch,))
        self.d_ci = [z((batch, D)), z((batch, D))]; self.d_aos = z((batch, ACT)); self.d_ao = z((batch, 2 * ACT))
        self.a_pre = z((batch, ACT)); self.a_lp = z((batch,)); self.a_act = z((batch, ACT))
        A = capi.SacAgent()
        A.batch, A.observation_dim, A.action_dim, A.n_actor_layers, A.n_critic_layers = batch, OBS, ACT, 3, 3
        A.gamma, A.polyak = 0.99, float(np.float32(1.0 - 0.005))
        A.sas = capi.SasParameters(-20.0, 2.0, 1e-6, -float(ACT))
        A.actor_adam = A.critic_adam = A.alpha_adam = capi.adam_parameters(epsilon=adam_eps)
        A.actor = self.actor.layers
        A.actor_adam_tensors, A.n_actor_adam_tensors = self.actor.adam, self.actor.n_adam
        for k in range(2):
            A.critics[k] = self.critics[k].layers; A.critics_target[k] = self.targets[k].layers
            A.critic_adam_tensors[k] = self.critics[k].adam; A.critic_age[k] = self.critics[k].age.ptr
            A.next_q[k] = self.next_q[k].ptr; A.d_output_critic[k] = self.d_out_c[k].ptr; A.d_critic_input[k] = self.d_ci[k].ptr
        A.n_critic_adam_tensors = self.critics[0].n_adam
        la = self.log_alpha
        A.log_alpha = capi.AdamTensor(la.offset(0), la.offset(1), la.offset(2), la.offset(3), None, 1, 0)
        A.actor_age, A.alpha_age = self.actor.age.ptr, self.alpha_age.ptr
        A.observations_actions_base, A.rewards, A.terminated = self.oab.ptr, self.rewards.ptr, self.terminated.ptr
        if masks:
            A.final_step_mask, A.next_final_step_mask, A.reset = self.m_final.ptr, self.m_next_final.ptr, self.m_reset.ptr
        A.next_state_action_value_input, A.next_log_probabilities, A.target_action_value = self.nsavi.ptr, self.next_lp.ptr, self.target_q.ptr
        A.state_action_value_input, A.d_output_actor_critics = self.savi.ptr, self.d_out_a.ptr
        A.d_actor_output_squashing, A.d_actor_output = self.d_aos.ptr, self.d_ao.ptr
        A.actor_pre_squashing, A.actor_log_probabilities, A.actor_actions = self.a_pre.ptr, self.a_lp.ptr, self.a_act.ptr
        if backend.name == "rocm":
            lib = backend.device.lib
            nbytes = max(lib.rlt_rocm_mlp_workspace_bytes(self.actor.layers, 3, batch), lib.rlt_rocm_mlp_workspace_bytes(self.critics[0].layers, 3, batch))
            nbytes += batch * 2 * ACT * 4 + 1024
            self.ws = backend.device.empty((nbytes,), np.uint8)
            A.workspace, A.workspace_bytes = self.ws.ptr, self.ws.nbytes
        self.c = A

    def parameters(self):
        parts = [self.actor.params.numpy()] + [c.params.numpy() for c in self.critics] + [t.params.numpy() for t in self.targets]
        return np.concatenate(parts + [self.log_alpha.numpy()[:1]])

    def set_batch(self, oab, rewards, terminated):
        self.oab.upload(oab); self.rewards.upload(rewards); self.terminated.upload(terminated)


def rel_err(a, ref):
    """max |a - ref| relative to the largest magnitude of the reference tensor (per-tensor scale)."""
    a = np.asarray(a, np.float64); ref = np.asarray(ref, np.float64)
    scale = max(np.abs(ref).max(), 1e-30)
    return np.abs(a - ref).max() / scale


def np_from(ptr, shape, dtype=np.float32):
    n = int(np.prod(shape))
    return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(np.ctypeslib.as_ctypes_type(dtype))), (n,)).reshape(shape).copy()


class Td3OnBackend:
    """All TD3 state for the Pendulum shapes (observation 3, action 1) on one backend. `params` is the flat vector
    [actor, actor_target, critic 0, critic 1, critic target 0, critic target 1], each [W|b] per layer."""

    def __init__(self, backend, batch, hidden, params, hyper=None, masks=False, obs=3, act=1, hidden_act="relu"):
        OBS, ACT, D = obs, act, obs + act
        self.backend, self.batch, self.OBS, self.ACT = backend, batch, OBS, ACT
        adims, cdims = [OBS, hidden, hidden, ACT], [D, hidden, hidden, 1]
        na, nc = mlp_param_count(adims), mlp_param_count(cdims)
        assert params.size == 2 * na + 4 * nc
        o = 0
        self.actor = Mlp(backend, adims, params[o:o + na], batch, hidden_act, out_act="tanh"); o += na
        self.actor_target = Mlp(backend, adims, params[o:o + na], batch, hidden_act, out_act="tanh", trainable=False); o += na
        self.critics = []
        for _ in range(2):
            self.critics.append(Mlp(backend, cdims, params[o:o + nc], batch, hidden_act)); o += nc
        self.targets = []
        for _ in range(2):
            self.targets.append(Mlp(backend, cdims, params[o:o + nc], batch, hidden_act, trainable=False)); o += nc
        z = backend.zeros
        self.oab = z((2, batch, D)); self.rewards = z((batch,)); self.terminated = z((batch,), np.uint8)
        self.m_final = backend.array(np.ones(batch, np.uint8)); self.m_next_final = backend.array(np.ones(batch, np.uint8))
        self.target_noise = z((batch, ACT)); self.nsavi = z((batch, D)); self.next_q = [z((batch,)), z((batch,))]; self.target_q = z((batch,))
        self.d_out_c = z((batch,)); self.savi = z((batch, D)); self.pre_clip = z((batch, ACT)); self.d_out_a = z((batch,))
        self.d_ci = z((batch, D)); self.d_ao = z((batch, ACT))
        h = hyper if hyper is not None else dict(gamma=0.99, actor_polyak=float(np.float32(1.0 - 0.005)), critic_polyak=float(np.float32(1.0 - 0.005)),
                                                 sampling_std=0.1, adam=capi.adam_parameters(epsilon=1e-7))
        A = capi.Td3Agent()
        A.batch, A.observation_dim, A.action_dim, A.n_actor_layers, A.n_critic_layers, A.ignore_termination = batch, OBS, ACT, 3, 3, 0
        A.gamma, A.actor_polyak, A.critic_polyak, A.sampling_std = h["gamma"], h["actor_polyak"], h["critic_polyak"], h["sampling_std"]
        A.actor_adam = A.critic_adam = h["adam"]
        A.actor, A.actor_target = self.actor.layers, self.actor_target.layers
        A.actor_adam_tensors, A.n_actor_adam_tensors, A.actor_age = self.actor.adam, self.actor.n_adam, self.actor.age.ptr
        for k in range(2):
            A.critics[k] = self.critics[k].layers; A.critics_target[k] = self.targets[k].layers
            A.critic_adam_tensors[k] = self.critics[k].adam; A.critic_age[k] = self.critics[k].age.ptr
            A.next_q[k] = self.next_q[k].ptr
        A.n_critic_adam_tensors = self.critics[0].n_adam
        A.observations_actions_base, A.rewards, A.terminated = self.oab.ptr, self.rewards.ptr, self.terminated.ptr
        if masks:
            A.final_step_mask, A.next_final_step_mask = self.m_final.ptr, self.m_next_final.ptr
        A.target_next_action_noise, A.next_state_action_value_input, A.target_action_value = self.target_noise.ptr, self.nsavi.ptr, self.target_q.ptr
        A.d_output_critic, A.state_action_value_input, A.actor_pre_clip = self.d_out_c.ptr, self.savi.ptr, self.pre_clip.ptr
        A.d_output_actor, A.d_critic_input, A.d_actor_output = self.d_out_a.ptr, self.d_ci.ptr, self.d_ao.ptr
        if backend.name == "rocm":
            lib = backend.device.lib
            nbytes = max(lib.rlt_rocm_mlp_workspace_bytes(self.actor.layers, 3, batch), lib.rlt_rocm_mlp_workspace_bytes(self.critics[0].layers, 3, batch))
            nbytes += batch * ACT * 4 + 1024
            self.ws = backend.device.empty((nbytes,), np.uint8)
            A.workspace, A.workspace_bytes = self.ws.ptr, self.ws.nbytes
        else:
            self.ws = backend.zeros((64,), np.uint8)
            A.workspace, A.workspace_bytes = self.ws.ptr, 64
        self.c = A

    def parameters(self):
        nets = [self.actor, self.actor_target] + self.critics + self.targets
        return np.concatenate([n.params.numpy() for n in nets])

    def ages(self):
        return np.array([self.actor.age.numpy()[0], self.critics[0].age.numpy()[0], self.critics[1].age.numpy()[0]], np.uint32)

    def state(self):
        """Everything an update reads and writes: parameters of all six networks, Adam moments and ages of the three trained ones."""
        nets = [self.actor] + self.critics
        return dict(params=[n.params.numpy() for n in [self.actor, self.actor_target] + self.critics + self.targets],
                    m=[n.m.numpy() for n in nets], v=[n.v.numpy() for n in nets], age=[n.age.numpy() for n in nets])

    def push(self, st):
        nets = [self.actor] + self.critics
        for n, p in zip([self.actor, self.actor_target] + self.critics + self.targets, st["params"]):
            n.params.upload(p)
        for n, m, v, a in zip(nets, st["m"], st["v"], st["age"]):
            n.m.upload(m); n.v.upload(v); n.age.upload(a)

    def gradients(self):
        return np.concatenate([n.grads.numpy() for n in [self.actor] + self.critics])

    def set_batch(self, oab, rewards, terminated, target_noise):
        self.oab.upload(oab); self.rewards.upload(rewards); self.terminated.upload(terminated); self.target_noise.upload(target_noise)

    def loop_step(self, flags, noise_c0, noise_c1, noise_a, both_critics_in_one_call=False):
        """The training half of td3::loop::core::step (rl/algorithms/td3/loop/core/operations_generic.h:98-133) on the batch set before."""
        b = self.backend
        if flags[0] and both_critics_in_one_call:
            n0, n1 = b.array(noise_c0.astype(np.float32)), b.array(noise_c1.astype(np.float32))
            b.call("td3_train_critics", C.byref(self.c), n0.ptr, n1.ptr)
            b.sync()
        elif flags[0]:
            for k, nz in enumerate((noise_c0, noise_c1)):
                n = b.array(nz.astype(np.float32))
                b.call("td3_train_critic", C.byref(self.c), k, n.ptr)
                b.sync()
        if flags[1]:
            b.call("td3_update_critic_targets", C.byref(self.c))
        if flags[2]:
            n = b.array(noise_a.astype(np.float32))
            b.call("td3_train_actor", C.byref(self.c), n.ptr)
            b.sync()
        if flags[3]:
            b.call("td3_update_actor_target", C.byref(self.c))
        b.sync()


class OnPolicyOnBackend:
    """Pendulum on-policy runner state and one dataset (all columns in one [rows + n_envs, ld] array, the reference's layout) on a backend."""

    def __init__(self, backend, n_envs, steps, ld, col, limit, runner_state=None):
        self.backend, self.n, self.steps, self.ld, self.col = backend, n_envs, steps, ld, col
        rs = runner_state or dict(states=np.zeros((n_envs, 2), np.float32), episode_step=np.zeros(n_envs, np.uint32), episode_return=np.zeros(n_envs, np.float32),
                                  truncated=np.ones(n_envs, np.uint8))
        self.states, self.ep_step, self.ep_ret, self.trunc = (backend.array(rs[k]) for k in ("states", "episode_step", "episode_return", "truncated"))
        self.c = capi.PendulumRunner(self.states.ptr, self.ep_step.ptr, self.ep_ret.ptr, self.trunc.ptr, n_envs, limit, capi.pendulum_parameters())
        self.data = backend.zeros(((steps + 1) * n_envs, ld))
        o = self.data.offset
        self.d = capi.OnPolicyDataset(o(col["observations"]), o(col["actions_mean"]), o(col["actions"]), o(col["action_log_probs"]), o(col["rewards"]), o(col["terminated"]),
                                      o(col["truncated"]), o(col["all_reset"]), ld, steps)

    def runner_state(self):
        return dict(states=self.states.numpy(), episode_step=self.ep_step.numpy(), episode_return=self.ep_ret.numpy(), truncated=self.trunc.numpy())

    def load_runner(self, rs):
        self.states.upload(rs["states"]); self.ep_step.upload(rs["episode_step"]); self.ep_ret.upload(rs["episode_return"]); self.trunc.upload(rs["truncated"])

    def collect(self, actor, log_std, noise, initial_states, standardize=None, truncate_on_each_iteration=0):
        b = self.backend
        ls, nz, ini = b.array(log_std), b.array(noise), b.array(initial_states)
        sm = b.array(standardize[0]) if standardize else None; sp = b.array(standardize[1]) if standardize else None
        ws, wsn = (None, 0)
        if b.name == "rocm":
            wsn = b.device.lib.rlt_rocm_on_policy_collect_workspace_bytes(C.byref(self.c), actor.layers, actor.n)
            ws, wsn = b.workspace(wsn)
        b.call("on_policy_collect", C.byref(self.c), C.byref(self.d), actor.layers, actor.n, ls.ptr, sm.ptr if sm else None, sp.ptr if sp else None, nz.ptr, ini.ptr,
               truncate_on_each_iteration, ws, wsn)
        b.sync()


SEQUENCE_BATCH_FIELDS = ("observations_actions_base", "rewards", "terminated", "reset", "next_reset_base", "final_step_mask", "next_final_step_mask_base")


class SequenceBatchOnBackend:
    """A SequentialBatch on a backend, pre-filled the way the reference harness fills its own before gather_batch (what the gather does not write
    stays: -777 in the float tensors, 0 in the flags)."""

    def __init__(self, backend, batch, sequence_length, data_dim):
        S, PS = sequence_length, sequence_length + 1
        self.backend = backend
        self.arrays = dict(observations_actions_base=backend.array(np.full((PS, batch, data_dim), -777.0, np.float32)), rewards=backend.array(np.full((S, batch), -777.0, np.float32)),
                           terminated=backend.zeros((S, batch), np.uint8), reset=backend.zeros((S, batch), np.uint8), next_reset_base=backend.zeros((PS, batch), np.uint8),
                           final_step_mask=backend.zeros((S, batch), np.uint8), next_final_step_mask_base=backend.zeros((PS, batch), np.uint8))
        self.c = capi.SequenceBatch(*[self.arrays[k].ptr for k in SEQUENCE_BATCH_FIELDS], batch, sequence_length)

    def numpy(self):
        return {k: v.numpy() for k, v in self.arrays.items()}


def seq_param_count(specs):
    """specs: list of (kind, in, out, activation name); dense [W | b], GRU [W_i | b_i | W_h | b_h | h0]."""
    return sum((i * o + o) if kind == 0 else (3 * o * i + 3 * o + 3 * o * o + 3 * o + o) for kind, i, o, _ in specs)


def random_seq_params(rng, specs):
    parts = []
    for kind, i, o, _ in specs:
        if kind == 0:
            parts += [rng.uniform(-1, 1, o * i) / np.sqrt(i), rng.uniform(-0.1, 0.1, o)]
        else:
            parts += [rng.uniform(-1, 1, 3 * o * i) / np.sqrt(i), rng.uniform(-0.1, 0.1, 3 * o), rng.uniform(-1, 1, 3 * o * o) / np.sqrt(o), rng.uniform(-0.1, 0.1, 3 * o), np.zeros(o)]
    return np.concatenate(parts).astype(np.float32)


class SeqNet:
    """A sequential model of dense and GRU layers on a backend: flat arenas (parameters, gradients, Adam moments), kept intermediates for `steps`
    x `batch` rows, described to the C ABI by an array of rlt_seq_layer."""

    def __init__(self, backend, specs, params, steps, batch, trainable=True, fast_tanh=True):
        self.backend, self.specs, self.steps, self.batch, self.n = backend, list(specs), steps, batch, len(specs)
        total = seq_param_count(specs)
        assert params.size == total, (params.size, total)
        self.params = backend.array(params.astype(np.float32))
        self.grads, self.m, self.v = (backend.zeros((total,)) for _ in range(3)) if trainable else (None, None, None)
        self.age = backend.array(np.array([1], np.uint32))
        self.layers = (capi.SeqLayer * self.n)()
        self.keep, adam, off = [], [], 0
        z = backend.zeros
        g = lambda o: self.grads.offset(o) if trainable else None
        def tensor(o, n, flags):
            if trainable:
                adam.append(capi.AdamTensor(self.params.offset(o), self.grads.offset(o), self.m.offset(o), self.v.offset(o), None, n, flags))
        for l, (kind, i, o, act) in enumerate(specs):
            L = self.layers[l]
            L.kind = kind
            if kind == 0:
                pre, out = z((steps * batch, o)), z((steps * batch, o))
                self.keep.append((pre, out))
                L.dense = capi.DenseLayer(self.params.offset(off), self.params.offset(off + i * o), g(off), g(off + i * o), pre.ptr, out.ptr, i, o, capi.ACT[act], 0)
                tensor(off, i * o, 1); tensor(off + i * o, o, 2)
                off += i * o + o
            else:
                post, npp, out = z((steps, batch, 3 * o)), z((steps, batch, o)), z((steps, batch, o))
                self.keep.append((post, npp, out))
                o_wi, o_bi, o_wh, o_bh, o_h0 = off, off + 3 * o * i, off + 3 * o * i + 3 * o, off + 3 * o * i + 3 * o + 3 * o * o, off + 3 * o * i + 3 * o + 3 * o * o + 3 * o
                L.gru = capi.GruLayer(self.params.offset(o_wi), self.params.offset(o_bi), self.params.offset(o_wh), self.params.offset(o_bh), self.params.offset(o_h0),
                                      g(o_wi), g(o_bi), g(o_wh), g(o_bh), post.ptr, npp.ptr, out.ptr, i, o, int(fast_tanh), 0)
                for oo, n, fl in ((o_wi, 3 * o * i, 1), (o_bi, 3 * o, 2), (o_wh, 3 * o * o, 1), (o_bh, 3 * o, 2), (o_h0, o, 2)):
                    tensor(oo, n, fl)
                off = o_h0 + o
        self.adam = (capi.AdamTensor * max(len(adam), 1))(*adam)
        self.n_adam = len(adam)

    def output(self):
        return self.keep[-1][-1].numpy()

    def workspace(self):
        if self.backend.name != "rocm":
            return None, 0
        return self.backend.workspace(self.backend.device.lib.rlt_rocm_seq_workspace_bytes(self.layers, self.n, self.steps, self.batch))


class SeqStateOnBackend:
    """The rollout state of a sequential model's GRU layers (hidden state and step counter per batch row) on a backend."""

    def __init__(self, backend, specs, batch):
        self.backend, self.specs, self.batch = backend, list(specs), batch
        self.hidden, self.step = {}, {}
        self.c = capi.SeqState()
        for l, (kind, _, o, _) in enumerate(specs):
            if kind == 1:
                self.hidden[l], self.step[l] = backend.zeros((batch, o)), backend.zeros((batch,), np.uint32)
                self.c.hidden[l], self.c.step[l] = self.hidden[l].ptr, self.step[l].ptr

    def set(self, hidden, steps):
        """hidden: list of [batch x H] per GRU layer, steps: list of [batch], in layer order."""
        for k, l in enumerate(sorted(self.hidden)):
            self.hidden[l].upload(hidden[k]); self.step[l].upload(np.asarray(steps[k], np.uint32))

    def numpy(self):
        ls = sorted(self.hidden)
        return [self.hidden[l].numpy() for l in ls], [self.step[l].numpy() for l in ls]


class RecurrentRunnerOnBackend:
    """Pendulum off-policy runner (n environments, one replay ring each) with a sequential policy and its rollout state on a backend."""

    def __init__(self, backend, specs, params, n_envs, capacity, episode_limit, auto_reset_period):
        self.backend, self.n, self.period = backend, n_envs, auto_reset_period
        self.policy = SeqNet(backend, specs, params, 1, n_envs, trainable=False)
        self.state = SeqStateOnBackend(backend, specs, n_envs)
        self.rb = ReplayOnBackend(backend, n_envs, capacity)
        self.states, self.ep_step, self.ep_ret = backend.zeros((n_envs, 2)), backend.zeros((n_envs,), np.uint32), backend.zeros((n_envs,))
        self.trunc = backend.array(np.ones(n_envs, np.uint8))
        self.c = capi.PendulumRunner(self.states.ptr, self.ep_step.ptr, self.ep_ret.ptr, self.trunc.ptr, n_envs, episode_limit, capi.pendulum_parameters())
        self.sas = capi.SasParameters(-20.0, 2.0, 1e-6, -1.0)
        self.ws, self.wsn = (None, 0)
        if backend.name == "rocm":
            n = int(backend.device.lib.rlt_rocm_pendulum_runner_step_recurrent_workspace_bytes(self.policy.layers, self.policy.n, n_envs))
            self._ws = backend.device.empty((n,), np.uint8)
            self.ws, self.wsn = self._ws.ptr, n

    def load(self, runner, rings):
        """runner: dict states / episode_step / episode_return / truncated / hidden / steps; rings: list of (data, position, full, current_episode_start, episode_start)."""
        self.states.upload(runner["states"]); self.ep_step.upload(runner["episode_step"]); self.ep_ret.upload(runner["episode_return"]); self.trunc.upload(runner["truncated"])
        self.state.set(runner["hidden"], runner["steps"])
        self.rb.data.upload(np.concatenate([r[0] for r in rings])); self.rb.position.upload(np.array([r[1] for r in rings], np.uint32))
        self.rb.full.upload(np.array([r[2] for r in rings], np.uint8)); self.rb.current_episode_start.upload(np.array([r[3] for r in rings], np.uint32))
        self.rb.episode_start.upload(np.concatenate([r[4] for r in rings]).astype(np.uint32))

    def step(self, action_noise, initial_states):
        be = self.backend
        nz, ini = be.array(np.ascontiguousarray(action_noise, np.float32)), be.array(np.ascontiguousarray(initial_states, np.float32))
        be.call("pendulum_runner_step_recurrent", C.byref(self.c), C.byref(self.rb.c), self.policy.layers, self.policy.n, C.byref(self.state.c), self.period, C.byref(self.sas),
                nz.ptr, ini.ptr, self.ws, self.wsn)
        be.sync()

    def numpy(self):
        hidden, steps = self.state.numpy()
        return dict(states=self.states.numpy(), episode_step=self.ep_step.numpy(), episode_return=self.ep_ret.numpy(), truncated=self.trunc.numpy(), hidden=hidden, steps=steps,
                    data=self.rb.data.numpy(), position=self.rb.position.numpy(), full=self.rb.full.numpy(), current_episode_start=self.rb.current_episode_start.numpy(),
                    episode_start=self.rb.episode_start.numpy())


class SacSequenceOnBackend:
    """All state of a SAC agent with sequential (recurrent) networks on one backend. params: flat [actor, critic 0, critic 1, target 0, target 1,
    log_alpha] with every network laid out layer after layer (the order the reference harness exports)."""

    def __init__(self, backend, actor_specs, critic_specs, params, S, B, obs_dim, act_dim, include_first=True, hyper=None):
        self.backend, self.S, self.B = backend, S, B
        T, D = S + (1 if include_first else 0), obs_dim + act_dim
        self.T = T
        na, nc = seq_param_count(actor_specs), seq_param_count(critic_specs)
        o = 0
        self.actor = SeqNet(backend, actor_specs, params[o:o + na], T, B); o += na
        self.critics = [SeqNet(backend, critic_specs, params[o + k * nc:o + (k + 1) * nc], S, B) for k in range(2)]; o += 2 * nc
        self.targets = [SeqNet(backend, critic_specs, params[o + k * nc:o + (k + 1) * nc], T, B, trainable=False) for k in range(2)]; o += 2 * nc
        self.log_alpha = backend.array(np.array([params[o], 0, 0, 0], np.float32))
        self.alpha_age = backend.array(np.array([1], np.uint32))
        self.batch = SequenceBatchOnBackend(backend, B, S, D)
        z = backend.zeros
        self.buf = dict(nsavi=z((T, B, D)), next_q0=z((T, B)), next_q1=z((T, B)), next_lp=z((T, B)), target=z((S, B)), d_output=z((S, B)), savi=z((S, B, D)),
                        d_ci0=z((S, B, D)), d_ci1=z((S, B, D)), d_aos=z((S, B, act_dim)), d_ao=z((S, B, 2 * act_dim)), a_act=z((T, B, act_dim)), a_pre=z((S, B, act_dim)), a_lp=z((S, B)))
        A = capi.SacSequenceAgent()
        A.observation_dim, A.action_dim, A.n_actor_layers, A.n_critic_layers, A.include_first_step_in_targets = obs_dim, act_dim, len(actor_specs), len(critic_specs), int(include_first)
        hyper = hyper or {}
        A.gamma, A.polyak = hyper.get("gamma", 0.99), hyper.get("polyak", float(np.float32(1.0 - 0.005)))
        A.sas = hyper.get("sas", capi.SasParameters(-20.0, 2.0, 1e-6, -float(act_dim)))
        A.actor_adam, A.critic_adam, A.alpha_adam = (hyper.get(k, capi.adam_parameters()) for k in ("actor_adam", "critic_adam", "alpha_adam"))
        A.actor, A.actor_adam_tensors, A.n_actor_adam_tensors, A.actor_age = self.actor.layers, self.actor.adam, self.actor.n_adam, self.actor.age.ptr
        b = self.buf
        for k in range(2):
            A.critics[k], A.critics_target[k] = self.critics[k].layers, self.targets[k].layers
            A.critic_adam_tensors[k], A.critic_age[k] = self.critics[k].adam, self.critics[k].age.ptr
            A.next_q[k], A.d_critic_input[k] = b[f"next_q{k}"].ptr, b[f"d_ci{k}"].ptr
        A.n_critic_adam_tensors = self.critics[0].n_adam
        la = self.log_alpha
        A.log_alpha = capi.AdamTensor(la.offset(0), la.offset(1), la.offset(2), la.offset(3), None, 1, 0)
        A.alpha_age = self.alpha_age.ptr
        A.batch = self.batch.c
        A.next_state_action_value_input, A.next_log_probabilities, A.target_action_value, A.d_output = b["nsavi"].ptr, b["next_lp"].ptr, b["target"].ptr, b["d_output"].ptr
        A.state_action_value_input, A.d_actor_output_squashing, A.d_actor_output = b["savi"].ptr, b["d_aos"].ptr, b["d_ao"].ptr
        A.actor_actions, A.actor_pre_squashing, A.actor_log_probabilities = b["a_act"].ptr, b["a_pre"].ptr, b["a_lp"].ptr
        if backend.name == "rocm":
            n = int(backend.device.lib.rlt_rocm_sac_sequence_workspace_bytes(C.byref(A)))
            self.ws = backend.device.empty((max(n, 4),), np.uint8)
            A.workspace, A.workspace_bytes = self.ws.ptr, n
        self.c = A

    def set_batch(self, data):
        for k in SEQUENCE_BATCH_FIELDS:
            self.batch.arrays[k].upload(data[k])

    def train(self, noise_critic, noise_actor, both_critics_in_one_call=False):
        """The training part of one loop step with a shared batch (rl/algorithms/sac/loop/core/operations_generic.h:127-154)."""
        be = self.backend
        nc, na = be.array(np.ascontiguousarray(noise_critic, np.float32)), be.array(np.ascontiguousarray(noise_actor, np.float32))
        if both_critics_in_one_call:
            be.call("sac_sequence_train_critics", C.byref(self.c), nc.ptr)
        for k in range(0 if both_critics_in_one_call else 2):
            be.call("sac_sequence_train_critic", C.byref(self.c), k, nc.ptr)
        be.call("sac_sequence_update_critic_targets", C.byref(self.c))
        be.call("sac_sequence_train_actor", C.byref(self.c), na.ptr)
        be.sync()

    def parameters(self):
        parts = [self.actor.params.numpy()] + [c.params.numpy() for c in self.critics] + [t.params.numpy() for t in self.targets]
        return np.concatenate(parts + [self.log_alpha.numpy()[:1]])

    def ages(self):
        return [int(x.numpy()[0]) for x in (self.actor.age, self.critics[0].age, self.critics[1].age, self.alpha_age)]


class Td3SequenceOnBackend:
    """All state of a TD3 agent with sequential (recurrent) networks on one backend. params: flat [actor, critic 0, critic 1, actor target, critic target 0,
    critic target 1] with every network laid out layer after layer (the order the reference harness exports)."""

    def __init__(self, backend, actor_specs, critic_specs, params, S, B, obs_dim, act_dim, include_first=True, hyper=None):
        self.backend, self.S, self.B = backend, S, B
        T, D = S + (1 if include_first else 0), obs_dim + act_dim
        self.T = T
        na, nc = seq_param_count(actor_specs), seq_param_count(critic_specs)
        o = 0
        self.actor = SeqNet(backend, actor_specs, params[o:o + na], S, B); o += na
        self.critics = [SeqNet(backend, critic_specs, params[o + k * nc:o + (k + 1) * nc], S, B) for k in range(2)]; o += 2 * nc
        self.actor_target = SeqNet(backend, actor_specs, params[o:o + na], T, B, trainable=False); o += na
        self.targets = [SeqNet(backend, critic_specs, params[o + k * nc:o + (k + 1) * nc], T, B, trainable=False) for k in range(2)]; o += 2 * nc
        self.batch = SequenceBatchOnBackend(backend, B, S, D)
        z = backend.zeros
        self.buf = dict(noise=z((T, B, act_dim)), nsavi=z((T, B, D)), next_q0=z((T, B)), next_q1=z((T, B)), target=z((S, B)), d_output=z((S, B)), savi=z((S, B, D)),
                        d_ci=z((S, B, D)), d_ao=z((S, B, act_dim)), a_in=z((T, B, obs_dim)))
        A = capi.Td3SequenceAgent()
        A.observation_dim, A.action_dim, A.n_actor_layers, A.n_critic_layers, A.include_first_step_in_targets = obs_dim, act_dim, len(actor_specs), len(critic_specs), int(include_first)
        hyper = hyper or {}
        polyak = float(np.float32(1.0 - 0.005))
        A.gamma, A.actor_polyak, A.critic_polyak = hyper.get("gamma", 0.99), hyper.get("actor_polyak", polyak), hyper.get("critic_polyak", polyak)
        A.ignore_termination = int(hyper.get("ignore_termination", 0))
        A.actor_adam, A.critic_adam = (hyper.get(k, capi.adam_parameters()) for k in ("actor_adam", "critic_adam"))
        A.actor, A.actor_target, A.actor_adam_tensors, A.n_actor_adam_tensors, A.actor_age = self.actor.layers, self.actor_target.layers, self.actor.adam, self.actor.n_adam, self.actor.age.ptr
        b = self.buf
        for k in range(2):
            A.critics[k], A.critics_target[k] = self.critics[k].layers, self.targets[k].layers
            A.critic_adam_tensors[k], A.critic_age[k] = self.critics[k].adam, self.critics[k].age.ptr
            A.next_q[k] = b[f"next_q{k}"].ptr
        A.n_critic_adam_tensors = self.critics[0].n_adam
        A.batch = self.batch.c
        A.target_next_action_noise, A.next_state_action_value_input, A.target_action_value, A.d_output = b["noise"].ptr, b["nsavi"].ptr, b["target"].ptr, b["d_output"].ptr
        A.state_action_value_input, A.d_critic_input, A.d_actor_output, A.actor_input = b["savi"].ptr, b["d_ci"].ptr, b["d_ao"].ptr, b["a_in"].ptr
        if backend.name == "rocm":
            n = int(backend.device.lib.rlt_rocm_td3_sequence_workspace_bytes(C.byref(A)))
            self.ws = backend.device.empty((max(n, 4),), np.uint8)
            A.workspace, A.workspace_bytes = self.ws.ptr, n
        self.c = A

    def set_batch(self, data):
        for k in SEQUENCE_BATCH_FIELDS:
            self.batch.arrays[k].upload(data[k])

    def train(self, noise, flags=(1, 1, 1, 1), both_critics_in_one_call=False):
        """The training part of one loop step with a shared batch (rl/algorithms/td3/loop/core/operations_generic.h:91-127); noise: the clamped target-action
        noise [T x B x act]; flags: (train critics, update critic targets, train actor, update actor target)."""
        be = self.backend
        self.buf["noise"].upload(np.ascontiguousarray(noise, np.float32).reshape(self.buf["noise"].shape))
        if flags[0] and both_critics_in_one_call:
            be.call("td3_sequence_train_critics", C.byref(self.c))
        elif flags[0]:
            for k in range(2):
                be.call("td3_sequence_train_critic", C.byref(self.c), k)
        if flags[1]:
            be.call("td3_sequence_update_critic_targets", C.byref(self.c))
        if flags[2]:
            be.call("td3_sequence_train_actor", C.byref(self.c))
        if flags[3]:
            be.call("td3_sequence_update_actor_target", C.byref(self.c))
        be.sync()

    def parameters(self):
        return np.concatenate([self.actor.params.numpy()] + [c.params.numpy() for c in self.critics] + [self.actor_target.params.numpy()] + [t.params.numpy() for t in self.targets])

    def ages(self):
        return [int(x.numpy()[0]) for x in (self.actor.age, self.critics[0].age, self.critics[1].age)]
