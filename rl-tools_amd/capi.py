"""ctypes binding of include/rlt_rocm.h: structure mirrors, prototypes and a thin device-array helper.

This is plumbing for tests, the smoke check and the benchmark; the product is the shared library itself.
The HIP library must exist (built by build.py): loading fails loudly otherwise, there is no CPU fallback.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "librlt_rocm.so")

c_float_p = C.POINTER(C.c_float)
c_u8_p = C.POINTER(C.c_uint8)
c_u32_p = C.POINTER(C.c_uint32)

ACT = {"identity": 0, "relu": 1, "gelu": 2, "tanh": 3, "fast_tanh": 4, "sigmoid": 5}


class DenseLayer(C.Structure):
    _fields_ = [("weights", C.c_void_p), ("biases", C.c_void_p), ("d_weights", C.c_void_p), ("d_biases", C.c_void_p),
                ("pre_activations", C.c_void_p), ("output", C.c_void_p),
                ("in_dim", C.c_int32), ("out_dim", C.c_int32), ("activation", C.c_int32), ("reserved", C.c_int32)]


class AdamParameters(C.Structure):
    _fields_ = [("alpha", C.c_float), ("beta_1", C.c_float), ("beta_2", C.c_float), ("epsilon", C.c_float), ("epsilon_sqrt", C.c_float),
                ("weight_decay", C.c_float), ("bias_lr_factor", C.c_float), ("enable_weight_decay", C.c_int32),
                ("enable_bias_lr_factor", C.c_int32), ("enable_gradient_clipping", C.c_int32), ("gradient_clip_value", C.c_float)]


def adam_parameters(alpha=1e-3, beta_1=0.9, beta_2=0.999, epsilon=1e-7, epsilon_sqrt=None):
    return AdamParameters(alpha, beta_1, beta_2, epsilon, epsilon if epsilon_sqrt is None else epsilon_sqrt, 0.0, 1.0, 0, 0, 0, 1.0)


class AdamTensor(C.Structure):
    _fields_ = [("parameters", C.c_void_p), ("gradient", C.c_void_p), ("first_moment", C.c_void_p), ("second_moment", C.c_void_p),
                ("polyak_target", C.c_void_p), ("count", C.c_uint32), ("flags", C.c_uint32)]


class SasParameters(C.Structure):
    _fields_ = [("log_std_lower_bound", C.c_float), ("log_std_upper_bound", C.c_float), ("log_probability_epsilon", C.c_float),
                ("target_entropy", C.c_float)]


class SacAgent(C.Structure):
    _fields_ = [("batch", C.c_int32), ("observation_dim", C.c_int32), ("action_dim", C.c_int32), ("n_actor_layers", C.c_int32),
                ("n_critic_layers", C.c_int32), ("gamma", C.c_float), ("polyak", C.c_float), ("reserved0", C.c_float),
                ("sas", SasParameters), ("actor_adam", AdamParameters), ("critic_adam", AdamParameters), ("alpha_adam", AdamParameters),
                ("actor", C.POINTER(DenseLayer)), ("critics", C.POINTER(DenseLayer) * 2), ("critics_target", C.POINTER(DenseLayer) * 2),
                ("actor_adam_tensors", C.POINTER(AdamTensor)), ("n_actor_adam_tensors", C.c_int32), ("pad0", C.c_int32),
                ("critic_adam_tensors", C.POINTER(AdamTensor) * 2), ("n_critic_adam_tensors", C.c_int32), ("pad1", C.c_int32),
                ("log_alpha", AdamTensor),
                ("actor_age", C.c_void_p), ("critic_age", C.c_void_p * 2), ("alpha_age", C.c_void_p),
                ("observations_actions_base", C.c_void_p), ("rewards", C.c_void_p), ("terminated", C.c_void_p),
                ("final_step_mask", C.c_void_p), ("next_final_step_mask", C.c_void_p), ("reset", C.c_void_p),
                ("next_state_action_value_input", C.c_void_p), ("next_q", C.c_void_p * 2), ("next_log_probabilities", C.c_void_p),
                ("target_action_value", C.c_void_p), ("d_output_critic", C.c_void_p * 2), ("state_action_value_input", C.c_void_p),
                ("d_output_actor_critics", C.c_void_p), ("d_critic_input", C.c_void_p * 2), ("d_actor_output_squashing", C.c_void_p),
                ("d_actor_output", C.c_void_p), ("actor_pre_squashing", C.c_void_p), ("actor_log_probabilities", C.c_void_p),
                ("actor_actions", C.c_void_p), ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t)]


class ReplayBuffer(C.Structure):
    _fields_ = [("data", C.c_void_p), ("episode_start", C.c_void_p), ("position", C.c_void_p), ("current_episode_start", C.c_void_p),
                ("full", C.c_void_p), ("n_envs", C.c_int32), ("capacity", C.c_int32), ("observation_dim", C.c_int32), ("action_dim", C.c_int32)]


class SequenceBatch(C.Structure):
    _fields_ = [("observations_actions_base", C.c_void_p), ("rewards", C.c_void_p), ("terminated", C.c_void_p), ("reset", C.c_void_p), ("next_reset_base", C.c_void_p),
                ("final_step_mask", C.c_void_p), ("next_final_step_mask_base", C.c_void_p), ("batch", C.c_int32), ("sequence_length", C.c_int32)]


class SequenceSampling(C.Structure):
    _fields_ = [("always_sample_from_initial_state", C.c_int32), ("random_seq_length", C.c_int32), ("enable_nominal_sequence_length_probability", C.c_int32),
                ("nominal_sequence_length_probability", C.c_float), ("include_first_step_in_targets", C.c_int32)]


class SequenceDraws(C.Structure):
    _fields_ = [("env_indices", C.c_void_p), ("sample_offsets", C.c_void_p), ("nominal", C.c_void_p), ("lengths", C.c_void_p)]


class PendulumParameters(C.Structure):
    _fields_ = [("g", C.c_float), ("max_speed", C.c_float), ("max_torque", C.c_float), ("dt", C.c_float), ("m", C.c_float), ("l", C.c_float)]


def pendulum_parameters():
    return PendulumParameters(10.0, 8.0, 2.0, 0.05, 1.0, 1.0)


class AcrobotParameters(C.Structure):
    _fields_ = [(name, C.c_float) for name in ("dt", "link_length_1", "link_length_2", "link_mass_1", "link_mass_2", "link_com_pos_1", "link_com_pos_2", "link_moi",
                                               "max_vel_1", "max_vel_2", "min_torque", "max_torque")]


def acrobot_parameters(easy=False):
    """rl/environments/acrobot/acrobot.h:14-37 DefaultParameters (EasyParameters: torque range +-10)"""
    import math
    t = 10.0 if easy else 5.0
    pi = C.c_float(math.pi).value
    return AcrobotParameters(0.2, 1.0, 1.0, 1.0, 1.0, 0.5, 0.5, 1.0, 4 * pi, 9 * pi, -t, t)


class CarParameters(C.Structure):
    _fields_ = [(name, C.c_float) for name in ("g", "m", "I", "lf", "lr", "tf_B", "tf_C", "tf_D", "tr_B", "tr_C", "tr_D", "cm", "cr0", "cr2", "vt", "dt")]


def car_parameters():
    """rl/environments/car/car.h:19-33"""
    return CarParameters(9.81, 0.041, 27.8e-6, 0.029, 0.033, 2.5790, 1.2000, 0.1920, 3.3852, 1.2691, 0.1737, 0.287, 0.0, 0.00035, 0.01, 0.01)


class PendulumRunner(C.Structure):
    _fields_ = [("states", C.c_void_p), ("episode_step", C.c_void_p), ("episode_return", C.c_void_p), ("truncated", C.c_void_p),
                ("n_envs", C.c_int32), ("episode_step_limit", C.c_int32), ("env", PendulumParameters)]


UNARY = dict(negate=0, abs=1, constant=2, sigmoid=3, fast_sigmoid=4, exp=5, tanh=6, fast_tanh=7, one_minus=8, scale=9, scale_reciprocal=10)
BINARY = dict(add=0, subtract=1, multiply=2, divide=3)
ENV_PENDULUM, ENV_ACROBOT, ENV_ACROBOT_SWINGUP, ENV_CAR, ENV_PENDULUM_POSITION = 0, 1, 2, 3, 4
ENV_DIMS = {ENV_PENDULUM: (2, 3, 1), ENV_ACROBOT: (4, 6, 1), ENV_ACROBOT_SWINGUP: (4, 6, 1), ENV_CAR: (6, 6, 2), ENV_PENDULUM_POSITION: (3, 2, 1)}      # state, observation, action widths


class EnvRunner(C.Structure):
    _fields_ = [("env_kind", C.c_int32), ("n_envs", C.c_int32), ("episode_step_limit", C.c_int32), ("reserved", C.c_int32),
                ("states", C.c_void_p), ("episode_step", C.c_void_p), ("episode_return", C.c_void_p), ("truncated", C.c_void_p),
                ("pendulum", PendulumParameters), ("acrobot", AcrobotParameters), ("car", CarParameters),
                ("observations", C.c_void_p), ("actions", C.c_void_p), ("next_observations", C.c_void_p), ("rewards", C.c_void_p), ("terminated", C.c_void_p)]


class SacLoopInputs(C.Structure):
    _fields_ = [("rollout_noise", C.c_void_p), ("initial_states", C.c_void_p), ("sample_offsets", C.c_void_p), ("noise_critic", C.c_void_p),
                ("noise_actor", C.c_void_p)]


class SacLoopOutputs(C.Structure):
    _fields_ = [("critic_loss", C.c_void_p), ("observations_actions_base", C.c_void_p), ("rewards", C.c_void_p), ("terminated", C.c_void_p),
                ("target_action_value", C.c_void_p), ("phase_ticks", C.c_void_p),
                ("drawn_rollout_noise", C.c_void_p), ("drawn_initial_states", C.c_void_p), ("drawn_sample_offsets", C.c_void_p),
                ("drawn_noise_critic", C.c_void_p), ("drawn_noise_actor", C.c_void_p), ("stage_ticks", C.c_void_p)]


class SacLoopScratch(C.Structure):
    _fields_ = [("rollout_noise", C.c_void_p), ("noise_critic", C.c_void_p), ("noise_actor", C.c_void_p), ("env_indices", C.c_void_p), ("sample_offsets", C.c_void_p)]


class PpoParameters(C.Structure):
    _fields_ = [("epsilon_clip", C.c_float), ("action_entropy_coefficient", C.c_float), ("advantage_epsilon", C.c_float),
                ("normalize_advantage", C.c_int32), ("learn_action_std", C.c_int32), ("reserved", C.c_int32 * 3)]


def ppo_parameters(epsilon_clip=0.2, action_entropy_coefficient=0.01, advantage_epsilon=1e-8, normalize_advantage=1, learn_action_std=1):
    return PpoParameters(epsilon_clip, action_entropy_coefficient, advantage_epsilon, normalize_advantage, learn_action_std)


class PpoAgent(C.Structure):
    _fields_ = [("actor", C.POINTER(DenseLayer)), ("n_actor_layers", C.c_int32), ("critic", C.POINTER(DenseLayer)), ("n_critic_layers", C.c_int32),
                ("log_std", C.c_void_p), ("d_log_std", C.c_void_p),
                ("actor_adam_tensors", C.POINTER(AdamTensor)), ("n_actor_adam_tensors", C.c_int32),
                ("critic_adam_tensors", C.POINTER(AdamTensor)), ("n_critic_adam_tensors", C.c_int32),
                ("actor_adam", AdamParameters), ("critic_adam", AdamParameters), ("actor_age", C.c_void_p), ("critic_age", C.c_void_p),
                ("observation_dim", C.c_int32), ("observation_privileged_dim", C.c_int32), ("action_dim", C.c_int32), ("batch", C.c_int32),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
                ("actor_standardize_mean", C.c_void_p), ("actor_standardize_precision", C.c_void_p),
                ("critic_standardize_mean", C.c_void_p), ("critic_standardize_precision", C.c_void_p)]


class GruLayer(C.Structure):
    _fields_ = [("weights_input", C.c_void_p), ("biases_input", C.c_void_p), ("weights_hidden", C.c_void_p), ("biases_hidden", C.c_void_p),
                ("initial_hidden_state", C.c_void_p), ("d_weights_input", C.c_void_p), ("d_biases_input", C.c_void_p), ("d_weights_hidden", C.c_void_p),
                ("d_biases_hidden", C.c_void_p), ("post_activation", C.c_void_p), ("n_pre_pre_activation", C.c_void_p), ("output", C.c_void_p),
                ("input_dim", C.c_int32), ("hidden_dim", C.c_int32), ("fast_tanh", C.c_int32), ("reserved", C.c_int32)]


class SeqLayer(C.Structure):
    _fields_ = [("kind", C.c_int32), ("reserved", C.c_int32), ("dense", DenseLayer), ("gru", GruLayer)]


RLT_SEQ_MAX_LAYERS = 8


class SeqState(C.Structure):
    _fields_ = [("hidden", C.c_void_p * RLT_SEQ_MAX_LAYERS), ("step", C.c_void_p * RLT_SEQ_MAX_LAYERS)]


class SacSequenceAgent(C.Structure):
    _fields_ = [("observation_dim", C.c_int32), ("action_dim", C.c_int32), ("n_actor_layers", C.c_int32), ("n_critic_layers", C.c_int32),
                ("include_first_step_in_targets", C.c_int32), ("reserved0", C.c_int32), ("gamma", C.c_float), ("polyak", C.c_float),
                ("sas", SasParameters), ("actor_adam", AdamParameters), ("critic_adam", AdamParameters), ("alpha_adam", AdamParameters),
                ("actor", C.POINTER(SeqLayer)), ("critics", C.POINTER(SeqLayer) * 2), ("critics_target", C.POINTER(SeqLayer) * 2),
                ("actor_adam_tensors", C.POINTER(AdamTensor)), ("n_actor_adam_tensors", C.c_int32), ("pad0", C.c_int32),
                ("critic_adam_tensors", C.POINTER(AdamTensor) * 2), ("n_critic_adam_tensors", C.c_int32), ("pad1", C.c_int32),
                ("log_alpha", AdamTensor),
                ("actor_age", C.c_void_p), ("critic_age", C.c_void_p * 2), ("alpha_age", C.c_void_p),
                ("batch", SequenceBatch),
                ("next_state_action_value_input", C.c_void_p), ("next_q", C.c_void_p * 2), ("next_log_probabilities", C.c_void_p),
                ("target_action_value", C.c_void_p), ("d_output", C.c_void_p), ("state_action_value_input", C.c_void_p),
                ("d_critic_input", C.c_void_p * 2), ("d_actor_output_squashing", C.c_void_p), ("d_actor_output", C.c_void_p),
                ("actor_actions", C.c_void_p), ("actor_pre_squashing", C.c_void_p), ("actor_log_probabilities", C.c_void_p),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t)]


class Td3SequenceAgent(C.Structure):
    _fields_ = [("observation_dim", C.c_int32), ("action_dim", C.c_int32), ("n_actor_layers", C.c_int32), ("n_critic_layers", C.c_int32),
                ("include_first_step_in_targets", C.c_int32), ("ignore_termination", C.c_int32),
                ("gamma", C.c_float), ("actor_polyak", C.c_float), ("critic_polyak", C.c_float), ("reserved0", C.c_float),
                ("actor_adam", AdamParameters), ("critic_adam", AdamParameters),
                ("actor", C.POINTER(SeqLayer)), ("actor_target", C.POINTER(SeqLayer)), ("critics", C.POINTER(SeqLayer) * 2), ("critics_target", C.POINTER(SeqLayer) * 2),
                ("actor_adam_tensors", C.POINTER(AdamTensor)), ("n_actor_adam_tensors", C.c_int32), ("pad0", C.c_int32),
                ("critic_adam_tensors", C.POINTER(AdamTensor) * 2), ("n_critic_adam_tensors", C.c_int32), ("pad1", C.c_int32),
                ("actor_age", C.c_void_p), ("critic_age", C.c_void_p * 2),
                ("batch", SequenceBatch),
                ("target_next_action_noise", C.c_void_p), ("next_state_action_value_input", C.c_void_p), ("next_q", C.c_void_p * 2),
                ("target_action_value", C.c_void_p), ("d_output", C.c_void_p), ("state_action_value_input", C.c_void_p),
                ("d_critic_input", C.c_void_p), ("d_actor_output", C.c_void_p), ("actor_input", C.c_void_p),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t)]


class Td3CriticDraws(C.Structure):
    _fields_ = [("seed", C.c_uint64), ("target_noise_stream", C.c_uint64), ("sampling_stream", C.c_uint64 * 2), ("target_noise_std", C.c_float), ("target_noise_clip", C.c_float)]


class Td3Agent(C.Structure):
    _fields_ = [("batch", C.c_int32), ("observation_dim", C.c_int32), ("action_dim", C.c_int32), ("n_actor_layers", C.c_int32),
                ("n_critic_layers", C.c_int32), ("ignore_termination", C.c_int32),
                ("gamma", C.c_float), ("actor_polyak", C.c_float), ("critic_polyak", C.c_float), ("sampling_std", C.c_float),
                ("actor_adam", AdamParameters), ("critic_adam", AdamParameters),
                ("actor", C.POINTER(DenseLayer)), ("actor_target", C.POINTER(DenseLayer)),
                ("critics", C.POINTER(DenseLayer) * 2), ("critics_target", C.POINTER(DenseLayer) * 2),
                ("actor_adam_tensors", C.POINTER(AdamTensor)), ("n_actor_adam_tensors", C.c_int32), ("pad0", C.c_int32),
                ("critic_adam_tensors", C.POINTER(AdamTensor) * 2), ("n_critic_adam_tensors", C.c_int32), ("pad1", C.c_int32),
                ("actor_age", C.c_void_p), ("critic_age", C.c_void_p * 2),
                ("observations_actions_base", C.c_void_p), ("rewards", C.c_void_p), ("terminated", C.c_void_p),
                ("final_step_mask", C.c_void_p), ("next_final_step_mask", C.c_void_p),
                ("target_next_action_noise", C.c_void_p), ("next_state_action_value_input", C.c_void_p), ("next_q", C.c_void_p * 2),
                ("target_action_value", C.c_void_p), ("d_output_critic", C.c_void_p),
                ("state_action_value_input", C.c_void_p), ("actor_pre_clip", C.c_void_p), ("d_output_actor", C.c_void_p),
                ("d_critic_input", C.c_void_p), ("d_actor_output", C.c_void_p),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t)]


class OnPolicyDataset(C.Structure):
    _fields_ = [("observations", C.c_void_p), ("actions_mean", C.c_void_p), ("actions", C.c_void_p), ("action_log_probs", C.c_void_p), ("rewards", C.c_void_p),
                ("terminated", C.c_void_p), ("truncated", C.c_void_p), ("all_reset", C.c_void_p), ("ld", C.c_int32), ("steps_per_env", C.c_int32)]


I, F, P, S, U64 = C.c_int, C.c_float, C.c_void_p, C.c_size_t, C.c_uint64
LP = C.POINTER(DenseLayer)
# return codes of the C ABI (include/rlt_rocm.h)
RLT_E_INVALID_ARGUMENT, RLT_E_UNSUPPORTED, RLT_E_NOT_INITIALISED, RLT_E_DEVICE_TIMEOUT, RLT_E_WORKSPACE_TOO_SMALL = -1, -2, -3, -4, -5
STATIC_SCRATCH_BYTES = 16 << 20

# name -> argument types after the leading device handle (shared by the HIP library and, minus the handle, the CPU checker)
PROTOTYPES = {
    "dense_evaluate": [LP, P, I, P, I, I],
    "dense_forward": [LP, P, I, P, I, I],
    "dense_backward_input": [LP, P, I, P, I, I],
    "dense_backward": [LP, P, I, P, I, I],
    "dense_backward_full": [LP, P, I, P, I, P, I, I],
    "mlp_evaluate": [LP, I, P, I, P, I, I, P, S],
    "mlp_forward": [LP, I, P, I, I],
    "mlp_backward": [LP, I, P, I, P, I, P, I, I, I, P, S],
    "mlp_zero_gradient": [LP, I],
    "mlp_forward_backward": [LP, I, P, I, P, I, P, I, P, I, F, I, P, S],
    "mlp_forward_backward_input": [LP, I, P, I, P, I, P, I, P, I, F, P, I, I, P, S],
    "adam_step": [C.POINTER(AdamTensor), I, C.POINTER(AdamParameters), P, F, P],
    "adam_reset": [C.POINTER(AdamTensor), I, P],
    "polyak_update": [P, P, S, F, I],
    "mse_gradient": [P, I, P, I, P, I, I, I, F, P],
    "mse_evaluate": [P, I, P, I, I, I, F, P],
    "sas_forward": [C.POINTER(SasParameters), P, I, P, I, P, I, P, I, P, I, I],
    "sas_backward": [C.POINTER(SasParameters), P, I, P, I, P, I, P, I, P, I, P, I, P, P, I, I],
    "sac_target_action_values": [P, P, P, P, P, P, F, I, P, I],
    "sac_min_value_d_output": [P, P, P, P, I, I, I, P, I, I],
    "mask_copy": [P, I, P, I, P, I, I, I],
    "mask_zero": [P, I, P, I, I, I],
    "scale_f32": [P, S, F, I],
    "unary_f32": [I, F, P, I, P, I, I, I],
    "binary_f32": [I, P, I, P, I, P, I, I, I],
    "multiply_accumulate_f32": [P, I, P, I, P, I, P, I, I, I],
    "reduce_abs_max_f32": [P, S, P],
    "cast_reduce_sum_u8": [P, S, P],
    "sac_train_critic": [C.POINTER(SacAgent), I, P],
    "sac_update_critic_targets": [C.POINTER(SacAgent)],
    "sac_train_actor": [C.POINTER(SacAgent), P],
    "replay_add": [C.POINTER(ReplayBuffer), P, P, P, P, P, P],
    "gather_batch": [C.POINTER(ReplayBuffer), P, P, I, I, I, P, P, P, P, P, P, P],
    "pendulum_step": [C.POINTER(PendulumParameters), P, P, P, P, P, I],
    "gather_sequence_batch": [C.POINTER(ReplayBuffer), C.POINTER(SequenceSampling), C.POINTER(SequenceDraws), I, C.POINTER(SequenceBatch)],
    "gather_sequence_draw": [C.POINTER(ReplayBuffer), C.POINTER(SequenceSampling), I, I, I, U64, U64, P, P, P, P],
    "acrobot_step": [C.POINTER(AcrobotParameters), I, P, P, P, P, P, P, I],
    "car_step": [C.POINTER(CarParameters), P, P, P, P, P, P, I],
    "env_runner_step": [C.POINTER(EnvRunner), C.POINTER(ReplayBuffer), I, LP, I, C.POINTER(SasParameters), P, P, P, P, S],
    "env_runner_step_sequential": [C.POINTER(EnvRunner), C.POINTER(ReplayBuffer), C.POINTER(SeqLayer), I, C.POINTER(SeqState), I, I, C.POINTER(SasParameters), F, P, P, P, S],
    "env_on_policy_collect": [C.POINTER(EnvRunner), C.POINTER(OnPolicyDataset), C.POINTER(SeqLayer), I, C.POINTER(SeqState), I, P, P, P, P, P, I, P, S],
    "env_evaluate": [C.POINTER(EnvRunner), I, C.POINTER(SeqLayer), I, C.POINTER(SeqState), I, P, P, P, I, I, P, P, P, P, S],
    "car_track_step": [C.POINTER(CarParameters), P, I, I, F, P, P, P, P, P, P, I],
    "pendulum_evaluate": [C.POINTER(PendulumParameters), I, LP, I, P, I, I, P, P, P],
    "pendulum_evaluate_standardized": [C.POINTER(PendulumParameters), I, LP, I, P, P, P, I, I, P, P, P],
    "ppo_gae": [P, P, P, P, P, P, I, I, I, F, F, I],
    "gru_forward": [C.POINTER(GruLayer), P, P, I, I, P, S],
    "gru_backward": [C.POINTER(GruLayer), P, P, P, P, I, I, I, P, S],
    "ppo_surrogate_gradient": [P, I, P, P, I, P, I, P, I, C.POINTER(PpoParameters), P, I, P, I, I],
    "ppo_train_minibatch": [C.POINTER(PpoAgent), C.POINTER(PpoParameters), P, P, P, P, P, P, I, P, P],
    "ppo_train_epoch": [C.POINTER(PpoAgent), C.POINTER(PpoParameters), P, P, P, P, P, P, I, P, I, P],
    "standardize_set_statistics": [P, P, P, P, I],
    "standardize_forward": [P, P, P, I, P, I, I, I],
    "standardize_backward_input": [P, P, I, P, I, I, I],
    "running_normalizer_update": [P, I, I, I, P, P, P],
    "on_policy_collect": [C.POINTER(PendulumRunner), C.POINTER(OnPolicyDataset), LP, I, P, P, P, P, P, I, P, S],
    "seq_forward": [C.POINTER(SeqLayer), I, P, I, P, I, I, P, S],
    "seq_backward": [C.POINTER(SeqLayer), I, P, I, P, P, P, I, I, I, I, P, S],
    "seq_zero_gradient": [C.POINTER(SeqLayer), I],
    "seq_reset_state": [C.POINTER(SeqLayer), I, C.POINTER(SeqState), P, I],
    "seq_evaluate_step": [C.POINTER(SeqLayer), I, P, I, C.POINTER(SeqState), I, P, I, I, P, S],
    "pendulum_evaluate_recurrent": [C.POINTER(PendulumParameters), I, C.POINTER(SeqLayer), I, C.POINTER(SeqState), I, P, I, I, P, P, P, P, S],
    "pendulum_runner_step_recurrent": [C.POINTER(PendulumRunner), C.POINTER(ReplayBuffer), C.POINTER(SeqLayer), I, C.POINTER(SeqState), I, C.POINTER(SasParameters), P, P, P, S],
    "td3_sequence_train_critic": [C.POINTER(Td3SequenceAgent), I],
    "td3_sequence_train_actor": [C.POINTER(Td3SequenceAgent)],
    "td3_sequence_update_critic_targets": [C.POINTER(Td3SequenceAgent)],
    "td3_sequence_update_actor_target": [C.POINTER(Td3SequenceAgent)],
    "sac_sequence_train_critic": [C.POINTER(SacSequenceAgent), I, P],
    "sac_sequence_update_critic_targets": [C.POINTER(SacSequenceAgent)],
    "sac_sequence_train_actor": [C.POINTER(SacSequenceAgent), P],
    "td3_sampling_forward": [P, I, P, I, F, P, I, P, I, I, I],
    "td3_sampling_backward": [P, I, P, I, P, I, I, I],
    "td3_target_action_noise": [P, F, F, P, S],
    "td3_noisy_next_actions": [P, I, P, I, I, I],
    "td3_target_action_values": [P, P, P, P, F, I, P, I],
    "td3_train_critic": [C.POINTER(Td3Agent), I, P],
    "td3_train_actor": [C.POINTER(Td3Agent), P],
    "td3_update_critic_targets": [C.POINTER(Td3Agent)],
    "td3_update_actor_target": [C.POINTER(Td3Agent)],
}
# workspace arguments exist only in the device ABI (the CPU checker allocates its own)
ROCM_ONLY = {
    "init": ([I, C.POINTER(P)], I), "destroy": ([P], I), "check_status": ([P], I), "set_stream": ([P, P], I), "get_stream": ([P], P),
    "error_string": ([I], C.c_char_p), "device_info": ([P, C.POINTER(I), C.POINTER(I), C.c_char_p, I], I),
    "malloc": ([P, C.POINTER(P), S], I), "free": ([P, P], I),
    "memcpy_h2d": ([P, P, P, S], I), "memcpy_d2h": ([P, P, P, S], I), "memcpy_d2d": ([P, P, P, S], I),
    "memcpy2d": ([P, P, S, P, S, S, S, I], I),
    "fill_f32": ([P, P, I, I, I, F], I), "fill_from_f32": ([P, P, I, I, I, P], I), "fill_u8": ([P, P, S, C.c_uint8], I),
    "env_runner_step_drawn": ([P, C.POINTER(EnvRunner), C.POINTER(ReplayBuffer), C.POINTER(SeqLayer), I, I, C.POINTER(SasParameters), F, P, P, P, U64, U64, U64], I),
    "randn_f32": ([P, P, S, U64, U64], I), "rand_f32": ([P, P, S, F, F, U64, U64], I), "rand_bits_u32": ([P, P, S, U64, U64], I),
    "reduce_sum_f32": ([P, P, S, I, P], I),
    "dense_backward_static": ([P, LP, P, I, P, I, I], I),
    "sac_sequence_train_critics": ([P, C.POINTER(SacSequenceAgent), P], I),
    "td3_sequence_train_critics": ([P, C.POINTER(Td3SequenceAgent)], I),
    "td3_train_critics": ([P, C.POINTER(Td3Agent), P, P], I),
    "td3_train_critics_drawn": ([P, C.POINTER(Td3Agent), C.POINTER(Td3CriticDraws), P, I], I),
    "td3_train_actor_drawn": ([P, C.POINTER(Td3Agent), C.c_uint64, C.c_uint64, P], I),
    "sac_set_per_operation": ([P, I], I),
    "polyak_update_list": ([P, P, P, P, I, F], I),
    "env_dims": ([I, C.POINTER(I), C.POINTER(I), C.POINTER(I)], I),
    "env_runner_step_workspace_bytes": ([C.POINTER(EnvRunner), I, LP, I], S),
    "env_runner_step_sequential_workspace_bytes": ([C.POINTER(EnvRunner), C.POINTER(SeqLayer), I], S),
    "env_evaluate_workspace_bytes": ([I, C.POINTER(SeqLayer), I, I], S),
    "env_on_policy_collect_workspace_bytes": ([C.POINTER(EnvRunner), C.POINTER(SeqLayer), I], S),
    "mlp_workspace_bytes": ([LP, I, I], S),
    "ppo_workspace_bytes": ([C.POINTER(PpoAgent)], S),
    "gru_workspace_bytes": ([C.POINTER(GruLayer), I, I], S),
    "seq_workspace_bytes": ([C.POINTER(SeqLayer), I, I, I], S),
    "seq_evaluate_step_workspace_bytes": ([C.POINTER(SeqLayer), I, I], S),
    "pendulum_runner_step_recurrent_workspace_bytes": ([C.POINTER(SeqLayer), I, I], S),
    "pendulum_evaluate_recurrent_workspace_bytes": ([C.POINTER(SeqLayer), I, I], S),
    "sac_sequence_workspace_bytes": ([C.POINTER(SacSequenceAgent)], S),
    "td3_sequence_workspace_bytes": ([C.POINTER(Td3SequenceAgent)], S),
    "on_policy_collect_workspace_bytes": ([C.POINTER(PendulumRunner), LP, I], S),
    "gather_draw": ([P, C.POINTER(ReplayBuffer), I, U64, U64, P, P], I),
    "sac_pendulum_loop_by_calls": ([P, C.POINTER(SacAgent), C.POINTER(PendulumRunner), C.POINTER(ReplayBuffer), I, U64, U64, C.POINTER(SacLoopScratch)], I),
    "sac_pendulum_loop": ([P, C.POINTER(SacAgent), C.POINTER(PendulumRunner), C.POINTER(ReplayBuffer), I, U64, U64, C.POINTER(SacLoopInputs),
                           C.POINTER(SacLoopOutputs)], I),
    "pendulum_runner_step": ([P, C.POINTER(PendulumRunner), C.POINTER(ReplayBuffer), I, LP, I, C.POINTER(SasParameters), P, P, P, U64, U64], I),
    "pendulum_runner_step_drawn": ([P, C.POINTER(PendulumRunner), C.POINTER(ReplayBuffer), LP, I, C.POINTER(SasParameters), P, U64, U64, U64], I),
    "gather_batch_drawn": ([P, C.POINTER(ReplayBuffer), U64, U64, P, P, I, I, P, P, P, P, P, P, P], I),
    "sac_train_critics": ([P, C.POINTER(SacAgent), P, I], I),
    "sac_train_critics_drawn": ([P, C.POINTER(SacAgent), P, U64, U64, I], I),
    "sac_train_actor_drawn": ([P, C.POINTER(SacAgent), P, U64, U64], I),
    "set_update_options": ([P, I, I], I), "set_wait_limit": ([P, C.c_uint32], I),
    "graph_begin_capture": ([P], I), "graph_end_capture": ([P, C.POINTER(P)], I), "graph_launch": ([P, P], I), "graph_destroy": ([P, P], I),
    "advance_streams": ([P, U64], I), "set_stream_offset": ([P, U64], I),
}


def load_library(path=LIB_PATH):
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build it with `python rl-tools_amd/build.py` (there is no CPU fallback)")
    lib = C.CDLL(path)
    for name, args in PROTOTYPES.items():
        fn = getattr(lib, "rlt_rocm_" + name)
        fn.argtypes = [P] + args
        fn.restype = I
    for name, (args, res) in ROCM_ONLY.items():
        fn = getattr(lib, "rlt_rocm_" + name)
        fn.argtypes = args
        fn.restype = res
    return lib


class RltError(RuntimeError):
    pass


class DeviceArray:
    """A device allocation with a numpy-like shape/dtype; `ptr` is what the C ABI takes."""

    def __init__(self, device, shape, dtype):
        self.device, self.shape, self.dtype = device, tuple(shape), np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = C.c_void_p()
        device.check(device.lib.rlt_rocm_malloc(device.handle, C.byref(p), max(self.nbytes, 4)))
        self.ptr = p.value

    def upload(self, array):
        a = np.ascontiguousarray(array, dtype=self.dtype)
        assert a.nbytes == self.nbytes, (a.shape, self.shape)
        if self.nbytes:
            self.device.check(self.device.lib.rlt_rocm_memcpy_h2d(self.device.handle, self.ptr, a.ctypes.data, self.nbytes))
        return self

    def numpy(self):
        out = np.empty(self.shape, self.dtype)
        if self.nbytes:
            self.device.check(self.device.lib.rlt_rocm_memcpy_d2h(self.device.handle, out.ctypes.data, self.ptr, self.nbytes))
        return out

    def offset(self, elements):
        return self.ptr + int(elements) * self.dtype.itemsize

    def free(self):
        if self.ptr:
            self.device.lib.rlt_rocm_free(self.device.handle, self.ptr)
            self.ptr = None


class Device:
    """rlt_rocm_device handle plus convenience allocation/call helpers."""

    def __init__(self, index=0, lib=None):
        self.lib = lib or load_library()
        h = C.c_void_p()
        rc = self.lib.rlt_rocm_init(index, C.byref(h))
        if rc != 0:
            raise RltError(f"rlt_rocm_init failed: {self.lib.rlt_rocm_error_string(rc).decode()}")
        self.handle = h
        self._arrays = []

    def check(self, rc):
        if rc != 0:
            raise RltError(f"rlt_rocm call failed ({rc}): {self.lib.rlt_rocm_error_string(rc).decode()}")

    def call(self, name, *args):
        self.check(getattr(self.lib, "rlt_rocm_" + name)(self.handle, *args))

    def sync(self):
        self.check(self.lib.rlt_rocm_check_status(self.handle))

    def empty(self, shape, dtype=np.float32):
        a = DeviceArray(self, shape, dtype)
        self._arrays.append(a)
        return a

    def zeros(self, shape, dtype=np.float32):
        return self.empty(shape, dtype).upload(np.zeros(shape, dtype))

    def array(self, host):
        host = np.asarray(host)
        return self.empty(host.shape, host.dtype).upload(host)

    def info(self):
        cu, lds = C.c_int(), C.c_int()
        name = C.create_string_buffer(128)
        self.check(self.lib.rlt_rocm_device_info(self.handle, C.byref(cu), C.byref(lds), name, 128))
        return {"compute_units": cu.value, "lds_bytes": lds.value, "name": name.value.decode()}

    def close(self):
        for a in self._arrays:
            a.free()
        self._arrays = []
        if self.handle:
            self.lib.rlt_rocm_destroy(self.handle)
            self.handle = None
