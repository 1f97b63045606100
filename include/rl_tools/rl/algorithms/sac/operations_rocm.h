// SAC's element-wise steps on devices::ROCM: target_action_values, min_value_d_output, mask_actions, mask_gradient (the counterpart of
// rl/algorithms/sac/operations_cuda.h:9-128). train_critic / train_actor / update_critic_targets are the reference's generic functions
// (rl/algorithms/sac/operations_generic.h:243-337,395-468,524-527): with these overloads and those of the layers, the optimiser and
// the containers every call they make resolves to this backend.
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/rl/algorithms/sac/sac.h>
#include <rl_tools/rl/components/off_policy_runner/off_policy_runner.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools{
    // target_action_values    sac/operations_cuda.h:10-43: y = r + gamma * (1 - terminated) * (min(Q1', Q2') - alpha * log pi(a'|s'))
    template <typename DEV_SPEC, typename BATCH_SPEC, typename TRAINING_BUFFER_SPEC, typename NEXT_ACTION_LOG_PROBS_SPEC, typename LOG_ALPHA_PARAMETER>
    void target_action_values(devices::ROCM<DEV_SPEC>& device, rl::components::off_policy_runner::SequentialBatch<BATCH_SPEC>& batch, rl::algorithms::sac::CriticTrainingBuffers<TRAINING_BUFFER_SPEC>& training_buffers, const Matrix<NEXT_ACTION_LOG_PROBS_SPEC>& next_action_log_probs, LOG_ALPHA_PARAMETER& log_alpha){
        using SPEC = typename TRAINING_BUFFER_SPEC::SPEC;
        using BUFFERS = rl::algorithms::sac::CriticTrainingBuffers<TRAINING_BUFFER_SPEC>;
        constexpr auto BATCH_SIZE = BATCH_SPEC::BATCH_SIZE;
        constexpr auto SEQUENCE_LENGTH = BATCH_SPEC::SEQUENCE_LENGTHH;
        static_assert(BATCH_SIZE == BUFFERS::BATCH_SIZE);
        static_assert(SPEC::PARAMETERS::ENTROPY_BONUS && SPEC::PARAMETERS::ENTROPY_BONUS_NEXT_STEP, "the ROCM kernel adds the entropy bonus of the next step inside the discounted term");
        static_assert(NEXT_ACTION_LOG_PROBS_SPEC::COL_PITCH == 1);
        constexpr auto TARGET_OFFSET = BATCH_SPEC::PARAMETERS::INCLUDE_FIRST_STEP_IN_TARGETS ? BATCH_SIZE : 0;      // the target of step t takes the target critics' value at t + 1 ...
        devices::rocm::check(rlt_rocm_sac_target_action_values(device.handle, training_buffers.next_state_action_value_critic_1._data + TARGET_OFFSET, training_buffers.next_state_action_value_critic_2._data + TARGET_OFFSET,
                                                               batch.rewards._data, (const uint8_t*)batch.terminated._data, next_action_log_probs._data /* ... and the log-probability at index t */, log_alpha.parameters._data,
                                                               (float)SPEC::PARAMETERS::GAMMA, SPEC::PARAMETERS::IGNORE_TERMINATION ? 1 : 0, training_buffers.target_action_value._data, SEQUENCE_LENGTH * BATCH_SIZE), "target_action_values");
    }
    // min_value_d_output      sac/operations_cuda.h:45-72: per sample, the action columns of the input gradient of the critic with the smaller value
    template <typename DEV_SPEC, typename SPEC, typename TRAINING_BUFFERS_SPEC>
    void min_value_d_output(devices::ROCM<DEV_SPEC>& device, rl::algorithms::sac::ActorCritic<SPEC>& actor_critic, rl::algorithms::sac::ActorTrainingBuffers<TRAINING_BUFFERS_SPEC>& training_buffers){
        using BUFFERS = rl::algorithms::sac::ActorTrainingBuffers<TRAINING_BUFFERS_SPEC>;
        constexpr int ROWS = BUFFERS::BATCH_SIZE * SPEC::PARAMETERS::SEQUENCE_LENGTH;
        constexpr int CRITIC_INPUT_DIM = get_last(typename SPEC::CRITIC_NETWORK_TYPE::INPUT_SHAPE{});
        constexpr int ACTION_DIM = SPEC::ENVIRONMENT::ACTION_DIM;
        auto critic_1_output = output(device, actor_critic.critics[0]);
        auto critic_2_output = output(device, actor_critic.critics[1]);
        devices::rocm::check(rlt_rocm_sac_min_value_d_output(device.handle, critic_1_output._data, critic_2_output._data, training_buffers.d_critic_1_input._data, training_buffers.d_critic_2_input._data,
                                                             CRITIC_INPUT_DIM, CRITIC_INPUT_DIM, ACTION_DIM, training_buffers.d_actor_output_squashing._data, ACTION_DIM, ROWS), "min_value_d_output");
    }
    // mask_actions            sac/operations_cuda.h:73-99: rows of `source` replace rows of `target` where the mask (or its inverse) is set
    template <typename DEV_SPEC, typename SOURCE_SPEC, typename TARGET_SPEC, typename MASK_SPEC>
    void mask_actions(devices::ROCM<DEV_SPEC>& device, Tensor<SOURCE_SPEC>& source, Tensor<TARGET_SPEC>& target, Tensor<MASK_SPEC>& mask, bool invert_mask = false){
        static_assert(SOURCE_SPEC::SHAPE::LENGTH == 3 && tensor::same_dimensions<SOURCE_SPEC, TARGET_SPEC>());
        static_assert(tensor::dense_row_major_layout<MASK_SPEC>() && sizeof(typename MASK_SPEC::T) == 1);
        constexpr int ROWS = SOURCE_SPEC::SHAPE::template GET<0> * SOURCE_SPEC::SHAPE::template GET<1>, COLS = SOURCE_SPEC::SHAPE::template GET<2>;
        static_assert(SOURCE_SPEC::STRIDE::template GET<2> == 1 && TARGET_SPEC::STRIDE::template GET<2> == 1);
        static_assert(SOURCE_SPEC::STRIDE::template GET<0> == SOURCE_SPEC::STRIDE::template GET<1> * SOURCE_SPEC::SHAPE::template GET<1> && TARGET_SPEC::STRIDE::template GET<0> == TARGET_SPEC::STRIDE::template GET<1> * TARGET_SPEC::SHAPE::template GET<1>,
                      "sequence steps follow each other with the row stride");
        devices::rocm::check(rlt_rocm_mask_copy(device.handle, source._data, SOURCE_SPEC::STRIDE::template GET<1>, target._data, TARGET_SPEC::STRIDE::template GET<1>, (const uint8_t*)mask._data, invert_mask ? 1 : 0, ROWS, COLS), "mask_actions");
    }
    // mask_gradient           sac/operations_cuda.h:100-128: rows are zeroed where the mask (or its inverse) is set
    template <typename DEV_SPEC, typename SOURCE_SPEC, typename MASK_SPEC>
    void mask_gradient(devices::ROCM<DEV_SPEC>& device, Tensor<SOURCE_SPEC>& source, Tensor<MASK_SPEC>& mask, bool invert_mask = false){
        static_assert(SOURCE_SPEC::SHAPE::LENGTH == 3);
        static_assert(tensor::dense_row_major_layout<MASK_SPEC>() && sizeof(typename MASK_SPEC::T) == 1);
        constexpr int ROWS = SOURCE_SPEC::SHAPE::template GET<0> * SOURCE_SPEC::SHAPE::template GET<1>, COLS = SOURCE_SPEC::SHAPE::template GET<2>;
        static_assert(SOURCE_SPEC::STRIDE::template GET<2> == 1 && SOURCE_SPEC::STRIDE::template GET<0> == SOURCE_SPEC::STRIDE::template GET<1> * SOURCE_SPEC::SHAPE::template GET<1>);
        devices::rocm::check(rlt_rocm_mask_zero(device.handle, source._data, SOURCE_SPEC::STRIDE::template GET<1>, (const uint8_t*)mask._data, invert_mask ? 1 : 0, ROWS, COLS), "mask_gradient");
    }
}
RL_TOOLS_NAMESPACE_WRAPPER_END
