// The environments whose step, reward, observation and termination the library has kernels for, described to its entry points
// (rlt_env_runner: a kind and that kind's parameters) from the reference's environment types, with their initial states drawn on the device:
//   rl::environments::Pendulum        rl/environments/pendulum/pendulum.h,  sample_initial_state operations_generic.h:58-61
//   rl::environments::PendulumPosition (pendulum.h:117-124: the velocity is hidden from the observation, the state remembers the last action), :62-66
//   rl::environments::Acrobot         rl/environments/acrobot/acrobot.h,    sample_initial_state operations_generic.h:39-44
//   rl::environments::AcrobotSwingup  (the same dynamics, another reward),  sample_initial_state operations_generic.h:46-52
//   rl::environments::Car             rl/environments/car/car.h (the variant without a track), sample_initial_state operations_generic.h:70-78
// The parameters of the first four are static members of ENVIRONMENT::SPEC::PARAMETERS. The Car's are the member initialisers of its Parameters struct
// (car.h:19-33; initial_parameters leaves them as they are, operations_generic.h:52-54), so a value-initialised Parameters object holds them: a description needs
// the type only here too. CarTrack (a track bitmap in the environment object) has a kernel (rlt_rocm_car_track_step) and no description.
#pragma once
#include <rl_tools/devices/rocm.h>
#include <rl_tools/rl/environments/pendulum/pendulum.h>
#include <rl_tools/rl/environments/acrobot/acrobot.h>
#include <rl_tools/rl/environments/car/car.h>
RL_TOOLS_NAMESPACE_WRAPPER_START
namespace rl_tools::rl::environments::rocm{
    template <typename ENVIRONMENT>
    struct Description{
        static constexpr bool SUPPORTED = false;
    };
    template <typename SPEC>
    struct Description<rl::environments::Pendulum<SPEC>>{
        using P = typename SPEC::PARAMETERS;
        static constexpr bool SUPPORTED = true;
        static constexpr int KIND = RLT_ENV_PENDULUM;
        static constexpr size_t STATE_DIM = 2;
        static_assert(P::initial_state_min_angle == -P::initial_state_max_angle && P::initial_state_min_speed == -P::initial_state_max_speed, "initial states are drawn from ranges that are symmetric about zero");
        static rlt_pendulum_parameters parameters(){
            return rlt_pendulum_parameters{(float)P::g, (float)P::max_speed, (float)P::max_torque, (float)P::dt, (float)P::m, (float)P::l};
        }
        static void set_parameters(rlt_env_runner& runner){ runner.env_kind = KIND; runner.pendulum = parameters(); }
        // uniform in +- the largest angle and speed
        template <typename DEV_SPEC, typename RNG>
        static void sample_initial_states(devices::ROCM<DEV_SPEC>& device, float* initial, size_t n, RNG& rng){
            devices::rocm::check(rlt_rocm_rand_f32(device.handle, initial, n * 2, -1.0f, 1.0f, rng.seed, random::next_stream(rng)), "sample_initial_state (Pendulum)");
            devices::rocm::check(rlt_rocm_unary_f32(device.handle, RLT_UNARY_SCALE, (float)P::initial_state_max_angle, initial, 2, initial, 2, (int)n, 1), "sample_initial_state (Pendulum)");
            if constexpr(P::initial_state_max_speed != 1){
                devices::rocm::check(rlt_rocm_unary_f32(device.handle, RLT_UNARY_SCALE, (float)P::initial_state_max_speed, initial + 1, 2, initial + 1, 2, (int)n, 1), "sample_initial_state (Pendulum)");
            }
        }
        // the same ranges per state component, for the runner step that draws inside its launch
        static void initial_ranges(float* low, float* high){
            high[0] = (float)P::initial_state_max_angle; high[1] = (float)P::initial_state_max_speed; low[0] = -high[0]; low[1] = -high[1];
        }
        // initial_state (rl/environments/pendulum/operations_generic.h:38-41): hanging down, at rest
        static void initial_state(float* host){ host[0] = -math::PI<float>; host[1] = 0; }
    };
    template <typename SPEC>
    struct Description<rl::environments::PendulumPosition<SPEC>>{
        using P = typename SPEC::PARAMETERS;
        static constexpr bool SUPPORTED = true;
        static constexpr int KIND = RLT_ENV_PENDULUM_POSITION;
        static constexpr size_t STATE_DIM = 3;      // theta, theta_dot, last_action
        static_assert(P::initial_state_min_angle == -P::initial_state_max_angle && P::initial_state_min_speed == -P::initial_state_max_speed, "initial states are drawn from ranges that are symmetric about zero");
        static_assert(P::OBSERVATION_NOISE_POSITION == 0, "the library's kernels observe without noise");
        static void set_parameters(rlt_env_runner& runner){ runner.env_kind = KIND; runner.pendulum = Description<rl::environments::Pendulum<SPEC>>::parameters(); }
        // angle and speed uniform in +- their largest values, last_action = 0 (operations_generic.h:62-66)
        template <typename DEV_SPEC, typename RNG>
        static void sample_initial_states(devices::ROCM<DEV_SPEC>& device, float* initial, size_t n, RNG& rng){
            devices::rocm::check(rlt_rocm_rand_f32(device.handle, initial, n * 3, -1.0f, 1.0f, rng.seed, random::next_stream(rng)), "sample_initial_state (PendulumPosition)");
            devices::rocm::check(rlt_rocm_unary_f32(device.handle, RLT_UNARY_SCALE, (float)P::initial_state_max_angle, initial, 3, initial, 3, (int)n, 1), "sample_initial_state (PendulumPosition)");
            if constexpr(P::initial_state_max_speed != 1){
                devices::rocm::check(rlt_rocm_unary_f32(device.handle, RLT_UNARY_SCALE, (float)P::initial_state_max_speed, initial + 1, 3, initial + 1, 3, (int)n, 1), "sample_initial_state (PendulumPosition)");
            }
            devices::rocm::check(rlt_rocm_fill_f32(device.handle, initial + 2, (int)n, 1, 3, 0.0f), "sample_initial_state (PendulumPosition)");
        }
        static void initial_ranges(float* low, float* high){
            high[0] = (float)P::initial_state_max_angle; high[1] = (float)P::initial_state_max_speed; low[0] = -high[0]; low[1] = -high[1]; low[2] = high[2] = 0;
        }
        // initial_state (operations_generic.h:42-46): hanging down, at rest, no action yet
        static void initial_state(float* host){ host[0] = -math::PI<float>; host[1] = 0; host[2] = 0; }
    };
    namespace acrobot{
        template <typename P>
        rlt_acrobot_parameters parameters(){
            return rlt_acrobot_parameters{(float)P::DT, (float)P::LINK_LENGTH_1, (float)P::LINK_LENGTH_2, (float)P::LINK_MASS_1, (float)P::LINK_MASS_2, (float)P::LINK_COM_POS_1,
                                          (float)P::LINK_COM_POS_2, (float)P::LINK_MOI, (float)P::MAX_VEL_1, (float)P::MAX_VEL_2, (float)P::MIN_TORQUE, (float)P::MAX_TORQUE};
        }
    }
    template <typename SPEC>
    struct Description<rl::environments::Acrobot<SPEC>>{
        static constexpr bool SUPPORTED = true;
        static constexpr int KIND = RLT_ENV_ACROBOT;
        static constexpr size_t STATE_DIM = 4;
        static void set_parameters(rlt_env_runner& runner){ runner.env_kind = KIND; runner.acrobot = acrobot::parameters<typename SPEC::PARAMETERS>(); }
        // both angles and both velocities uniform in +- 0.1
        template <typename DEV_SPEC, typename RNG>
        static void sample_initial_states(devices::ROCM<DEV_SPEC>& device, float* initial, size_t n, RNG& rng){
            devices::rocm::check(rlt_rocm_rand_f32(device.handle, initial, n * 4, -0.1f, 0.1f, rng.seed, random::next_stream(rng)), "sample_initial_state (Acrobot)");
        }
        static void initial_ranges(float* low, float* high){ for(int i = 0; i < 4; i++){ low[i] = -0.1f; high[i] = 0.1f; } }
        // initial_state (rl/environments/acrobot/operations_generic.h:54-59): hanging down, at rest
        static void initial_state(float* host){ host[0] = host[1] = host[2] = host[3] = 0; }
    };
    template <typename SPEC>
    struct Description<rl::environments::AcrobotSwingup<SPEC>>{
        static constexpr bool SUPPORTED = true;
        static constexpr int KIND = RLT_ENV_ACROBOT_SWINGUP;
        static constexpr size_t STATE_DIM = 4;
        static void set_parameters(rlt_env_runner& runner){ runner.env_kind = KIND; runner.acrobot = acrobot::parameters<typename SPEC::PARAMETERS>(); }
        // both angles uniform over the circle, at rest
        template <typename DEV_SPEC, typename RNG>
        static void sample_initial_states(devices::ROCM<DEV_SPEC>& device, float* initial, size_t n, RNG& rng){
            devices::rocm::check(rlt_rocm_rand_f32(device.handle, initial, n * 4, -math::PI<float>, math::PI<float>, rng.seed, random::next_stream(rng)), "sample_initial_state (AcrobotSwingup)");
            devices::rocm::check(rlt_rocm_fill_f32(device.handle, initial + 2, (int)n, 2, 4, 0.0f), "sample_initial_state (AcrobotSwingup)");
        }
        static void initial_ranges(float* low, float* high){ low[0] = low[1] = -math::PI<float>; high[0] = high[1] = math::PI<float>; low[2] = low[3] = high[2] = high[3] = 0; }
        static void initial_state(float* host){ host[0] = host[1] = host[2] = host[3] = 0; }
    };
    template <typename SPEC>
    struct Description<rl::environments::Car<SPEC>>{
        static constexpr bool SUPPORTED = true;
        static constexpr int KIND = RLT_ENV_CAR;
        static constexpr size_t STATE_DIM = 6;      // x, y, mu, vx, vy, omega
        static rlt_car_parameters parameters(){
            const typename SPEC::PARAMETERS p{};
            return rlt_car_parameters{(float)p.g, (float)p.m, (float)p.I, (float)p.lf, (float)p.lr, (float)p.tf.B, (float)p.tf.C, (float)p.tf.D, (float)p.tr.B, (float)p.tr.C, (float)p.tr.D,
                                      (float)p.cm, (float)p.cr0, (float)p.cr2, (float)p.vt, (float)p.dt};
        }
        static void set_parameters(rlt_env_runner& runner){ runner.env_kind = KIND; runner.car = parameters(); }
        // position uniform in +- 0.2, heading uniform over the circle, at rest
        static void initial_ranges(float* low, float* high){
            low[0] = low[1] = -0.2f; high[0] = high[1] = 0.2f; low[2] = -math::PI<float>; high[2] = math::PI<float>; low[3] = low[4] = low[5] = high[3] = high[4] = high[5] = 0;
        }
        template <typename DEV_SPEC, typename RNG>
        static void sample_initial_states(devices::ROCM<DEV_SPEC>& device, float* initial, size_t n, RNG& rng){
            devices::rocm::check(rlt_rocm_rand_f32(device.handle, initial, n * 6, -0.2f, 0.2f, rng.seed, random::next_stream(rng)), "sample_initial_state (Car)");
            devices::rocm::check(rlt_rocm_unary_f32(device.handle, RLT_UNARY_SCALE, math::PI<float> / 0.2f, initial + 2, 6, initial + 2, 6, (int)n, 1), "sample_initial_state (Car)");
            devices::rocm::check(rlt_rocm_fill_f32(device.handle, initial + 3, (int)n, 3, 6, 0.0f), "sample_initial_state (Car)");
        }
        // initial_state (rl/environments/car/operations_generic.h:61-69): at the origin, at rest
        static void initial_state(float* host){ for(int i = 0; i < 6; i++){ host[i] = 0; } }
    };
}
RL_TOOLS_NAMESPACE_WRAPPER_END
