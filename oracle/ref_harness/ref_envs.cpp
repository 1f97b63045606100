// Harness around the REAL reference's analytic environments other than the Pendulum (compiled from /root/reference/include where it lies; nothing
// of it is copied here): batched step / reward / observe / terminated of the Acrobot and the AcrobotSwingup with their default parameters, and of
// the Car, without a track and on the reference's default track. Built by oracle/Makefile into oracle/_ref/librlt_ref_envs_generic.so.
#include <rl_tools/operations/cpu_mux.h>
#include <rl_tools/rl/environments/acrobot/operations_cpu.h>
#include <rl_tools/rl/environments/car/operations_generic.h>   // (the CPU header of the car reads a bitmap file through a member the environment no longer has)

#include <cstdint>

namespace rlt = rl_tools;

namespace {
using DEVICE = rlt::devices::DEVICE_FACTORY<>;
using RNG = DEVICE::SPEC::RANDOM::ENGINE<>;
using TI = typename DEVICE::index_t;
using SPEC = rlt::rl::environments::acrobot::Specification<float, TI, rlt::rl::environments::acrobot::DefaultParameters<float>>;
using EASY_SPEC = rlt::rl::environments::acrobot::Specification<float, TI, rlt::rl::environments::acrobot::EasyParameters<float>>;

template <typename ENVIRONMENT>
void steps(const float* states, const float* actions, float* next_states, float* observations, float* next_observations, float* rewards, uint8_t* terminated, int n) {
    DEVICE device;
    RNG rng;
    rlt::malloc(device, rng);
    rlt::init(device, rng, 0);
    ENVIRONMENT env;
    typename ENVIRONMENT::Parameters parameters;
    rlt::Matrix<rlt::matrix::Specification<float, TI, 1, 1, false>> action;
    rlt::Matrix<rlt::matrix::Specification<float, TI, 1, 6, false>> observation;
    for (int e = 0; e < n; e++) {
        typename ENVIRONMENT::State state, next;
        state.theta_1 = states[4 * e]; state.theta_2 = states[4 * e + 1]; state.theta_1_dot = states[4 * e + 2]; state.theta_2_dot = states[4 * e + 3];
        rlt::set(action, 0, 0, actions[e]);
        rlt::observe(device, env, parameters, state, typename ENVIRONMENT::Observation{}, observation, rng);
        for (TI i = 0; i < 6; i++) observations[6 * e + i] = rlt::get(observation, 0, i);
        rlt::step(device, env, parameters, state, action, next, rng);
        rewards[e] = rlt::reward(device, env, parameters, state, action, next, rng);
        terminated[e] = rlt::terminated(device, env, parameters, next, rng);
        rlt::observe(device, env, parameters, next, typename ENVIRONMENT::Observation{}, observation, rng);
        for (TI i = 0; i < 6; i++) next_observations[6 * e + i] = rlt::get(observation, 0, i);
        next_states[4 * e] = next.theta_1; next_states[4 * e + 1] = next.theta_2; next_states[4 * e + 2] = next.theta_1_dot; next_states[4 * e + 3] = next.theta_2_dot;
    }
    rlt::free(device, rng);
}
}  // namespace

namespace {
using CAR_SPEC = rlt::rl::environments::car::Specification<float, TI>;
using CAR = rlt::rl::environments::Car<CAR_SPEC>;
using TRACK_SPEC = rlt::rl::environments::car::SpecificationTrack<float, TI, 100, 100, 20>;
using TRACK_CAR = rlt::rl::environments::CarTrack<TRACK_SPEC>;
}  // namespace

extern "C" {
// states [n x 6] = (x, y, mu, vx, vy, omega), actions [n x 2] = (throttle / brake, steering)
int rlt_ref_car_steps(const float* states, const float* actions, float* next_states, float* observations, float* next_observations, float* rewards, uint8_t* terminated, int n) {
    DEVICE device;
    RNG rng;
    rlt::malloc(device, rng);
    rlt::init(device, rng, 0);
    CAR env;
    CAR::Parameters parameters;
    rlt::initial_parameters(device, env, parameters);
    rlt::Matrix<rlt::matrix::Specification<float, TI, 1, 2, false>> action;
    rlt::Matrix<rlt::matrix::Specification<float, TI, 1, 6, false>> observation;
    for (int e = 0; e < n; e++) {
        CAR::State state, next;
        const float* s = states + 6 * e;
        state.x = s[0]; state.y = s[1]; state.mu = s[2]; state.vx = s[3]; state.vy = s[4]; state.omega = s[5];
        rlt::set(action, 0, 0, actions[2 * e]); rlt::set(action, 0, 1, actions[2 * e + 1]);
        rlt::observe(device, env, parameters, state, CAR::Observation{}, observation, rng);
        for (TI i = 0; i < 6; i++) observations[6 * e + i] = rlt::get(observation, 0, i);
        rlt::step(device, env, parameters, state, action, next, rng);
        rewards[e] = rlt::reward(device, env, parameters, state, action, next, rng);
        terminated[e] = rlt::terminated(device, env, parameters, next, rng);
        rlt::observe(device, env, parameters, next, CAR::Observation{}, observation, rng);
        for (TI i = 0; i < 6; i++) next_observations[6 * e + i] = rlt::get(observation, 0, i);
        float* o = next_states + 6 * e;
        o[0] = next.x; o[1] = next.y; o[2] = next.mu; o[3] = next.vx; o[4] = next.vy; o[5] = next.omega;
    }
    rlt::free(device, rng);
    return 0;
}
// The car on the reference's default track (100 x 100 cells of 20 mm): the track bitmap as the environment holds it after init ...
void rlt_ref_car_track_bitmap(uint8_t* track) {
    DEVICE device;
    TRACK_CAR env;
    rlt::init(device, env);
    for (TI r = 0; r < 100; r++) for (TI c = 0; c < 100; c++) track[r * 100 + c] = env.track[r][c];
}
// ... and batched observe / step / reward / terminated; states [n x 6], actions [n x 2], observations [n x 9]. The reference's observe reads the bitmap
// without a bounds check, so callers keep the states where the three rays (50 cells long) stay inside it.
int rlt_ref_car_track_steps(const float* states, const float* actions, float* next_states, float* observations, float* next_observations, float* rewards, uint8_t* terminated, int n) {
    DEVICE device;
    RNG rng;
    rlt::malloc(device, rng);
    rlt::init(device, rng, 0);
    TRACK_CAR env;
    rlt::init(device, env);
    static TRACK_CAR::Parameters parameters;
    rlt::initial_parameters(device, env, parameters);
    rlt::Matrix<rlt::matrix::Specification<float, TI, 1, 2, false>> action;
    rlt::Matrix<rlt::matrix::Specification<float, TI, 1, 9, false>> observation;
    for (int e = 0; e < n; e++) {
        TRACK_CAR::State state, next;
        const float* s = states + 6 * e;
        state.x = s[0]; state.y = s[1]; state.mu = s[2]; state.vx = s[3]; state.vy = s[4]; state.omega = s[5];
        rlt::set(action, 0, 0, actions[2 * e]); rlt::set(action, 0, 1, actions[2 * e + 1]);
        rlt::observe(device, env, parameters, state, TRACK_CAR::Observation{}, observation, rng);
        for (TI i = 0; i < 9; i++) observations[9 * e + i] = rlt::get(observation, 0, i);
        rlt::step(device, env, parameters, state, action, next, rng);
        rewards[e] = rlt::reward(device, env, parameters, state, action, next, rng);
        terminated[e] = rlt::terminated(device, env, parameters, next, rng);
        if (next_observations) {
            rlt::observe(device, env, parameters, next, TRACK_CAR::Observation{}, observation, rng);
            for (TI i = 0; i < 9; i++) next_observations[9 * e + i] = rlt::get(observation, 0, i);
        }
        float* o = next_states + 6 * e;
        o[0] = next.x; o[1] = next.y; o[2] = next.mu; o[3] = next.vx; o[4] = next.vy; o[5] = next.omega;
    }
    rlt::free(device, rng);
    return 0;
}
// kind 0: Acrobot, 1: AcrobotSwingup, 2: AcrobotSwingup with EasyParameters (torque +-10)
int rlt_ref_acrobot_steps(int kind, const float* states, const float* actions, float* next_states, float* observations, float* next_observations, float* rewards,
                          uint8_t* terminated, int n) {
    if (kind == 0) steps<rlt::rl::environments::Acrobot<SPEC>>(states, actions, next_states, observations, next_observations, rewards, terminated, n);
    else if (kind == 1) steps<rlt::rl::environments::AcrobotSwingup<SPEC>>(states, actions, next_states, observations, next_observations, rewards, terminated, n);
    else if (kind == 2) steps<rlt::rl::environments::AcrobotSwingup<EASY_SPEC>>(states, actions, next_states, observations, next_observations, rewards, terminated, n);
    else return -1;
    return 0;
}
}
