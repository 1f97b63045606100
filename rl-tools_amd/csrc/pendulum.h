// The Pendulum's transition as device code shared by the kernels that step it.
#pragma once
#include "common.h"

namespace {
__device__ __forceinline__ float clampf(float x, float lo, float hi) { return fminf(fmaxf(x, lo), hi); }

struct Transition { float obs[3]; float next_obs[3]; float action, reward; float theta, theta_dot; };

// pendulum/operations_generic.h:79-101 (step), :131-139 (reward from the pre-step state and the un-clamped action),
// :142-160 (Fourier observation)
__device__ __forceinline__ void pendulum_transition(const rlt_pendulum_parameters& p, float theta, float theta_dot, float action, Transition& t) {
    sincosf(theta, &t.obs[1], &t.obs[0]);
    t.obs[2] = theta_dot;
    float u = p.max_torque * clampf(action, -1.0f, 1.0f);
    u = clampf(u, -p.max_torque, p.max_torque);
    float newthdot = theta_dot + (3.0f * p.g / (2.0f * p.l) * t.obs[1] + 3.0f / (p.m * p.l * p.l) * u) * p.dt;
    newthdot = clampf(newthdot, -p.max_speed, p.max_speed);
    float newth = theta + newthdot * p.dt;
    const float PI = 3.14159265358979323846f;
    float a = theta + PI, b = 2.0f * PI;
    float angle_norm = (a - b * floorf(a / b)) - PI;
    float ur = p.max_torque * action;
    t.reward = -(angle_norm * angle_norm + 0.1f * theta_dot * theta_dot + 0.001f * (ur * ur));
    sincosf(newth, &t.next_obs[1], &t.next_obs[0]);
    t.next_obs[2] = newthdot;
    t.theta = newth; t.theta_dot = newthdot; t.action = action;
}
}  // namespace
