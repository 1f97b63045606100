/*
 * rlt_oracle_sac_loop.h -- CPU restatement of the reference's seeded SAC-on-Pendulum training loop
 * (rl/algorithms/sac/loop/core/operations_generic.h:110-155). TEST INFRASTRUCTURE ONLY, see rlt_oracle.h.
 */
#ifndef RLT_ORACLE_SAC_LOOP_H
#define RLT_ORACLE_SAC_LOOP_H
#include "rlt_oracle.h"
#ifdef __cplusplus
extern "C" {
#endif

typedef struct rlt_oracle_sac_loop_config {
    uint32_t seed;
    int32_t batch;               /* 256 for the benchmark configuration, 100 in the reference's example */
    int32_t hidden_dim;          /* 64 */
    int32_t replay_capacity;     /* 10000 */
    int32_t n_warmup_steps;      /* 100 */
    int32_t episode_step_limit;  /* 200 */
    float adam_epsilon;          /* 1e-7 (the loop's TENSORFLOW defaults) */
} rlt_oracle_sac_loop_config;

typedef struct rlt_oracle_sac_loop rlt_oracle_sac_loop;

rlt_oracle_sac_loop* rlt_oracle_sac_loop_create(const rlt_oracle_sac_loop_config* config);
void rlt_oracle_sac_loop_destroy(rlt_oracle_sac_loop* loop);
int rlt_oracle_sac_loop_step(rlt_oracle_sac_loop* loop);

/* Views into the loop's state; pointers stay valid until destroy. */
const rlt_sac_agent* rlt_oracle_sac_loop_agent(rlt_oracle_sac_loop* loop);
const rlt_replay_buffer* rlt_oracle_sac_loop_replay(rlt_oracle_sac_loop* loop);
const rlt_pendulum_runner* rlt_oracle_sac_loop_runner(rlt_oracle_sac_loop* loop);
const float* rlt_oracle_sac_loop_noise_critic(rlt_oracle_sac_loop* loop);   /* [batch x 1] of the last step */
const float* rlt_oracle_sac_loop_noise_actor(rlt_oracle_sac_loop* loop);
const uint32_t* rlt_oracle_sac_loop_env_indices(rlt_oracle_sac_loop* loop);  /* draws of the last gather */
const uint32_t* rlt_oracle_sac_loop_sample_offsets(rlt_oracle_sac_loop* loop);
uint32_t rlt_oracle_sac_loop_step_count(rlt_oracle_sac_loop* loop);
float rlt_oracle_sac_loop_critic_loss(rlt_oracle_sac_loop* loop, int critic_index);
/* {reset happened, initial theta, initial theta_dot, rollout noise, action taken, episode return} of the last env step */
void rlt_oracle_sac_loop_last_env_step(rlt_oracle_sac_loop* loop, float* out6);
size_t rlt_oracle_sac_loop_parameter_count(rlt_oracle_sac_loop* loop);
/* flat order: actor, critic 0, critic 1, target 0, target 1, log_alpha; per network per layer [weights, biases] */
void rlt_oracle_sac_loop_get_parameters(rlt_oracle_sac_loop* loop, float* out);

#ifdef __cplusplus
}
#endif
#endif
