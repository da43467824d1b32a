// Kernel argument block of the fused control-step kernel (device pointers, passed by value).
#pragma once
#include <stdint.h>

#include "../../include/ksim_hip.h"

namespace ks {

struct DevModel;

struct StepArgs {
  const DevModel* model;
  int64_t N;
  int substeps, actuator_period, actuator_type;
  float action_scale;
  float *qpos, *qvel, *qacc_warmstart, *time, *last_ctrl;
  const float *action, *ctrl_in, *latency, *zero_offset;
  const uint8_t* drop;
  const float *kp, *kd, *ctrl_clip, *kp_scale, *kd_scale, *torque_limit_scale;
  const float *action_bias, *torque_bias, *action_noise, *torque_noise;
  const float *friction, *mass_scale;
  const uint8_t* env_mask;
  const uint8_t* fresh;
  float *qacc, *ctrl_out, *xpos, *xquat, *cvel, *traj_ctrl, *traj_xpos, *traj_xquat;
  int32_t *solver_niter, *nefc;
  float *dbg_M, *dbg_bias, *dbg_qacc_smooth, *contact_dist, *cinert, *cfrc_ext;
  const float *armature_scale, *damping_scale;
  const float *frictionloss, *body_ipos, *body_inertia, *sph_pos, *sph_radius;
  const int32_t* env_order;
  int32_t* work;
  int n_events;
  KsEventDesc events[KS_MAX_EVENTS];
  float* event_state;
  const float* event_uniform;
  KsRng event_rng;
  float* event_force;
  int n_force_events;
};

}  // namespace ks
