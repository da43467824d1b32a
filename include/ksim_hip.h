/* ksim_hip.h — C ABI of libksimhip.so: the MI355X (gfx950) rollout hot path of ksim.
 *
 * Every entry point is asynchronous on the caller's HIP stream, allocates nothing,
 * never synchronises the host, keeps no mutable global state (re-entrant) and
 * returns 0 on success or a negative KS_E* code; ks_last_error() gives the
 * calling thread's last message.  All pointers are DEVICE pointers unless a
 * parameter says "host".  The caller owns every buffer.
 *
 * Each declaration cites the reference (kscalelabs/ksim 0.2.10) interface it
 * replaces as file:line.
 */
#ifndef KSIM_HIP_H_
#define KSIM_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* ks_stream_t; /* a hipStream_t; NULL = the default stream */

enum {
  KS_OK = 0,
  KS_EINVAL = -1,  /* bad size / flag / null pointer */
  KS_ELAUNCH = -2, /* HIP reported a launch error */
  KS_ELIMIT = -3   /* size beyond a compiled-in maximum */
};

/* Library identity / error text (host). */
const char* ks_version(void);
const char* ks_last_error(void);

/* ------------------------------------------------------------------ GAE / returns
 * Replaces compute_ppo_inputs, ksim/task/ppo.py:54-121.
 * Layout "bt": arrays are (B, T) row-major like the reference's *_bt arguments;
 * one wavefront scans one env row with shuffles (segmented reverse scan).
 * Layout "tn": arrays are (T, N) time-major with env fastest (the rollout
 * buffer's own layout); one lane walks one env back in time.
 *   values, rewards : f32     dones, successes : 1 byte per element, non-zero = true
 *   successes may be NULL (treated as all false).
 *   gae, returns, targets : f32 outputs (targets = returns when monte_carlo_returns
 *   else gae + values, ppo.py:107).  Any output may be NULL.
 */
int ks_gae_bt(ks_stream_t stream, int64_t B, int64_t T, const float* values, const float* rewards,
              const uint8_t* dones, const uint8_t* successes, float gamma, float lam,
              int monte_carlo_returns, float* gae, float* returns, float* targets);
int ks_gae_tn(ks_stream_t stream, int64_t T, int64_t N, const float* values, const float* rewards,
              const uint8_t* dones, const uint8_t* successes, float gamma, float lam,
              int monte_carlo_returns, float* gae, float* returns, float* targets);

/* Advantage normalisation over ALL n elements, population std clipped at 1e-6
 * (ppo.py:116-119).  workspace: >= KS_REDUCE_WORKSPACE_BYTES bytes of device memory. */
#define KS_REDUCE_WORKSPACE_BYTES (2 * 1024 * 8 + 64)
int ks_normalize_advantages(ks_stream_t stream, int64_t n, const float* gae, float* advantages,
                            void* workspace);

/* ------------------------------------------------------------------ PPO loss
 * Replaces compute_ppo_loss + clipped_value_loss (ppo.py:124-135,149-246) and the
 * total "mean over (B,T) of the summed terms" (ppo.py:473-486).
 *   n = B*T elements, A = action dims; log-probs / entropy are (n, A) row-major.
 *   entropy may be NULL (term omitted, ppo.py:237-239).
 *   policy/value/kl/entropy_loss: per-element outputs (n), each may be NULL.
 *   loss_out: one f32 (device), may be NULL.  workspace as above.
 */
typedef struct KsPpoLossParams {
  float clip_param;      /* ppo.py:259 default 0.2 */
  float value_loss_coef; /* 0.5 */
  float entropy_coef;    /* 0.008 */
  float kl_coef;         /* 1e-3 */
  float log_clip_value;  /* 5.0 */
  float kl_scale;        /* adaptive-KL runtime factor, ppo.py:475; 1.0 */
  int32_t use_clipped_value_loss; /* 1 */
} KsPpoLossParams;
int ks_ppo_loss(ks_stream_t stream, int64_t n, int32_t A, const KsPpoLossParams* params /*host*/,
                const float* advantages, const float* value_targets, const float* on_log_probs,
                const float* on_values, const float* off_log_probs, const float* off_values,
                const float* off_entropy, float* policy_loss, float* value_loss, float* kl_loss,
                float* entropy_loss, float* loss_out, void* workspace);

/* ------------------------------------------------------------------ reward total + done/success
 * Replaces the scale/sum/clip of get_rewards (ksim/task/rl.py:219-239) and the
 * ternary -> boolean combination of terminations (rl.py:1049-1050).
 *   components: (K, n) f32, scales: K host floats (sign already folded for *Penalty).
 *   use_clip_min/max: 0 = no clip.  total: (n) f32, may be NULL.
 *   terminations: (k, n) int8 in {-1,0,+1}; done/success: (n) uint8; pass k = 0 to skip.
 */
#define KS_MAX_REWARD_TERMS 32
int ks_reward_total(ks_stream_t stream, int64_t n, int32_t K, const float* components,
                    const float* scales /*host*/, int32_t use_clip_min, float clip_min,
                    int32_t use_clip_max, float clip_max, float* total, int32_t k,
                    const int8_t* terminations, uint8_t* done, uint8_t* success);

/* ------------------------------------------------------------------ physics model
 * Replaces the mjx.Model produced by ksim/utils/mujoco.py:388-391 (mjx.put_model) for the
 * model subset of the rollout configs: a kinematic tree whose bodies (depth-first order,
 * body 0 = world) each carry one free or hinge joint, motor actuators (one per dof at
 * most) and contact spheres against the ground plane z = 0 with pyramidal friction cones.
 * ks_model_create copies the description to the current HIP device (the only call that
 * allocates); the handle is immutable afterwards.
 */
#define KS_MAX_BODIES 32
#define KS_MAX_QPOS 40
#define KS_MAX_DOFS 32
#define KS_MAX_ACTUATORS 32
#define KS_MAX_SPHERES 16
enum { KS_JNT_NONE = 0, KS_JNT_FREE = 1, KS_JNT_HINGE = 2 };

typedef struct KsModelDesc {
  int32_t nb, nq, nv, nu, ns;
  int32_t iterations, ls_iterations; /* Newton / line-search limits (ksim/task/rl.py:717-748 sets opt.*) */
  int32_t eulerdamp;                 /* must be 0: ksim disables EULERDAMP (rl.py:575-578,745-746) */
  double dt, gravity[3], tolerance, ls_tolerance, impratio, meaninertia, friction;
  double solref[2], solimp[5];
  int32_t body_parent[KS_MAX_BODIES], body_jtype[KS_MAX_BODIES], body_qadr[KS_MAX_BODIES],
      body_dofadr[KS_MAX_BODIES], body_subtree_end[KS_MAX_BODIES];
  double body_pos[KS_MAX_BODIES][3], body_quat[KS_MAX_BODIES][4], body_mass[KS_MAX_BODIES],
      body_ipos[KS_MAX_BODIES][3], body_iquat[KS_MAX_BODIES][4], body_inertia[KS_MAX_BODIES][3],
      jnt_axis[KS_MAX_BODIES][3], jnt_pos[KS_MAX_BODIES][3], body_invweight0[KS_MAX_BODIES];
  double qpos0[KS_MAX_QPOS];
  int32_t dof_body[KS_MAX_DOFS], dof_parent[KS_MAX_DOFS];
  double dof_damping[KS_MAX_DOFS], dof_armature[KS_MAX_DOFS];
  int32_t act_dof[KS_MAX_ACTUATORS];
  double act_gear[KS_MAX_ACTUATORS], act_lo[KS_MAX_ACTUATORS], act_hi[KS_MAX_ACTUATORS];
  int32_t sph_body[KS_MAX_SPHERES];
  double sph_pos[KS_MAX_SPHERES][3], sph_radius[KS_MAX_SPHERES];
} KsModelDesc;

typedef struct KsModel KsModel;
int ks_model_create(const KsModelDesc* desc /*host*/, KsModel** out);
int ks_model_destroy(KsModel* model);
int ks_model_lds_bytes(const KsModel* model); /* LDS one env needs in the step kernel */

/* ------------------------------------------------------------------ control step / forward
 * ks_step replaces MjxEngine.step (ksim/engine.py:259-361): `substeps` physics steps of
 * mjx.step (engine.py:257) with the latency blend (287-288), the actuator update every
 * `actuator_period` substeps (290-318) and last_ctrl <- action (355), for N envs at once
 * (the reference vmaps the per-env call, ksim/task/rl.py:1615).
 * ks_forward replaces the mjx.forward of MjxEngine.reset (engine.py:213): derived fields
 * and the warm start for the given qpos/qvel/ctrl_in, without integrating.
 *
 * All arrays are env-major rows: (N, dim) f32, like the reference's vmapped pytrees.
 * Nullable inputs fall back to: latency 0, zero_offset 0, no drops, scales 1, no noise,
 * no bias, model friction, mass scale 1.  Noise arrays are explicit pre-sampled draws,
 * (substeps, N, nu), so that results can be compared on identical seeded inputs.
 */
enum { KS_ACT_TORQUE = 0, KS_ACT_POSITION = 1 }; /* actuators.py:70-87 / 98-238 */

typedef struct KsStepIO {
  int64_t N;
  int32_t substeps;        /* EngineData.phys_steps_per_ctrl_steps, engine.py:150 */
  int32_t actuator_period; /* EngineData.phys_steps_per_actuator_step, engine.py:151 */
  int32_t actuator_type;
  float action_scale;      /* PositionActuators.action_scale, actuators.py:107 */
  /* state, in/out */
  float* qpos;             /* (N, nq) */
  float* qvel;             /* (N, nv) */
  float* qacc_warmstart;   /* (N, nv) */
  float* time;             /* (N) nullable */
  float* last_ctrl;        /* (N, nu) PhysicsState.last_ctrl, ksim/types.py:33-43 */
  /* inputs */
  const float* action;      /* (N, nu) */
  const float* ctrl_in;     /* (N, nu) ks_forward only: data.ctrl; nullable = 0 */
  const float* latency;     /* (N) PhysicsState.action_latency in substeps */
  const float* zero_offset; /* (N, nu) */
  const uint8_t* drop;      /* (N, nu) drop_action mask, engine.py:277-278 */
  const float* kp;          /* (nu) */
  const float* kd;          /* (nu) */
  const float* ctrl_clip;   /* (nu), +inf = unlimited */
  const float* kp_scale;    /* (N) ActuatorState, actuators.py:90-95 */
  const float* kd_scale;    /* (N) */
  const float* torque_limit_scale; /* (N) */
  const float* action_bias; /* (N, nu) */
  const float* torque_bias; /* (N, nu) */
  const float* action_noise; /* (substeps, N, nu) */
  const float* torque_noise; /* (substeps, N, nu) */
  const float* friction;    /* (N) per-env contact friction (FloorFrictionRandomizer, randomization.py:74-104) */
  const float* mass_scale;  /* (N, nb) per-env body mass factor (randomization.py:207-222) */
  /* outputs, each nullable */
  float* qacc;              /* (N, nv) of the last substep */
  float* ctrl_out;          /* (N, nu) torques applied in the last substep = data.ctrl */
  float* xpos;              /* (N, nb*3) body positions at the start of the last substep */
  float* xquat;             /* (N, nb*4) */
  float* cvel;              /* (N, nb*6) com-based body velocities [angular; linear] */
  int32_t* solver_niter;    /* (N) Newton iterations of the last substep */
  int32_t* nefc;            /* (N) active constraint rows of the last substep */
  /* intermediate quantities for parity tests, each nullable */
  float* dbg_M;             /* (N, nv*nv) */
  float* dbg_bias;          /* (N, nv) */
  float* dbg_qacc_smooth;   /* (N, nv) */
  float* dbg_con_dist;      /* (N, ns) */
} KsStepIO;

int ks_step(const KsModel* model, ks_stream_t stream, const KsStepIO* io /*host*/);
int ks_forward(const KsModel* model, ks_stream_t stream, const KsStepIO* io /*host*/);

#ifdef __cplusplus
}
#endif
#endif /* KSIM_HIP_H_ */
