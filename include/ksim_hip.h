/* ksim_hip.h — C ABI of libksimhip.so: the MI355X (gfx950) rollout hot path of ksim.
 *
 * Compute entry points are asynchronous on the caller's HIP stream, allocate nothing,
 * never synchronise the host, keep no mutable global state (re-entrant) and
 * return 0 on success or a negative KS_E* code; ks_last_error() gives the
 * calling thread's last message.  All pointers are DEVICE pointers unless a
 * parameter says "host".  The caller owns every buffer.
 *
 * The set-up calls are the exception, and the only ones that allocate device memory
 * and block the host (uploads, one stream synchronisation in ks_mlp_train_init):
 *   ks_model_create, ks_terms_create, ks_mlp_create, ks_gru_create, ks_lstm_create   (tables and weights of a handle)
 *   ks_mlp_train_init, ks_gru_train_init, ks_lstm_train_init   (master weights, gradients, Adam moments, transposes)
 * Their memory belongs to the handle and is released by the matching *_destroy; a set-up call that fails releases
 * what it had allocated.  Call them outside graph capture and outside timed loops.  Gradients and optimiser state
 * live in the handle, so two streams must not train one handle at once.
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
/* sizeof() of a public struct as this library was compiled, for binding self-checks:
 * 0 KsPpoLossParams, 1 KsModelDesc, 2 KsStepIO, 3 KsTermsDesc, 4 KsObserveIO, 5 KsTerminateIO, 6 KsMlpDesc,
 * 7 KsRewardIO, 8 KsObsElem, 9 KsTermDesc, 10 KsRewardDesc, 11 KsRng, 12 KsAdamParams, 13 KsEventDesc,
 * 14 KsRewardScanIO, 15 KsRewardScanDesc, 16 KsGruDesc, 17 KsLstmDesc, 18 KsGaussianHead, 19 KsCommandIO,
 * 20 KsMixtureHead, 21 KsNoiseStage, 22 KsRandomVar;
 * -1 for anything else. */
int64_t ks_abi_sizeof(int32_t which);

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
/* The same result with no workspace argument and no allocation of any kind.  No counterpart in the reference: it is for
 * callers that cannot allocate device memory (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  The block partials live in a device array of KS_REDUCE_WORKSPACE_BYTES bytes inside the library, one copy
 * per GPU, held until the process ends; n above KS_NORMALIZE_STATIC_MAX_N is rejected with KS_ELIMIT.  All calls on one
 * GPU share that array: calls that overlap on one GPU (two streams, two threads) race; calls on one stream do not. */
#define KS_NORMALIZE_STATIC_MAX_N ((int64_t)1 << 28)
int ks_normalize_advantages_static(ks_stream_t stream, int64_t n, const float* gae, float* advantages);

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
  const float* kl_scale_device; /* when not NULL: a device float read in place of kl_scale (see ks_ppo_adapt_kl) */
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
  int32_t eulerdamp;                 /* 1: the velocity update is implicit in joint damping, (M + dt diag(damping)) a = M qacc.
                                        That is MuJoCo's Euler step with EULERDAMP and also, for models whose smooth forces
                                        depend on velocity only through joint damping (torque motors), its implicitfast
                                        integrator, which ksim selects (rl.py:555-578,730-748).  0: plain semi-implicit Euler */
  int32_t condim;                    /* contact dimension of every sphere-floor contact: 3 (0 means 3) = friction pyramid, four
                                        rows per contact; 1 = frictionless, one normal row regularised with the body's
                                        translational inverse weight (MuJoCo condim, as examples/data/scene.mjcf:19,72 uses) */
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
  /* Joint limits of hinges, by body (MuJoCo jnt_limited / jnt_range; the real K-Bot limits every joint,
   * examples/kbot/robot/kbot-headless/robot.mjcf:66-217), and dry joint friction (dof_frictionloss, robot.mjcf:5-18).
   * A violated limit is one constraint row J = +-e_j, friction one row J = e_j whose force saturates at
   * +-frictionloss; both are regularised with dof_invweight0[j], the diagonal of the inverse mass matrix at qpos0,
   * and use dof_solref / dof_solimp (MuJoCo's per-joint solreflimit, solimplimit, solreffriction, solimpfriction, one
   * pair for all of them here; all zero = the contacts' solref / solimp).  Everything zero: neither limits nor friction. */
  int32_t jnt_limited[KS_MAX_BODIES];
  double jnt_range[KS_MAX_BODIES][2], dof_invweight0[KS_MAX_DOFS], dof_frictionloss[KS_MAX_DOFS];
  double dof_solref[2], dof_solimp[5];
  double dof_stiffness[KS_MAX_DOFS]; /* joint springs of hinges about qpos0 (MuJoCo jnt_stiffness, springref = qpos0;
                                        examples/data/scene.mjcf:43-66): passive force -stiffness (q - qpos0) */
} KsModelDesc;

typedef struct KsModel KsModel;
int ks_model_create(const KsModelDesc* desc /*host*/, KsModel** out);
int ks_model_destroy(KsModel* model);
int ks_model_lds_bytes(const KsModel* model); /* LDS one env needs in the step kernel */

/* Random draws: every entry point that needs randomness takes either explicit pre-sampled
 * buffers (so both sides of a parity test see identical draws) or, when they are NULL, a
 * counter-based Philox-4x32-10 stream keyed by (seed, env, step, purpose). */
typedef struct KsRng {
  uint64_t seed;
  uint64_t step;
  const uint64_t* step_base; /* device, nullable: added to `step` when the kernel runs, so that a captured
                                HIP graph of a rollout draws fresh numbers on every replay */
} KsRng;

/* Velocity events inside the substep loop (ksim/events.py:58-237, called per physics step at
 * ksim/engine.py:322-333): every substep the time remaining of an event is decremented by dt; when it reaches
 * zero the root velocity gets an impulse and a new interval is drawn.
 *   linear push : qvel[0:3] += (cos t, sin t, 0) * (lo + u1 (hi - lo)) * mag * level_scale, t = 2 pi u0
 *   angular push: qvel[5]   += +-(lo + u1 (hi - lo)) * mag * level_scale, minus when u0 < 0.5
 *   jump        : qvel[0:3] += sqrt(2 * -gravity * (lo + u0 (hi - lo)) * level_scale)
 *   all         : time remaining = interval_lo + u2 (interval_hi - interval_lo)
 * The force push (ForcePushEvent, events.py:240-365) holds a Cartesian force and torque on one body, applied at
 * its centre of mass in the world frame like MuJoCo's xfrc_applied, for a drawn duration.  Per env it carries,
 * besides the time remaining, KS_EVENT_FORCE_STATE floats: [force duration left, force(3), torque(3), unused].
 * Every substep: both timers lose dt; the stored wrench is multiplied by level_scale (events.py:296 rescales the
 * carried value itself); while the duration is positive the body receives stored * level_scale (events.py:297-299);
 * when the interval runs out a new wrench is drawn (events.py:320-358):
 *   force  = dir(u0,u1,u2) * s * mag,  torque = dir(u4,u5,u6) * s * mag2,  dir(.) = unit vector of 2u - 1,
 *   s = lo + u3 (hi - lo);  case floor(3 u7): 0 force only, 1 torque only, 2 both;
 *   time remaining = interval_lo + u8 (interval_hi - interval_lo);  duration = duration_lo + u9 (duration_hi - duration_lo).
 * As in the reference, each force push first clears the applied forces of all bodies, so with several of them only
 * the last one in the list acts. */
#define KS_MAX_EVENTS 4
#define KS_EVENT_DRAWS 12      /* uniforms per (substep, env, event) in an explicit draw buffer */
#define KS_EVENT_FORCE_STATE 8 /* floats per (event, env) of force-push state */
enum { KS_EVENT_LINEAR_PUSH = 0, KS_EVENT_ANGULAR_PUSH = 1, KS_EVENT_JUMP = 2, KS_EVENT_FORCE_PUSH = 3 };
typedef struct KsEventDesc {
  int32_t kind;
  float mag;          /* linvel | angvel | unused | max_force */
  float lo, hi;       /* vel_range | jump_height_range | force_range */
  float interval_lo, interval_hi;
  float level_scale;  /* event.scale.get_scale(curriculum_level) */
  float mag2;         /* force push: max_torque */
  float duration_lo, duration_hi; /* force push: duration_range */
  int32_t body;       /* force push: body index (0 = world) */
} KsEventDesc;

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
enum { KS_ACT_TORQUE = 0, KS_ACT_POSITION = 1, /* actuators.py:70-87 / 98-238 */
       KS_ACT_POSITION_VELOCITY = 2 /* actuators.py:241-293: the action is (position targets, velocity targets), 2 nu wide;
                                       tau = kp (target_pos - q) + kd (target_vel - qd), noise, clipped.  action, last_ctrl,
                                       drop and action_noise are then 2 nu wide (the second half of action_noise is the
                                       velocity-target noise) */ };

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
  const uint8_t* env_mask;  /* (N) nullable: envs with 0 are skipped entirely (reset-under-cond, rl.py:1072-1080) */
  /* outputs, each nullable */
  float* qacc;              /* (N, nv) of the last substep */
  float* ctrl_out;          /* (N, nu) torques applied in the last substep = data.ctrl */
  float* xpos;              /* (N, nb*3) body positions at the start of the last substep */
  float* xquat;             /* (N, nb*4) */
  float* cvel;              /* (N, nb*6) com-based body velocities [angular; linear] */
  float* traj_ctrl;         /* (N, nu)   second copies of ctrl_out / xpos / xquat for the transition record */
  float* traj_xpos;         /* (N, nb*3) (Trajectory.ctrl/xpos/xquat, ksim/task/rl.py:1054-1070) */
  float* traj_xquat;        /* (N, nb*4) */
  int32_t* solver_niter;    /* (N) Newton iterations of the last substep */
  int32_t* nefc;            /* (N) active constraint rows of the last substep */
  /* intermediate quantities for parity tests, each nullable */
  float* dbg_M;             /* (N, nv*nv) */
  float* dbg_bias;          /* (N, nv) */
  float* dbg_qacc_smooth;   /* (N, nv) */
  float* contact_dist;      /* (N, ns) signed distance sphere - floor of the last substep's collision pass (negative =
                               touching): the data.contact.dist that contact observations read (ksim/utils/mujoco.py:175-217) */
  float* cinert;            /* (N, nb*10) com-based body inertias of the last substep, mjData.cinert's layout: the six
                               entries of the symmetric inertia about the tree's centre of mass (xx yy zz xy xz yz), mass times
                               the offset of the body's centre (3), mass (ksim/observation.py:285-290); nullable */
  float* cfrc_ext;          /* (N, nb*6) contact force on each body of the last substep as a spatial force about the tree's
                               centre of mass, world axes, torque then force: mjData.cfrc_ext, which the feet force / torque
                               observations read (ksim/observation.py:563-616); nullable */
  /* more per-env model parameters (inputs, nullable = 1): factors on the joints' armature and damping
     (ArmatureRandomizer, JointDampingRandomizer, ksim/randomization.py:108-123,226-243; the root's six dofs keep 1) */
  const float* armature_scale; /* (N, nv) */
  const float* damping_scale;  /* (N, nv) */
  /* per-env replacements of model fields (inputs, nullable = the model's own values): dry joint friction
     (StaticFrictionRandomizer, randomization.py:56-71), centres of mass (COMRandomizer, AllBodiesCOMRandomizer, 290-356),
     principal inertias (AllBodiesInertiaRandomizer, 359-383, together with mass_scale), and the contact spheres
     (CollisionBodyRandomizer, 386-487: a jittered capsule is two jittered spheres).  frictionloss selects the kernel
     variant with dof-lane rows even for a model without dry friction of its own. */
  const float* frictionloss;   /* (N, nv) */
  const float* body_ipos;      /* (N, nb*3) */
  const float* body_inertia;   /* (N, nb*3) */
  const float* sph_pos;        /* (N, ns*3); with sph_radius */
  const float* sph_radius;     /* (N, ns) */
  /* launch order (no counterpart in the reference: its vmapped solver runs all envs in lock step).  Envs differ a lot in
     cost (contacts, Newton iterations), and with only a few wavefronts per hardware slot the launch ends with the last heavy
     env.  `work` returns an estimate of each env's cost in this step; ks_work_order turns it into a heaviest-first
     permutation that the next step takes as `env_order`, so the heavy envs start first and the light ones fill the gaps.
     Results do not depend on the order. */
  const int32_t* env_order;    /* (N) a permutation of 0..N-1: workgroup i steps env env_order[i]; nullable = the natural order
                                  dealt to the XCDs in contiguous eighths (workgroup i steps env (i % 8) (N / 8) + i / 8 when
                                  N is a multiple of 8) */
  int32_t* work;               /* (N) nullable */
  /* events (ks_step only) */
  int32_t n_events;
  KsEventDesc events[KS_MAX_EVENTS];
  float* event_state;          /* (n_events, N) time remaining, in/out */
  const float* event_uniform;  /* (substeps, N, n_events, KS_EVENT_DRAWS) U[0,1) draws, nullable -> Philox */
  KsRng event_rng;
  float* event_force;          /* (n_events, N, KS_EVENT_FORCE_STATE) in/out; required when a force push is listed */
  /* ks_step only, nullable: envs flagged here were reset by the termination pass and still owe the forward pass of
     MjxEngine.reset (engine.py:213: mjx.forward on the reset state, whose solution becomes the new episode's warm
     start).  The step runs that pass for them first, inside the same launch, with zero controls and without integrating;
     what it leaves in qacc_warmstart is what a masked ks_forward before the step would have left.  The derived outputs of
     the reset state itself (xpos, xquat ...) are not written: a caller whose terms read those runs ks_forward instead. */
  const uint8_t* fresh;        /* (N) */
} KsStepIO;

int ks_step(const KsModel* model, ks_stream_t stream, const KsStepIO* io /*host*/);
/* order = the envs sorted by work, heaviest first (counting sort over buckets of four work units; ties in arbitrary order).  When N is a multiple of 8 (and at
 * least 512) the sort runs inside the eight regions [r N / 8, (r + 1) N / 8) and region r's envs go to order[r], order[r + 8],
 * ...: workgroup b of the step launch runs on XCD b % 8, so every XCD then steps one contiguous eighth of the env arrays,
 * heaviest first, and the 128-byte lines that neighbouring envs' rows share stay in one L2. */
int ks_work_order(ks_stream_t stream, int64_t N, const int32_t* work, int32_t* order);
int ks_forward(const KsModel* model, ks_stream_t stream, const KsStepIO* io /*host*/);

/* ------------------------------------------------------------------ per-env terms
 * One spec holds the compiled tables of the task's observations, terminations and
 * resets; ks_terms_create copies it to the device (allocates), after which
 * ks_observe / ks_terminate_reset / ks_sample_action allocate nothing.
 *
 * Observations (replaces get_observation + Observation.observe/add_noise,
 * ksim/task/rl.py:153-186, ksim/observation.py:89-145,184-257,300-352,705-713): every
 * element k of the concatenated observation vector is described by one KsObsElem.
 */
enum { /* KsObsElem.src: which per-env array the element reads, all (N, dim) f32 */
  KS_SRC_QPOS = 0, KS_SRC_QVEL = 1, KS_SRC_QACC = 2, KS_SRC_CTRL = 3, KS_SRC_LAST_ACTION = 4,
  KS_SRC_COMMAND = 5, KS_SRC_TIME = 6, KS_SRC_XPOS = 7, KS_SRC_XQUAT = 8, KS_SRC_CVEL = 9,
  KS_SRC_CONST = 10, KS_SRC_CONTACT_DIST = 11 /* (N, ns) KsStepIO.contact_dist */,
  KS_SRC_CINERT = 12 /* (N, nb*10) KsStepIO.cinert */,
  KS_SRC_CFRC_EXT = 13 /* (N, nb*6) KsStepIO.cfrc_ext */, KS_SRC_COUNT = 14
};
enum { /* KsObsElem.kind */
  KS_OBS_COPY = 0,      /* src[index]                                  (observation.py:185-195,254-257,300-303,343-352) */
  KS_OBS_JOINT_POS = 1, /* qpos[index] - zero_offset[index - 7]        (observation.py:220-225) */
  KS_OBS_ROT_INV = 2,   /* component `comp` of q^-1 v q, q = qpos[3:7], v = src[index..index+2] or (c0,c1,c2)
                           (in_robot_frame velocities, observation.py:198-217; gravity in the body frame) */
  KS_OBS_CONTACT = 3,   /* 1 when src[index] < 0 else 0: geoms_colliding of one sphere with the floor
                           (observation.py:481-521, utils/mujoco.py:175-217) */
  KS_OBS_DELAYED = 4,   /* the value `comp` control steps ago (observation.py:228-252,260-283): the element owns the
                           column carry[carry + d * stride], d = 0..comp-1, oldest first; it emits slot 0 (minus
                           zero_offset when src is qpos), shifts the column down and appends src[index].  A fresh
                           episode fills the column with the current value. */
  KS_OBS_GRAVITY_EMA = 5, /* component `comp` of the lagged, biased gravity reading (observation.py:355-442):
                           p = R(euler bias) (q^-1 (c0,c1,c2) q), x <- x lag + p (1 - lag), emits x.
                           carry[carry .. carry+6] = x(3), lag, bias(3); a fresh episode sets x = 0,
                           lag ~ U(q0, q1), bias ~ U(-q2, q2)^3 from four draws. */
  KS_OBS_SITE_GYRO = 6,  /* component `comp` of a gyro at a site of body `index` (MuJoCo's gyro sensor, which
                           SensorObservation reads from sensordata, observation.py:307-340): the body's angular velocity in
                           the site frame, (q_body q_site)^-1 w, with q_body = xquat[index], w = cvel[index][0:3] (both of
                           the last substep's forward pass, as sensordata is) and q_site = (e0, e1, e2, e3) */
  KS_OBS_SITE_ACCEL = 7, /* component `comp` of an accelerometer at a site of the floating base (body `index`, the one the
                           free joint moves): the site's acceleration minus gravity in the site frame,
                           (q_body q_site)^-1 (qacc[0:3] + alpha x r + w x (w x r) - g), alpha = R_body qacc[3:6],
                           r = R_body (c0, c1, c2), g = (q0, q1, q2), q_site = (e0, e1, e2, e3) */
  KS_OBS_SITE_ROT6D = 8, /* entry `comp` (0..5) of the 6-D rotation of a site of body `index` (SiteOrientationObservation,
                           observation.py:645-669): the first two rows of R(q_body q_site), row-major */
  KS_OBS_CONTACT_ANY = 9, /* 1 when any contact sphere whose bit is set in `index` touches the floor: the floor's own entry of
                           ContactObservation (observation.py:452-478), whose geom list holds the floor and some spheres */
  /* MuJoCo's framepos / framequat / magnetometer sensors of a site of body `index` (read by SensorObservation like the
     two above): component `comp` of xpos[index] + R_body (c0, c1, c2); component `comp` (0..3) of q_body q_site; component
     `comp` of (q_body q_site)^-1 (q0, q1, q2), the model's magnetic field in the site frame.  (frameangvel needs no kind: it
     is cvel[index][0:3], a KS_OBS_COPY.) */
  KS_OBS_SITE_POS = 10, KS_OBS_SITE_QUAT = 11, KS_OBS_SITE_MAGNETOMETER = 12
};
/* Site kinds with env_site = 1 read the site's pose per env from KsObserveIO.site_pose instead of (e0..e3) and (c0, c1, c2):
 * the IMU mounting error of IMUAlignmentRandomizer (ksim/randomization.py:245-284) is a model field there, one per env. */
/* Noise and bias of an observation (ksim/noise.py:129-229, applied by Observation.add_noise, ksim/observation.py:110-142:
 * first the noise, then the per-episode bias).  A stage draws rv = mean + level (scale z + scale2 w) with z ~ N(0,1),
 * w ~ U(-1,1) (Gaussian kinds: scale = std; uniform kinds: scale2 = mag; the uniform-Gaussian kinds of
 * UniformGaussianRandomVariable, noise.py:106-121, use both) and adds it to the observation or multiplies the observation
 * by it.  ChainedNoise (noise.py:222-229) applies several stages with ONE key: all stages of an element see the same z and w.
 * One key also ties w to z inside a stage: jax.random builds a normal draw as sqrt(2) erfinv of the uniform the same bits
 * give, so w = erf(z / sqrt 2).  The in-kernel Philox stream draws z and derives w that way; explicit noise_normal /
 * noise_uniform buffers are taken as they are (a caller comparing with the reference passes a consistent pair). */
enum { KS_NOISE_NONE = 0, KS_NOISE_ADD_GAUSSIAN = 1, KS_NOISE_ADD_UNIFORM = 2, KS_NOISE_MUL_GAUSSIAN = 3,
       KS_NOISE_MUL_UNIFORM = 4, KS_NOISE_ADD_UNIFORM_GAUSSIAN = 5, KS_NOISE_MUL_UNIFORM_GAUSSIAN = 6 };
#define KS_MAX_NOISE_CHAIN 4
typedef struct KsNoiseStage {
  int32_t kind;
  float mean, scale, scale2; /* scale: std (Gaussian kinds) or mag (uniform kinds); scale2: mag of the uniform-Gaussian kinds */
} KsNoiseStage;
typedef struct KsObsElem {
  int32_t kind, src, index, comp;
  float c0, c1, c2;
  int32_t n_noise;               /* stages in use, 0 = no noise */
  KsNoiseStage noise[KS_MAX_NOISE_CHAIN];
  KsNoiseStage bias;             /* per-episode bias (KS_NOISE_NONE: none): the same kinds, evaluated every step from the env's
                                    stored standard draw (KsObserveIO.bias_draw) at the current curriculum level, which is what
                                    re-drawing with the episode's key gives (observation.py:136-141, ksim/task/rl.py:263-271) */
  int32_t carry, stride;         /* stateful kinds: offset into the env's carry row, distance between delay slots */
  float q0, q1, q2;              /* KS_OBS_GRAVITY_EMA: min_lag, max_lag, imu_bias; KS_OBS_SITE_ACCEL: gravity; KS_OBS_SITE_MAGNETOMETER: field */
  float e0, e1, e2, e3;          /* site kinds: the site's orientation in its body, wxyz */
  int32_t env_site;              /* site kinds: 1 = take the site's pose from KsObserveIO.site_pose */
} KsObsElem;

/* Terminations (replaces get_terminations + terms, rl.py:288-299, ksim/terminations.py:60-192). */
enum { KS_TERM_MIN_HEIGHT = 0, KS_TERM_BAD_Z = 1, KS_TERM_NOT_UPRIGHT = 2, KS_TERM_BAD_VELOCITY = 3,
       KS_TERM_FAR_FROM_ORIGIN = 4, KS_TERM_EPISODE_LENGTH = 5,
       KS_TERM_ILLEGAL_CONTACT = 6 /* a listed contact sphere is deeper than contact_eps into the floor: some
                                      contact_dist[s] < p0 with bit s of the sphere mask (int)p1 set (terminations.py:84-99) */ };
typedef struct KsTermDesc {
  int32_t kind;
  int32_t value; /* what a firing term reports: -1 or +1 */
  float p0, p1, p2, p3; /* min_height | min_z,max_z,final_min_z,final_max_z | max_radians | max_vel | max_dist | max_sec,disable_level(<0: never) */
} KsTermDesc;

/* Resets (replaces the Reset list applied in MjxEngine.reset, engine.py:207-220, ksim/resets.py:44-189,
 * 284-354): qpos[i] <- clip(start[i] + u*mag[i]*(level if by_level[i]), lo[i], hi[i]) with u ~ U(-1,1) and
 * start[i] = base[i], or for elements marked reset_from_motion the reference-motion frame drawn for the env plus base[i]
 * (InitialMotionStateReset, resets.py:284-306; time <- frame * ctrl_dt then, otherwise 0);
 * reset_hfield: z <- hfield[ix, iy] + base[2] with the cell looked up from the new x, y (HFieldXYPositionReset, resets.py:45-90);
 * then the base orientation: quat <- quat * yaw(U(-pi,pi)) (RandomHeadingReset, resets.py:309-320) and
 * quat <- quat * euler(roll, pitch, 0) with roll and pitch from ONE uniform draw mapped to their ranges, as one key
 * gives them (RandomPitchRollReset, resets.py:338-354), in the order reset_pitch_roll says;
 * qvel, warm start and last_ctrl <- 0. */
#define KS_MAX_OBS 512
#define KS_MAX_TERMS 16
typedef struct KsTermsDesc {
  int32_t nq, nv, nu, nb;
  int32_t obs_dim, n_terms, command_dim, random_heading;
  int32_t ns;        /* contact spheres of the model (width of KS_SRC_CONTACT_DIST) */
  int32_t carry_dim; /* floats of observation carry per env (0: no stateful observation) */
  int32_t action_dim; /* width of the action vector = of last_ctrl and of KS_SRC_LAST_ACTION; 0 means nu
                         (2 nu for position-velocity actuators) */
  int32_t nonfinite_terminates; /* 1: an env whose qpos/qvel is not finite counts as failed (done, no success);
                                   the reference has no such guard and would carry the NaNs forever */
  KsObsElem obs[KS_MAX_OBS];
  KsTermDesc terms[KS_MAX_TERMS];
  float reset_base[KS_MAX_QPOS], reset_mag[KS_MAX_QPOS], reset_lo[KS_MAX_QPOS], reset_hi[KS_MAX_QPOS];
  int32_t reset_by_level[KS_MAX_QPOS];
  int32_t reset_from_motion[KS_MAX_QPOS]; /* 1: start from the reference-motion frame (KsTerminateIO.reset_motion_qpos) */
  int32_t reset_pitch_roll;               /* 0 none, 1 applied after the heading, 2 applied before it */
  float reset_pitch[2], reset_roll[2];    /* (min, max) in radians */
  int32_t reset_hfield;                   /* 1: base height from the height field (KsTerminateIO.reset_hfield) */
  float hfield_bound[2];                  /* half extents (x, y) of the height field */
} KsTermsDesc;
typedef struct KsTerms KsTerms;
int ks_terms_create(const KsTermsDesc* desc /*host*/, KsTerms** out);
int ks_terms_destroy(KsTerms* terms);

typedef struct KsObserveIO {
  int64_t N;
  float level;               /* curriculum level */
  const float* src[KS_SRC_COUNT]; /* indexed by KS_SRC_*; an unused source may be NULL */
  const float* zero_offset;  /* (N, nu) nullable */
  float* bias_draw;          /* (N, obs_dim, 2) in/out: the episode's standard draws (z, w) behind each element's bias; required
                                when an element has a bias.  Envs flagged in `fresh` get new ones first (the reference re-keys
                                the biases of an env that was reset, ksim/task/rl.py:1110-1117) */
  const float* bias_redraw;  /* (N, obs_dim, 2) the (z, w) that fresh envs take, nullable -> Philox */
  const float* noise_normal; /* (N, obs_dim) standard normal draws, nullable -> Philox */
  const float* noise_uniform;/* (N, obs_dim) U[0,1) draws, nullable -> Philox */
  KsRng rng;
  float* obs;                /* (N, obs_dim) clean, nullable */
  float* noisy_obs;          /* (N, obs_dim) noisy copy, nullable (rl.py:181-184) */
  /* stateful observations (rl.py:166-176: observe_stateful with the carry of the previous control step) */
  float* carry;               /* (N, carry_dim) in/out; required when carry_dim > 0 */
  const uint8_t* fresh;       /* (N) nullable: non-zero = the env starts an episode, its carries are initialised from the
                                 current state before observing (initial_carry, rl.py:1034-1080) and its bias draws are
                                 renewed; NULL = none */
  const float* carry_uniform; /* (N, carry_dim) U[0,1) draws for the initial carries, nullable -> Philox */
  const float* site_pose;     /* (N, 7) per-env orientation (wxyz) and position of the randomised site in its body; required
                                 when an element has env_site set */
} KsObserveIO;
int ks_observe(const KsTerms* terms, ks_stream_t stream, const KsObserveIO* io /*host*/);

/* A random variable of ksim/noise.py:50-121 as parameters: value = mean + s (std z + mag w), z ~ N(0,1), w ~ U(-1,1),
 * s = the curriculum level where the reference passes one, else 1.  same_key: both parts come from one key
 * (UniformGaussianRandomVariable, noise.py:106-121), so w = erf(z / sqrt 2) as described at KsNoiseStage. */
typedef struct KsRandomVar {
  float mean, mag, std;
  int32_t same_key;
} KsRandomVar;

/* Terminations, trajectory record and reset predication for the post-step state
 * (replaces RLTask._get_step_env_state, rl.py:1023-1136, for the physics part):
 * writes done/success/components and the transition copies, then overwrites the state of
 * finished envs with a fresh episode.  reset_mask marks them for a following ks_forward. */
typedef struct KsTerminateIO {
  int64_t N;
  float level;
  float* qpos; float* qvel; float* qacc_warmstart; float* time; float* last_ctrl; /* state, in/out */
  int8_t* components;        /* (n_terms, N) int8 in {-1,0,1}, nullable */
  uint8_t* done; uint8_t* success; /* (N) */
  float* traj_qpos; float* traj_qvel; float* traj_time; /* transition copies of the pre-reset state, nullable */
  uint8_t* reset_mask;       /* (N) = done, nullable */
  int32_t* episode_length;   /* (N) control steps in the current episode, in/out, nullable */
  const float* reset_uniform; /* (N, nq + 1) U(-1,1) draws (last one: heading), nullable -> Philox */
  const float* reset_pitch_roll_uniform; /* (N) U[0,1) draws of RandomPitchRollReset, nullable -> Philox */
  const float* reset_motion_qpos;  /* (reset_motion_frames, nq) reference motion, required when the table marks elements */
  int32_t reset_motion_frames;
  float reset_motion_dt;           /* ctrl_dt of the motion: time <- frame * dt */
  const int32_t* reset_frame;      /* (N) frame per env, nullable -> floor(U[0,1) * frames) from Philox */
  const float* reset_hfield;       /* (hfield_nx, hfield_ny) heights, required when reset_hfield is set */
  int32_t hfield_nx, hfield_ny;
  KsRng rng;
  int32_t apply_reset;       /* 0: report terminations only; 1: reset finished envs; 2: reset every env (initial reset) */
  /* event timers of the envs that start a fresh episode: a new interval each (engine.py:226-232) */
  int32_t n_events;
  float event_interval[KS_MAX_EVENTS][2];
  float* event_state;               /* (n_events, N), nullable when n_events == 0 */
  const float* event_reset_uniform; /* (N, n_events) U[0,1) draws, nullable -> Philox */
  float* event_force;               /* (n_events, N, KS_EVENT_FORCE_STATE), nullable: zeroed for the reset envs */
  const float* contact_dist;        /* (N, ns) KsStepIO.contact_dist of the step just taken; KS_TERM_ILLEGAL_CONTACT only */
  /* Per-episode quantities of the envs that start a fresh episode, re-drawn like MjxEngine.reset does under cond(done)
   * (ksim/engine.py:222-245, ksim/task/rl.py:1072-1080).  Every buffer is nullable = left alone. */
  float* action_latency;            /* (N) <- U(latency_lo level, latency_hi level), in physics steps (engine.py:233-237) */
  float latency_lo, latency_hi;
  float* zero_offset;               /* (N, nu) <- zero_offset_rv at the curriculum level (engine.py:238-242) */
  KsRandomVar zero_offset_rv;
  /* ActuatorState of PositionActuators.get_initial_state (ksim/actuators.py:219-238), drawn at level 1 */
  float* act_action_bias;           /* (N, nu) */
  float* act_torque_bias;           /* (N, nu) */
  float* act_kp_scale;              /* (N) */
  float* act_kd_scale;              /* (N) */
  float* act_torque_limit_scale;    /* (N) */
  KsRandomVar action_bias_rv, torque_bias_rv, kp_scale_rv, kd_scale_rv, torque_limit_scale_rv;
  /* explicit draws, (N, 3 nu + 4) each, nullable -> Philox; columns: latency, zero offset (nu), action bias (nu),
   * torque bias (nu), kp scale, kd scale, torque limit scale */
  const float* episode_uniform;     /* U(-1,1); the latency takes lo + (u + 1) / 2 (hi - lo) */
  const float* episode_normal;      /* N(0,1) */
} KsTerminateIO;
int ks_terminate_reset(const KsTerms* terms, ks_stream_t stream, const KsTerminateIO* io /*host*/);
/* ks_terminate_reset of control step t and ks_observe of step t + 1 in one launch (the tail of step_engine followed by the
 * head of the next one, ksim/task/rl.py:1049-1080 then 1164-1176 / 153-186): a workgroup takes the decisions for its envs,
 * resets the finished ones and observes the same envs in the state the next step starts from.  oio->fresh, when given, must
 * be tio->reset_mask (the observation's episode starts are what this call's first half decides); the observation's random
 * numbers are keyed by oio->rng, which the caller sets to the next step's.  Same results as the two calls in a row. */
int ks_terminate_reset_observe(const KsTerms* terms, ks_stream_t stream, const KsTerminateIO* tio /*host*/,
                               const KsObserveIO* oio /*host*/);

/* Commands (replaces get_commands / get_initial_commands, ksim/task/rl.py:302-332, called per control step at
 * rl.py:1082-1098, for the velocity commands of the shipped tasks, ksim/commands.py:281-391,451-507).  The env's command
 * vector is the concatenation of the commands' values:
 *   linear velocity : vel, yaw, xvel, yvel, target_vel, target_yaw     angular velocity : vel, target_vel
 *   constant        : `dim` floats that are left alone
 * Per step and command, in this order: an env that starts an episode (fresh) draws its initial command from its
 * (reset) state: targets at random, current values measured (base speed and heading in the robot frame; yaw rate).
 * Otherwise, with probability switch_prob new targets are drawn and the current values stay; else the current
 * values move towards the targets by at most accel * ctrl_dt.  Draws u0..: linear = target speed, target yaw, zero,
 * backward, switch; angular = target speed, flip, zero, switch. */
#define KS_MAX_COMMANDS 8
#define KS_COMMAND_DRAWS 20
#define KS_MAX_VECTOR_COMMAND 16
enum { KS_CMD_CONST = 0, KS_CMD_LINEAR_VELOCITY = 1, KS_CMD_ANGULAR_VELOCITY = 2,
       /* FloatVectorCommand / IntVectorCommand (commands.py:97-170): `dim` <= KS_MAX_VECTOR_COMMAND scalars, each uniform in
          [lo, hi] (integers: lo..hi inclusive), all zero with probability zero_prob; redrawn at an episode start and with
          probability switch_prob per step, otherwise kept.  Draws: u0 switch, u1 zero, u2.. one per scalar. */
       KS_CMD_FLOAT_VECTOR = 3, KS_CMD_INT_VECTOR = 4,
       /* StartPositionCommand / StartQuaternionCommand (commands.py:173-215): qpos[0:3] / qpos[3:7] of the state an episode
          starts from, kept until the next start (dim 3 / 4). */
       KS_CMD_START_POSITION = 5, KS_CMD_START_QUATERNION = 6,
       /* BaseHeightCommand (commands.py:773-796): a height uniform in [lo[0], hi[0]] at an episode start; afterwards one draw
          u0 decides both: replaced by lo + u0 (hi - lo) when u0 < switch_prob (the reference passes one key to both its
          uniform and its Bernoulli draw, so the two are the same number). */
       KS_CMD_BASE_HEIGHT = 7,
       /* SinusoidalGaitCommand (commands.py:696-770): moving flag, phase, then one target foot height per foot (dim = 2 + feet,
          feet <= KS_MAX_VECTOR_COMMAND).  lo[0..4] = gait_period, max_height, height_offset, stance_ratio, moving_threshold.
          Start: flag 1, phase 0.  Step: phase <- (phase + ctrl_dt / gait_period) mod 1 while the flag is set, else 0; when
          |qvel[0:2]| <= moving_threshold the flag and the phase drop to 0 (the flag stays down until the next start).
          Foot f at phase p_f = (phase + f / feet) mod 1 gets height_offset + max_height sin(pi (p_f - stance) / (1 - stance))
          in swing (p_f >= stance), height_offset in stance. */
       KS_CMD_SINUSOIDAL_GAIT = 8,
       /* JointPositionCommand (commands.py:821-914): n = (dim - 3) / 2 <= KS_MAX_VECTOR_COMMAND joints; the value is the
          reference's JointPositionCommandValue flattened: start (n), target (n), total_time, num_steps, step_id.  At an
          episode start: target_j uniform in [lo[j], hi[j]] (u_j), start_j = qpos[7 + joints[j]], total_time uniform in
          [min_time, max_time] (u_n), num_steps = ceil(total_time / ctrl_dt), step_id = 0.  Afterwards step_id += 1, and once
          step_id > num_steps a new value is drawn the same way from the current state. */
       KS_CMD_JOINT_POSITION = 9,
       /* CartesianCoordinateCommand (commands.py:537-694): current (3), target (3), speed (dim 7).  lo / hi [0..2] = the box
          (already scaled by the curriculum level), min_vel / max_vel = the speed range, ctrl_dt = the command's dt.  At an
          episode start target = current = a point of the box (u0..u2) and speed uniform (u3).  Afterwards, with
          d = |target - current|: when (d < dt speed / 2 and u4 < switch_prob) or u4 < jump_prob (one draw decides both) a
          new target and speed are drawn; then current moves towards the target by min(speed dt, d) with d the distance to
          the OLD target (commands.py:640-653). */
       KS_CMD_CARTESIAN_COORDINATE = 10 };
typedef struct KsCommandDesc {
  int32_t kind, index, dim;    /* offset and length inside the command vector */
  float min_vel, max_vel, max_yaw, zero_prob, backward_prob, switch_prob; /* scales already evaluated at the curriculum level */
  float ctrl_dt, linear_accel, angular_accel;
  float lo[KS_MAX_VECTOR_COMMAND], hi[KS_MAX_VECTOR_COMMAND]; /* vector commands: the ranges */
  int32_t joints[KS_MAX_VECTOR_COMMAND]; /* joint position command: actuated-joint indices (qpos[7 + j]) */
  float min_time, max_time;              /* joint position command: range of the time to reach a target */
  float jump_prob;                       /* cartesian command */
} KsCommandDesc;
typedef struct KsCommandIO {
  int64_t N;
  int32_t command_dim, n_commands, nq, nv;
  KsCommandDesc commands[KS_MAX_COMMANDS];
  float* command;            /* (N, command_dim) in/out */
  float* traj_command;       /* (N, command_dim) nullable: receives the incoming commands, i.e. the ones the step that is
                                being recorded was taken under (Trajectory.command, rl.py:1113-1128) */
  const float* qpos;         /* (N, nq) */
  const float* qvel;         /* (N, nv) */
  const uint8_t* fresh;      /* (N) nullable: envs that start an episode */
  int32_t all_fresh;         /* 1: every env draws an initial command (first step of a task) */
  const float* uniform;      /* (N, n_commands, KS_COMMAND_DRAWS) U[0,1) draws, nullable -> Philox */
  KsRng rng;
} KsCommandIO;
int ks_commands(ks_stream_t stream, const KsCommandIO* io /*host*/);

/* Action post-processing (replaces the sampling tail of RLTask._sample_action, rl.py:998-1001):
 * action = mean + std * noise, NaN -> 0, clip to +-clip_max.  log_std (nu) nullable = deterministic. */
int ks_sample_action(ks_stream_t stream, int64_t N, int32_t nu, const float* mean, const float* log_std,
                     const float* noise_normal /*(N,nu) nullable -> Philox*/, KsRng rng, float clip_max,
                     float* action);

/* The same tail for a network that also emits the standard deviation (examples/kbot/train.py:915-932): raw is
 * (N, 2 nu) = means then raw deviations; mean = raw_mean + mean_bias, std = min((softplus(raw_std) + min_std) * var_scale,
 * max_std), action = mean + std * noise.  Optionally returns mean, std and the per-dimension log-probability of the sample
 * before the NaN scrub and clip, which is what the task stores as the old policy's log-probability.  The example's low-pass
 * filter on the mean and its command-dependent bias are task code and stay outside. */
typedef struct KsGaussianHead {
  float min_std, max_std, var_scale;
  int32_t deterministic;   /* 1: action = mean (argmax_action) */
  const float* mean_bias;  /* device (nu), nullable */
} KsGaussianHead;
int ks_sample_action_head(ks_stream_t stream, int64_t N, int32_t nu, const float* raw /*(N, 2 nu)*/,
                          const KsGaussianHead* head /*host*/, const float* noise_normal /*(N,nu) nullable -> Philox*/,
                          KsRng rng, float clip_max, float* action /*(N,nu)*/, float* mean_out /*nullable*/,
                          float* std_out /*nullable*/, float* log_prob_out /*(N,nu) nullable*/);

/* Action filters between the network output and the sampled action (ksim/actions.py:31-257): small per-env recursions on
 * the target positions, whose state is part of the model carry and restarts with the episode.
 *   KS_FILTER_LOWPASS               y = y_last + alpha (x - y_last), alpha = dt / (1 / (2 pi p0) + dt)   (actions.py:248-257)
 *   KS_FILTER_CLIP_ACCELERATION     v = (x - pos) / dt, a = clip((v - vel) / dt, +-p0), vel += a dt, pos += vel dt (54-80)
 *   KS_FILTER_INTEGRATE_VELOCITY    pos += x dt                                                          (108-133)
 *   KS_FILTER_INTEGRATE_ACCELERATION vel = clip(vel + x dt, +-p0), pos += vel dt                         (162-191)
 *   KS_FILTER_CLIP_POSITIONS        y = clip(x, lo, hi)                                                  (194-214)
 *   KS_FILTER_TANH_POSITIONS        y = tanh(x) (hi - lo) + lo                                           (217-241)
 * state is (N, 2 nu) = position-like part | velocity-like part (the low-pass keeps y_last in the first half); y is the
 * filter's output (the new position-like part for the stateful kinds).  Envs flagged in fresh restart from init (N, nu),
 * or from zero, with zero velocity, before the step is applied. */
enum { KS_FILTER_LOWPASS = 0, KS_FILTER_CLIP_ACCELERATION = 1, KS_FILTER_INTEGRATE_VELOCITY = 2,
       KS_FILTER_INTEGRATE_ACCELERATION = 3, KS_FILTER_CLIP_POSITIONS = 4, KS_FILTER_TANH_POSITIONS = 5 };
int ks_action_filter(ks_stream_t stream, int64_t N, int32_t nu, int32_t kind, float ctrl_dt, float p0,
                     const float* lo /*(nu) device, range kinds*/, const float* hi, const float* x /*(N,nu)*/,
                     float* state /*(N, 2 nu) in-out, stateful kinds*/, const uint8_t* fresh /*(N) nullable*/,
                     const float* init /*(N,nu) nullable*/, float* y /*(N,nu)*/);

/* Mixture-of-Gaussians head of the walking example's actor (examples/walking.py:127-144): raw is (N, 3 nu K) = component
 * means (nu, K), raw deviations (nu, K), logits (nu, K) per env.  mean = clip(raw_mean + mean_bias, clip_lo, clip_hi)
 * (zero bias and ClipPositions, walking.py:138-142), std = min((softplus(raw_std) + min_std) * var_scale, max_std).  Per
 * action dimension one component is drawn from softmax(logits) with the uniform draw u (first k whose cumulative
 * probability exceeds u), then action = mean_k + std_k * z; log_prob = logsumexp_k(log softmax(logits)_k + log N(action;
 * mean_k, std_k)) of the sample before the NaN scrub and clip.  deterministic: the mean of the most probable component.
 * The distribution itself (xax.MixtureOfGaussians) is a third-party class that is not part of the reference tree; this
 * is the textbook mixture. */
#define KS_MAX_MIXTURES 16
typedef struct KsMixtureHead {
  int32_t num_mixtures;   /* K in 1..KS_MAX_MIXTURES */
  float min_std, max_std, var_scale;
  int32_t deterministic;
  const float* mean_bias; /* device (nu), nullable */
  const float* clip_lo;   /* device (nu), nullable (then clip_hi must be NULL too) */
  const float* clip_hi;
} KsMixtureHead;
int ks_sample_action_mixture(ks_stream_t stream, int64_t N, int32_t nu, const float* raw /*(N, 3 nu K)*/,
                             const KsMixtureHead* head /*host*/, const float* uniform /*(N,nu) nullable -> Philox*/,
                             const float* noise_normal /*(N,nu) nullable -> Philox*/, KsRng rng, float clip_max,
                             float* action /*(N,nu)*/, float* log_prob_out /*(N,nu) nullable*/,
                             int32_t* component_out /*(N,nu) nullable*/);

/* ------------------------------------------------------------------ policy / critic / discriminator MLP
 * The dense contraction of the path: the network a task's sample_action calls
 * (ksim/task/rl.py:892-926,986-996; plain MLP stacks as in examples/walking.py:40-208's
 * heads) and the AMP discriminator forward (ksim/task/amp.py:327-358).
 * y = W_L act(... act(W_1 x + b_1) ...) + b_L, weights (out, in) row-major like the
 * reference's linear layers.  KS_MLP_BF16 rounds weights and activations to bf16 and
 * accumulates in fp32 on the matrix cores; KS_MLP_F32 keeps fp32 throughout.
 * ks_mlp_create uploads (allocates); ks_mlp_forward allocates nothing: the caller
 * provides ks_mlp_workspace_bytes(mlp, M) bytes of device scratch.
 */
#define KS_MAX_LAYERS 8
enum { KS_ACT_NONE = 0, KS_ACT_ELU = 1, KS_ACT_RELU = 2, KS_ACT_TANH = 3,
       KS_ACT_GELU = 4 /* tanh form, jax.nn.gelu's default (examples/walking.py:103) */ };
enum { KS_MLP_F32 = 0, KS_MLP_BF16 = 1 };
typedef struct KsMlpDesc {
  int32_t n_layers;
  int32_t dims[KS_MAX_LAYERS + 1];  /* in, hidden..., out */
  int32_t activation;               /* applied after every layer but the last */
  int32_t dtype;
  const float* weights[KS_MAX_LAYERS]; /* host, (dims[l+1], dims[l]) */
  const float* biases[KS_MAX_LAYERS];  /* host, (dims[l+1]) */
} KsMlpDesc;
typedef struct KsMlp KsMlp;
int ks_mlp_create(const KsMlpDesc* desc /*host*/, KsMlp** out);
int ks_mlp_destroy(KsMlp* mlp);
int64_t ks_mlp_workspace_bytes(const KsMlp* mlp, int64_t M);
int ks_mlp_forward(const KsMlp* mlp, ks_stream_t stream, int64_t M, const float* x /*(M, in)*/,
                   float* y /*(M, out)*/, void* workspace);
/* Two networks over the same M rows, e.g. the actor on the noisy observations and the critic on the clean ones
 * (ksim/task/rl.py:892-926 and the value call of examples/walking.py:626-638, which XLA schedules side by side).  Same
 * results as two ks_mlp_forward calls; when both networks run as whole-network kernels with one activation and M is
 * below 16384 they share a single launch, so the second network's workgroups overlap the first one's. */
int ks_mlp_forward_pair(const KsMlp* mlp0, const KsMlp* mlp1, ks_stream_t stream, int64_t M, const float* x0,
                        float* y0, const float* x1, float* y1, void* workspace0, void* workspace1);

/* ------------------------------------------------------------------ GRU cell (recurrent policies, forward)
 * The recurrent actors / critics of the shipped examples (examples/walking.py:40-208: input projection, a stack of
 * eqx.nn.GRUCell, output MLP) step once per control step inside the rollout (ksim/task/rl.py:892-926).  One cell:
 *   gi = W_ih x + bias, gh = W_hh h;  r = sigmoid(gi_r + gh_r), z = sigmoid(gi_z + gh_z),
 *   n = tanh(gi_n + r (gh_n + bias_n)),  h' = n + z (h - n)        (gate order r | z | n along the 3H rows)
 * `fresh` marks envs that start an episode: their carry is taken as zero (get_initial_model_carry after a reset,
 * rl.py:1072-1080).  h_out may alias h_in.  Forward only: backpropagation through time is not built. */
typedef struct KsGruDesc {
  int32_t input_size, hidden_size, dtype; /* dtype: KS_MLP_F32 | KS_MLP_BF16 for the two projections */
  const float* weight_ih; /* host (3H, input_size) */
  const float* weight_hh; /* host (3H, H) */
  const float* bias;      /* host (3H), nullable */
  const float* bias_n;    /* host (H), nullable */
} KsGruDesc;
typedef struct KsGru KsGru;
int ks_gru_create(const KsGruDesc* desc /*host*/, KsGru** out);
int ks_gru_destroy(KsGru* gru);
int64_t ks_gru_workspace_bytes(const KsGru* gru, int64_t M);
int ks_gru_forward(const KsGru* gru, ks_stream_t stream, int64_t M, const float* x /*(M, input_size)*/,
                   const float* h_in /*(M, H)*/, const uint8_t* fresh /*(M) nullable*/, float* h_out /*(M, H)*/,
                   void* workspace);

/* LSTM cell (eqx.nn.LSTMCell, the recurrent layer of examples/kbot/train.py:837-995): g = W_ih x + W_hh h + bias with the
 * 4H rows in gate order input | forget | cell | output; c' = sigmoid(f) c + sigmoid(i) tanh(g), h' = sigmoid(o) tanh(c').
 * Envs marked fresh start from h = c = 0.  h_out / c_out may alias h_in / c_in.  Forward only. */
typedef struct KsLstmDesc {
  int32_t input_size, hidden_size, dtype;
  const float* weight_ih; /* host (4H, input_size) */
  const float* weight_hh; /* host (4H, H) */
  const float* bias;      /* host (4H), nullable */
} KsLstmDesc;
typedef struct KsLstm KsLstm;
int ks_lstm_create(const KsLstmDesc* desc /*host*/, KsLstm** out);
int ks_lstm_destroy(KsLstm* lstm);
int64_t ks_lstm_workspace_bytes(const KsLstm* lstm, int64_t M);
int ks_lstm_forward(const KsLstm* lstm, ks_stream_t stream, int64_t M, const float* x /*(M, input_size)*/,
                    const float* h_in /*(M, H)*/, const float* c_in /*(M, H)*/, const uint8_t* fresh /*(M) nullable*/,
                    float* h_out, float* c_out, void* workspace);

/* ------------------------------------------------------------------ policy update: gradients and optimiser
 * The native pieces of PPOTask._single_step / update_model (ksim/task/ppo.py:495-565, 572-694) for an
 * MLP actor / critic with a Gaussian head: the backward pass that jax.grad performs through
 * _get_ppo_loss_and_metrics (ppo.py:412-492) and the optax chain of the examples' get_optimizer
 * (examples/walking.py:373-387: zero_nans, clip_by_global_norm, add_decayed_weights, scale_by_adam,
 * learning rate, -1).  ks_mlp_train_init keeps fp32 master weights, gradients and Adam moments beside
 * the working-precision copies that ks_mlp_forward reads; after ks_mlp_adam_step every copy is refreshed.
 *   ks_mlp_train_forward  y = net(x), hidden activations kept in `workspace` for the backward pass
 *   ks_mlp_train_backward gradients of sum(dy * y) w.r.t. every weight and bias, into the handle.  It follows the
 *                         ks_mlp_train_forward of the same rows on the same workspace, whose contents (and layout: large
 *                         bf16 batches keep their activations transposed for a one-launch backward pass) belong to the pair
 *   ks_grad_sqnorm        adds the squared norm of n floats (NaNs skipped) to *acc (device double)
 *   ks_mlp_grad_sqnorm    the same over all gradients of a network
 *   ks_mlp_adam_step      one optimiser step with `sqnorm` = squared global gradient norm over everything
 *                         that is optimised together (NULL or max_grad_norm <= 0: no clipping)
 *   ks_adam_step          the same chain on a bare parameter vector (e.g. the log standard deviations) */
typedef struct KsAdamParams {
  float lr, b1, b2, eps, weight_decay, max_grad_norm;
  int64_t step; /* 1 for the first update (bias correction) */
} KsAdamParams;
int ks_mlp_train_init(KsMlp* mlp);
int64_t ks_mlp_train_workspace_bytes(const KsMlp* mlp, int64_t M);
int ks_mlp_train_forward(KsMlp* mlp, ks_stream_t stream, int64_t M, const float* x, float* y, void* workspace);
int ks_mlp_train_backward(KsMlp* mlp, ks_stream_t stream, int64_t M, const float* x, const float* dy /*(M, out)*/,
                          void* workspace);
/* ks_mlp_train_backward that also returns dx (M, in), the gradient with respect to the network input (added to dx when
 * accumulate_dx, rows flagged in zero_rows written as zero); weight_gradients = 0 skips the weight and bias gradients
 * (then x may be NULL).  For a one-layer network no preceding ks_mlp_train_forward is needed. */
int ks_mlp_train_backward_dx(KsMlp* mlp, ks_stream_t stream, int64_t M, const float* x, const float* dy, float* dx,
                             int32_t weight_gradients, int32_t accumulate_dx, const uint8_t* zero_rows /*(M) nullable*/,
                             void* workspace);
/* The first `count` bias entries of a layer are constants: the optimiser and the gradient norm skip them. */
int ks_mlp_freeze_bias_prefix(KsMlp* mlp, int32_t layer, int32_t count);

/* ksim/task/amp.py:360-438 (get_disc_losses, _grad_penalty, _get_amp_disc_loss_and_metrics): gradient of the AMP
 * discriminator's loss
 *   0.5 sum (D(real) - 1)^2 + 0.5 sum (D(sim) + 1)^2 + grad_penalty_coef / 2 * mean_motions sum_frames |dD/dx (real frame)|^2
 * with respect to every weight and bias of the discriminator, an MLP with one output applied to each frame (ELU, ReLU, tanh or
 * no activation), into the handle's gradient buffers (then ks_mlp_grad_sqnorm / ks_mlp_adam_step as for any network).
 * real (n_real, in) holds n_motions reference motions of n_real / n_motions frames each, sim (n_sim, in) the frames of
 * the simulated trajectories.  losses[3] (device) receives the real, simulated and penalty terms.  Computed in fp32 on the
 * master weights whatever the network's working precision. */
int64_t ks_mlp_disc_workspace_bytes(const KsMlp* mlp, int64_t n_real, int64_t n_sim);
int ks_mlp_disc_loss_grad(KsMlp* mlp, ks_stream_t stream, int64_t n_real, const float* real, int64_t n_sim, const float* sim,
                          float grad_penalty_coef, int64_t n_motions, float* losses, void* workspace);
int ks_grad_sqnorm(ks_stream_t stream, int64_t n, const float* g, double* acc);
/* Mirror (left / right symmetry) losses of a task, examples/kbot/train.py:1458-1477, for networks applied to flat rows.
 * A mirror map is a signed permutation: mirrored[j] = sign[j] * x[perm[j]] (mirror_joints / mirror_obs / mirror_cmd,
 * train.py:1565-1760, each negate and reorder entries of their vector).
 *   ks_signed_permute     out[r][j] = sign[j] * x[r][perm[j]]: the mirrored rows that the networks see
 *   ks_mirror_loss_grad   with y (rows, n) the network's output on the rows and ym (rows, n) its output on the mirrored
 *                         rows:  loss[r] = scale * mean_j (y[r][j] - sign[j] ym[r][perm[j]])^2  (train.py:1466-1469; for
 *                         a critic n = 1, perm = {0}, sign = {1}: scale * (v - vm)^2, train.py:1477), and the gradient of
 *                         mean_r loss[r] is ADDED to dy and WRITTEN to dym.  perm must be a permutation of 0..n-1.
 * The loss joins the PPO loss as an auxiliary term (ksim/task/ppo.py:241-244, 485-486: mean over rows of the sum of terms). */
/* The low-pass filter on the actor's means inside the loss of the K-Bot task: run_actor filters the biased means with
 * ksim.lowpass_one_pole (examples/kbot/train.py:923-929, ksim/actions.py:248-257) and the filter state `lpf_params` is part
 * of the model carry that the scan over the trajectory threads through time and restarts with the episode
 * (train.py:1439-1451, 1506-1515, 1529-1533).
 *   ks_lowpass_scan           rows (t, m) of ld floats; the first nu columns are the means:
 *                             y_t = y_{t-1} + alpha (x_t + mean_bias + add_t - y_{t-1}), alpha = dt / (1 / (2 pi cutoff) + dt),
 *                             y_{-1} = y0[m] (NULL: zero), and y_{t-1} = 0 at the steps flagged in fresh (T, M).  `add`
 *                             (nullable) is the command-dependent bias read from the observation rows (train.py:920-921):
 *                             add[(t M + m) add_ld + k] joins joint add_first + k, k < add_count.  Columns nu..ld-1 are
 *                             copied (x == y is allowed and filters in place).  y_last (M, nu), nullable, receives the carry
 *                             after the last step.  With T = 1 this is the rollout's own filter step.
 *   ks_lowpass_scan_backward  the reverse sweep jax.grad derives through that scan: g holds dL/dy in its first nu columns
 *                             on entry and dL/dx on return (G_t = g_t + (1 - alpha) G_{t+1}, cut where step t + 1 is
 *                             fresh; dx_t = alpha G_t); d_y0 (M, nu), nullable, receives the gradient of the initial carry. */
int ks_lowpass_scan(ks_stream_t stream, int64_t T, int64_t M, int32_t nu, int32_t ld, float ctrl_dt, float cutoff,
                    const float* x, const float* mean_bias /*(nu) nullable*/, const float* add /*nullable*/, int64_t add_ld,
                    int32_t add_first, int32_t add_count, const float* y0 /*(M,nu) nullable*/,
                    const uint8_t* fresh /*(T,M) nullable*/, float* y, float* y_last /*(M,nu) nullable*/);
int ks_lowpass_scan_backward(ks_stream_t stream, int64_t T, int64_t M, int32_t nu, int32_t ld, float ctrl_dt, float cutoff,
                             const uint8_t* fresh /*(T,M) nullable*/, float* g /*(T,M,ld) in place*/, float* d_y0 /*nullable*/);
int ks_signed_permute(ks_stream_t stream, int64_t rows, int32_t n, const float* x, const int32_t* perm, const float* sign,
                      float* out);
int ks_mirror_loss_grad(ks_stream_t stream, int64_t rows, int32_t n, float scale, const float* y, const float* ym,
                        const int32_t* perm, const float* sign, float* dy, float* dym, float* loss /*(rows), nullable*/);
/* ksim/task/ppo.py:546-563 (adaptive KL in _single_step), without a trip to the host: with
 * kl_mean = mean_rows(sum_a(on_log_probs - log_probs)) * kl_coef * *kl_scale, the coefficient kl_coef * *kl_scale is
 * multiplied by 1.5 when kl_mean > 1.5 desired_kl, divided by 1.5 when kl_mean < desired_kl / 1.5, clipped to
 * [1e-8, 1e2], and *kl_scale (device, in/out) becomes that coefficient / kl_coef.  The next ks_ppo_loss_grad reads it
 * through KsPpoLossParams.kl_scale_device.  workspace: 256 floats (device).  Sums in a fixed order. */
int ks_ppo_adapt_kl(ks_stream_t stream, int64_t rows, int32_t A, const float* on_log_probs, const float* log_probs,
                    float kl_coef, float desired_kl, float* kl_scale, float* workspace);
int ks_mlp_grad_sqnorm(const KsMlp* mlp, ks_stream_t stream, double* acc);
int ks_mlp_adam_step(KsMlp* mlp, ks_stream_t stream, const KsAdamParams* params /*host*/, const double* sqnorm);
int ks_adam_step(ks_stream_t stream, int64_t n, float* param, const float* grad, float* m1, float* m2,
                 const KsAdamParams* params /*host*/, const double* sqnorm);
/* Copies of the parameters and gradients in the caller's (out, in) layout, for checks and checkpoints. */
int ks_mlp_get_params(const KsMlp* mlp, ks_stream_t stream, int32_t layer, float* weight /*(out,in) dev*/, float* bias /*(out) dev*/,
                      int32_t gradients /*0: parameters, 1: gradients*/);

/* Backward pass through time of a GRU stack (the jax.grad through the lax.scan over the trajectory in
 * PPOTask._single_step, ksim/task/ppo.py:572-694, for the recurrent actors and critics of examples/walking.py:40-208).
 * Forward over the trajectory with ks_gru_train_forward, which keeps per step saved (M, 5H) = r | z | n | hn | h.  Then per
 * step, last to first, ks_gru_backward_step takes dh_out (M, H) = gradient from the layer above at that step + dh_in of
 * the step after it, and returns d_gi, d_gh (M, 3H), the gradients of the two projections' outputs, and dh_in (M, H), the
 * gradient of the step's incoming hidden state (zero for an env that started an episode there).  With d_gi, d_gh and
 * saved[..., 4H:] stacked over all steps, one ks_mlp_train_backward_dx per projection (ks_gru_projections hands them
 * out) yields the weight gradients and the gradient of the layer's inputs.  ks_gru_adam_step updates both. */
int ks_gru_train_init(KsGru* gru);
int ks_gru_projections(KsGru* gru, KsMlp** input_projection, KsMlp** hidden_projection);
int ks_gru_train_forward(const KsGru* gru, ks_stream_t stream, int64_t M, const float* x, const float* h_in,
                         const uint8_t* fresh, float* h_out, float* saved /*(M, 5H)*/, void* workspace /*ks_gru_workspace_bytes*/);
int64_t ks_gru_backward_workspace_bytes(const KsGru* gru, int64_t M);
int ks_gru_backward_step(KsGru* gru, ks_stream_t stream, int64_t M, const float* dh_out, const float* saved,
                         const uint8_t* fresh, float* d_gi, float* d_gh, float* dh_in, void* workspace);
int ks_gru_grad_sqnorm(const KsGru* gru, ks_stream_t stream, double* acc);
int ks_gru_adam_step(KsGru* gru, ks_stream_t stream, const KsAdamParams* params /*host*/, const double* sqnorm);
/* The same for LSTM stacks (the recurrent actor and critic of examples/kbot/train.py:903-915): saved is (M, 7H) =
 * i | f | g | o | tanh(c') | c | h; a step takes dh_out and dc_out and returns d_g (M, 4H), the gradient of both
 * projections' outputs, with dh_in and dc_in. */
int ks_lstm_train_init(KsLstm* lstm);
int ks_lstm_projections(KsLstm* lstm, KsMlp** input_projection, KsMlp** hidden_projection);
int ks_lstm_train_forward(const KsLstm* lstm, ks_stream_t stream, int64_t M, const float* x, const float* h_in,
                          const float* c_in, const uint8_t* fresh, float* h_out, float* c_out, float* saved /*(M, 7H)*/,
                          void* workspace /*ks_lstm_workspace_bytes*/);
int64_t ks_lstm_backward_workspace_bytes(const KsLstm* lstm, int64_t M);
int ks_lstm_backward_step(KsLstm* lstm, ks_stream_t stream, int64_t M, const float* dh_out, const float* dc_out,
                          const float* saved, const uint8_t* fresh, float* d_g, float* dh_in, float* dc_in, void* workspace);
int ks_lstm_grad_sqnorm(const KsLstm* lstm, ks_stream_t stream, double* acc);
int ks_lstm_adam_step(KsLstm* lstm, ks_stream_t stream, const KsAdamParams* params /*host*/, const double* sqnorm);
/* A whole trajectory of one LSTM layer in one launch each way: the lax.scan over the T steps of the trajectory inside the loss
 * (ksim/task/ppo.py:572-694 around the model's forward, examples/kbot/train.py:903-915) and what jax.grad derives for it, for
 * fp32 cells of hidden size 128 (ks_lstm_sequence_supported returns 1; other cells take the step-by-step entry points above).
 *   ks_lstm_sequence_forward   gi (T, M, 4H) = W_ih x_t + bias for every step (one product over all T M rows through the
 *                              input projection); h0, c0 (M, H) the carry the slice starts from; fresh (T, M) nullable;
 *                              hs, cs (T, M, H) the states after every step (cs nullable), saved (T, M, 7H) nullable, in the
 *                              layout of ks_lstm_train_forward.  With T = 1, hs / cs may alias h0 / c0; ks_lstm_forward and
 *                              ks_lstm_train_forward are this launch with T = 1 for such cells, so a rollout's steps and the
 *                              replay of its trajectory agree bit for bit.  The gates are evaluated with the hardware
 *                              exponential and reciprocal (about 1 ulp each; 3e-7 from the library's expf / tanhf on unit-scale
 *                              states).
 *   ks_lstm_sequence_backward  dH (T, M, H) the gradient reaching h_t from the layer above; d_g (T, M, 4H) out, as
 *                              ks_lstm_backward_step returns it per step; dh0, dc0 (M, H), nullable, the gradient of the
 *                              initial carry.  Needs ks_lstm_train_init (the transposed weights). */
int ks_lstm_sequence_supported(const KsLstm* lstm);
int ks_lstm_sequence_forward(const KsLstm* lstm, ks_stream_t stream, int64_t T, int64_t M, const float* gi, const float* h0,
                             const float* c0, const uint8_t* fresh, float* hs, float* cs, float* saved);
int ks_lstm_sequence_backward(const KsLstm* lstm, ks_stream_t stream, int64_t T, int64_t M, const float* dH, const float* saved,
                              const uint8_t* fresh, float* d_g, float* dh0, float* dc0);

/* Gaussian policy head and the gradient of the PPO objective (ppo.py:149-246, total 473-486):
 *   ks_gaussian_log_prob: per action dimension log N(action; mean, exp(log_std)) and entropy
 *   ks_ppo_loss_grad: d(total loss)/d(mean), d/d(value), d/d(log_std) for the mean over the M rows of
 *   policy + value + kl + entropy terms, with the new log-probabilities taken from (mean, log_std, action).
 *   d_log_std is overwritten; workspace >= KS_PPO_GRAD_WORKSPACE_BYTES(nu). */
int ks_gaussian_log_prob(ks_stream_t stream, int64_t M, int32_t nu, const float* mean, const float* log_std,
                         const float* action, float* log_prob /*(M,nu)*/, float* entropy /*(M,nu) nullable*/);
#define KS_MAX_ACTIONS 32
#define KS_PPO_GRAD_BLOCKS 256
#define KS_PPO_GRAD_WORKSPACE_BYTES(nu) ((size_t)KS_PPO_GRAD_BLOCKS * (nu) * 4)
int ks_ppo_loss_grad(ks_stream_t stream, int64_t M, int32_t nu, const KsPpoLossParams* params /*host*/,
                     const float* mean, const float* log_std, const float* action, const float* on_log_probs /*(M,nu)*/,
                     const float* advantages, const float* value_targets, const float* on_values,
                     const float* values, float* d_mean /*(M,nu)*/, float* d_value /*(M)*/, float* d_log_std /*(nu)*/,
                     void* workspace);

/* ks_ppo_loss_grad for a network with the mean | raw deviation head of ks_sample_action_head (examples/kbot/train.py:
 * 915-932): raw is (M, 2 nu); d_raw (M, 2 nu) receives the gradient with respect to both halves (through the softplus,
 * the scale and the cap of the deviation), which is what the network's backward pass takes. */
int ks_gaussian_head_log_prob(ks_stream_t stream, int64_t M, int32_t nu, const KsGaussianHead* head /*host*/,
                              const float* raw /*(M, 2 nu)*/, const float* action, float* log_prob /*(M,nu)*/,
                              float* entropy /*(M,nu) nullable*/);
int ks_ppo_loss_grad_head(ks_stream_t stream, int64_t M, int32_t nu, const KsPpoLossParams* params /*host*/,
                          const KsGaussianHead* head /*host*/, const float* raw, const float* action,
                          const float* on_log_probs /*(M,nu)*/, const float* advantages, const float* value_targets,
                          const float* on_values, const float* values, float* d_raw /*(M, 2 nu)*/, float* d_value /*(M)*/);

/* The same for the mixture-of-Gaussians head of ks_sample_action_mixture (examples/walking.py:127-144): raw and d_raw are
 * (M, 3 nu K).  The policy and KL terms differentiate the mixture's log-density exactly (responsibilities); the entropy
 * term uses the upper bound sum_k pi_k H_k + H(pi) of a mixture's entropy, which has no closed form (what
 * xax.MixtureOfGaussians.entropy computes is outside the reference tree: unpinned).  on_log_probs are the per-action
 * log-densities that ks_sample_action_mixture returned when the actions were drawn. */
int ks_mixture_head_log_prob(ks_stream_t stream, int64_t M, int32_t nu, const KsMixtureHead* head /*host*/,
                             const float* raw /*(M, 3 nu K)*/, const float* action /*(M,nu)*/, float* log_prob /*(M,nu)*/);
int ks_ppo_loss_grad_mixture(ks_stream_t stream, int64_t M, int32_t nu, const KsPpoLossParams* params /*host*/,
                             const KsMixtureHead* head /*host*/, const float* raw, const float* action,
                             const float* on_log_probs /*(M,nu)*/, const float* advantages, const float* value_targets,
                             const float* on_values, const float* values, float* d_raw /*(M, 3 nu K)*/, float* d_value /*(M)*/);

/* ------------------------------------------------------------------ rewards over a rollout
 * Replaces get_rewards + the stateless Reward.get_reward terms the configs name
 * (ksim/task/rl.py:189-245; ksim/rewards.py:166-188 StayAlive, 374-401 BaseHeight / BaseHeightRange,
 * 404-460 ActionVelocity / Acceleration / Jerk penalties, 746-777 Upright).
 * Trajectory arrays are time-major (T, N, dim); outputs are (T, N).  Each descriptor yields one
 * component scaled by `scale` (sign already folded for *Penalty classes, rl.py:219-221); the total is
 * their sum in order, optionally clipped (rl.py:235-239).
 */
enum { KS_REW_STAY_ALIVE = 0, KS_REW_BASE_HEIGHT = 1, KS_REW_BASE_HEIGHT_RANGE = 2, KS_REW_ACTION_VEL = 3,
       KS_REW_ACTION_ACC = 4, KS_REW_ACTION_JERK = 5, KS_REW_UPRIGHT_ANGVEL = 6, KS_REW_UPRIGHT_LINVEL = 7,
       KS_REW_UPRIGHT_POSE = 8,
       KS_REW_AMP = 9, /* max(0, 1 - 0.25 (logit - 1)^2) of the discriminator logits, ksim/task/amp.py:99-112 */
       KS_REW_STATEFUL = 10, /* a value ks_reward_scan computed: stateful[norm] (norm = slot index) */
       /* command tracking (ksim/rewards.py:84-88,236-372).  k(x) = -abs |x| - sq x^2 + exp(-x^2 / (2 scale^2)), p0 = scale,
        * p1 = sq, p2 = abs, p3 = zero_threshold; the command entries sit at command[index ...]. */
       KS_REW_LINVEL_CMD = 11, /* base velocity in the robot frame against a LinearVelocityCommandValue (vel, yaw, xvel,
                                  yvel at index + 0..3); norm picks the component: 0 vel = k(|v_xy| - vel), 1 yaw =
                                  k(atan2(v_y, v_x) - yaw), 2 x = k(v_x - xvel), 3 y = k(v_y - yvel); components 1-3 are
                                  zero while |vel command| < p3 */
       KS_REW_ANGVEL_CMD = 12, /* yaw rate qvel[5] against command[index]: norm 0 mag = k(w - cmd); norm 1 dir = +1 when
                                  the signs (zero inside +-p3) agree, else -1 */
       KS_REW_OFF_AXIS = 13,   /* exp(-v^2 / (2 p0^2)) of v = qvel[2] (norm 0), qvel[4] (norm 1), qvel[5] (norm 2) */
       KS_REW_MOTIONLESS = 14, /* |qvel[6:]| while |qvel[0:2]| < p0 and qvel[5] < p1, else 0 (rewards.py:1206-1221) */
       KS_REW_FORCE = 15,      /* max over `norm` bodies of (max(|obs[index + 3 b .. +3]| - p1, 0) / p0)^2 (rewards.py:1224-1240) */
       /* The kinds below read per-term constants from the table `params` of KsRewardIO at param_offset. */
       KS_REW_JOINT_SMOOTH = 16, /* SmallJointVelocity / Acceleration / JerkReward (rewards.py:463-508): mean over the joints
                                    qpos[7:] of exp(-x^2 / (2 p0^2)), x the first / second / third (norm = 1 / 2 / 3) difference
                                    along the rollout, edge-padded at its start and zeroed after a step that was done */
       KS_REW_AVOID_LIMITS = 17, /* mean over the joints of -min(q - lo, 0) + max(q - hi, 0); params (nq - 7, 2) (rewards.py:521-533) */
       KS_REW_TORQUE = 18,       /* mean |ctrl / params[u]| (rewards.py:556-581) */
       KS_REW_ENERGY = 19,       /* mean |ctrl / params[u] * qvel[6 + u]| (rewards.py:584-592) */
       KS_REW_JOINT_DEVIATION = 20, /* sum over `count` joints of norm((qpos[7 + index_k] - target_k) weight_k); params
                                       (count, 3) = index, target, weight (rewards.py:595-639) */
       KS_REW_FLAT_BODY = 21,    /* mean over `count` bodies of (R(xquat_b)^T p) . p; params = count body indices, then p
                                    (rewards.py:665-682) */
       KS_REW_POSITION_TRACKING = 22, /* exp(-e^2 / (2 p0^2)), e = sum_i norm((xpos[index2] - xpos[count])_i - command[index + i])
                                         (rewards.py:703-719); index2 = tracked body, count = base body */
       KS_REW_NO_ROLL_ANGVEL = 23, /* k(qvel[3]) (rewards.py:779-804) */
       KS_REW_NO_ROLL_POSE = 24,   /* k(-atan2(z_b.y, z_b.z)), z_b the world's z axis in the base frame */
       KS_REW_LINK_SMOOTH = 25,  /* LinkAcceleration / JerkPenalty (rewards.py:808-840): mean over the bodies 1.. of
                                    norm(second / third (p0 = 2 / 3) difference of |xpos(t) - xpos(t - 1)|), padded and
                                    zeroed like KS_REW_JOINT_SMOOTH; `norm` is the l1 / l2 choice */
       KS_REW_FEET_SLIP = 26,    /* sum over `norm` feet of |obs[index2 + 6 f .. + 6]| while any of the foot's `count` contact
                                    flags obs[index + c * norm + f] > 0.5 (rewards.py:1088-1105) */
       KS_REW_REACHABILITY = 27, /* sum over the joints of norm(max(0, |action - qpos[7:]| - params[u])) (rewards.py:1108-1129) */
       KS_REW_SINUSOIDAL_GAIT = 29, /* 1 - sum over `norm` feet of |obs[index + 3 f + 2] - command[index2 + f]| / p0
                                       (rewards.py:1320-1335); index2 = where the command's heights start */
       KS_REW_INTERSECTION = 28, /* 1 when two of the `norm` points obs[index + 3 i .. + 3] are closer than p0, else 0
                                    (rewards.py:1417-1430) */
       KS_REW_JOINT_POSITION = 30, /* JointPositionReward "pos" (rewards.py:1352-1380): mean over the `count` joints params[k]
                                      of kernel_with_penalty(current_position_k - qpos[7 + joint]; p0, p1, p2), where the
                                      command block at `index` holds a JointPositionCommandValue (commands.py:795-818) as
                                      [start (count), target (count), total_time, num_steps, step_id] and
                                      current_position = start + (target - start) step_id / num_steps */
       KS_REW_JOINT_VELOCITY_CMD = 31 /* its "vel" part: current_velocity = (target - start) / total_time against qvel[6 + joint] */ };
enum { KS_NORM_L1 = 0, KS_NORM_L2 = 1 }; /* xax.get_norm: l1 = |x|, l2 = x^2 (reference tests/test_rewards.py:95-98) */
#define KS_MAX_REWARD_PARAMS 320
typedef struct KsRewardDesc {
  int32_t kind;
  int32_t norm;   /* action-difference penalties */
  float scale;
  float p0, p1, p2; /* balance,success_reward,has_success_reward | target,kernel_scale | lo,hi,dropoff | scale,sq,abs */
  float p3;
  int32_t index;    /* offset into the command or observation vector, for the kinds that read one */
  int32_t index2, param_offset, count; /* see the kinds that name them */
} KsRewardDesc;
typedef struct KsRewardIO {
  int64_t T, N;
  int32_t nq, nv, nu, n_rewards;
  KsRewardDesc rewards[KS_MAX_REWARD_TERMS];
  int32_t use_clip_min, use_clip_max;
  float clip_min, clip_max;
  const float* qpos;   /* (T, N, nq) */
  const float* qvel;   /* (T, N, nv) */
  const float* action; /* (T, N, nu) */
  const uint8_t* done; /* (T, N) */
  const uint8_t* success; /* (T, N) */
  const float* disc_logits; /* (T, N) discriminator output per frame (ks_mlp_forward on the motion frames), KS_REW_AMP only */
  float* components;   /* (n_rewards, T, N) nullable */
  float* total;        /* (T, N) */
  const float* stateful; /* (n_slots, T, N) output of ks_reward_scan, KS_REW_STATEFUL only */
  int32_t command_dim, obs_dim;
  const float* command;  /* (T, N, command_dim), command-tracking kinds only */
  const float* obs;      /* (T, N, obs_dim), KS_REW_FORCE and KS_REW_FEET_SLIP */
  int32_t nb, n_params;
  const float* ctrl;     /* (T, N, nu) applied torques, KS_REW_TORQUE / KS_REW_ENERGY */
  const float* xpos;     /* (T, N, nb, 3) */
  const float* xquat;    /* (T, N, nb, 4) */
  float params[KS_MAX_REWARD_PARAMS]; /* per-term constants, n_params of them in use */
} KsRewardIO;
int ks_rewards(ks_stream_t stream, const KsRewardIO* io /*host*/);

/* Stateful rewards (StatefulReward.get_reward_stateful, ksim/rewards.py:127-163): sequential scans over the T steps of
 * a rollout with a per-env carry that persists between rollouts.  One lane walks one env forward in time.  As in
 * get_rewards (rl.py:206-214) the carry an env starts from is the initial one when the LAST step of this rollout is
 * done.  Outputs are unscaled; KS_REW_STATEFUL terms of ks_rewards pick them up in dict order.
 *   KS_SCAN_FEET_AIR_TIME (rewards.py:992-1085): carry = 3 n counters (air, ground, stationary ground; whole numbers
 *     kept as f32), three output slots (air, gnd, stationary_gnd).
 *   KS_SCAN_SPARSE_TARGET_HEIGHT (rewards.py:1148-1192): carry = n running maximum heights, one output slot.
 * Contact flags are the (n_contact, n) block of 0/1 values at obs[contact_index...] (any over n_contact, > 0.5);
 * positions the (n, 3) block at obs[position_index...]. */
#define KS_MAX_REWARD_SCANS 8
#define KS_MAX_SCAN_BODIES 8
#define KS_MAX_SCAN_JOINTS 32
enum { KS_SCAN_FEET_AIR_TIME = 0, KS_SCAN_SPARSE_TARGET_HEIGHT = 1,
       KS_SCAN_SYMMETRY = 2,          /* SymmetryReward (rewards.py:843-896): with x[t][j] = qpos[t][7 + joints[j]] - targets[j],
                                         carry <- carry (1 - alpha) + mean_t x[t] alpha once per rollout, then
                                         out[t] = -sum_j x[t][j] carry[j]; n joints, carry of n floats, one slot; a carry
                                         that restarts begins at the targets (initial_carry) */
       KS_SCAN_PAIRWISE_SYMMETRY = 3  /* PairwiseSymmetryReward (rewards.py:899-936): joints[0..1] = left, right,
                                         targets[0..1] their zeros, right negated when `flipped`; slot "lr" =
                                         kernel_with_penalty(left - right; kernel_scale, sq_scale, abs_scale), slot "self" as
                                         KS_SCAN_SYMMETRY over the pair; carry of 2 floats restarting at the zeros */ };
typedef struct KsRewardScanDesc {
  int32_t kind;
  int32_t n;               /* feet / bodies */
  int32_t n_contact;       /* contact geoms per foot */
  int32_t contact_index, position_index;
  int32_t slot;            /* first output slot */
  int32_t carry_index;     /* offset into the env's carry row */
  int32_t linvel_cmd_index, angvel_cmd_index; /* feet air time: index into the command vector whose |value| decides
                                                 "moving", or -1 to use |qvel[0:2]| and qvel[5] (rewards.py:1020-1037) */
  float air_steps, gnd_steps; /* round(gait_period * air_time_percent / ctrl_dt), round(gait_period * (1 - pct) / ctrl_dt) */
  float bias, ground_penalty;
  float linvel_threshold, angvel_threshold;
  float height;            /* sparse target height: the reward is clipped at it */
  int32_t joints[KS_MAX_SCAN_JOINTS]; /* symmetry kinds: joint indices (qpos address - 7) */
  float targets[KS_MAX_SCAN_JOINTS];
  float alpha, kernel_scale, sq_scale, abs_scale;
  int32_t flipped;
} KsRewardScanDesc;
typedef struct KsRewardScanIO {
  int64_t T, N;
  int32_t obs_dim, nv, command_dim, n_scans, carry_dim, n_slots;
  KsRewardScanDesc scans[KS_MAX_REWARD_SCANS];
  const float* obs;      /* (T, N, obs_dim) */
  const float* qvel;     /* (T, N, nv) */
  const float* qpos;     /* (T, N, nq), required by the symmetry kinds */
  int32_t nq;
  const float* command;  /* (T, N, command_dim) nullable unless a *_cmd_index is set */
  const uint8_t* done;   /* (T, N) */
  float* carry;          /* (N, carry_dim) in/out */
  float* out;            /* (n_slots, T, N) */
} KsRewardScanIO;
int ks_reward_scan(ks_stream_t stream, const KsRewardScanIO* io /*host*/);

/* ------------------------------------------------------------------ measurement aid
 * A plain f32 copy of n elements (reads 4n bytes, writes 4n bytes): the known-size kernel that hardware
 * traffic counters are calibrated against.  No counterpart in the reference. */
int ks_copy_f32(ks_stream_t stream, int64_t n, const float* src, float* dst);
/* The matrix cores' own yardstick: `workgroups` workgroups of four wavefronts, each wavefront issuing `iters` x 8
 * v_mfma_f32_32x32x16_bf16 on register operands (eight independent accumulator tiles, 32768 flop per instruction) and
 * nothing else.  out (workgroups x 256 floats) receives checksums; stamps (2 per workgroup, nullable) the shader-clock
 * cycles of the loop and the same interval in ticks of the constant 100 MHz counter, from which the clock under matrix
 * load follows.  What this reaches is the ceiling of any kernel built on that instruction.  No counterpart in the
 * reference. */
int ks_mfma_yardstick(ks_stream_t stream, int32_t workgroups, int32_t iters, float* out, int64_t* stamps);

#ifdef __cplusplus
}
#endif
#endif /* KSIM_HIP_H_ */
