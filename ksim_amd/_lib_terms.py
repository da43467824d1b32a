"""ctypes signatures of the per-env-term and MLP entry points (include/ksim_hip.h)."""
from __future__ import annotations

import ctypes
from ctypes import POINTER, c_float, c_int8, c_int32, c_int64, c_uint8, c_uint64, c_void_p

KS_MAX_OBS, KS_MAX_TERMS, KS_MAX_QPOS, KS_MAX_LAYERS = 512, 16, 40, 8
(SRC_QPOS, SRC_QVEL, SRC_QACC, SRC_CTRL, SRC_LAST_ACTION, SRC_COMMAND, SRC_TIME, SRC_XPOS, SRC_XQUAT, SRC_CVEL,
 SRC_CONST, SRC_CONTACT_DIST, SRC_CINERT, SRC_CFRC_EXT, SRC_COUNT) = range(15)
(OBS_COPY, OBS_JOINT_POS, OBS_ROT_INV, OBS_CONTACT, OBS_DELAYED, OBS_GRAVITY_EMA, OBS_SITE_GYRO, OBS_SITE_ACCEL,
 OBS_SITE_ROT6D, OBS_CONTACT_ANY, OBS_SITE_POS, OBS_SITE_QUAT, OBS_SITE_MAGNETOMETER) = range(13)
(NOISE_NONE, NOISE_ADD_GAUSSIAN, NOISE_ADD_UNIFORM, NOISE_MUL_GAUSSIAN, NOISE_MUL_UNIFORM, NOISE_ADD_UNIFORM_GAUSSIAN,
 NOISE_MUL_UNIFORM_GAUSSIAN) = range(7)
KS_MAX_NOISE_CHAIN = 4
(TERM_MIN_HEIGHT, TERM_BAD_Z, TERM_NOT_UPRIGHT, TERM_BAD_VELOCITY, TERM_FAR_FROM_ORIGIN,
 TERM_EPISODE_LENGTH, TERM_ILLEGAL_CONTACT) = range(7)
ACT_NONE, ACT_ELU, ACT_RELU, ACT_TANH, ACT_GELU = range(5)
MLP_F32, MLP_BF16 = 0, 1


class KsNoiseStage(ctypes.Structure):
    _fields_ = [("kind", c_int32), ("mean", c_float), ("scale", c_float), ("scale2", c_float)]


class KsRandomVar(ctypes.Structure):
    _fields_ = [("mean", c_float), ("mag", c_float), ("std", c_float), ("same_key", c_int32)]


class KsObsElem(ctypes.Structure):
    _fields_ = [("kind", c_int32), ("src", c_int32), ("index", c_int32), ("comp", c_int32), ("c0", c_float),
                ("c1", c_float), ("c2", c_float), ("n_noise", c_int32), ("noise", KsNoiseStage * KS_MAX_NOISE_CHAIN),
                ("bias", KsNoiseStage), ("carry", c_int32), ("stride", c_int32), ("q0", c_float), ("q1", c_float),
                ("q2", c_float), ("e0", c_float), ("e1", c_float), ("e2", c_float), ("e3", c_float), ("env_site", c_int32)]


class KsTermDesc(ctypes.Structure):
    _fields_ = [("kind", c_int32), ("value", c_int32), ("p0", c_float), ("p1", c_float), ("p2", c_float),
                ("p3", c_float)]


class KsTermsDesc(ctypes.Structure):
    _fields_ = [("nq", c_int32), ("nv", c_int32), ("nu", c_int32), ("nb", c_int32), ("obs_dim", c_int32),
                ("n_terms", c_int32), ("command_dim", c_int32), ("random_heading", c_int32),
                ("ns", c_int32), ("carry_dim", c_int32), ("action_dim", c_int32), ("nonfinite_terminates", c_int32),
                ("obs", KsObsElem * KS_MAX_OBS), ("terms", KsTermDesc * KS_MAX_TERMS),
                ("reset_base", c_float * KS_MAX_QPOS), ("reset_mag", c_float * KS_MAX_QPOS),
                ("reset_lo", c_float * KS_MAX_QPOS), ("reset_hi", c_float * KS_MAX_QPOS),
                ("reset_by_level", c_int32 * KS_MAX_QPOS), ("reset_from_motion", c_int32 * KS_MAX_QPOS),
                ("reset_pitch_roll", c_int32), ("reset_pitch", c_float * 2), ("reset_roll", c_float * 2),
                ("reset_hfield", c_int32), ("hfield_bound", c_float * 2)]


class KsRng(ctypes.Structure):
    _fields_ = [("seed", c_uint64), ("step", c_uint64), ("step_base", c_void_p)]


KS_MAX_EVENTS = 4
KS_EVENT_DRAWS, KS_EVENT_FORCE_STATE = 12, 8
EVENT_LINEAR_PUSH, EVENT_ANGULAR_PUSH, EVENT_JUMP, EVENT_FORCE_PUSH = range(4)


class KsEventDesc(ctypes.Structure):
    _fields_ = [("kind", c_int32), ("mag", c_float), ("lo", c_float), ("hi", c_float), ("interval_lo", c_float),
                ("interval_hi", c_float), ("level_scale", c_float), ("mag2", c_float), ("duration_lo", c_float),
                ("duration_hi", c_float), ("body", c_int32)]


class KsObserveIO(ctypes.Structure):
    _fields_ = [("N", c_int64), ("level", c_float), ("src", c_void_p * SRC_COUNT), ("zero_offset", c_void_p),
                ("bias_draw", c_void_p), ("bias_redraw", c_void_p), ("noise_normal", c_void_p), ("noise_uniform", c_void_p),
                ("rng", KsRng),
                ("obs", c_void_p), ("noisy_obs", c_void_p), ("carry", c_void_p), ("fresh", c_void_p),
                ("carry_uniform", c_void_p), ("site_pose", c_void_p)]


class KsTerminateIO(ctypes.Structure):
    _fields_ = [("N", c_int64), ("level", c_float), ("qpos", c_void_p), ("qvel", c_void_p),
                ("qacc_warmstart", c_void_p), ("time", c_void_p), ("last_ctrl", c_void_p), ("components", c_void_p),
                ("done", c_void_p), ("success", c_void_p), ("traj_qpos", c_void_p), ("traj_qvel", c_void_p),
                ("traj_time", c_void_p), ("reset_mask", c_void_p), ("episode_length", c_void_p),
                ("reset_uniform", c_void_p), ("reset_pitch_roll_uniform", c_void_p), ("reset_motion_qpos", c_void_p),
                ("reset_motion_frames", c_int32), ("reset_motion_dt", c_float), ("reset_frame", c_void_p),
                ("reset_hfield", c_void_p), ("hfield_nx", c_int32), ("hfield_ny", c_int32),
                ("rng", KsRng), ("apply_reset", c_int32), ("n_events", c_int32),
                ("event_interval", (c_float * 2) * KS_MAX_EVENTS), ("event_state", c_void_p),
                ("event_reset_uniform", c_void_p), ("event_force", c_void_p), ("contact_dist", c_void_p),
                ("action_latency", c_void_p), ("latency_lo", c_float), ("latency_hi", c_float), ("zero_offset", c_void_p),
                ("zero_offset_rv", KsRandomVar), ("act_action_bias", c_void_p), ("act_torque_bias", c_void_p),
                ("act_kp_scale", c_void_p), ("act_kd_scale", c_void_p), ("act_torque_limit_scale", c_void_p),
                ("action_bias_rv", KsRandomVar), ("torque_bias_rv", KsRandomVar), ("kp_scale_rv", KsRandomVar),
                ("kd_scale_rv", KsRandomVar), ("torque_limit_scale_rv", KsRandomVar), ("episode_uniform", c_void_p),
                ("episode_normal", c_void_p)]


class KsMlpDesc(ctypes.Structure):
    _fields_ = [("n_layers", c_int32), ("dims", c_int32 * (KS_MAX_LAYERS + 1)), ("activation", c_int32),
                ("dtype", c_int32), ("weights", c_void_p * KS_MAX_LAYERS), ("biases", c_void_p * KS_MAX_LAYERS)]


(REW_STAY_ALIVE, REW_BASE_HEIGHT, REW_BASE_HEIGHT_RANGE, REW_ACTION_VEL, REW_ACTION_ACC, REW_ACTION_JERK,
 REW_UPRIGHT_ANGVEL, REW_UPRIGHT_LINVEL, REW_UPRIGHT_POSE, REW_AMP, REW_STATEFUL, REW_LINVEL_CMD, REW_ANGVEL_CMD,
 REW_OFF_AXIS, REW_MOTIONLESS, REW_FORCE, REW_JOINT_SMOOTH, REW_AVOID_LIMITS, REW_TORQUE, REW_ENERGY, REW_JOINT_DEVIATION,
 REW_FLAT_BODY, REW_POSITION_TRACKING, REW_NO_ROLL_ANGVEL, REW_NO_ROLL_POSE, REW_LINK_SMOOTH, REW_FEET_SLIP,
 REW_REACHABILITY, REW_INTERSECTION, REW_SINUSOIDAL_GAIT, REW_JOINT_POSITION, REW_JOINT_VELOCITY_CMD) = range(32)
KS_MAX_REWARD_PARAMS = 320
KS_MAX_REWARD_SCANS, KS_MAX_SCAN_BODIES, KS_MAX_SCAN_JOINTS = 8, 8, 32
SCAN_FEET_AIR_TIME, SCAN_SPARSE_TARGET_HEIGHT, SCAN_SYMMETRY, SCAN_PAIRWISE_SYMMETRY = 0, 1, 2, 3
NORM_L1, NORM_L2 = 0, 1
KS_MAX_REWARD_TERMS = 32


class KsRewardDesc(ctypes.Structure):
    _fields_ = [("kind", c_int32), ("norm", c_int32), ("scale", c_float), ("p0", c_float), ("p1", c_float),
                ("p2", c_float), ("p3", c_float), ("index", c_int32), ("index2", c_int32), ("param_offset", c_int32),
                ("count", c_int32)]


class KsRewardIO(ctypes.Structure):
    _fields_ = [("T", c_int64), ("N", c_int64), ("nq", c_int32), ("nv", c_int32), ("nu", c_int32),
                ("n_rewards", c_int32), ("rewards", KsRewardDesc * KS_MAX_REWARD_TERMS), ("use_clip_min", c_int32),
                ("use_clip_max", c_int32), ("clip_min", c_float), ("clip_max", c_float), ("qpos", c_void_p),
                ("qvel", c_void_p), ("action", c_void_p), ("done", c_void_p), ("success", c_void_p),
                ("disc_logits", c_void_p), ("components", c_void_p), ("total", c_void_p), ("stateful", c_void_p),
                ("command_dim", c_int32), ("obs_dim", c_int32), ("command", c_void_p), ("obs", c_void_p),
                ("nb", c_int32), ("n_params", c_int32), ("ctrl", c_void_p), ("xpos", c_void_p), ("xquat", c_void_p),
                ("params", c_float * KS_MAX_REWARD_PARAMS)]


class KsRewardScanDesc(ctypes.Structure):
    _fields_ = [("kind", c_int32), ("n", c_int32), ("n_contact", c_int32), ("contact_index", c_int32),
                ("position_index", c_int32), ("slot", c_int32), ("carry_index", c_int32),
                ("linvel_cmd_index", c_int32), ("angvel_cmd_index", c_int32), ("air_steps", c_float),
                ("gnd_steps", c_float), ("bias", c_float), ("ground_penalty", c_float), ("linvel_threshold", c_float),
                ("angvel_threshold", c_float), ("height", c_float), ("joints", c_int32 * KS_MAX_SCAN_JOINTS),
                ("targets", c_float * KS_MAX_SCAN_JOINTS), ("alpha", c_float), ("kernel_scale", c_float),
                ("sq_scale", c_float), ("abs_scale", c_float), ("flipped", c_int32)]


class KsRewardScanIO(ctypes.Structure):
    _fields_ = [("T", c_int64), ("N", c_int64), ("obs_dim", c_int32), ("nv", c_int32), ("command_dim", c_int32),
                ("n_scans", c_int32), ("carry_dim", c_int32), ("n_slots", c_int32),
                ("scans", KsRewardScanDesc * KS_MAX_REWARD_SCANS), ("obs", c_void_p), ("qvel", c_void_p),
                ("qpos", c_void_p), ("nq", c_int32), ("command", c_void_p), ("done", c_void_p), ("carry", c_void_p), ("out", c_void_p)]


class KsGruDesc(ctypes.Structure):
    _fields_ = [("input_size", c_int32), ("hidden_size", c_int32), ("dtype", c_int32), ("weight_ih", c_void_p),
                ("weight_hh", c_void_p), ("bias", c_void_p), ("bias_n", c_void_p)]


KS_MAX_COMMANDS, KS_COMMAND_DRAWS = 8, 20
KS_MAX_VECTOR_COMMAND = 16
(CMD_CONST, CMD_LINEAR_VELOCITY, CMD_ANGULAR_VELOCITY, CMD_FLOAT_VECTOR, CMD_INT_VECTOR, CMD_START_POSITION,
 CMD_START_QUATERNION, CMD_BASE_HEIGHT, CMD_SINUSOIDAL_GAIT, CMD_JOINT_POSITION, CMD_CARTESIAN_COORDINATE) = range(11)


class KsCommandDesc(ctypes.Structure):
    _fields_ = [("kind", c_int32), ("index", c_int32), ("dim", c_int32), ("min_vel", c_float), ("max_vel", c_float),
                ("max_yaw", c_float), ("zero_prob", c_float), ("backward_prob", c_float), ("switch_prob", c_float),
                ("ctrl_dt", c_float), ("linear_accel", c_float), ("angular_accel", c_float),
                ("lo", c_float * KS_MAX_VECTOR_COMMAND), ("hi", c_float * KS_MAX_VECTOR_COMMAND),
                ("joints", c_int32 * KS_MAX_VECTOR_COMMAND), ("min_time", c_float), ("max_time", c_float), ("jump_prob", c_float)]


class KsCommandIO(ctypes.Structure):
    _fields_ = [("N", c_int64), ("command_dim", c_int32), ("n_commands", c_int32), ("nq", c_int32), ("nv", c_int32),
                ("commands", KsCommandDesc * KS_MAX_COMMANDS), ("command", c_void_p), ("traj_command", c_void_p),
                ("qpos", c_void_p), ("qvel", c_void_p), ("fresh", c_void_p), ("all_fresh", c_int32), ("uniform", c_void_p),
                ("rng", KsRng)]


class KsGaussianHead(ctypes.Structure):
    _fields_ = [("min_std", c_float), ("max_std", c_float), ("var_scale", c_float), ("deterministic", c_int32),
                ("mean_bias", c_void_p)]


class KsMixtureHead(ctypes.Structure):
    _fields_ = [("num_mixtures", c_int32), ("min_std", c_float), ("max_std", c_float), ("var_scale", c_float),
                ("deterministic", c_int32), ("mean_bias", c_void_p), ("clip_lo", c_void_p), ("clip_hi", c_void_p)]


class KsLstmDesc(ctypes.Structure):
    _fields_ = [("input_size", c_int32), ("hidden_size", c_int32), ("dtype", c_int32), ("weight_ih", c_void_p),
                ("weight_hh", c_void_p), ("bias", c_void_p)]


class KsAdamParams(ctypes.Structure):
    _fields_ = [("lr", c_float), ("b1", c_float), ("b2", c_float), ("eps", c_float), ("weight_decay", c_float),
                ("max_grad_norm", c_float), ("step", c_int64)]


def bind(lib) -> None:
    lib.ks_rewards.argtypes = [c_void_p, POINTER(KsRewardIO)]
    lib.ks_rewards.restype = c_int32
    lib.ks_gru_create.argtypes = [POINTER(KsGruDesc), POINTER(c_void_p)]
    lib.ks_gru_destroy.argtypes = [c_void_p]
    lib.ks_gru_workspace_bytes.argtypes = [c_void_p, c_int64]
    lib.ks_gru_workspace_bytes.restype = c_int64
    lib.ks_gru_forward.argtypes = [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.ks_lstm_create.argtypes = [POINTER(KsLstmDesc), POINTER(c_void_p)]
    lib.ks_lstm_destroy.argtypes = [c_void_p]
    lib.ks_lstm_workspace_bytes.argtypes = [c_void_p, c_int64]
    lib.ks_lstm_workspace_bytes.restype = c_int64
    lib.ks_lstm_forward.argtypes = [c_void_p, c_void_p, c_int64] + [c_void_p] * 7
    for name in ("ks_gru_create", "ks_gru_destroy", "ks_gru_forward", "ks_lstm_create", "ks_lstm_destroy", "ks_lstm_forward"):
        getattr(lib, name).restype = c_int32
    lib.ks_reward_scan.argtypes = [c_void_p, POINTER(KsRewardScanIO)]
    lib.ks_reward_scan.restype = c_int32
    lib.ks_terms_create.argtypes = [POINTER(KsTermsDesc), POINTER(c_void_p)]
    lib.ks_terms_destroy.argtypes = [c_void_p]
    lib.ks_observe.argtypes = [c_void_p, c_void_p, POINTER(KsObserveIO)]
    lib.ks_terminate_reset.argtypes = [c_void_p, c_void_p, POINTER(KsTerminateIO)]
    lib.ks_terminate_reset_observe.argtypes = [c_void_p, c_void_p, POINTER(KsTerminateIO), POINTER(KsObserveIO)]
    lib.ks_terminate_reset_observe.restype = c_int32
    lib.ks_sample_action.argtypes = [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_void_p, KsRng, c_float,
                                     c_void_p]
    lib.ks_commands.argtypes = [c_void_p, POINTER(KsCommandIO)]
    lib.ks_commands.restype = c_int32
    lib.ks_sample_action_head.argtypes = [c_void_p, c_int64, c_int32, c_void_p, POINTER(KsGaussianHead), c_void_p, KsRng,
                                          c_float, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.ks_sample_action_head.restype = c_int32
    lib.ks_action_filter.argtypes = [c_void_p, c_int64, c_int32, c_int32, c_float, c_float] + [c_void_p] * 7
    lib.ks_action_filter.restype = c_int32
    lib.ks_sample_action_mixture.argtypes = [c_void_p, c_int64, c_int32, c_void_p, POINTER(KsMixtureHead), c_void_p, c_void_p,
                                             KsRng, c_float, c_void_p, c_void_p, c_void_p]
    lib.ks_sample_action_mixture.restype = c_int32
    lib.ks_mlp_create.argtypes = [POINTER(KsMlpDesc), POINTER(c_void_p)]
    lib.ks_mlp_destroy.argtypes = [c_void_p]
    lib.ks_mlp_workspace_bytes.argtypes = [c_void_p, c_int64]
    lib.ks_mlp_workspace_bytes.restype = c_int64
    lib.ks_mlp_forward.argtypes = [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p]
    lib.ks_mlp_forward_pair.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
                                        c_void_p, c_void_p]
    lib.ks_mlp_train_init.argtypes = [c_void_p]
    lib.ks_mlp_train_workspace_bytes.argtypes = [c_void_p, c_int64]
    lib.ks_mlp_train_workspace_bytes.restype = c_int64
    lib.ks_mlp_train_forward.argtypes = [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p]
    lib.ks_mlp_train_backward.argtypes = [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p]
    lib.ks_grad_sqnorm.argtypes = [c_void_p, c_int64, c_void_p, c_void_p]
    lib.ks_mlp_train_backward_dx.argtypes = [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int32, c_int32,
                                             c_void_p, c_void_p]
    lib.ks_mlp_freeze_bias_prefix.argtypes = [c_void_p, c_int32, c_int32]
    lib.ks_gru_train_init.argtypes = [c_void_p]
    lib.ks_gru_projections.argtypes = [c_void_p, POINTER(c_void_p), POINTER(c_void_p)]
    lib.ks_gru_train_forward.argtypes = [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.ks_gru_backward_workspace_bytes.argtypes = [c_void_p, c_int64]
    lib.ks_gru_backward_workspace_bytes.restype = c_int64
    lib.ks_gru_backward_step.argtypes = [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                         c_void_p]
    lib.ks_gru_grad_sqnorm.argtypes = [c_void_p, c_void_p, c_void_p]
    lib.ks_gru_adam_step.argtypes = [c_void_p, c_void_p, POINTER(KsAdamParams), c_void_p]
    lib.ks_ppo_loss_grad_head.argtypes = [c_void_p, c_int64, c_int32, c_void_p, POINTER(KsGaussianHead)] + [c_void_p] * 9
    lib.ks_ppo_loss_grad_head.restype = c_int32
    lib.ks_ppo_loss_grad_mixture.argtypes = [c_void_p, c_int64, c_int32, c_void_p, POINTER(KsMixtureHead)] + [c_void_p] * 9
    lib.ks_ppo_loss_grad_mixture.restype = c_int32
    lib.ks_mixture_head_log_prob.argtypes = [c_void_p, c_int64, c_int32, POINTER(KsMixtureHead), c_void_p, c_void_p, c_void_p]
    lib.ks_mixture_head_log_prob.restype = c_int32
    lib.ks_gaussian_head_log_prob.argtypes = [c_void_p, c_int64, c_int32, POINTER(KsGaussianHead), c_void_p, c_void_p, c_void_p, c_void_p]
    lib.ks_gaussian_head_log_prob.restype = c_int32
    lib.ks_lstm_train_init.argtypes = [c_void_p]
    lib.ks_lstm_projections.argtypes = [c_void_p, POINTER(c_void_p), POINTER(c_void_p)]
    lib.ks_lstm_train_forward.argtypes = [c_void_p, c_void_p, c_int64] + [c_void_p] * 8
    lib.ks_lstm_backward_workspace_bytes.argtypes = [c_void_p, c_int64]
    lib.ks_lstm_backward_workspace_bytes.restype = c_int64
    lib.ks_lstm_backward_step.argtypes = [c_void_p, c_void_p, c_int64] + [c_void_p] * 8
    lib.ks_lstm_grad_sqnorm.argtypes = [c_void_p, c_void_p, c_void_p]
    lib.ks_lstm_sequence_supported.argtypes = [c_void_p]
    lib.ks_lstm_sequence_supported.restype = c_int32
    lib.ks_lstm_sequence_forward.argtypes = [c_void_p, c_void_p, c_int64, c_int64] + [c_void_p] * 7
    lib.ks_lstm_sequence_forward.restype = c_int32
    lib.ks_lstm_sequence_backward.argtypes = [c_void_p, c_void_p, c_int64, c_int64] + [c_void_p] * 6
    lib.ks_lstm_sequence_backward.restype = c_int32
    lib.ks_lstm_adam_step.argtypes = [c_void_p, c_void_p, POINTER(KsAdamParams), c_void_p]
    for name in ("ks_mlp_train_backward_dx", "ks_mlp_freeze_bias_prefix", "ks_gru_train_init", "ks_gru_projections",
                 "ks_gru_train_forward", "ks_gru_backward_step", "ks_gru_grad_sqnorm", "ks_gru_adam_step",
                 "ks_lstm_train_init", "ks_lstm_projections", "ks_lstm_train_forward", "ks_lstm_backward_step",
                 "ks_lstm_grad_sqnorm", "ks_lstm_adam_step"):
        getattr(lib, name).restype = c_int32
    lib.ks_mlp_disc_workspace_bytes.argtypes = [c_void_p, c_int64, c_int64]
    lib.ks_mlp_disc_workspace_bytes.restype = c_int64
    lib.ks_mlp_disc_loss_grad.argtypes = [c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_float, c_int64, c_void_p, c_void_p]
    lib.ks_mlp_disc_loss_grad.restype = c_int32
    lib.ks_mlp_grad_sqnorm.argtypes = [c_void_p, c_void_p, c_void_p]
    lib.ks_mlp_adam_step.argtypes = [c_void_p, c_void_p, POINTER(KsAdamParams), c_void_p]
    lib.ks_adam_step.argtypes = [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, POINTER(KsAdamParams), c_void_p]
    lib.ks_mlp_get_params.argtypes = [c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_int32]
    lib.ks_gaussian_log_prob.argtypes = [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]
    for name in ("ks_mlp_train_init", "ks_mlp_train_forward", "ks_mlp_train_backward", "ks_grad_sqnorm",
                 "ks_mlp_grad_sqnorm", "ks_mlp_adam_step", "ks_adam_step", "ks_mlp_get_params", "ks_gaussian_log_prob"):
        getattr(lib, name).restype = c_int32
    for name in ("ks_terms_create", "ks_terms_destroy", "ks_observe", "ks_terminate_reset", "ks_sample_action",
                 "ks_mlp_create", "ks_mlp_destroy", "ks_mlp_forward", "ks_mlp_forward_pair"):
        getattr(lib, name).restype = c_int32
