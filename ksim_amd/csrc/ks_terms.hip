// Fused per-env terms: observation assembly + noise, terminations + trajectory record + reset
// predication, and action sampling.  Streaming kernels over (N, dim) env-major rows.
#include "ks_common.h"
#include "ks_philox.h"

#include <cstring>

namespace ks {

struct DevTerms {
  KsTermsDesc d;
};

__device__ inline void rot_inv(const float* q4, float vx, float vy, float vz, float* out) {
  // q^-1 v q for the (normalised) wxyz quaternion q
  float w = q4[0], x = q4[1], y = q4[2], z = q4[3];
  const float n = sqrtf(w * w + x * x + y * y + z * z);
  const float inv = n > 0.f ? 1.0f / n : 0.f;
  w *= inv; x = -x * inv; y = -y * inv; z = -z * inv;  // conjugate
  // t = 2 * (qv x v); v' = v + w t + qv x t
  const float tx = 2.f * (y * vz - z * vy), ty = 2.f * (z * vx - x * vz), tz = 2.f * (x * vy - y * vx);
  out[0] = vx + w * tx + (y * tz - z * ty);
  out[1] = vy + w * ty + (z * tx - x * tz);
  out[2] = vz + w * tz + (x * ty - y * tx);
}

struct ObserveArgs {
  const DevTerms* t;
  int64_t N;
  float level;
  const float* src[KS_SRC_COUNT];
  int src_dim[KS_SRC_COUNT];
  const float *zero_offset, *bias_redraw, *noise_normal, *noise_uniform;
  float* bias_draw;
  KsRng rng;
  float *obs, *noisy;
  int obs_dim, nq, nu;
  float* carry;
  const uint8_t* fresh;
  const float* carry_uniform;
  const float* site_pose;
  int carry_dim;
};

// v rotated by the (normalised) wxyz quaternion q
__device__ inline void rot_fwd(const float* q4, const float* v, float* out) {
  const float w = q4[0], x = q4[1], y = q4[2], z = q4[3];
  const float tx = 2.f * (y * v[2] - z * v[1]), ty = 2.f * (z * v[0] - x * v[2]), tz = 2.f * (x * v[1] - y * v[0]);
  out[0] = v[0] + w * tx + (y * tz - z * ty);
  out[1] = v[1] + w * ty + (z * tx - x * tz);
  out[2] = v[2] + w * tz + (x * ty - y * tx);
}

// one noise or bias stage on the value v with the standard draws z ~ N(0,1), w ~ U(-1,1) (ksim/noise.py:74-121,184-213)
__device__ inline float apply_stage(const KsNoiseStage& st, float v, float z, float w, float level) {
  float rv = st.mean;
  switch (st.kind) {
    case KS_NOISE_ADD_GAUSSIAN: case KS_NOISE_MUL_GAUSSIAN: rv += z * (st.scale * level); break;
    case KS_NOISE_ADD_UNIFORM: case KS_NOISE_MUL_UNIFORM: rv += w * (st.scale * level); break;
    case KS_NOISE_ADD_UNIFORM_GAUSSIAN: case KS_NOISE_MUL_UNIFORM_GAUSSIAN: rv += z * (st.scale * level) + w * (st.scale2 * level); break;
    default: return v;
  }
  const bool add = st.kind == KS_NOISE_ADD_GAUSSIAN || st.kind == KS_NOISE_ADD_UNIFORM || st.kind == KS_NOISE_ADD_UNIFORM_GAUSSIAN;
  return add ? v + rv : v * rv;
}

// One observation element: idx = env * obs_dim + element.
__device__ __forceinline__ void observe_one(const ObserveArgs& a, int64_t idx) {
  const int64_t e = idx / a.obs_dim;
  const int k = (int)(idx - e * a.obs_dim);
  // read in place (the table sits in the caches): a private copy of the element, whose noise chain is indexed at run
  // time, would live in scratch memory and cost a write and a read of the whole element per thread
  const KsObsElem& el = a.t->d.obs[k];
  float v;
  if (el.kind == KS_OBS_COPY) {
    v = (el.src == KS_SRC_CONST) ? el.c0 : a.src[el.src][e * a.src_dim[el.src] + el.index];
  } else if (el.kind == KS_OBS_JOINT_POS) {
    v = a.src[KS_SRC_QPOS][e * a.nq + el.index] - (a.zero_offset ? a.zero_offset[e * a.nu + (el.index - 7)] : 0.f);
  } else if (el.kind == KS_OBS_CONTACT) {
    v = a.src[el.src][e * a.src_dim[el.src] + el.index] < 0.f ? 1.f : 0.f;
  } else if (el.kind == KS_OBS_DELAYED) {
    // this thread owns one column of the delay buffer: nobody else reads or writes it
    float* col = a.carry + e * a.carry_dim + el.carry;
    const float cur = a.src[el.src][e * a.src_dim[el.src] + el.index];
    const bool fresh = a.fresh && a.fresh[e];
    v = fresh ? cur : col[0];
    for (int d = 0; d + 1 < el.comp; ++d) col[d * el.stride] = fresh ? cur : col[(d + 1) * el.stride];
    col[(el.comp - 1) * el.stride] = cur;
    if (el.src == KS_SRC_QPOS && a.zero_offset) v -= a.zero_offset[e * a.nu + (el.index - 7)];
  } else if (el.kind == KS_OBS_GRAVITY_EMA) {
    // the three components of one reading run in three threads; each recomputes the vector and owns x[comp]
    float* c = a.carry + e * a.carry_dim + el.carry;
    float x = c[el.comp], lag = c[3], b[3] = {c[4], c[5], c[6]};
    if (a.fresh && a.fresh[e]) {
      float u[4];
      if (a.carry_uniform) {
        for (int j = 0; j < 4; ++j) u[j] = a.carry_uniform[e * a.carry_dim + el.carry + 3 + j];
      } else {
        const Philox4 r = draw(a.rng.seed, a.rng.step + (a.rng.step_base ? *a.rng.step_base : 0ull), kRngObsCarry, (uint64_t)e, (uint32_t)el.carry);
        u[0] = u01(r.x); u[1] = u01(r.y); u[2] = u01(r.z); u[3] = u01(r.w);
      }
      x = 0.f;
      lag = el.q0 + u[0] * (el.q1 - el.q0);
      for (int j = 0; j < 3; ++j) b[j] = -el.q2 + u[1 + j] * (2.f * el.q2);
      if (el.comp == 0) { c[3] = lag; c[4] = b[0]; c[5] = b[1]; c[6] = b[2]; }
    }
    float g[3], p[3];
    rot_inv(a.src[KS_SRC_QPOS] + e * a.nq + 3, el.c0, el.c1, el.c2, g);
    // roll-pitch-yaw (x, y, z angles; z applied last) to a quaternion
    const float cr = cosf(0.5f * b[0]), sr = sinf(0.5f * b[0]), cp = cosf(0.5f * b[1]), sp = sinf(0.5f * b[1]);
    const float cy = cosf(0.5f * b[2]), sy = sinf(0.5f * b[2]);
    const float bq[4] = {cr * cp * cy + sr * sp * sy, sr * cp * cy - cr * sp * sy, cr * sp * cy + sr * cp * sy, cr * cp * sy - sr * sp * cy};
    rot_fwd(bq, g, p);
    x = x * lag + p[el.comp] * (1.f - lag);
    c[el.comp] = x;
    v = x;
  } else if (el.kind == KS_OBS_CONTACT_ANY) {
    bool any = false;
    for (int sidx = 0; sidx < a.src_dim[KS_SRC_CONTACT_DIST]; ++sidx)
      any |= ((el.index >> sidx) & 1) && a.src[KS_SRC_CONTACT_DIST][e * a.src_dim[KS_SRC_CONTACT_DIST] + sidx] < 0.f;
    v = any ? 1.f : 0.f;
  } else if (el.kind == KS_OBS_SITE_ROT6D) {
    const float* qb = a.src[KS_SRC_XQUAT] + e * a.src_dim[KS_SRC_XQUAT] + 4 * el.index;
    float qs[4] = {el.e0, el.e1, el.e2, el.e3};
    if (el.env_site) for (int k = 0; k < 4; ++k) qs[k] = a.site_pose[e * 7 + k];
    // world orientation of the site: q = q_body q_site; row i of R(q) is what the inverse rotation makes of axis i
    const float q[4] = {qb[0] * qs[0] - qb[1] * qs[1] - qb[2] * qs[2] - qb[3] * qs[3],
                        qb[0] * qs[1] + qb[1] * qs[0] + qb[2] * qs[3] - qb[3] * qs[2],
                        qb[0] * qs[2] - qb[1] * qs[3] + qb[2] * qs[0] + qb[3] * qs[1],
                        qb[0] * qs[3] + qb[1] * qs[2] - qb[2] * qs[1] + qb[3] * qs[0]};
    const int row = el.comp / 3, col = el.comp - 3 * row;
    float col_vec[3], axis[3] = {0.f, 0.f, 0.f};
    axis[col] = 1.f;
    rot_fwd(q, axis, col_vec);  // column `col` of R
    v = col_vec[row];
  } else if (el.kind == KS_OBS_SITE_POS || el.kind == KS_OBS_SITE_QUAT || el.kind == KS_OBS_SITE_MAGNETOMETER) {
    const float* qb = a.src[KS_SRC_XQUAT] + e * a.src_dim[KS_SRC_XQUAT] + 4 * el.index;
    float qs[4] = {el.e0, el.e1, el.e2, el.e3}, r_l[3] = {el.c0, el.c1, el.c2};
    if (el.env_site) {
      for (int k = 0; k < 4; ++k) qs[k] = a.site_pose[e * 7 + k];
      for (int k = 0; k < 3; ++k) r_l[k] = a.site_pose[e * 7 + 4 + k];
    }
    if (el.kind == KS_OBS_SITE_POS) {
      float r[3];
      rot_fwd(qb, r_l, r);
      v = a.src[KS_SRC_XPOS][e * a.src_dim[KS_SRC_XPOS] + 3 * el.index + el.comp] + r[el.comp];
    } else if (el.kind == KS_OBS_SITE_QUAT) {
      const float q[4] = {qb[0] * qs[0] - qb[1] * qs[1] - qb[2] * qs[2] - qb[3] * qs[3],
                          qb[0] * qs[1] + qb[1] * qs[0] + qb[2] * qs[3] - qb[3] * qs[2],
                          qb[0] * qs[2] - qb[1] * qs[3] + qb[2] * qs[0] + qb[3] * qs[1],
                          qb[0] * qs[3] + qb[1] * qs[2] - qb[2] * qs[1] + qb[3] * qs[0]};
      v = q[el.comp];
    } else {
      float in_body[3], out[3];
      rot_inv(qb, el.q0, el.q1, el.q2, in_body);
      rot_inv(qs, in_body[0], in_body[1], in_body[2], out);
      v = out[el.comp];
    }
  } else if (el.kind == KS_OBS_SITE_GYRO || el.kind == KS_OBS_SITE_ACCEL) {
    const float* qb = a.src[KS_SRC_XQUAT] + e * a.src_dim[KS_SRC_XQUAT] + 4 * el.index;
    const float* w = a.src[KS_SRC_CVEL] + e * a.src_dim[KS_SRC_CVEL] + 6 * el.index;  // angular velocity, world axes
    float vec[3] = {w[0], w[1], w[2]};
    if (el.kind == KS_OBS_SITE_ACCEL) {
      const float* qa = a.src[KS_SRC_QACC] + e * a.src_dim[KS_SRC_QACC];
      float r[3], al[3];
      const float al_l[3] = {qa[3], qa[4], qa[5]};
      float r_l[3] = {el.c0, el.c1, el.c2};
      if (el.env_site) for (int k = 0; k < 3; ++k) r_l[k] = a.site_pose[e * 7 + 4 + k];
      rot_fwd(qb, r_l, r);
      rot_fwd(qb, al_l, al);
      // w x r, then alpha x r + w x (w x r)
      const float wr[3] = {w[1] * r[2] - w[2] * r[1], w[2] * r[0] - w[0] * r[2], w[0] * r[1] - w[1] * r[0]};
      vec[0] = qa[0] + (al[1] * r[2] - al[2] * r[1]) + (w[1] * wr[2] - w[2] * wr[1]) - el.q0;
      vec[1] = qa[1] + (al[2] * r[0] - al[0] * r[2]) + (w[2] * wr[0] - w[0] * wr[2]) - el.q1;
      vec[2] = qa[2] + (al[0] * r[1] - al[1] * r[0]) + (w[0] * wr[1] - w[1] * wr[0]) - el.q2;
    }
    float in_body[3], out[3];
    float qs[4] = {el.e0, el.e1, el.e2, el.e3};
    if (el.env_site) for (int k = 0; k < 4; ++k) qs[k] = a.site_pose[e * 7 + k];
    rot_inv(qb, vec[0], vec[1], vec[2], in_body);
    rot_inv(qs, in_body[0], in_body[1], in_body[2], out);
    v = out[el.comp];
  } else {
    float vec[3] = {el.c0, el.c1, el.c2}, out[3];
    if (el.src != KS_SRC_CONST) {
      const float* p = a.src[el.src] + e * a.src_dim[el.src] + el.index;
      vec[0] = p[0]; vec[1] = p[1]; vec[2] = p[2];
    }
    rot_inv(a.src[KS_SRC_QPOS] + e * a.nq + 3, vec[0], vec[1], vec[2], out);
    v = out[el.comp];
  }
  if (a.obs) a.obs[idx] = v;
  const uint64_t step = a.rng.step + (a.rng.step_base ? *a.rng.step_base : 0ull);
  if (el.bias.kind != KS_NOISE_NONE && a.fresh && a.fresh[e]) {  // a new episode: new bias draws (rl.py:1110-1117)
    float z, w;
    if (a.bias_redraw) {
      z = a.bias_redraw[2 * idx];
      w = a.bias_redraw[2 * idx + 1];
    } else {
      const Philox4 r = draw(a.rng.seed, step, kRngObsBias, (uint64_t)e, (uint32_t)k);
      z = normal_from(r.x, r.y);
      w = erff(z * 0.70710678118654752440f);
    }
    a.bias_draw[2 * idx] = z;
    a.bias_draw[2 * idx + 1] = w;
  }
  if (a.noisy) {
    float nv = v;
    if (el.n_noise > 0) {
      float z, w;
      if (a.noise_normal && a.noise_uniform) {
        z = a.noise_normal[idx];
        w = 2.f * a.noise_uniform[idx] - 1.f;
      } else {
        const Philox4 r = draw(a.rng.seed, step, kRngObsNoise, (uint64_t)e, (uint32_t)k);
        z = normal_from(r.x, r.y);
        w = erff(z * 0.70710678118654752440f);  // the uniform that the same random bits give
      }
      for (int j = 0; j < el.n_noise; ++j) nv = apply_stage(el.noise[j], nv, z, w, a.level);
    }
    if (el.bias.kind != KS_NOISE_NONE) nv = apply_stage(el.bias, nv, a.bias_draw[2 * idx], a.bias_draw[2 * idx + 1], a.level);
    a.noisy[idx] = nv;
  }
}

__global__ __launch_bounds__(256) void observe_kernel(ObserveArgs a) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= a.N * a.obs_dim) return;
  observe_one(a, idx);
}

struct TerminateArgs {
  const DevTerms* t;
  int64_t N;
  float level;
  float *qpos, *qvel, *warm, *time, *last_ctrl;
  int8_t* components;
  uint8_t *done, *success;
  float *traj_qpos, *traj_qvel, *traj_time;
  uint8_t* reset_mask;
  int32_t* episode_length;
  const float* reset_uniform;
  KsRng rng;
  int apply_reset, nq, nv, nu, n_terms, random_heading, nonfinite_terminates;
  int n_events;
  float event_interval[KS_MAX_EVENTS][2];
  float* event_state;
  const float* event_reset_uniform;
  float* event_force;
  const float* contact_dist;
  int ns, na;
  float *action_latency, *zero_offset, *act_action_bias, *act_torque_bias, *act_kp_scale, *act_kd_scale, *act_torque_limit_scale;
  float latency_lo, latency_hi;
  KsRandomVar zero_offset_rv, action_bias_rv, torque_bias_rv, kp_scale_rv, kd_scale_rv, torque_limit_scale_rv;
  const float *episode_uniform, *episode_normal;
  int redraw;  // any of the per-episode buffers is given
  const float *reset_pitch_roll_uniform, *reset_motion_qpos, *reset_hfield;
  const int32_t* reset_frame;
  int reset_motion_frames, hfield_nx, hfield_ny;
  float reset_motion_dt;
};

// value of a random variable from its standard draws (ksim/noise.py:74-121)
__device__ inline float rv_value(const KsRandomVar& rv, float u, float z, float s) {
  const float w = rv.same_key ? erff(z * 0.70710678118654752440f) : u;
  return rv.mean + s * (rv.std * z + rv.mag * w);
}

// A 256-thread workgroup owns kTermEnvs consecutive envs.  The state rows of those envs are contiguous in memory,
// so the transition copies, the finiteness check and the reset writes all walk them as flat, coalesced
// arrays; the per-env decisions (one lane per env, a handful of scalars each) sit between the flat passes.
// Termination comparisons are strict and done in fp32 on the stored state, so the integer outputs are
// reproducible bit for bit.
constexpr int kTermEnvs = 32;
// In the launch that also observes, a workgroup takes fewer envs: the observation is one thread per element, and with 32
// envs per workgroup a launch over a few thousand envs would be too few workgroups to fill the chip.
constexpr int kTermObsEnvs = 8;

// s_bad: non-finite state seen; s_reset: env starts a fresh episode; s_frame: its frame of the reference motion
template <int ENVS>
__device__ __forceinline__ void terminate_block(const TerminateArgs& a, int* s_bad, int* s_reset, int* s_frame) {
  const KsTermsDesc& d = a.t->d;
  const int tid = threadIdx.x;
  const int64_t e0 = (int64_t)blockIdx.x * ENVS;
  const int ne = a.N - e0 < ENVS ? (int)(a.N - e0) : ENVS;
  const int nq = a.nq, nv = a.nv, nu = a.nu;
  if (tid < ENVS) s_bad[tid] = 0;
  __syncthreads();
  // ---- flat pass 1: transition record (post-step state) and finiteness
  float* qb = a.qpos + e0 * nq;
  float* vb = a.qvel + e0 * nv;
  for (int idx = tid; idx < ne * nq; idx += 256) {
    const float x = qb[idx];
    if (a.traj_qpos) a.traj_qpos[e0 * nq + idx] = x;
    if (a.nonfinite_terminates && !(fabsf(x) <= 3.0e38f)) s_bad[idx / nq] = 1;  // true for NaN and inf
  }
  for (int idx = tid; idx < ne * nv; idx += 256) {
    const float x = vb[idx];
    if (a.traj_qvel) a.traj_qvel[e0 * nv + idx] = x;
    if (a.nonfinite_terminates && !(fabsf(x) <= 3.0e38f)) s_bad[idx / nv] = 1;
  }
  __syncthreads();
  // ---- one lane per env: terminations, done / success, reset decision
  if (tid < ne) {
    const int64_t e = e0 + tid;
    const float* q = qb + tid * nq;
    const float* v = vb + tid * nv;
    const float tm = a.time ? a.time[e] : 0.f;
    bool done = false, succ = true;
    for (int j = 0; j < a.n_terms; ++j) {
      const KsTermDesc td = d.terms[j];
      bool fire = false;
      switch (td.kind) {
        case KS_TERM_MIN_HEIGHT: fire = q[2] < td.p0; break;
        case KS_TERM_BAD_Z: {
          const float lo = (td.p2 - td.p0) * a.level + td.p0, hi = (td.p3 - td.p1) * a.level + td.p1;
          fire = (q[2] < lo) || (q[2] > hi);
        } break;
        case KS_TERM_NOT_UPRIGHT: {
          float out[3];
          rot_inv(q + 3, 0.f, 0.f, 1.f, out);
          fire = acosf(fminf(fmaxf(out[2], -1.f), 1.f)) > td.p0;
        } break;
        case KS_TERM_BAD_VELOCITY: fire = sqrtf(v[0] * v[0] + v[1] * v[1] + v[2] * v[2]) > td.p0; break;
        case KS_TERM_FAR_FROM_ORIGIN: fire = sqrtf(q[0] * q[0] + q[1] * q[1] + q[2] * q[2]) > td.p0; break;
        case KS_TERM_EPISODE_LENGTH: fire = (tm > td.p0) && !(td.p1 >= 0.f && a.level < td.p1); break;
        case KS_TERM_ILLEGAL_CONTACT: {
          const unsigned mask = (unsigned)td.p1;
          for (int sidx = 0; sidx < a.ns; ++sidx)
            fire |= ((mask >> sidx) & 1u) && a.contact_dist[e * a.ns + sidx] < td.p0;
        } break;
        default: break;
      }
      const int8_t val = fire ? (int8_t)td.value : (int8_t)0;
      if (a.components) a.components[(int64_t)j * a.N + e] = val;
      done |= val != 0;
      succ &= val != -1;
    }
    if (s_bad[tid]) { done = true; succ = false; }
    succ = succ && done;
    if (a.done) a.done[e] = done ? 1 : 0;
    if (a.success) a.success[e] = succ ? 1 : 0;
    if (a.traj_time) a.traj_time[e] = tm;
    const bool do_reset = a.apply_reset == 2 || (done && a.apply_reset == 1);
    s_reset[tid] = do_reset ? 1 : 0;
    if (a.reset_mask) a.reset_mask[e] = do_reset ? 1 : 0;
    if (a.episode_length) a.episode_length[e] = do_reset ? 0 : a.episode_length[e] + 1;
    int frame = 0;
    if (do_reset && a.reset_motion_qpos) {  // resets.py:291: randint(0, num_frames)
      if (a.reset_frame) frame = a.reset_frame[e];
      else {
        const uint64_t st = a.rng.step + (a.rng.step_base ? *a.rng.step_base : 0ull);
        frame = (int)(u01(draw(a.rng.seed, st, kRngReset, (uint64_t)e, (uint32_t)nq + 2u).x) * (float)a.reset_motion_frames);
      }
      frame = frame < 0 ? 0 : (frame >= a.reset_motion_frames ? a.reset_motion_frames - 1 : frame);
    }
    s_frame[tid] = frame;
    if (do_reset && a.time) a.time[e] = a.reset_motion_qpos ? (float)frame * a.reset_motion_dt : 0.f;
    if (do_reset)
      for (int k = 0; k < a.n_events; ++k) {
        float u;
        if (a.event_reset_uniform) u = a.event_reset_uniform[e * a.n_events + k];
        else u = u01(draw(a.rng.seed, a.rng.step + (a.rng.step_base ? *a.rng.step_base : 0ull), kRngEvent, (uint64_t)e, 0x10000u + k).x);
        a.event_state[(int64_t)k * a.N + e] = a.event_interval[k][0] + u * (a.event_interval[k][1] - a.event_interval[k][0]);
        if (a.event_force)  // no force held at the start of an episode (events.py:360-365)
          for (int j = 0; j < KS_EVENT_FORCE_STATE; ++j) a.event_force[((int64_t)k * a.N + e) * KS_EVENT_FORCE_STATE + j] = 0.f;
      }
  }
  __syncthreads();
  // ---- flat pass 2: fresh episodes (engine.py:207-246): qpos from the reset table, everything else zero
  const uint64_t step = a.rng.step + (a.rng.step_base ? *a.rng.step_base : 0ull);
  for (int idx = tid; idx < ne * nq; idx += 256) {
    const int le = idx / nq, i = idx - le * nq;
    if (!s_reset[le]) continue;
    const int64_t e = e0 + le;
    float u;
    if (a.reset_uniform) u = a.reset_uniform[e * (nq + 1) + i];
    else u = 2.f * u01(draw(a.rng.seed, step, kRngReset, (uint64_t)e, (uint32_t)i).x) - 1.f;
    const float mag = d.reset_mag[i] * (d.reset_by_level[i] ? a.level : 1.f);
    float start = d.reset_base[i];
    if (d.reset_from_motion[i] && a.reset_motion_qpos) start += a.reset_motion_qpos[(int64_t)s_frame[le] * nq + i];
    const float x = start + u * mag;
    qb[idx] = fminf(fmaxf(x, d.reset_lo[i]), d.reset_hi[i]);
  }
  if (d.reset_hfield && a.reset_hfield && nq >= 3) {
    __syncthreads();  // x and y written above are read back by the env's own lane
    if (tid < ne && s_reset[tid]) {
      float* q = qb + tid * nq;
      const int nx = a.hfield_nx, ny = a.hfield_ny;
      int ix = (int)(((q[0] + d.hfield_bound[0]) / (2.f * d.hfield_bound[0])) * (float)(nx - 1));  // truncation, as astype(int32)
      int iy = (int)(((q[1] + d.hfield_bound[1]) / (2.f * d.hfield_bound[1])) * (float)(ny - 1));
      ix = ix < 0 ? 0 : (ix > nx - 1 ? nx - 1 : ix);
      iy = iy < 0 ? 0 : (iy > ny - 1 ? ny - 1 : iy);
      q[2] = a.reset_hfield[(int64_t)ix * ny + iy] + d.reset_base[2];
    }
  }
  for (int idx = tid; idx < ne * nv; idx += 256) {
    if (!s_reset[idx / nv]) continue;
    vb[idx] = 0.f;
    if (a.warm) a.warm[e0 * nv + idx] = 0.f;
  }
  if (a.last_ctrl)
    for (int idx = tid; idx < ne * a.na; idx += 256)
      if (s_reset[idx / a.na]) a.last_ctrl[e0 * a.na + idx] = 0.f;
  // ---- per-episode quantities of the fresh episodes (engine.py:222-245, actuators.py:219-238)
  if (a.redraw) {
    const int ned = 3 * nu + 4;
    for (int idx = tid; idx < ne * ned; idx += 256) {
      const int le = idx / ned, j = idx - le * ned;
      if (!s_reset[le]) continue;
      const int64_t e = e0 + le;
      float u, z;
      if (a.episode_uniform && a.episode_normal) {
        u = a.episode_uniform[e * ned + j];
        z = a.episode_normal[e * ned + j];
      } else {
        const Philox4 r = draw(a.rng.seed, step, kRngEpisode, (uint64_t)e, (uint32_t)j);
        u = a.episode_uniform ? a.episode_uniform[e * ned + j] : 2.f * u01(r.x) - 1.f;
        z = a.episode_normal ? a.episode_normal[e * ned + j] : normal_from(r.y, r.z);
      }
      if (j == 0) {
        if (a.action_latency) a.action_latency[e] = a.latency_lo * a.level + 0.5f * (u + 1.f) * ((a.latency_hi - a.latency_lo) * a.level);
      } else if (j <= nu) {
        if (a.zero_offset) a.zero_offset[e * nu + (j - 1)] = rv_value(a.zero_offset_rv, u, z, a.level);
      } else if (j <= 2 * nu) {
        if (a.act_action_bias) a.act_action_bias[e * nu + (j - 1 - nu)] = rv_value(a.action_bias_rv, u, z, 1.f);
      } else if (j <= 3 * nu) {
        if (a.act_torque_bias) a.act_torque_bias[e * nu + (j - 1 - 2 * nu)] = rv_value(a.torque_bias_rv, u, z, 1.f);
      } else if (j == 3 * nu + 1) {
        if (a.act_kp_scale) a.act_kp_scale[e] = rv_value(a.kp_scale_rv, u, z, 1.f);
      } else if (j == 3 * nu + 2) {
        if (a.act_kd_scale) a.act_kd_scale[e] = rv_value(a.kd_scale_rv, u, z, 1.f);
      } else {
        if (a.act_torque_limit_scale) a.act_torque_limit_scale[e] = rv_value(a.torque_limit_scale_rv, u, z, 1.f);
      }
    }
  }
  if ((a.random_heading || d.reset_pitch_roll) && nq >= 7) {
    __syncthreads();  // the base orientation written above is read back by the env's own lane
    if (tid < ne && s_reset[tid]) {
      const int64_t e = e0 + tid;
      float* q = qb + tid * nq;
      auto heading = [&]() {
        float u;
        if (a.reset_uniform) u = a.reset_uniform[e * (nq + 1) + nq];
        else u = 2.f * u01(draw(a.rng.seed, step, kRngReset, (uint64_t)e, (uint32_t)nq).x) - 1.f;
        const float h = 0.5f * 3.14159265358979323846f * u;  // yaw/2, yaw ~ U(-pi, pi)
        const float cw = cosf(h), sz = sinf(h);
        const float w = q[3], x = q[4], y = q[5], z = q[6];
        q[3] = w * cw - z * sz; q[4] = x * cw + y * sz; q[5] = y * cw - x * sz; q[6] = z * cw + w * sz;
      };
      auto pitch_roll = [&]() {
        // one draw for both angles: the reference samples pitch and roll from the same key (resets.py:348-349)
        float u;
        if (a.reset_pitch_roll_uniform) u = a.reset_pitch_roll_uniform[e];
        else u = u01(draw(a.rng.seed, step, kRngReset, (uint64_t)e, (uint32_t)nq + 1u).x);
        const float pitch = d.reset_pitch[0] + u * (d.reset_pitch[1] - d.reset_pitch[0]);
        const float roll = d.reset_roll[0] + u * (d.reset_roll[1] - d.reset_roll[0]);
        const float cr = cosf(0.5f * roll), sr = sinf(0.5f * roll), cp = cosf(0.5f * pitch), sp = sinf(0.5f * pitch);
        const float bw = cr * cp, bx = sr * cp, by = cr * sp, bz = -sr * sp;  // euler (roll, pitch, 0) as a quaternion
        const float w = q[3], x = q[4], y = q[5], z = q[6];
        q[3] = w * bw - x * bx - y * by - z * bz;
        q[4] = w * bx + x * bw + y * bz - z * by;
        q[5] = w * by - x * bz + y * bw + z * bx;
        q[6] = w * bz + x * by - y * bx + z * bw;
      };
      if (d.reset_pitch_roll == 2) pitch_roll();
      if (a.random_heading) heading();
      if (d.reset_pitch_roll == 1) pitch_roll();
    }
  }
}

__global__ __launch_bounds__(256) void terminate_kernel(TerminateArgs a) {
  __shared__ int s_bad[kTermEnvs], s_reset[kTermEnvs], s_frame[kTermEnvs];
  terminate_block<kTermEnvs>(a, s_bad, s_reset, s_frame);
}

// The termination pass of control step t and the observation of step t + 1 in one launch: a workgroup takes the decisions
// for its envs, resets the finished ones, and then observes those same envs in the state the next step will start from
// (one thread per element, striding over the workgroup's envs).  What the first half wrote (state rows, the reset mask that
// the observation takes as its `fresh` flags) is read back by other threads of the same workgroup only.
__global__ __launch_bounds__(256) void terminate_observe_kernel(TerminateArgs a, ObserveArgs o) {
  __shared__ int s_bad[kTermObsEnvs], s_reset[kTermObsEnvs], s_frame[kTermObsEnvs];
  terminate_block<kTermObsEnvs>(a, s_bad, s_reset, s_frame);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  const int64_t e0 = (int64_t)blockIdx.x * kTermObsEnvs;
  const int ne = a.N - e0 < kTermObsEnvs ? (int)(a.N - e0) : kTermObsEnvs;
  for (int i = threadIdx.x; i < ne * o.obs_dim; i += 256) observe_one(o, e0 * o.obs_dim + i);
}

__global__ __launch_bounds__(256) void sample_action_kernel(int64_t n, int nu, const float* __restrict__ mean,
                                                            const float* __restrict__ log_std,
                                                            const float* __restrict__ noise, KsRng rng, float clip_max,
                                                            float* __restrict__ action) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  const int64_t e = idx / nu;
  const int u = (int)(idx - e * nu);
  float a = mean[idx];
  if (log_std) {
    float z;
    if (noise) z = noise[idx];
    else {
      const Philox4 r = draw(rng.seed, rng.step + (rng.step_base ? *rng.step_base : 0ull), kRngAction, (uint64_t)e, (uint32_t)u);
      z = normal_from(r.x, r.y);
    }
    a += expf(log_std[u]) * z;
  }
  if (a != a) a = 0.f;                         // NaN -> 0, rl.py:999-1000
  a = fminf(fmaxf(a, -clip_max), clip_max);    // rl.py:1001
  action[idx] = a;
}

// Gaussian head with a state-dependent standard deviation: the network emits (mean, raw std) per actuator.
__global__ __launch_bounds__(256) void sample_action_head_kernel(int64_t n, int nu, const float* __restrict__ raw,
                                                                 KsGaussianHead hd, const float* __restrict__ noise,
                                                                 KsRng rng, float clip_max, float* __restrict__ action,
                                                                 float* __restrict__ mean_out, float* __restrict__ std_out,
                                                                 float* __restrict__ logp_out) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  const int64_t e = idx / nu;
  const int u = (int)(idx - e * nu);
  const float mean = raw[e * 2 * nu + u] + (hd.mean_bias ? hd.mean_bias[u] : 0.f);
  const float r = raw[e * 2 * nu + nu + u];
  const float sp = r > 20.f ? r : log1pf(expf(r));  // softplus, linear where exp would overflow
  const float sd = fminf((sp + hd.min_std) * hd.var_scale, hd.max_std);
  float z = 0.f;
  if (!hd.deterministic) {
    if (noise) z = noise[idx];
    else {
      const Philox4 p = draw(rng.seed, rng.step + (rng.step_base ? *rng.step_base : 0ull), kRngAction, (uint64_t)e, (uint32_t)u);
      z = normal_from(p.x, p.y);
    }
  }
  float a = mean + sd * z;
  if (logp_out) logp_out[idx] = -0.5f * z * z - logf(sd) - 0.91893853320467274178f;  // log N(a; mean, sd), (a - mean) / sd = z
  if (mean_out) mean_out[idx] = mean;
  if (std_out) std_out[idx] = sd;
  if (a != a) a = 0.f;                         // NaN -> 0, rl.py:999-1000
  a = fminf(fmaxf(a, -clip_max), clip_max);    // rl.py:1001
  action[idx] = a;
}

// Action filters: one lane per (env, joint); the state row of an env is position-like | velocity-like.
__global__ __launch_bounds__(256) void action_filter_kernel(int64_t n, int nu, int kind, float dt, float p0,
                                                            const float* __restrict__ lo, const float* __restrict__ hi,
                                                            const float* __restrict__ x, float* __restrict__ state,
                                                            const uint8_t* __restrict__ fresh, const float* __restrict__ init,
                                                            float* __restrict__ y) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  const int64_t e = idx / nu;
  const int j = (int)(idx - e * nu);
  const float v = x[idx];
  if (kind == KS_FILTER_CLIP_POSITIONS) { y[idx] = fminf(fmaxf(v, lo[j]), hi[j]); return; }
  if (kind == KS_FILTER_TANH_POSITIONS) { y[idx] = tanhf(v) * (hi[j] - lo[j]) + lo[j]; return; }
  float* st = state + e * 2 * nu;
  float pos = st[j], vel = st[nu + j];
  if (fresh && fresh[e]) { pos = init ? init[idx] : 0.f; vel = 0.f; }
  if (kind == KS_FILTER_LOWPASS) {
    const float alpha = dt / (1.f / (6.28318530717958647692f * p0) + dt);
    pos = pos + alpha * (v - pos);
  } else if (kind == KS_FILTER_CLIP_ACCELERATION) {
    const float cv = (v - pos) / dt;
    const float ca = fminf(fmaxf((cv - vel) / dt, -p0), p0);
    vel = vel + ca * dt;
    pos = pos + vel * dt;
  } else if (kind == KS_FILTER_INTEGRATE_VELOCITY) {
    pos = pos + v * dt;
  } else {  // KS_FILTER_INTEGRATE_ACCELERATION
    vel = fminf(fmaxf(vel + v * dt, -p0), p0);
    pos = pos + vel * dt;
  }
  st[j] = pos;
  st[nu + j] = vel;
  y[idx] = pos;
}

// Mixture-of-Gaussians head: one lane per (env, action dimension) walks its K components three times (softmax
// normaliser, component pick by inverse CDF, log-density of the sample), all in registers.
__global__ __launch_bounds__(256) void sample_action_mixture_kernel(int64_t n, int nu, const float* __restrict__ raw,
                                                                    KsMixtureHead hd, const float* __restrict__ uniform,
                                                                    const float* __restrict__ noise, KsRng rng,
                                                                    float clip_max, float* __restrict__ action,
                                                                    float* __restrict__ logp_out, int* __restrict__ comp_out,
                                                                    const float* __restrict__ given) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  const int64_t e = idx / nu;
  const int u = (int)(idx - e * nu);
  const int K = hd.num_mixtures;
  const float* rm = raw + e * 3 * nu * K + (int64_t)u * K;
  const float* rs = rm + (int64_t)nu * K;
  const float* rl = rs + (int64_t)nu * K;
  const float bias = hd.mean_bias ? hd.mean_bias[u] : 0.f;
  const float lo = hd.clip_lo ? hd.clip_lo[u] : -INFINITY, hi = hd.clip_hi ? hd.clip_hi[u] : INFINITY;
  float mean[KS_MAX_MIXTURES], sd[KS_MAX_MIXTURES], lg[KS_MAX_MIXTURES];
  float lmax = -INFINITY;
  int best = 0;
#pragma unroll
  for (int k = 0; k < KS_MAX_MIXTURES; ++k) {
    if (k < K) {
      mean[k] = fminf(fmaxf(rm[k] + bias, lo), hi);
      const float r = rs[k];
      const float sp = r > 20.f ? r : log1pf(expf(r));
      sd[k] = fminf((sp + hd.min_std) * hd.var_scale, hd.max_std);
      lg[k] = rl[k];
      if (lg[k] > lmax) { lmax = lg[k]; best = k; }
    } else {
      mean[k] = 0.f; sd[k] = 1.f; lg[k] = -INFINITY;
    }
  }
  float zsum = 0.f;
#pragma unroll
  for (int k = 0; k < KS_MAX_MIXTURES; ++k) zsum += k < K ? expf(lg[k] - lmax) : 0.f;
  const float lse = lmax + logf(zsum);  // log of the softmax normaliser
  float uu = 0.f, z = 0.f;
  int pick = best;
  if (!hd.deterministic) {
    if (uniform && noise) { uu = uniform[idx]; z = noise[idx]; }
    else {
      const Philox4 p = draw(rng.seed, rng.step + (rng.step_base ? *rng.step_base : 0ull), kRngAction, (uint64_t)e, (uint32_t)u);
      z = noise ? noise[idx] : normal_from(p.x, p.y);
      uu = uniform ? uniform[idx] : u01(p.z);
    }
    // inverse CDF: the first component whose cumulative probability exceeds the draw (the last one on rounding)
    float cum = 0.f;
    pick = K - 1;
    bool found = false;
#pragma unroll
    for (int k = 0; k < KS_MAX_MIXTURES; ++k) {
      if (k < K) {
        cum += expf(lg[k] - lse);
        if (!found && cum > uu) { pick = k; found = true; }
      }
    }
  }
  float pm = 0.f, ps = 1.f;
#pragma unroll
  for (int k = 0; k < KS_MAX_MIXTURES; ++k)
    if (k == pick) { pm = mean[k]; ps = sd[k]; }
  float a = hd.deterministic ? pm : pm + ps * z;
  if (given) a = given[idx];  // log-density of a recorded action instead of a fresh sample
  if (logp_out) {
    float t[KS_MAX_MIXTURES], tmax = -INFINITY;
#pragma unroll
    for (int k = 0; k < KS_MAX_MIXTURES; ++k) {
      const float d = (a - mean[k]) / sd[k];
      t[k] = k < K ? (lg[k] - lse) - 0.5f * d * d - logf(sd[k]) - 0.91893853320467274178f : -INFINITY;
      tmax = fmaxf(tmax, t[k]);
    }
    float acc = 0.f;
#pragma unroll
    for (int k = 0; k < KS_MAX_MIXTURES; ++k) acc += k < K ? expf(t[k] - tmax) : 0.f;
    logp_out[idx] = tmax + logf(acc);
  }
  if (comp_out) comp_out[idx] = pick;
  if (!action) return;
  if (a != a) a = 0.f;
  a = fminf(fmaxf(a, -clip_max), clip_max);
  action[idx] = a;
}

// ---------------------------------------------------------------------------------------------
// Rewards over a time-major rollout.  One lane per (t, env).
// Action differences follow rewards.py:410-460: v(t) = a[t]-a[t-1], A(t) = v(t)-v(t-1),
// J(t) = A(t)-A(t-1), each zeroed when the step before it ended an episode, and the first
// 1 / 2 / 3 steps of the rollout masked to zero.
// ---------------------------------------------------------------------------------------------
__device__ inline float kernel_with_penalty(float x, float scale, float sq, float ab) {
  return fabsf(x) * -ab + x * x * -sq + expf(-(x * x) / (2.f * scale * scale));
}

__device__ inline float dist3(const float* a, const float* b) {
  const float x = a[0] - b[0], y = a[1] - b[1], z = a[2] - b[2];
  return sqrtf(x * x + y * y + z * z);
}

// first / second / third difference (order 1 / 2 / 3) of x along the rollout from x(t), x(t-1), x(t-2), x(t-3) (already clamped to
// the rollout's first step, which is the reference's edge padding); d_k says that step t - k was done, which zeroes every
// difference taken across it (rewards.py:469-508)
__device__ inline float smooth_difference(int order, float x0, float x1, float x2, float x3, bool d1, bool d2, bool d3) {
  const float v0 = d1 ? 0.f : x0 - x1;
  if (order == 1) return v0;
  const float v1 = d2 ? 0.f : x1 - x2;
  const float A0 = d1 ? 0.f : v0 - v1;
  if (order == 2) return A0;
  const float v2 = d3 ? 0.f : x2 - x3;
  const float A1 = d2 ? 0.f : v1 - v2;
  return d1 ? 0.f : A0 - A1;
}

__global__ __launch_bounds__(256) void rewards_kernel(KsRewardIO io) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t TN = io.T * io.N;
  if (idx >= TN) return;
  const int64_t t = idx / io.N;
  const float* q = io.qpos ? io.qpos + idx * io.nq : nullptr;
  const float* v = io.qvel ? io.qvel + idx * io.nv : nullptr;
  const bool dn = io.done[idx] != 0, sc = io.success && io.success[idx] != 0;
  const bool d1 = t >= 1 && io.done[idx - io.N] != 0;
  const bool d2 = t >= 2 && io.done[idx - 2 * io.N] != 0;
  const bool d3 = t >= 3 && io.done[idx - 3 * io.N] != 0;
  float total = 0.f;
  for (int j = 0; j < io.n_rewards; ++j) {
    const KsRewardDesc r = io.rewards[j];
    float val = 0.f;
    switch (r.kind) {
      case KS_REW_STAY_ALIVE: {
        const float alive = 1.0f / r.p0;
        val = dn ? (sc ? (r.p2 != 0.f ? r.p1 : alive) : -1.0f) : alive;
      } break;
      case KS_REW_BASE_HEIGHT: {
        const float x = q[2] - r.p0;
        val = expf(-(x * x) / (2.f * r.p1 * r.p1));
      } break;
      case KS_REW_BASE_HEIGHT_RANGE: {
        const float z = q[2];
        val = fmaxf(1.0f - fmaxf(fmaxf(r.p0 - z, z - r.p1), 0.f) * r.p2, 0.f);
      } break;
      case KS_REW_ACTION_VEL:
      case KS_REW_ACTION_ACC:
      case KS_REW_ACTION_JERK: {
        const int order = r.kind - KS_REW_ACTION_VEL + 1;
        float s = 0.f;
        if (t >= order) {
          const float* a0 = io.action + idx * io.nu;
          for (int u = 0; u < io.nu; ++u) {
            const float x0 = a0[u], x1 = a0[u - io.N * io.nu];
            const float v0 = d1 ? 0.f : x0 - x1;
            float x = v0;
            if (order >= 2) {
              const float x2 = a0[u - 2 * io.N * io.nu];
              const float v1 = d2 ? 0.f : x1 - x2;
              const float A0 = d1 ? 0.f : v0 - v1;
              x = A0;
              if (order == 3) {
                const float x3 = a0[u - 3 * io.N * io.nu];
                const float v2 = d3 ? 0.f : x2 - x3;
                const float A1 = d2 ? 0.f : v1 - v2;
                x = d1 ? 0.f : A0 - A1;
              }
            }
            s += r.norm == KS_NORM_L1 ? fabsf(x) : x * x;
          }
          s /= (float)io.nu;
        }
        val = s;
      } break;
      case KS_REW_UPRIGHT_ANGVEL: val = kernel_with_penalty(v[4], r.p0, r.p1, r.p2); break;
      case KS_REW_UPRIGHT_LINVEL: val = kernel_with_penalty(v[2], r.p0, r.p1, r.p2); break;
      case KS_REW_UPRIGHT_POSE: {
        float zb[3];
        rot_inv(q + 3, 0.f, 0.f, 1.f, zb);
        val = kernel_with_penalty(atan2f(zb[0], zb[2]), r.p0, r.p1, r.p2);
      } break;
      case KS_REW_AMP: {
        const float d = io.disc_logits[idx] - 1.0f;
        val = fmaxf(0.f, 1.0f - 0.25f * d * d);
      } break;
      case KS_REW_STATEFUL: val = io.stateful[(int64_t)r.norm * TN + idx]; break;
      case KS_REW_LINVEL_CMD: {
        const float* cmd = io.command + idx * io.command_dim + r.index;
        float lv[3];
        rot_inv(q + 3, v[0], v[1], v[2], lv);
        float x;
        if (r.norm == 0) x = sqrtf(lv[0] * lv[0] + lv[1] * lv[1]) - cmd[0];
        else if (r.norm == 1) x = atan2f(lv[1], lv[0]) - cmd[1];
        else if (r.norm == 2) x = lv[0] - cmd[2];
        else x = lv[1] - cmd[3];
        val = kernel_with_penalty(x, r.p0, r.p1, r.p2);
        if (r.norm != 0 && fabsf(cmd[0]) < r.p3) val = 0.f;
      } break;
      case KS_REW_ANGVEL_CMD: {
        const float c = io.command[idx * io.command_dim + r.index], w = v[5];
        if (r.norm == 0) {
          val = kernel_with_penalty(w - c, r.p0, r.p1, r.p2);
        } else {
          const float sw = fabsf(w) < r.p3 ? 0.f : (w > 0.f ? 1.f : -1.f);
          const float sc2 = fabsf(c) < r.p3 ? 0.f : (c > 0.f ? 1.f : -1.f);
          val = sw == sc2 ? 1.f : -1.f;
        }
      } break;
      case KS_REW_OFF_AXIS: {
        const float x = v[r.norm == 0 ? 2 : (r.norm == 1 ? 4 : 5)];
        val = expf(-(x * x) / (2.f * r.p0 * r.p0));
      } break;
      case KS_REW_MOTIONLESS: {
        const bool still = sqrtf(v[0] * v[0] + v[1] * v[1]) < r.p0 && v[5] < r.p1;
        float s2 = 0.f;
        for (int j = 6; j < io.nv; ++j) s2 += v[j] * v[j];
        val = still ? sqrtf(s2) : 0.f;
      } break;
      case KS_REW_FORCE: {
        const float* ob = io.obs + idx * io.obs_dim + r.index;
        float best = 0.f;
        for (int b = 0; b < r.norm; ++b) {
          const float n = sqrtf(ob[3 * b] * ob[3 * b] + ob[3 * b + 1] * ob[3 * b + 1] + ob[3 * b + 2] * ob[3 * b + 2]);
          const float e = fmaxf(n - r.p1, 0.f) / r.p0;
          best = b == 0 ? e * e : fmaxf(best, e * e);
        }
        val = best;
      } break;
      case KS_REW_JOINT_SMOOTH: {
        const int nj = io.nq - 7;
        const int64_t s1 = t >= 1 ? io.N * io.nq : 0, s2 = s1 + (t >= 2 ? io.N * io.nq : 0), s3 = s2 + (t >= 3 ? io.N * io.nq : 0);
        float s = 0.f;
        for (int u = 0; u < nj; ++u) {
          const float* a0 = q + 7 + u;
          const float x = smooth_difference(r.norm, a0[0], a0[-s1], a0[-s2], a0[-s3], d1, d2, d3);
          s += expf(-(x * x) / (2.f * r.p0 * r.p0));
        }
        val = s / (float)nj;
      } break;
      case KS_REW_AVOID_LIMITS: {
        const int nj = io.nq - 7;
        const float* lim = io.params + r.param_offset;
        float s = 0.f;
        for (int u = 0; u < nj; ++u) s += -fminf(q[7 + u] - lim[2 * u], 0.f) + fmaxf(q[7 + u] - lim[2 * u + 1], 0.f);
        val = s / (float)nj;
      } break;
      case KS_REW_TORQUE:
      case KS_REW_ENERGY: {
        const float* c = io.ctrl + idx * io.nu;
        const float* sc = io.params + r.param_offset;
        float s = 0.f;
        for (int u = 0; u < io.nu; ++u) s += fabsf(r.kind == KS_REW_TORQUE ? c[u] / sc[u] : c[u] / sc[u] * v[6 + u]);
        val = s / (float)io.nu;
      } break;
      case KS_REW_JOINT_DEVIATION: {
        const float* pr = io.params + r.param_offset;
        float s = 0.f;
        for (int k = 0; k < r.count; ++k) {
          const float x = (q[7 + (int)pr[3 * k]] - pr[3 * k + 1]) * pr[3 * k + 2];
          s += r.norm == KS_NORM_L1 ? fabsf(x) : x * x;
        }
        val = s;
      } break;
      case KS_REW_FLAT_BODY: {
        const float* pr = io.params + r.param_offset;
        const float* pl = pr + r.count;
        float s = 0.f;
        for (int k = 0; k < r.count; ++k) {
          float uv[3];
          rot_inv(io.xquat + (idx * io.nb + (int)pr[k]) * 4, pl[0], pl[1], pl[2], uv);
          s += uv[0] * pl[0] + uv[1] * pl[1] + uv[2] * pl[2];
        }
        val = s / (float)r.count;
      } break;
      case KS_REW_POSITION_TRACKING: {
        const float* pb = io.xpos + (idx * io.nb + r.index2) * 3;
        const float* p0 = io.xpos + (idx * io.nb + r.count) * 3;
        const float* cmd = io.command + idx * io.command_dim + r.index;
        float e = 0.f;
        for (int i = 0; i < 3; ++i) {
          const float x = (pb[i] - p0[i]) - cmd[i];
          e += r.norm == KS_NORM_L1 ? fabsf(x) : x * x;
        }
        val = expf(-(e * e) / (2.f * r.p0 * r.p0));
      } break;
      case KS_REW_NO_ROLL_ANGVEL: val = kernel_with_penalty(v[3], r.p0, r.p1, r.p2); break;
      case KS_REW_NO_ROLL_POSE: {
        float zb[3];
        rot_inv(q + 3, 0.f, 0.f, 1.f, zb);
        val = kernel_with_penalty(-atan2f(zb[1], zb[2]), r.p0, r.p1, r.p2);
      } break;
      case KS_REW_LINK_SMOOTH: {
        const int order = (int)r.p0;
        const int64_t st = io.N * io.nb * 3;
        const int64_t s1 = t >= 1 ? st : 0, s2 = s1 + (t >= 2 ? st : 0), s3 = s2 + (t >= 3 ? st : 0);
        float s = 0.f;
        for (int b = 1; b < io.nb; ++b) {
          const float* p = io.xpos + (idx * io.nb + b) * 3;
          // speeds |p(t - k) - p(t - k - 1)|, zeroed after a done step, then plain differences of those
          const float w0 = d1 ? 0.f : dist3(p, p - s1), w1 = d2 ? 0.f : dist3(p - s1, p - s2), w2 = d3 ? 0.f : dist3(p - s2, p - s3);
          const float A0 = d1 ? 0.f : w0 - w1;
          float x = A0;
          if (order == 3) {
            const float A1 = d2 ? 0.f : w1 - w2;
            x = d1 ? 0.f : A0 - A1;
          }
          s += r.norm == KS_NORM_L1 ? fabsf(x) : x * x;
        }
        val = s / (float)(io.nb - 1);
      } break;
      case KS_REW_FEET_SLIP: {
        const float* ob = io.obs + idx * io.obs_dim;
        float s = 0.f;
        for (int f = 0; f < r.norm; ++f) {
          bool touching = false;
          for (int c = 0; c < r.count; ++c) touching = touching || ob[r.index + c * r.norm + f] > 0.5f;
          const float* w = ob + r.index2 + 6 * f;
          const float n2 = w[0] * w[0] + w[1] * w[1] + w[2] * w[2] + w[3] * w[3] + w[4] * w[4] + w[5] * w[5];
          s += touching ? sqrtf(n2) : 0.f;
        }
        val = s;
      } break;
      case KS_REW_REACHABILITY: {
        const float* dm = io.params + r.param_offset;
        const float* a0 = io.action + idx * io.nu;
        float s = 0.f;
        for (int u = 0; u < io.nu; ++u) {
          const float x = fmaxf(0.f, fabsf(a0[u] - q[7 + u]) - dm[u]);
          s += r.norm == KS_NORM_L1 ? x : x * x;
        }
        val = s;
      } break;
      case KS_REW_JOINT_POSITION:
      case KS_REW_JOINT_VELOCITY_CMD: {
        const float* pr = io.params + r.param_offset;
        const float* cm = io.command + idx * io.command_dim + r.index;  // [start, target, total_time, num_steps, step_id]
        const float total_time = cm[2 * r.count], num_steps = cm[2 * r.count + 1], step_id = cm[2 * r.count + 2];
        float sum = 0.f;
        for (int k = 0; k < r.count; ++k) {
          const int jn = (int)pr[k];
          const float start = cm[k], target = cm[r.count + k];
          const float diff = r.kind == KS_REW_JOINT_POSITION ? start + (target - start) * step_id / num_steps - q[7 + jn]
                                                             : (target - start) / total_time - v[6 + jn];
          sum += kernel_with_penalty(diff, r.p0, r.p1, r.p2);
        }
        val = sum / (float)r.count;
      } break;
      case KS_REW_SINUSOIDAL_GAIT: {
        const float* ob = io.obs + idx * io.obs_dim + r.index;
        const float* hc = io.command + idx * io.command_dim + r.index2;
        float s = 0.f;
        for (int f = 0; f < r.norm; ++f) s += fabsf(ob[3 * f + 2] - hc[f]);
        val = 1.f - s / r.p0;
      } break;
      case KS_REW_INTERSECTION: {
        const float* ob = io.obs + idx * io.obs_dim + r.index;
        bool close = false;
        for (int i = 1; i < r.norm; ++i)
          for (int k = 0; k < i; ++k) close = close || dist3(ob + 3 * i, ob + 3 * k) < r.p0;
        val = close ? 1.f : 0.f;
      } break;
      default: break;
    }
    val *= r.scale;
    if (io.components) io.components[(int64_t)j * TN + idx] = val;
    total = j == 0 ? val : total + val;
  }
  if (io.use_clip_min) total = fmaxf(total, io.clip_min);
  if (io.use_clip_max) total = fminf(total, io.clip_max);
  if (io.total) io.total[idx] = total;
}

// One lane walks one env through the T steps of the rollout; every load of a step is coalesced over envs for the
// (T, N) arrays and strided by the row length for the (T, N, dim) ones.
__global__ __launch_bounds__(256) void reward_scan_kernel(KsRewardScanIO io) {
  const int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= io.N) return;
  const int64_t TN = io.T * io.N;
  const bool restart = io.done[(io.T - 1) * io.N + e] != 0;  // ksim/task/rl.py:206-214
  for (int sidx = 0; sidx < io.n_scans; ++sidx) {
    const KsRewardScanDesc& s = io.scans[sidx];
    float* cr = io.carry + e * io.carry_dim + s.carry_index;
    if (s.kind == KS_SCAN_SYMMETRY || s.kind == KS_SCAN_PAIRWISE_SYMMETRY) {
      // one update of the carry per rollout with the rollout's mean, then a second walk for the rewards; the carry row
      // itself is the accumulator, so any number of joints needs no registers
      const int n = s.kind == KS_SCAN_SYMMETRY ? s.n : 2;
      const float inv_t = 1.f / (float)io.T;
      for (int j = 0; j < n; ++j) {
        const float sign = (s.kind == KS_SCAN_PAIRWISE_SYMMETRY && j == 1 && s.flipped) ? -1.f : 1.f;
        float sum = 0.f;
        for (int64_t t = 0; t < io.T; ++t) sum += sign * (io.qpos[(t * io.N + e) * io.nq + 7 + s.joints[j]] - s.targets[j]);
        const float old = restart ? s.targets[j] : cr[j];
        cr[j] = old * (1.0f - s.alpha) + (sum * inv_t) * s.alpha;
      }
      for (int64_t t = 0; t < io.T; ++t) {
        const int64_t idx = t * io.N + e;
        const float* q = io.qpos + idx * io.nq + 7;
        float acc = 0.f;
        for (int j = 0; j < n; ++j) {
          const float sign = (s.kind == KS_SCAN_PAIRWISE_SYMMETRY && j == 1 && s.flipped) ? -1.f : 1.f;
          acc += sign * (q[s.joints[j]] - s.targets[j]) * -cr[j];
        }
        if (s.kind == KS_SCAN_SYMMETRY) {
          io.out[(int64_t)s.slot * TN + idx] = acc;
        } else {
          const float ql = q[s.joints[0]] - s.targets[0];
          const float qr = (s.flipped ? -1.f : 1.f) * (q[s.joints[1]] - s.targets[1]);
          io.out[(int64_t)s.slot * TN + idx] = kernel_with_penalty(ql - qr, s.kernel_scale, s.sq_scale, s.abs_scale);
          io.out[(int64_t)(s.slot + 1) * TN + idx] = acc;
        }
      }
      continue;
    }
    float c[3 * KS_MAX_SCAN_BODIES];  // counter k of body f at c[k * KS_MAX_SCAN_BODIES + f]; packed as k * n + f in memory
    const int nk = s.kind == KS_SCAN_FEET_AIR_TIME ? 3 : 1;
    for (int k = 0; k < 3; ++k)
      for (int f = 0; f < KS_MAX_SCAN_BODIES; ++f)
        c[k * KS_MAX_SCAN_BODIES + f] = (k < nk && f < s.n && !restart) ? cr[k * s.n + f] : 0.f;
    for (int64_t t = 0; t < io.T; ++t) {
      const int64_t idx = t * io.N + e;
      const float* ob = io.obs + idx * io.obs_dim;
      const float* qv = io.qvel + idx * io.nv;
      const bool dn = io.done[idx] != 0;
      if (s.kind == KS_SCAN_FEET_AIR_TIME) {
        const float* cmd = io.command ? io.command + idx * io.command_dim : nullptr;
        const bool lin = s.linvel_cmd_index >= 0 ? fabsf(cmd[s.linvel_cmd_index]) > s.linvel_threshold
                                                 : sqrtf(qv[0] * qv[0] + qv[1] * qv[1]) > s.linvel_threshold;
        const bool ang = s.angvel_cmd_index >= 0 ? fabsf(cmd[s.angvel_cmd_index]) > s.angvel_threshold
                                                 : qv[5] > s.angvel_threshold;
        const bool moving = (lin || ang) && !dn;
        float air = -INFINITY, gnd = -INFINITY, stat = -INFINITY;
        for (int f = 0; f < KS_MAX_SCAN_BODIES; ++f) {
          if (f >= s.n) break;
          bool contact = false;
          for (int g = 0; g < s.n_contact; ++g) contact |= ob[s.contact_index + g * s.n + f] > 0.5f;
          const float a_ = (!contact && moving) ? c[f] + 1.f : 0.f;
          const float g_ = (contact && moving) ? c[KS_MAX_SCAN_BODIES + f] + 1.f : 0.f;
          const float s_ = (contact && !moving) ? c[2 * KS_MAX_SCAN_BODIES + f] + 1.f : 0.f;
          c[f] = a_; c[KS_MAX_SCAN_BODIES + f] = g_; c[2 * KS_MAX_SCAN_BODIES + f] = s_;
          air = fmaxf(air, a_ < s.air_steps ? a_ / s.air_steps + s.bias : 0.f);
          gnd = fmaxf(gnd, g_ < s.gnd_steps ? g_ / s.gnd_steps + s.bias : -s.ground_penalty);
          stat = fmaxf(stat, fminf(fmaxf(s_ / s.gnd_steps, 0.f), 1.f) + s.bias);
        }
        io.out[(int64_t)s.slot * TN + idx] = air;
        io.out[(int64_t)(s.slot + 1) * TN + idx] = gnd;
        io.out[(int64_t)(s.slot + 2) * TN + idx] = stat;
      } else {
        const bool still = (sqrtf(qv[0] * qv[0] + qv[1] * qv[1]) < s.linvel_threshold && qv[5] < s.angvel_threshold) || dn;
        float best = -INFINITY;
        for (int f = 0; f < KS_MAX_SCAN_BODIES; ++f) {
          if (f >= s.n) break;
          bool contact = false;
          for (int g = 0; g < s.n_contact; ++g) contact |= ob[s.contact_index + g * s.n + f] > 0.5f;
          const float h = ob[s.position_index + 3 * f + 2];
          best = fmaxf(best, fminf(contact ? c[f] : 0.f, s.height));
          c[f] = (still || contact) ? 0.f : fmaxf(c[f], h);
        }
        io.out[(int64_t)s.slot * TN + idx] = best;
      }
    }
    if (s.kind == KS_SCAN_FEET_AIR_TIME) {
      for (int k = 0; k < 3; ++k)
        for (int f = 0; f < KS_MAX_SCAN_BODIES; ++f)
          if (f < s.n) cr[k * s.n + f] = c[k * KS_MAX_SCAN_BODIES + f];
    } else {
      for (int f = 0; f < KS_MAX_SCAN_BODIES; ++f)
        if (f < s.n) cr[f] = c[f];
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Commands: one thread per (env, command).
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void command_kernel(KsCommandIO io) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= io.N * io.n_commands) return;
  const int64_t e = idx / io.n_commands;
  const int k = (int)(idx - e * io.n_commands);
  const KsCommandDesc& c = io.commands[k];  // read in place: a copy of a runtime-indexed element would go through scratch memory
  float* cmd = io.command + e * io.command_dim + c.index;
  if (io.traj_command)
    for (int j = 0; j < c.dim; ++j) io.traj_command[e * io.command_dim + c.index + j] = cmd[j];
  if (c.kind == KS_CMD_CONST) return;
  float u[KS_COMMAND_DRAWS];
  if (io.uniform) {
    for (int j = 0; j < KS_COMMAND_DRAWS; ++j) u[j] = io.uniform[idx * KS_COMMAND_DRAWS + j];
  } else {
    const uint64_t step = io.rng.step + (io.rng.step_base ? *io.rng.step_base : 0ull);
    for (int j = 0; j < KS_COMMAND_DRAWS / 4; ++j) {
      const Philox4 a = draw(io.rng.seed, step, kRngCommand, (uint64_t)e, (uint32_t)((KS_COMMAND_DRAWS / 4) * k + j));
      u[4 * j] = u01(a.x); u[4 * j + 1] = u01(a.y); u[4 * j + 2] = u01(a.z); u[4 * j + 3] = u01(a.w);
    }
  }
  const bool fresh = io.all_fresh || (io.fresh && io.fresh[e]);
  const float* qv = io.qvel + e * io.nv;
  if (c.kind == KS_CMD_LINEAR_VELOCITY) {
    float vel = cmd[0], yaw = cmd[1], tv = cmd[4], ty = cmd[5];
    const bool redraw = fresh || u[4] < c.switch_prob;
    if (fresh) {  // measured speed and heading in the robot frame (commands.py:316-323)
      float lv[3];
      rot_inv(io.qpos + e * io.nq + 3, qv[0], qv[1], qv[2], lv);
      vel = sqrtf(lv[0] * lv[0] + lv[1] * lv[1]);
      yaw = atan2f(lv[1], lv[0]);
    }
    if (redraw) {  // commands.py:328-335
      tv = c.min_vel + u[0] * (c.max_vel - c.min_vel);
      ty = -c.max_yaw + u[1] * (2.f * c.max_yaw);
      const bool zero = u[2] < c.zero_prob, back = u[3] < c.backward_prob;
      tv = zero ? 0.f : (back ? -tv : tv);
      ty = zero ? 0.f : ty;
    } else {       // commands.py:349-357
      vel += fminf(fmaxf(tv - vel, -c.linear_accel), c.linear_accel) * c.ctrl_dt;
      yaw += fminf(fmaxf(ty - yaw, -c.angular_accel), c.angular_accel) * c.ctrl_dt;
    }
    cmd[0] = vel; cmd[1] = yaw; cmd[2] = vel * cosf(yaw); cmd[3] = vel * sinf(yaw); cmd[4] = tv; cmd[5] = ty;
  } else if (c.kind == KS_CMD_START_POSITION || c.kind == KS_CMD_START_QUATERNION) {
    if (fresh) {
      const float* q = io.qpos + e * io.nq + (c.kind == KS_CMD_START_POSITION ? 0 : 3);
      for (int j = 0; j < c.dim; ++j) cmd[j] = q[j];
    }
  } else if (c.kind == KS_CMD_SINUSOIDAL_GAIT) {
    const int feet = c.dim - 2;
    const float period = c.lo[0], max_h = c.lo[1], offset = c.lo[2], stance = c.lo[3], threshold = c.lo[4];
    float flag = 1.f, phase = 0.f;
    if (!fresh) {
      flag = cmd[0];
      const float stepped = cmd[1] + c.ctrl_dt / period;
      phase = flag != 0.f ? stepped - floorf(stepped) : 0.f;
      const bool moving = sqrtf(qv[0] * qv[0] + qv[1] * qv[1]) > threshold;
      if (!moving) { flag = 0.f; phase = 0.f; }
    }
    cmd[0] = flag; cmd[1] = phase;
    for (int f = 0; f < feet; ++f) {
      float pf = phase + (float)f / (float)feet;
      pf -= floorf(pf);
      const float prog = fminf(fmaxf((pf - stance) / (1.f - stance), 0.f), 1.f);
      cmd[2 + f] = (pf >= stance ? max_h * sinf(3.14159265358979323846f * prog) : 0.f) + offset;
    }
  } else if (c.kind == KS_CMD_JOINT_POSITION) {
    const int n = (c.dim - 3) / 2;
    const float step_id = cmd[2 * n + 2] + 1.f;
    if (fresh || step_id > cmd[2 * n + 1]) {  // commands.py:852-893: a new target, from where the joints are now
      const float* q = io.qpos + e * io.nq + 7;
      for (int j = 0; j < KS_MAX_VECTOR_COMMAND; ++j)
        if (j < n) {
          cmd[j] = q[c.joints[j]];
          cmd[n + j] = c.lo[j] + u[j] * (c.hi[j] - c.lo[j]);
        }
      float total = 0.f;
      for (int j = 0; j <= KS_MAX_VECTOR_COMMAND; ++j)
        if (j == n) total = c.min_time + u[j] * (c.max_time - c.min_time);  // the draw after the targets'
      cmd[2 * n] = total;
      cmd[2 * n + 1] = ceilf(total / c.ctrl_dt);
      cmd[2 * n + 2] = 0.f;
    } else {
      cmd[2 * n + 2] = step_id;
    }
  } else if (c.kind == KS_CMD_CARTESIAN_COORDINATE) {
    float box[3], new_speed = c.min_vel + u[3] * (c.max_vel - c.min_vel);
    for (int j = 0; j < 3; ++j) box[j] = c.lo[j] + u[j] * (c.hi[j] - c.lo[j]);
    if (fresh) {
      for (int j = 0; j < 3; ++j) cmd[j] = cmd[3 + j] = box[j];
      cmd[6] = new_speed;
    } else {
      float speed = cmd[6];
      const float dx = cmd[3] - cmd[0], dy = cmd[4] - cmd[1], dz = cmd[5] - cmd[2];
      const float dist = sqrtf(dx * dx + dy * dy + dz * dz);
      const bool reached = dist < c.ctrl_dt * speed * 0.5f;
      if ((reached && u[4] < c.switch_prob) || u[4] < c.jump_prob) {
        for (int j = 0; j < 3; ++j) cmd[3 + j] = box[j];
        speed = new_speed;
      }
      float dir[3] = {cmd[3] - cmd[0], cmd[4] - cmd[1], cmd[5] - cmd[2]};
      const float norm = sqrtf(dir[0] * dir[0] + dir[1] * dir[1] + dir[2] * dir[2]);
      const float move = fminf(speed * c.ctrl_dt, dist);  // the distance to the target held before this step
      for (int j = 0; j < 3; ++j) cmd[j] += (norm > 0.f ? dir[j] / norm : dir[j]) * move;
      cmd[6] = speed;
    }
  } else if (c.kind == KS_CMD_BASE_HEIGHT) {
    if (fresh || u[0] < c.switch_prob) cmd[0] = c.lo[0] + u[0] * (c.hi[0] - c.lo[0]);
  } else if (c.kind == KS_CMD_FLOAT_VECTOR || c.kind == KS_CMD_INT_VECTOR) {
    if (fresh || u[0] < c.switch_prob) {
      const bool zero = u[1] < c.zero_prob;
      for (int j = 0; j < c.dim; ++j) {
        float val;
        if (c.kind == KS_CMD_INT_VECTOR) val = fminf(floorf(c.lo[j] + u[2 + j] * (c.hi[j] + 1.f - c.lo[j])), c.hi[j]);
        else val = c.lo[j] + u[2 + j] * (c.hi[j] - c.lo[j]);
        cmd[j] = zero ? 0.f : val;
      }
    }
  } else {
    float vel = cmd[0], tv = cmd[1];
    const bool redraw = fresh || u[3] < c.switch_prob;
    if (redraw) {  // commands.py:470-478: on a switch the current value is re-read from the state as well
      tv = c.min_vel + u[0] * (c.max_vel - c.min_vel);
      tv = u[1] < 0.5f ? -tv : tv;
      tv = u[2] < c.zero_prob ? 0.f : tv;
      vel = qv[5];
    } else {
      vel += fminf(fmaxf(tv - vel, -c.angular_accel), c.angular_accel) * c.ctrl_dt;
    }
    cmd[0] = vel; cmd[1] = tv;
  }
}

}  // namespace ks

using namespace ks;

struct KsTerms {
  KsTermsDesc host;
  DevTerms* dev;
};

extern "C" int ks_terms_create(const KsTermsDesc* d, KsTerms** out) {
  if (!d || !out) return fail(KS_EINVAL, "ks_terms_create: null argument");
  if (d->obs_dim < 0 || d->obs_dim > KS_MAX_OBS) return fail(KS_ELIMIT, "ks_terms_create: obs_dim %d > %d", d->obs_dim, KS_MAX_OBS);
  if (d->n_terms < 0 || d->n_terms > KS_MAX_TERMS) return fail(KS_ELIMIT, "ks_terms_create: %d terminations > %d", d->n_terms, KS_MAX_TERMS);
  if (d->nq < 0 || d->nq > KS_MAX_QPOS || d->nv < 0 || d->nu < 0 || d->nb < 1) return fail(KS_EINVAL, "ks_terms_create: bad sizes");
  const int src_dim[KS_SRC_COUNT] = {d->nq, d->nv, d->nv, d->nu, d->action_dim > 0 ? d->action_dim : d->nu, d->command_dim, 1, d->nb * 3, d->nb * 4, d->nb * 6, 0, d->ns, d->nb * 10, d->nb * 6};
  if (d->ns < 0 || d->carry_dim < 0) return fail(KS_EINVAL, "ks_terms_create: negative sphere count or carry size");
  if (d->reset_pitch_roll < 0 || d->reset_pitch_roll > 2) return fail(KS_EINVAL, "ks_terms_create: reset_pitch_roll must be 0, 1 or 2");
  if ((d->reset_pitch_roll || d->random_heading) && d->nq < 7) return fail(KS_EINVAL, "ks_terms_create: an orientation reset needs a floating base");
  if (d->reset_hfield && (d->nq < 3 || !(d->hfield_bound[0] > 0.f) || !(d->hfield_bound[1] > 0.f)))
    return fail(KS_EINVAL, "ks_terms_create: the height-field reset needs a floating base and positive half extents");
  for (int k = 0; k < d->obs_dim; ++k) {
    const KsObsElem& el = d->obs[k];
    if (el.src < 0 || el.src >= KS_SRC_COUNT) return fail(KS_EINVAL, "ks_terms_create: obs %d: bad source %d", k, el.src);
    if (el.kind < KS_OBS_COPY || el.kind > KS_OBS_SITE_MAGNETOMETER) return fail(KS_EINVAL, "ks_terms_create: obs %d: bad kind", k);
    if (el.kind == KS_OBS_CONTACT_ANY) {
      // a 31-bit mask in an int field, walked with a shift per sphere: more spheres than that cannot be expressed
      if (d->ns > 31) return fail(KS_ELIMIT, "ks_terms_create: obs %d: a contact list covers at most 31 spheres, the model has %d", k, d->ns);
      if (d->ns < 1 || el.index <= 0 || (el.index >> d->ns) != 0) return fail(KS_EINVAL, "ks_terms_create: obs %d: sphere mask 0x%x outside the model's %d spheres", k, el.index, d->ns);
      continue;
    }
    if (el.kind == KS_OBS_SITE_ROT6D) {
      if (el.comp < 0 || el.comp > 5 || el.index < 0 || el.index >= d->nb) return fail(KS_EINVAL, "ks_terms_create: obs %d: bad site orientation entry (component %d, body %d)", k, el.comp, el.index);
      if (!(el.e0 * el.e0 + el.e1 * el.e1 + el.e2 * el.e2 + el.e3 * el.e3 > 0.f)) return fail(KS_EINVAL, "ks_terms_create: obs %d: the site orientation is not a quaternion", k);
      continue;
    }
    if (el.kind == KS_OBS_SITE_POS || el.kind == KS_OBS_SITE_QUAT || el.kind == KS_OBS_SITE_MAGNETOMETER) {
      if (el.comp < 0 || el.comp > (el.kind == KS_OBS_SITE_QUAT ? 3 : 2) || el.index < 0 || el.index >= d->nb) return fail(KS_EINVAL, "ks_terms_create: obs %d: bad site frame sensor (component %d, body %d)", k, el.comp, el.index);
      if (!(el.e0 * el.e0 + el.e1 * el.e1 + el.e2 * el.e2 + el.e3 * el.e3 > 0.f)) return fail(KS_EINVAL, "ks_terms_create: obs %d: the site orientation is not a quaternion", k);
      continue;
    }
    if (el.kind == KS_OBS_SITE_GYRO || el.kind == KS_OBS_SITE_ACCEL) {
      if (el.comp < 0 || el.comp > 2 || el.index < 0 || el.index >= d->nb) return fail(KS_EINVAL, "ks_terms_create: obs %d: bad site sensor (component %d, body %d)", k, el.comp, el.index);
      if (!(el.e0 * el.e0 + el.e1 * el.e1 + el.e2 * el.e2 + el.e3 * el.e3 > 0.f)) return fail(KS_EINVAL, "ks_terms_create: obs %d: the site orientation is not a quaternion", k);
      if (el.kind == KS_OBS_SITE_ACCEL && d->nv < 6) return fail(KS_EINVAL, "ks_terms_create: obs %d: an accelerometer needs a floating base", k);
      continue;
    }
    if (el.kind == KS_OBS_DELAYED) {
      if (el.comp < 1 || el.stride < 1 || el.carry < 0 || el.carry + (el.comp - 1) * el.stride >= d->carry_dim)
        return fail(KS_EINVAL, "ks_terms_create: obs %d: delay buffer outside the carry row", k);
      if (el.src == KS_SRC_CONST) return fail(KS_EINVAL, "ks_terms_create: obs %d: a delayed constant", k);
      if (el.src == KS_SRC_QPOS && (el.index < 7 || el.index - 7 >= d->nu)) return fail(KS_EINVAL, "ks_terms_create: obs %d: delayed joint position index %d out of range", k, el.index);
    }
    if (el.kind == KS_OBS_GRAVITY_EMA) {
      if (el.comp < 0 || el.comp > 2 || d->nq < 7 || el.src != KS_SRC_CONST) return fail(KS_EINVAL, "ks_terms_create: obs %d: bad gravity reading", k);
      if (el.carry < 0 || el.carry + 7 > d->carry_dim) return fail(KS_EINVAL, "ks_terms_create: obs %d: carry outside the carry row", k);
      if (!(el.q0 >= 0.f && el.q0 < 1.f && el.q1 >= 0.f && el.q1 < 1.f && el.q2 >= 0.f)) return fail(KS_EINVAL, "ks_terms_create: obs %d: lag outside [0, 1) or negative bias", k);
    }
    const int span = el.kind == KS_OBS_ROT_INV ? 3 : 1;
    if (el.src != KS_SRC_CONST && (el.index < 0 || el.index + span > src_dim[el.src]))
      return fail(KS_EINVAL, "ks_terms_create: obs %d reads [%d,%d) of a source with %d columns", k, el.index, el.index + span, src_dim[el.src]);
    if (el.kind == KS_OBS_JOINT_POS && (el.src != KS_SRC_QPOS || el.index < 7 || el.index - 7 >= d->nu))
      return fail(KS_EINVAL, "ks_terms_create: obs %d: joint position index %d out of range", k, el.index);
    if (el.kind == KS_OBS_ROT_INV && (el.comp < 0 || el.comp > 2 || d->nq < 7))
      return fail(KS_EINVAL, "ks_terms_create: obs %d: bad rotation component", k);
  }
  for (int k = 0; k < d->obs_dim; ++k) {
    const KsObsElem& el = d->obs[k];
    if (el.n_noise < 0 || el.n_noise > KS_MAX_NOISE_CHAIN) return fail(KS_ELIMIT, "ks_terms_create: obs %d: %d noise stages (0..%d)", k, el.n_noise, KS_MAX_NOISE_CHAIN);
    for (int j = 0; j < el.n_noise; ++j)
      if (el.noise[j].kind <= KS_NOISE_NONE || el.noise[j].kind > KS_NOISE_MUL_UNIFORM_GAUSSIAN) return fail(KS_EINVAL, "ks_terms_create: obs %d: bad noise kind", k);
    if (el.bias.kind < KS_NOISE_NONE || el.bias.kind > KS_NOISE_MUL_UNIFORM_GAUSSIAN) return fail(KS_EINVAL, "ks_terms_create: obs %d: bad bias kind", k);
  }
  for (int j = 0; j < d->n_terms; ++j) {
    const KsTermDesc& t = d->terms[j];
    if (t.kind < KS_TERM_MIN_HEIGHT || t.kind > KS_TERM_ILLEGAL_CONTACT) return fail(KS_EINVAL, "ks_terms_create: termination %d: bad kind", j);
    if (t.kind == KS_TERM_ILLEGAL_CONTACT && (d->ns < 1 || d->ns > 24 || t.p1 < 0.f || t.p1 >= (float)(1u << d->ns)))
      return fail(KS_EINVAL, "ks_terms_create: termination %d: sphere mask outside the model's %d spheres", j, d->ns);
    if (t.value != 1 && t.value != -1) return fail(KS_EINVAL, "ks_terms_create: termination %d must report +1 or -1", j);
    if ((t.kind == KS_TERM_NOT_UPRIGHT) && d->nq < 7) return fail(KS_EINVAL, "ks_terms_create: termination %d needs a free root", j);
    if (d->nq < 3 || d->nv < 3) return fail(KS_EINVAL, "ks_terms_create: terminations need a floating base");
  }
  KsTerms* t = new KsTerms();
  t->host = *d;
  if (hipMalloc((void**)&t->dev, sizeof(DevTerms)) != hipSuccess) { delete t; return fail(KS_ELAUNCH, "ks_terms_create: hipMalloc failed"); }
  if (hipMemcpy(t->dev, d, sizeof(KsTermsDesc), hipMemcpyHostToDevice) != hipSuccess) {
    (void)hipFree(t->dev); delete t; return fail(KS_ELAUNCH, "ks_terms_create: upload failed");
  }
  *out = t;
  return KS_OK;
}

extern "C" int ks_terms_destroy(KsTerms* t) {
  if (!t) return KS_OK;
  (void)hipFree(t->dev);
  delete t;
  return KS_OK;
}

// Checks a ks_observe call on the host and fills the kernel arguments; `empty` when there is nothing to launch.
static int fill_observe(const KsTerms* t, const KsObserveIO* io, ObserveArgs& a, bool& empty) {
  empty = false;
  if (!t || !io) return fail(KS_EINVAL, "ks_observe: null argument");
  const KsTermsDesc& d = t->host;
  if (io->N < 0) return fail(KS_EINVAL, "ks_observe: negative env count");
  if (io->N == 0 || d.obs_dim == 0) { empty = true; return KS_OK; }
  const int src_dim[KS_SRC_COUNT] = {d.nq, d.nv, d.nv, d.nu, d.action_dim > 0 ? d.action_dim : d.nu, d.command_dim, 1, d.nb * 3, d.nb * 4, d.nb * 6, 0, d.ns, d.nb * 10, d.nb * 6};
  if (d.carry_dim > 0 && !io->carry) return fail(KS_EINVAL, "ks_observe: the stateful observations need a carry buffer");
  std::memset(&a, 0, sizeof(a));
  bool needs_quat = false, needs_noise = false;
  for (int k = 0; k < d.obs_dim; ++k) {
    const KsObsElem& el = d.obs[k];
    const bool frame_kind = el.kind == KS_OBS_SITE_POS || el.kind == KS_OBS_SITE_QUAT || el.kind == KS_OBS_SITE_MAGNETOMETER;
    const bool site_kind = el.kind == KS_OBS_SITE_GYRO || el.kind == KS_OBS_SITE_ACCEL || el.kind == KS_OBS_SITE_ROT6D || frame_kind;
    if (site_kind && el.env_site && !io->site_pose) return fail(KS_EINVAL, "ks_observe: observation %d reads the per-env site pose, which is NULL", k);
    if (el.kind == KS_OBS_SITE_GYRO || el.kind == KS_OBS_SITE_ACCEL) {
      if (!io->src[KS_SRC_XQUAT] || !io->src[KS_SRC_CVEL] || (el.kind == KS_OBS_SITE_ACCEL && !io->src[KS_SRC_QACC]))
        return fail(KS_EINVAL, "ks_observe: observation %d (site sensor) needs xquat, cvel and, for an accelerometer, qacc", k);
      continue;
    }
    if (el.kind == KS_OBS_SITE_ROT6D) {
      if (!io->src[KS_SRC_XQUAT]) return fail(KS_EINVAL, "ks_observe: observation %d (site orientation) needs xquat", k);
      continue;
    }
    if (frame_kind) {
      if (!io->src[KS_SRC_XQUAT] || (el.kind == KS_OBS_SITE_POS && !io->src[KS_SRC_XPOS]))
        return fail(KS_EINVAL, "ks_observe: observation %d (site frame sensor) needs xquat and, for a position, xpos", k);
      continue;
    }
    if (el.kind == KS_OBS_CONTACT_ANY) {
      if (!io->src[KS_SRC_CONTACT_DIST]) return fail(KS_EINVAL, "ks_observe: observation %d reads contact_dist, which is NULL", k);
      continue;
    }
    if (el.src != KS_SRC_CONST && !io->src[el.src]) return fail(KS_EINVAL, "ks_observe: observation %d reads source %d, which is NULL", k, el.src);
    needs_quat |= el.kind == KS_OBS_ROT_INV || el.kind == KS_OBS_GRAVITY_EMA;
  }
  bool needs_bias = false;
  for (int k = 0; k < d.obs_dim; ++k) {
    const KsObsElem& el = d.obs[k];
    needs_noise |= el.n_noise > 0;
    needs_bias |= el.bias.kind != KS_NOISE_NONE;
  }
  // the bias is applied when noisy_obs is written and re-drawn for the envs `fresh` marks: either use touches bias_draw
  if (needs_bias && (io->noisy_obs || io->fresh) && !io->bias_draw) return fail(KS_EINVAL, "ks_observe: observations with a bias need the bias_draw buffer");
  if (needs_quat && !io->src[KS_SRC_QPOS]) return fail(KS_EINVAL, "ks_observe: qpos is required for body-frame observations");
  if ((io->noise_normal == nullptr) != (io->noise_uniform == nullptr)) return fail(KS_EINVAL, "ks_observe: pass both explicit noise buffers or neither");
  (void)needs_noise;
  a.t = t->dev; a.N = io->N; a.level = io->level;
  for (int s = 0; s < KS_SRC_COUNT; ++s) { a.src[s] = io->src[s]; a.src_dim[s] = src_dim[s]; }
  a.zero_offset = io->zero_offset; a.bias_draw = needs_bias ? io->bias_draw : nullptr; a.bias_redraw = io->bias_redraw; a.noise_normal = io->noise_normal; a.noise_uniform = io->noise_uniform;
  a.rng = io->rng; a.obs = io->obs; a.noisy = io->noisy_obs; a.obs_dim = d.obs_dim; a.nq = d.nq; a.nu = d.nu;
  a.carry = io->carry; a.fresh = io->fresh; a.carry_uniform = io->carry_uniform; a.carry_dim = d.carry_dim;
  a.site_pose = io->site_pose;
  return KS_OK;
}

extern "C" int ks_observe(const KsTerms* t, ks_stream_t stream, const KsObserveIO* io) {
  ObserveArgs a;
  bool empty;
  const int rc = fill_observe(t, io, a, empty);
  if (rc != KS_OK || empty) return rc;
  const int64_t n = a.N * a.obs_dim;
  const int64_t grid = (n + 255) / 256;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_observe: too many elements");
  hipLaunchKernelGGL(observe_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, a);
  return check_launch("ks_observe");
}


static int fill_terminate(const KsTerms* t, const KsTerminateIO* io, TerminateArgs& a, bool& empty) {
  empty = false;
  if (!t || !io) return fail(KS_EINVAL, "ks_terminate_reset: null argument");
  const KsTermsDesc& d = t->host;
  if (io->N < 0) return fail(KS_EINVAL, "ks_terminate_reset: negative env count");
  if (io->N == 0) { empty = true; return KS_OK; }
  if (!io->qpos || !io->qvel) return fail(KS_EINVAL, "ks_terminate_reset: qpos and qvel are required");
  std::memset(&a, 0, sizeof(a));
  a.t = t->dev; a.N = io->N; a.level = io->level;
  a.qpos = io->qpos; a.qvel = io->qvel; a.warm = io->qacc_warmstart; a.time = io->time; a.last_ctrl = io->last_ctrl;
  a.components = io->components; a.done = io->done; a.success = io->success;
  a.traj_qpos = io->traj_qpos; a.traj_qvel = io->traj_qvel; a.traj_time = io->traj_time;
  a.reset_mask = io->reset_mask; a.episode_length = io->episode_length; a.reset_uniform = io->reset_uniform;
  a.rng = io->rng; a.apply_reset = io->apply_reset; a.nq = d.nq; a.nv = d.nv; a.nu = d.nu; a.n_terms = d.n_terms;
  a.random_heading = d.random_heading; a.nonfinite_terminates = d.nonfinite_terminates;
  if (io->n_events < 0 || io->n_events > KS_MAX_EVENTS) return fail(KS_ELIMIT, "ks_terminate_reset: %d events (0..%d)", io->n_events, KS_MAX_EVENTS);
  if (io->n_events > 0 && !io->event_state) return fail(KS_EINVAL, "ks_terminate_reset: events need event_state");
  a.contact_dist = io->contact_dist; a.ns = d.ns; a.na = d.action_dim > 0 ? d.action_dim : d.nu;
  for (int j = 0; j < d.n_terms; ++j)
    if (d.terms[j].kind == KS_TERM_ILLEGAL_CONTACT && !io->contact_dist) return fail(KS_EINVAL, "ks_terminate_reset: termination %d reads contact_dist", j);
  a.n_events = io->n_events; a.event_state = io->event_state; a.event_reset_uniform = io->event_reset_uniform; a.event_force = io->event_force;
  for (int k = 0; k < io->n_events; ++k) { a.event_interval[k][0] = io->event_interval[k][0]; a.event_interval[k][1] = io->event_interval[k][1]; }
  a.action_latency = io->action_latency; a.zero_offset = io->zero_offset; a.act_action_bias = io->act_action_bias;
  a.act_torque_bias = io->act_torque_bias; a.act_kp_scale = io->act_kp_scale; a.act_kd_scale = io->act_kd_scale;
  a.act_torque_limit_scale = io->act_torque_limit_scale;
  a.latency_lo = io->latency_lo; a.latency_hi = io->latency_hi;
  a.zero_offset_rv = io->zero_offset_rv; a.action_bias_rv = io->action_bias_rv; a.torque_bias_rv = io->torque_bias_rv;
  a.kp_scale_rv = io->kp_scale_rv; a.kd_scale_rv = io->kd_scale_rv; a.torque_limit_scale_rv = io->torque_limit_scale_rv;
  a.episode_uniform = io->episode_uniform; a.episode_normal = io->episode_normal;
  a.reset_pitch_roll_uniform = io->reset_pitch_roll_uniform; a.reset_frame = io->reset_frame;
  bool from_motion = false;
  for (int i = 0; i < d.nq; ++i) from_motion |= d.reset_from_motion[i] != 0;
  if (from_motion && io->apply_reset) {
    if (!io->reset_motion_qpos || io->reset_motion_frames < 1)
      return fail(KS_EINVAL, "ks_terminate_reset: the reset table starts from a reference motion: reset_motion_qpos and its frame count are required");
    a.reset_motion_qpos = io->reset_motion_qpos; a.reset_motion_frames = io->reset_motion_frames; a.reset_motion_dt = io->reset_motion_dt;
  }
  if (d.reset_hfield && io->apply_reset) {
    if (!io->reset_hfield || io->hfield_nx < 1 || io->hfield_ny < 1)
      return fail(KS_EINVAL, "ks_terminate_reset: the reset table reads a height field: reset_hfield and its shape are required");
    a.reset_hfield = io->reset_hfield; a.hfield_nx = io->hfield_nx; a.hfield_ny = io->hfield_ny;
  }
  a.redraw = (a.action_latency || a.zero_offset || a.act_action_bias || a.act_torque_bias || a.act_kp_scale || a.act_kd_scale ||
              a.act_torque_limit_scale) ? 1 : 0;
  if (a.action_latency && !(io->latency_lo >= 0.f && io->latency_hi >= io->latency_lo))
    return fail(KS_EINVAL, "ks_terminate_reset: latency range must satisfy 0 <= lo <= hi");
  return KS_OK;
}

extern "C" int ks_terminate_reset(const KsTerms* t, ks_stream_t stream, const KsTerminateIO* io) {
  TerminateArgs a;
  bool empty;
  const int rc = fill_terminate(t, io, a, empty);
  if (rc != KS_OK || empty) return rc;
  const int64_t grid = (a.N + kTermEnvs - 1) / kTermEnvs;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_terminate_reset: too many envs");
  hipLaunchKernelGGL(terminate_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, a);
  return check_launch("ks_terminate_reset");
}

extern "C" int ks_terminate_reset_observe(const KsTerms* t, ks_stream_t stream, const KsTerminateIO* tio, const KsObserveIO* oio) {
  TerminateArgs a;
  ObserveArgs o;
  bool empty_t, empty_o;
  int rc = fill_terminate(t, tio, a, empty_t);
  if (rc != KS_OK) return rc;
  rc = fill_observe(t, oio, o, empty_o);
  if (rc != KS_OK) return rc;
  if (tio->N != oio->N) return fail(KS_EINVAL, "ks_terminate_reset_observe: the two halves disagree about the env count (%lld, %lld)", (long long)tio->N, (long long)oio->N);
  if (empty_t) return KS_OK;
  // the observation half takes the episode starts from the mask the termination half writes in the same launch
  if (oio->fresh && oio->fresh != tio->reset_mask) return fail(KS_EINVAL, "ks_terminate_reset_observe: the observation's fresh flags must be the reset mask of this call");
  if (empty_o) { o.obs_dim = 0; }
  const int64_t grid = (a.N + kTermObsEnvs - 1) / kTermObsEnvs;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_terminate_reset_observe: too many envs");
  hipLaunchKernelGGL(terminate_observe_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, a, o);
  return check_launch("ks_terminate_reset_observe");
}


extern "C" int ks_sample_action(ks_stream_t stream, int64_t N, int32_t nu, const float* mean, const float* log_std,
                                const float* noise_normal, KsRng rng, float clip_max, float* action) {
  if (N < 0 || nu < 0) return fail(KS_EINVAL, "ks_sample_action: negative size");
  if (N == 0 || nu == 0) return KS_OK;
  if (!mean || !action) return fail(KS_EINVAL, "ks_sample_action: null pointer");
  const int64_t n = N * nu, grid = (n + 255) / 256;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_sample_action: too many elements");
  hipLaunchKernelGGL(sample_action_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, n, (int)nu, mean,
                     log_std, noise_normal, rng, clip_max, action);
  return check_launch("ks_sample_action");
}

extern "C" int ks_sample_action_head(ks_stream_t stream, int64_t N, int32_t nu, const float* raw, const KsGaussianHead* head,
                                     const float* noise_normal, KsRng rng, float clip_max, float* action, float* mean_out,
                                     float* std_out, float* log_prob_out) {
  if (N < 0 || nu < 1) return fail(KS_EINVAL, "ks_sample_action_head: bad sizes");
  if (N == 0) return KS_OK;
  if (!raw || !head || !action) return fail(KS_EINVAL, "ks_sample_action_head: raw, head and action are required");
  if (!(head->max_std > 0.f) || head->min_std < 0.f || !(head->var_scale > 0.f)) return fail(KS_EINVAL, "ks_sample_action_head: standard deviation limits must be positive");
  if (!(clip_max > 0.f)) return fail(KS_EINVAL, "ks_sample_action_head: clip_max must be positive");
  const int64_t n = N * nu, grid = (n + 255) / 256;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_sample_action_head: too many elements");
  hipLaunchKernelGGL(sample_action_head_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, n, (int)nu, raw, *head,
                     noise_normal, rng, clip_max, action, mean_out, std_out, log_prob_out);
  return check_launch("ks_sample_action_head");
}

extern "C" int ks_action_filter(ks_stream_t stream, int64_t N, int32_t nu, int32_t kind, float ctrl_dt, float p0, const float* lo,
                                const float* hi, const float* x, float* state, const uint8_t* fresh, const float* init, float* y) {
  using namespace ks;
  if (N < 0 || nu < 1) return fail(KS_EINVAL, "ks_action_filter: bad sizes");
  if (kind < KS_FILTER_LOWPASS || kind > KS_FILTER_TANH_POSITIONS) return fail(KS_EINVAL, "ks_action_filter: unknown kind %d", kind);
  if (N == 0) return KS_OK;
  if (!x || !y) return fail(KS_EINVAL, "ks_action_filter: null pointer");
  const bool ranged = kind == KS_FILTER_CLIP_POSITIONS || kind == KS_FILTER_TANH_POSITIONS;
  if (ranged && (!lo || !hi)) return fail(KS_EINVAL, "ks_action_filter: the range kinds need lo and hi");
  if (!ranged && !state) return fail(KS_EINVAL, "ks_action_filter: the stateful kinds need their state");
  if (!ranged && !(ctrl_dt > 0.f)) return fail(KS_EINVAL, "ks_action_filter: ctrl_dt must be positive");
  if ((kind == KS_FILTER_LOWPASS || kind == KS_FILTER_CLIP_ACCELERATION || kind == KS_FILTER_INTEGRATE_ACCELERATION) && !(p0 > 0.f))
    return fail(KS_EINVAL, "ks_action_filter: the cutoff frequency / acceleration / velocity bound must be positive");
  const int64_t n = N * nu, grid = (n + 255) / 256;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_action_filter: too many elements");
  hipLaunchKernelGGL(action_filter_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, n, (int)nu, (int)kind, ctrl_dt, p0, lo,
                     hi, x, state, fresh, init, y);
  return check_launch("ks_action_filter");
}

extern "C" int ks_sample_action_mixture(ks_stream_t stream, int64_t N, int32_t nu, const float* raw, const KsMixtureHead* head,
                                        const float* uniform, const float* noise_normal, KsRng rng, float clip_max,
                                        float* action, float* log_prob_out, int32_t* component_out) {
  using namespace ks;
  if (N < 0 || nu < 1) return fail(KS_EINVAL, "ks_sample_action_mixture: bad sizes");
  if (N == 0) return KS_OK;
  if (!raw || !head || !action) return fail(KS_EINVAL, "ks_sample_action_mixture: null pointer");
  if (head->num_mixtures < 1 || head->num_mixtures > KS_MAX_MIXTURES)
    return fail(KS_ELIMIT, "ks_sample_action_mixture: %d components, 1..%d are built", head->num_mixtures, KS_MAX_MIXTURES);
  if (!(head->max_std > 0.f) || head->min_std < 0.f || !(head->var_scale > 0.f))
    return fail(KS_EINVAL, "ks_sample_action_mixture: bad deviation bounds");
  if ((head->clip_lo == nullptr) != (head->clip_hi == nullptr)) return fail(KS_EINVAL, "ks_sample_action_mixture: clip_lo and clip_hi come together");
  if (!(clip_max > 0.f)) return fail(KS_EINVAL, "ks_sample_action_mixture: clip_max must be positive");
  const int64_t n = N * nu, grid = (n + 255) / 256;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_sample_action_mixture: too many elements");
  hipLaunchKernelGGL(sample_action_mixture_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, n, (int)nu, raw, *head,
                     uniform, noise_normal, rng, clip_max, action, log_prob_out, component_out, (const float*)nullptr);
  return check_launch("ks_sample_action_mixture");
}

extern "C" int ks_mixture_head_log_prob(ks_stream_t stream, int64_t M, int32_t nu, const KsMixtureHead* head, const float* raw,
                                        const float* action, float* log_prob) {
  using namespace ks;
  if (M < 0 || nu < 1) return fail(KS_EINVAL, "ks_mixture_head_log_prob: bad sizes");
  if (M == 0) return KS_OK;
  if (!raw || !head || !action || !log_prob) return fail(KS_EINVAL, "ks_mixture_head_log_prob: null pointer");
  if (head->num_mixtures < 1 || head->num_mixtures > KS_MAX_MIXTURES)
    return fail(KS_ELIMIT, "ks_mixture_head_log_prob: %d components, 1..%d are built", head->num_mixtures, KS_MAX_MIXTURES);
  if (!(head->max_std > 0.f) || head->min_std < 0.f || !(head->var_scale > 0.f)) return fail(KS_EINVAL, "ks_mixture_head_log_prob: bad deviation bounds");
  if ((head->clip_lo == nullptr) != (head->clip_hi == nullptr)) return fail(KS_EINVAL, "ks_mixture_head_log_prob: clip_lo and clip_hi come together");
  const int64_t n = M * nu, grid = (n + 255) / 256;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_mixture_head_log_prob: too many elements");
  KsMixtureHead hd = *head;
  hd.deterministic = 1;  // no draws: only the density of the given action is wanted
  KsRng none = {0, 0, nullptr};
  hipLaunchKernelGGL(sample_action_mixture_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, n, (int)nu, raw, hd,
                     (const float*)nullptr, (const float*)nullptr, none, 1.f, (float*)nullptr, log_prob, (int*)nullptr, action);
  return check_launch("ks_mixture_head_log_prob");
}

extern "C" int ks_rewards(ks_stream_t stream, const KsRewardIO* io) {
  if (!io) return fail(KS_EINVAL, "ks_rewards: null argument");
  if (io->T < 0 || io->N < 0) return fail(KS_EINVAL, "ks_rewards: negative size");
  if (io->n_rewards < 0 || io->n_rewards > KS_MAX_REWARD_TERMS) return fail(KS_ELIMIT, "ks_rewards: more than %d terms", KS_MAX_REWARD_TERMS);
  if (io->T == 0 || io->N == 0) return KS_OK;
  if (!io->done) return fail(KS_EINVAL, "ks_rewards: done is required");
  for (int j = 0; j < io->n_rewards; ++j) {
    const int k = io->rewards[j].kind;
    if (k < KS_REW_STAY_ALIVE || k > KS_REW_JOINT_VELOCITY_CMD) return fail(KS_EINVAL, "ks_rewards: term %d: bad kind", j);
    const KsRewardDesc& rd = io->rewards[j];
    if (k == KS_REW_LINVEL_CMD || k == KS_REW_ANGVEL_CMD) {
      const int span = k == KS_REW_LINVEL_CMD ? 4 : 1;
      if (!io->command || rd.index < 0 || rd.index + span > io->command_dim) return fail(KS_EINVAL, "ks_rewards: term %d reads command[%d..%d) of %d entries", j, rd.index, rd.index + span, io->command_dim);
      if (rd.norm < 0 || rd.norm >= (k == KS_REW_LINVEL_CMD ? 4 : 2) || !(rd.p0 > 0.f)) return fail(KS_EINVAL, "ks_rewards: term %d: bad component or length scale", j);
    }
    if (k == KS_REW_OFF_AXIS && (rd.norm < 0 || rd.norm > 2 || !(rd.p0 > 0.f))) return fail(KS_EINVAL, "ks_rewards: term %d: bad component or length scale", j);
    if (k == KS_REW_FORCE && (!io->obs || rd.norm < 1 || rd.index < 0 || rd.index + 3 * rd.norm > io->obs_dim || !(rd.p0 > 0.f)))
      return fail(KS_EINVAL, "ks_rewards: term %d: force block outside the observation or zero expected weight", j);
    if (k == KS_REW_STATEFUL && (!io->stateful || io->rewards[j].norm < 0)) return fail(KS_EINVAL, "ks_rewards: term %d needs the scanned values", j);
    const bool needs_q = k == KS_REW_BASE_HEIGHT || k == KS_REW_BASE_HEIGHT_RANGE || k == KS_REW_UPRIGHT_POSE || k == KS_REW_LINVEL_CMD;
    const bool needs_v = k == KS_REW_UPRIGHT_ANGVEL || k == KS_REW_UPRIGHT_LINVEL || (k >= KS_REW_LINVEL_CMD && k <= KS_REW_MOTIONLESS);
    const bool needs_a = k >= KS_REW_ACTION_VEL && k <= KS_REW_ACTION_JERK;
    if (needs_q && (!io->qpos || io->nq < 7)) return fail(KS_EINVAL, "ks_rewards: term %d needs qpos of a floating base", j);
    if (needs_v && (!io->qvel || io->nv < 6)) return fail(KS_EINVAL, "ks_rewards: term %d needs qvel of a floating base", j);
    if (needs_a && (!io->action || io->nu < 1)) return fail(KS_EINVAL, "ks_rewards: term %d needs actions", j);
    {
      const KsRewardDesc& r = io->rewards[j];
      const int nj = io->nq - 7;
      int need_params = 0;
      bool uses_params = true;
      switch (k) {
        case KS_REW_JOINT_SMOOTH:
          if (!io->qpos || nj < 1 || r.norm < 1 || r.norm > 3 || !(r.p0 > 0.f))
            return fail(KS_EINVAL, "ks_rewards: term %d: joint smoothness needs joints behind a floating base, order 1..3 and a positive scale", j);
          uses_params = false;
          break;
        case KS_REW_AVOID_LIMITS:
          if (!io->qpos || nj < 1) return fail(KS_EINVAL, "ks_rewards: term %d needs joints behind a floating base", j);
          need_params = 2 * nj;
          break;
        case KS_REW_TORQUE:
        case KS_REW_ENERGY:
          if (!io->ctrl || io->nu < 1) return fail(KS_EINVAL, "ks_rewards: term %d needs the applied torques", j);
          if (k == KS_REW_ENERGY && (!io->qvel || io->nv != io->nu + 6)) return fail(KS_EINVAL, "ks_rewards: term %d needs qvel with one entry per actuator behind a floating base", j);
          need_params = io->nu;
          break;
        case KS_REW_JOINT_DEVIATION:
          if (!io->qpos || nj < 1 || r.count < 1) return fail(KS_EINVAL, "ks_rewards: term %d needs joints behind a floating base", j);
          need_params = 3 * r.count;
          break;
        case KS_REW_FLAT_BODY:
          if (!io->xquat || io->nb < 1 || r.count < 1) return fail(KS_EINVAL, "ks_rewards: term %d needs body orientations", j);
          need_params = r.count + 3;
          break;
        case KS_REW_POSITION_TRACKING:
          if (!io->xpos || r.index2 < 0 || r.index2 >= io->nb || r.count < 0 || r.count >= io->nb)
            return fail(KS_EINVAL, "ks_rewards: term %d: body outside the trajectory's positions", j);
          if (!io->command || r.index < 0 || r.index + 3 > io->command_dim) return fail(KS_EINVAL, "ks_rewards: term %d: command block outside the command vector", j);
          if (!(r.p0 > 0.f)) return fail(KS_EINVAL, "ks_rewards: term %d: the kernel scale must be positive", j);
          uses_params = false;
          break;
        case KS_REW_NO_ROLL_ANGVEL:
          if (!io->qvel || io->nv < 6) return fail(KS_EINVAL, "ks_rewards: term %d needs qvel of a floating base", j);
          uses_params = false;
          break;
        case KS_REW_NO_ROLL_POSE:
          if (!io->qpos || io->nq < 7) return fail(KS_EINVAL, "ks_rewards: term %d needs qpos of a floating base", j);
          uses_params = false;
          break;
        case KS_REW_LINK_SMOOTH:
          if (!io->xpos || io->nb < 2 || (r.p0 != 2.f && r.p0 != 3.f)) return fail(KS_EINVAL, "ks_rewards: term %d needs body positions and order 2 or 3", j);
          uses_params = false;
          break;
        case KS_REW_FEET_SLIP:
          if (!io->obs || r.norm < 1 || r.count < 1 || r.index < 0 || r.index + r.count * r.norm > io->obs_dim || r.index2 < 0 ||
              r.index2 + 6 * r.norm > io->obs_dim)
            return fail(KS_EINVAL, "ks_rewards: term %d: contact or velocity block outside the observation", j);
          uses_params = false;
          break;
        case KS_REW_REACHABILITY:
          if (!io->qpos || !io->action || io->nu < 1 || io->nq != io->nu + 7) return fail(KS_EINVAL, "ks_rewards: term %d needs actions and qpos with one joint per action behind a floating base", j);
          need_params = io->nu;
          break;
        case KS_REW_JOINT_POSITION:
        case KS_REW_JOINT_VELOCITY_CMD:
          if (!io->qpos || !io->qvel || nj < 1 || r.count < 1) return fail(KS_EINVAL, "ks_rewards: term %d needs joints behind a floating base", j);
          if (!io->command || r.index < 0 || r.index + 2 * r.count + 3 > io->command_dim)
            return fail(KS_EINVAL, "ks_rewards: term %d: the joint-position command block (2 n + 3 numbers) lies outside the command vector", j);
          if (!(r.p0 > 0.f)) return fail(KS_EINVAL, "ks_rewards: term %d: the kernel scale must be positive", j);
          need_params = r.count;
          break;
        case KS_REW_SINUSOIDAL_GAIT:
          if (!io->obs || !io->command || r.norm < 1 || r.index < 0 || r.index + 3 * r.norm > io->obs_dim || r.index2 < 0 ||
              r.index2 + r.norm > io->command_dim || !(r.p0 != 0.f))
            return fail(KS_EINVAL, "ks_rewards: term %d: foot positions or target heights outside their vectors, or zero max height", j);
          uses_params = false;
          break;
        case KS_REW_INTERSECTION:
          if (!io->obs || r.norm < 2 || r.index < 0 || r.index + 3 * r.norm > io->obs_dim) return fail(KS_EINVAL, "ks_rewards: term %d: position block outside the observation", j);
          uses_params = false;
          break;
        default: uses_params = false; break;
      }
      if (uses_params) {
        if (io->n_params < 0 || io->n_params > KS_MAX_REWARD_PARAMS || r.param_offset < 0 || r.param_offset + need_params > io->n_params)
          return fail(KS_EINVAL, "ks_rewards: term %d: its %d constants do not fit the table of %d", j, need_params, io->n_params);
        const float* pr = io->params + r.param_offset;
        if (k == KS_REW_TORQUE || k == KS_REW_ENERGY)
          for (int u = 0; u < io->nu; ++u)
            if (!(pr[u] != 0.f)) return fail(KS_EINVAL, "ks_rewards: term %d: zero control scale for actuator %d", j, u);
        if (k == KS_REW_JOINT_DEVIATION)
          for (int c = 0; c < r.count; ++c)
            if (!(pr[3 * c] >= 0.f && pr[3 * c] < (float)nj)) return fail(KS_EINVAL, "ks_rewards: term %d: joint %d outside 0..%d", j, (int)pr[3 * c], nj - 1);
        if (k == KS_REW_JOINT_POSITION || k == KS_REW_JOINT_VELOCITY_CMD)
          for (int c = 0; c < r.count; ++c)
            if (!(pr[c] >= 0.f && pr[c] < (float)nj)) return fail(KS_EINVAL, "ks_rewards: term %d: joint %d outside 0..%d", j, (int)pr[c], nj - 1);
        if (k == KS_REW_FLAT_BODY)
          for (int c = 0; c < r.count; ++c)
            if (!(pr[c] >= 0.f && pr[c] < (float)io->nb)) return fail(KS_EINVAL, "ks_rewards: term %d: body %d outside 0..%d", j, (int)pr[c], io->nb - 1);
      }
    }
    if (k == KS_REW_AMP && !io->disc_logits) return fail(KS_EINVAL, "ks_rewards: term %d needs the discriminator logits", j);
    if (k == KS_REW_STAY_ALIVE && !(io->rewards[j].p0 != 0.f)) return fail(KS_EINVAL, "ks_rewards: term %d: zero balance", j);
  }
  const int64_t n = io->T * io->N, grid = (n + 255) / 256;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_rewards: too many elements");
  hipLaunchKernelGGL(rewards_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, *io);
  return check_launch("ks_rewards");
}

extern "C" int ks_reward_scan(ks_stream_t stream, const KsRewardScanIO* io) {
  using namespace ks;
  if (!io) return fail(KS_EINVAL, "ks_reward_scan: null argument");
  if (io->T < 0 || io->N < 0) return fail(KS_EINVAL, "ks_reward_scan: negative size");
  if (io->n_scans < 0 || io->n_scans > KS_MAX_REWARD_SCANS) return fail(KS_ELIMIT, "ks_reward_scan: more than %d scans", KS_MAX_REWARD_SCANS);
  if (io->T == 0 || io->N == 0 || io->n_scans == 0) return KS_OK;
  if (!io->done || !io->carry || !io->out) return fail(KS_EINVAL, "ks_reward_scan: done, carry and out are required");
  for (int j = 0; j < io->n_scans; ++j) {
    const KsRewardScanDesc& s = io->scans[j];
    if (s.kind == KS_SCAN_SYMMETRY || s.kind == KS_SCAN_PAIRWISE_SYMMETRY) {
      const bool pair = s.kind == KS_SCAN_PAIRWISE_SYMMETRY;
      const int n = pair ? 2 : s.n;
      if (!io->qpos || io->nq < 8) return fail(KS_EINVAL, "ks_reward_scan: scan %d reads the joints behind a floating base (qpos)", j);
      if (n < 1 || n > KS_MAX_SCAN_JOINTS) return fail(KS_ELIMIT, "ks_reward_scan: scan %d: %d joints (1..%d)", j, n, KS_MAX_SCAN_JOINTS);
      for (int k = 0; k < n; ++k)
        if (s.joints[k] < 0 || s.joints[k] + 7 >= io->nq) return fail(KS_EINVAL, "ks_reward_scan: scan %d: joint %d outside 0..%d", j, s.joints[k], io->nq - 8);
      if (s.slot < 0 || s.slot + (pair ? 2 : 1) > io->n_slots) return fail(KS_EINVAL, "ks_reward_scan: scan %d: output slot outside n_slots", j);
      if (s.carry_index < 0 || s.carry_index + n > io->carry_dim) return fail(KS_EINVAL, "ks_reward_scan: scan %d: carry outside the carry row", j);
      if (pair && (!(s.kernel_scale > 0.f) || !(s.sq_scale > 0.f) || !(s.abs_scale > 0.f))) return fail(KS_EINVAL, "ks_reward_scan: scan %d: the kernel scales must be positive", j);
      continue;
    }
    if (!io->obs || !io->qvel) return fail(KS_EINVAL, "ks_reward_scan: scan %d reads obs and qvel", j);
    if (io->nv < 6) return fail(KS_EINVAL, "ks_reward_scan: the rewards read the velocity of a floating base");
    if (s.kind != KS_SCAN_FEET_AIR_TIME && s.kind != KS_SCAN_SPARSE_TARGET_HEIGHT) return fail(KS_EINVAL, "ks_reward_scan: scan %d: bad kind", j);
    const bool feet = s.kind == KS_SCAN_FEET_AIR_TIME;
    if (s.n < 1 || s.n > KS_MAX_SCAN_BODIES || s.n_contact < 1) return fail(KS_ELIMIT, "ks_reward_scan: scan %d: %d bodies (1..%d), %d contact rows", j, s.n, KS_MAX_SCAN_BODIES, s.n_contact);
    if (s.contact_index < 0 || s.contact_index + s.n_contact * s.n > io->obs_dim) return fail(KS_EINVAL, "ks_reward_scan: scan %d: contact block outside the observation", j);
    if (!feet && (s.position_index < 0 || s.position_index + 3 * s.n > io->obs_dim)) return fail(KS_EINVAL, "ks_reward_scan: scan %d: position block outside the observation", j);
    if (s.slot < 0 || s.slot + (feet ? 3 : 1) > io->n_slots) return fail(KS_EINVAL, "ks_reward_scan: scan %d: output slot outside n_slots", j);
    if (s.carry_index < 0 || s.carry_index + (feet ? 3 : 1) * s.n > io->carry_dim) return fail(KS_EINVAL, "ks_reward_scan: scan %d: carry outside the carry row", j);
    if (feet) {
      for (int idx : {s.linvel_cmd_index, s.angvel_cmd_index})
        if (idx >= 0 && (!io->command || idx >= io->command_dim)) return fail(KS_EINVAL, "ks_reward_scan: scan %d: command index %d without such a command", j, idx);
      if (!(s.air_steps > 0.f) || !(s.gnd_steps > 0.f)) return fail(KS_EINVAL, "ks_reward_scan: scan %d: the gait needs at least one step in the air and one on the ground", j);
    }
  }
  const int64_t grid = (io->N + 255) / 256;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_reward_scan: too many envs");
  hipLaunchKernelGGL(reward_scan_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, *io);
  return check_launch("ks_reward_scan");
}

extern "C" int ks_commands(ks_stream_t stream, const KsCommandIO* io) {
  using namespace ks;
  if (!io) return fail(KS_EINVAL, "ks_commands: null argument");
  if (io->N < 0 || io->n_commands < 0 || io->n_commands > KS_MAX_COMMANDS) return fail(KS_ELIMIT, "ks_commands: %d commands (0..%d)", io->n_commands, KS_MAX_COMMANDS);
  if (io->N == 0 || io->n_commands == 0) return KS_OK;
  if (!io->command) return fail(KS_EINVAL, "ks_commands: the command buffer is required");
  for (int k = 0; k < io->n_commands; ++k) {
    const KsCommandDesc& c = io->commands[k];
    int need = c.dim;
    if (c.kind == KS_CMD_LINEAR_VELOCITY) need = 6;
    if (c.kind == KS_CMD_ANGULAR_VELOCITY) need = 2;
    if (c.kind == KS_CMD_START_POSITION) need = 3;
    if (c.kind == KS_CMD_START_QUATERNION) need = 4;
    if (c.kind == KS_CMD_BASE_HEIGHT) need = 1;
    if (c.kind == KS_CMD_SINUSOIDAL_GAIT) {
      if (c.dim < 3 || c.dim > 2 + KS_MAX_VECTOR_COMMAND) return fail(KS_ELIMIT, "ks_commands: command %d: 1..%d feet", k, KS_MAX_VECTOR_COMMAND);
      if (!(c.lo[0] > 0.f) || !(c.lo[3] < 1.f) || !io->qvel || io->nv < 2) return fail(KS_EINVAL, "ks_commands: command %d: gait period, stance ratio or the base velocity missing", k);
    }
    if (c.kind == KS_CMD_CARTESIAN_COORDINATE) need = 7;
    if (c.kind == KS_CMD_JOINT_POSITION) {
      const int n = (c.dim - 3) / 2;
      if (c.dim < 5 || c.dim != 2 * n + 3 || n > KS_MAX_VECTOR_COMMAND) return fail(KS_ELIMIT, "ks_commands: command %d: a joint position command holds 2 n + 3 values, 1 <= n <= %d", k, KS_MAX_VECTOR_COMMAND);
      if (!io->qpos || !(c.ctrl_dt > 0.f) || !(c.min_time > 0.f) || !(c.max_time >= c.min_time)) return fail(KS_EINVAL, "ks_commands: command %d: joint positions, ctrl_dt or the time range missing", k);
      for (int j = 0; j < n; ++j)
        if (c.joints[j] < 0 || 7 + c.joints[j] >= io->nq) return fail(KS_EINVAL, "ks_commands: command %d: joint %d outside qpos[7:%d]", k, c.joints[j], io->nq);
    }
    if (c.kind < KS_CMD_CONST || c.kind > KS_CMD_CARTESIAN_COORDINATE) return fail(KS_EINVAL, "ks_commands: command %d: bad kind", k);
    if ((c.kind == KS_CMD_START_POSITION || c.kind == KS_CMD_START_QUATERNION) && (!io->qpos || io->nq < 7))
      return fail(KS_EINVAL, "ks_commands: command %d reads the pose of a floating base", k);
    if ((c.kind == KS_CMD_FLOAT_VECTOR || c.kind == KS_CMD_INT_VECTOR) && c.dim > KS_MAX_VECTOR_COMMAND) return fail(KS_ELIMIT, "ks_commands: command %d: %d scalars (at most %d)", k, c.dim, KS_MAX_VECTOR_COMMAND);
    if (c.dim != need || c.dim < 1 || c.index < 0 || c.index + c.dim > io->command_dim) return fail(KS_EINVAL, "ks_commands: command %d: [%d,%d) outside the %d-wide command vector or of the wrong length", k, c.index, c.index + c.dim, io->command_dim);
    if ((c.kind == KS_CMD_LINEAR_VELOCITY || c.kind == KS_CMD_ANGULAR_VELOCITY) && (!io->qpos || !io->qvel || io->nq < 7 || io->nv < 6))
      return fail(KS_EINVAL, "ks_commands: velocity commands read the state of a floating base");
  }
  const int64_t n = io->N * io->n_commands, grid = (n + 255) / 256;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_commands: too many elements");
  hipLaunchKernelGGL(command_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, *io);
  return check_launch("ks_commands");
}
