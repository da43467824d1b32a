// Fused control-step kernel: S physics substeps of one env per wavefront, state resident in LDS.
//
// One 64-lane wavefront owns one env.  Lanes map to bodies, dofs, constraint rows or matrix
// entries depending on the phase; all cross-lane traffic goes through LDS or DPP reductions and
// every branch on solver progress (Newton iterations, line-search refinements, contact count) is
// wave-uniform, so a converged env stops iterating.  Phases of one substep:
//   kinematics (per-body chain walk) -> centre of mass -> com-based inertias and motion axes ->
//   composite inertias -> dense mass matrix -> body velocities + RNE bias -> smooth forces ->
//   sphere/plane contacts and pyramidal constraint rows -> Cholesky of M -> Newton solver with
//   exact line search -> semi-implicit Euler.
// The arithmetic follows the MuJoCo model that ksim/engine.py:257 invokes through mjx.step.
#include "ks_common.h"
#include "ks_model.h"
#include "ks_step_args.h"

#include <cstring>

namespace ks {

#define KS_SYNC() __syncthreads()

struct Lds {
  float *qpos, *qvel, *warm, *tau, *sc, *bmass;
  float *xpos, *xquat, *xmat, *xipos, *ximat, *xanchor, *xaxis;
  float *cinert, *crb, *cdof, *cvel, *cfrc, *fsub, *buf;
  float *M, *H, *J;
  float *vbuf, *fbuf, *wbuf, *qfs, *qacc;
  float *con_off, *con_D, *con_kip;
  int* con_body;
};

__host__ __device__ inline int lds_floats(int nb, int nq, int nv, int nu, int ns) {
  const int nvs = nv | 1;
  int n = 0;
  n += nq + nv + nv + nu + 2 * nq + nb;                   // qpos qvel warm tau sc bmass
  n += nb * (3 + 4 + 9 + 3 + 9 + 3 + 3);                  // xpos xquat xmat xipos ximat xanchor xaxis
  n += nb * 10 * 2 + nv * 6 + nb * 6 * 3 + nv * 6;        // cinert crb cdof cvel cfrc fsub buf
  n += nv * nvs * 2 + 4 * ns * nvs;                       // M H J
  n += nv + 4 * ns + 4 * ns + nv + nv;                    // vbuf fbuf wbuf qfs qacc
  n += ns * 3 + ns + ns + ns;                             // con_off con_D con_kip con_body
  return n + 8;
}

__device__ inline Lds carve(float* p, const DevModel& m) {
  const int nb = m.nb, nq = m.nq, nv = m.nv, nu = m.nu, ns = m.ns, nvs = m.nvs;
  Lds l;
  auto take = [&](int n) {
    float* r = p;
    p += n;
    return r;
  };
  l.qpos = take(nq); l.qvel = take(nv); l.warm = take(nv); l.tau = take(nu); l.sc = take(2 * nq); l.bmass = take(nb);
  l.xpos = take(nb * 3); l.xquat = take(nb * 4); l.xmat = take(nb * 9); l.xipos = take(nb * 3);
  l.ximat = take(nb * 9); l.xanchor = take(nb * 3); l.xaxis = take(nb * 3);
  l.cinert = take(nb * 10); l.crb = take(nb * 10); l.cdof = take(nv * 6); l.cvel = take(nb * 6);
  l.cfrc = take(nb * 6); l.fsub = take(nb * 6); l.buf = take(nv * 6);
  l.M = take(nv * nvs); l.H = take(nv * nvs); l.J = take(4 * ns * nvs);
  l.vbuf = take(nv); l.fbuf = take(4 * ns); l.wbuf = take(4 * ns); l.qfs = take(nv); l.qacc = take(nv);
  l.con_off = take(ns * 3); l.con_D = take(ns); l.con_kip = take(ns);
  l.con_body = reinterpret_cast<int*>(take(ns));
  return l;
}

// ------------------------------------------------------------------------------------------- position stage
__device__ inline void kinematics(const DevModel& m, const Lds& l, int lane) {
  // half-angle sines/cosines of every hinge coordinate
  for (int i = lane; i < m.nq; i += 64) {
    const float h = 0.5f * (l.qpos[i] - m.qpos0[i]);
    l.sc[2 * i] = sinf(h);
    l.sc[2 * i + 1] = cosf(h);
  }
  KS_SYNC();
  if (lane == 0) {
    for (int k = 0; k < 3; ++k) { l.xpos[k] = 0.f; l.xipos[k] = 0.f; l.xanchor[k] = 0.f; l.xaxis[k] = 0.f; }
    l.xquat[0] = 1.f; l.xquat[1] = l.xquat[2] = l.xquat[3] = 0.f;
    for (int k = 0; k < 9; ++k) { l.xmat[k] = (k % 4 == 0) ? 1.f : 0.f; l.ximat[k] = l.xmat[k]; }
  } else if (lane < m.nb) {
    const int b = lane;
    V3 pos = {0.f, 0.f, 0.f}, anchor = {0.f, 0.f, 0.f}, axis = {0.f, 0.f, 1.f};
    Quat quat = {1.f, 0.f, 0.f, 0.f};
    Mat3 R = q2mat(quat);
    const int depth = m.body_depth[b];
    for (int d = 0; d < depth; ++d) {
      const int c = m.body_chain[b][d];
      const int jt = m.body_jtype[c];
      if (jt == kJntFree) {
        const int qa = m.body_qadr[c];
        pos = ld3(l.qpos + qa);
        quat = qnormalize({l.qpos[qa + 3], l.qpos[qa + 4], l.qpos[qa + 5], l.qpos[qa + 6]});
        anchor = pos;
        axis = {0.f, 0.f, 1.f};
      } else {
        V3 npos = pos + mul(R, ld3(m.body_pos[c]));
        Quat nq = qmul(quat, {m.body_quat[c][0], m.body_quat[c][1], m.body_quat[c][2], m.body_quat[c][3]});
        if (jt == kJntHinge) {
          const V3 jpos = ld3(m.jnt_pos[c]), jax = ld3(m.jnt_axis[c]);
          const Mat3 Rn = q2mat(nq);
          anchor = npos + mul(Rn, jpos);
          axis = mul(Rn, jax);
          const float s = l.sc[2 * m.body_qadr[c]], co = l.sc[2 * m.body_qadr[c] + 1];
          nq = qmul(nq, {co, jax.x * s, jax.y * s, jax.z * s});
          npos = anchor - mul(q2mat(nq), jpos);
        }
        quat = qnormalize(nq);
        pos = npos;
      }
      R = q2mat(quat);
    }
    st3(l.xpos + 3 * b, pos);
    l.xquat[4 * b] = quat.w; l.xquat[4 * b + 1] = quat.x; l.xquat[4 * b + 2] = quat.y; l.xquat[4 * b + 3] = quat.z;
    for (int k = 0; k < 9; ++k) l.xmat[9 * b + k] = R.m[k];
    st3(l.xanchor + 3 * b, anchor);
    st3(l.xaxis + 3 * b, axis);
    st3(l.xipos + 3 * b, pos + mul(R, ld3(m.body_ipos[b])));
    const Mat3 Ri = q2mat(qnormalize(
        qmul(quat, {m.body_iquat[b][0], m.body_iquat[b][1], m.body_iquat[b][2], m.body_iquat[b][3]})));
    for (int k = 0; k < 9; ++k) l.ximat[9 * b + k] = Ri.m[k];
  }
  KS_SYNC();
}

// centre of mass of the tree (wave-uniform result), com-based inertias, motion axes
__device__ inline V3 com_pos(const DevModel& m, const Lds& l, int lane, const float* mass_scale) {
  float mass = 0.f;
  V3 mp = {0.f, 0.f, 0.f};
  if (lane > 0 && lane < m.nb) {
    mass = m.body_mass[lane] * (mass_scale ? mass_scale[lane] : 1.f);
    mp = ld3(l.xipos + 3 * lane) * mass;
    l.bmass[lane] = mass;
  }
  const float mt = wave_sum(mass);
  const float inv = mt > 1e-15f ? 1.0f / mt : 0.f;
  const V3 com = {wave_sum(mp.x) * inv, wave_sum(mp.y) * inv, wave_sum(mp.z) * inv};
  if (lane == 0) {
    for (int k = 0; k < 10; ++k) l.cinert[k] = 0.f;
  } else if (lane < m.nb) {
    const int b = lane;
    const float* R = l.ximat + 9 * b;
    const float I0 = m.body_inertia[b][0], I1 = m.body_inertia[b][1], I2 = m.body_inertia[b][2];
    const V3 d = ld3(l.xipos + 3 * b) - com;
    const float xx = R[0] * I0 * R[0] + R[1] * I1 * R[1] + R[2] * I2 * R[2];
    const float yy = R[3] * I0 * R[3] + R[4] * I1 * R[4] + R[5] * I2 * R[5];
    const float zz = R[6] * I0 * R[6] + R[7] * I1 * R[7] + R[8] * I2 * R[8];
    const float xy = R[0] * I0 * R[3] + R[1] * I1 * R[4] + R[2] * I2 * R[5];
    const float xz = R[0] * I0 * R[6] + R[1] * I1 * R[7] + R[2] * I2 * R[8];
    const float yz = R[3] * I0 * R[6] + R[4] * I1 * R[7] + R[5] * I2 * R[8];
    const float d2 = dot(d, d);
    float* ci = l.cinert + 10 * b;
    ci[0] = xx + mass * (d2 - d.x * d.x);
    ci[1] = yy + mass * (d2 - d.y * d.y);
    ci[2] = zz + mass * (d2 - d.z * d.z);
    ci[3] = xy - mass * d.x * d.y;
    ci[4] = xz - mass * d.x * d.z;
    ci[5] = yz - mass * d.y * d.z;
    ci[6] = mass * d.x; ci[7] = mass * d.y; ci[8] = mass * d.z;
    ci[9] = mass;
  }
  if (lane < m.nv) {
    const int j = lane, b = m.dof_body[j];
    const V3 off = com - ld3(l.xanchor + 3 * b);
    Sp cd;
    if (m.body_jtype[b] == kJntFree) {
      const int k = j - m.body_dofadr[b];
      if (k < 3) {
        cd.a = {0.f, 0.f, 0.f};
        cd.l = {k == 0 ? 1.f : 0.f, k == 1 ? 1.f : 0.f, k == 2 ? 1.f : 0.f};
      } else {
        const float* R = l.xmat + 9 * b;
        const V3 ax = {R[k - 3], R[3 + k - 3], R[6 + k - 3]};
        cd.a = ax;
        cd.l = cross(ax, off);
      }
    } else {
      const V3 ax = ld3(l.xaxis + 3 * b);
      cd.a = ax;
      cd.l = cross(ax, off);
    }
    st6(l.cdof + 6 * j, cd);
  }
  KS_SYNC();
  return com;
}

// composite inertias (subtree sums over the depth-first body order) and the dense mass matrix
__device__ inline void crb_mass_matrix(const DevModel& m, const Lds& l, int lane) {
  for (int idx = lane; idx < m.nb * 10; idx += 64) {
    const int b = idx / 10, k = idx - 10 * b;
    float s = 0.f;
    if (b > 0) {
      const int e = m.body_subtree_end[b];
      for (int c = b; c < e; ++c) s += l.cinert[10 * c + k];
    }
    l.crb[idx] = s;
  }
  for (int idx = lane; idx < m.nv * m.nvs; idx += 64) l.M[idx] = 0.f;
  KS_SYNC();
  if (lane < m.nv) st6(l.buf + 6 * lane, inert_mul(l.crb + 10 * m.dof_body[lane], ld6(l.cdof + 6 * lane)));
  KS_SYNC();
  for (int p = lane; p < m.npairs; p += 64) {
    const int i = m.pair_i[p], j = m.pair_j[p];
    float v = dot(ld6(l.cdof + 6 * j), ld6(l.buf + 6 * i));
    if (i == j) v += m.dof_armature[i];
    l.M[i * m.nvs + j] = v;
    l.M[j * m.nvs + i] = v;
  }
  KS_SYNC();
}

// ------------------------------------------------------------------------------------------- velocity stage
// body velocities, axis derivatives and RNE with zero joint acceleration; leaves qfrc_bias in l.vbuf
__device__ inline void velocity_and_bias(const DevModel& m, const Lds& l, int lane) {
  if (lane == 0) {
    for (int k = 0; k < 6; ++k) { l.cvel[k] = 0.f; l.cfrc[k] = 0.f; }
  } else if (lane < m.nb) {
    const int b = lane;
    Sp v = {{0.f, 0.f, 0.f}, {0.f, 0.f, 0.f}};
    Sp acc = {{0.f, 0.f, 0.f}, {-m.gravity[0], -m.gravity[1], -m.gravity[2]}};
    const int depth = m.body_depth[b];
    for (int d = 0; d < depth; ++d) {
      const int c = m.body_chain[b][d];
      const int da = m.body_dofadr[c];
      if (m.body_jtype[c] == kJntFree) {
        for (int k = 0; k < 3; ++k) v = v + ld6(l.cdof + 6 * (da + k)) * l.qvel[da + k];
        Sp dv = {{0.f, 0.f, 0.f}, {0.f, 0.f, 0.f}};
        for (int k = 3; k < 6; ++k) {
          const Sp cd = ld6(l.cdof + 6 * (da + k));
          acc = acc + cross_motion(v, cd) * l.qvel[da + k];
          dv = dv + cd * l.qvel[da + k];
        }
        v = v + dv;
      } else if (m.body_jtype[c] == kJntHinge) {
        const Sp cd = ld6(l.cdof + 6 * da);
        acc = acc + cross_motion(v, cd) * l.qvel[da];
        v = v + cd * l.qvel[da];
      }
    }
    st6(l.cvel + 6 * b, v);
    const float* ci = l.cinert + 10 * b;
    st6(l.cfrc + 6 * b, inert_mul(ci, acc) + cross_force(v, inert_mul(ci, v)));
  }
  KS_SYNC();
  for (int idx = lane; idx < m.nb * 6; idx += 64) {
    const int b = idx / 6, k = idx - 6 * b;
    float s = 0.f;
    if (b > 0) {
      const int e = m.body_subtree_end[b];
      for (int c = b; c < e; ++c) s += l.cfrc[6 * c + k];
    }
    l.fsub[idx] = s;
  }
  KS_SYNC();
}

// ------------------------------------------------------------------------------------------- dense linear algebra in LDS
// In-place Cholesky of the lower triangle of A (row stride nvs): lane i owns row i.
__device__ inline void cholesky_inplace(float* A, int n, int nvs, int lane) {
  for (int j = 0; j < n; ++j) {
    float s = 0.f;
    if (lane >= j && lane < n) {
      const float* ri = A + lane * nvs;
      const float* rj = A + j * nvs;
      s = ri[j];
      for (int k = 0; k < j; ++k) s -= ri[k] * rj[k];
    }
    const float piv = lane_bcast(s, j);
    const float d = sqrtf(fmaxf(piv, 1e-30f));
    const float inv = 1.0f / d;
    if (lane == j) A[j * nvs + j] = d;
    else if (lane > j && lane < n) A[lane * nvs + j] = s * inv;
    KS_SYNC();
  }
}

// x = (L L^T)^-1 b with lane i holding b_i / x_i in a register
__device__ inline float cholesky_solve(const float* L, int n, int nvs, int lane, float b) {
  float r = b;
  for (int j = 0; j < n; ++j) {
    const float xj = lane_bcast(r, j) / L[j * nvs + j];
    if (lane == j) r = xj;
    else if (lane > j && lane < n) r -= L[lane * nvs + j] * xj;
  }
  for (int j = n - 1; j >= 0; --j) {
    const float xj = lane_bcast(r, j) / L[j * nvs + j];
    if (lane == j) r = xj;
    else if (lane < j) r -= L[j * nvs + lane] * xj;
  }
  return r;
}

struct LsPoint {
  float alpha, cost, d0, d1;
};

__device__ __forceinline__ bool in_bracket(const LsPoint& x, const LsPoint& y) {
  return ((x.d0 < y.d0) && (y.d0 < 0.f)) || ((x.d0 > y.d0) && (y.d0 > 0.f));
}

// ------------------------------------------------------------------------------------------- the fused kernel
// FWD = true is the forward-only variant (derived fields + warm start of a given state, no actuation, no
// integration) that replaces the mjx.forward of a reset.
template <bool FWD>
__global__ __launch_bounds__(64) void step_kernel(StepArgs a) {
  extern __shared__ float lds_raw[];
  const DevModel& m = *a.model;
  const int lane = threadIdx.x;
  const int64_t env = blockIdx.x;
  if (a.env_mask && !a.env_mask[env]) return;  // wave-uniform
  const int nb = m.nb, nq = m.nq, nv = m.nv, nu = m.nu, ns = m.ns, nvs = m.nvs;
  const Lds l = carve(lds_raw, m);
  const int rq = (nb > 1 && m.body_jtype[1] == kJntFree) ? 7 : 0;
  const int rv = rq ? 6 : 0;

  for (int i = lane; i < nq; i += 64) l.qpos[i] = a.qpos[env * nq + i];
  for (int i = lane; i < nv; i += 64) {
    l.qvel[i] = a.qvel[env * nv + i];
    l.warm[i] = a.qacc_warmstart ? a.qacc_warmstart[env * nv + i] : 0.f;
  }
  for (int i = lane; i < nu; i += 64) l.tau[i] = a.ctrl_in ? a.ctrl_in[env * nu + i] : 0.f;
  const float mu = a.friction ? a.friction[env] : m.friction;
  const float* mass_scale = a.mass_scale ? a.mass_scale + env * nb : nullptr;
  float time = a.time ? a.time[env] : 0.f;
  const float latency = a.latency ? a.latency[env] : 0.f;
  const float kp_scale = a.kp_scale ? a.kp_scale[env] : 1.f;
  const float kd_scale = a.kd_scale ? a.kd_scale[env] : 1.f;
  const float lim_scale = a.torque_limit_scale ? a.torque_limit_scale[env] : 1.f;
  const float scale = 1.0f / (m.meaninertia * (float)(nv > 1 ? nv : 1));
  int niter_out = 0, nefc_out = 0;
  float my_qacc = 0.f;
  KS_SYNC();

  const int nsub = FWD ? 1 : a.substeps;
  for (int sub = 0; sub < nsub; ++sub) {
    // ---- actuators (ksim/engine.py:287-320, ksim/actuators.py:198-217)
    if (!FWD && (sub % a.actuator_period) == 0 && lane < nu) {
      const int u = lane;
      const int64_t eu = env * nu + u;
      float prct = (float)sub - latency;
      prct = fminf(fmaxf(prct, 0.f), 1.f);
      const float last = a.last_ctrl[eu], act = a.action[eu];
      const bool drop = a.drop && a.drop[eu];
      const float c = drop ? last : last * (1.0f - prct) + act * prct;
      const int64_t su = ((int64_t)sub * a.N + env) * nu + u;
      float t;
      if (a.actuator_type == KS_ACT_TORQUE) {
        t = c + (a.torque_noise ? a.torque_noise[su] : 0.f);
      } else {
        const float target = c * a.action_scale + (a.action_noise ? a.action_noise[su] : 0.f) +
                             (a.action_bias ? a.action_bias[eu] : 0.f);
        const float q = l.qpos[rq + u] - (a.zero_offset ? a.zero_offset[eu] : 0.f);
        t = (a.kp[u] * kp_scale) * (target - q) + (a.kd[u] * kd_scale) * (0.f - l.qvel[rv + u]);
        t = t + (a.torque_noise ? a.torque_noise[su] : 0.f) + (a.torque_bias ? a.torque_bias[eu] : 0.f);
        const float lim = a.ctrl_clip[u] * lim_scale;
        t = fminf(fmaxf(t, -lim), lim);
      }
      l.tau[u] = t;
    }
    KS_SYNC();

    // ---- position and velocity stages
    kinematics(m, l, lane);
    const V3 com = com_pos(m, l, lane, mass_scale);
    crb_mass_matrix(m, l, lane);
    velocity_and_bias(m, l, lane);

    // smooth forces: passive - bias + actuator
    float qfs = 0.f, my_qvel = 0.f;
    if (lane < nv) {
      const int j = lane;
      my_qvel = l.qvel[j];
      const float bias = dot(ld6(l.cdof + 6 * j), ld6(l.fsub + 6 * m.dof_body[j]));
      float f = -m.dof_damping[j] * my_qvel - bias;
      const int u = m.dof_act[j];
      if (u >= 0) {
        const float c = fminf(fmaxf(l.tau[u], m.act_lo[u]), m.act_hi[u]);
        f += m.act_gear[u] * c;
      }
      qfs = f;
      l.qfs[j] = f;
      if (a.dbg_bias) a.dbg_bias[env * nv + j] = bias;
    }

    // ---- contacts: sphere vs plane z = 0, compacted to the penetrating ones
    float dist = 1.f;
    V3 cpos = {0.f, 0.f, 0.f};
    if (lane < ns) {
      const int b = m.sph_body[lane];
      const float* R = l.xmat + 9 * b;
      const V3 lp = ld3(m.sph_pos[lane]);
      const V3 c = ld3(l.xpos + 3 * b) + V3{R[0] * lp.x + R[1] * lp.y + R[2] * lp.z,
                                           R[3] * lp.x + R[4] * lp.y + R[5] * lp.z,
                                           R[6] * lp.x + R[7] * lp.y + R[8] * lp.z};
      const float r = m.sph_radius[lane];
      dist = c.z - r;
      cpos = {c.x, c.y, c.z - r - 0.5f * dist};
      if (a.dbg_con_dist) a.dbg_con_dist[env * ns + lane] = dist;
    }
    const bool touching = (lane < ns) && (dist < 0.f);
    const unsigned long long cmask = __ballot(touching);
    const int ncon = __popcll(cmask);
    const int nefc = 4 * ncon;
    if (touching) {
      const int c = __popcll(cmask & ((1ull << lane) - 1ull));
      const int b = m.sph_body[lane];
      l.con_body[c] = b;
      st3(l.con_off + 3 * c, cpos - com);
      const float t = m.body_invweight0[b];
      const float invweight = (t + mu * mu * t) * 2.f * mu * mu / m.impratio;
      const float ix = fabsf(dist) / m.width;
      const float ia = (1.0f / powf(m.mid, m.power - 1.f)) * powf(ix, m.power);
      const float ib = 1.f - (1.0f / powf(1.f - m.mid, m.power - 1.f)) * powf(1.f - ix, m.power);
      const float iy = ix < m.mid ? ia : ib;
      float imp = m.dmin + iy * (m.dmax - m.dmin);
      imp = fminf(fmaxf(imp, m.dmin), m.dmax);
      if (ix > 1.f) imp = m.dmax;
      float Rr = invweight * (1.f - imp) / imp;
      Rr = fmaxf(Rr, 1e-15f);
      l.con_D[c] = 1.0f / Rr;
      l.con_kip[c] = m.con_k * imp * dist;
    }
    KS_SYNC();
    for (int idx = lane; idx < nefc * nv; idx += 64) {
      const int r = idx / nv, j = idx - r * nv;
      const int c = r >> 2, q = r & 3;
      const int b = l.con_body[c];
      float val = 0.f;
      if ((m.body_dofmask[b] >> j) & 1u) {
        const Sp cd = ld6(l.cdof + 6 * j);
        const V3 jac = cd.l + cross(cd.a, ld3(l.con_off + 3 * c));
        const float tang = (q < 2) ? jac.y : -jac.x;
        val = jac.z + ((q & 1) ? -mu : mu) * tang;
      }
      l.J[r * nvs + j] = val;
    }
    // ---- factor M (into H) and the unconstrained acceleration
    for (int idx = lane; idx < nv * nvs; idx += 64) l.H[idx] = l.M[idx];
    if (a.dbg_M) for (int idx = lane; idx < nv * nv; idx += 64) a.dbg_M[env * nv * nv + idx] = l.M[(idx / nv) * nvs + idx % nv];
    KS_SYNC();
    cholesky_inplace(l.H, nv, nvs, lane);
    const float qas = cholesky_solve(l.H, nv, nvs, lane, qfs);
    if (a.dbg_qacc_smooth && lane < nv) a.dbg_qacc_smooth[env * nv + lane] = qas;

    // ---- constraint rows: reference acceleration and regulariser (lane = row)
    float aref = 0.f, D = 0.f;
    if (lane < nefc) {
      const float* Jr = l.J + lane * nvs;
      float vel = 0.f;
      for (int j = 0; j < nv; ++j) vel += Jr[j] * l.qvel[j];
      aref = -m.con_b * vel - l.con_kip[lane >> 2];
      D = l.con_D[lane >> 2];
    }

    // ---- Newton solver (wave-uniform control flow)
    float qacc = qas;
    int niter = 0;
    if (nefc > 0) {
      const float warm = (lane < nv) ? l.warm[lane] : 0.f;
      // cost of the warm start and of the unconstrained acceleration
      float Ma_w = 0.f, Ma_s = 0.f, Jar_w = 0.f, Jar_s = 0.f;
      KS_SYNC();
      if (lane < nv) l.vbuf[lane] = warm;
      KS_SYNC();
      if (lane < nv) { const float* Mr = l.M + lane * nvs; for (int j = 0; j < nv; ++j) Ma_w += Mr[j] * l.vbuf[j]; }
      if (lane < nefc) { const float* Jr = l.J + lane * nvs; for (int j = 0; j < nv; ++j) Jar_w += Jr[j] * l.vbuf[j]; Jar_w -= aref; }
      KS_SYNC();
      if (lane < nv) l.vbuf[lane] = qas;
      KS_SYNC();
      if (lane < nv) { const float* Mr = l.M + lane * nvs; for (int j = 0; j < nv; ++j) Ma_s += Mr[j] * l.vbuf[j]; }
      if (lane < nefc) { const float* Jr = l.J + lane * nvs; for (int j = 0; j < nv; ++j) Jar_s += Jr[j] * l.vbuf[j]; Jar_s -= aref; }
      const float cost_w = wave_sum((lane < nefc && Jar_w < 0.f) ? 0.5f * D * Jar_w * Jar_w : 0.f) +
                           0.5f * wave_sum((lane < nv) ? (Ma_w - qfs) * (warm - qas) : 0.f);
      const float cost_s = wave_sum((lane < nefc && Jar_s < 0.f) ? 0.5f * D * Jar_s * Jar_s : 0.f) +
                           0.5f * wave_sum((lane < nv) ? (Ma_s - qfs) * (qas - qas) : 0.f);
      const bool use_warm = cost_w < cost_s;
      qacc = use_warm ? warm : qas;
      float Ma = use_warm ? Ma_w : Ma_s;
      float Jaref = use_warm ? Jar_w : Jar_s;
      float cost = use_warm ? cost_w : cost_s;
      float prev_cost = INFINITY;
      float gauss = 0.f, grad = 0.f, search = 0.f, qfc = 0.f;
      bool active = false;

      auto update_constraint_and_gradient = [&](bool first) {
        active = (lane < nefc) && (Jaref < 0.f);
        const float force = active ? -D * Jaref : 0.f;
        KS_SYNC();
        if (lane < nefc) { l.fbuf[lane] = force; l.wbuf[lane] = active ? D : 0.f; }
        KS_SYNC();
        qfc = 0.f;
        if (lane < nv) for (int r = 0; r < nefc; ++r) qfc += l.J[r * nvs + lane] * l.fbuf[r];
        gauss = 0.5f * wave_sum((lane < nv) ? (Ma - qfs) * (qacc - qas) : 0.f);
        if (!first) {
          prev_cost = cost;
          cost = wave_sum(active ? 0.5f * D * Jaref * Jaref : 0.f) + gauss;
        }
        grad = (lane < nv) ? Ma - qfs - qfc : 0.f;
        // H = M + J^T diag(D active) J  (lower triangle), then factor and solve
        for (int idx = lane; idx < nv * nv; idx += 64) {
          const int i = idx / nv, j = idx - i * nv;
          if (j <= i) {
            float h = l.M[i * nvs + j];
            for (int r = 0; r < nefc; ++r) h += l.wbuf[r] * l.J[r * nvs + i] * l.J[r * nvs + j];
            l.H[i * nvs + j] = h;
          }
        }
        KS_SYNC();
        cholesky_inplace(l.H, nv, nvs, lane);
        const float mgrad = cholesky_solve(l.H, nv, nvs, lane, grad);
        search = -mgrad;
      };
      update_constraint_and_gradient(true);

      while (true) {
        const float improvement = scale * (prev_cost - cost);
        const float gradient = scale * sqrtf(wave_sum(grad * grad));
        bool done = niter >= m.iterations;
        done |= improvement < m.tolerance;
        done |= gradient < m.tolerance;
        if (done && !(m.iterations == 1 && niter == 0)) break;

        // ---- exact line search along `search`
        KS_SYNC();
        if (lane < nv) l.vbuf[lane] = search;
        KS_SYNC();
        float mv = 0.f, jv = 0.f;
        if (lane < nv) { const float* Mr = l.M + lane * nvs; for (int j = 0; j < nv; ++j) mv += Mr[j] * l.vbuf[j]; }
        if (lane < nefc) { const float* Jr = l.J + lane * nvs; for (int j = 0; j < nv; ++j) jv += Jr[j] * l.vbuf[j]; }
        const float smag = sqrtf(wave_sum(search * search)) * m.meaninertia * (float)(nv > 1 ? nv : 1);
        const float gtol = m.tolerance * m.ls_tolerance * smag;
        const float q0r = 0.5f * Jaref * Jaref * D, q1r = jv * Jaref * D, q2r = 0.5f * jv * jv * D;
        const float g0 = gauss;
        const float g1 = wave_sum((lane < nv) ? search * (Ma - qfs) : 0.f);
        const float g2 = 0.5f * wave_sum((lane < nv) ? search * mv : 0.f);
        auto point = [&](float alpha) {
          const bool on = (lane < nefc) && (Jaref + alpha * jv < 0.f);
          const float q0 = g0 + wave_sum(on ? q0r : 0.f);
          const float q1 = g1 + wave_sum(on ? q1r : 0.f);
          const float q2 = g2 + wave_sum(on ? q2r : 0.f);
          LsPoint p;
          p.alpha = alpha;
          p.cost = alpha * alpha * q2 + alpha * q1 + q0;
          p.d0 = 2.f * alpha * q2 + q1;
          p.d1 = 2.f * q2 + (q2 == 0.f ? 1e-15f : 0.f);
          return p;
        };
        const LsPoint p0 = point(0.f);
        LsPoint lo = point(p0.alpha - p0.d0 / p0.d1);
        LsPoint hi;
        if (lo.d0 < p0.d0) { hi = p0; } else { hi = lo; lo = p0; }
        bool swap = true;
        int it = 0;
        while (true) {
          bool ls_done = it >= m.ls_iterations;
          ls_done |= !swap;
          ls_done |= (lo.d0 < 0.f) && (lo.d0 > -gtol);
          ls_done |= (hi.d0 > 0.f) && (hi.d0 < gtol);
          if (ls_done) break;
          const LsPoint lo_next = point(lo.alpha - lo.d0 / lo.d1);
          const LsPoint hi_next = point(hi.alpha - hi.d0 / hi.d1);
          const LsPoint mid = point(0.5f * (lo.alpha + hi.alpha));
          LsPoint nlo = lo, nhi = hi;
          const bool s1 = in_bracket(nlo, lo_next); if (s1) nlo = lo_next;
          const bool s2 = in_bracket(nlo, mid);     if (s2) nlo = mid;
          const bool s3 = in_bracket(nlo, hi_next); if (s3) nlo = hi_next;
          const bool t1 = in_bracket(nhi, hi_next); if (t1) nhi = hi_next;
          const bool t2 = in_bracket(nhi, mid);     if (t2) nhi = mid;
          const bool t3 = in_bracket(nhi, lo_next); if (t3) nhi = lo_next;
          lo = nlo; hi = nhi;
          swap = s1 | s2 | s3 | t1 | t2 | t3;
          ++it;
        }
        const bool improved = (lo.cost < p0.cost) || (hi.cost < p0.cost);
        float alpha = lo.cost < hi.cost ? lo.alpha : hi.alpha;
        if (!improved) alpha = 0.f;
        qacc += alpha * search;
        Ma += alpha * mv;
        Jaref += alpha * jv;
        update_constraint_and_gradient(false);
        ++niter;
      }
    }
    niter_out = niter;
    nefc_out = nefc;
    my_qacc = qacc;
    KS_SYNC();
    if (lane < nv) { l.warm[lane] = qacc; l.qacc[lane] = qacc; }

    // ---- semi-implicit Euler
    if (!FWD) {
      if (lane < nv) l.qvel[lane] = my_qvel + m.dt * qacc;
      KS_SYNC();
      if (lane > 0 && lane < nb) {
        const int b = lane, qa = m.body_qadr[b], da = m.body_dofadr[b];
        if (m.body_jtype[b] == kJntFree) {
          for (int k = 0; k < 3; ++k) l.qpos[qa + k] += m.dt * l.qvel[da + k];
          const V3 w = ld3(l.qvel + da + 3);
          const float n = sqrtf(dot(w, w));
          Quat q = {l.qpos[qa + 3], l.qpos[qa + 4], l.qpos[qa + 5], l.qpos[qa + 6]};
          if (n > 1e-15f) {
            const float h = 0.5f * n * m.dt, s = sinf(h) / n;
            q = qmul(q, {cosf(h), w.x * s, w.y * s, w.z * s});
          }
          q = qnormalize(q);
          l.qpos[qa + 3] = q.w; l.qpos[qa + 4] = q.x; l.qpos[qa + 5] = q.y; l.qpos[qa + 6] = q.z;
        } else if (m.body_jtype[b] == kJntHinge) {
          l.qpos[qa] += m.dt * l.qvel[da];
        }
      }
      time += m.dt;
    }
    KS_SYNC();
  }

  // ---- write back
  if (!FWD) {
    for (int i = lane; i < nq; i += 64) a.qpos[env * nq + i] = l.qpos[i];
    for (int i = lane; i < nv; i += 64) a.qvel[env * nv + i] = l.qvel[i];
    if (a.time && lane == 0) a.time[env] = time;
    if (a.last_ctrl) for (int i = lane; i < nu; i += 64) a.last_ctrl[env * nu + i] = a.action[env * nu + i];
  }
  if (a.qacc_warmstart) for (int i = lane; i < nv; i += 64) a.qacc_warmstart[env * nv + i] = l.warm[i];
  if (a.qacc && lane < nv) a.qacc[env * nv + lane] = my_qacc;
  if (a.ctrl_out) for (int i = lane; i < nu; i += 64) a.ctrl_out[env * nu + i] = l.tau[i];
  if (a.xpos) for (int i = lane; i < nb * 3; i += 64) a.xpos[env * nb * 3 + i] = l.xpos[i];
  if (a.xquat) for (int i = lane; i < nb * 4; i += 64) a.xquat[env * nb * 4 + i] = l.xquat[i];
  if (a.cvel) for (int i = lane; i < nb * 6; i += 64) a.cvel[env * nb * 6 + i] = l.cvel[i];
  if (a.traj_ctrl) for (int i = lane; i < nu; i += 64) a.traj_ctrl[env * nu + i] = l.tau[i];
  if (a.traj_xpos) for (int i = lane; i < nb * 3; i += 64) a.traj_xpos[env * nb * 3 + i] = l.xpos[i];
  if (a.traj_xquat) for (int i = lane; i < nb * 4; i += 64) a.traj_xquat[env * nb * 4 + i] = l.xquat[i];
  if (a.solver_niter && lane == 0) a.solver_niter[env] = niter_out;
  if (a.nefc && lane == 0) a.nefc[env] = nefc_out;
}

}  // namespace ks

using namespace ks;

// ---------------------------------------------------------------------------------------------
// C ABI: model upload and the step / forward entry points
// ---------------------------------------------------------------------------------------------
struct KsModel {
  DevModel host;
  DevModel* dev;
  int device;
};

extern "C" int ks_model_create(const KsModelDesc* d, KsModel** out) {
  if (!d || !out) return fail(KS_EINVAL, "ks_model_create: null argument");
  if (d->nb < 1 || d->nb > kMaxB || d->nq < 0 || d->nq > kMaxQ || d->nv < 0 || d->nv > kMaxV || d->nu < 0 ||
      d->nu > kMaxU || d->ns < 0 || d->ns > kMaxS)
    return fail(KS_ELIMIT, "ks_model_create: sizes nb=%d nq=%d nv=%d nu=%d ns=%d exceed %d/%d/%d/%d/%d", d->nb, d->nq,
                d->nv, d->nu, d->ns, kMaxB, kMaxQ, kMaxV, kMaxU, kMaxS);
  if (d->nv > 64 || 4 * d->ns > 64) return fail(KS_ELIMIT, "ks_model_create: more than 64 dofs or constraint rows");
  if (d->eulerdamp) return fail(KS_EINVAL, "ks_model_create: the implicit-damping Euler variant is not implemented");
  if (!(d->dt > 0.0)) return fail(KS_EINVAL, "ks_model_create: dt must be positive");
  KsModel* km = new KsModel();
  DevModel& m = km->host;
  std::memset(&m, 0, sizeof(m));
  m.nb = d->nb; m.nq = d->nq; m.nv = d->nv; m.nu = d->nu; m.ns = d->ns;
  m.iterations = d->iterations; m.ls_iterations = d->ls_iterations; m.eulerdamp = d->eulerdamp;
  m.nvs = d->nv | 1;
  m.dt = (float)d->dt;
  for (int k = 0; k < 3; ++k) m.gravity[k] = (float)d->gravity[k];
  m.tolerance = (float)d->tolerance; m.ls_tolerance = (float)d->ls_tolerance;
  m.meaninertia = (float)d->meaninertia; m.friction = (float)d->friction; m.impratio = (float)d->impratio;
  {  // solref / solimp -> (k, b) and clamped impedance parameters
    double timeconst = d->solref[0], dampratio = d->solref[1];
    double dmin = d->solimp[0], dmax = d->solimp[1], width = d->solimp[2], mid = d->solimp[3], power = d->solimp[4];
    if (timeconst < 2 * d->dt) timeconst = 2 * d->dt;
    auto clampd = [](double x, double lo, double hi) { return x < lo ? lo : (x > hi ? hi : x); };
    dmin = clampd(dmin, 1e-4, 0.9999); dmax = clampd(dmax, 1e-4, 0.9999);
    width = width < 1e-15 ? 1e-15 : width; mid = clampd(mid, 1e-4, 0.9999); power = power < 1 ? 1 : power;
    double k = 1.0 / (dmax * dmax * timeconst * timeconst * dampratio * dampratio), b = 2.0 / (dmax * timeconst);
    if (d->solref[0] <= 0) k = -d->solref[0] / (dmax * dmax);
    if (d->solref[1] <= 0) b = -d->solref[1] / dmax;
    m.con_k = (float)k; m.con_b = (float)b; m.dmin = (float)dmin; m.dmax = (float)dmax; m.width = (float)width;
    m.mid = (float)mid; m.power = (float)power;
  }
  for (int b = 0; b < d->nb; ++b) {
    m.body_parent[b] = d->body_parent[b]; m.body_jtype[b] = d->body_jtype[b]; m.body_qadr[b] = d->body_qadr[b];
    m.body_dofadr[b] = d->body_dofadr[b]; m.body_subtree_end[b] = d->body_subtree_end[b];
    if (b > 0 && (d->body_parent[b] < 0 || d->body_parent[b] >= b)) { delete km; return fail(KS_EINVAL, "ks_model_create: body %d has parent %d (must precede it)", b, d->body_parent[b]); }
    if (d->body_subtree_end[b] <= b || d->body_subtree_end[b] > d->nb) { delete km; return fail(KS_EINVAL, "ks_model_create: bad subtree_end for body %d", b); }
    if (b > 0 && d->body_jtype[b] != kJntFree && d->body_jtype[b] != kJntHinge) { delete km; return fail(KS_EINVAL, "ks_model_create: body %d needs a free or hinge joint", b); }
    for (int k = 0; k < 3; ++k) {
      m.body_pos[b][k] = (float)d->body_pos[b][k]; m.body_ipos[b][k] = (float)d->body_ipos[b][k];
      m.body_inertia[b][k] = (float)d->body_inertia[b][k]; m.jnt_axis[b][k] = (float)d->jnt_axis[b][k];
      m.jnt_pos[b][k] = (float)d->jnt_pos[b][k];
    }
    for (int k = 0; k < 4; ++k) { m.body_quat[b][k] = (float)d->body_quat[b][k]; m.body_iquat[b][k] = (float)d->body_iquat[b][k]; }
    m.body_mass[b] = (float)d->body_mass[b];
    m.body_invweight0[b] = (float)d->body_invweight0[b];
    // chain from the root down to b
    int chain[kMaxB], n = 0;
    for (int c = b; c > 0; c = d->body_parent[c]) chain[n++] = c;
    if (n > kMaxDepth) { delete km; return fail(KS_ELIMIT, "ks_model_create: tree deeper than %d", kMaxDepth); }
    m.body_depth[b] = n;
    for (int k = 0; k < n; ++k) m.body_chain[b][k] = chain[n - 1 - k];
  }
  for (int q = 0; q < d->nq; ++q) m.qpos0[q] = (float)d->qpos0[q];
  for (int j = 0; j < d->nv; ++j) {
    m.dof_body[j] = d->dof_body[j]; m.dof_parent[j] = d->dof_parent[j]; m.dof_act[j] = -1;
    m.dof_damping[j] = (float)d->dof_damping[j]; m.dof_armature[j] = (float)d->dof_armature[j];
    if (d->dof_parent[j] >= j || d->dof_body[j] < 1 || d->dof_body[j] >= d->nb) { delete km; return fail(KS_EINVAL, "ks_model_create: bad dof %d", j); }
  }
  for (int u = 0; u < d->nu; ++u) {
    const int j = d->act_dof[u];
    if (j < 0 || j >= d->nv) { delete km; return fail(KS_EINVAL, "ks_model_create: actuator %d drives dof %d", u, j); }
    if (m.dof_act[j] >= 0) { delete km; return fail(KS_EINVAL, "ks_model_create: dof %d has two actuators", j); }
    m.dof_act[j] = u; m.act_dof[u] = j; m.act_gear[u] = (float)d->act_gear[u];
    m.act_lo[u] = (float)d->act_lo[u]; m.act_hi[u] = (float)d->act_hi[u];
  }
  for (int s = 0; s < d->ns; ++s) {
    if (d->sph_body[s] < 1 || d->sph_body[s] >= d->nb) { delete km; return fail(KS_EINVAL, "ks_model_create: sphere %d on body %d", s, d->sph_body[s]); }
    m.sph_body[s] = d->sph_body[s]; m.sph_radius[s] = (float)d->sph_radius[s];
    for (int k = 0; k < 3; ++k) m.sph_pos[s][k] = (float)d->sph_pos[s][k];
  }
  // dof masks and (i, ancestor j) pairs
  int np = 0;
  for (int i = 0; i < d->nv; ++i)
    for (int j = i; j >= 0; j = d->dof_parent[j]) {
      m.pair_i[np] = (short)i; m.pair_j[np] = (short)j; ++np;
    }
  m.npairs = np;
  for (int b = 1; b < d->nb; ++b) {
    unsigned mask = 0;
    for (int j = 0; j < d->nv; ++j) {
      for (int c = b; c > 0; c = d->body_parent[c])
        if (c == d->dof_body[j]) { mask |= 1u << j; break; }
    }
    m.body_dofmask[b] = mask;
  }
  if (hipGetDevice(&km->device) != hipSuccess) { delete km; return fail(KS_ELAUNCH, "ks_model_create: no HIP device"); }
  if (hipMalloc((void**)&km->dev, sizeof(DevModel)) != hipSuccess) { delete km; return fail(KS_ELAUNCH, "ks_model_create: hipMalloc failed"); }
  if (hipMemcpy(km->dev, &m, sizeof(DevModel), hipMemcpyHostToDevice) != hipSuccess) {
    (void)hipFree(km->dev); delete km; return fail(KS_ELAUNCH, "ks_model_create: upload failed");
  }
  *out = km;
  return KS_OK;
}

extern "C" int ks_model_destroy(KsModel* m) {
  if (!m) return KS_OK;
  (void)hipFree(m->dev);
  delete m;
  return KS_OK;
}

extern "C" int ks_model_lds_bytes(const KsModel* m) {
  if (!m) return 0;
  return lds_floats(m->host.nb, m->host.nq, m->host.nv, m->host.nu, m->host.ns) * 4;
}

static int launch_step(const KsModel* km, ks_stream_t stream, const KsStepIO* io, bool forward_only) {
  if (!km || !io) return fail(KS_EINVAL, "ks_step: null argument");
  const DevModel& m = km->host;
  if (io->N < 0) return fail(KS_EINVAL, "ks_step: negative env count");
  if (io->N == 0) return KS_OK;
  if (io->N > 0x7fffffff) return fail(KS_ELIMIT, "ks_step: too many envs");
  if (!io->qpos || !io->qvel) return fail(KS_EINVAL, "ks_step: qpos and qvel are required");
  StepArgs a;
  std::memset(&a, 0, sizeof(a));
  a.model = km->dev;
  a.N = io->N;
  a.qpos = io->qpos; a.qvel = io->qvel; a.qacc_warmstart = io->qacc_warmstart; a.time = io->time;
  a.friction = io->friction; a.mass_scale = io->mass_scale; a.env_mask = io->env_mask;
  a.qacc = io->qacc; a.ctrl_out = io->ctrl_out; a.xpos = io->xpos; a.xquat = io->xquat; a.cvel = io->cvel;
  a.traj_ctrl = io->traj_ctrl; a.traj_xpos = io->traj_xpos; a.traj_xquat = io->traj_xquat;
  a.solver_niter = io->solver_niter; a.nefc = io->nefc;
  a.dbg_M = io->dbg_M; a.dbg_bias = io->dbg_bias; a.dbg_qacc_smooth = io->dbg_qacc_smooth;
  a.dbg_con_dist = io->dbg_con_dist;
  a.ctrl_in = io->ctrl_in;
  if (!forward_only) {
    if (io->substeps < 1 || io->substeps > 64) return fail(KS_EINVAL, "ks_step: substeps must be in 1..64");
    if (io->actuator_period < 1) return fail(KS_EINVAL, "ks_step: actuator_period must be >= 1");
    if (m.nu > 0 && (!io->action || !io->last_ctrl)) return fail(KS_EINVAL, "ks_step: action and last_ctrl are required");
    if (io->actuator_type != KS_ACT_TORQUE && io->actuator_type != KS_ACT_POSITION)
      return fail(KS_EINVAL, "ks_step: unknown actuator type %d", io->actuator_type);
    if (io->actuator_type == KS_ACT_POSITION && m.nu > 0 && (!io->kp || !io->kd || !io->ctrl_clip))
      return fail(KS_EINVAL, "ks_step: position actuators need kp, kd and ctrl_clip");
    if (io->actuator_type == KS_ACT_POSITION && m.nu + (m.body_jtype[1] == kJntFree ? 7 : 0) > m.nq)
      return fail(KS_EINVAL, "ks_step: position actuators assume one actuator per joint after the root");
    a.substeps = io->substeps; a.actuator_period = io->actuator_period; a.actuator_type = io->actuator_type;
    a.action = io->action; a.last_ctrl = io->last_ctrl; a.latency = io->latency; a.zero_offset = io->zero_offset;
    a.drop = io->drop; a.kp = io->kp; a.kd = io->kd; a.ctrl_clip = io->ctrl_clip;
    a.kp_scale = io->kp_scale; a.kd_scale = io->kd_scale; a.torque_limit_scale = io->torque_limit_scale;
    a.action_scale = io->action_scale;
    a.action_noise = io->action_noise; a.torque_noise = io->torque_noise; a.action_bias = io->action_bias;
    a.torque_bias = io->torque_bias;
  }
  const int bytes = lds_floats(m.nb, m.nq, m.nv, m.nu, m.ns) * 4;
  if (bytes > 160 * 1024) return fail(KS_ELIMIT, "ks_step: model needs %d bytes of LDS", bytes);
  const void* fn = forward_only ? (const void*)step_kernel<true> : (const void*)step_kernel<false>;
  if (bytes > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return fail(KS_ELAUNCH, "ks_step: cannot raise the LDS limit: %s", hipGetErrorString(e));
  }
  if (forward_only) hipLaunchKernelGGL(step_kernel<true>, dim3((unsigned)io->N), dim3(64), bytes, (hipStream_t)stream, a);
  else hipLaunchKernelGGL(step_kernel<false>, dim3((unsigned)io->N), dim3(64), bytes, (hipStream_t)stream, a);
  return check_launch("ks_step");
}

extern "C" int ks_step(const KsModel* model, ks_stream_t stream, const KsStepIO* io) {
  return launch_step(model, stream, io, false);
}

extern "C" int ks_forward(const KsModel* model, ks_stream_t stream, const KsStepIO* io) {
  return launch_step(model, stream, io, true);
}
