/* CPU oracle of the per-env dynamics step — see ks_dyn_oracle.h.  TEST INFRASTRUCTURE.
 *
 * Build: gcc -O2 -DREAL=double -DSUF=_f64 ...  and  -DREAL=float -DSUF=_f32 (oracle/Makefile).
 * Spatial vectors are [angular(3); linear(3)], expressed in world axes about the
 * centre of mass of the whole tree (MuJoCo's "com-based" frame).
 */
#include "ks_dyn_oracle.h"

#include <math.h>
#include <string.h>

#ifndef REAL
#define REAL double
#define SUF _f64
#endif
#define CAT_(a, b) a##b
#define CAT(a, b) CAT_(a, b)
#define FN(name) CAT(name, SUF)

#define MINVAL ((REAL)1e-15)
#define MINIMP ((REAL)0.0001)
#define MAXIMP ((REAL)0.9999)

typedef struct FN(KsorData) {
  /* state (in/out) */
  REAL qpos[KSOR_MAXQ], qvel[KSOR_MAXV], ctrl[KSOR_MAXU], qacc_warmstart[KSOR_MAXV], time;
  /* per-env parameters */
  REAL mass_scale[KSOR_MAXB], friction;
  REAL armature_scale[KSOR_MAXV], damping_scale[KSOR_MAXV]; /* ksim/randomization.py:108-123, 226-243 */
  /* per-env replacements of model fields, used when their flag is set (ksim/randomization.py:56-71 dof_frictionloss,
   * 290-356 body_ipos, 359-383 body_inertia, 386-487 collision geometry, here the contact spheres) */
  int has_ipos, has_inertia, has_frictionloss, has_spheres;
  REAL body_ipos[KSOR_MAXB][3], body_inertia[KSOR_MAXB][3], dof_frictionloss[KSOR_MAXV], sph_pos[KSOR_MAXS][3],
      sph_radius[KSOR_MAXS];
  /* Cartesian force (3) and torque (3) per body, world frame, acting at the body's centre of mass: MuJoCo's
   * xfrc_applied, which ForcePushEvent writes (ksim/events.py:302-307) */
  REAL xfrc_applied[KSOR_MAXB][6];
  /* position-dependent */
  REAL xpos[KSOR_MAXB][3], xquat[KSOR_MAXB][4], xmat[KSOR_MAXB][9], xipos[KSOR_MAXB][3], ximat[KSOR_MAXB][9],
      xanchor[KSOR_MAXB][3], xaxis[KSOR_MAXB][3], com[3];
  REAL cinert[KSOR_MAXB][10], crb[KSOR_MAXB][10], cdof[KSOR_MAXV][6];
  REAL M[KSOR_MAXV * KSOR_MAXV], L[KSOR_MAXV * KSOR_MAXV];
  /* velocity-dependent */
  REAL cvel[KSOR_MAXB][6], cdof_dot[KSOR_MAXV][6];
  REAL qfrc_bias[KSOR_MAXV], qfrc_passive[KSOR_MAXV], qfrc_actuator[KSOR_MAXV], actuator_force[KSOR_MAXU],
      qfrc_smooth[KSOR_MAXV], qacc_smooth[KSOR_MAXV];
  /* constraints */
  int nefc, solver_niter;
  REAL con_dist[KSOR_MAXS], con_pos[KSOR_MAXS][3];
  REAL efc_J[KSOR_MAXR * KSOR_MAXV], efc_pos[KSOR_MAXR], efc_aref[KSOR_MAXR], efc_D[KSOR_MAXR],
      efc_force[KSOR_MAXR], efc_floss[KSOR_MAXR]; /* efc_floss > 0 marks a dry-friction row */
  REAL qfrc_constraint[KSOR_MAXV], qacc[KSOR_MAXV];
  /* contact forces on each body as a spatial force about the tree's centre of mass, world axes, torque then force
   * (MuJoCo's cfrc_ext, which FeetForceObservation / FeetTorqueObservation read, ksim/observation.py:563-616) */
  REAL cfrc_ext[KSOR_MAXB][6];
} FN(KsorData);
typedef FN(KsorData) Data;

int FN(ksor_sizeof_data)(void) { return (int)sizeof(Data); }

/* ------------------------------------------------------------------ small math */
static void cross3(REAL* r, const REAL* a, const REAL* b) {
  REAL x = a[1] * b[2] - a[2] * b[1], y = a[2] * b[0] - a[0] * b[2], z = a[0] * b[1] - a[1] * b[0];
  r[0] = x; r[1] = y; r[2] = z;
}
static REAL dot3(const REAL* a, const REAL* b) { return a[0] * b[0] + a[1] * b[1] + a[2] * b[2]; }
static void quat_mul(REAL* r, const REAL* a, const REAL* b) {
  REAL w = a[0] * b[0] - a[1] * b[1] - a[2] * b[2] - a[3] * b[3];
  REAL x = a[0] * b[1] + a[1] * b[0] + a[2] * b[3] - a[3] * b[2];
  REAL y = a[0] * b[2] - a[1] * b[3] + a[2] * b[0] + a[3] * b[1];
  REAL z = a[0] * b[3] + a[1] * b[2] - a[2] * b[1] + a[3] * b[0];
  r[0] = w; r[1] = x; r[2] = y; r[3] = z;
}
static void quat_norm(REAL* q) {
  REAL n = (REAL)sqrt(q[0] * q[0] + q[1] * q[1] + q[2] * q[2] + q[3] * q[3]);
  if (n < MINVAL) { q[0] = 1; q[1] = q[2] = q[3] = 0; return; }
  q[0] /= n; q[1] /= n; q[2] /= n; q[3] /= n;
}
static void quat2mat(REAL* m, const REAL* q) {
  REAL w = q[0], x = q[1], y = q[2], z = q[3];
  m[0] = w * w + x * x - y * y - z * z; m[1] = 2 * (x * y - w * z); m[2] = 2 * (x * z + w * y);
  m[3] = 2 * (x * y + w * z); m[4] = w * w - x * x + y * y - z * z; m[5] = 2 * (y * z - w * x);
  m[6] = 2 * (x * z - w * y); m[7] = 2 * (y * z + w * x); m[8] = w * w - x * x - y * y + z * z;
}
static void mat_vec(REAL* r, const REAL* m, const REAL* v) {
  REAL x = m[0] * v[0] + m[1] * v[1] + m[2] * v[2], y = m[3] * v[0] + m[4] * v[1] + m[5] * v[2],
       z = m[6] * v[0] + m[7] * v[1] + m[8] * v[2];
  r[0] = x; r[1] = y; r[2] = z;
}
static void rot_vec_quat(REAL* r, const REAL* v, const REAL* q) {
  REAL m[9];
  quat2mat(m, q);
  mat_vec(r, m, v);
}
static void axis_angle_quat(REAL* q, const REAL* axis, REAL angle) {
  REAL s = (REAL)sin(angle * (REAL)0.5);
  q[0] = (REAL)cos(angle * (REAL)0.5); q[1] = axis[0] * s; q[2] = axis[1] * s; q[3] = axis[2] * s;
}
/* spatial inertia (10: xx yy zz xy xz yz, m*c(3), m) times motion vector -> force vector */
static void inert_mul(REAL* r, const REAL* i, const REAL* v) {
  r[0] = i[0] * v[0] + i[3] * v[1] + i[4] * v[2] - i[8] * v[4] + i[7] * v[5];
  r[1] = i[3] * v[0] + i[1] * v[1] + i[5] * v[2] + i[8] * v[3] - i[6] * v[5];
  r[2] = i[4] * v[0] + i[5] * v[1] + i[2] * v[2] - i[7] * v[3] + i[6] * v[4];
  r[3] = i[8] * v[1] - i[7] * v[2] + i[9] * v[3];
  r[4] = i[6] * v[2] - i[8] * v[0] + i[9] * v[4];
  r[5] = i[7] * v[0] - i[6] * v[1] + i[9] * v[5];
}
static void cross_motion(REAL* r, const REAL* vel, const REAL* v) {
  REAL a[3], b[3], c[3];
  cross3(a, vel, v);          /* w x a */
  cross3(b, vel, v + 3);      /* w x b */
  cross3(c, vel + 3, v);      /* vl x a */
  r[0] = a[0]; r[1] = a[1]; r[2] = a[2];
  r[3] = b[0] + c[0]; r[4] = b[1] + c[1]; r[5] = b[2] + c[2];
}
static void cross_force(REAL* r, const REAL* vel, const REAL* f) {
  REAL a[3], b[3], c[3];
  cross3(a, vel, f);          /* w x tau */
  cross3(b, vel + 3, f + 3);  /* vl x F */
  cross3(c, vel, f + 3);      /* w x F */
  r[0] = a[0] + b[0]; r[1] = a[1] + b[1]; r[2] = a[2] + b[2];
  r[3] = c[0]; r[4] = c[1]; r[5] = c[2];
}

/* ------------------------------------------------------------------ kinematics */
void FN(ksor_kinematics)(const KsorModel* m, Data* d) {
  for (int k = 0; k < 3; ++k) { d->xpos[0][k] = 0; d->xipos[0][k] = 0; d->xanchor[0][k] = 0; d->xaxis[0][k] = 0; }
  d->xquat[0][0] = 1; d->xquat[0][1] = d->xquat[0][2] = d->xquat[0][3] = 0;
  quat2mat(d->xmat[0], d->xquat[0]);
  quat2mat(d->ximat[0], d->xquat[0]);
  for (int b = 1; b < m->nb; ++b) {
    const int p = m->body_parent[b];
    REAL pos[3], quat[4];
    REAL bpos[3] = {(REAL)m->body_pos[b][0], (REAL)m->body_pos[b][1], (REAL)m->body_pos[b][2]};
    REAL bquat[4] = {(REAL)m->body_quat[b][0], (REAL)m->body_quat[b][1], (REAL)m->body_quat[b][2], (REAL)m->body_quat[b][3]};
    REAL jpos[3] = {(REAL)m->jnt_pos[b][0], (REAL)m->jnt_pos[b][1], (REAL)m->jnt_pos[b][2]};
    REAL jaxis[3] = {(REAL)m->jnt_axis[b][0], (REAL)m->jnt_axis[b][1], (REAL)m->jnt_axis[b][2]};
    if (m->body_jtype[b] == KSOR_JNT_FREE) {
      const int qa = m->body_qadr[b];
      for (int k = 0; k < 3; ++k) pos[k] = d->qpos[qa + k];
      for (int k = 0; k < 4; ++k) quat[k] = d->qpos[qa + 3 + k];
      quat_norm(quat);
      for (int k = 0; k < 3; ++k) { d->xanchor[b][k] = pos[k]; d->xaxis[b][k] = (k == 2); }
    } else {
      mat_vec(pos, d->xmat[p], bpos);
      for (int k = 0; k < 3; ++k) pos[k] += d->xpos[p][k];
      quat_mul(quat, d->xquat[p], bquat);
      if (m->body_jtype[b] == KSOR_JNT_HINGE) {
        REAL anchor[3], qloc[4], v[3];
        rot_vec_quat(anchor, jpos, quat);
        for (int k = 0; k < 3; ++k) anchor[k] += pos[k];
        rot_vec_quat(d->xaxis[b], jaxis, quat);
        axis_angle_quat(qloc, jaxis, d->qpos[m->body_qadr[b]] - (REAL)m->qpos0[m->body_qadr[b]]);
        quat_mul(quat, quat, qloc);
        rot_vec_quat(v, jpos, quat);
        for (int k = 0; k < 3; ++k) { pos[k] = anchor[k] - v[k]; d->xanchor[b][k] = anchor[k]; }
      }
      quat_norm(quat);
    }
    for (int k = 0; k < 3; ++k) d->xpos[b][k] = pos[k];
    for (int k = 0; k < 4; ++k) d->xquat[b][k] = quat[k];
    quat2mat(d->xmat[b], quat);
    REAL ipos[3] = {(REAL)m->body_ipos[b][0], (REAL)m->body_ipos[b][1], (REAL)m->body_ipos[b][2]};
    if (d->has_ipos) for (int k = 0; k < 3; ++k) ipos[k] = d->body_ipos[b][k];
    REAL iquat[4] = {(REAL)m->body_iquat[b][0], (REAL)m->body_iquat[b][1], (REAL)m->body_iquat[b][2], (REAL)m->body_iquat[b][3]};
    REAL v[3], q2[4];
    mat_vec(v, d->xmat[b], ipos);
    for (int k = 0; k < 3; ++k) d->xipos[b][k] = pos[k] + v[k];
    quat_mul(q2, quat, iquat);
    quat_norm(q2);
    quat2mat(d->ximat[b], q2);
  }
}

/* centre of mass of the tree, com-based inertias and motion axes */
void FN(ksor_com_pos)(const KsorModel* m, Data* d) {
  REAL mt = 0, c[3] = {0, 0, 0};
  for (int b = 1; b < m->nb; ++b) {
    const REAL mass = (REAL)m->body_mass[b] * d->mass_scale[b];
    mt += mass;
    for (int k = 0; k < 3; ++k) c[k] += mass * d->xipos[b][k];
  }
  for (int k = 0; k < 3; ++k) d->com[k] = mt > MINVAL ? c[k] / mt : 0;
  memset(d->cinert[0], 0, sizeof(d->cinert[0]));
  for (int b = 1; b < m->nb; ++b) {
    const REAL mass = (REAL)m->body_mass[b] * d->mass_scale[b];
    const REAL* R = d->ximat[b];
    REAL I[3] = {(REAL)m->body_inertia[b][0], (REAL)m->body_inertia[b][1], (REAL)m->body_inertia[b][2]};
    if (d->has_inertia) for (int k = 0; k < 3; ++k) I[k] = d->body_inertia[b][k];
    REAL dif[3];
    for (int k = 0; k < 3; ++k) dif[k] = d->xipos[b][k] - d->com[k];
    REAL* ci = d->cinert[b];
    /* R diag(I) R^T */
    REAL xx = 0, yy = 0, zz = 0, xy = 0, xz = 0, yz = 0;
    for (int k = 0; k < 3; ++k) {
      xx += R[0 + k] * I[k] * R[0 + k]; yy += R[3 + k] * I[k] * R[3 + k]; zz += R[6 + k] * I[k] * R[6 + k];
      xy += R[0 + k] * I[k] * R[3 + k]; xz += R[0 + k] * I[k] * R[6 + k]; yz += R[3 + k] * I[k] * R[6 + k];
    }
    const REAL d2 = dot3(dif, dif);
    ci[0] = xx + mass * (d2 - dif[0] * dif[0]);
    ci[1] = yy + mass * (d2 - dif[1] * dif[1]);
    ci[2] = zz + mass * (d2 - dif[2] * dif[2]);
    ci[3] = xy - mass * dif[0] * dif[1];
    ci[4] = xz - mass * dif[0] * dif[2];
    ci[5] = yz - mass * dif[1] * dif[2];
    ci[6] = mass * dif[0]; ci[7] = mass * dif[1]; ci[8] = mass * dif[2];
    ci[9] = mass;
  }
  for (int b = 1; b < m->nb; ++b) {
    const int da = m->body_dofadr[b];
    REAL off[3];
    for (int k = 0; k < 3; ++k) off[k] = d->com[k] - d->xanchor[b][k];
    if (m->body_jtype[b] == KSOR_JNT_FREE) {
      for (int k = 0; k < 3; ++k) {
        REAL* t = d->cdof[da + k];
        t[0] = t[1] = t[2] = 0; t[3] = (k == 0); t[4] = (k == 1); t[5] = (k == 2);
        REAL* r = d->cdof[da + 3 + k];
        REAL axis[3] = {d->xmat[b][0 + k], d->xmat[b][3 + k], d->xmat[b][6 + k]};
        r[0] = axis[0]; r[1] = axis[1]; r[2] = axis[2];
        cross3(r + 3, axis, off);
      }
    } else if (m->body_jtype[b] == KSOR_JNT_HINGE) {
      REAL* r = d->cdof[da];
      for (int k = 0; k < 3; ++k) r[k] = d->xaxis[b][k];
      cross3(r + 3, d->xaxis[b], off);
    }
  }
}

/* composite rigid body inertias and the dense joint-space inertia matrix */
void FN(ksor_crb)(const KsorModel* m, Data* d) {
  const int nv = m->nv;
  for (int b = 0; b < m->nb; ++b) memcpy(d->crb[b], d->cinert[b], sizeof(d->crb[b]));
  for (int b = m->nb - 1; b > 0; --b) {
    const int p = m->body_parent[b];
    if (p > 0) for (int k = 0; k < 10; ++k) d->crb[p][k] += d->crb[b][k];
  }
  for (int i = 0; i < nv * nv; ++i) d->M[i] = 0;
  for (int i = 0; i < nv; ++i) {
    REAL buf[6];
    inert_mul(buf, d->crb[m->dof_body[i]], d->cdof[i]);
    for (int j = i; j >= 0; j = m->dof_parent[j]) {
      REAL s = 0;
      for (int k = 0; k < 6; ++k) s += d->cdof[j][k] * buf[k];
      d->M[i * nv + j] = s;
      d->M[j * nv + i] = s;
    }
    d->M[i * nv + i] += (REAL)m->dof_armature[i] * d->armature_scale[i];
  }
}

/* dense Cholesky A = L L^T (lower); returns 0 on success */
static int chol(REAL* L, const REAL* A, int n) {
  for (int j = 0; j < n; ++j) {
    REAL s = A[j * n + j];
    for (int k = 0; k < j; ++k) s -= L[j * n + k] * L[j * n + k];
    if (s <= 0) return -1;
    const REAL dj = (REAL)sqrt(s);
    L[j * n + j] = dj;
    for (int i = j + 1; i < n; ++i) {
      REAL t = A[i * n + j];
      for (int k = 0; k < j; ++k) t -= L[i * n + k] * L[j * n + k];
      L[i * n + j] = t / dj;
    }
    for (int i = 0; i < j; ++i) L[i * n + j] = 0;
  }
  return 0;
}
static void chol_solve(REAL* x, const REAL* L, const REAL* b, int n) {
  for (int i = 0; i < n; ++i) {
    REAL s = b[i];
    for (int k = 0; k < i; ++k) s -= L[i * n + k] * x[k];
    x[i] = s / L[i * n + i];
  }
  for (int i = n - 1; i >= 0; --i) {
    REAL s = x[i];
    for (int k = i + 1; k < n; ++k) s -= L[k * n + i] * x[k];
    x[i] = s / L[i * n + i];
  }
}

/* body velocities and the time derivatives of the motion axes */
void FN(ksor_com_vel)(const KsorModel* m, Data* d) {
  memset(d->cvel[0], 0, sizeof(d->cvel[0]));
  for (int b = 1; b < m->nb; ++b) {
    REAL v[6];
    memcpy(v, d->cvel[m->body_parent[b]], sizeof(v));
    const int da = m->body_dofadr[b];
    if (m->body_jtype[b] == KSOR_JNT_FREE) {
      for (int k = 0; k < 3; ++k) {
        memset(d->cdof_dot[da + k], 0, sizeof(d->cdof_dot[0]));
        for (int c = 0; c < 6; ++c) v[c] += d->cdof[da + k][c] * d->qvel[da + k];
      }
      for (int k = 3; k < 6; ++k) cross_motion(d->cdof_dot[da + k], v, d->cdof[da + k]);
      for (int k = 3; k < 6; ++k)
        for (int c = 0; c < 6; ++c) v[c] += d->cdof[da + k][c] * d->qvel[da + k];
    } else if (m->body_jtype[b] == KSOR_JNT_HINGE) {
      cross_motion(d->cdof_dot[da], v, d->cdof[da]);
      for (int c = 0; c < 6; ++c) v[c] += d->cdof[da][c] * d->qvel[da];
    }
    memcpy(d->cvel[b], v, sizeof(v));
  }
}

/* recursive Newton-Euler with zero joint acceleration: Coriolis, centrifugal and gravity forces */
void FN(ksor_rne)(const KsorModel* m, Data* d) {
  REAL cacc[KSOR_MAXB][6], cfrc[KSOR_MAXB][6];
  memset(cacc, 0, sizeof(cacc));
  memset(cfrc, 0, sizeof(cfrc));
  for (int k = 0; k < 3; ++k) cacc[0][3 + k] = -(REAL)m->gravity[k];
  for (int b = 1; b < m->nb; ++b) {
    memcpy(cacc[b], cacc[m->body_parent[b]], sizeof(cacc[b]));
    const int da = m->body_dofadr[b];
    const int nd = m->body_jtype[b] == KSOR_JNT_FREE ? 6 : (m->body_jtype[b] == KSOR_JNT_HINGE ? 1 : 0);
    for (int k = 0; k < nd; ++k)
      for (int c = 0; c < 6; ++c) cacc[b][c] += d->cdof_dot[da + k][c] * d->qvel[da + k];
    REAL iv[6], ia[6], cf[6];
    inert_mul(ia, d->cinert[b], cacc[b]);
    inert_mul(iv, d->cinert[b], d->cvel[b]);
    cross_force(cf, d->cvel[b], iv);
    for (int c = 0; c < 6; ++c) cfrc[b][c] = ia[c] + cf[c];
  }
  for (int b = m->nb - 1; b > 0; --b) {
    const int p = m->body_parent[b];
    if (p > 0) for (int c = 0; c < 6; ++c) cfrc[p][c] += cfrc[b][c];
  }
  for (int i = 0; i < m->nv; ++i) {
    REAL s = 0;
    for (int c = 0; c < 6; ++c) s += d->cdof[i][c] * cfrc[m->dof_body[i]][c];
    d->qfrc_bias[i] = s;
  }
}

/* ------------------------------------------------------------------ constraints */
/* translational Jacobian (3 x nv) of a world point attached to body b */
static void jac_point(const KsorModel* m, const Data* d, REAL* jacp, const REAL* point, int b) {
  const int nv = m->nv;
  for (int i = 0; i < 3 * nv; ++i) jacp[i] = 0;
  REAL off[3];
  for (int k = 0; k < 3; ++k) off[k] = point[k] - d->com[k];
  /* last dof of the body, then up the chain */
  int j = -1;
  for (int bb = b; bb > 0 && j < 0; bb = m->body_parent[bb]) {
    if (m->body_jtype[bb] == KSOR_JNT_FREE) j = m->body_dofadr[bb] + 5;
    else if (m->body_jtype[bb] == KSOR_JNT_HINGE) j = m->body_dofadr[bb];
  }
  for (; j >= 0; j = m->dof_parent[j]) {
    REAL c[3];
    cross3(c, d->cdof[j], off);
    for (int k = 0; k < 3; ++k) jacp[k * nv + j] = d->cdof[j][3 + k] + c[k];
  }
}

/* constraint impedance d(|pos|) of MuJoCo's solimp = (dmin, dmax, width, midpoint, power) */
static REAL impedance(REAL pos, REAL dmin, REAL dmax, REAL width, REAL mid, REAL power) {
  const REAL ix = (REAL)fabs(pos) / width;
  const REAL ia = (1 / (REAL)pow(mid, power - 1)) * (REAL)pow(ix, power);
  const REAL ib = 1 - (1 / (REAL)pow(1 - mid, power - 1)) * (REAL)pow(1 - ix, power);
  const REAL iy = ix < mid ? ia : ib;
  REAL imp = dmin + iy * (dmax - dmin);
  imp = imp < dmin ? dmin : (imp > dmax ? dmax : imp);
  if (ix > 1) imp = dmax;
  return imp;
}

static void sol_params(const double* solref, const double* solimp, double dt, REAL* kk, REAL* bb, REAL* dmin, REAL* dmax,
                       REAL* width, REAL* mid, REAL* power) {
  REAL timeconst = (REAL)solref[0], dampratio = (REAL)solref[1];
  *dmin = (REAL)solimp[0]; *dmax = (REAL)solimp[1]; *width = (REAL)solimp[2]; *mid = (REAL)solimp[3]; *power = (REAL)solimp[4];
  if (timeconst < 2 * (REAL)dt) timeconst = 2 * (REAL)dt;
  *dmin = *dmin < MINIMP ? MINIMP : (*dmin > MAXIMP ? MAXIMP : *dmin);
  *dmax = *dmax < MINIMP ? MINIMP : (*dmax > MAXIMP ? MAXIMP : *dmax);
  *width = *width < MINVAL ? MINVAL : *width;
  *mid = *mid < MINIMP ? MINIMP : (*mid > MAXIMP ? MAXIMP : *mid);
  *power = *power < 1 ? 1 : *power;
  *kk = 1 / (*dmax * *dmax * timeconst * timeconst * dampratio * dampratio);
  *bb = 2 / (*dmax * timeconst);
  if (solref[0] <= 0) *kk = -(REAL)solref[0] / (*dmax * *dmax);
  if (solref[1] <= 0) *bb = -(REAL)solref[1] / *dmax;
}

/* Rows in the order contacts, joint limits, dry friction (MuJoCo orders them friction, limits, contacts; the order
 * only changes the order of summation). */
void FN(ksor_make_constraint)(const KsorModel* m, Data* d) {
  const int nv = m->nv;
  int nefc = 0;
  const REAL mu = d->friction;
  /* solref / solimp -> stiffness k, damping b (refsafe) and clamped impedance parameters: one set for the contact rows,
   * one for the rows of joint limits and dry friction (dof_solref / dof_solimp; all zero = the contact set) */
  REAL kk, bb, dmin, dmax, width, mid, power;
  sol_params(m->solref, m->solimp, m->dt, &kk, &bb, &dmin, &dmax, &width, &mid, &power);
  int own = 0;
  for (int k = 0; k < 2; ++k) own |= m->dof_solref[k] != 0;
  for (int k = 0; k < 5; ++k) own |= m->dof_solimp[k] != 0;
  REAL jk = kk, jb = bb, jdmin = dmin, jdmax = dmax, jwidth = width, jmid = mid, jpower = power;
  if (own) sol_params(m->dof_solref, m->dof_solimp, m->dt, &jk, &jb, &jdmin, &jdmax, &jwidth, &jmid, &jpower);

  for (int s = 0; s < m->ns; ++s) {
    const int b = m->sph_body[s];
    REAL lp[3] = {(REAL)m->sph_pos[s][0], (REAL)m->sph_pos[s][1], (REAL)m->sph_pos[s][2]}, c[3];
    if (d->has_spheres) for (int k = 0; k < 3; ++k) lp[k] = d->sph_pos[s][k];
    mat_vec(c, d->xmat[b], lp);
    for (int k = 0; k < 3; ++k) c[k] += d->xpos[b][k];
    const REAL r = d->has_spheres ? d->sph_radius[s] : (REAL)m->sph_radius[s];
    const REAL dist = c[2] - r;
    d->con_dist[s] = dist;
    d->con_pos[s][0] = c[0]; d->con_pos[s][1] = c[1]; d->con_pos[s][2] = c[2] - r - dist * (REAL)0.5;
    if (!(dist < 0)) continue; /* inactive contacts contribute nothing */
    REAL jacp[3 * KSOR_MAXV];
    jac_point(m, d, jacp, d->con_pos[s], b);
    /* contact frame: normal z, tangents (0,1,0) and (-1,0,0) */
    const REAL* Jn = jacp + 2 * nv;
    const REAL* Jy = jacp + 1 * nv;
    const REAL* Jx = jacp;
    const REAL t = (REAL)m->body_invweight0[b];
    const REAL pos = dist;
    const REAL imp = impedance(pos, dmin, dmax, width, mid, power);
    if (m->condim == 1) {
      /* frictionless contact (MJX _instantiate_contact_frictionless): the normal row alone, regularised with the
       * body's translational inverse weight */
      REAL R = t * (1 - imp) / imp;
      if (R < MINVAL) R = MINVAL;
      REAL* row = d->efc_J + nefc * nv;
      REAL vel = 0;
      for (int j = 0; j < nv; ++j) { row[j] = Jn[j]; vel += row[j] * d->qvel[j]; }
      d->efc_pos[nefc] = pos;
      d->efc_aref[nefc] = -bb * vel - kk * imp * pos;
      d->efc_D[nefc] = 1 / R;
      d->efc_floss[nefc] = 0;
      nefc += 1;
      continue;
    }
    const REAL invweight = (t + mu * mu * t) * 2 * mu * mu / (REAL)m->impratio;
    REAL R = invweight * (1 - imp) / imp;
    if (R < MINVAL) R = MINVAL;
    for (int q = 0; q < 4; ++q) {
      REAL* row = d->efc_J + (nefc + q) * nv;
      for (int j = 0; j < nv; ++j) {
        const REAL tang = (q < 2) ? Jy[j] : -Jx[j];
        row[j] = Jn[j] + ((q & 1) ? -mu : mu) * tang;
      }
      REAL vel = 0;
      for (int j = 0; j < nv; ++j) vel += row[j] * d->qvel[j];
      d->efc_pos[nefc + q] = pos;
      d->efc_aref[nefc + q] = -bb * vel - kk * imp * pos;
      d->efc_D[nefc + q] = 1 / R;
      d->efc_floss[nefc + q] = 0;
    }
    nefc += 4;
  }
  /* joint limits of hinges: one row for the nearer side once it is violated (margin 0), J = +1 on the lower side and
   * -1 on the upper side, regularised with the dof's inverse weight */
  for (int b = 1; b < m->nb; ++b) {
    if (m->body_jtype[b] != KSOR_JNT_HINGE || !m->jnt_limited[b]) continue;
    const int j = m->body_dofadr[b];
    const REAL q = d->qpos[m->body_qadr[b]];
    const REAL dlo = q - (REAL)m->jnt_range[b][0], dhi = (REAL)m->jnt_range[b][1] - q;
    const REAL pos = dlo < dhi ? dlo : dhi;
    if (!(pos < 0)) continue;
    const REAL side = dlo < dhi ? 1 : -1;
    REAL* row = d->efc_J + nefc * nv;
    for (int i = 0; i < nv; ++i) row[i] = 0;
    row[j] = side;
    const REAL imp = impedance(pos, jdmin, jdmax, jwidth, jmid, jpower);
    REAL R = (REAL)m->dof_invweight0[j] * (1 - imp) / imp;
    if (R < MINVAL) R = MINVAL;
    d->efc_pos[nefc] = pos;
    d->efc_aref[nefc] = -jb * side * d->qvel[j] - jk * imp * pos;
    d->efc_D[nefc] = 1 / R;
    d->efc_floss[nefc] = 0;
    ++nefc;
  }
  /* dry joint friction: a row J = e_j at pos = 0 whose force saturates at +-frictionloss */
  for (int j = 0; j < nv; ++j) {
    const REAL fl = d->has_frictionloss ? d->dof_frictionloss[j] : (REAL)m->dof_frictionloss[j];
    if (!(fl > 0)) continue;
    REAL* row = d->efc_J + nefc * nv;
    for (int i = 0; i < nv; ++i) row[i] = 0;
    row[j] = 1;
    const REAL imp = impedance(0, jdmin, jdmax, jwidth, jmid, jpower);
    REAL R = (REAL)m->dof_invweight0[j] * (1 - imp) / imp;
    if (R < MINVAL) R = MINVAL;
    d->efc_pos[nefc] = 0;
    d->efc_aref[nefc] = -jb * d->qvel[j];
    d->efc_D[nefc] = 1 / R;
    d->efc_floss[nefc] = fl;
    ++nefc;
  }
  d->nefc = nefc;
}

/* ------------------------------------------------------------------ Newton solver */
typedef struct {
  REAL qacc[KSOR_MAXV], Ma[KSOR_MAXV], Jaref[KSOR_MAXR], grad[KSOR_MAXV], Mgrad[KSOR_MAXV], search[KSOR_MAXV];
  REAL efc_force[KSOR_MAXR], qfrc_constraint[KSOR_MAXV];
  int active[KSOR_MAXR];
  REAL gauss, cost, prev_cost;
} Ctx;

static void mul_M(const KsorModel* m, const Data* d, REAL* r, const REAL* v) {
  const int nv = m->nv;
  for (int i = 0; i < nv; ++i) {
    REAL s = 0;
    for (int j = 0; j < nv; ++j) s += d->M[i * nv + j] * v[j];
    r[i] = s;
  }
}

static void update_constraint(const KsorModel* m, const Data* d, Ctx* c) {
  const int nv = m->nv, ne = d->nefc;
  REAL cost = 0;
  for (int i = 0; i < nv; ++i) c->qfrc_constraint[i] = 0;
  for (int r = 0; r < ne; ++r) {
    const REAL fl = d->efc_floss[r], x = c->Jaref[r];
    if (fl > 0) {
      /* dry friction: quadratic inside |x| < R f, linear (constant force -+f) outside */
      const REAL rf = fl / d->efc_D[r];
      if (x <= -rf) { c->active[r] = 0; c->efc_force[r] = fl; cost += fl * (-(REAL)0.5 * rf - x); }
      else if (x >= rf) { c->active[r] = 0; c->efc_force[r] = -fl; cost += fl * (-(REAL)0.5 * rf + x); }
      else { c->active[r] = 1; c->efc_force[r] = -d->efc_D[r] * x; cost += (REAL)0.5 * d->efc_D[r] * x * x; }
    } else {
      c->active[r] = x < 0;
      c->efc_force[r] = c->active[r] ? -d->efc_D[r] * x : 0;
      if (c->active[r]) cost += (REAL)0.5 * d->efc_D[r] * x * x;
    }
    for (int j = 0; j < nv; ++j) c->qfrc_constraint[j] += d->efc_J[r * nv + j] * c->efc_force[r];
  }
  REAL g = 0;
  for (int i = 0; i < nv; ++i) g += (c->Ma[i] - d->qfrc_smooth[i]) * (c->qacc[i] - d->qacc_smooth[i]);
  c->gauss = (REAL)0.5 * g;
  c->prev_cost = c->cost;
  c->cost = cost + c->gauss;
}

static void update_gradient(const KsorModel* m, const Data* d, Ctx* c) {
  const int nv = m->nv, ne = d->nefc;
  REAL H[KSOR_MAXV * KSOR_MAXV], Lh[KSOR_MAXV * KSOR_MAXV];
  for (int i = 0; i < nv; ++i) c->grad[i] = c->Ma[i] - d->qfrc_smooth[i] - c->qfrc_constraint[i];
  for (int i = 0; i < nv * nv; ++i) H[i] = d->M[i];
  for (int r = 0; r < ne; ++r) {
    if (!c->active[r]) continue;
    const REAL* J = d->efc_J + r * nv;
    for (int i = 0; i < nv; ++i) {
      const REAL s = J[i] * d->efc_D[r];
      if (s == 0) continue;
      for (int j = 0; j < nv; ++j) H[i * nv + j] += s * J[j];
    }
  }
  chol(Lh, H, nv);
  chol_solve(c->Mgrad, Lh, c->grad, nv);
}

static void ctx_create(const KsorModel* m, const Data* d, Ctx* c, const REAL* qacc, int grad) {
  const int nv = m->nv, ne = d->nefc;
  for (int i = 0; i < nv; ++i) c->qacc[i] = qacc[i];
  mul_M(m, d, c->Ma, qacc);
  for (int r = 0; r < ne; ++r) {
    REAL s = 0;
    for (int j = 0; j < nv; ++j) s += d->efc_J[r * nv + j] * qacc[j];
    c->Jaref[r] = s - d->efc_aref[r];
  }
  c->cost = (REAL)INFINITY;
  c->prev_cost = 0;
  for (int i = 0; i < nv; ++i) c->search[i] = c->grad[i] = c->Mgrad[i] = 0;
  update_constraint(m, d, c);
  if (grad) {
    update_gradient(m, d, c);
    for (int i = 0; i < nv; ++i) c->search[i] = -c->Mgrad[i];
  }
}

typedef struct { REAL alpha, cost, deriv0, deriv1; } LSPoint;

static LSPoint ls_point(const Data* d, const Ctx* c, REAL alpha, const REAL* jv, const REAL (*quad)[3],
                        const REAL* quad_gauss) {
  REAL q0 = quad_gauss[0], q1 = quad_gauss[1], q2 = quad_gauss[2];
  for (int r = 0; r < d->nefc; ++r) {
    const REAL x = c->Jaref[r] + alpha * jv[r];
    const REAL fl = d->efc_floss[r];
    if (fl > 0) {
      const REAL rf = fl / d->efc_D[r];
      if (x <= -rf) { q0 += fl * (-(REAL)0.5 * rf - c->Jaref[r]); q1 += -fl * jv[r]; }
      else if (x >= rf) { q0 += fl * (-(REAL)0.5 * rf + c->Jaref[r]); q1 += fl * jv[r]; }
      else { q0 += quad[r][0]; q1 += quad[r][1]; q2 += quad[r][2]; }
    } else if (x < 0) { q0 += quad[r][0]; q1 += quad[r][1]; q2 += quad[r][2]; }
  }
  LSPoint p;
  p.alpha = alpha;
  p.cost = alpha * alpha * q2 + alpha * q1 + q0;
  p.deriv0 = 2 * alpha * q2 + q1;
  p.deriv1 = 2 * q2 + (q2 == 0 ? MINVAL : 0);
  return p;
}
static int in_bracket(const LSPoint* x, const LSPoint* y) {
  return ((x->deriv0 < y->deriv0) && (y->deriv0 < 0)) || ((x->deriv0 > y->deriv0) && (y->deriv0 > 0));
}

static void linesearch(const KsorModel* m, const Data* d, Ctx* c) {
  const int nv = m->nv, ne = d->nefc;
  REAL mv[KSOR_MAXV], jv[KSOR_MAXR], quad[KSOR_MAXR][3], quad_gauss[3];
  REAL sn = 0;
  for (int i = 0; i < nv; ++i) sn += c->search[i] * c->search[i];
  const REAL smag = (REAL)sqrt(sn) * (REAL)m->meaninertia * (REAL)(nv > 1 ? nv : 1);
  const REAL gtol = (REAL)m->tolerance * (REAL)m->ls_tolerance * smag;
  mul_M(m, d, mv, c->search);
  for (int r = 0; r < ne; ++r) {
    REAL s = 0;
    for (int j = 0; j < nv; ++j) s += d->efc_J[r * nv + j] * c->search[j];
    jv[r] = s;
    quad[r][0] = (REAL)0.5 * c->Jaref[r] * c->Jaref[r] * d->efc_D[r];
    quad[r][1] = jv[r] * c->Jaref[r] * d->efc_D[r];
    quad[r][2] = (REAL)0.5 * jv[r] * jv[r] * d->efc_D[r];
  }
  REAL sMa = 0, sq = 0, smv = 0;
  for (int i = 0; i < nv; ++i) {
    sMa += c->search[i] * c->Ma[i];
    sq += c->search[i] * d->qfrc_smooth[i];
    smv += c->search[i] * mv[i];
  }
  quad_gauss[0] = c->gauss; quad_gauss[1] = sMa - sq; quad_gauss[2] = (REAL)0.5 * smv;

  const LSPoint p0 = ls_point(d, c, 0, jv, quad, quad_gauss);
  LSPoint lo = ls_point(d, c, p0.alpha - p0.deriv0 / p0.deriv1, jv, quad, quad_gauss);
  LSPoint hi;
  if (lo.deriv0 < p0.deriv0) { hi = p0; } else { hi = lo; lo = p0; }
  int swap = 1, it = 0;
  while (1) {
    int done = it >= m->ls_iterations;
    done |= !swap;
    done |= (lo.deriv0 < 0) && (lo.deriv0 > -gtol);
    done |= (hi.deriv0 > 0) && (hi.deriv0 < gtol);
    if (done) break;
    const LSPoint lo_next = ls_point(d, c, lo.alpha - lo.deriv0 / lo.deriv1, jv, quad, quad_gauss);
    const LSPoint hi_next = ls_point(d, c, hi.alpha - hi.deriv0 / hi.deriv1, jv, quad, quad_gauss);
    const LSPoint mid = ls_point(d, c, (REAL)0.5 * (lo.alpha + hi.alpha), jv, quad, quad_gauss);
    int s1, s2, s3, t1, t2, t3;
    LSPoint nlo = lo, nhi = hi;
    s1 = in_bracket(&nlo, &lo_next); if (s1) nlo = lo_next;
    s2 = in_bracket(&nlo, &mid);     if (s2) nlo = mid;
    s3 = in_bracket(&nlo, &hi_next); if (s3) nlo = hi_next;
    t1 = in_bracket(&nhi, &hi_next); if (t1) nhi = hi_next;
    t2 = in_bracket(&nhi, &mid);     if (t2) nhi = mid;
    t3 = in_bracket(&nhi, &lo_next); if (t3) nhi = lo_next;
    lo = nlo; hi = nhi;
    swap = s1 | s2 | s3 | t1 | t2 | t3;
    ++it;
  }
  const int improved = (lo.cost < p0.cost) || (hi.cost < p0.cost);
  REAL alpha = lo.cost < hi.cost ? lo.alpha : hi.alpha;
  if (!improved) alpha = 0;
  for (int i = 0; i < nv; ++i) { c->qacc[i] += alpha * c->search[i]; c->Ma[i] += alpha * mv[i]; }
  for (int r = 0; r < ne; ++r) c->Jaref[r] += alpha * jv[r];
}

void FN(ksor_solve)(const KsorModel* m, Data* d) {
  const int nv = m->nv;
  Ctx cw, cs, c;
  const REAL scale = 1 / ((REAL)m->meaninertia * (REAL)(nv > 1 ? nv : 1));
  const REAL* start = d->qacc_smooth;
  if (d->nefc == 0) {
    /* unconstrained: the minimiser is qacc_smooth */
    for (int i = 0; i < nv; ++i) { d->qacc[i] = d->qacc_smooth[i]; d->qfrc_constraint[i] = 0; d->qacc_warmstart[i] = d->qacc[i]; }
    d->solver_niter = 0;
    return;
  }
  ctx_create(m, d, &cw, d->qacc_warmstart, 0);
  ctx_create(m, d, &cs, d->qacc_smooth, 0);
  if (cw.cost < cs.cost) start = d->qacc_warmstart;
  ctx_create(m, d, &c, start, 1);
  int niter = 0;
  while (1) {
    REAL gn = 0;
    for (int i = 0; i < nv; ++i) gn += c.grad[i] * c.grad[i];
    const REAL improvement = scale * (c.prev_cost - c.cost);
    const REAL gradient = scale * (REAL)sqrt(gn);
    int done = niter >= m->iterations;
    done |= improvement < (REAL)m->tolerance;
    done |= gradient < (REAL)m->tolerance;
    if (done && !(m->iterations == 1 && niter == 0)) break;
    linesearch(m, d, &c);
    update_constraint(m, d, &c);
    update_gradient(m, d, &c);
    for (int i = 0; i < nv; ++i) c.search[i] = -c.Mgrad[i];
    ++niter;
  }
  d->solver_niter = niter;
  for (int i = 0; i < nv; ++i) {
    d->qacc[i] = c.qacc[i];
    d->qacc_warmstart[i] = c.qacc[i];
    d->qfrc_constraint[i] = c.qfrc_constraint[i];
  }
  for (int r = 0; r < d->nefc; ++r) d->efc_force[r] = c.efc_force[r];
}

/* ------------------------------------------------------------------ forward + integrate */
void FN(ksor_forward)(const KsorModel* m, Data* d) {
  const int nv = m->nv;
  FN(ksor_kinematics)(m, d);
  FN(ksor_com_pos)(m, d);
  FN(ksor_crb)(m, d);
  chol(d->L, d->M, nv);
  FN(ksor_make_constraint)(m, d); /* uses qvel for aref, like make_constraint after fwd_position in MJX */
  FN(ksor_com_vel)(m, d);
  FN(ksor_rne)(m, d);
  for (int i = 0; i < nv; ++i) { d->qfrc_passive[i] = -(REAL)m->dof_damping[i] * d->damping_scale[i] * d->qvel[i]; d->qfrc_actuator[i] = 0; }
  for (int b = 1; b < m->nb; ++b) { /* joint springs (hinges): the spring's rest position is the joint's qpos0 */
    if (m->body_jtype[b] != KSOR_JNT_HINGE) continue;
    const int j = m->body_dofadr[b], qa = m->body_qadr[b];
    d->qfrc_passive[j] -= (REAL)m->dof_stiffness[j] * (d->qpos[qa] - (REAL)m->qpos0[qa]);
  }
  for (int u = 0; u < m->nu; ++u) {
    REAL c = d->ctrl[u];
    if (c < (REAL)m->act_lo[u]) c = (REAL)m->act_lo[u];
    if (c > (REAL)m->act_hi[u]) c = (REAL)m->act_hi[u];
    d->actuator_force[u] = (REAL)m->act_gear[u] * c;
    d->qfrc_actuator[m->act_dof[u]] += d->actuator_force[u];
  }
  for (int i = 0; i < nv; ++i) d->qfrc_smooth[i] = d->qfrc_passive[i] - d->qfrc_bias[i] + d->qfrc_actuator[i];
  /* applied Cartesian forces: qfrc += Jp(xipos)^T f + Jr^T t over the dofs of the body's ancestor chain */
  for (int b = 1; b < m->nb; ++b) {
    const REAL* w = d->xfrc_applied[b];
    int any = 0;
    for (int k = 0; k < 6; ++k) any |= w[k] != 0;
    if (!any) continue;
    REAL jacp[3 * KSOR_MAXV];
    jac_point(m, d, jacp, d->xipos[b], b);
    int j = -1;
    for (int bb = b; bb > 0 && j < 0; bb = m->body_parent[bb]) {
      if (m->body_jtype[bb] == KSOR_JNT_FREE) j = m->body_dofadr[bb] + 5;
      else if (m->body_jtype[bb] == KSOR_JNT_HINGE) j = m->body_dofadr[bb];
    }
    for (; j >= 0; j = m->dof_parent[j]) {
      REAL q = 0;
      for (int k = 0; k < 3; ++k) q += jacp[k * nv + j] * w[k] + d->cdof[j][k] * w[3 + k];
      d->qfrc_smooth[j] += q;
    }
  }
  chol_solve(d->qacc_smooth, d->L, d->qfrc_smooth, nv);
  FN(ksor_solve)(m, d);
  /* Cartesian contact forces: a pyramid row with force f pushes along normal +- mu tangent, so a contact's force is
   * the sum of its four edge forces; it acts on the sphere's body at the contact point */
  memset(d->cfrc_ext, 0, sizeof(d->cfrc_ext));
  int row = 0;
  for (int s = 0; s < m->ns; ++s) {
    if (!(d->con_dist[s] < 0)) continue;
    REAL F[3] = {0, 0, 0};
    if (m->condim == 1) {
      F[2] = d->efc_force[row];
      row += 1;
    } else {
      for (int q = 0; q < 4; ++q) {
        const REAL f = d->efc_force[row + q], smu = (q & 1) ? -d->friction : d->friction;
        F[2] += f;
        if (q < 2) F[1] += smu * f; else F[0] -= smu * f;
      }
      row += 4;
    }
    REAL off[3], tq[3];
    for (int k = 0; k < 3; ++k) off[k] = d->con_pos[s][k] - d->com[k];
    cross3(tq, off, F);
    const int b = m->sph_body[s];
    for (int k = 0; k < 3; ++k) { d->cfrc_ext[b][k] += tq[k]; d->cfrc_ext[b][3 + k] += F[k]; }
  }
}

void FN(ksor_euler)(const KsorModel* m, Data* d) {
  const int nv = m->nv;
  const REAL dt = (REAL)m->dt;
  REAL qacc[KSOR_MAXV];
  for (int i = 0; i < nv; ++i) qacc[i] = d->qacc[i];
  if (m->eulerdamp) {
    /* implicit in joint damping: (M + dt diag(damping)) qacc' = qfrc_smooth + qfrc_constraint */
    REAL H[KSOR_MAXV * KSOR_MAXV], Lh[KSOR_MAXV * KSOR_MAXV], rhs[KSOR_MAXV];
    for (int i = 0; i < nv * nv; ++i) H[i] = d->M[i];
    for (int i = 0; i < nv; ++i) H[i * nv + i] += dt * (REAL)m->dof_damping[i] * d->damping_scale[i];
    for (int i = 0; i < nv; ++i) rhs[i] = d->qfrc_smooth[i] + d->qfrc_constraint[i];
    chol(Lh, H, nv);
    chol_solve(qacc, Lh, rhs, nv);
  }
  for (int i = 0; i < nv; ++i) d->qvel[i] += dt * qacc[i];
  for (int b = 1; b < m->nb; ++b) {
    const int qa = m->body_qadr[b], da = m->body_dofadr[b];
    if (m->body_jtype[b] == KSOR_JNT_FREE) {
      for (int k = 0; k < 3; ++k) d->qpos[qa + k] += dt * d->qvel[da + k];
      /* quaternion integration with the body-frame angular velocity */
      REAL w[3] = {d->qvel[da + 3], d->qvel[da + 4], d->qvel[da + 5]};
      REAL n = (REAL)sqrt(dot3(w, w));
      REAL q[4] = {d->qpos[qa + 3], d->qpos[qa + 4], d->qpos[qa + 5], d->qpos[qa + 6]};
      if (n > MINVAL) {
        REAL axis[3] = {w[0] / n, w[1] / n, w[2] / n}, dq[4], r[4];
        axis_angle_quat(dq, axis, n * dt);
        quat_mul(r, q, dq);
        for (int k = 0; k < 4; ++k) q[k] = r[k];
      }
      quat_norm(q);
      for (int k = 0; k < 4; ++k) d->qpos[qa + 3 + k] = q[k];
    } else if (m->body_jtype[b] == KSOR_JNT_HINGE) {
      d->qpos[qa] += dt * d->qvel[da];
    }
  }
  d->time += dt;
}

void FN(ksor_step)(const KsorModel* m, Data* d) {
  FN(ksor_forward)(m, d);
  FN(ksor_euler)(m, d);
}

/* ------------------------------------------------------------------ batched control step (CPU baseline + tests)
 * One control step of N envs = S physics substeps with the engine's latency blend and
 * PD actuator (ksim/engine.py:287-320, ksim/actuators.py:198-217 without noise).
 * Arrays are env-major (N, dim).  nroot_q/nroot_v: 7/6 with a free root, else 0/0.
 */
void FN(ksor_ctrl_step_batch)(const KsorModel* m, int N, int S, int actuator_period, Data* data /*N*/,
                              const REAL* action /*N,nu*/, REAL* last_ctrl /*N,nu*/, const REAL* latency /*N*/,
                              const REAL* zero_offset /*N,nu or NULL*/, const REAL* kp /*N,nu*/,
                              const REAL* kd /*N,nu*/, const REAL* ctrl_clip /*nu*/, int nthreads,
                              const REAL* qvel_impulse /*S,N,nv or NULL: events, ksim/engine.py:322-333*/) {
  const int nu = m->nu;
  const int rq = (m->nb > 1 && m->body_jtype[1] == KSOR_JNT_FREE) ? 7 : 0;
  const int rv = rq ? 6 : 0;
#pragma omp parallel for num_threads(nthreads) schedule(static)
  for (int e = 0; e < N; ++e) {
    Data* d = data + e;
    REAL torque[KSOR_MAXU];
    for (int u = 0; u < nu; ++u) torque[u] = 0;
    for (int s = 0; s < S; ++s) {
      REAL prct = (REAL)s - latency[e];
      prct = prct < 0 ? 0 : (prct > 1 ? 1 : prct);
      if (s % actuator_period == 0) {
        for (int u = 0; u < nu; ++u) {
          const REAL target = last_ctrl[e * nu + u] * (1 - prct) + action[e * nu + u] * prct;
          const REAL q = d->qpos[rq + u] - (zero_offset ? zero_offset[e * nu + u] : 0);
          REAL t = kp[e * nu + u] * (target - q) + kd[e * nu + u] * (0 - d->qvel[rv + u]);
          const REAL lim = ctrl_clip[u];
          t = t < -lim ? -lim : (t > lim ? lim : t);
          torque[u] = t;
        }
      }
      for (int u = 0; u < nu; ++u) d->ctrl[u] = torque[u];
      if (qvel_impulse)
        for (int j = 0; j < m->nv; ++j) d->qvel[j] += qvel_impulse[((size_t)s * N + e) * m->nv + j];
      FN(ksor_step)(m, d);
    }
    for (int u = 0; u < nu; ++u) last_ctrl[e * nu + u] = action[e * nu + u];
  }
}
