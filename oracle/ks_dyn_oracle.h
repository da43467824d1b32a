/* CPU oracle of the per-env dynamics step — TEST INFRASTRUCTURE, not shipped code.
 *
 * Restates, in plain scalar C, what `mjx.step` computes at ksim/engine.py:257 for the
 * model subset the rollout configs use (kinematic tree of free/hinge joints, motor
 * actuators, sphere-plane contacts with pyramidal cones, joint limits, dry joint friction,
 * Newton solver, Euler).
 * MJX itself is third-party and not vendored in the reference (ksim/requirements.txt:20-21,
 * unpinned); the algorithm follows the public MuJoCo "Computation" documentation.
 * Parity with MJX of the Newton iterates, impedance details and pyramidal regulariser
 * scaling is UNPINNED; the mathematics (kinematics, mass matrix, bias forces, contact
 * geometry, solver fixed point, integrator) is pinned by tests/test_oracle_dyn.py.
 *
 * Compiled twice (REAL = double / float); symbols carry the suffix _f64 / _f32.
 */
#ifndef KS_DYN_ORACLE_H_
#define KS_DYN_ORACLE_H_

#define KSOR_MAXB 32  /* bodies incl. world */
#define KSOR_MAXQ 40
#define KSOR_MAXV 32
#define KSOR_MAXU 32
#define KSOR_MAXS 16  /* contact spheres */
#define KSOR_MAXR 128 /* constraint rows: 4 per sphere, one per limited joint at its limit, one per dof with dry friction */

enum { KSOR_JNT_NONE = 0, KSOR_JNT_FREE = 1, KSOR_JNT_HINGE = 2 };

/* Model: always double; shared by both precisions. */
typedef struct KsorModel {
  int nb, nq, nv, nu, ns;
  int iterations, ls_iterations, eulerdamp;
  int condim; /* 3 (or 0): pyramidal friction, four rows per contact; 1: frictionless, one normal row */
  double dt, gravity[3], tolerance, ls_tolerance, impratio, meaninertia;
  double solref[2], solimp[5];
  int body_parent[KSOR_MAXB], body_jtype[KSOR_MAXB], body_qadr[KSOR_MAXB], body_dofadr[KSOR_MAXB];
  int body_subtree_end[KSOR_MAXB];
  double body_pos[KSOR_MAXB][3], body_quat[KSOR_MAXB][4], body_mass[KSOR_MAXB], body_ipos[KSOR_MAXB][3],
      body_iquat[KSOR_MAXB][4], body_inertia[KSOR_MAXB][3], jnt_axis[KSOR_MAXB][3], jnt_pos[KSOR_MAXB][3],
      body_invweight0[KSOR_MAXB];
  double qpos0[KSOR_MAXQ];
  int dof_body[KSOR_MAXV], dof_parent[KSOR_MAXV];
  double dof_damping[KSOR_MAXV], dof_armature[KSOR_MAXV];
  /* joint limits of hinges (MuJoCo jnt_limited / jnt_range, by body) and dry joint friction (dof_frictionloss);
   * dof_invweight0 is the diagonal of the inverse mass matrix at qpos0, which scales their regularisation */
  int jnt_limited[KSOR_MAXB];
  double jnt_range[KSOR_MAXB][2], dof_invweight0[KSOR_MAXV], dof_frictionloss[KSOR_MAXV];
  double dof_solref[2], dof_solimp[5]; /* solref / solimp of the limit and friction rows; all zero = those of the contacts */
  double dof_stiffness[KSOR_MAXV];     /* joint springs about qpos0: passive force -stiffness (q - qpos0) on hinges */
  int act_dof[KSOR_MAXU];
  double act_gear[KSOR_MAXU], act_lo[KSOR_MAXU], act_hi[KSOR_MAXU];
  int sph_body[KSOR_MAXS];
  double sph_pos[KSOR_MAXS][3], sph_radius[KSOR_MAXS];
} KsorModel;

#endif
