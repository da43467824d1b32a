// Device-side model constants (float) and the wave-level helpers shared by the dynamics kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ks {

constexpr int kMaxB = 32;      // bodies incl. world
constexpr int kMaxQ = 40;
constexpr int kMaxV = 32;
constexpr int kMaxU = 32;
constexpr int kMaxS = 16;      // contact spheres
constexpr int kMaxR = 64;      // constraint rows (4 per sphere)
constexpr int kMaxDepth = 12;  // longest root-to-leaf body chain
constexpr int kMaxPairs = kMaxV * (kMaxV + 1) / 2;

enum { kJntNone = 0, kJntFree = 1, kJntHinge = 2 };

// Immutable after ks_model_create(); lives in device global memory and is read through the
// vector L1 / scalar cache (it is ~10 KB and shared by every wavefront).
struct DevModel {
  int nb, nq, nv, nu, ns, iterations, ls_iterations, eulerdamp, npairs, nvs /* row stride of the mass matrix in LDS, a multiple of 4 */, max_depth,
      js /* row stride of the constraint Jacobian in LDS, a multiple of 4 */,
      dofrows /* 1 when a joint is limited or has dry friction */, nfriction /* dofs with dry friction */,
      invw_ok /* 1 when every hinge dof has a positive inverse weight (what rows on the dof lanes are regularised with) */,
      frictionless /* 1: condim 1, one normal row per contact instead of the four pyramid edges */;
  float dt, gravity[3], tolerance, ls_tolerance, meaninertia, friction, impratio;
  // contact impedance constants, already clamped the way the constraint builder wants them
  float con_k, con_b, dmin, dmax, width, mid, power;
  float imp_a, imp_b;  // 1 / mid^(power-1) and 1 / (1-mid)^(power-1), the constant factors of the impedance curve
  // the same constants for the rows of joint limits and dry friction
  float dr_k, dr_b, dr_dmin, dr_dmax, dr_width, dr_mid, dr_power, dr_imp_a, dr_imp_b;
  int body_parent[kMaxB], body_jtype[kMaxB], body_qadr[kMaxB], body_dofadr[kMaxB], body_subtree_end[kMaxB],
      body_depth[kMaxB];
  int body_chain[kMaxB][kMaxDepth];  // ancestors from the tree root down to the body itself
  unsigned body_dofmask[kMaxB];      // bit j set when dof j moves the body
  float body_pos[kMaxB][3], body_quat[kMaxB][4], body_mass[kMaxB], body_ipos[kMaxB][3], body_iquat[kMaxB][4],
      body_inertia[kMaxB][3], jnt_axis[kMaxB][3], jnt_pos[kMaxB][3], body_invweight0[kMaxB];
  float qpos0[kMaxQ];
  int dof_body[kMaxV], dof_parent[kMaxV], dof_act[kMaxV];
  float dof_damping[kMaxV], dof_armature[kMaxV];
  int act_dof[kMaxU];
  float act_gear[kMaxU], act_lo[kMaxU], act_hi[kMaxU];
  int sph_body[kMaxS];
  float sph_pos[kMaxS][3], sph_radius[kMaxS];
  short pair_i[kMaxPairs], pair_j[kMaxPairs];  // (i, j): j is i or an ancestor dof of i
  // What lane L reads at the top of every substep, gathered into one 64-dword record so that it arrives in
  // sixteen 16-byte loads from one base address (layout: LaneRec in ks_dynamics.hip).
  unsigned lane_rec[64][64];
};

// ---------------------------------------------------------------- wavefront reductions (DPP, no LDS)
__device__ __forceinline__ float dpp_add(float x, int /*unused*/) { return x; }

template <int kCtrl, int kRowMask>
__device__ __forceinline__ float dpp_shift(float x) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), kCtrl, kRowMask, 0xf, false));
}

// Sum over the 64 lanes; the result is wave-uniform (read from lane 63 into a scalar register).
__device__ __forceinline__ float wave_sum(float x) {
  x += dpp_shift<0x111, 0xf>(x);  // row_shr:1
  x += dpp_shift<0x112, 0xf>(x);  // row_shr:2
  x += dpp_shift<0x114, 0xf>(x);  // row_shr:4
  x += dpp_shift<0x118, 0xf>(x);  // row_shr:8   -> lane 15 of each row holds the row total
  x += dpp_shift<0x142, 0xa>(x);  // row_bcast:15 into rows 1 and 3
  x += dpp_shift<0x143, 0xc>(x);  // row_bcast:31 into rows 2 and 3 -> lane 63 holds the total
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 63));
}

__device__ __forceinline__ float lane_bcast(float x, int lane /*uniform*/) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), lane));
}

// ---------------------------------------------------------------- 3-vectors, quaternions, spatial algebra
struct V3 {
  float x, y, z;
};
__device__ __forceinline__ V3 operator+(V3 a, V3 b) { return {a.x + b.x, a.y + b.y, a.z + b.z}; }
__device__ __forceinline__ V3 operator-(V3 a, V3 b) { return {a.x - b.x, a.y - b.y, a.z - b.z}; }
__device__ __forceinline__ V3 operator*(V3 a, float s) { return {a.x * s, a.y * s, a.z * s}; }
__device__ __forceinline__ V3 cross(V3 a, V3 b) {
  return {a.y * b.z - a.z * b.y, a.z * b.x - a.x * b.z, a.x * b.y - a.y * b.x};
}
__device__ __forceinline__ float dot(V3 a, V3 b) { return a.x * b.x + a.y * b.y + a.z * b.z; }
__device__ __forceinline__ V3 ld3(const float* p) { return {p[0], p[1], p[2]}; }
__device__ __forceinline__ void st3(float* p, V3 v) {
  p[0] = v.x;
  p[1] = v.y;
  p[2] = v.z;
}

struct Quat {
  float w, x, y, z;
};
__device__ __forceinline__ Quat qmul(Quat a, Quat b) {
  return {a.w * b.w - a.x * b.x - a.y * b.y - a.z * b.z, a.w * b.x + a.x * b.w + a.y * b.z - a.z * b.y,
          a.w * b.y - a.x * b.z + a.y * b.w + a.z * b.x, a.w * b.z + a.x * b.y - a.y * b.x + a.z * b.w};
}
__device__ __forceinline__ Quat qnormalize(Quat q) {
  const float n2 = q.w * q.w + q.x * q.x + q.y * q.y + q.z * q.z;
  if (n2 < 1e-30f) return {1.f, 0.f, 0.f, 0.f};
  const float inv = __builtin_amdgcn_rsqf(n2);  // one instruction, 1 ulp: the quaternions here are within rounding of unit length
  return {q.w * inv, q.x * inv, q.y * inv, q.z * inv};
}
struct Mat3 {
  float m[9];
};
__device__ __forceinline__ Mat3 q2mat(Quat q) {
  const float w = q.w, x = q.x, y = q.y, z = q.z;
  Mat3 r;
  r.m[0] = w * w + x * x - y * y - z * z;
  r.m[1] = 2 * (x * y - w * z);
  r.m[2] = 2 * (x * z + w * y);
  r.m[3] = 2 * (x * y + w * z);
  r.m[4] = w * w - x * x + y * y - z * z;
  r.m[5] = 2 * (y * z - w * x);
  r.m[6] = 2 * (x * z - w * y);
  r.m[7] = 2 * (y * z + w * x);
  r.m[8] = w * w - x * x - y * y + z * z;
  return r;
}
__device__ __forceinline__ V3 mul(const Mat3& m, V3 v) {
  return {m.m[0] * v.x + m.m[1] * v.y + m.m[2] * v.z, m.m[3] * v.x + m.m[4] * v.y + m.m[5] * v.z,
          m.m[6] * v.x + m.m[7] * v.y + m.m[8] * v.z};
}
__device__ __forceinline__ V3 qrot(Quat q, V3 v) { return mul(q2mat(q), v); }

// spatial vectors are [angular; linear] about the tree's centre of mass, world axes
struct Sp {
  V3 a, l;
};
__device__ __forceinline__ Sp ld6(const float* p) { return {{p[0], p[1], p[2]}, {p[3], p[4], p[5]}}; }
__device__ __forceinline__ void st6(float* p, Sp s) {
  st3(p, s.a);
  st3(p + 3, s.l);
}
__device__ __forceinline__ Sp operator+(Sp a, Sp b) { return {a.a + b.a, a.l + b.l}; }
__device__ __forceinline__ Sp operator*(Sp a, float s) { return {a.a * s, a.l * s}; }
__device__ __forceinline__ float dot(Sp a, Sp b) { return dot(a.a, b.a) + dot(a.l, b.l); }
__device__ __forceinline__ Sp cross_motion(Sp vel, Sp v) {
  return {cross(vel.a, v.a), cross(vel.a, v.l) + cross(vel.l, v.a)};
}
__device__ __forceinline__ Sp cross_force(Sp vel, Sp f) {
  return {cross(vel.a, f.a) + cross(vel.l, f.l), cross(vel.a, f.l)};
}
// inertia i = (xx yy zz xy xz yz, m*c(3), m) times a motion vector
__device__ __forceinline__ Sp inert_mul(const float* i, Sp v) {
  Sp r;
  r.a.x = i[0] * v.a.x + i[3] * v.a.y + i[4] * v.a.z - i[8] * v.l.y + i[7] * v.l.z;
  r.a.y = i[3] * v.a.x + i[1] * v.a.y + i[5] * v.a.z + i[8] * v.l.x - i[6] * v.l.z;
  r.a.z = i[4] * v.a.x + i[5] * v.a.y + i[2] * v.a.z - i[7] * v.l.x + i[6] * v.l.y;
  r.l.x = i[8] * v.a.y - i[7] * v.a.z + i[9] * v.l.x;
  r.l.y = i[6] * v.a.z - i[8] * v.a.x + i[9] * v.l.y;
  r.l.z = i[7] * v.a.x - i[6] * v.a.y + i[9] * v.l.z;
  return r;
}

}  // namespace ks
