// Fused control-step kernel: S physics substeps of one env per wavefront.
//
// One 64-lane wavefront owns one env (64-thread workgroups, so a workgroup barrier is a wave barrier).
// Where the data lives:
//   registers  the mass matrix / Newton Hessian as a 32x32 matrix-core accumulator tile while it is assembled and
//              factored, then row i of the factor for the substitutions; the lane's own body / dof / sphere
//              constants; all per-dof and per-row solver vectors
//   LDS        state (qpos, qvel, warm start, torques), body poses, com-based inertias and motion axes,
//              a staging copy of M and of J (column access), one broadcast vector
//   HBM        touched once at the start and once at the end of the control step
// Cross-lane traffic is v_readlane broadcasts (pivots, triangular solves), DPP reductions and LDS
// broadcasts; the rank updates of the Hessian and of its factorisation run as 32x32x2 fp32 MFMAs; every
// branch on solver progress is wave-uniform, so a converged env stops iterating.
// Phases of one substep: kinematics along ancestor chains -> centre of mass -> com-based inertias / motion
// axes -> composite inertias -> mass matrix -> velocities + RNE bias along ancestor chains -> smooth forces ->
// sphere/plane contacts, pyramidal rows -> Cholesky of M -> Newton with exact line search -> semi-implicit Euler.
// The arithmetic follows the MuJoCo model that ksim/engine.py:257 invokes through mjx.step.
#include "ks_common.h"
#include "ks_model.h"
#include "ks_philox.h"
#include "ks_step_args.h"

#include <cmath>
#include <cstring>

namespace ks {

typedef __attribute__((ext_vector_type(16))) float f32x16;

#define KS_SYNC() __syncthreads()
#ifndef KS_STEP_WAVES
#define KS_STEP_WAVES 4  // wavefronts per SIMD the register allocation aims at
#endif
// Phase timers for kernel tuning: compiled in only with -DKS_PROFILE, which reuses the dbg_M buffer for cycle counts.
#ifdef KS_PROFILE
#define KS_TICK(k) { const long long t_now = clock64(); prof[k] += (float)(t_now - t_last); t_last = t_now; }
#else
#define KS_TICK(k)
#endif
// A phase boundary of the step kernel.  The LDS layout is rebuilt from an offset the compiler cannot see through: the
// two dozen array addresses are then a few scalar additions at the start of each phase instead of values that stay live
// from the top of the kernel, where they do not fit the scalar registers and every use reads its address back out of a
// vector register lane.
#define KS_PHASE(k) { KS_TICK(k) int off_ = 0; asm volatile("" : "+s"(off_)); l = carve(lds_raw + off_, nb, nq, nv, nu, ns, nvs, js); }
// Register rows (mass matrix, Hessian, Jacobian) are padded from nv to a compile-time width NP, one kernel
// instantiation per width: the padding rows are unit rows and the padding columns zero, so the factorisation,
// the triangular solves and the row products run without any bound checks.
__host__ __device__ inline int padded_nv(int nv) { return nv <= 8 ? 8 : nv <= 16 ? 16 : nv <= 24 ? 24 : nv <= 28 ? 28 : 32; }
// Row stride of M and J in LDS: rows are 16-byte aligned (read with ds_read_b128, one row per lane) and the
// stride in 16-byte units is odd, which spreads 16 consecutive rows over all 64 banks.
__host__ __device__ inline int row_stride(int nv) { return (padded_nv(nv) / 4) % 2 ? padded_nv(nv) : padded_nv(nv) + 4; }
__host__ __device__ inline int m_stride(int nv) { return row_stride(nv); }
__host__ __device__ inline int j_stride(int nv) { return row_stride(nv); }

struct Lds {
  float *qpos, *qvel, *warm, *tau;
  float *xpos, *xquat, *xanchor, *xaxis;
  float *cinert, *crb, *cdof, *buf, *cvel, *cfrc, *fsub;
  float *M, *J, *vbuf, *drow;
  float *con_off, *con_D, *con_kip;
  int *con_body, *sub_end;
  unsigned* con_mask;
};

__host__ __device__ inline int up4(int n) { return (n + 3) & ~3; }

__host__ __device__ inline int lds_floats(int nb, int nq, int nv, int nu, int ns) {
  const int nvs = m_stride(nv), js = j_stride(nv);
  int n = 0;
  n += up4(nq) + 32 + up4(nv) + up4(nu);                             // qpos qvel(32) warm tau
  n += up4(nb * 3) + up4(nb * 4) + 2 * up4(nb * 3);                    // xpos xquat xanchor xaxis
  n += up4(nv * 6) + up4(nb * 6);                                    // cdof cvel
  const int scratch = 2 * up4(nb * 10) + up4(nv * 6) + 2 * up4(nb * 6);  // cinert crb buf fsub cfrc
  const int jsz = up4(4 * ns * js + 32);                             // J overlays that scratch once it is dead
  n += scratch > jsz ? scratch : jsz;
  n += up4(nv * nvs) + 32 + 64;                                      // M vbuf drow
  n += up4(ns * 3) + 4 * up4(ns) + up4(nb);                          // con_off con_D con_kip con_body con_mask sub_end
  return n + 8;
}

__device__ __forceinline__ Lds carve(float* p, int nb, int nq, int nv, int nu, int ns, int nvs, int js) {
  Lds l;
  auto take = [&](int n) {
    float* r = p;
    p += up4(n);
    return r;
  };
  l.qpos = take(nq); l.qvel = take(32); l.warm = take(nv); l.tau = take(nu);
  l.xpos = take(nb * 3); l.xquat = take(nb * 4); l.xanchor = take(nb * 3); l.xaxis = take(nb * 3);
  l.cdof = take(nv * 6); l.cvel = take(nb * 6);
  {
    float* base = p;
    l.cinert = take(nb * 10); l.crb = take(nb * 10); l.buf = take(nv * 6);
    l.fsub = take(nb * 6); l.cfrc = take(nb * 6);
    float* end = p;
    l.J = base;  // written only after the bias forces are out of fsub
    float* jend = base + up4(4 * ns * js + 32);
    p = end > jend ? end : jend;
  }
  l.M = take(nv * nvs); l.vbuf = take(32); l.drow = take(64);
  l.con_off = take(ns * 3); l.con_D = take(ns); l.con_kip = take(ns);
  l.con_body = reinterpret_cast<int*>(take(ns));
  l.con_mask = reinterpret_cast<unsigned*>(take(ns));
  l.sub_end = reinterpret_cast<int*>(take(nb));
  return l;
}

// NP consecutive floats from a 16-byte aligned LDS address
template <int NP>
__device__ __forceinline__ void load_row(const float* p, float (&v)[NP]) {
  const float4* q = reinterpret_cast<const float4*>(p);
#pragma unroll
  for (int k = 0; k < NP / 4; ++k) {
    const float4 t = q[k];
    v[4 * k] = t.x; v[4 * k + 1] = t.y; v[4 * k + 2] = t.z; v[4 * k + 3] = t.w;
  }
}


// Right-looking Cholesky of a symmetric matrix of up to 32 rows with the rank-1 updates on the matrix cores.
// The matrix sits in the accumulator layout of the 32x32x2 fp32 MFMA: lane c + 32 h holds, in register
// 4 g + e, the entry (row 8 g + 4 h + e, column c).  Step j reads the pivot from the lane that owns column j, scales row j (one register of the 32 lanes of one
// half) and feeds that scaled row to one MFMA as both operands, -l l^T, which updates every entry right of and
// below the pivot at once; the other lane half contributes zeros.  A step costs about eight vector instructions
// instead of two per updated column.  Column j below the diagonal is left as it was when the pivot was reached
// (L[k][j] * L[j][j]) and row j right of the diagonal holds L[k][j]: read down a lane, that is row c of L to the
// left of the diagonal and the scaled column c below it, exactly what the column-oriented substitutions take,
// once the upper lane half has handed its 16 registers to the lower one.  On return, in lane i < NP:
//   R[j], j < i : L[i][j]              R[k], k > i : L[k][i] * L[i][i]              myinv = 1 / L[i][i]
// `nv` (wave-uniform) is the real size: the steps of the padded columns, which would multiply zeros, are branched over
// (only steps past the next smaller instantiation's size carry the test).
constexpr int padded_from(int np) { return np > 28 ? 28 : (np > 24 ? 24 : (np > 16 ? 16 : (np > 8 ? 8 : 0))); }

template <int NP>
__device__ __forceinline__ void chol_tile(f32x16& T, float (&R)[NP], float& myinv, int lane, int nv) {
  // The lane id is made opaque so that the per-step lane masks are compared where they are used: shared between the call
  // sites they would be sixty-odd scalar register pairs that live across the solver and are read back from spill lanes.
  asm volatile("" : "+v"(lane));
  const int c = lane & 31, half = lane >> 5;
  myinv = 1.f;
#pragma unroll
  for (int j = 0; j < NP; ++j) {
    if (j >= padded_from(NP) && j >= nv) continue;  // a padded column: unit pivot, nothing below or right of it
    const int hj = (j >> 2) & 1, rho = 4 * (j >> 3) + (j & 3);
    // a pivot below 1e-30 (or not a number) counts as 1e-30: the reciprocal root is capped instead of the pivot floored,
    // which is the same number and one instruction less on the chain
    const float inv = fminf(__builtin_amdgcn_rsqf(lane_bcast(T[rho], j + 32 * hj)), 1e15f);
    myinv = lane == j ? inv : myinv;
    const bool sel = half == hj && c > j;
    const float t = T[rho] * inv;
    const float a = sel ? t : 0.f, na = sel ? -t : 0.f;
    T[rho] = sel ? t : T[rho];
    // the last real column has nothing right of or below it
    if (j + 1 < NP && !(j + 1 >= padded_from(NP) && j + 1 >= nv)) T = __builtin_amdgcn_mfma_f32_32x32x2f32(na, a, T, 0, 0, 0);
  }
#pragma unroll
  for (int g = 0; g < 4; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int jlo = 8 * g + e, jhi = 8 * g + 4 + e;
      if (jlo < NP) R[jlo] = T[4 * g + e];
      if (jhi < NP) R[jhi] = __shfl_xor(T[4 * g + e], 32);
    }
}

// Mass matrix (LDS, rows of `stride` floats, zero beyond nv) into the accumulator layout, unit diagonal on the padding.
__device__ __forceinline__ void load_mtile(f32x16& T, const float* __restrict__ M, int stride, int nv, int np, int lane) {
  // The lane id is made opaque here: otherwise the sixteen unit-diagonal constants below are computed once, shared by
  // all the call sites of a substep and kept (spilled) across the whole solver instead of being rebuilt in a few cycles.
  asm volatile("" : "+v"(lane));
  const int c = lane & 31, half = lane >> 5;
  const bool real = c < nv;
  const float* row = M + (real ? c : 0) * stride;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int r0 = 8 * g + 4 * half;
    const bool inside = r0 + 4 <= np;
    const float4 v = *reinterpret_cast<const float4*>(row + (inside ? r0 : 0));
    T[4 * g] = (real && inside) ? v.x : (r0 == c ? 1.f : 0.f);
    T[4 * g + 1] = (real && inside) ? v.y : (r0 + 1 == c ? 1.f : 0.f);
    T[4 * g + 2] = (real && inside) ? v.z : (r0 + 2 == c ? 1.f : 0.f);
    T[4 * g + 3] = (real && inside) ? v.w : (r0 + 3 == c ? 1.f : 0.f);
  }
}

// x = (L L^T)^-1 b, lane i holding b_i and returning x_i
template <int NP>
__device__ __forceinline__ float solve_regs(const float (&R)[NP], float myinv, int lane, float b, int nv) {
  asm volatile("" : "+v"(lane));  // as in chol_tile: the masks lane > j, lane < k are rebuilt here, not kept
  float r = b;
#pragma unroll
  for (int j = 0; j < NP; ++j) {  // L y = b; lane j keeps r_j = y_j * L[j][j]
    if (j >= padded_from(NP) && j >= nv) continue;  // padded unknowns are zero and couple to nothing
    const float yj = lane_bcast(r * myinv, j);
    r = lane > j ? r - R[j] * yj : r;
  }
  const float myinv2 = myinv * myinv;
#pragma unroll
  for (int k = NP - 1; k >= 0; --k) {  // L^T x = y in the scaled form  sum_{k>i} R[k] x_k + L[i][i]^2 x_i = r_i
    if (k >= padded_from(NP) && k >= nv) continue;
    const float xk = lane_bcast(r * myinv2, k);
    r = lane < k ? r - R[k] * xk : r;
  }
  return r * myinv2;
}

// dot product of an LDS row (per-lane address, 16-byte aligned) with a broadcast register vector
template <int NP>
__device__ __forceinline__ float row_dot(const float* row, const float (&vv)[NP]) {
  const float4* q = reinterpret_cast<const float4*>(row);
  float s0 = 0.f, s1 = 0.f;
#pragma unroll
  for (int k = 0; k < NP / 4; ++k) {  // two chains of fused multiply-adds, one instruction per product
    const float4 t = q[k];
    s0 = fmaf(t.x, vv[4 * k], s0);
    s1 = fmaf(t.y, vv[4 * k + 1], s1);
    s0 = fmaf(t.z, vv[4 * k + 2], s0);
    s1 = fmaf(t.w, vv[4 * k + 3], s1);
  }
  return s0 + s1;
}

// Per-lane constants of one substep, as stored in DevModel::lane_rec (64 dwords, filled by ks_model_create):
// lane L's body (L < nb), dof (L < nv), contact sphere (L < ns) and its share of the (i, ancestor j) dof pairs.
// Lanes beyond a range carry the entries of index 0 (or -1 / zero where the kernel tests for that).
struct LaneRec {
  int b_parent, b_jtype, b_qadr, b_dofadr;
  int b_depth;
  float b_q0, b_mass, d_stiffness;  // d_stiffness: spring of the hinge whose dof this lane holds
  float b_pos[3], b_ipos[3], b_inertia[3], b_jaxis[3], b_jpos[3], pad1;
  float b_quat[4], b_iquat[4];
  int d_body, d_act, d_jtype, d_k;
  float d_damping, d_armature, d_gear, d_lo, d_hi;
  int s_body;
  float s_rad, s_invw;
  float s_pos[3];
  unsigned s_mask;
  int pk[kMaxPairs / 64 + 1];
  // rows that live on the dof's own lane: hinge limit (range, inverse weight, address of the joint angle) and dry
  // friction (level and the constant stiffness 1 / R of its row)
  int d_limited, d_qadr;
  float d_rlo, d_rhi, d_invw, d_floss, d_frD;
};
static_assert(sizeof(LaneRec) == 256, "LaneRec must fill the 64-dword record");

struct LsPoint {
  float alpha, cost, d0, d1;
};

// constraint impedance d(|pos|) of a solimp whose parameters are already clamped
__device__ __forceinline__ float impedance_of(float pos, float dmin, float dmax, float width, float mid, float power, float imp_a,
                                              float imp_b) {
  const float ix = fabsf(pos) / width;
  // x^power: the default power of 2 (and 1) without the general power function
  const float ox = 1.f - ix;
  const float px = power == 2.f ? ix * ix : (power == 1.f ? ix : powf(ix, power));
  const float po = power == 2.f ? ox * ox : (power == 1.f ? ox : powf(ox, power));
  const float ia = imp_a * px;
  const float ib = 1.f - imp_b * po;
  const float iy = ix < mid ? ia : ib;
  float imp = dmin + iy * (dmax - dmin);
  imp = fminf(fmaxf(imp, dmin), dmax);
  if (ix > 1.f) imp = dmax;
  return imp;
}
// of the contact rows, and of the rows of joint limits and dry friction
__device__ __forceinline__ float impedance(const DevModel& m, float pos) {
  return impedance_of(pos, m.dmin, m.dmax, m.width, m.mid, m.power, m.imp_a, m.imp_b);
}
__device__ __forceinline__ float impedance_dof(const DevModel& m, float pos) {
  return impedance_of(pos, m.dr_dmin, m.dr_dmax, m.dr_width, m.dr_mid, m.dr_power, m.dr_imp_a, m.dr_imp_b);
}

// The rows a dof lane carries itself: the violated limit of its hinge (J = lim_s e_j, lim_s = +-1, 0 when none) and its
// dry friction (J = e_j, force clipped at +-fr_fl, 0 when none).  All zero on lanes that hold no dof.
struct DofRows {
  float lim_s, lim_aref, lim_D, fr_fl, fr_aref, fr_D, fr_rf;  // fr_rf = fr_fl / fr_D, where the friction force saturates
};

// Cost of the lane's rows at acceleration qa; their force on the dof, their Hessian diagonal and which of them are in
// their quadratic zone (bit 0 limit, bit 1 friction).
__device__ __forceinline__ float dofrow_eval(const DofRows& r, float qa, float& force, float& hdiag, int& zone) {
  float cost = 0.f;
  force = 0.f; hdiag = 0.f; zone = 0;
  const float xl = r.lim_s * qa - r.lim_aref;
  if (r.lim_s != 0.f && xl < 0.f) {
    cost = 0.5f * r.lim_D * xl * xl; force = -r.lim_D * xl * r.lim_s; hdiag = r.lim_D; zone = 1;
  }
  if (r.fr_fl > 0.f) {
    const float xf = qa - r.fr_aref, rf = r.fr_rf;
    if (xf <= -rf) { cost += r.fr_fl * (-0.5f * rf - xf); force += r.fr_fl; }
    else if (xf >= rf) { cost += r.fr_fl * (-0.5f * rf + xf); force -= r.fr_fl; }
    else { cost += 0.5f * r.fr_D * xf * xf; force -= r.fr_D * xf; hdiag += r.fr_D; zone |= 2; }
  }
  return cost;
}

// Coefficients of the rows' cost along qa + alpha s, in the zones the rows are in at that alpha.
__device__ __forceinline__ void dofrow_quad(const DofRows& r, float qa, float sdir, float alpha, float& t0, float& t1,
                                            float& t2) {
  t0 = 0.f; t1 = 0.f; t2 = 0.f;
  const float x0 = r.lim_s * qa - r.lim_aref, jv = r.lim_s * sdir;
  if (r.lim_s != 0.f && x0 + alpha * jv < 0.f) {
    t0 = 0.5f * x0 * x0 * r.lim_D; t1 = jv * x0 * r.lim_D; t2 = 0.5f * jv * jv * r.lim_D;
  }
  if (r.fr_fl > 0.f) {
    const float f0 = qa - r.fr_aref, rf = r.fr_rf, x = f0 + alpha * sdir;
    if (x <= -rf) { t0 += r.fr_fl * (-0.5f * rf - f0); t1 -= r.fr_fl * sdir; }
    else if (x >= rf) { t0 += r.fr_fl * (-0.5f * rf + f0); t1 += r.fr_fl * sdir; }
    else { t0 += 0.5f * f0 * f0 * r.fr_D; t1 += sdir * f0 * r.fr_D; t2 += 0.5f * sdir * sdir * r.fr_D; }
  }
}

__device__ __forceinline__ bool in_bracket(const LsPoint& x, const LsPoint& y) {
  return ((x.d0 < y.d0) && (y.d0 < 0.f)) || ((x.d0 > y.d0) && (y.d0 > 0.f));
}

// sum of one component over a contiguous subtree range of an array with `w` floats per body
__device__ __forceinline__ float range_sum(const float* base, int w, int b, int e) {
  float s0 = 0.f, s1 = 0.f;
  int c = b;
  for (; c + 1 < e; c += 2) {
    s0 += base[w * c];
    s1 += base[w * (c + 1)];
  }
  if (c < e) s0 += base[w * c];
  return s0 + s1;
}

// ------------------------------------------------------------------------------------------- the fused kernel
// FWD = true is the forward-only variant (derived fields + warm start of a given state, no actuation, no
// integration) that replaces the mjx.forward of a reset.
template <bool FWD, int NP, bool DR>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(KS_STEP_WAVES, KS_STEP_WAVES)))
void step_kernel(StepArgs a) {
  extern __shared__ __attribute__((aligned(16))) float lds_raw[];
  const DevModel& m = *a.model;
  const int lane = threadIdx.x;
  // heaviest envs first when an order is given (ks_work_order, which also keeps neighbouring envs on one XCD); without
  // one, workgroup b takes env (b % 8) (N / 8) + b / 8 for the same reason
  int64_t env = blockIdx.x;
  if (a.env_order) env = a.env_order[blockIdx.x];
  else if (a.N % 8 == 0) env = (int64_t)(blockIdx.x % 8) * (a.N / 8) + blockIdx.x / 8;
  if (a.env_mask && !a.env_mask[env]) return;  // wave-uniform
  int work = 0;  // wave-uniform cost estimate of this control step
  const int nb = m.nb, nq = m.nq, nv = m.nv, nu = m.nu, ns = m.ns, nvs = m.nvs, js = m.js;
  Lds l = carve(lds_raw, nb, nq, nv, nu, ns, nvs, js);
  const int rq = (nb > 1 && m.body_jtype[1] == kJntFree) ? 7 : 0;
  const int rv = rq ? 6 : 0;

  for (int i = lane; i < nq; i += 64) l.qpos[i] = a.qpos[env * nq + i];
  if (lane < 32) l.qvel[lane] = lane < nv ? a.qvel[env * nv + lane] : 0.f;
  if (lane < nv) l.warm[lane] = a.qacc_warmstart ? a.qacc_warmstart[env * nv + lane] : 0.f;
  for (int i = lane; i < nu; i += 64) l.tau[i] = a.ctrl_in ? a.ctrl_in[env * nu + i] : 0.f;
  for (int i = lane; i < nb; i += 64) l.sub_end[i] = m.body_subtree_end[i];
  if (lane == 0) {  // world body
    for (int k = 0; k < 3; ++k) { l.xpos[k] = 0.f; l.xanchor[k] = 0.f; l.xaxis[k] = 0.f; }
    l.xquat[0] = 1.f; l.xquat[1] = l.xquat[2] = l.xquat[3] = 0.f;
    for (int k = 0; k < 6; ++k) l.cvel[k] = 0.f;
  }
  const float mu = a.friction ? a.friction[env] : m.friction;
  const float latency = a.latency ? a.latency[env] : 0.f;
  const float scale = 1.0f / (m.meaninertia * (float)(nv > 1 ? nv : 1));
  KS_SYNC();
#ifdef KS_PROFILE
  float prof[16];
  for (int k = 0; k < 16; ++k) prof[k] = 0.f;
  long long t_last = clock64();
#endif

  const int nsub = FWD ? 1 : a.substeps;
  // An env that the termination pass has just reset still owes the forward pass of its reset (engine.py:213: derived
  // quantities and the warm start of the new episode, from the reset state with zero controls).  With `fresh` given the
  // step does it itself, as a pass `sub = -1` that neither actuates nor integrates, instead of a masked launch of the
  // forward-only kernel between the termination pass and this step.
  const bool fresh_env = !FWD && a.fresh && a.fresh[env];  // wave-uniform
  for (int sub = fresh_env ? -1 : 0; sub < nsub; ++sub) {
    const bool fwd = FWD || sub < 0;
    // The lane id is re-materialised per substep so that per-lane LDS addresses are recomputed inside the loop
    // instead of being hoisted out of it into ~130 long-lived registers (which would halve the occupancy).
    int lane_v = threadIdx.x;
    asm volatile("" : "+v"(lane_v));
    const int lane = lane_v;
      // ---- per-lane model constants: re-read every substep (they hit the vector L1) so that they do not stay live
      // across the solver, whose register rows set the occupancy
    const bool is_body = lane > 0 && lane < nb;
    const int bl = is_body ? lane : 0;
    const bool is_dof = lane < nv;
    const bool is_sph = lane < ns;
    LaneRec rec;
    {
      const uint4* src = reinterpret_cast<const uint4*>(m.lane_rec[lane]);
      uint4* dst = reinterpret_cast<uint4*>(&rec);
#pragma unroll
      for (int k = 0; k < 16; ++k) dst[k] = src[k];
    }
    const int b_parent = rec.b_parent, b_jtype = rec.b_jtype, b_qadr = rec.b_qadr, b_dofadr = rec.b_dofadr,
              b_depth = rec.b_depth;
    (void)b_parent;
    const V3 b_pos = {rec.b_pos[0], rec.b_pos[1], rec.b_pos[2]};
    V3 b_ipos = {rec.b_ipos[0], rec.b_ipos[1], rec.b_ipos[2]}, b_inertia = {rec.b_inertia[0], rec.b_inertia[1], rec.b_inertia[2]};
    if (a.body_ipos && is_body) b_ipos = ld3(a.body_ipos + (env * nb + bl) * 3);        // per-env centres of mass
    if (a.body_inertia && is_body) b_inertia = ld3(a.body_inertia + (env * nb + bl) * 3);  // and principal inertias
    const V3
             b_jaxis = {rec.b_jaxis[0], rec.b_jaxis[1], rec.b_jaxis[2]}, b_jpos = {rec.b_jpos[0], rec.b_jpos[1], rec.b_jpos[2]};
    const Quat b_quat = {rec.b_quat[0], rec.b_quat[1], rec.b_quat[2], rec.b_quat[3]};
    const Quat b_iquat = {rec.b_iquat[0], rec.b_iquat[1], rec.b_iquat[2], rec.b_iquat[3]};
    const float b_q0 = rec.b_q0;
    const float b_mass = is_body ? rec.b_mass * (a.mass_scale ? a.mass_scale[env * nb + bl] : 1.f) : 0.f;
    const int d_body = rec.d_body, d_act = rec.d_act, d_jtype = rec.d_jtype, d_k = rec.d_k;
    const float d_damping = rec.d_damping * ((a.damping_scale && is_dof) ? a.damping_scale[env * nv + lane] : 1.f);
    const float d_armature = rec.d_armature, d_gear = rec.d_gear, d_lo = rec.d_lo, d_hi = rec.d_hi;
    (void)d_armature;
    const int s_body = rec.s_body;
    V3 s_pos = {rec.s_pos[0], rec.s_pos[1], rec.s_pos[2]};
    float s_rad = rec.s_rad;
    const float s_invw = rec.s_invw;
    if (a.sph_pos && lane < ns) {  // per-env contact spheres
      s_pos = ld3(a.sph_pos + (env * ns + lane) * 3);
      s_rad = a.sph_radius[env * ns + lane];
    }
    const unsigned s_mask = rec.s_mask;
    int pk[kMaxPairs / 64 + 1];
#pragma unroll
    for (int k = 0; k < kMaxPairs / 64 + 1; ++k) pk[k] = rec.pk[k];

    // ---- actuators (ksim/engine.py:287-320, ksim/actuators.py:198-217)
    if (!fwd && (sub % a.actuator_period) == 0 && lane < nu) {
      const int u = lane;
      // the actuator inputs of this control step are read again at every actuator update (they stay in the caches):
      // held in registers they would be live across the solver of every substep
      const bool posvel = a.actuator_type == KS_ACT_POSITION_VELOCITY;
      const int na = posvel ? 2 * nu : nu;  // width of the action vector
      const int64_t ea = env * na + lane, eu = env * nu + lane;
      const float u_last = a.last_ctrl[ea], u_act = a.action[ea];
      const bool u_drop = a.drop && a.drop[ea];
      const float u_zero = a.zero_offset ? a.zero_offset[eu] : 0.f;
      float u_kp = 0.f, u_kd = 0.f, u_lim = 0.f, u_abias = 0.f, u_tbias = 0.f;
      if (a.actuator_type != KS_ACT_TORQUE) {
        u_kp = a.kp[lane] * (a.kp_scale ? a.kp_scale[env] : 1.f);
        u_kd = a.kd[lane] * (a.kd_scale ? a.kd_scale[env] : 1.f);
        u_lim = a.ctrl_clip[lane] * (a.torque_limit_scale ? a.torque_limit_scale[env] : 1.f);
        u_abias = a.action_bias ? a.action_bias[eu] : 0.f;
        u_tbias = a.torque_bias ? a.torque_bias[eu] : 0.f;
      }
      float prct = (float)sub - latency;
      prct = fminf(fmaxf(prct, 0.f), 1.f);
      const float c = u_drop ? u_last : u_last * (1.0f - prct) + u_act * prct;
      const int64_t su = ((int64_t)sub * a.N + env) * nu + u, sa = ((int64_t)sub * a.N + env) * na + u;
      float t;
      if (a.actuator_type == KS_ACT_TORQUE) {
        t = c + (a.torque_noise ? a.torque_noise[su] : 0.f);
      } else {
        float target_vel = 0.f;
        if (posvel) {  // the velocity targets ride in the second half of the action vector
          const float v_last = a.last_ctrl[ea + nu], v_act = a.action[ea + nu];
          const bool v_drop = a.drop && a.drop[ea + nu];
          target_vel = (v_drop ? v_last : v_last * (1.0f - prct) + v_act * prct) + (a.action_noise ? a.action_noise[sa + nu] : 0.f);
        }
        const float target = c * a.action_scale + (a.action_noise ? a.action_noise[sa] : 0.f) + u_abias;
        const float q = l.qpos[rq + u] - u_zero;
        t = u_kp * (target - q) + u_kd * (target_vel - l.qvel[rv + u]);
        t = t + (a.torque_noise ? a.torque_noise[su] : 0.f) + u_tbias;
        t = fminf(fmaxf(t, -u_lim), u_lim);
      }
      l.tau[u] = t;
    }

    // ---- events (ksim/engine.py:322-333, ksim/events.py): impulses on the root velocity when an interval runs out
    if (!fwd && a.n_events > 0) {
      const uint64_t ev_step = a.event_rng.step + (a.event_rng.step_base ? *a.event_rng.step_base : 0ull);
#pragma nounroll
      for (int e = 0; e < a.n_events; ++e) {  // a rolled loop: nothing of the event records is kept across the substeps
        if (a.events[e].kind != KS_EVENT_FORCE_PUSH) {
          const KsEventDesc ev = a.events[e];
          // the timer stays in memory between substeps (lane 0 owns it) so that it costs no register over the solver
          float* tleft = a.event_state + (int64_t)e * a.N + env;
          float left = lane_bcast(lane == 0 ? *tleft : 0.f, 0) - m.dt;
          if (left <= 0.f) {  // wave-uniform
            float u0, u1, u2;
            if (a.event_uniform) {
              const float* u = a.event_uniform + (((int64_t)sub * a.N + env) * a.n_events + e) * KS_EVENT_DRAWS;
              u0 = u[0]; u1 = u[1]; u2 = u[2];
            } else {
              const Philox4 r = draw(a.event_rng.seed, ev_step, kRngEvent, (uint64_t)env, (uint32_t)(sub * KS_MAX_EVENTS + e));
              u0 = u01(r.x); u1 = u01(r.y); u2 = u01(r.z);
            }
            if (lane == 0) {
              if (ev.kind == KS_EVENT_LINEAR_PUSH) {
                const float th = 6.28318530717958647692f * u0, mag = (ev.lo + u1 * (ev.hi - ev.lo)) * ev.mag * ev.level_scale;
                l.qvel[0] += cosf(th) * mag;
                l.qvel[1] += sinf(th) * mag;
              } else if (ev.kind == KS_EVENT_ANGULAR_PUSH) {
                const float mag = (ev.lo + u1 * (ev.hi - ev.lo)) * ev.mag;
                l.qvel[5] += (u0 < 0.5f ? -mag : mag) * ev.level_scale;
              } else if (ev.kind == KS_EVENT_JUMP) {
                const float h = (ev.lo + u0 * (ev.hi - ev.lo)) * ev.level_scale;
                for (int k = 0; k < 3; ++k) l.qvel[k] += sqrtf(2.f * -m.gravity[k] * h);
              }
            }
            left = ev.interval_lo + u2 * (ev.interval_hi - ev.interval_lo);
          }
          if (lane == 0) *tleft = left;
        }
      }
      KS_SYNC();
    }

    KS_PHASE(0)
    // ---- kinematics.  Every body first writes its pose relative to its parent (joint rotation included) to
    // LDS, then composes the poses along its own chain of ancestors from the root down: max_depth short
    // steps shared by all bodies instead of one full pass per tree level.
    V3 xipos = {0.f, 0.f, 0.f};
    Mat3 ximat;
#pragma unroll
    for (int k = 0; k < 9; ++k) ximat.m[k] = 0.f;
    float* lpose = l.cinert;  // 7 floats per body; the inertia scratch is not in use yet
    if (is_body) {
      V3 tl;
      Quat ql;
      if (b_jtype == kJntFree) {
        tl = ld3(l.qpos + b_qadr);
        ql = qnormalize({l.qpos[b_qadr + 3], l.qpos[b_qadr + 4], l.qpos[b_qadr + 5], l.qpos[b_qadr + 6]});
      } else {
        tl = b_pos;
        ql = b_quat;
        if (b_jtype == kJntHinge) {
          float hs, hc;
          sincosf(0.5f * (l.qpos[b_qadr] - b_q0), &hs, &hc);
          const Quat jr = {hc, b_jaxis.x * hs, b_jaxis.y * hs, b_jaxis.z * hs};
          // rotation about the joint anchor: p + R_b (a - R_j a) with a the anchor in the body frame
          const V3 ra = mul(q2mat(jr), b_jpos);
          tl = b_pos + mul(q2mat(b_quat), b_jpos - ra);
          ql = qmul(b_quat, jr);
        }
      }
      st3(lpose + 7 * lane, tl);
      lpose[7 * lane + 3] = ql.w; lpose[7 * lane + 4] = ql.x; lpose[7 * lane + 5] = ql.y; lpose[7 * lane + 6] = ql.z;
    }
    KS_SYNC();
    {
      V3 pos = {0.f, 0.f, 0.f};
      Quat quat = {1.f, 0.f, 0.f, 0.f};
      for (int k = 0; k < m.max_depth; ++k) {
        if (k < b_depth) {
          const int cb = m.body_chain[bl][k];
          const V3 tl = ld3(lpose + 7 * cb);
          const Quat ql = {lpose[7 * cb + 3], lpose[7 * cb + 4], lpose[7 * cb + 5], lpose[7 * cb + 6]};
          pos = pos + mul(q2mat(quat), tl);
          quat = qmul(quat, ql);
        }
      }
      if (is_body) {
        quat = qnormalize(quat);
        const Mat3 R = q2mat(quat);
        V3 anchor = pos, axis = {0.f, 0.f, 1.f};
        if (b_jtype == kJntHinge) {
          anchor = pos + mul(R, b_jpos);
          axis = mul(R, b_jaxis);
        }
        st3(l.xpos + 3 * lane, pos);
        l.xquat[4 * lane] = quat.w; l.xquat[4 * lane + 1] = quat.x; l.xquat[4 * lane + 2] = quat.y; l.xquat[4 * lane + 3] = quat.z;
        st3(l.xanchor + 3 * lane, anchor);
        st3(l.xaxis + 3 * lane, axis);
        xipos = pos + mul(R, b_ipos);
        ximat = q2mat(qnormalize(qmul(quat, b_iquat)));
      }
    }
    KS_SYNC();

    KS_PHASE(1)
    // ---- centre of mass of the tree (wave-uniform), com-based inertias and motion axes
    const float mt = wave_sum(b_mass);
    const float minv = mt > 1e-15f ? 1.0f / mt : 0.f;
    const V3 com = {wave_sum(b_mass * xipos.x) * minv, wave_sum(b_mass * xipos.y) * minv,
                    wave_sum(b_mass * xipos.z) * minv};
    if (lane == 0) {  // world body entries of the per-substep scratch (the scratch is reused by J later)
      for (int k = 0; k < 10; ++k) l.cinert[k] = 0.f;
      for (int k = 0; k < 6; ++k) l.cfrc[k] = 0.f;
    }
    float ci[10];
    {
      const float* R = ximat.m;
      const float I0 = b_inertia.x, I1 = b_inertia.y, I2 = b_inertia.z;
      const V3 d = xipos - com;
      const float d2 = dot(d, d);
      ci[0] = R[0] * I0 * R[0] + R[1] * I1 * R[1] + R[2] * I2 * R[2] + b_mass * (d2 - d.x * d.x);
      ci[1] = R[3] * I0 * R[3] + R[4] * I1 * R[4] + R[5] * I2 * R[5] + b_mass * (d2 - d.y * d.y);
      ci[2] = R[6] * I0 * R[6] + R[7] * I1 * R[7] + R[8] * I2 * R[8] + b_mass * (d2 - d.z * d.z);
      ci[3] = R[0] * I0 * R[3] + R[1] * I1 * R[4] + R[2] * I2 * R[5] - b_mass * d.x * d.y;
      ci[4] = R[0] * I0 * R[6] + R[1] * I1 * R[7] + R[2] * I2 * R[8] - b_mass * d.x * d.z;
      ci[5] = R[3] * I0 * R[6] + R[4] * I1 * R[7] + R[5] * I2 * R[8] - b_mass * d.y * d.z;
      ci[6] = b_mass * d.x; ci[7] = b_mass * d.y; ci[8] = b_mass * d.z;
      ci[9] = b_mass;
      if (is_body) {
#pragma unroll
        for (int k = 0; k < 10; ++k) l.cinert[10 * lane + k] = ci[k];
        if (a.cinert && sub == nsub - 1) {  // the LDS copy is scratch that the constraint rows reuse: export it here
#pragma unroll
          for (int k = 0; k < 10; ++k) a.cinert[((int64_t)env * nb + lane) * 10 + k] = ci[k];
        }
      }
      if (a.cinert && sub == nsub - 1 && lane == 0)
        for (int k = 0; k < 10; ++k) a.cinert[(int64_t)env * nb * 10 + k] = 0.f;  // world body
    }
    Sp my_cdof = {{0.f, 0.f, 0.f}, {0.f, 0.f, 0.f}};
    if (is_dof) {
      const V3 off = com - ld3(l.xanchor + 3 * d_body);
      if (d_jtype == kJntFree) {
        if (d_k < 3) {
          my_cdof.l = {d_k == 0 ? 1.f : 0.f, d_k == 1 ? 1.f : 0.f, d_k == 2 ? 1.f : 0.f};
        } else {
          const Mat3 Rb = q2mat({l.xquat[4 * d_body], l.xquat[4 * d_body + 1], l.xquat[4 * d_body + 2], l.xquat[4 * d_body + 3]});
          const float* R = Rb.m;
          const V3 ax = d_k == 3 ? V3{R[0], R[3], R[6]} : d_k == 4 ? V3{R[1], R[4], R[7]} : V3{R[2], R[5], R[8]};
          my_cdof = {ax, cross(ax, off)};
        }
      } else {
        const V3 ax = ld3(l.xaxis + 3 * d_body);
        my_cdof = {ax, cross(ax, off)};
      }
      st6(l.cdof + 6 * lane, my_cdof);
    }
    KS_SYNC();

    KS_PHASE(2)
    // ---- composite inertias (subtree = contiguous body range) and the mass matrix
    for (int idx = lane; idx < nb * 10; idx += 64) {
      const int b = idx / 10, k = idx - 10 * b;
      l.crb[idx] = b > 0 ? range_sum(l.cinert + k, 10, b, l.sub_end[b]) : 0.f;
    }
    for (int idx = lane; idx < nv * nvs; idx += 64) l.M[idx] = 0.f;
    KS_SYNC();
    if (is_dof) st6(l.buf + 6 * lane, inert_mul(l.crb + 10 * d_body, my_cdof));
    KS_SYNC();
#pragma unroll
    for (int k = 0; k < kMaxPairs / 64 + 1; ++k) {
      if (pk[k] >= 0) {
        const int i = pk[k] >> 8, j = pk[k] & 0xff;
        float v = dot(ld6(l.cdof + 6 * j), ld6(l.buf + 6 * i));
        if (i == j) v += m.dof_armature[i] * (a.armature_scale ? a.armature_scale[env * nv + i] : 1.f);
        l.M[i * nvs + j] = v;
        l.M[j * nvs + i] = v;
      }
    }

    KS_PHASE(3)
    // ---- body velocities and bias accelerations: the motion axes are all expressed in one frame, so every
    // body accumulates them over the dofs of its own ancestor chain, root first (no pass per tree level)
    {
      Sp v = {{0.f, 0.f, 0.f}, {0.f, 0.f, 0.f}};
      Sp acc = {{0.f, 0.f, 0.f}, {-m.gravity[0], -m.gravity[1], -m.gravity[2]}};
      for (int k = 0; k < m.max_depth; ++k) {
        if (k < b_depth) {
          const int cb = m.body_chain[bl][k];
          const int jt = m.body_jtype[cb], da = m.body_dofadr[cb];
          if (jt == kJntFree) {
            for (int c = 0; c < 3; ++c) v = v + ld6(l.cdof + 6 * (da + c)) * l.qvel[da + c];
            Sp dv = {{0.f, 0.f, 0.f}, {0.f, 0.f, 0.f}};
            for (int c = 3; c < 6; ++c) {
              const Sp cd = ld6(l.cdof + 6 * (da + c));
              const float qd = l.qvel[da + c];
              acc = acc + cross_motion(v, cd) * qd;
              dv = dv + cd * qd;
            }
            v = v + dv;
          } else if (jt == kJntHinge) {
            const Sp cd = ld6(l.cdof + 6 * da);
            const float qd = l.qvel[da];
            acc = acc + cross_motion(v, cd) * qd;
            v = v + cd * qd;
          }
        }
      }
      Sp cf = inert_mul(ci, acc) + cross_force(v, inert_mul(ci, v));
      // ---- force pushes (ksim/events.py:240-365): a wrench held on one body enters the Newton-Euler pass as an
      // external force on that body, so the subtree sums and the projection on the motion axes below turn it into
      // the generalised force J^T f.  Lane 0 owns the state in memory; the other lanes get it by broadcast.
      if (!fwd && a.n_force_events > 0) {
        const uint64_t ev_step = a.event_rng.step + (a.event_rng.step_base ? *a.event_rng.step_base : 0ull);
        Sp ext = {{0.f, 0.f, 0.f}, {0.f, 0.f, 0.f}};
#pragma nounroll
        for (int e = 0; e < a.n_events; ++e) {
          if (a.events[e].kind != KS_EVENT_FORCE_PUSH) continue;
          const KsEventDesc ev = a.events[e];
          float* st = a.event_force + ((int64_t)e * a.N + env) * KS_EVENT_FORCE_STATE;
          float* tleft = a.event_state + (int64_t)e * a.N + env;
          float s7[7];
#pragma unroll
          for (int k = 0; k < 7; ++k) s7[k] = lane_bcast(lane == 0 ? st[k] : 0.f, 0);
          float dur = s7[0] - m.dt, left = lane_bcast(lane == 0 ? *tleft : 0.f, 0) - m.dt;
#pragma unroll
          for (int k = 0; k < 6; ++k) s7[1 + k] *= ev.level_scale;   // events.py:296: the carried wrench itself is rescaled
          const bool on = dur > 0.f && lane == ev.body;                // events.py:297-299, 302-307
          const V3 f = {s7[1] * ev.level_scale, s7[2] * ev.level_scale, s7[3] * ev.level_scale};
          const V3 tq = {s7[4] * ev.level_scale, s7[5] * ev.level_scale, s7[6] * ev.level_scale};
          const V3 mom = tq + cross(xipos - com, f);                    // moment about the centre of mass of the tree
          ext = {{on ? mom.x : 0.f, on ? mom.y : 0.f, on ? mom.z : 0.f}, {on ? f.x : 0.f, on ? f.y : 0.f, on ? f.z : 0.f}};
          if (left <= 0.f) {  // wave-uniform: a new wrench (events.py:320-358)
            float u[10];
            if (a.event_uniform) {
              const float* up = a.event_uniform + (((int64_t)sub * a.N + env) * a.n_events + e) * KS_EVENT_DRAWS;
#pragma unroll
              for (int k = 0; k < 10; ++k) u[k] = up[k];
            } else {
#pragma unroll
              for (int q = 0; q < 3; ++q) {
                const Philox4 r = draw(a.event_rng.seed, ev_step, kRngEvent, (uint64_t)env, (uint32_t)((sub * KS_MAX_EVENTS + e) * 4 + 1 + q));
                u[4 * q] = u01(r.x); u[4 * q + 1] = u01(r.y);
                if (q < 2) { u[4 * q + 2] = u01(r.z); u[4 * q + 3] = u01(r.w); }
              }
            }
            const V3 d0 = {2.f * u[0] - 1.f, 2.f * u[1] - 1.f, 2.f * u[2] - 1.f}, d1 = {2.f * u[4] - 1.f, 2.f * u[5] - 1.f, 2.f * u[6] - 1.f};
            const float sc = ev.lo + u[3] * (ev.hi - ev.lo);
            const float kf = sc * ev.mag / sqrtf(dot(d0, d0)), kt = sc * ev.mag2 / sqrtf(dot(d1, d1));
            const int which = min(2, (int)(3.f * u[7]));
            const float wf = which == 1 ? 0.f : kf, wt = which == 0 ? 0.f : kt;
            s7[1] = d0.x * wf; s7[2] = d0.y * wf; s7[3] = d0.z * wf;
            s7[4] = d1.x * wt; s7[5] = d1.y * wt; s7[6] = d1.z * wt;
            left = ev.interval_lo + u[8] * (ev.interval_hi - ev.interval_lo);
            dur = ev.duration_lo + u[9] * (ev.duration_hi - ev.duration_lo);
          }
          if (lane == 0) {
            *tleft = left;
            st[0] = dur;
#pragma unroll
            for (int k = 1; k < 7; ++k) st[k] = s7[k];
          }
        }
        cf = {cf.a - ext.a, cf.l - ext.l};
      }
      if (is_body) {
        st6(l.cvel + 6 * lane, v);
        st6(l.cfrc + 6 * lane, cf);
      }
    }
    KS_SYNC();
    for (int idx = lane; idx < nb * 6; idx += 64) {
      const int b = idx / 6, k = idx - 6 * b;
      l.fsub[idx] = b > 0 ? range_sum(l.cfrc + k, 6, b, l.sub_end[b]) : 0.f;
    }
    KS_SYNC();

    KS_PHASE(4)
    // ---- mass-matrix row into registers; smooth forces: passive - bias + actuator
    const float* Mrow = l.M + (is_dof ? lane : 0) * nvs;
    float qfs = 0.f, my_qvel = 0.f;
    if (is_dof) {
      my_qvel = l.qvel[lane];
      const float bias = dot(my_cdof, ld6(l.fsub + 6 * d_body));
      float f = -d_damping * my_qvel - bias;
      if (rec.d_stiffness != 0.f) f -= rec.d_stiffness * (l.qpos[rec.d_qadr] - m.qpos0[rec.d_qadr]);  // joint spring about qpos0
      if (d_act >= 0) f += d_gear * fminf(fmaxf(l.tau[d_act], d_lo), d_hi);
      qfs = f;
      if (a.dbg_bias) a.dbg_bias[env * nv + lane] = bias;
#ifndef KS_PROFILE
      if (a.dbg_M) for (int j = 0; j < nv; ++j) a.dbg_M[env * nv * nv + lane * nv + j] = l.M[lane * nvs + j];
#endif
    }

    KS_PHASE(5)
    // ---- contacts: sphere vs plane z = 0, compacted to the penetrating ones
    float dist = 1.f;
    V3 cpos = {0.f, 0.f, 0.f};
    if (is_sph) {
      const Mat3 Rb = q2mat({l.xquat[4 * s_body], l.xquat[4 * s_body + 1], l.xquat[4 * s_body + 2], l.xquat[4 * s_body + 3]});
      const float* R = Rb.m;
      const V3 c = ld3(l.xpos + 3 * s_body) + V3{R[0] * s_pos.x + R[1] * s_pos.y + R[2] * s_pos.z,
                                                R[3] * s_pos.x + R[4] * s_pos.y + R[5] * s_pos.z,
                                                R[6] * s_pos.x + R[7] * s_pos.y + R[8] * s_pos.z};
      dist = c.z - s_rad;
      cpos = {c.x, c.y, c.z - s_rad - 0.5f * dist};
      if (a.contact_dist) a.contact_dist[env * ns + lane] = dist;
    }
    const bool touching = is_sph && (dist < 0.f);
    const unsigned long long cmask = __ballot(touching);
    const int ncon = __popcll(cmask);
    const bool frictionless = m.frictionless != 0;
    const int nefc = frictionless ? ncon : 4 * ncon;
    // A launch ends with its slowest wavefront, and an env with many contacts runs several times longer than an airborne
    // one: waves with more constraint rows get a higher issue priority on their SIMD, which shortens exactly those.
    if (nefc >= 20) __builtin_amdgcn_s_setprio(3);
    else if (nefc >= 12) __builtin_amdgcn_s_setprio(2);
    else if (nefc > 0) __builtin_amdgcn_s_setprio(1);
    else __builtin_amdgcn_s_setprio(0);
    if (touching) {
      const int c = __popcll(cmask & ((1ull << lane) - 1ull));
      l.con_body[c] = s_body;
      l.con_mask[c] = s_mask;
      st3(l.con_off + 3 * c, cpos - com);
      const float invweight = frictionless ? s_invw : (s_invw + mu * mu * s_invw) * 2.f * mu * mu / m.impratio;
      const float imp = impedance(m, dist);
      const float Rr = fmaxf(invweight * (1.f - imp) / imp, 1e-15f);
      l.con_D[c] = 1.0f / Rr;
      l.con_kip[c] = m.con_k * imp * dist;
    }
    KS_SYNC();

    KS_PHASE(6)
    // ---- Cholesky of M and the unconstrained acceleration (registers only)
    float R[NP];
    float myinv;
    {
      f32x16 T;
      load_mtile(T, l.M, nvs, nv, NP, lane);
      chol_tile<NP>(T, R, myinv, lane, nv);
    }
    const float qas_all = solve_regs<NP>(R, myinv, lane, qfs, nv);
    const float qas = is_dof ? qas_all : 0.f;  // lanes that hold no row carry meaningless numbers
    if (a.dbg_qacc_smooth && is_dof) a.dbg_qacc_smooth[env * nv + lane] = qas;

    KS_PHASE(7)
    float qacc = qas;
    float Mqacc = qfs;  // M qacc = smooth + constraint force: what the implicit integration step solves against
    int niter = 0;
    // ---- rows on the dof lanes (models with joint limits or dry friction only).  Their Jacobians are unit vectors, so
    // nothing of them is stored: lane j derives J a - aref of its rows from its own qacc wherever the solver needs it.
    DofRows dr = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    int ndr = 0;
    if (DR) {
      int lane_r = threadIdx.x;
      asm volatile("" : "+v"(lane_r));
      const LaneRec* rr = reinterpret_cast<const LaneRec*>(m.lane_rec[lane_r]);
      if (is_dof) {
        if (rr->d_limited) {
          const float q = l.qpos[rr->d_qadr];
          const float dlo = q - rr->d_rlo, dhi = rr->d_rhi - q;
          const float pos = fminf(dlo, dhi);
          if (pos < 0.f) {  // the nearer side, once violated
            dr.lim_s = dlo < dhi ? 1.f : -1.f;
            const float imp = impedance_dof(m, pos);
            dr.lim_D = 1.f / fmaxf(rr->d_invw * (1.f - imp) / imp, 1e-15f);
            dr.lim_aref = -m.dr_b * dr.lim_s * my_qvel - m.dr_k * imp * pos;
          }
        }
        dr.fr_fl = a.frictionloss ? ((rr->d_jtype == kJntHinge) ? a.frictionloss[env * nv + lane] : 0.f) : rr->d_floss;
        dr.fr_D = rr->d_frD;
        dr.fr_rf = dr.fr_fl / dr.fr_D;
        dr.fr_aref = -m.dr_b * my_qvel;
      }
      ndr = __popcll(__ballot(dr.lim_s != 0.f)) + __popcll(__ballot(dr.fr_fl > 0.f));
    }
    if (nefc > 0 || (DR && ndr > 0)) {
      // ---- constraint rows.  Lane j builds column j of J: the motion axis of dof j is one LDS read away, so a contact
      // costs the lane one cross product and its four pyramid edges, written to LDS row-wise (consecutive lanes,
      // consecutive addresses).  The row lanes then take their reference acceleration from a row product with qvel.
      const bool is_row = lane < nefc;
      float aref = 0.f, D = 0.f;
      {
        const bool col = lane < NP;  // the padding columns are written too (zeros): the row products read NP floats
        const Sp cd = ld6(l.cdof + 6 * (is_dof ? lane : 0));
        float* Jc = l.J + (col ? lane : 0);
        for (int k = 0; k < ncon; ++k) {  // wave-uniform
          const V3 off = ld3(l.con_off + 3 * k);
          const bool on = is_dof && ((l.con_mask[k] >> lane) & 1u);
          const V3 jac = cd.l + cross(cd.a, off);
          if (frictionless) {
            if (col) Jc[k * js] = on ? jac.z : 0.f;
          } else if (col) {  // rows of a contact: z + mu y, z - mu y, z - mu x, z + mu x
            Jc[(4 * k) * js] = on ? jac.z + mu * jac.y : 0.f;
            Jc[(4 * k + 1) * js] = on ? jac.z - mu * jac.y : 0.f;
            Jc[(4 * k + 2) * js] = on ? jac.z - mu * jac.x : 0.f;
            Jc[(4 * k + 3) * js] = on ? jac.z + mu * jac.x : 0.f;
          }
        }
        if (frictionless && col)  // whole blocks of four rows are read back below: the tail of the last block is zero
          for (int r = nefc; r < ((nefc + 3) & ~3); ++r) Jc[r * js] = 0.f;
        KS_SYNC();
        if (is_row) {
          const int c = frictionless ? lane : lane >> 2;
          float vv[NP];
          load_row<NP>(l.qvel, vv);
          const float vel = row_dot<NP>(l.J + lane * js, vv);
          aref = -m.con_b * vel - l.con_kip[c];
          D = l.con_D[c];
        }
      }
      const float warm = is_dof ? l.warm[lane] : 0.f;
      KS_SYNC();
      KS_PHASE(8)
      // cost of the warm start and of the unconstrained acceleration; start from the cheaper one
      float Ma_w = 0.f, Ma_s = 0.f, Jar_w = 0.f, Jar_s = 0.f;
      {
        float vv[NP];
        if (lane < 32) l.vbuf[lane] = warm;
        KS_SYNC();
        load_row<NP>(l.vbuf, vv);
        if (is_dof) Ma_w = row_dot<NP>(Mrow, vv);
        if (is_row) Jar_w = row_dot<NP>(l.J + (is_row ? lane : 0) * js, vv) - aref;
        KS_SYNC();
        if (lane < 32) l.vbuf[lane] = qas;
        KS_SYNC();
        load_row<NP>(l.vbuf, vv);
        if (is_dof) Ma_s = row_dot<NP>(Mrow, vv);
        if (is_row) Jar_s = row_dot<NP>(l.J + (is_row ? lane : 0) * js, vv) - aref;
      }
      float drc_w = 0.f, drc_s = 0.f;
      if (DR) {
        float f_, h_;
        int z_;
        drc_w = dofrow_eval(dr, warm, f_, h_, z_);
        drc_s = dofrow_eval(dr, qas, f_, h_, z_);
      }
      const float cost_w = wave_sum(((is_row && Jar_w < 0.f) ? 0.5f * D * Jar_w * Jar_w : 0.f) + drc_w) +
                           0.5f * wave_sum(is_dof ? (Ma_w - qfs) * (warm - qas) : 0.f);
      const float cost_s = wave_sum(((is_row && Jar_s < 0.f) ? 0.5f * D * Jar_s * Jar_s : 0.f) + drc_s);
      const bool use_warm = cost_w < cost_s;
      qacc = use_warm ? warm : qas;
      float Ma = use_warm ? Ma_w : Ma_s;
      float Jaref = use_warm ? Jar_w : Jar_s;
      float cost = use_warm ? cost_w : cost_s;
      float prev_cost = INFINITY;
      bool first = true;
      KS_PHASE(9)
      unsigned long long am_factored = 0ull;  // active set that R currently factors
      unsigned long long amd_factored = 0ull; // and the quadratic zones of the dof-lane rows
      bool have_factor = false;               // none yet: R holds the factor of M
      while (true) {
        // ---- constraint update: active set, forces, cost
        const bool active = is_row && (Jaref < 0.f);
        const float force = active ? -D * Jaref : 0.f;
        unsigned long long am = __ballot(active);
        float qfc = 0.f;
        if (nefc <= 32) {
          // J^T f with the rows split between the lane halves: the forces go through LDS (one 16-byte broadcast read per
          // block of four rows), lane j of half h sums the blocks 2 i + h of column j, and the halves meet at the end.
          if (lane < 32) l.vbuf[lane] = force;  // zero beyond the rows and on the inactive ones
          KS_SYNC();
          const int jc = (lane & 31) < nv ? (lane & 31) : 0, hh = lane >> 5;
          const int nblk = (nefc + 3) >> 2;
          for (int b0 = 0; b0 < nblk; b0 += 2) {
            const bool ok = b0 + hh < nblk;
            const int bb = ok ? b0 + hh : 0;
            const float4 f = *reinterpret_cast<const float4*>(l.vbuf + 4 * bb);
            const float* Jb = l.J + (4 * bb) * js + jc;
            const float sblk = (Jb[0] * f.x + Jb[js] * f.y) + (Jb[2 * js] * f.z + Jb[3 * js] * f.w);
            qfc += ok ? sblk : 0.f;
          }
          qfc += __shfl_xor(qfc, 32);
        } else {
          for (unsigned long long t = am; t; t &= t - 1) {
            const int r = __builtin_ctzll(t);
            qfc += l.J[r * js + (lane < nv ? lane : 0)] * lane_bcast(force, r);
          }
        }
        float dr_cost = 0.f, dr_force = 0.f, dr_h = 0.f;
        unsigned long long amd = 0ull;
        if (DR) {
          int zone;
          dr_cost = dofrow_eval(dr, qacc, dr_force, dr_h, zone);
          qfc += dr_force;
          amd = (__ballot(zone & 1) & 0xffffffffull) | (__ballot(zone & 2) << 32);
        }
        if (!is_dof) qfc = 0.f;
        const float gauss = 0.5f * wave_sum(is_dof ? (Ma - qfs) * (qacc - qas) : 0.f);
        if (!first) {
          prev_cost = cost;
          cost = wave_sum((active ? 0.5f * D * Jaref * Jaref : 0.f) + dr_cost) + gauss;
        }
        first = false;
        // ---- gradient; stop before paying for another Hessian when the solver is done
        const float grad = is_dof ? Ma - qfs - qfc : 0.f;
        const float improvement = scale * (prev_cost - cost);
        const float gradient = scale * sqrtf(wave_sum(grad * grad));
        bool done = niter >= m.iterations;
        done |= improvement < m.tolerance;
        done |= gradient < m.tolerance;
        if (done && !(m.iterations == 1 && niter == 0)) break;
        KS_PHASE(10)
        // ---- Newton direction: H = M + J^T diag(D active) J.  The rank-nefc term runs on the matrix cores: one
        // 32x32x2 fp32 MFMA per pair of constraint rows, operands straight from the LDS copy of J (lane = column,
        // lane half = row of the pair).  The accumulator tile holds, in lane c, rows {8g + 4 (lane / 32) + e} of
        // column c, which by symmetry is row c: the upper lane half hands its 16 entries to the lower one and
        // lane i < 32 ends up with row i of H in registers, as the factorisation wants it.
        // H depends on the iterate only through the active set: while that stays the same (the usual case once the
        // solver closes in) the factor of the previous iteration is still the factor of H and is kept.
        if (!have_factor || am != am_factored || (DR && amd != amd_factored)) {
          l.drow[lane] = active ? D : 0.f;
          KS_SYNC();
          f32x16 hc;
          load_mtile(hc, l.M, nvs, nv, NP, lane);
          const int col = lane & 31, half = lane >> 5;
          const bool col_ok = NP == 32 || col < NP;
          for (int r0 = 0; r0 < nefc; r0 += 2) {
            const int r = r0 + half;
            const float jv = (col_ok && r < nefc) ? l.J[r * js + col] : 0.f;
            hc = __builtin_amdgcn_mfma_f32_32x32x2f32(l.drow[r] * jv, jv, hc, 0, 0, 0);
          }
          if (DR) {  // unit-vector rows add their stiffness to the diagonal
            const float hd = __shfl(dr_h, col);
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
              for (int e = 0; e < 4; ++e) hc[4 * g + e] += (8 * g + 4 * half + e == col) ? hd : 0.f;
          }
          KS_PHASE(11)
          chol_tile<NP>(hc, R, myinv, lane, nv);
          am_factored = am;
          amd_factored = amd;
          have_factor = true;
        }
        const float search_all = -solve_regs<NP>(R, myinv, lane, grad, nv);
        const float search = is_dof ? search_all : 0.f;
        KS_PHASE(12)
        // ---- exact line search along `search`
        float mv = 0.f, jv = 0.f;
        {
          float vv[NP];
          KS_SYNC();
          if (lane < 32) l.vbuf[lane] = search;
          KS_SYNC();
          load_row<NP>(l.vbuf, vv);
          if (is_dof) mv = row_dot<NP>(Mrow, vv);
          if (is_row) jv = row_dot<NP>(l.J + (is_row ? lane : 0) * js, vv);
        }
        const float smag = sqrtf(wave_sum(search * search)) * m.meaninertia * (float)(nv > 1 ? nv : 1);
        const float gtol = m.tolerance * m.ls_tolerance * smag;
        const float q0r = 0.5f * Jaref * Jaref * D, q1r = jv * Jaref * D, q2r = 0.5f * jv * jv * D;
        const float g0 = gauss;
        const float g1 = wave_sum(is_dof ? search * (Ma - qfs) : 0.f);
        const float g2 = 0.5f * wave_sum(is_dof ? search * mv : 0.f);
        // With at most 16 constraint rows the three sums of a cost evaluation share one reduction: the 16-lane
        // groups 0, 1, 2 hold copies of the rows with the constant, linear and quadratic coefficient, and one
        // DPP reduction within the groups yields all three totals.
        // Rows 16..31 ride along as a second copy in the same lanes, so up to 32 rows need no more reduction steps.
        const bool packed = nefc <= 32, two = nefc > 16;
        float pk_j = 0.f, pk_jv = 0.f, pk_q = 0.f, pk_j2 = 0.f, pk_jv2 = 0.f, pk_q2 = 0.f;
        const int grp = lane >> 4;
        if (packed) {
          const int r = lane & 15;
          pk_j = __shfl(Jaref, r);
          pk_jv = __shfl(jv, r);
          const float c0 = __shfl(q0r, r), c1 = __shfl(q1r, r), c2 = __shfl(q2r, r);
          pk_q = grp == 0 ? c0 : (grp == 1 ? c1 : (grp == 2 ? c2 : 0.f));
          if (two) {
            pk_j2 = __shfl(Jaref, 16 + r);
            pk_jv2 = __shfl(jv, 16 + r);
            const float e0 = __shfl(q0r, 16 + r), e1 = __shfl(q1r, 16 + r), e2 = __shfl(q2r, 16 + r);
            pk_q2 = grp == 0 ? e0 : (grp == 1 ? e1 : (grp == 2 ? e2 : 0.f));
          }
        }
        auto point = [&](float alpha) {
          float q0, q1, q2;
          if (packed) {
            float x = (pk_j + alpha * pk_jv < 0.f) ? pk_q : 0.f;  // rows beyond nefc carry zeros
            if (two) x += (pk_j2 + alpha * pk_jv2 < 0.f) ? pk_q2 : 0.f;
            if (DR && ndr > 0) {
              // The rows on the dof lanes join the same reduction.  Lane j < 32 holds the three coefficients of its own rows:
              // the constant one belongs in group 0, the linear one in group 1, so each lane keeps the one of its own group
              // and swaps the other with the lane 16 away; the quadratic ones go to the upper lane half (groups 2 and 3).
              float t0, t1, t2;
              dofrow_quad(dr, qacc, search, alpha, t0, t1, t2);
              const float got = __shfl_xor(grp == 0 ? t1 : t0, 16);
              const float up = __shfl(t2, lane & 31);
              x += grp == 0 ? t0 + got : (grp == 1 ? t1 + got : up);
            }
            x += dpp_shift<0x111, 0xf>(x);
            x += dpp_shift<0x112, 0xf>(x);
            x += dpp_shift<0x114, 0xf>(x);
            x += dpp_shift<0x118, 0xf>(x);  // lane 15 of each 16-lane group holds the group's total
            q0 = g0 + lane_bcast(x, 15);
            q1 = g1 + lane_bcast(x, 31);
            q2 = g2 + lane_bcast(x, 47) + (DR ? lane_bcast(x, 63) : 0.f);
          } else {
            const bool on = is_row && (Jaref + alpha * jv < 0.f);
            q0 = g0 + wave_sum(on ? q0r : 0.f);
            q1 = g1 + wave_sum(on ? q1r : 0.f);
            q2 = g2 + wave_sum(on ? q2r : 0.f);
          }
          if (DR && ndr > 0 && !packed) {
            float t0, t1, t2;
            dofrow_quad(dr, qacc, search, alpha, t0, t1, t2);
            q0 += wave_sum(t0);
            q1 += wave_sum(t1);
            q2 += wave_sum(t2);
          }
          LsPoint p;
          p.alpha = alpha;
          p.cost = alpha * alpha * q2 + alpha * q1 + q0;
          p.d0 = 2.f * alpha * q2 + q1;
          p.d1 = 2.f * q2 + (q2 == 0.f ? 1e-15f : 0.f);
          return p;
        };
        const LsPoint p0 = point(0.f);
        // Newton estimates of the step length: d0 / d1 by reciprocal and product (1 ulp), a tenth of an IEEE division's instructions
        auto newton_alpha = [](const LsPoint& x) { return x.alpha - x.d0 * __builtin_amdgcn_rcpf(x.d1); };
        LsPoint lo = point(newton_alpha(p0));
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
          const LsPoint lo_next = point(newton_alpha(lo));
          const LsPoint hi_next = point(newton_alpha(hi));
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
        ++niter;
        KS_PHASE(13)
      }
      Mqacc = Ma;
      // ---- Cartesian contact forces on the bodies (mjData.cfrc_ext), only when asked for: a pyramid row with force f
      // pushes along normal +- mu tangent (rows of a contact: z + mu y, z - mu y, z - mu x, z + mu x)
      if (a.cfrc_ext && sub == nsub - 1) {
        const float f = (is_row && Jaref < 0.f) ? -D * Jaref : 0.f;
        const int q = lane & 3;
        float fx = 0.f, fy = 0.f, fz = f;
        if (!frictionless) {
          fx = q == 3 ? mu * f : (q == 2 ? -mu * f : 0.f);
          fy = q == 0 ? mu * f : (q == 1 ? -mu * f : 0.f);
          fx += __shfl_xor(fx, 1); fy += __shfl_xor(fy, 1); fz += __shfl_xor(fz, 1);
          fx += __shfl_xor(fx, 2); fy += __shfl_xor(fy, 2); fz += __shfl_xor(fz, 2);
        }
        KS_SYNC();  // the line search is done with drow
        const int cc = frictionless ? lane : lane >> 2;
        if (is_row && (frictionless || q == 0)) { l.drow[3 * cc] = fx; l.drow[3 * cc + 1] = fy; l.drow[3 * cc + 2] = fz; }
        KS_SYNC();
        if (lane < nb) {
          Sp w = {{0.f, 0.f, 0.f}, {0.f, 0.f, 0.f}};
          for (int k = 0; k < ncon; ++k)
            if (l.con_body[k] == lane) {
              const V3 F = ld3(l.drow + 3 * k);
              w.a = w.a + cross(ld3(l.con_off + 3 * k), F);
              w.l = w.l + F;
            }
          float* dst = a.cfrc_ext + ((int64_t)env * nb + lane) * 6;
          dst[0] = w.a.x; dst[1] = w.a.y; dst[2] = w.a.z; dst[3] = w.l.x; dst[4] = w.l.y; dst[5] = w.l.z;
        }
      }
    } else if (a.cfrc_ext && sub == nsub - 1) {
      for (int i = lane; i < nb * 6; i += 64) a.cfrc_ext[(int64_t)env * nb * 6 + i] = 0.f;
    }
    work += (1 + niter) * (16 + nefc + ndr);
    if (sub == nsub - 1) {  // outputs of the last substep go out here: nothing of them stays live to the end
      if (a.qacc && lane < nv) a.qacc[env * nv + lane] = qacc;
      if (a.solver_niter && lane == 0) a.solver_niter[env] = niter;
      if (a.nefc && lane == 0) a.nefc[env] = nefc + ndr;
    }
    KS_SYNC();
    if (is_dof) l.warm[lane] = qacc;

    KS_PHASE(14)
    // ---- semi-implicit Euler
    if (!fwd) {
      // What this stage needs of the lane's constants is read again here (through an opaque lane id, so that the loads
      // are not merged with those at the top of the substep): nothing of it stays live across the solver.
      int lane_e = threadIdx.x;
      asm volatile("" : "+v"(lane_e));
      const LaneRec* rec_e = reinterpret_cast<const LaneRec*>(m.lane_rec[lane_e]);
      const int b_jtype = rec_e->b_jtype, b_qadr = rec_e->b_qadr, b_dofadr = rec_e->b_dofadr;
      const float d_damping = rec_e->d_damping * ((a.damping_scale && lane_e < nv) ? a.damping_scale[env * nv + lane_e] : 1.f);
      const float my_qvel = lane_e < nv ? l.qvel[lane_e] : 0.f;
      float qacc_int = qacc;
      if (m.eulerdamp) {
        // implicit in the joint damping: (M + dt diag(damping)) a = M qacc.  For torque motors, whose force does
        // not depend on velocity, this is MuJoCo's implicitfast step; qacc itself (warm start, output) is unchanged.
        f32x16 T;
        load_mtile(T, l.M, nvs, nv, NP, lane);
        const int c = lane & 31, half = lane >> 5;
        const float hd = m.dt * __shfl(is_dof ? d_damping : 0.f, c);
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
          for (int e = 0; e < 4; ++e) T[4 * g + e] += (8 * g + 4 * half + e == c) ? hd : 0.f;
        float R2[NP];
        float inv2;
        chol_tile<NP>(T, R2, inv2, lane, nv);
        const float sol = solve_regs<NP>(R2, inv2, lane, is_dof ? Mqacc : 0.f, nv);
        qacc_int = is_dof ? sol : 0.f;
      }
      if (is_dof) l.qvel[lane] = my_qvel + m.dt * qacc_int;
      KS_SYNC();
      if (is_body) {
        const int qa = b_qadr, da = b_dofadr;
        if (b_jtype == kJntFree) {
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
        } else if (b_jtype == kJntHinge) {
          l.qpos[qa] += m.dt * l.qvel[da];
        }
      }
    }
    KS_SYNC();
  }

  KS_PHASE(15)
#ifdef KS_PROFILE
  if (a.dbg_M && lane == 0) for (int k = 0; k < 16; ++k) a.dbg_M[env * nv * nv + k] = prof[k];
#endif
  // ---- write back
  if (!FWD) {
    for (int i = lane; i < nq; i += 64) a.qpos[env * nq + i] = l.qpos[i];
    if (lane < nv) a.qvel[env * nv + lane] = l.qvel[lane];
    if (a.work && lane == 0) a.work[env] = work;
    if (a.time && lane == 0) {  // dt added once per substep in fp32, like the reference's accumulation
      float time = a.time[env];
      for (int k = 0; k < nsub; ++k) time += m.dt;
      a.time[env] = time;
    }
    if (a.last_ctrl) {
      const int na = a.actuator_type == KS_ACT_POSITION_VELOCITY ? 2 * nu : nu;
      for (int i = lane; i < na; i += 64) a.last_ctrl[env * na + i] = a.action[env * na + i];
    }
  }
  if (a.qacc_warmstart && lane < nv) a.qacc_warmstart[env * nv + lane] = l.warm[lane];
  if (a.ctrl_out) for (int i = lane; i < nu; i += 64) a.ctrl_out[env * nu + i] = l.tau[i];
  if (a.xpos) for (int i = lane; i < nb * 3; i += 64) a.xpos[env * nb * 3 + i] = l.xpos[i];
  if (a.xquat) for (int i = lane; i < nb * 4; i += 64) a.xquat[env * nb * 4 + i] = l.xquat[i];
  if (a.cvel) for (int i = lane; i < nb * 6; i += 64) a.cvel[env * nb * 6 + i] = l.cvel[i];
  if (a.traj_ctrl) for (int i = lane; i < nu; i += 64) a.traj_ctrl[env * nu + i] = l.tau[i];
  if (a.traj_xpos) for (int i = lane; i < nb * 3; i += 64) a.traj_xpos[env * nb * 3 + i] = l.xpos[i];
  if (a.traj_xquat) for (int i = lane; i < nb * 4; i += 64) a.traj_xquat[env * nb * 4 + i] = l.xquat[i];
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
  if (d->condim != 0 && d->condim != 1 && d->condim != 3) return fail(KS_EINVAL, "ks_model_create: condim %d (1 or 3)", d->condim);
  if (!(d->dt > 0.0)) return fail(KS_EINVAL, "ks_model_create: dt must be positive");
  KsModel* km = new KsModel();
  DevModel& m = km->host;
  std::memset(&m, 0, sizeof(m));
  m.nb = d->nb; m.nq = d->nq; m.nv = d->nv; m.nu = d->nu; m.ns = d->ns;
  m.iterations = d->iterations; m.ls_iterations = d->ls_iterations; m.eulerdamp = d->eulerdamp;
  m.frictionless = d->condim == 1 ? 1 : 0;
  m.nvs = m_stride(d->nv);
  m.js = j_stride(d->nv);
  m.dt = (float)d->dt;
  for (int k = 0; k < 3; ++k) m.gravity[k] = (float)d->gravity[k];
  m.tolerance = (float)d->tolerance; m.ls_tolerance = (float)d->ls_tolerance;
  m.meaninertia = (float)d->meaninertia; m.friction = (float)d->friction; m.impratio = (float)d->impratio;
  {  // solref / solimp -> (k, b) and clamped impedance parameters, for the contact rows and for the dof-lane rows
    auto convert = [&](const double* solref, const double* solimp, float* out /*k b dmin dmax width mid power imp_a imp_b*/) {
      double timeconst = solref[0], dampratio = solref[1];
      double dmin = solimp[0], dmax = solimp[1], width = solimp[2], mid = solimp[3], power = solimp[4];
      if (timeconst < 2 * d->dt) timeconst = 2 * d->dt;
      auto clampd = [](double x, double lo, double hi) { return x < lo ? lo : (x > hi ? hi : x); };
      dmin = clampd(dmin, 1e-4, 0.9999); dmax = clampd(dmax, 1e-4, 0.9999);
      width = width < 1e-15 ? 1e-15 : width; mid = clampd(mid, 1e-4, 0.9999); power = power < 1 ? 1 : power;
      double k = 1.0 / (dmax * dmax * timeconst * timeconst * dampratio * dampratio), b = 2.0 / (dmax * timeconst);
      if (solref[0] <= 0) k = -solref[0] / (dmax * dmax);
      if (solref[1] <= 0) b = -solref[1] / dmax;
      out[0] = (float)k; out[1] = (float)b; out[2] = (float)dmin; out[3] = (float)dmax; out[4] = (float)width;
      out[5] = (float)mid; out[6] = (float)power;
      out[7] = (float)(1.0 / std::pow(mid, power - 1.0)); out[8] = (float)(1.0 / std::pow(1.0 - mid, power - 1.0));
    };
    float c[9];
    convert(d->solref, d->solimp, c);
    m.con_k = c[0]; m.con_b = c[1]; m.dmin = c[2]; m.dmax = c[3]; m.width = c[4]; m.mid = c[5]; m.power = c[6]; m.imp_a = c[7]; m.imp_b = c[8];
    bool own = false;
    for (int k = 0; k < 2; ++k) own |= d->dof_solref[k] != 0.0;
    for (int k = 0; k < 5; ++k) own |= d->dof_solimp[k] != 0.0;
    if (own) convert(d->dof_solref, d->dof_solimp, c);
    m.dr_k = c[0]; m.dr_b = c[1]; m.dr_dmin = c[2]; m.dr_dmax = c[3]; m.dr_width = c[4]; m.dr_mid = c[5]; m.dr_power = c[6];
    m.dr_imp_a = c[7]; m.dr_imp_b = c[8];
  }
  for (int b = 0; b < d->nb; ++b) {
    m.body_parent[b] = d->body_parent[b]; m.body_jtype[b] = d->body_jtype[b]; m.body_qadr[b] = d->body_qadr[b];
    m.body_dofadr[b] = d->body_dofadr[b]; m.body_subtree_end[b] = d->body_subtree_end[b];
    if (b > 0 && (d->body_parent[b] < 0 || d->body_parent[b] >= b)) { delete km; return fail(KS_EINVAL, "ks_model_create: body %d has parent %d (must precede it)", b, d->body_parent[b]); }
    if (d->body_subtree_end[b] <= b || d->body_subtree_end[b] > d->nb) { delete km; return fail(KS_EINVAL, "ks_model_create: bad subtree_end for body %d", b); }
    if (b > 0 && d->body_jtype[b] != kJntFree && d->body_jtype[b] != kJntHinge) { delete km; return fail(KS_EINVAL, "ks_model_create: body %d needs a free or hinge joint", b); }
    if (b > 0) {  // the joint's coordinates and dofs must lie inside qpos / qvel: the kernel and the tables below index with them
      const int nqj = d->body_jtype[b] == kJntFree ? 7 : 1, nvj = d->body_jtype[b] == kJntFree ? 6 : 1;
      if (d->body_qadr[b] < 0 || d->body_qadr[b] + nqj > d->nq || d->body_dofadr[b] < 0 || d->body_dofadr[b] + nvj > d->nv) {
        delete km;
        return fail(KS_EINVAL, "ks_model_create: body %d has qpos address %d and dof address %d outside nq=%d / nv=%d", b,
                    d->body_qadr[b], d->body_dofadr[b], d->nq, d->nv);
      }
    }
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
    if (n > m.max_depth) m.max_depth = n;
    for (int k = 0; k < n; ++k) m.body_chain[b][k] = chain[n - 1 - k];
  }
  for (int q = 0; q < d->nq; ++q) m.qpos0[q] = (float)d->qpos0[q];
  for (int j = 0; j < d->nv; ++j) {
    m.dof_body[j] = d->dof_body[j]; m.dof_parent[j] = d->dof_parent[j]; m.dof_act[j] = -1;
    m.dof_damping[j] = (float)d->dof_damping[j]; m.dof_armature[j] = (float)d->dof_armature[j];
    if (d->dof_parent[j] >= j || d->dof_body[j] < 1 || d->dof_body[j] >= d->nb) { delete km; return fail(KS_EINVAL, "ks_model_create: bad dof %d", j); }
  }
  for (int b = 1; b < d->nb; ++b) {
    if (!d->jnt_limited[b]) continue;
    if (d->body_jtype[b] != kJntHinge) { delete km; return fail(KS_EINVAL, "ks_model_create: body %d: only hinges can be limited", b); }
    if (!(d->jnt_range[b][0] < d->jnt_range[b][1])) { delete km; return fail(KS_EINVAL, "ks_model_create: body %d: empty joint range", b); }
    if (!(d->dof_invweight0[d->body_dofadr[b]] > 0.0)) { delete km; return fail(KS_EINVAL, "ks_model_create: body %d: a limited joint needs dof_invweight0 > 0", b); }
    m.dofrows = 1;
  }
  m.invw_ok = 1;
  for (int j = 0; j < d->nv; ++j)
    if (d->body_jtype[d->dof_body[j]] == kJntHinge && !(d->dof_invweight0[j] > 0.0)) m.invw_ok = 0;
  for (int j = 0; j < d->nv; ++j) {
    if (d->dof_frictionloss[j] == 0.0) continue;
    if (!(d->dof_frictionloss[j] > 0.0) || d->body_jtype[d->dof_body[j]] != kJntHinge) { delete km; return fail(KS_EINVAL, "ks_model_create: dof %d: frictionloss must be positive and on a hinge", j); }
    if (!(d->dof_invweight0[j] > 0.0)) { delete km; return fail(KS_EINVAL, "ks_model_create: dof %d: dry friction needs dof_invweight0 > 0", j); }
    m.dofrows = 1;
    ++m.nfriction;
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
  for (int L = 0; L < 64; ++L) {
    LaneRec r;
    std::memset(&r, 0, sizeof(r));
    const bool is_body = L > 0 && L < d->nb;
    const int bl = is_body ? L : 0;
    r.b_parent = m.body_parent[bl]; r.b_jtype = m.body_jtype[bl]; r.b_qadr = m.body_qadr[bl]; r.b_dofadr = m.body_dofadr[bl];
    r.b_depth = is_body ? m.body_depth[bl] : -1;
    r.b_q0 = (is_body && r.b_jtype == kJntHinge) ? m.qpos0[r.b_qadr] : 0.f;
    r.b_mass = m.body_mass[bl];
    for (int k = 0; k < 3; ++k) {
      r.b_pos[k] = m.body_pos[bl][k]; r.b_ipos[k] = m.body_ipos[bl][k]; r.b_inertia[k] = m.body_inertia[bl][k];
      r.b_jaxis[k] = m.jnt_axis[bl][k]; r.b_jpos[k] = m.jnt_pos[bl][k];
    }
    for (int k = 0; k < 4; ++k) { r.b_quat[k] = m.body_quat[bl][k]; r.b_iquat[k] = m.body_iquat[bl][k]; }
    const bool is_dof = L < d->nv;
    const int dl = is_dof ? L : 0;
    r.d_body = d->nv > 0 ? m.dof_body[dl] : 0;
    r.d_act = is_dof ? m.dof_act[dl] : -1;
    r.d_jtype = m.body_jtype[r.d_body];
    r.d_k = dl - m.body_dofadr[r.d_body];
    r.d_damping = m.dof_damping[dl]; r.d_armature = m.dof_armature[dl];
    r.d_stiffness = 0.f;
    const int ua = r.d_act >= 0 ? r.d_act : 0;
    r.d_gear = m.act_gear[ua]; r.d_lo = m.act_lo[ua]; r.d_hi = m.act_hi[ua];
    r.d_limited = 0; r.d_qadr = 0; r.d_rlo = 0.f; r.d_rhi = 0.f; r.d_invw = 0.f; r.d_floss = 0.f; r.d_frD = 0.f;
    if (is_dof && r.d_jtype == kJntHinge) {
      r.d_limited = d->jnt_limited[r.d_body] != 0;
      r.d_qadr = m.body_qadr[r.d_body];
      r.d_stiffness = (float)d->dof_stiffness[dl];
      r.d_rlo = (float)d->jnt_range[r.d_body][0]; r.d_rhi = (float)d->jnt_range[r.d_body][1];
      r.d_invw = (float)d->dof_invweight0[dl];
      r.d_floss = (float)d->dof_frictionloss[dl];
      const double imp0 = m.dr_dmin;  // impedance at pos = 0
      r.d_frD = (float)(1.0 / std::max(d->dof_invweight0[dl] * (1.0 - imp0) / imp0, 1e-15));
    }
    const int sl = L < d->ns ? L : 0;
    r.s_body = m.sph_body[sl]; r.s_rad = m.sph_radius[sl]; r.s_invw = m.body_invweight0[r.s_body];
    for (int k = 0; k < 3; ++k) r.s_pos[k] = m.sph_pos[sl][k];
    r.s_mask = m.body_dofmask[r.s_body];
    for (int k = 0; k < kMaxPairs / 64 + 1; ++k) {
      const int p = L + 64 * k;
      r.pk[k] = p < m.npairs ? ((int)m.pair_i[p] << 8) | (int)m.pair_j[p] : -1;
    }
    std::memcpy(m.lane_rec[L], &r, sizeof(r));
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
  a.friction = io->friction; a.mass_scale = io->mass_scale; a.env_mask = io->env_mask; a.fresh = io->fresh;
  a.qacc = io->qacc; a.ctrl_out = io->ctrl_out; a.xpos = io->xpos; a.xquat = io->xquat; a.cvel = io->cvel;
  a.traj_ctrl = io->traj_ctrl; a.traj_xpos = io->traj_xpos; a.traj_xquat = io->traj_xquat;
  a.solver_niter = io->solver_niter; a.nefc = io->nefc;
  a.dbg_M = io->dbg_M; a.dbg_bias = io->dbg_bias; a.dbg_qacc_smooth = io->dbg_qacc_smooth;
  a.contact_dist = io->contact_dist; a.cinert = io->cinert; a.cfrc_ext = io->cfrc_ext;
  a.armature_scale = io->armature_scale; a.damping_scale = io->damping_scale;
  a.frictionloss = io->frictionloss; a.body_ipos = io->body_ipos; a.body_inertia = io->body_inertia;
  a.sph_pos = io->sph_pos; a.sph_radius = io->sph_radius;
  if ((io->sph_pos == nullptr) != (io->sph_radius == nullptr)) return fail(KS_EINVAL, "ks_step: sph_pos and sph_radius come together");
  if (io->frictionloss && !m.invw_ok) return fail(KS_EINVAL, "ks_step: per-env frictionloss needs dof_invweight0 > 0 on every hinge");
  a.env_order = forward_only ? nullptr : io->env_order; a.work = io->work;
  a.ctrl_in = io->ctrl_in;
  if (!forward_only) {
    if (io->substeps < 1 || io->substeps > 64) return fail(KS_EINVAL, "ks_step: substeps must be in 1..64");
    if (io->actuator_period < 1) return fail(KS_EINVAL, "ks_step: actuator_period must be >= 1");
    if (m.nu > 0 && (!io->action || !io->last_ctrl)) return fail(KS_EINVAL, "ks_step: action and last_ctrl are required");
    if (io->actuator_type < KS_ACT_TORQUE || io->actuator_type > KS_ACT_POSITION_VELOCITY)
      return fail(KS_EINVAL, "ks_step: unknown actuator type %d", io->actuator_type);
    if (io->actuator_type != KS_ACT_TORQUE && m.nu > 0 && (!io->kp || !io->kd || !io->ctrl_clip))
      return fail(KS_EINVAL, "ks_step: position actuators need kp, kd and ctrl_clip");
    if (io->actuator_type != KS_ACT_TORQUE && m.nu + (m.body_jtype[1] == kJntFree ? 7 : 0) > m.nq)
      return fail(KS_EINVAL, "ks_step: position actuators assume one actuator per joint after the root");
    a.substeps = io->substeps; a.actuator_period = io->actuator_period; a.actuator_type = io->actuator_type;
    a.action = io->action; a.last_ctrl = io->last_ctrl; a.latency = io->latency; a.zero_offset = io->zero_offset;
    a.drop = io->drop; a.kp = io->kp; a.kd = io->kd; a.ctrl_clip = io->ctrl_clip;
    a.kp_scale = io->kp_scale; a.kd_scale = io->kd_scale; a.torque_limit_scale = io->torque_limit_scale;
    a.action_scale = io->action_scale;
    a.action_noise = io->action_noise; a.torque_noise = io->torque_noise; a.action_bias = io->action_bias;
    a.torque_bias = io->torque_bias;
    if (io->n_events < 0 || io->n_events > KS_MAX_EVENTS) return fail(KS_ELIMIT, "ks_step: %d events (0..%d)", io->n_events, KS_MAX_EVENTS);
    if (io->n_events > 0) {
      if (!io->event_state) return fail(KS_EINVAL, "ks_step: events need event_state");
      for (int e = 0; e < io->n_events; ++e) {
        const KsEventDesc& ev = io->events[e];
        if (ev.kind < KS_EVENT_LINEAR_PUSH || ev.kind > KS_EVENT_FORCE_PUSH)
          return fail(KS_EINVAL, "ks_step: event %d: unknown kind %d", e, ev.kind);
        if (ev.kind == KS_EVENT_FORCE_PUSH) {
          if (ev.body < 1 || ev.body >= m.nb) return fail(KS_EINVAL, "ks_step: event %d: body %d outside 1..%d", e, ev.body, m.nb - 1);
          if (!io->event_force) return fail(KS_EINVAL, "ks_step: a force push needs event_force");
          ++a.n_force_events;
        } else if (m.nv < 6 || m.body_jtype[1] != kJntFree) {
          return fail(KS_EINVAL, "ks_step: velocity events push a floating base");
        }
      }
      a.event_force = io->event_force;
      a.n_events = io->n_events;
      for (int e = 0; e < io->n_events; ++e) a.events[e] = io->events[e];
      a.event_state = io->event_state; a.event_uniform = io->event_uniform; a.event_rng = io->event_rng;
    }
  }
  const int bytes = lds_floats(m.nb, m.nq, m.nv, m.nu, m.ns) * 4;
  if (bytes > 160 * 1024) return fail(KS_ELIMIT, "ks_step: model needs %d bytes of LDS", bytes);
  void (*fn)(StepArgs) = nullptr;
  switch (padded_nv(m.nv)) {
#define KS_CASE(W)                                                                                       \
  case W:                                                                                                \
    fn = (m.dofrows || io->frictionloss) ? (forward_only ? step_kernel<true, W, true> : step_kernel<false, W, true>)           \
                   : (forward_only ? step_kernel<true, W, false> : step_kernel<false, W, false>);        \
    break;
    KS_CASE(8) KS_CASE(16) KS_CASE(24) KS_CASE(28) KS_CASE(32)
#undef KS_CASE
    default: return fail(KS_ELIMIT, "ks_step: no kernel for %d dofs", m.nv);
  }
  if (bytes > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return fail(KS_ELAUNCH, "ks_step: cannot raise the LDS limit: %s", hipGetErrorString(e));
  }
  hipLaunchKernelGGL(fn, dim3((unsigned)io->N), dim3(64), bytes, (hipStream_t)stream, a);
  return check_launch("ks_step");
}

extern "C" int ks_step(const KsModel* model, ks_stream_t stream, const KsStepIO* io) {
  return launch_step(model, stream, io, false);
}

extern "C" int ks_forward(const KsModel* model, ks_stream_t stream, const KsStepIO* io) {
  return launch_step(model, stream, io, true);
}

namespace ks {
constexpr int kWorkBuckets = 512, kWorkShift = 2, kWorkThreads = 256;  // buckets of four work units
constexpr int kXcds = 8;  // workgroup b of a launch runs on XCD b % 8, each XCD with an L2 of its own
__device__ __forceinline__ int work_bucket(int w) { return min(max(w, 0) >> kWorkShift, kWorkBuckets - 1); }
// Counting sort of envs by descending work in one workgroup: histogram, suffix sums, scatter.
// With gridDim.x == 8 (N a multiple of 8) workgroup r sorts the envs of region r = [r N / 8, (r + 1) N / 8) and writes them
// to order[r], order[r + 8], ...: the step kernel's workgroup b = r + 8 k then runs on XCD r and finds there only envs of
// region r.  The state rows of neighbouring envs share 128-byte lines (an env's qpos row is 108 bytes); kept inside one XCD
// such a line is fetched into, and written back from, one L2 instead of two.
// Four wavefronts and 4 KB of LDS: in a rollout on several streams this launch has to find room on a CU that another group's
// physics launch fills, and a small workgroup finds it as soon as one wavefront per SIMD has left.
__global__ __launch_bounds__(kWorkThreads) void work_order_kernel(int64_t N, const int32_t* __restrict__ work, int32_t* __restrict__ order) {
  __shared__ int hist[kWorkBuckets];
  __shared__ int scan[kWorkBuckets];
  const int t = threadIdx.x;
  const int regions = gridDim.x, region = blockIdx.x;
  const int64_t n = N / regions, first = region * n;
  for (int b = t; b < kWorkBuckets; b += kWorkThreads) hist[b] = 0;
  __syncthreads();
  for (int64_t i = t; i < n; i += kWorkThreads) atomicAdd(&hist[work_bucket(work[first + i])], 1);
  __syncthreads();
  // inclusive suffix sums (heaviest bucket first) by doubling
  for (int b = t; b < kWorkBuckets; b += kWorkThreads) scan[b] = hist[b];
  __syncthreads();
  for (int off = 1; off < kWorkBuckets; off <<= 1) {
    int v[kWorkBuckets / kWorkThreads];
    for (int k = 0; k < kWorkBuckets / kWorkThreads; ++k) {
      const int b = t + kWorkThreads * k;
      v[k] = scan[b] + (b + off < kWorkBuckets ? scan[b + off] : 0);
    }
    __syncthreads();
    for (int k = 0; k < kWorkBuckets / kWorkThreads; ++k) scan[t + kWorkThreads * k] = v[k];
    __syncthreads();
  }
  // bucket b starts after all heavier buckets: scan[b] - hist[b]
  for (int b = t; b < kWorkBuckets; b += kWorkThreads) hist[b] = scan[b] - hist[b];
  __syncthreads();
  for (int64_t i = t; i < n; i += kWorkThreads) {
    const int pos = atomicAdd(&hist[work_bucket(work[first + i])], 1);
    order[(int64_t)pos * regions + region] = (int32_t)(first + i);
  }
}
}  // namespace ks

extern "C" int ks_work_order(ks_stream_t stream, int64_t N, const int32_t* work, int32_t* order) {
  using namespace ks;
  if (N < 0 || N > 0x7fffffff) return fail(KS_EINVAL, "ks_work_order: bad env count");
  if (N == 0) return KS_OK;
  if (!work || !order) return fail(KS_EINVAL, "ks_work_order: null argument");
  const int regions = (N % kXcds == 0 && N >= 64 * kXcds) ? kXcds : 1;
  hipLaunchKernelGGL(work_order_kernel, dim3(regions), dim3(kWorkThreads), 0, (hipStream_t)stream, N, work, order);
  return check_launch("ks_work_order");
}
