// GAE / returns scan, advantage normalisation, PPO loss and reward/termination
// reduction for gfx950.  Streaming, HBM-bound kernels: every array is read or
// written exactly once per launch, with 64 consecutive elements per wavefront.
#include "ks_common.h"
#include <mutex>

namespace ks {

static thread_local char g_err[256] = "";
char* err_buf() { return g_err; }

// ---------------------------------------------------------------------------------------------
// GAE, (B, T) layout.  One wavefront per env row.  The recurrences R_t = r'_t + g m_t R_{t+1} and
// A_t = d_t + g l m_t A_{t+1} (ksim/task/ppo.py:66-75) are compositions of affine maps x -> d + c x, which are
// associative.  Lanes hold time in DESCENDING order (lane i of a 64-step chunk holds t = chunk_end - i), so the
// reverse scan over time is a forward scan over lanes: four DPP row_shr steps inside 16-lane rows, then
// row_bcast:15 and row_bcast:31 to chain the rows; no LDS traffic.  Chunks are chained from the end of the row
// through a wave-uniform carry read from lane 63.
// ---------------------------------------------------------------------------------------------
template <int kCtrl, int kRowMask>
__device__ __forceinline__ float dpp_take(float old, float x) {  // lanes without a valid source keep `old`
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, x),
                                                                kCtrl, kRowMask, 0xf, false));
}

// one scan step: (c, d) <- (c, d) o (c, d)[source lane]; identity where there is no source
template <int kCtrl, int kRowMask>
__device__ __forceinline__ void scan_step(float& c, float& d) {
  const float pc = dpp_take<kCtrl, kRowMask>(1.0f, c);
  const float pd = dpp_take<kCtrl, kRowMask>(0.0f, d);
  d = d + c * pd;
  c = c * pc;
}

__device__ __forceinline__ void affine_scan64(float& c, float& d) {
  scan_step<0x111, 0xf>(c, d);  // row_shr:1
  scan_step<0x112, 0xf>(c, d);  // row_shr:2
  scan_step<0x114, 0xf>(c, d);  // row_shr:4
  scan_step<0x118, 0xf>(c, d);  // row_shr:8
  scan_step<0x142, 0xa>(c, d);  // row_bcast:15 -> rows 1 and 3
  scan_step<0x143, 0xc>(c, d);  // row_bcast:31 -> rows 2 and 3
}

__device__ __forceinline__ float lane63(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), 63));
}

constexpr int kGaeMaxChunks = 4;  // rows of up to 256 steps keep every load in flight at once

__global__ __launch_bounds__(256) void gae_bt_kernel(
    int64_t B, int64_t T, const float* __restrict__ values, const float* __restrict__ rewards,
    const uint8_t* __restrict__ dones, const uint8_t* __restrict__ successes, float gamma, float lam,
    int mc, float* __restrict__ gae, float* __restrict__ returns, float* __restrict__ targets) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= B) return;  // whole wavefront leaves together
  const int64_t base = row * T;
  const float v_last = values[base + T - 1];  // bootstrap = last value repeated, ppo.py:79
  const float gl = gamma * lam;
  const float omg = 1.0f - gamma;
  float carry_r = 0.f, carry_a = 0.f, v_after = v_last;  // v_after: value at the first step after the chunk
  const int64_t nchunk = (T + 63) >> 6;
  for (int64_t c0 = nchunk - 1; c0 >= 0; c0 -= kGaeMaxChunks) {
    // issue the loads of up to kGaeMaxChunks chunks before any of them is scanned
    float v[kGaeMaxChunks], r[kGaeMaxChunks];
    uint8_t dn[kGaeMaxChunks], sc[kGaeMaxChunks];
#pragma unroll
    for (int k = 0; k < kGaeMaxChunks; ++k) {
      const int64_t c = c0 - k;
      const int64_t t = (c << 6) + 63 - lane;  // descending time across lanes
      const bool valid = c >= 0 && t < T;
      v[k] = valid ? values[base + t] : 0.f;
      r[k] = valid ? rewards[base + t] : 0.f;
      dn[k] = valid ? dones[base + t] : (uint8_t)0;
      sc[k] = (valid && successes) ? successes[base + t] : (uint8_t)0;
    }
#pragma unroll
    for (int k = 0; k < kGaeMaxChunks; ++k) {
      const int64_t c = c0 - k;
      if (c < 0) break;
      const int64_t t = (c << 6) + 63 - lane;
      const bool valid = t < T;
      // V(s_{t+1}) sits one lane down; lane 0 takes the first value after the chunk (wave_shr:1 keeps `old` there)
      float v_up = dpp_take<0x138, 0xf>(v_after, v[k]);
      if (t + 1 >= T) v_up = v_last;
      const float mask = dn[k] ? 0.f : 1.f;
      const float rb = omg * r[k] + gamma * v[k] * (sc[k] ? 1.f : 0.f);  // ppo.py:82-83
      const float delta = rb + gamma * v_up * mask - v[k];                // ppo.py:86
      float c_r = valid ? gamma * mask : 1.f, d_r = valid ? rb : 0.f;
      float c_a = valid ? gl * mask : 1.f, d_a = valid ? delta : 0.f;
      affine_scan64(c_r, d_r);
      affine_scan64(c_a, d_a);
      const float R = d_r + c_r * carry_r;
      const float A = d_a + c_a * carry_a;
      if (valid) {
        if (gae) gae[base + t] = A;
        if (returns) returns[base + t] = R;
        if (targets) targets[base + t] = mc ? R : A + v[k];  // ppo.py:107
      }
      carry_r = lane63(R);
      carry_a = lane63(A);
      v_after = lane63(v[k]);
    }
  }
}

// GAE, (T, N) layout.  A workgroup owns 32 consecutive envs and walks back in time in chunks of 32 steps: all 256
// threads load the chunk's (32 steps x 32 envs) tiles into LDS (128-byte rows, every load independent of the
// recurrence), the first 32 threads run the recurrence out of LDS, one env each, and all threads write the results
// back.  With one lane per env doing its own loads, 8192 envs would be 128 wavefronts with one dependent stream of
// loads each; here every CU has eight times as many loads in flight and N / 32 workgroups spread over the chip.
constexpr int kTnEnvs = 32, kTnSteps = 32;
__global__ __launch_bounds__(256) void gae_tn_kernel(
    int64_t T, int64_t N, const float* __restrict__ values, const float* __restrict__ rewards,
    const uint8_t* __restrict__ dones, const uint8_t* __restrict__ successes, float gamma, float lam,
    int mc, float* __restrict__ gae, float* __restrict__ returns, float* __restrict__ targets) {
  __shared__ float sv[kTnSteps][kTnEnvs], sr[kTnSteps][kTnEnvs], oa[kTnSteps][kTnEnvs], orr[kTnSteps][kTnEnvs];
  __shared__ uint8_t sd[kTnSteps][kTnEnvs], ss[kTnSteps][kTnEnvs];
  const int tx = threadIdx.x & (kTnEnvs - 1), ty = threadIdx.x / kTnEnvs;
  // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Four neighbouring tiles share every 128-byte
  // line of the byte arrays, so neighbouring tiles go to one XCD: workgroup b takes tile (b % 8) * (grid / 8) + b / 8.
  int64_t tile = blockIdx.x;
  if (gridDim.x % 8 == 0) tile = (int64_t)(blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8;
  const int64_t e = tile * kTnEnvs + tx;
  const bool in = e < N;
  const float gl = gamma * lam, omg = 1.0f - gamma;
  float R = 0.f, A = 0.f, v_up = 0.f;
  for (int64_t t1 = T; t1 > 0; t1 -= kTnSteps) {
    const int64_t t0 = t1 > kTnSteps ? t1 - kTnSteps : 0;
    const int n = (int)(t1 - t0);
    for (int k = ty; k < n; k += 256 / kTnEnvs) {
      const int64_t i = (t0 + k) * N + e;
      sv[k][tx] = in ? values[i] : 0.f;
      sr[k][tx] = in ? rewards[i] : 0.f;
      sd[k][tx] = in ? dones[i] : (uint8_t)0;
      ss[k][tx] = (in && successes) ? successes[i] : (uint8_t)0;
    }
    __syncthreads();
    if (threadIdx.x < kTnEnvs) {
      if (t1 == T) v_up = sv[n - 1][tx];
      for (int k = n - 1; k >= 0; --k) {
        const float v = sv[k][tx], r = sr[k][tx];
        const float mask = sd[k][tx] ? 0.f : 1.f;
        const float sc = ss[k][tx] ? 1.f : 0.f;
        const float rb = omg * r + gamma * v * sc;
        const float delta = rb + gamma * v_up * mask - v;
        R = rb + gamma * mask * R;
        A = delta + gl * mask * A;
        oa[k][tx] = A;
        orr[k][tx] = R;
        v_up = v;
      }
    }
    __syncthreads();
    if (in)
      for (int k = ty; k < n; k += 256 / kTnEnvs) {
        const int64_t i = (t0 + k) * N + e;
        const float a = oa[k][tx], rr = orr[k][tx];
        if (gae) gae[i] = a;
        if (returns) returns[i] = rr;
        if (targets) targets[i] = mc ? rr : a + sv[k][tx];
      }
    __syncthreads();
  }
}

// ---------------------------------------------------------------------------------------------
// Deterministic two-stage reductions (no atomics): stage 1 writes one partial per block,
// stage 2 re-reads the <= 1024 partials in a fixed order.
// ---------------------------------------------------------------------------------------------
constexpr int kMaxPartials = 1024;

__device__ inline double wave_sum(double x) {
#pragma unroll
  for (int s = 32; s > 0; s >>= 1) x += __shfl_down(x, s);
  return x;
}

// Sum over a 256-thread block; result valid in thread 0.
__device__ inline double block_sum(double x, double* lds4) {
  x = wave_sum(x);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) lds4[threadIdx.x >> 6] = x;
  __syncthreads();
  return lds4[0] + lds4[1] + lds4[2] + lds4[3];
}

__global__ __launch_bounds__(256) void moments_kernel(int64_t n, const float* __restrict__ x,
                                                       double* __restrict__ partial) {
  __shared__ double lds[4];
  double s = 0.0, ss = 0.0;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const double v = x[i];
    s += v;
    ss += v * v;
  }
  s = block_sum(s, lds);
  ss = block_sum(ss, lds);
  if (threadIdx.x == 0) {
    partial[blockIdx.x] = s;
    partial[kMaxPartials + blockIdx.x] = ss;
  }
}

__global__ __launch_bounds__(256) void normalize_kernel(int64_t n, int nparts, const float* __restrict__ x,
                                                         const double* __restrict__ partial,
                                                         float* __restrict__ out) {
  __shared__ double lds[4];
  __shared__ float s_mean, s_inv;
  double s = 0.0, ss = 0.0;
  for (int i = threadIdx.x; i < nparts; i += blockDim.x) {
    s += partial[i];
    ss += partial[kMaxPartials + i];
  }
  s = block_sum(s, lds);
  ss = block_sum(ss, lds);
  if (threadIdx.x == 0) {
    const double mean = s / (double)n;
    double var = ss / (double)n - mean * mean;
    if (var < 0.0) var = 0.0;
    double sd = sqrt(var);
    if (sd < 1e-6) sd = 1e-6;  // ppo.py:118
    s_mean = (float)mean;
    s_inv = (float)(1.0 / sd);
  }
  __syncthreads();
  const float mean = s_mean, inv = s_inv;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
    out[i] = (x[i] - mean) * inv;
}

// the adaptive-KL factor: a device scalar when the caller keeps it there, otherwise the host's number
__device__ __forceinline__ float kl_scale_of(const KsPpoLossParams& p) { return p.kl_scale_device ? *p.kl_scale_device : p.kl_scale; }

// ---------------------------------------------------------------------------------------------
// PPO loss (ppo.py:207-246).  One lane per (b, t) element; the A log-probs of an element are
// contiguous, so a wavefront touches one contiguous 64*A*4-byte span per array.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void ppo_loss_kernel(
    int64_t n, int A, KsPpoLossParams p, const float* __restrict__ adv, const float* __restrict__ tgt,
    const float* __restrict__ lp_on, const float* __restrict__ v_on, const float* __restrict__ lp_off,
    const float* __restrict__ v_off, const float* __restrict__ ent, float* __restrict__ o_policy,
    float* __restrict__ o_value, float* __restrict__ o_kl, float* __restrict__ o_ent,
    double* __restrict__ partial) {
  __shared__ double lds[4];
  double acc = 0.0;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    float log_ratio = 0.f, kl = 0.f, es = 0.f;
    const float* a_on = lp_on + i * A;
    const float* a_off = lp_off + i * A;
    for (int a = 0; a < A; ++a) {
      const float on = a_on[a], off = a_off[a];
      log_ratio += off - on;
      kl += on - off;
    }
    if (ent) {
      const float* e = ent + i * A;
      for (int a = 0; a < A; ++a) es += e[a];
    }
    const float lr = fminf(fmaxf(log_ratio, -p.log_clip_value), p.log_clip_value);
    const float ratio = expf(lr);
    const float cr = fminf(fmaxf(ratio, 1.f - p.clip_param), 1.f + p.clip_param);
    const float ad = adv[i];
    const float policy = -fminf(ratio * ad, cr * ad);
    const float von = v_on[i], voff = v_off[i], tg = tgt[i];
    float vobj;
    if (p.use_clipped_value_loss) {
      const float vc = von + fminf(fmaxf(voff - von, -p.clip_param), p.clip_param);
      const float ce = vc - tg, er = voff - tg;
      vobj = 0.5f * fmaxf(er * er, ce * ce);
    } else {
      const float er = tg - voff;
      vobj = 0.5f * er * er;
    }
    const float value = vobj * p.value_loss_coef;
    const float klv = kl * p.kl_coef * kl_scale_of(p);
    const float entv = ent ? -es * p.entropy_coef : 0.f;
    if (o_policy) o_policy[i] = policy;
    if (o_value) o_value[i] = value;
    if (o_kl) o_kl[i] = klv;
    if (o_ent && ent) o_ent[i] = entv;
    acc += (double)(policy + value + klv + entv);
  }
  acc = block_sum(acc, lds);
  if (threadIdx.x == 0) partial[blockIdx.x] = acc;
}

__global__ __launch_bounds__(256) void mean_finish_kernel(int nparts, int64_t n, const double* __restrict__ partial,
                                                           float* __restrict__ out) {
  __shared__ double lds[4];
  double s = 0.0;
  for (int i = threadIdx.x; i < nparts; i += blockDim.x) s += partial[i];
  s = block_sum(s, lds);
  if (threadIdx.x == 0) out[0] = (float)(s / (double)n);
}

// ---------------------------------------------------------------------------------------------
// Reward total (rl.py:219-239) and done/success (rl.py:1049-1050).
// ---------------------------------------------------------------------------------------------
struct RewardScales {
  float s[KS_MAX_REWARD_TERMS];
};

__global__ __launch_bounds__(256) void reward_total_kernel(
    int64_t n, int K, const float* __restrict__ comps, RewardScales sc, int use_min, float cmin, int use_max,
    float cmax, float* __restrict__ total, int k, const int8_t* __restrict__ terms, uint8_t* __restrict__ done,
    uint8_t* __restrict__ success) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  if (total) {
    float t = 0.f;
    for (int j = 0; j < K; ++j) {
      const float term = comps[(int64_t)j * n + i] * sc.s[j];
      t = (j == 0) ? term : t + term;  // insertion-order sum, rl.py:235
    }
    if (use_min) t = fmaxf(t, cmin);
    if (use_max) t = fminf(t, cmax);
    total[i] = t;
  }
  if (k > 0) {
    bool d = false, s = true;
    for (int j = 0; j < k; ++j) {
      const int8_t t = terms[(int64_t)j * n + i];
      d |= t != 0;
      s &= t != -1;
    }
    if (done) done[i] = d ? 1 : 0;
    if (success) success[i] = (s && d) ? 1 : 0;
  }
}

__global__ __launch_bounds__(256) void copy_f32_kernel(int64_t n, const float* __restrict__ src, float* __restrict__ dst) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) dst[i] = src[i];
}

static inline int grid_for(int64_t n, int block, int cap) {
  int64_t g = (n + block - 1) / block;
  if (g > cap) g = cap;
  if (g < 1) g = 1;
  return (int)g;
}

}  // namespace ks

using namespace ks;

extern "C" const char* ks_version(void) { return "ksim_hip 0.1 (gfx950)"; }
extern "C" const char* ks_last_error(void) { return ks::err_buf(); }
extern "C" int64_t ks_abi_sizeof(int32_t which) {
  switch (which) {
    case 0: return sizeof(KsPpoLossParams);
    case 1: return sizeof(KsModelDesc);
    case 2: return sizeof(KsStepIO);
    case 3: return sizeof(KsTermsDesc);
    case 4: return sizeof(KsObserveIO);
    case 5: return sizeof(KsTerminateIO);
    case 6: return sizeof(KsMlpDesc);
    case 7: return sizeof(KsRewardIO);
    case 8: return sizeof(KsObsElem);
    case 9: return sizeof(KsTermDesc);
    case 10: return sizeof(KsRewardDesc);
    case 11: return sizeof(KsRng);
    case 12: return sizeof(KsAdamParams);
    case 13: return sizeof(KsEventDesc);
    case 14: return sizeof(KsRewardScanIO);
    case 15: return sizeof(KsRewardScanDesc);
    case 16: return sizeof(KsGruDesc);
    case 17: return sizeof(KsLstmDesc);
    case 18: return sizeof(KsGaussianHead);
    case 19: return sizeof(KsCommandIO);
    case 20: return sizeof(KsMixtureHead);
    case 21: return sizeof(KsNoiseStage);
    case 22: return sizeof(KsRandomVar);
    default: return -1;
  }
}

static int check_gae_args(int64_t n0, int64_t n1, const float* v, const float* r, const uint8_t* d) {
  if (n0 < 0 || n1 < 0) return fail(KS_EINVAL, "ks_gae: negative size");
  if (n0 > 0 && n1 > 0 && (!v || !r || !d)) return fail(KS_EINVAL, "ks_gae: null input");
  if (n0 > (int64_t)1 << 40 || n1 > (int64_t)1 << 40) return fail(KS_ELIMIT, "ks_gae: size too large");
  return KS_OK;
}

extern "C" int ks_gae_bt(ks_stream_t stream, int64_t B, int64_t T, const float* values, const float* rewards,
                         const uint8_t* dones, const uint8_t* successes, float gamma, float lam,
                         int monte_carlo_returns, float* gae, float* returns, float* targets) {
  if (int rc = check_gae_args(B, T, values, rewards, dones)) return rc;
  if (B == 0 || T == 0) return KS_OK;
  const int rows_per_block = 4;
  const int64_t grid = (B + rows_per_block - 1) / rows_per_block;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_gae_bt: B too large");
  hipLaunchKernelGGL(gae_bt_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, B, T, values, rewards,
                     dones, successes, gamma, lam, monte_carlo_returns, gae, returns, targets);
  return check_launch("ks_gae_bt");
}

extern "C" int ks_gae_tn(ks_stream_t stream, int64_t T, int64_t N, const float* values, const float* rewards,
                         const uint8_t* dones, const uint8_t* successes, float gamma, float lam,
                         int monte_carlo_returns, float* gae, float* returns, float* targets) {
  if (int rc = check_gae_args(T, N, values, rewards, dones)) return rc;
  if (N == 0 || T == 0) return KS_OK;
  const int64_t grid = (N + kTnEnvs - 1) / kTnEnvs;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_gae_tn: N too large");
  hipLaunchKernelGGL(gae_tn_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, T, N, values, rewards,
                     dones, successes, gamma, lam, monte_carlo_returns, gae, returns, targets);
  return check_launch("ks_gae_tn");
}

extern "C" int ks_normalize_advantages(ks_stream_t stream, int64_t n, const float* gae, float* advantages,
                                       void* workspace) {
  if (n < 0) return fail(KS_EINVAL, "ks_normalize_advantages: negative size");
  if (n == 0) return KS_OK;
  if (!gae || !advantages || !workspace) return fail(KS_EINVAL, "ks_normalize_advantages: null pointer");
  const int g = grid_for(n, 256 * 4, kMaxPartials);
  double* partial = (double*)workspace;
  hipLaunchKernelGGL(moments_kernel, dim3(g), dim3(256), 0, (hipStream_t)stream, n, gae, partial);
  hipLaunchKernelGGL(normalize_kernel, dim3(grid_for(n, 256, 4096)), dim3(256), 0, (hipStream_t)stream, n, g, gae,
                     partial, advantages);
  return check_launch("ks_normalize_advantages");
}

// ---------------------------------------------------------------------------------------------
// ks_normalize_advantages without a workspace argument: the block partials live in a file-scope device array.
// The array's name is only a host-side handle; its device address is looked up once per device with
// hipGetSymbolAddress (each GPU holds its own copy) and that pointer is what the kernels receive.
// ---------------------------------------------------------------------------------------------
namespace ks {
static __device__ __align__(256) unsigned char scratch[KS_REDUCE_WORKSPACE_BYTES];
constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices] = {};
static std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device.
static int scratch_on_current_device(const char* who, void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(KS_ELAUNCH, "%s: hipGetDevice: %s", who, hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices)
    return fail(KS_ELIMIT, "%s: device %d beyond the %d this library keeps scratch for", who, dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) return fail(KS_ELAUNCH, "%s: hipGetSymbolAddress: %s", who, hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return KS_OK;
}
}  // namespace ks

extern "C" int ks_normalize_advantages_static(ks_stream_t stream, int64_t n, const float* gae, float* advantages) {
  if (n < 0) return fail(KS_EINVAL, "ks_normalize_advantages_static: negative size");
  if (n > KS_NORMALIZE_STATIC_MAX_N)
    return fail(KS_ELIMIT, "ks_normalize_advantages_static: n = %lld beyond the maximum of %lld elements", (long long)n,
                (long long)KS_NORMALIZE_STATIC_MAX_N);
  if (n == 0) return KS_OK;
  if (!gae || !advantages) return fail(KS_EINVAL, "ks_normalize_advantages_static: null pointer");
  void* ptr = nullptr;
  if (int rc = scratch_on_current_device("ks_normalize_advantages_static", &ptr)) return rc;
  double* partial = (double*)ptr;
  // every partial that stage 2 reads is written by stage 1 of the same call, so nothing has to be cleared
  const int g = grid_for(n, 256 * 4, kMaxPartials);
  hipLaunchKernelGGL(moments_kernel, dim3(g), dim3(256), 0, (hipStream_t)stream, n, gae, partial);
  hipLaunchKernelGGL(normalize_kernel, dim3(grid_for(n, 256, 4096)), dim3(256), 0, (hipStream_t)stream, n, g, gae,
                     partial, advantages);
  return check_launch("ks_normalize_advantages_static");
}

extern "C" int ks_ppo_loss(ks_stream_t stream, int64_t n, int32_t A, const KsPpoLossParams* params,
                           const float* advantages, const float* value_targets, const float* on_log_probs,
                           const float* on_values, const float* off_log_probs, const float* off_values,
                           const float* off_entropy, float* policy_loss, float* value_loss, float* kl_loss,
                           float* entropy_loss, float* loss_out, void* workspace) {
  if (n < 0 || A < 1) return fail(KS_EINVAL, "ks_ppo_loss: bad size n=%lld A=%d", (long long)n, A);
  if (!params) return fail(KS_EINVAL, "ks_ppo_loss: null params");
  if (n == 0) return KS_OK;
  if (!advantages || !value_targets || !on_log_probs || !on_values || !off_log_probs || !off_values || !workspace)
    return fail(KS_EINVAL, "ks_ppo_loss: null pointer");
  const int g = grid_for(n, 256, kMaxPartials);
  double* partial = (double*)workspace;
  hipLaunchKernelGGL(ppo_loss_kernel, dim3(g), dim3(256), 0, (hipStream_t)stream, n, (int)A, *params, advantages,
                     value_targets, on_log_probs, on_values, off_log_probs, off_values, off_entropy, policy_loss,
                     value_loss, kl_loss, entropy_loss, partial);
  if (loss_out)
    hipLaunchKernelGGL(mean_finish_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, g, n, partial, loss_out);
  return check_launch("ks_ppo_loss");
}

extern "C" int ks_reward_total(ks_stream_t stream, int64_t n, int32_t K, const float* components,
                               const float* scales, int32_t use_clip_min, float clip_min, int32_t use_clip_max,
                               float clip_max, float* total, int32_t k, const int8_t* terminations, uint8_t* done,
                               uint8_t* success) {
  if (n < 0 || K < 0 || k < 0) return fail(KS_EINVAL, "ks_reward_total: negative size");
  if (K > KS_MAX_REWARD_TERMS || k > KS_MAX_REWARD_TERMS)
    return fail(KS_ELIMIT, "ks_reward_total: more than %d terms", KS_MAX_REWARD_TERMS);
  if (n == 0) return KS_OK;
  if (total && (K == 0 || !components || !scales)) return fail(KS_EINVAL, "ks_reward_total: total needs K>0 components");
  if (k > 0 && !terminations) return fail(KS_EINVAL, "ks_reward_total: null terminations");
  RewardScales sc{};
  for (int j = 0; j < K && scales; ++j) sc.s[j] = scales[j];
  const int64_t grid = (n + 255) / 256;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_reward_total: n too large");
  hipLaunchKernelGGL(reward_total_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, n, (int)K,
                     components, sc, use_clip_min, clip_min, use_clip_max, clip_max, total, (int)k, terminations, done,
                     success);
  return check_launch("ks_reward_total");
}

extern "C" int ks_copy_f32(ks_stream_t stream, int64_t n, const float* src, float* dst) {
  if (n < 0) return fail(KS_EINVAL, "ks_copy_f32: negative size");
  if (n == 0) return KS_OK;
  if (!src || !dst) return fail(KS_EINVAL, "ks_copy_f32: null pointer");
  hipLaunchKernelGGL(copy_f32_kernel, dim3(grid_for(n, 256, 65536)), dim3(256), 0, (hipStream_t)stream, n, src, dst);
  return check_launch("ks_copy_f32");
}

// ---------------------------------------------------------------------------------------------
// Gaussian policy head and the gradient of the PPO objective
// ---------------------------------------------------------------------------------------------
namespace ks {

constexpr float kHalfLog2Pi = 0.91893853320467274178f;

__global__ __launch_bounds__(256) void gaussian_log_prob_kernel(int64_t n, int nu, const float* __restrict__ mean,
                                                               const float* __restrict__ log_std,
                                                               const float* __restrict__ action, float* __restrict__ lp,
                                                               float* __restrict__ ent) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n) return;
  const int a = (int)(idx % nu);
  const float ls = log_std[a];
  const float z = (action[idx] - mean[idx]) * __expf(-ls);
  lp[idx] = -0.5f * z * z - ls - kHalfLog2Pi;
  if (ent) ent[idx] = 0.5f + kHalfLog2Pi + ls;
}

// One thread per row m; every workgroup also accumulates the log-std gradient of its rows, reduced in a fixed
// order (block partials, then ppo_grad_finish_kernel), so the result does not depend on scheduling.
__global__ __launch_bounds__(256) void ppo_loss_grad_kernel(int64_t M, int nu, KsPpoLossParams p, const float* __restrict__ mean,
                                                           const float* __restrict__ log_std, const float* __restrict__ action,
                                                           const float* __restrict__ on_lp, const float* __restrict__ adv,
                                                           const float* __restrict__ tgt, const float* __restrict__ on_v,
                                                           const float* __restrict__ v, float* __restrict__ d_mean,
                                                           float* __restrict__ d_value, float* __restrict__ partial) {
  __shared__ float red[256];
  float dls[KS_MAX_ACTIONS];
#pragma unroll
  for (int a = 0; a < KS_MAX_ACTIONS; ++a) dls[a] = 0.f;
  const float inv_m = 1.0f / (float)M;
  for (int64_t m = (int64_t)blockIdx.x * 256 + threadIdx.x; m < M; m += (int64_t)gridDim.x * 256) {
    // new log-probabilities and the log ratio
    float logr = 0.f;
    for (int a = 0; a < nu; ++a) {
      const float ls = log_std[a];
      const float z = (action[m * nu + a] - mean[m * nu + a]) * __expf(-ls);
      logr += (-0.5f * z * z - ls - kHalfLog2Pi) - on_lp[m * nu + a];
    }
    const bool log_inside = logr > -p.log_clip_value && logr < p.log_clip_value;
    const float ratio = __expf(fminf(fmaxf(logr, -p.log_clip_value), p.log_clip_value));
    const float A = adv[m];
    const float lo = 1.f - p.clip_param, hi = 1.f + p.clip_param;
    const float s1 = ratio * A, s2 = fminf(fmaxf(ratio, lo), hi) * A;
    // d(-min(s1, s2)) / d(log ratio); inside the clip range both surrogates coincide
    const bool ratio_inside = ratio > lo && ratio < hi;
    float g_logr = 0.f;
    if (log_inside) {
      if (s1 < s2 || ratio_inside) g_logr = -A * ratio;   // the unclipped surrogate is active (or both are the same)
    }
    // kl term: (on_lp - lp) * kl_coef * kl_scale per action
    const float g_lp = (g_logr - p.kl_coef * kl_scale_of(p)) * inv_m;
    const float g_ent = -p.entropy_coef * inv_m;
    for (int a = 0; a < nu; ++a) {
      const float ls = log_std[a];
      const float is = __expf(-ls);
      const float z = (action[m * nu + a] - mean[m * nu + a]) * is;
      d_mean[m * nu + a] = g_lp * z * is;
      dls[a] += g_lp * (z * z - 1.f) + g_ent;
    }
    // value term
    const float vv = v[m], vo = on_v[m], t = tgt[m];
    float gv;
    if (p.use_clipped_value_loss) {
      const float dvv = vv - vo;
      const float vc = vo + fminf(fmaxf(dvv, -p.clip_param), p.clip_param);
      const float e = vv - t, ec = vc - t;
      if (e * e >= ec * ec) gv = e;
      else gv = (dvv > -p.clip_param && dvv < p.clip_param) ? ec : 0.f;
    } else {
      gv = vv - t;
    }
    d_value[m] = p.value_loss_coef * gv * inv_m;
  }
  for (int a = 0; a < nu; ++a) {
    red[threadIdx.x] = dls[a];
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
      if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
      __syncthreads();
    }
    if (threadIdx.x == 0) partial[(int64_t)blockIdx.x * nu + a] = red[0];
    __syncthreads();
  }
}

// log N(action; mean, std) and the entropy per action for the mean | raw deviation head
__global__ __launch_bounds__(256) void gaussian_head_log_prob_kernel(int64_t n, int nu, KsGaussianHead hd, const float* __restrict__ raw,
                                                                    const float* __restrict__ action, float* __restrict__ lp,
                                                                    float* __restrict__ ent) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n) return;
  const int64_t m = idx / nu;
  const int a = (int)(idx - m * nu);
  const float mean = raw[m * 2 * nu + a] + (hd.mean_bias ? hd.mean_bias[a] : 0.f);
  const float r = raw[m * 2 * nu + nu + a];
  const float sp = r > 20.f ? r : log1pf(expf(r));
  const float sd = fminf((sp + hd.min_std) * hd.var_scale, hd.max_std);
  const float z = (action[idx] - mean) / sd, ls = logf(sd);
  lp[idx] = -0.5f * z * z - ls - kHalfLog2Pi;
  if (ent) ent[idx] = 0.5f + kHalfLog2Pi + ls;
}

// The same objective for a network that emits its own deviations: raw (M, 2 nu) = means | raw deviations,
// std = min((softplus(raw_std) + min_std) * var_scale, max_std).  One thread per row; d_raw receives the gradient of both halves.
__global__ __launch_bounds__(256) void ppo_loss_grad_head_kernel(int64_t M, int nu, KsPpoLossParams p, KsGaussianHead hd,
                                                                const float* __restrict__ raw, const float* __restrict__ action,
                                                                const float* __restrict__ on_lp, const float* __restrict__ adv,
                                                                const float* __restrict__ tgt, const float* __restrict__ on_v,
                                                                const float* __restrict__ v, float* __restrict__ d_raw,
                                                                float* __restrict__ d_value) {
  const int64_t m = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (m >= M) return;
  const float inv_m = 1.0f / (float)M;
  const float* rm = raw + m * 2 * nu;
  float logr = 0.f;
  for (int a = 0; a < nu; ++a) {
    const float mean = rm[a] + (hd.mean_bias ? hd.mean_bias[a] : 0.f);
    const float r = rm[nu + a];
    const float sp = r > 20.f ? r : log1pf(expf(r));
    const float sd = fminf((sp + hd.min_std) * hd.var_scale, hd.max_std);
    const float z = (action[m * nu + a] - mean) / sd;
    logr += (-0.5f * z * z - logf(sd) - kHalfLog2Pi) - on_lp[m * nu + a];
  }
  const bool log_inside = logr > -p.log_clip_value && logr < p.log_clip_value;
  const float ratio = __expf(fminf(fmaxf(logr, -p.log_clip_value), p.log_clip_value));
  const float A = adv[m];
  const float lo = 1.f - p.clip_param, hi = 1.f + p.clip_param;
  const float s1 = ratio * A, s2 = fminf(fmaxf(ratio, lo), hi) * A;
  const bool ratio_inside = ratio > lo && ratio < hi;
  float g_logr = 0.f;
  if (log_inside && (s1 < s2 || ratio_inside)) g_logr = -A * ratio;
  const float g_lp = (g_logr - p.kl_coef * kl_scale_of(p)) * inv_m;
  const float g_ent = -p.entropy_coef * inv_m;
  for (int a = 0; a < nu; ++a) {
    const float mean = rm[a] + (hd.mean_bias ? hd.mean_bias[a] : 0.f);
    const float r = rm[nu + a];
    const float sp = r > 20.f ? r : log1pf(expf(r));
    const float pre = (sp + hd.min_std) * hd.var_scale;
    const bool capped = pre >= hd.max_std;
    const float sd = capped ? hd.max_std : pre;
    const float z = (action[m * nu + a] - mean) / sd;
    d_raw[m * 2 * nu + a] = g_lp * z / sd;
    // d/d log(std) of the log-density is z^2 - 1 and of the entropy 1; then through the cap, the scale and the softplus
    const float d_ls = g_lp * (z * z - 1.f) + g_ent;
    const float sig = r > 20.f ? 1.f : 1.f / (1.f + expf(-r));
    d_raw[m * 2 * nu + nu + a] = capped ? 0.f : d_ls / sd * hd.var_scale * sig;
  }
  const float vv = v[m], vo = on_v[m], t = tgt[m];
  float gv;
  if (p.use_clipped_value_loss) {
    const float dvv = vv - vo;
    const float vc = vo + fminf(fmaxf(dvv, -p.clip_param), p.clip_param);
    const float e = vv - t, ec = vc - t;
    if (e * e >= ec * ec) gv = e;
    else gv = (dvv > -p.clip_param && dvv < p.clip_param) ? ec : 0.f;
  } else {
    gv = vv - t;
  }
  d_value[m] = p.value_loss_coef * gv * inv_m;
}

// The same objective for the mixture-of-Gaussians head: raw (M, 3 nu K) = component means, raw deviations and logits per
// action.  One thread per row walks its actions twice (log ratio, then gradients).  The entropy term uses the usual
// upper bound of a mixture's entropy, sum_k pi_k H_k + H(pi).
__global__ __launch_bounds__(128) void ppo_loss_grad_mixture_kernel(int64_t M, int nu, KsPpoLossParams p, KsMixtureHead hd,
                                                                   const float* __restrict__ raw, const float* __restrict__ action,
                                                                   const float* __restrict__ on_lp, const float* __restrict__ adv,
                                                                   const float* __restrict__ tgt, const float* __restrict__ on_v,
                                                                   const float* __restrict__ v, float* __restrict__ d_raw,
                                                                   float* __restrict__ d_value) {
  const int64_t m = (int64_t)blockIdx.x * 128 + threadIdx.x;
  if (m >= M) return;
  const int K = hd.num_mixtures;
  const float inv_m = 1.0f / (float)M;
  const float* rm = raw + m * 3 * nu * K;
  float* dm = d_raw + m * 3 * nu * K;
  auto component = [&](int a, int k, float& mean, float& sd, bool& mean_clipped, bool& sd_capped, float& sig) {
    const float r0 = rm[a * K + k] + (hd.mean_bias ? hd.mean_bias[a] : 0.f);
    const float lo = hd.clip_lo ? hd.clip_lo[a] : -INFINITY, hi = hd.clip_hi ? hd.clip_hi[a] : INFINITY;
    mean = fminf(fmaxf(r0, lo), hi);
    mean_clipped = r0 < lo || r0 > hi;
    const float r = rm[(nu + a) * K + k];
    const float sp = r > 20.f ? r : log1pf(expf(r));
    const float pre = (sp + hd.min_std) * hd.var_scale;
    sd_capped = pre >= hd.max_std;
    sd = sd_capped ? hd.max_std : pre;
    sig = r > 20.f ? 1.f : 1.f / (1.f + expf(-r));
  };
  auto log_mix = [&](int a, float x, float& lse_logits) {  // log density of the mixture at x, and the logits' normaliser
    float lmax = -INFINITY;
    for (int k = 0; k < K; ++k) lmax = fmaxf(lmax, rm[(2 * nu + a) * K + k]);
    float zs = 0.f;
    for (int k = 0; k < K; ++k) zs += expf(rm[(2 * nu + a) * K + k] - lmax);
    lse_logits = lmax + logf(zs);
    float tmax = -INFINITY, t[KS_MAX_MIXTURES];
    for (int k = 0; k < K; ++k) {
      float mean, sd, sg; bool c1, c2;
      component(a, k, mean, sd, c1, c2, sg);
      const float z = (x - mean) / sd;
      t[k] = (rm[(2 * nu + a) * K + k] - lse_logits) - 0.5f * z * z - logf(sd) - kHalfLog2Pi;
      tmax = fmaxf(tmax, t[k]);
    }
    float acc = 0.f;
    for (int k = 0; k < K; ++k) acc += expf(t[k] - tmax);
    return tmax + logf(acc);
  };
  float logr = 0.f;
  for (int a = 0; a < nu; ++a) {
    float lse;
    logr += log_mix(a, action[m * nu + a], lse) - on_lp[m * nu + a];
  }
  const bool log_inside = logr > -p.log_clip_value && logr < p.log_clip_value;
  const float ratio = __expf(fminf(fmaxf(logr, -p.log_clip_value), p.log_clip_value));
  const float A = adv[m];
  const float lo_r = 1.f - p.clip_param, hi_r = 1.f + p.clip_param;
  const float s1 = ratio * A, s2 = fminf(fmaxf(ratio, lo_r), hi_r) * A;
  const bool ratio_inside = ratio > lo_r && ratio < hi_r;
  float g_logr = 0.f;
  if (log_inside && (s1 < s2 || ratio_inside)) g_logr = -A * ratio;
  const float g_lp = (g_logr - p.kl_coef * kl_scale_of(p)) * inv_m;
  const float g_ent = -p.entropy_coef * inv_m;
  for (int a = 0; a < nu; ++a) {
    const float x = action[m * nu + a];
    float lse;
    const float lp = log_mix(a, x, lse);
    // entropy bound: sum_k pi_k (h_k - log pi_k), h_k = 1/2 + log sqrt(2 pi) + log sd_k
    float gbar = 0.f;
    for (int k = 0; k < K; ++k) {
      float mean, sd, sg; bool c1, c2;
      component(a, k, mean, sd, c1, c2, sg);
      const float lpi = rm[(2 * nu + a) * K + k] - lse;
      gbar += expf(lpi) * (0.5f + kHalfLog2Pi + logf(sd) - lpi);
    }
    for (int k = 0; k < K; ++k) {
      float mean, sd, sg; bool mean_clipped, sd_capped;
      component(a, k, mean, sd, mean_clipped, sd_capped, sg);
      const float lpi = rm[(2 * nu + a) * K + k] - lse, pi = expf(lpi);
      const float z = (x - mean) / sd;
      const float resp = expf(lpi - 0.5f * z * z - logf(sd) - kHalfLog2Pi - lp);  // responsibility of component k
      dm[a * K + k] = mean_clipped ? 0.f : g_lp * resp * z / sd;
      const float d_ls = g_lp * resp * (z * z - 1.f) + g_ent * pi;
      dm[(nu + a) * K + k] = sd_capped ? 0.f : d_ls / sd * hd.var_scale * sg;
      const float gk = 0.5f + kHalfLog2Pi + logf(sd) - lpi;
      dm[(2 * nu + a) * K + k] = g_lp * (resp - pi) + g_ent * pi * (gk - gbar);
    }
  }
  const float vv = v[m], vo = on_v[m], t = tgt[m];
  float gv;
  if (p.use_clipped_value_loss) {
    const float dvv = vv - vo;
    const float vc = vo + fminf(fmaxf(dvv, -p.clip_param), p.clip_param);
    const float e = vv - t, ec = vc - t;
    if (e * e >= ec * ec) gv = e;
    else gv = (dvv > -p.clip_param && dvv < p.clip_param) ? ec : 0.f;
  } else {
    gv = vv - t;
  }
  d_value[m] = p.value_loss_coef * gv * inv_m;
}

// d_log_std[a] = sum over the blocks' partial sums: one workgroup per action, a fixed tree over up to 256 partials (one
// thread walking them one after the other spends 256 dependent load latencies on it)
__global__ __launch_bounds__(256) void ppo_grad_finish_kernel(int nblocks, int nu, const float* __restrict__ partial, float* __restrict__ d_log_std) {
  __shared__ float red[256];
  const int a = blockIdx.x;
  float s = 0.f;
  for (int b = threadIdx.x; b < nblocks; b += 256) s += partial[(int64_t)b * nu + a];
  red[threadIdx.x] = s;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) d_log_std[a] = red[0];
}

// adaptive KL: partial[b] = sum over the block's strided share of (on_lp - lp), every element of every row
__global__ __launch_bounds__(256) void kl_parts_kernel(int64_t n, const float* __restrict__ on_lp, const float* __restrict__ lp,
                                                       float* __restrict__ partial) {
  __shared__ float red[256];
  float s = 0.f;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) s += on_lp[i] - lp[i];
  red[threadIdx.x] = s;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) partial[blockIdx.x] = red[0];
}

__global__ __launch_bounds__(256) void kl_adapt_kernel(int nblocks, float inv_rows, float kl_coef, float desired,
                                                       const float* __restrict__ partial, float* __restrict__ kl_scale) {
  __shared__ float red[256];
  red[threadIdx.x] = (int)threadIdx.x < nblocks ? partial[threadIdx.x] : 0.f;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const float coef = kl_coef * *kl_scale;
    const float kl_mean = red[0] * inv_rows * coef;
    float c = coef;
    if (kl_mean > desired * 1.5f) c = coef * 1.5f;
    if (kl_mean < desired / 1.5f) c = c / 1.5f;
    c = fminf(fmaxf(c, 1e-8f), 1e2f);
    *kl_scale = c / kl_coef;
  }
}

// One-pole low-pass along the time axis of a trajectory, one thread per (env column, joint), walking the T steps in order:
// y_t = y_{t-1} + alpha (x_t + bias - y_{t-1}), y_{t-1} = 0 at the steps flagged fresh (the carry restarts with the
// episode) and y0 before the first step.  Rows are (t, m) with ld floats each; the first nu columns hold the signal, the
// others travel unchanged.  `add` is an observation-dependent part of the bias: add[(t M + m) add_ld + k] joins joint
// add_first + k.
__global__ __launch_bounds__(256) void lowpass_scan_kernel(int64_t T, int64_t M, int nu, int ld, float alpha,
                                                           const float* __restrict__ x, const float* __restrict__ mean_bias,
                                                           const float* __restrict__ add, int64_t add_ld, int add_first, int add_count,
                                                           const float* __restrict__ y0, const uint8_t* __restrict__ fresh,
                                                           float* __restrict__ y, float* __restrict__ y_last) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= M * (int64_t)ld) return;
  const int64_t m = idx / ld;
  const int j = (int)(idx - m * ld);
  constexpr int kAhead = 8;  // steps whose loads are in flight together: the recursion itself is a few instructions per step
  if (j >= nu) {  // the columns behind the signal (raw deviations of the head): copied when the output is another buffer
    if (x != y)
      for (int64_t t0 = 0; t0 < T; t0 += kAhead) {
        float v[kAhead];
#pragma unroll
        for (int k = 0; k < kAhead; ++k) v[k] = t0 + k < T ? x[((t0 + k) * M + m) * ld + j] : 0.f;
#pragma unroll
        for (int k = 0; k < kAhead; ++k)
          if (t0 + k < T) y[((t0 + k) * M + m) * ld + j] = v[k];
      }
    return;
  }
  const float b = mean_bias ? mean_bias[j] : 0.f;
  const bool has_add = add && j >= add_first && j < add_first + add_count;
  float last = y0 ? y0[m * nu + j] : 0.f;
  for (int64_t t0 = 0; t0 < T; t0 += kAhead) {
    float v[kAhead];
    bool f[kAhead];
#pragma unroll
    for (int k = 0; k < kAhead; ++k) {
      const bool in = t0 + k < T;
      const int64_t r = in ? (t0 + k) * M + m : m;
      v[k] = x[r * ld + j] + b;
      if (has_add) v[k] += add[r * add_ld + (j - add_first)];
      f[k] = fresh && fresh[r];
    }
#pragma unroll
    for (int k = 0; k < kAhead; ++k)
      if (t0 + k < T) {
        if (f[k]) last = 0.f;
        last = last + alpha * (v[k] - last);
        y[((t0 + k) * M + m) * ld + j] = last;
      }
  }
  if (y_last) y_last[m * nu + j] = last;
}

// Reverse sweep of the same recursion: with g_t = dL/dy_t on entry, the gradient reaching y_t is
// G_t = g_t + (1 - alpha) G_{t+1} unless step t + 1 is fresh (the carry was cut there), and dL/dx_t = alpha G_t, written in
// place.  d_y0 receives (1 - alpha) G_0 unless step 0 is fresh.
__global__ __launch_bounds__(256) void lowpass_scan_backward_kernel(int64_t T, int64_t M, int nu, int ld, float alpha,
                                                                    const uint8_t* __restrict__ fresh, float* __restrict__ g,
                                                                    float* __restrict__ d_y0) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= M * (int64_t)nu) return;
  const int64_t m = idx / nu;
  const int j = (int)(idx - m * nu);
  float carry = 0.f;  // (1 - alpha) G_{t+1}, or 0 across an episode start
  constexpr int kAhead = 8;  // steps whose loads are in flight together
  for (int64_t t0 = T - 1; t0 >= 0; t0 -= kAhead) {
    float v[kAhead];
    bool f[kAhead];
#pragma unroll
    for (int k = 0; k < kAhead; ++k) {
      const int64_t r = (t0 - k >= 0 ? t0 - k : 0) * M + m;
      v[k] = g[r * ld + j];
      f[k] = fresh && fresh[r];
    }
#pragma unroll
    for (int k = 0; k < kAhead; ++k)
      if (t0 - k >= 0) {
        const float G = v[k] + carry;
        g[((t0 - k) * M + m) * ld + j] = alpha * G;
        carry = f[k] ? 0.f : (1.f - alpha) * G;
      }
  }
  if (d_y0) d_y0[idx] = carry;
}

// mirrored rows: out[r][j] = sign[j] * x[r][perm[j]]
__global__ __launch_bounds__(256) void signed_permute_kernel(int64_t total, int n, const float* __restrict__ x, const int* __restrict__ perm,
                                                             const float* __restrict__ sign, float* __restrict__ out) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int64_t r = idx / n;
  const int j = (int)(idx - r * n);
  out[idx] = sign[j] * x[r * n + perm[j]];
}

// One thread per (row, j): diff = y[r][j] - sign[j] ym[r][perm[j]].  perm is a bijection, so the thread owns dym[r][perm[j]].
// The row's loss is summed by the thread of j = 0 over the row, in index order.
__global__ __launch_bounds__(256) void mirror_loss_grad_kernel(int64_t rows, int n, float scale, const float* __restrict__ y,
                                                               const float* __restrict__ ym, const int* __restrict__ perm,
                                                               const float* __restrict__ sign, float* __restrict__ dy,
                                                               float* __restrict__ dym, float* __restrict__ loss) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= rows * n) return;
  const int64_t r = idx / n;
  const int j = (int)(idx - r * n);
  const float c = 2.f * scale / ((float)n * (float)rows);
  const int pj = perm[j];
  const float sj = sign[j];
  const float diff = y[idx] - sj * ym[r * n + pj];
  dy[idx] += c * diff;
  dym[r * n + pj] = -c * sj * diff;
  if (loss && j == 0) {
    float s = 0.f;
    for (int k = 0; k < n; ++k) {
      const float d = y[r * n + k] - sign[k] * ym[r * n + perm[k]];
      s += d * d;
    }
    loss[r] = scale * s / (float)n;
  }
}

}  // namespace ks

static float lowpass_alpha(float ctrl_dt, float cutoff) {  // actions.py:254-255, in float like ks_action_filter
  return ctrl_dt / (1.f / (6.28318530717958647692f * cutoff) + ctrl_dt);
}

extern "C" int ks_lowpass_scan(ks_stream_t stream, int64_t T, int64_t M, int32_t nu, int32_t ld, float ctrl_dt, float cutoff,
                               const float* x, const float* mean_bias, const float* add, int64_t add_ld, int32_t add_first,
                               int32_t add_count, const float* y0, const uint8_t* fresh, float* y, float* y_last) {
  if (T < 0 || M < 0 || nu < 1 || ld < nu) return ks::fail(KS_EINVAL, "ks_lowpass_scan: bad shape (T %lld, M %lld, nu %d, ld %d)", (long long)T, (long long)M, nu, ld);
  if (!(ctrl_dt > 0.f) || !(cutoff > 0.f)) return ks::fail(KS_EINVAL, "ks_lowpass_scan: ctrl_dt and the cutoff frequency must be positive");
  if (T == 0 || M == 0) return KS_OK;
  if (!x || !y) return ks::fail(KS_EINVAL, "ks_lowpass_scan: null pointer");
  if (add && (add_first < 0 || add_count < 1 || add_first + add_count > nu || add_ld < add_count))
    return ks::fail(KS_EINVAL, "ks_lowpass_scan: the additive bias covers joints [%d, %d) of %d with rows of %lld floats", add_first,
                    add_first + add_count, nu, (long long)add_ld);
  const int64_t total = M * ld, grid = (total + 255) / 256;
  if (grid > 0x7fffffff) return ks::fail(KS_ELIMIT, "ks_lowpass_scan: too many elements");
  hipLaunchKernelGGL(ks::lowpass_scan_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, T, M, nu, ld,
                     lowpass_alpha(ctrl_dt, cutoff), x, mean_bias, add, add_ld, add_first, add_count, y0, fresh, y, y_last);
  return ks::check_launch("ks_lowpass_scan");
}

extern "C" int ks_lowpass_scan_backward(ks_stream_t stream, int64_t T, int64_t M, int32_t nu, int32_t ld, float ctrl_dt, float cutoff,
                                        const uint8_t* fresh, float* g, float* d_y0) {
  if (T < 0 || M < 0 || nu < 1 || ld < nu) return ks::fail(KS_EINVAL, "ks_lowpass_scan_backward: bad shape");
  if (!(ctrl_dt > 0.f) || !(cutoff > 0.f)) return ks::fail(KS_EINVAL, "ks_lowpass_scan_backward: ctrl_dt and the cutoff frequency must be positive");
  if (T == 0 || M == 0) return KS_OK;
  if (!g) return ks::fail(KS_EINVAL, "ks_lowpass_scan_backward: null pointer");
  const int64_t total = M * nu, grid = (total + 255) / 256;
  if (grid > 0x7fffffff) return ks::fail(KS_ELIMIT, "ks_lowpass_scan_backward: too many elements");
  hipLaunchKernelGGL(ks::lowpass_scan_backward_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, T, M, nu, ld,
                     lowpass_alpha(ctrl_dt, cutoff), fresh, g, d_y0);
  return ks::check_launch("ks_lowpass_scan_backward");
}

extern "C" int ks_signed_permute(ks_stream_t stream, int64_t rows, int32_t n, const float* x, const int32_t* perm, const float* sign,
                                 float* out) {
  if (rows < 0 || n < 1) return ks::fail(KS_EINVAL, "ks_signed_permute: bad shape");
  if (rows == 0) return KS_OK;
  if (!x || !perm || !sign || !out || x == out) return ks::fail(KS_EINVAL, "ks_signed_permute: null pointer, or in place");
  const int64_t total = rows * n, grid = (total + 255) / 256;
  if (grid > 0x7fffffff) return ks::fail(KS_ELIMIT, "ks_signed_permute: too many elements");
  hipLaunchKernelGGL(ks::signed_permute_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, total, n, x, perm, sign, out);
  return ks::check_launch("ks_signed_permute");
}

extern "C" int ks_mirror_loss_grad(ks_stream_t stream, int64_t rows, int32_t n, float scale, const float* y, const float* ym,
                                   const int32_t* perm, const float* sign, float* dy, float* dym, float* loss) {
  if (rows < 1 || n < 1) return ks::fail(KS_EINVAL, "ks_mirror_loss_grad: bad shape");
  if (!y || !ym || !perm || !sign || !dy || !dym) return ks::fail(KS_EINVAL, "ks_mirror_loss_grad: null pointer");
  const int64_t total = rows * n, grid = (total + 255) / 256;
  if (grid > 0x7fffffff) return ks::fail(KS_ELIMIT, "ks_mirror_loss_grad: too many elements");
  hipLaunchKernelGGL(ks::mirror_loss_grad_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, rows, n, scale, y, ym, perm,
                     sign, dy, dym, loss);
  return ks::check_launch("ks_mirror_loss_grad");
}

extern "C" int ks_ppo_adapt_kl(ks_stream_t stream, int64_t rows, int32_t A, const float* on_log_probs, const float* log_probs,
                               float kl_coef, float desired_kl, float* kl_scale, float* workspace) {
  if (rows < 1 || A < 1) return ks::fail(KS_EINVAL, "ks_ppo_adapt_kl: bad shape");
  if (!on_log_probs || !log_probs || !kl_scale || !workspace) return ks::fail(KS_EINVAL, "ks_ppo_adapt_kl: null pointer");
  if (!(kl_coef > 0.f) || !(desired_kl > 0.f)) return ks::fail(KS_EINVAL, "ks_ppo_adapt_kl: kl_coef and desired_kl must be positive");
  const int64_t n = rows * A;
  const int64_t want = (n + 1023) / 1024;
  const int blocks = (int)(want < 256 ? want : 256);
  hipLaunchKernelGGL(ks::kl_parts_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, n, on_log_probs, log_probs, workspace);
  hipLaunchKernelGGL(ks::kl_adapt_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, blocks, 1.f / (float)rows, kl_coef, desired_kl,
                     (const float*)workspace, kl_scale);
  return ks::check_launch("ks_ppo_adapt_kl");
}

extern "C" int ks_gaussian_log_prob(ks_stream_t stream, int64_t M, int32_t nu, const float* mean, const float* log_std,
                                    const float* action, float* log_prob, float* entropy) {
  if (M < 0 || nu < 1) return ks::fail(KS_EINVAL, "ks_gaussian_log_prob: bad shape");
  if (M == 0) return KS_OK;
  if (!mean || !log_std || !action || !log_prob) return ks::fail(KS_EINVAL, "ks_gaussian_log_prob: null pointer");
  const int64_t n = M * nu;
  hipLaunchKernelGGL(ks::gaussian_log_prob_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, n, nu, mean,
                     log_std, action, log_prob, entropy);
  return ks::check_launch("ks_gaussian_log_prob");
}

extern "C" int ks_ppo_loss_grad(ks_stream_t stream, int64_t M, int32_t nu, const KsPpoLossParams* params, const float* mean,
                                const float* log_std, const float* action, const float* on_log_probs,
                                const float* advantages, const float* value_targets, const float* on_values,
                                const float* values, float* d_mean, float* d_value, float* d_log_std, void* workspace) {
  if (!params) return ks::fail(KS_EINVAL, "ks_ppo_loss_grad: null parameters");
  if (M < 1 || nu < 1 || nu > KS_MAX_ACTIONS) return ks::fail(KS_EINVAL, "ks_ppo_loss_grad: bad shape (1..%d actions)", KS_MAX_ACTIONS);
  if (!mean || !log_std || !action || !on_log_probs || !advantages || !value_targets || !on_values || !values || !d_mean ||
      !d_value || !d_log_std || !workspace)
    return ks::fail(KS_EINVAL, "ks_ppo_loss_grad: null pointer");
  const int64_t want = (M + 255) / 256;
  const int blocks = (int)(want < KS_PPO_GRAD_BLOCKS ? want : KS_PPO_GRAD_BLOCKS);
  hipLaunchKernelGGL(ks::ppo_loss_grad_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, M, nu, *params, mean, log_std, action,
                     on_log_probs, advantages, value_targets, on_values, values, d_mean, d_value, (float*)workspace);
  hipLaunchKernelGGL(ks::ppo_grad_finish_kernel, dim3(nu), dim3(256), 0, (hipStream_t)stream, blocks, nu, (const float*)workspace,
                     d_log_std);
  return ks::check_launch("ks_ppo_loss_grad");
}

extern "C" int ks_ppo_loss_grad_head(ks_stream_t stream, int64_t M, int32_t nu, const KsPpoLossParams* params,
                                     const KsGaussianHead* head, const float* raw, const float* action, const float* on_log_probs,
                                     const float* advantages, const float* value_targets, const float* on_values,
                                     const float* values, float* d_raw, float* d_value) {
  if (!params || !head) return ks::fail(KS_EINVAL, "ks_ppo_loss_grad_head: null parameters");
  if (M < 1 || nu < 1) return ks::fail(KS_EINVAL, "ks_ppo_loss_grad_head: bad shape");
  if (!raw || !action || !on_log_probs || !advantages || !value_targets || !on_values || !values || !d_raw || !d_value)
    return ks::fail(KS_EINVAL, "ks_ppo_loss_grad_head: null pointer");
  if (!(head->max_std > 0.f) || head->min_std < 0.f || !(head->var_scale > 0.f))
    return ks::fail(KS_EINVAL, "ks_ppo_loss_grad_head: bad deviation bounds");
  const int64_t grid = (M + 255) / 256;
  if (grid > 0x7fffffff) return ks::fail(KS_ELIMIT, "ks_ppo_loss_grad_head: too many rows");
  hipLaunchKernelGGL(ks::ppo_loss_grad_head_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, M, nu, *params, *head, raw,
                     action, on_log_probs, advantages, value_targets, on_values, values, d_raw, d_value);
  return ks::check_launch("ks_ppo_loss_grad_head");
}

extern "C" int ks_gaussian_head_log_prob(ks_stream_t stream, int64_t M, int32_t nu, const KsGaussianHead* head, const float* raw,
                                         const float* action, float* log_prob, float* entropy) {
  if (M < 0 || nu < 1) return ks::fail(KS_EINVAL, "ks_gaussian_head_log_prob: bad shape");
  if (M == 0) return KS_OK;
  if (!head || !raw || !action || !log_prob) return ks::fail(KS_EINVAL, "ks_gaussian_head_log_prob: null pointer");
  if (!(head->max_std > 0.f) || head->min_std < 0.f || !(head->var_scale > 0.f))
    return ks::fail(KS_EINVAL, "ks_gaussian_head_log_prob: bad deviation bounds");
  const int64_t n = M * nu, grid = (n + 255) / 256;
  if (grid > 0x7fffffff) return ks::fail(KS_ELIMIT, "ks_gaussian_head_log_prob: too many elements");
  hipLaunchKernelGGL(ks::gaussian_head_log_prob_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, n, nu, *head, raw, action,
                     log_prob, entropy);
  return ks::check_launch("ks_gaussian_head_log_prob");
}

extern "C" int ks_ppo_loss_grad_mixture(ks_stream_t stream, int64_t M, int32_t nu, const KsPpoLossParams* params,
                                        const KsMixtureHead* head, const float* raw, const float* action, const float* on_log_probs,
                                        const float* advantages, const float* value_targets, const float* on_values,
                                        const float* values, float* d_raw, float* d_value) {
  if (!params || !head) return ks::fail(KS_EINVAL, "ks_ppo_loss_grad_mixture: null parameters");
  if (M < 1 || nu < 1) return ks::fail(KS_EINVAL, "ks_ppo_loss_grad_mixture: bad shape");
  if (head->num_mixtures < 1 || head->num_mixtures > KS_MAX_MIXTURES)
    return ks::fail(KS_ELIMIT, "ks_ppo_loss_grad_mixture: %d components, 1..%d are built", head->num_mixtures, KS_MAX_MIXTURES);
  if (!raw || !action || !on_log_probs || !advantages || !value_targets || !on_values || !values || !d_raw || !d_value)
    return ks::fail(KS_EINVAL, "ks_ppo_loss_grad_mixture: null pointer");
  if (!(head->max_std > 0.f) || head->min_std < 0.f || !(head->var_scale > 0.f))
    return ks::fail(KS_EINVAL, "ks_ppo_loss_grad_mixture: bad deviation bounds");
  if ((head->clip_lo == nullptr) != (head->clip_hi == nullptr)) return ks::fail(KS_EINVAL, "ks_ppo_loss_grad_mixture: clip_lo and clip_hi come together");
  const int64_t grid = (M + 127) / 128;
  if (grid > 0x7fffffff) return ks::fail(KS_ELIMIT, "ks_ppo_loss_grad_mixture: too many rows");
  hipLaunchKernelGGL(ks::ppo_loss_grad_mixture_kernel, dim3((unsigned)grid), dim3(128), 0, (hipStream_t)stream, M, nu, *params, *head, raw,
                     action, on_log_probs, advantages, value_targets, on_values, values, d_raw, d_value);
  return ks::check_launch("ks_ppo_loss_grad_mixture");
}
