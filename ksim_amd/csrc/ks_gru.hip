// GRU and LSTM cells for recurrent policies in the rollout, and the GRU's backward pass through time.  The two gate projections are plain linear
// layers and run through the MLP entry points (matrix cores for bf16); one streaming kernel then combines the gates.
#include "ks_common.h"

#include <vector>

namespace ks {

// gi = W_ih x + b (M, 3H), gh = W_hh h + (0, 0, b_n) (M, 3H), gate order reset | update | candidate:
//   r = sigmoid(gi_r + gh_r), z = sigmoid(gi_z + gh_z), n = tanh(gi_n + r * gh_n), h' = n + z (h - n)
// An env that starts an episode (fresh[m] != 0) takes h = 0; gh was computed from the stored h, so its
// contribution is replaced by the bias part alone, which for zero h is (0, 0, b_n).
__global__ __launch_bounds__(256) void gru_gate_kernel(int64_t M, int H, const float* __restrict__ gi,
                                                       const float* __restrict__ gh, const float* __restrict__ h_in,
                                                       const float* __restrict__ bias_n, const uint8_t* __restrict__ fresh,
                                                       float* __restrict__ h_out) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= M * H) return;
  const int64_t m = idx / H;
  const int j = (int)(idx - m * H);
  const bool f = fresh && fresh[m];
  const float* a = gi + m * 3 * H;
  const float* b = gh + m * 3 * H;
  const float hr = f ? 0.f : b[j], hz = f ? 0.f : b[H + j], hn = f ? bias_n[j] : b[2 * H + j];
  const float h = f ? 0.f : h_in[idx];
  const float r = 1.f / (1.f + expf(-(a[j] + hr)));
  const float z = 1.f / (1.f + expf(-(a[H + j] + hz)));
  const float n = tanhf(a[2 * H + j] + r * hn);
  h_out[idx] = n + z * (h - n);
}

// The same cell for training: also keeps what the backward pass needs, saved (M, 5H) = r | z | n | hn | h, where hn is the
// hidden part of the candidate (what r multiplies) and h the hidden state the cell actually used (zero for a fresh env).
__global__ __launch_bounds__(256) void gru_gate_train_kernel(int64_t M, int H, const float* __restrict__ gi,
                                                             const float* __restrict__ gh, const float* __restrict__ h_in,
                                                             const float* __restrict__ bias_n, const uint8_t* __restrict__ fresh,
                                                             float* __restrict__ h_out, float* __restrict__ saved) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= M * H) return;
  const int64_t m = idx / H;
  const int j = (int)(idx - m * H);
  const bool f = fresh && fresh[m];
  const float* a = gi + m * 3 * H;
  const float* b = gh + m * 3 * H;
  const float hr = f ? 0.f : b[j], hz = f ? 0.f : b[H + j], hn = f ? bias_n[j] : b[2 * H + j];
  const float h = f ? 0.f : h_in[idx];
  const float r = 1.f / (1.f + expf(-(a[j] + hr)));
  const float z = 1.f / (1.f + expf(-(a[H + j] + hz)));
  const float n = tanhf(a[2 * H + j] + r * hn);
  h_out[idx] = n + z * (h - n);
  float* sv = saved + m * 5 * H;
  sv[j] = r; sv[H + j] = z; sv[2 * H + j] = n; sv[3 * H + j] = hn; sv[4 * H + j] = h;
}

// Backward through the gates of one step.  dh_out is the gradient reaching h' (from the layer above at this step plus
// from the next step).  d_gi (M, 3H) is the gradient of the input projection's output, d_gh (M, 3H) that of the hidden
// projection's output (its n part is also the gradient of bias_n, fresh rows included); dh_in = dh_out * z is the direct
// path to the previous hidden state, zero for a fresh env (the hidden projection adds its share afterwards).
__global__ __launch_bounds__(256) void gru_gate_backward_kernel(int64_t M, int H, const float* __restrict__ dh_out,
                                                                const float* __restrict__ saved, const uint8_t* __restrict__ fresh,
                                                                float* __restrict__ d_gi, float* __restrict__ d_gh,
                                                                float* __restrict__ dh_in) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= M * H) return;
  const int64_t m = idx / H;
  const int j = (int)(idx - m * H);
  const bool f = fresh && fresh[m];
  const float* sv = saved + m * 5 * H;
  const float r = sv[j], z = sv[H + j], n = sv[2 * H + j], hn = sv[3 * H + j], h = sv[4 * H + j];
  const float d = dh_out[idx];
  const float dn_pre = d * (1.f - z) * (1.f - n * n);
  const float dz_pre = d * (h - n) * z * (1.f - z);
  const float dr_pre = dn_pre * hn * r * (1.f - r);
  float* a = d_gi + m * 3 * H;
  float* b = d_gh + m * 3 * H;
  a[j] = dr_pre; a[H + j] = dz_pre; a[2 * H + j] = dn_pre;
  b[j] = dr_pre; b[H + j] = dz_pre; b[2 * H + j] = dn_pre * r;
  dh_in[idx] = f ? 0.f : d * z;
}

// LSTM: g = W_ih x + W_hh h + b (M, 4H) in gate order input | forget | cell | output:
//   c' = sigmoid(f) c + sigmoid(i) tanh(g),  h' = sigmoid(o) tanh(c').  A fresh env starts from h = c = 0, which
// leaves only the input projection (it carries the whole bias).
__global__ __launch_bounds__(256) void lstm_gate_kernel(int64_t M, int H, const float* __restrict__ gi,
                                                        const float* __restrict__ gh, const float* __restrict__ c_in,
                                                        const uint8_t* __restrict__ fresh, float* __restrict__ h_out,
                                                        float* __restrict__ c_out) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= M * H) return;
  const int64_t m = idx / H;
  const int j = (int)(idx - m * H);
  const bool f = fresh && fresh[m];
  const float* a = gi + m * 4 * H;
  const float* b = gh + m * 4 * H;
  float g[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) g[k] = a[k * H + j] + (f ? 0.f : b[k * H + j]);
  const float c = f ? 0.f : c_in[idx];
  const float si = 1.f / (1.f + expf(-g[0])), sf = 1.f / (1.f + expf(-g[1])), so = 1.f / (1.f + expf(-g[3]));
  const float cn = sf * c + si * tanhf(g[2]);
  c_out[idx] = cn;
  h_out[idx] = so * tanhf(cn);
}

// The LSTM cell for training: saved (M, 7H) = i | f | g | o | tanh(c') | c | h with the gate activations, the cell and
// hidden state the step actually used (zero for a fresh env).
__global__ __launch_bounds__(256) void lstm_gate_train_kernel(int64_t M, int H, const float* __restrict__ gi,
                                                              const float* __restrict__ gh, const float* __restrict__ h_in,
                                                              const float* __restrict__ c_in, const uint8_t* __restrict__ fresh,
                                                              float* __restrict__ h_out, float* __restrict__ c_out,
                                                              float* __restrict__ saved) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= M * H) return;
  const int64_t m = idx / H;
  const int j = (int)(idx - m * H);
  const bool f = fresh && fresh[m];
  const float* a = gi + m * 4 * H;
  const float* b = gh + m * 4 * H;
  float g[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) g[k] = a[k * H + j] + (f ? 0.f : b[k * H + j]);
  const float c = f ? 0.f : c_in[idx], h = f ? 0.f : h_in[idx];
  const float si = 1.f / (1.f + expf(-g[0])), sf = 1.f / (1.f + expf(-g[1])), so = 1.f / (1.f + expf(-g[3]));
  const float tg = tanhf(g[2]);
  const float cn = sf * c + si * tg;
  const float tc = tanhf(cn);
  c_out[idx] = cn;
  h_out[idx] = so * tc;
  float* sv = saved + m * 7 * H;
  sv[j] = si; sv[H + j] = sf; sv[2 * H + j] = tg; sv[3 * H + j] = so; sv[4 * H + j] = tc; sv[5 * H + j] = c; sv[6 * H + j] = h;
}

// Backward through the gates of one LSTM step: dh_out, dc_out are the gradients reaching h' and c'.  d_g (M, 4H) is the
// gradient of the summed gate pre-activations, hence of both projections' outputs; dc_in = dc f is the gradient of the
// incoming cell state and dh_in starts at zero (the hidden projection adds its share afterwards); both are zero for a fresh env.
__global__ __launch_bounds__(256) void lstm_gate_backward_kernel(int64_t M, int H, const float* __restrict__ dh_out,
                                                                 const float* __restrict__ dc_out, const float* __restrict__ saved,
                                                                 const uint8_t* __restrict__ fresh, float* __restrict__ d_g,
                                                                 float* __restrict__ dh_in, float* __restrict__ dc_in) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= M * H) return;
  const int64_t m = idx / H;
  const int j = (int)(idx - m * H);
  const bool f = fresh && fresh[m];
  const float* sv = saved + m * 7 * H;
  const float si = sv[j], sf = sv[H + j], tg = sv[2 * H + j], so = sv[3 * H + j], tc = sv[4 * H + j], c = sv[5 * H + j];
  const float dh = dh_out[idx];
  const float dc = dc_out[idx] + dh * so * (1.f - tc * tc);
  float* a = d_g + m * 4 * H;
  a[j] = dc * tg * si * (1.f - si);
  a[H + j] = dc * c * sf * (1.f - sf);
  a[2 * H + j] = dc * si * (1.f - tg * tg);
  a[3 * H + j] = dh * tc * so * (1.f - so);
  dc_in[idx] = f ? 0.f : dc * sf;
  dh_in[idx] = 0.f;
}

// ---------------------------------------------------------------- a whole trajectory of one LSTM layer in one launch
// The step-by-step path costs two GEMM launches and a gate kernel per step, layer and network: a minibatch of 100 control steps
// is thousands of launches of a few microseconds each.  Here a workgroup of eight wavefronts owns 4 rows (envs) for all T
// steps, so that a minibatch of a thousand rows is one workgroup per CU.  The product runs on v_mfma_f32_4x4x1 (sixteen
// independent 4x4 outer products per instruction): block b = lane / 4 of wavefront w is hidden unit 16 w + b, its four B entries
// are that unit's input / forget / cell / output rows of W_hh and the four A entries, the same for every block and therefore
// broadcast from one block, the four rows' hidden state; after K = 128 instructions and a 4 x 4 transpose inside each group of
// four lanes, lane (b, j) holds the four gate pre-activations of its unit for row j.  The wavefront's slice of W_hh stays in
// 128 vector registers per lane for the whole sequence, the hidden state of the 4 rows lives in LDS (double buffered), the
// cell state in a register; a step is 128 MFMAs (the fp32 matrix rate: 4 rows x 512 x 128 multiply-adds per CU), the gate
// arithmetic of one (unit, row) per lane, and one barrier.  fp32 cells of hidden size 128.
typedef __attribute__((ext_vector_type(4))) float f32x4;
constexpr int kSeqRows = 4, kSeqH = 128, kSeqWaves = 8, kSeqPadH = kSeqH + 4, kSeqPadG = 4 * kSeqH + 4;

__device__ __forceinline__ float sigmoid_ks(float x) { return 1.f / (1.f + expf(-x)); }

// 1 / (1 + e^-x) and tanh x = 1 - 2 / (e^2x + 1) on v_exp_f32 and v_rcp_f32; both saturate correctly (e^y = inf gives 0 and -1 + 2 = 1)
__device__ __forceinline__ float seq_sigmoid(float x) { return __builtin_amdgcn_rcpf(1.f + __expf(-x)); }
__device__ __forceinline__ float seq_tanh(float x) { return 1.f - 2.f * __builtin_amdgcn_rcpf(__expf(2.f * x) + 1.f); }

// Barrier for data that the wavefronts of a workgroup hand each other through LDS only: it waits for this wavefront's LDS
// traffic, not for its global loads and stores.  __syncthreads() would also drain the step's stores (and the loads fetched
// ahead for the next step) before every barrier, a memory round trip per step of the sequence.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// where hidden unit u of a row sits in the LDS copy of the state: unit u = 16 q + b is register q of block b (see the forward
// kernel), and a lane reads its block's 8 registers as 8 consecutive floats
__device__ __forceinline__ int seq_slot(int u) { return 8 * (u & 15) + (u >> 4); }

// Transpose of a 4 x 4 block held by four neighbouring lanes (lane j of the group holds a0..a3): out[g] = a_j of lane g.
// Three lane exchanges within the group (DPP quad permutes): for d = 1, 2, 3 lane s sends its entry s ^ d to lane s ^ d.
__device__ __forceinline__ float pick4(float a0, float a1, float a2, float a3, int i) {
  return i == 0 ? a0 : (i == 1 ? a1 : (i == 2 ? a2 : a3));
}
__device__ __forceinline__ void quad_transpose(float a0, float a1, float a2, float a3, int j, float (&out)[4]) {
  const float own = pick4(a0, a1, a2, a3, j);
  const float s1 = pick4(a0, a1, a2, a3, j ^ 1), s2 = pick4(a0, a1, a2, a3, j ^ 2), s3 = pick4(a0, a1, a2, a3, j ^ 3);
  const float r1 = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, s1), 0xB1, 0xf, 0xf, true));  // quad_perm [1,0,3,2]
  const float r2 = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, s2), 0x4E, 0xf, 0xf, true));  // quad_perm [2,3,0,1]
  const float r3 = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, s3), 0x1B, 0xf, 0xf, true));  // quad_perm [3,2,1,0]
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int d = g ^ j;
    out[g] = d == 0 ? own : (d == 1 ? r1 : (d == 2 ? r2 : r3));
  }
}

__global__ __launch_bounds__(64 * kSeqWaves) __attribute__((amdgpu_waves_per_eu(2, 2)))
void lstm_seq_forward_kernel(int T, int64_t M, int groups, const float* __restrict__ gi, const float* __restrict__ W, int ldw,
                             const float* h0, const float* c0, const uint8_t* __restrict__ fresh,
                             float* hs, float* cs, float* __restrict__ saved) {  // with T = 1, hs / cs may be h0 / c0
  constexpr int H = kSeqH;
  __shared__ __attribute__((aligned(16))) float sh[2][kSeqRows][kSeqPadH];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int j = lane & 3, unit = 16 * wave + (lane >> 2);
  // The weights are the B operand: block b, entry lane % 4: W_hh[gate lane % 4, unit][k].  The hidden state is the A operand and
  // is the same for all sixteen blocks, so it is broadcast from one block per instruction (CBSZ = 4, ABID = k % 16): the four
  // lanes of block k % 16 hold h[row 0..3][k] in register k / 16, i.e. the 512 values of the state sit once in 8 registers of the
  // wavefront instead of once per block.  In LDS the state is stored in that order (row, block, register), two 16-byte reads per
  // lane and step.
  float wa[H];
  {
    const float4* src = reinterpret_cast<const float4*>(W + (int64_t)(j * H + unit) * ldw);
#pragma unroll
    for (int k4 = 0; k4 < H / 4; ++k4) {
      const float4 v = src[k4];
      wa[4 * k4] = v.x; wa[4 * k4 + 1] = v.y; wa[4 * k4 + 2] = v.z; wa[4 * k4 + 3] = v.w;
    }
  }
  // A workgroup takes `groups` sets of 4 rows one after the other with the same registers of weights: a single step over
  // thousands of rows (the rollout's call) would otherwise fetch the 256 KB of W_hh once per 4 rows.
  for (int grp = 0; grp < groups; ++grp) {
  const int64_t r0 = ((int64_t)blockIdx.x * groups + grp) * kSeqRows;
  if (r0 >= M) break;  // the same for every thread of the workgroup
  const int64_t m = r0 + j;
  const bool row_ok = m < M;
  const int64_t mc = row_ok ? m : M - 1;  // loads of the rows past the batch are clamped, their stores dropped
  if (grp > 0) __syncthreads();  // the previous set's last read of the state buffers is over
  float c = c0[mc * H + unit];
  float hprev = h0[mc * H + unit];  // the state this lane's (unit, row) enters the step with
  sh[0][j][seq_slot(unit)] = hprev;
  __syncthreads();
  int cur = 0;
  // the step's inputs from memory are fetched one step ahead: their latency would otherwise stand between the matrix work and the gates
  float gnext[4];
  uint8_t fnext = 0;
#pragma unroll
  for (int g = 0; g < 4; ++g) gnext[g] = gi[mc * 4 * H + g * H + unit];
  if (fresh) fnext = fresh[mc];
  for (int t = 0; t < T; ++t) {
    float gin[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) gin[g] = gnext[g];
    const bool f = fnext != 0;
    if (t + 1 < T) {
      const int64_t tn = (int64_t)(t + 1) * M + mc;
#pragma unroll
      for (int g = 0; g < 4; ++g) gnext[g] = gi[tn * 4 * H + g * H + unit];
      if (fresh) fnext = fresh[tn];
    }
    f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
    float ha[8];
    {
      const float4 a0 = *reinterpret_cast<const float4*>(&sh[cur][j][8 * (lane >> 2)]);
      const float4 a1 = *reinterpret_cast<const float4*>(&sh[cur][j][8 * (lane >> 2) + 4]);
      ha[0] = a0.x; ha[1] = a0.y; ha[2] = a0.z; ha[3] = a0.w; ha[4] = a1.x; ha[5] = a1.y; ha[6] = a1.z; ha[7] = a1.w;
    }
    // k runs 0..127 in order, even k into one accumulator and odd k into the other
#define KS_SEQ_MFMA(K0)                                                                                            \
    acc0 = __builtin_amdgcn_mfma_f32_4x4x1f32(ha[(K0) >> 4], wa[(K0)], acc0, 4, (K0) & 15, 0);                       \
    acc1 = __builtin_amdgcn_mfma_f32_4x4x1f32(ha[((K0) + 1) >> 4], wa[(K0) + 1], acc1, 4, ((K0) + 1) & 15, 0);
#define KS_SEQ_MFMA8(K0) KS_SEQ_MFMA(K0) KS_SEQ_MFMA((K0) + 2) KS_SEQ_MFMA((K0) + 4) KS_SEQ_MFMA((K0) + 6)
#define KS_SEQ_MFMA32(K0) KS_SEQ_MFMA8(K0) KS_SEQ_MFMA8((K0) + 8) KS_SEQ_MFMA8((K0) + 16) KS_SEQ_MFMA8((K0) + 24)
    KS_SEQ_MFMA32(0) KS_SEQ_MFMA32(32) KS_SEQ_MFMA32(64) KS_SEQ_MFMA32(96)
#undef KS_SEQ_MFMA32
#undef KS_SEQ_MFMA8
#undef KS_SEQ_MFMA
    // lane (unit, gate lane % 4) now holds that gate for the four rows in its four registers; the gates want the transpose
    // within each group of four lanes: lane (unit, row j) with the four gates
    float pre[4];
    quad_transpose(acc0[0] + acc1[0], acc0[1] + acc1[1], acc0[2] + acc1[2], acc0[3] + acc1[3], j, pre);
    const float cp = f ? 0.f : c, hu = f ? 0.f : hprev;
    // the hardware exponential and reciprocal (about 1 ulp each) instead of the library's expf, tanhf and IEEE division: a
    // fifth of the instructions, and the gates are as many instructions per step as the matrix work is cycles
    const float si = seq_sigmoid(gin[0] + (f ? 0.f : pre[0]));
    const float sf = seq_sigmoid(gin[1] + (f ? 0.f : pre[1]));
    const float tg = seq_tanh(gin[2] + (f ? 0.f : pre[2]));
    const float so = seq_sigmoid(gin[3] + (f ? 0.f : pre[3]));
    c = sf * cp + si * tg;
    const float tc = seq_tanh(c);
    const float hn = so * tc;
    hprev = hn;
    sh[cur ^ 1][j][seq_slot(unit)] = hn;
    if (row_ok) {
      const int64_t o = (int64_t)t * M + m;
      hs[o * H + unit] = hn;
      if (cs) cs[o * H + unit] = c;
      if (saved) {
        float* sv = saved + o * 7 * H + unit;
        sv[0] = si; sv[H] = sf; sv[2 * H] = tg; sv[3 * H] = so; sv[4 * H] = tc; sv[5 * H] = cp; sv[6 * H] = hu;
      }
    }
    lds_barrier();  // the new hidden state is complete; the buffer just read is free for the step after next
    cur ^= 1;
  }
  }
}

// The reverse sweep of the same layer: dH (T, M, H) is the gradient reaching h_t from the layer above; the gradient through
// W_hh and that of the cell state are carried in registers.  Per step: the gate derivatives from the saved activations
// (lstm_gate_backward_kernel's formulas) into d_g (T, M, 4H) and LDS, then dh_{t-1} = d_g W_hh over the transposed weights.
// Here the sixteen blocks of an MFMA are four groups of four units (entries i) times four quarters of the 4H gate rows
// (K split four ways): lane (b, j) accumulates, for row j, the partial sums over gate rows [128 (b / 4), 128 (b / 4) + 128) of the
// units 16 w + 4 (b % 4) + {0..3}; two lane exchanges add the quarters, and the lane keeps the unit 16 w + 4 (b % 4) + b / 4.
__global__ __launch_bounds__(64 * kSeqWaves) __attribute__((amdgpu_waves_per_eu(2, 2)))
void lstm_seq_backward_kernel(int T, int64_t M, const float* __restrict__ dH, const float* __restrict__ saved,
                              const uint8_t* __restrict__ fresh, const float* __restrict__ Wt, int ldwt,
                              float* __restrict__ d_g, float* __restrict__ dh0, float* __restrict__ dc0) {
  constexpr int H = kSeqH;
  __shared__ __attribute__((aligned(16))) float sg[kSeqRows][kSeqPadG];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int j = lane & 3, ug = (lane >> 2) & 3, kg = lane >> 4;
  const int unit = 16 * wave + 4 * ug + kg;  // the (unit, row j) whose gate arithmetic and carried gradients this lane owns
  const int64_t r0 = (int64_t)blockIdx.x * kSeqRows;
  const int64_t m = r0 + j;
  const bool row_ok = m < M;
  const int64_t mc = row_ok ? m : M - 1;
  // A operand of block b, entry i = lane % 4: Wt[unit 16 w + 4 ug + i][gate row 128 kg + s]
  float wa[128];
  {
    const float4* src = reinterpret_cast<const float4*>(Wt + (int64_t)(16 * wave + 4 * ug + j) * ldwt + 128 * kg);
#pragma unroll
    for (int s4 = 0; s4 < 32; ++s4) {
      const float4 v = src[s4];
      wa[4 * s4] = v.x; wa[4 * s4 + 1] = v.y; wa[4 * s4 + 2] = v.z; wa[4 * s4 + 3] = v.w;
    }
  }
  float dhc = 0.f, dc = 0.f;
  // the step's inputs from memory are fetched one step ahead, under the matrix work of the step before
  float nx[7];
  uint8_t fnext = 0;
  {
    const int64_t o = (int64_t)(T - 1) * M + mc;
    const float* sv = saved + o * 7 * H + unit;
#pragma unroll
    for (int k = 0; k < 6; ++k) nx[k] = sv[k * H];
    nx[6] = dH[o * H + unit];
    if (fresh) fnext = fresh[o];
  }
  for (int t = T - 1; t >= 0; --t) {
    const bool f = fnext != 0;
    const float si = nx[0], sf = nx[1], tg = nx[2], so = nx[3], tc = nx[4], cp = nx[5];
    const float dh = nx[6] + dhc;
    if (t > 0) {
      const int64_t o = (int64_t)(t - 1) * M + mc;
      const float* sv = saved + o * 7 * H + unit;
#pragma unroll
      for (int k = 0; k < 6; ++k) nx[k] = sv[k * H];
      nx[6] = dH[o * H + unit];
      if (fresh) fnext = fresh[o];
    }
    const float dct = dc + dh * so * (1.f - tc * tc);
    const float gI = dct * tg * si * (1.f - si), gF = dct * cp * sf * (1.f - sf), gG = dct * si * (1.f - tg * tg),
                gO = dh * tc * so * (1.f - so);
    dc = f ? 0.f : dct * sf;
    sg[j][unit] = gI; sg[j][H + unit] = gF; sg[j][2 * H + unit] = gG; sg[j][3 * H + unit] = gO;
    if (row_ok) {
      float* dg = d_g + ((int64_t)t * M + m) * 4 * H + unit;
      dg[0] = gI; dg[H] = gF; dg[2 * H] = gG; dg[3 * H] = gO;
    }
    lds_barrier();
    f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
    const float* grow = &sg[j][128 * kg];
#pragma unroll
    for (int s4 = 0; s4 < 32; ++s4) {
      const float4 gb = *reinterpret_cast<const float4*>(grow + 4 * s4);
      acc0 = __builtin_amdgcn_mfma_f32_4x4x1f32(wa[4 * s4], gb.x, acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_4x4x1f32(wa[4 * s4 + 1], gb.y, acc1, 0, 0, 0);
      acc0 = __builtin_amdgcn_mfma_f32_4x4x1f32(wa[4 * s4 + 2], gb.z, acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_4x4x1f32(wa[4 * s4 + 3], gb.w, acc1, 0, 0, 0);
    }
    float part[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float v = acc0[r] + acc1[r];
      v += __shfl_xor(v, 16);
      v += __shfl_xor(v, 32);
      part[r] = v;
    }
    const float mine = kg == 0 ? part[0] : (kg == 1 ? part[1] : (kg == 2 ? part[2] : part[3]));
    dhc = f ? 0.f : mine;
    lds_barrier();  // every wavefront has read this step's gate gradients
  }
  if (row_ok) {
    if (dh0) dh0[m * H + unit] = dhc;
    if (dc0) dc0[m * H + unit] = dc;
  }
}

}  // namespace ks

using namespace ks;

struct KsGru {
  int I, H;
  KsMlp *proj_i, *proj_h;
  float* bias_n;    // device (H)
  float* bias_tmp;  // device (3H), training only
};

extern "C" int ks_gru_create(const KsGruDesc* d, KsGru** out) {
  if (!d || !out) return fail(KS_EINVAL, "ks_gru_create: null argument");
  if (d->input_size < 1 || d->hidden_size < 1 || d->hidden_size > 21845) return fail(KS_EINVAL, "ks_gru_create: bad sizes %d -> %d", d->input_size, d->hidden_size);
  if (!d->weight_ih || !d->weight_hh) return fail(KS_EINVAL, "ks_gru_create: weights are required");
  const int H = d->hidden_size, I = d->input_size;
  std::vector<float> zero(3 * (size_t)H, 0.f), bh(3 * (size_t)H, 0.f);
  if (d->bias_n) for (int j = 0; j < H; ++j) bh[2 * (size_t)H + j] = d->bias_n[j];
  KsGru* g = new KsGru{I, H, nullptr, nullptr, nullptr, nullptr};
  KsMlpDesc md = {};
  md.n_layers = 1; md.activation = KS_ACT_NONE; md.dtype = d->dtype;
  md.dims[0] = I; md.dims[1] = 3 * H; md.weights[0] = d->weight_ih; md.biases[0] = d->bias ? d->bias : zero.data();
  int rc = ks_mlp_create(&md, &g->proj_i);
  if (rc == KS_OK) {
    md.dims[0] = H; md.weights[0] = d->weight_hh; md.biases[0] = bh.data();
    rc = ks_mlp_create(&md, &g->proj_h);
  }
  if (rc == KS_OK && (hipMalloc((void**)&g->bias_n, H * 4) != hipSuccess ||
                      hipMemcpy(g->bias_n, bh.data() + 2 * (size_t)H, H * 4, hipMemcpyHostToDevice) != hipSuccess))
    rc = fail(KS_ELAUNCH, "ks_gru_create: upload failed");
  if (rc != KS_OK) { ks_gru_destroy(g); return rc; }
  *out = g;
  return KS_OK;
}

extern "C" int ks_gru_destroy(KsGru* g) {
  if (!g) return KS_OK;
  ks_mlp_destroy(g->proj_i);
  ks_mlp_destroy(g->proj_h);
  if (g->bias_n) (void)hipFree(g->bias_n);
  if (g->bias_tmp) (void)hipFree(g->bias_tmp);
  delete g;
  return KS_OK;
}

static int64_t up256(int64_t n) { return (n + 255) / 256 * 256; }

extern "C" int64_t ks_gru_workspace_bytes(const KsGru* g, int64_t M) {
  if (!g || M < 0) return -1;
  const int64_t gates = up256(M * 3 * g->H * 4);
  return 2 * gates + up256(ks_mlp_workspace_bytes(g->proj_i, M)) + up256(ks_mlp_workspace_bytes(g->proj_h, M));
}

extern "C" int ks_gru_forward(const KsGru* g, ks_stream_t stream, int64_t M, const float* x, const float* h_in,
                              const uint8_t* fresh, float* h_out, void* workspace) {
  if (!g || !x || !h_in || !h_out) return fail(KS_EINVAL, "ks_gru_forward: null argument");
  if (M < 0) return fail(KS_EINVAL, "ks_gru_forward: negative row count");
  if (M == 0) return KS_OK;
  if (!workspace) return fail(KS_EINVAL, "ks_gru_forward: workspace is required");
  const int64_t gates = up256(M * 3 * g->H * 4);
  char* w = (char*)workspace;
  float* gi = (float*)w;
  float* gh = (float*)(w + gates);
  void* wi = w + 2 * gates;
  void* wh = w + 2 * gates + up256(ks_mlp_workspace_bytes(g->proj_i, M));
  int rc = ks_mlp_forward(g->proj_i, stream, M, x, gi, wi);
  if (rc != KS_OK) return rc;
  rc = ks_mlp_forward(g->proj_h, stream, M, h_in, gh, wh);
  if (rc != KS_OK) return rc;
  const int64_t n = M * g->H, grid = (n + 255) / 256;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_gru_forward: too many elements");
  hipLaunchKernelGGL(gru_gate_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, M, g->H, gi, gh, h_in,
                     g->bias_n, fresh, h_out);
  return check_launch("ks_gru_forward");
}

extern "C" int ks_gru_train_init(KsGru* g) {
  if (!g) return fail(KS_EINVAL, "ks_gru_train_init: null handle");
  int rc = ks_mlp_train_init(g->proj_i);
  if (rc == KS_OK) rc = ks_mlp_train_init(g->proj_h);
  // the hidden projection's bias is (0, 0, b_n): only its candidate part is a parameter of the cell
  if (rc == KS_OK) rc = ks_mlp_freeze_bias_prefix(g->proj_h, 0, 2 * g->H);
  if (rc == KS_OK && !g->bias_tmp && hipMalloc((void**)&g->bias_tmp, 3 * (size_t)g->H * 4) != hipSuccess)
    rc = fail(KS_ELAUNCH, "ks_gru_train_init: allocation failed");
  return rc;
}

extern "C" int ks_gru_projections(KsGru* g, KsMlp** input_projection, KsMlp** hidden_projection) {
  if (!g || !input_projection || !hidden_projection) return fail(KS_EINVAL, "ks_gru_projections: null argument");
  *input_projection = g->proj_i;
  *hidden_projection = g->proj_h;
  return KS_OK;
}

extern "C" int ks_gru_grad_sqnorm(const KsGru* g, ks_stream_t stream, double* acc) {
  if (!g || !acc) return fail(KS_EINVAL, "ks_gru_grad_sqnorm: null argument");
  const int rc = ks_mlp_grad_sqnorm(g->proj_i, stream, acc);
  return rc != KS_OK ? rc : ks_mlp_grad_sqnorm(g->proj_h, stream, acc);
}

extern "C" int ks_gru_adam_step(KsGru* g, ks_stream_t stream, const KsAdamParams* params, const double* sqnorm) {
  if (!g || !g->bias_tmp) return fail(KS_EINVAL, "ks_gru_adam_step: call ks_gru_train_init first");
  int rc = ks_mlp_adam_step(g->proj_i, stream, params, sqnorm);
  if (rc == KS_OK) rc = ks_mlp_adam_step(g->proj_h, stream, params, sqnorm);
  // the gate kernel's own copy of b_n (used for envs that start an episode) follows the hidden projection's bias
  if (rc == KS_OK) rc = ks_mlp_get_params(g->proj_h, stream, 0, nullptr, g->bias_tmp, 0);
  if (rc == KS_OK && hipMemcpyAsync(g->bias_n, g->bias_tmp + 2 * (size_t)g->H, (size_t)g->H * 4, hipMemcpyDeviceToDevice,
                                    (hipStream_t)stream) != hipSuccess)
    rc = fail(KS_ELAUNCH, "ks_gru_adam_step: bias copy failed");
  return rc;
}

extern "C" int ks_gru_train_forward(const KsGru* g, ks_stream_t stream, int64_t M, const float* x, const float* h_in,
                                    const uint8_t* fresh, float* h_out, float* saved, void* workspace) {
  if (!g || !x || !h_in || !h_out || !saved) return fail(KS_EINVAL, "ks_gru_train_forward: null argument");
  if (M < 0) return fail(KS_EINVAL, "ks_gru_train_forward: negative row count");
  if (M == 0) return KS_OK;
  if (!workspace) return fail(KS_EINVAL, "ks_gru_train_forward: workspace is required");
  const int64_t gates = up256(M * 3 * g->H * 4);
  char* w = (char*)workspace;
  float* gi = (float*)w;
  float* gh = (float*)(w + gates);
  void* wi = w + 2 * gates;
  void* wh = w + 2 * gates + up256(ks_mlp_workspace_bytes(g->proj_i, M));
  int rc = ks_mlp_forward(g->proj_i, stream, M, x, gi, wi);
  if (rc != KS_OK) return rc;
  rc = ks_mlp_forward(g->proj_h, stream, M, h_in, gh, wh);
  if (rc != KS_OK) return rc;
  const int64_t n = M * g->H, grid = (n + 255) / 256;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_gru_train_forward: too many elements");
  hipLaunchKernelGGL(gru_gate_train_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, M, g->H, gi, gh, h_in,
                     g->bias_n, fresh, h_out, saved);
  return check_launch("ks_gru_train_forward");
}

extern "C" int64_t ks_gru_backward_workspace_bytes(const KsGru* g, int64_t M) {
  if (!g || M < 0) return -1;
  return ks_mlp_train_workspace_bytes(g->proj_h, M);
}

extern "C" int ks_gru_backward_step(KsGru* g, ks_stream_t stream, int64_t M, const float* dh_out, const float* saved,
                                    const uint8_t* fresh, float* d_gi, float* d_gh, float* dh_in, void* workspace) {
  if (!g || !dh_out || !saved || !d_gi || !d_gh || !dh_in || !workspace) return fail(KS_EINVAL, "ks_gru_backward_step: null argument");
  if (M < 0) return fail(KS_EINVAL, "ks_gru_backward_step: negative row count");
  if (M == 0) return KS_OK;
  const int64_t n = M * g->H, grid = (n + 255) / 256;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_gru_backward_step: too many elements");
  hipLaunchKernelGGL(gru_gate_backward_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, M, g->H, dh_out, saved, fresh,
                     d_gi, d_gh, dh_in);
  int rc = check_launch("ks_gru_backward_step");
  if (rc != KS_OK) return rc;
  // dh_in += d_gh W_hh, except across an episode boundary
  return ks_mlp_train_backward_dx(g->proj_h, stream, M, nullptr, d_gh, dh_in, 0, 1, fresh, workspace);
}

struct KsLstm {
  int I, H;
  KsMlp *proj_i, *proj_h;
};

extern "C" int ks_lstm_create(const KsLstmDesc* d, KsLstm** out) {
  if (!d || !out) return fail(KS_EINVAL, "ks_lstm_create: null argument");
  if (d->input_size < 1 || d->hidden_size < 1 || d->hidden_size > 16384) return fail(KS_EINVAL, "ks_lstm_create: bad sizes %d -> %d", d->input_size, d->hidden_size);
  if (!d->weight_ih || !d->weight_hh) return fail(KS_EINVAL, "ks_lstm_create: weights are required");
  const int H = d->hidden_size, I = d->input_size;
  std::vector<float> zero(4 * (size_t)H, 0.f);
  KsLstm* g = new KsLstm{I, H, nullptr, nullptr};
  KsMlpDesc md = {};
  md.n_layers = 1; md.activation = KS_ACT_NONE; md.dtype = d->dtype;
  md.dims[0] = I; md.dims[1] = 4 * H; md.weights[0] = d->weight_ih; md.biases[0] = d->bias ? d->bias : zero.data();
  int rc = ks_mlp_create(&md, &g->proj_i);
  if (rc == KS_OK) {
    md.dims[0] = H; md.weights[0] = d->weight_hh; md.biases[0] = zero.data();
    rc = ks_mlp_create(&md, &g->proj_h);
  }
  if (rc != KS_OK) { ks_lstm_destroy(g); return rc; }
  *out = g;
  return KS_OK;
}

extern "C" int ks_lstm_destroy(KsLstm* g) {
  if (!g) return KS_OK;
  ks_mlp_destroy(g->proj_i);
  ks_mlp_destroy(g->proj_h);
  delete g;
  return KS_OK;
}

extern "C" int64_t ks_lstm_workspace_bytes(const KsLstm* g, int64_t M) {
  if (!g || M < 0) return -1;
  const int64_t gates = up256(M * 4 * g->H * 4);
  return 2 * gates + up256(ks_mlp_workspace_bytes(g->proj_i, M)) + up256(ks_mlp_workspace_bytes(g->proj_h, M));
}

extern "C" int ks_lstm_forward(const KsLstm* g, ks_stream_t stream, int64_t M, const float* x, const float* h_in,
                               const float* c_in, const uint8_t* fresh, float* h_out, float* c_out, void* workspace) {
  if (!g || !x || !h_in || !c_in || !h_out || !c_out) return fail(KS_EINVAL, "ks_lstm_forward: null argument");
  if (M < 0) return fail(KS_EINVAL, "ks_lstm_forward: negative row count");
  if (M == 0) return KS_OK;
  if (!workspace) return fail(KS_EINVAL, "ks_lstm_forward: workspace is required");
  const int64_t gates = up256(M * 4 * g->H * 4);
  char* w = (char*)workspace;
  float* gi = (float*)w;
  float* gh = (float*)(w + gates);
  void* wi = w + 2 * gates;
  void* wh = w + 2 * gates + up256(ks_mlp_workspace_bytes(g->proj_i, M));
  int rc = ks_mlp_forward(g->proj_i, stream, M, x, gi, wi);
  if (rc != KS_OK) return rc;
  // one step of the sequence kernel where it applies: a rollout's steps and the replay of its trajectory then give the same bits
  if (ks_lstm_sequence_supported(g)) return ks_lstm_sequence_forward(g, stream, 1, M, gi, h_in, c_in, fresh, h_out, c_out, nullptr);
  rc = ks_mlp_forward(g->proj_h, stream, M, h_in, gh, wh);
  if (rc != KS_OK) return rc;
  const int64_t n = M * g->H, grid = (n + 255) / 256;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_lstm_forward: too many elements");
  hipLaunchKernelGGL(lstm_gate_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, M, g->H, gi, gh, c_in, fresh,
                     h_out, c_out);
  return check_launch("ks_lstm_forward");
}

// whether the one-launch sequence kernels cover this cell: fp32, hidden size 128
static bool lstm_seq_weights(const KsLstm* g, const float** W, int* ldw, const float** Wt, int* ldwt) {
  const void *w = nullptr, *wt = nullptr;
  int np = 0, kp = 0, dt = 0;
  if (!g || g->H != kSeqH) return false;
  if (mlp_peek_layer(g->proj_h, 0, &w, &wt, &np, &kp, &dt) != KS_OK) return false;
  if (dt != KS_MLP_F32 || np != 4 * kSeqH || kp < kSeqH || (kp & 3)) return false;
  *W = (const float*)w; *ldw = kp;
  *Wt = (const float*)wt; *ldwt = np;
  return w != nullptr;
}

extern "C" int ks_lstm_sequence_supported(const KsLstm* g) {
  const float *W, *Wt;
  int a, b;
  return lstm_seq_weights(g, &W, &a, &Wt, &b) ? 1 : 0;
}

extern "C" int ks_lstm_sequence_forward(const KsLstm* g, ks_stream_t stream, int64_t T, int64_t M, const float* gi, const float* h0,
                                        const float* c0, const uint8_t* fresh, float* hs, float* cs, float* saved) {
  if (!g || !gi || !h0 || !c0 || !hs) return fail(KS_EINVAL, "ks_lstm_sequence_forward: null argument");
  if (T < 0 || M < 0) return fail(KS_EINVAL, "ks_lstm_sequence_forward: negative size");
  if (T == 0 || M == 0) return KS_OK;
  const float *W, *Wt;
  int ldw, ldwt;
  if (!lstm_seq_weights(g, &W, &ldw, &Wt, &ldwt)) return fail(KS_EINVAL, "ks_lstm_sequence_forward: needs an fp32 cell of hidden size %d", kSeqH);
  if (T > 1 && (hs == h0 || (cs && cs == c0))) return fail(KS_EINVAL, "ks_lstm_sequence_forward: outputs may alias the initial state only for T = 1");
  // sets of 4 rows per workgroup: one while there is at most one set per CU (long sequences want every CU), more when a short
  // call covers so many rows that re-reading the weights per set would dominate it
  const int64_t sets = (M + kSeqRows - 1) / kSeqRows;
  int groups = 1;
  if (T * 8 <= 64) while (groups < 8 && sets > (int64_t)256 * groups) groups *= 2;
  const int64_t grid = (sets + groups - 1) / groups;
  if (grid > 0x7fffffff || T > 0x7fffffff) return fail(KS_ELIMIT, "ks_lstm_sequence_forward: too many rows or steps");
  hipLaunchKernelGGL(lstm_seq_forward_kernel, dim3((unsigned)grid), dim3(64 * kSeqWaves), 0, (hipStream_t)stream, (int)T, M, groups, gi, W,
                     ldw, h0, c0, fresh, hs, cs, saved);
  return check_launch("ks_lstm_sequence_forward");
}

extern "C" int ks_lstm_sequence_backward(const KsLstm* g, ks_stream_t stream, int64_t T, int64_t M, const float* dH, const float* saved,
                                         const uint8_t* fresh, float* d_g, float* dh0, float* dc0) {
  if (!g || !dH || !saved || !d_g) return fail(KS_EINVAL, "ks_lstm_sequence_backward: null argument");
  if (T < 0 || M < 0) return fail(KS_EINVAL, "ks_lstm_sequence_backward: negative size");
  if (T == 0 || M == 0) return KS_OK;
  const float *W, *Wt;
  int ldw, ldwt;
  if (!lstm_seq_weights(g, &W, &ldw, &Wt, &ldwt)) return fail(KS_EINVAL, "ks_lstm_sequence_backward: needs an fp32 cell of hidden size %d", kSeqH);
  if (!Wt) return fail(KS_EINVAL, "ks_lstm_sequence_backward: ks_lstm_train_init has not run");
  const int64_t grid = (M + kSeqRows - 1) / kSeqRows;
  if (grid > 0x7fffffff || T > 0x7fffffff) return fail(KS_ELIMIT, "ks_lstm_sequence_backward: too many rows or steps");
  hipLaunchKernelGGL(lstm_seq_backward_kernel, dim3((unsigned)grid), dim3(64 * kSeqWaves), 0, (hipStream_t)stream, (int)T, M, dH, saved,
                     fresh, Wt, ldwt, d_g, dh0, dc0);
  return check_launch("ks_lstm_sequence_backward");
}

extern "C" int ks_lstm_train_init(KsLstm* g) {
  if (!g) return fail(KS_EINVAL, "ks_lstm_train_init: null handle");
  int rc = ks_mlp_train_init(g->proj_i);
  if (rc == KS_OK) rc = ks_mlp_train_init(g->proj_h);
  // the cell has one bias, carried by the input projection: the hidden projection's stays zero
  if (rc == KS_OK) rc = ks_mlp_freeze_bias_prefix(g->proj_h, 0, 4 * g->H);
  return rc;
}

extern "C" int ks_lstm_projections(KsLstm* g, KsMlp** input_projection, KsMlp** hidden_projection) {
  if (!g || !input_projection || !hidden_projection) return fail(KS_EINVAL, "ks_lstm_projections: null argument");
  *input_projection = g->proj_i;
  *hidden_projection = g->proj_h;
  return KS_OK;
}

extern "C" int ks_lstm_train_forward(const KsLstm* g, ks_stream_t stream, int64_t M, const float* x, const float* h_in,
                                     const float* c_in, const uint8_t* fresh, float* h_out, float* c_out, float* saved,
                                     void* workspace) {
  if (!g || !x || !h_in || !c_in || !h_out || !c_out || !saved) return fail(KS_EINVAL, "ks_lstm_train_forward: null argument");
  if (M < 0) return fail(KS_EINVAL, "ks_lstm_train_forward: negative row count");
  if (M == 0) return KS_OK;
  if (!workspace) return fail(KS_EINVAL, "ks_lstm_train_forward: workspace is required");
  const int64_t gates = up256(M * 4 * g->H * 4);
  char* w = (char*)workspace;
  float* gi = (float*)w;
  float* gh = (float*)(w + gates);
  void* wi = w + 2 * gates;
  void* wh = w + 2 * gates + up256(ks_mlp_workspace_bytes(g->proj_i, M));
  int rc = ks_mlp_forward(g->proj_i, stream, M, x, gi, wi);
  if (rc != KS_OK) return rc;
  if (ks_lstm_sequence_supported(g)) return ks_lstm_sequence_forward(g, stream, 1, M, gi, h_in, c_in, fresh, h_out, c_out, saved);
  rc = ks_mlp_forward(g->proj_h, stream, M, h_in, gh, wh);
  if (rc != KS_OK) return rc;
  const int64_t n = M * g->H, grid = (n + 255) / 256;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_lstm_train_forward: too many elements");
  hipLaunchKernelGGL(lstm_gate_train_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, M, g->H, gi, gh, h_in, c_in,
                     fresh, h_out, c_out, saved);
  return check_launch("ks_lstm_train_forward");
}

extern "C" int64_t ks_lstm_backward_workspace_bytes(const KsLstm* g, int64_t M) {
  if (!g || M < 0) return -1;
  return ks_mlp_train_workspace_bytes(g->proj_h, M);
}

extern "C" int ks_lstm_backward_step(KsLstm* g, ks_stream_t stream, int64_t M, const float* dh_out, const float* dc_out,
                                     const float* saved, const uint8_t* fresh, float* d_g, float* dh_in, float* dc_in,
                                     void* workspace) {
  if (!g || !dh_out || !dc_out || !saved || !d_g || !dh_in || !dc_in || !workspace) return fail(KS_EINVAL, "ks_lstm_backward_step: null argument");
  if (M < 0) return fail(KS_EINVAL, "ks_lstm_backward_step: negative row count");
  if (M == 0) return KS_OK;
  const int64_t n = M * g->H, grid = (n + 255) / 256;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_lstm_backward_step: too many elements");
  hipLaunchKernelGGL(lstm_gate_backward_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, M, g->H, dh_out, dc_out,
                     saved, fresh, d_g, dh_in, dc_in);
  const int rc = check_launch("ks_lstm_backward_step");
  if (rc != KS_OK) return rc;
  // dh_in = d_g W_hh, except across an episode boundary
  return ks_mlp_train_backward_dx(g->proj_h, stream, M, nullptr, d_g, dh_in, 0, 1, fresh, workspace);
}

extern "C" int ks_lstm_grad_sqnorm(const KsLstm* g, ks_stream_t stream, double* acc) {
  if (!g || !acc) return fail(KS_EINVAL, "ks_lstm_grad_sqnorm: null argument");
  const int rc = ks_mlp_grad_sqnorm(g->proj_i, stream, acc);
  return rc != KS_OK ? rc : ks_mlp_grad_sqnorm(g->proj_h, stream, acc);
}

extern "C" int ks_lstm_adam_step(KsLstm* g, ks_stream_t stream, const KsAdamParams* params, const double* sqnorm) {
  if (!g) return fail(KS_EINVAL, "ks_lstm_adam_step: null handle");
  const int rc = ks_mlp_adam_step(g->proj_i, stream, params, sqnorm);
  return rc != KS_OK ? rc : ks_mlp_adam_step(g->proj_h, stream, params, sqnorm);
}
