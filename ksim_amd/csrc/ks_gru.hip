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
  rc = ks_mlp_forward(g->proj_h, stream, M, h_in, gh, wh);
  if (rc != KS_OK) return rc;
  const int64_t n = M * g->H, grid = (n + 255) / 256;
  if (grid > 0x7fffffff) return fail(KS_ELIMIT, "ks_lstm_forward: too many elements");
  hipLaunchKernelGGL(lstm_gate_kernel, dim3((unsigned)grid), dim3(256), 0, (hipStream_t)stream, M, g->H, gi, gh, c_in, fresh,
                     h_out, c_out);
  return check_launch("ks_lstm_forward");
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
