// GRU and LSTM cells for recurrent policies in the rollout (forward only).  The two gate projections are plain linear
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

}  // namespace ks

using namespace ks;

struct KsGru {
  int I, H;
  KsMlp *proj_i, *proj_h;
  float* bias_n;  // device (H)
};

extern "C" int ks_gru_create(const KsGruDesc* d, KsGru** out) {
  if (!d || !out) return fail(KS_EINVAL, "ks_gru_create: null argument");
  if (d->input_size < 1 || d->hidden_size < 1 || d->hidden_size > 21845) return fail(KS_EINVAL, "ks_gru_create: bad sizes %d -> %d", d->input_size, d->hidden_size);
  if (!d->weight_ih || !d->weight_hh) return fail(KS_EINVAL, "ks_gru_create: weights are required");
  const int H = d->hidden_size, I = d->input_size;
  std::vector<float> zero(3 * (size_t)H, 0.f), bh(3 * (size_t)H, 0.f);
  if (d->bias_n) for (int j = 0; j < H; ++j) bh[2 * (size_t)H + j] = d->bias_n[j];
  KsGru* g = new KsGru{I, H, nullptr, nullptr, nullptr};
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
