// MLP forward on the gfx950 matrix cores: one fused GEMM + bias + activation kernel per layer.
//
// Tile: a 256-thread workgroup (4 wavefronts, 2 x 2) owns a 128 x 128 block of the layer output;
// each wavefront accumulates a 64 x 64 sub-block as 2 x 2 MFMA 32x32 tiles in 64 fp32 registers.
// The K loop stages 128 x BK slices of the activations and of the weights through LDS.
//   bf16 path: v_mfma_f32_32x32x16_bf16 (A/B fragments: 8 consecutive k per lane), BK = 32
//   fp32 path: v_mfma_f32_32x32x2_f32   (A/B fragments: 1 k per lane),             BK = 16
// Output fragment layout (both): lane l, register r -> row 8*(r/4) + 4*(l/32) + r%4, column l%32.
#include "ks_common.h"

#include <cmath>
#include <cstring>
#include <vector>

namespace ks {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int kBM = 128, kBN = 128;

template <int ACT>
__device__ __forceinline__ float activate(float x) {
  if (ACT == KS_ACT_ELU) return x > 0.f ? x : expm1f(x);
  if (ACT == KS_ACT_RELU) return fmaxf(x, 0.f);
  if (ACT == KS_ACT_TANH) return tanhf(x);
  return x;
}

__device__ __forceinline__ __bf16 to_bf16(float x) { return (__bf16)x; }

// T = math/storage type of activations and weights (__bf16 or float).
// FIRST: x is the caller's unpadded fp32 input (row stride ldx = in_dim).
// LAST: y is the caller's unpadded fp32 output (row stride ldy = out_dim).
template <typename T, bool FIRST, bool LAST, int ACT>
__global__ __launch_bounds__(256) void mlp_layer_kernel(int64_t M, int K /*padded*/, int Kreal, int Nreal,
                                                        const void* __restrict__ xin, int64_t ldx,
                                                        const T* __restrict__ W /*(Np, K)*/,
                                                        const float* __restrict__ bias /*(Np)*/,
                                                        void* __restrict__ yout, int64_t ldy) {
  constexpr bool BF = sizeof(T) == 2;
  constexpr int BK = BF ? 32 : 16;
  constexpr int PAD = BF ? 8 : 4;  // keeps 16-byte alignment of rows and spreads LDS banks
  __shared__ __attribute__((aligned(16))) T As[kBM][BK + PAD];
  __shared__ __attribute__((aligned(16))) T Bs[kBN][BK + PAD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int64_t m0 = (int64_t)blockIdx.x * kBM;
  const int n0 = blockIdx.y * kBN;
  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int lrow = tid >> 1;               // 0..127
  const int lcol = (tid & 1) * (BK / 2);   // each thread stages BK/2 elements of one row
  for (int k0 = 0; k0 < K; k0 += BK) {
    // ---- stage A (activations)
    {
      const int64_t m = m0 + lrow;
      T* dst = &As[lrow][lcol];
      if (FIRST) {
        const float* x = (const float*)xin;
#pragma unroll
        for (int c = 0; c < BK / 2; ++c) {
          const int k = k0 + lcol + c;
          const float v = (m < M && k < Kreal) ? x[m * ldx + k] : 0.f;
          dst[c] = BF ? (T)to_bf16(v) : (T)v;
        }
      } else {
        const T* x = (const T*)xin;
        if (m < M) {
          const uint4* src = (const uint4*)(x + m * ldx + k0 + lcol);
#pragma unroll
          for (int c = 0; c < (BK / 2) * (int)sizeof(T) / 16; ++c) ((uint4*)dst)[c] = src[c];
        } else {
#pragma unroll
          for (int c = 0; c < (BK / 2) * (int)sizeof(T) / 16; ++c) ((uint4*)dst)[c] = make_uint4(0, 0, 0, 0);
        }
      }
    }
    // ---- stage B (weights, padded so no guards are needed)
    {
      const uint4* src = (const uint4*)(W + (int64_t)(n0 + lrow) * K + k0 + lcol);
      uint4* dst = (uint4*)&Bs[lrow][lcol];
#pragma unroll
      for (int c = 0; c < (BK / 2) * (int)sizeof(T) / 16; ++c) dst[c] = src[c];
    }
    __syncthreads();
    if constexpr (BF) {
#pragma unroll
      for (int kk = 0; kk < BK; kk += 16) {
        bf16x8 af[2], bfr[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) af[i] = *(const bf16x8*)&As[wm * 64 + i * 32 + (lane & 31)][kk + (lane >> 5) * 8];
#pragma unroll
        for (int j = 0; j < 2; ++j) bfr[j] = *(const bf16x8*)&Bs[wn * 64 + j * 32 + (lane & 31)][kk + (lane >> 5) * 8];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int kk = 0; kk < BK; kk += 2) {
        float af[2], bfr[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) af[i] = (float)As[wm * 64 + i * 32 + (lane & 31)][kk + (lane >> 5)];
#pragma unroll
        for (int j = 0; j < 2; ++j) bfr[j] = (float)Bs[wn * 64 + j * 32 + (lane & 31)][kk + (lane >> 5)];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bfr[j], acc[i][j], 0, 0, 0);
      }
    }
    __syncthreads();
  }
  // ---- epilogue: bias + activation + store
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = n0 + wn * 64 + j * 32 + (lane & 31);
      const float b = bias[col];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t row = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (row >= M) continue;
        const float v = acc[i][j][r] + b;
        if (LAST) {
          if (col < Nreal) ((float*)yout)[row * ldy + col] = v;
        } else {
          const float h = activate<ACT>(v);
          ((T*)yout)[row * ldy + col] = BF ? (T)to_bf16(h) : (T)h;
        }
      }
    }
}

struct DevMlp {
  int n_layers, activation, dtype;
  int dims[KS_MAX_LAYERS + 1];
  int kpad[KS_MAX_LAYERS];  // padded input width of layer l
  int npad[KS_MAX_LAYERS];  // padded output width of layer l
  void* W[KS_MAX_LAYERS];
  float* b[KS_MAX_LAYERS];
};

static inline int round_up(int x, int m) { return (x + m - 1) / m * m; }

static uint16_t f32_to_bf16_rne(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);  // NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

template <typename T, bool FIRST, bool LAST>
static void launch_layer(int act, dim3 grid, hipStream_t s, int64_t M, int K, int Kreal, int Nreal, const void* x,
                         int64_t ldx, const void* W, const float* b, void* y, int64_t ldy) {
#define KS_LAUNCH(A)                                                                                             \
  hipLaunchKernelGGL((mlp_layer_kernel<T, FIRST, LAST, A>), grid, dim3(256), 0, s, M, K, Kreal, Nreal, x, ldx, \
                     (const T*)W, b, y, ldy)
  if (LAST) { KS_LAUNCH(KS_ACT_NONE); return; }
  switch (act) {
    case KS_ACT_ELU: KS_LAUNCH(KS_ACT_ELU); break;
    case KS_ACT_RELU: KS_LAUNCH(KS_ACT_RELU); break;
    case KS_ACT_TANH: KS_LAUNCH(KS_ACT_TANH); break;
    default: KS_LAUNCH(KS_ACT_NONE); break;
  }
#undef KS_LAUNCH
}

}  // namespace ks

using namespace ks;

struct KsMlp {
  DevMlp m;
};

extern "C" int ks_mlp_create(const KsMlpDesc* d, KsMlp** out) {
  if (!d || !out) return fail(KS_EINVAL, "ks_mlp_create: null argument");
  if (d->n_layers < 1 || d->n_layers > KS_MAX_LAYERS) return fail(KS_ELIMIT, "ks_mlp_create: %d layers (1..%d)", d->n_layers, KS_MAX_LAYERS);
  if (d->dtype != KS_MLP_F32 && d->dtype != KS_MLP_BF16) return fail(KS_EINVAL, "ks_mlp_create: unknown dtype");
  if (d->activation < KS_ACT_NONE || d->activation > KS_ACT_TANH) return fail(KS_EINVAL, "ks_mlp_create: unknown activation");
  for (int l = 0; l <= d->n_layers; ++l)
    if (d->dims[l] < 1 || d->dims[l] > 65536) return fail(KS_EINVAL, "ks_mlp_create: bad width %d", d->dims[l]);
  KsMlp* h = new KsMlp();
  DevMlp& m = h->m;
  std::memset(&m, 0, sizeof(m));
  m.n_layers = d->n_layers; m.activation = d->activation; m.dtype = d->dtype;
  const int bk = d->dtype == KS_MLP_BF16 ? 32 : 16;
  const size_t esz = d->dtype == KS_MLP_BF16 ? 2 : 4;
  for (int l = 0; l <= d->n_layers; ++l) m.dims[l] = d->dims[l];
  for (int l = 0; l < d->n_layers; ++l) {
    if (!d->weights[l] || !d->biases[l]) { ks_mlp_destroy(h); return fail(KS_EINVAL, "ks_mlp_create: layer %d has no weights", l); }
    m.npad[l] = round_up(d->dims[l + 1], kBN);
    // hidden activations are stored with the producer's padded width, so the consumer's K equals it
    m.kpad[l] = l == 0 ? round_up(d->dims[0], bk) : m.npad[l - 1];
    const size_t n = (size_t)m.npad[l] * m.kpad[l];
    std::vector<unsigned char> w(n * esz, 0);
    for (int o = 0; o < d->dims[l + 1]; ++o)
      for (int i = 0; i < d->dims[l]; ++i) {
        const float v = d->weights[l][(size_t)o * d->dims[l] + i];
        if (esz == 2) ((uint16_t*)w.data())[(size_t)o * m.kpad[l] + i] = f32_to_bf16_rne(v);
        else ((float*)w.data())[(size_t)o * m.kpad[l] + i] = v;
      }
    std::vector<float> b(m.npad[l], 0.f);
    for (int o = 0; o < d->dims[l + 1]; ++o) b[o] = d->biases[l][o];
    if (hipMalloc(&m.W[l], n * esz) != hipSuccess || hipMalloc((void**)&m.b[l], b.size() * 4) != hipSuccess ||
        hipMemcpy(m.W[l], w.data(), n * esz, hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(m.b[l], b.data(), b.size() * 4, hipMemcpyHostToDevice) != hipSuccess) {
      ks_mlp_destroy(h);
      return fail(KS_ELAUNCH, "ks_mlp_create: upload of layer %d failed", l);
    }
  }
  *out = h;
  return KS_OK;
}

extern "C" int ks_mlp_destroy(KsMlp* h) {
  if (!h) return KS_OK;
  for (int l = 0; l < KS_MAX_LAYERS; ++l) {
    if (h->m.W[l]) (void)hipFree(h->m.W[l]);
    if (h->m.b[l]) (void)hipFree(h->m.b[l]);
  }
  delete h;
  return KS_OK;
}

extern "C" int64_t ks_mlp_workspace_bytes(const KsMlp* h, int64_t M) {
  if (!h || M < 0) return 0;
  int widest = 0;
  for (int l = 0; l + 1 < h->m.n_layers; ++l) widest = h->m.npad[l] > widest ? h->m.npad[l] : widest;
  const int64_t esz = h->m.dtype == KS_MLP_BF16 ? 2 : 4;
  return 2 * M * widest * esz + 256;
}

extern "C" int ks_mlp_forward(const KsMlp* h, ks_stream_t stream, int64_t M, const float* x, float* y, void* workspace) {
  if (!h) return fail(KS_EINVAL, "ks_mlp_forward: null handle");
  if (M < 0) return fail(KS_EINVAL, "ks_mlp_forward: negative row count");
  if (M == 0) return KS_OK;
  if (!x || !y) return fail(KS_EINVAL, "ks_mlp_forward: null pointer");
  const DevMlp& m = h->m;
  if (m.n_layers > 1 && !workspace) return fail(KS_EINVAL, "ks_mlp_forward: workspace required");
  if ((M + kBM - 1) / kBM > 0x7fffffff) return fail(KS_ELIMIT, "ks_mlp_forward: too many rows");
  const int64_t esz = m.dtype == KS_MLP_BF16 ? 2 : 4;
  int widest = 0;
  for (int l = 0; l + 1 < m.n_layers; ++l) widest = m.npad[l] > widest ? m.npad[l] : widest;
  char* buf[2] = {(char*)workspace, (char*)workspace + ((M * widest * esz + 255) / 256) * 256};
  const void* in = x;
  int64_t ldin = m.dims[0];
  hipStream_t s = (hipStream_t)stream;
  for (int l = 0; l < m.n_layers; ++l) {
    const bool first = l == 0, last = l == m.n_layers - 1;
    void* outp = last ? (void*)y : (void*)buf[l & 1];
    const int64_t ldo = last ? m.dims[l + 1] : m.npad[l];
    const dim3 grid((unsigned)((M + kBM - 1) / kBM), (unsigned)(m.npad[l] / kBN));
#define KS_GO(T)                                                                                                 \
  if (first && last) launch_layer<T, true, true>(m.activation, grid, s, M, m.kpad[l], m.dims[l], m.dims[l + 1], in, ldin, m.W[l], m.b[l], outp, ldo); \
  else if (first) launch_layer<T, true, false>(m.activation, grid, s, M, m.kpad[l], m.dims[l], m.dims[l + 1], in, ldin, m.W[l], m.b[l], outp, ldo);   \
  else if (last) launch_layer<T, false, true>(m.activation, grid, s, M, m.kpad[l], m.dims[l], m.dims[l + 1], in, ldin, m.W[l], m.b[l], outp, ldo);    \
  else launch_layer<T, false, false>(m.activation, grid, s, M, m.kpad[l], m.dims[l], m.dims[l + 1], in, ldin, m.W[l], m.b[l], outp, ldo);
    if (m.dtype == KS_MLP_BF16) { KS_GO(__bf16) } else { KS_GO(float) }
#undef KS_GO
    in = outp;
    ldin = ldo;
  }
  return check_launch("ks_mlp_forward");
}
