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
#include <cstdlib>
#include <vector>

namespace ks {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;  // a 16-byte register vector (plain vector type, so arrays of it stay in registers)

constexpr int kBM = 128, kBN = 128;  // kBM: the largest row tile

// FAST: the result is rounded to bf16 right away, so the hardware exponential (abs. error ~1e-7 near zero) is
// exact enough; the fp32 path keeps expm1f.
template <int ACT, bool FAST>
__device__ __forceinline__ float activate(float x) {
  if (ACT == KS_ACT_ELU) {
    // exp(x) - 1 >= x everywhere, so ELU is the median of (x, 0, exp(x) - 1): one instruction instead of compare + select
    if (FAST) return __builtin_amdgcn_fmed3f(x, 0.f, __expf(x) - 1.0f);
    return x > 0.f ? x : expm1f(x);
  }
  if (ACT == KS_ACT_RELU) return fmaxf(x, 0.f);
  if (ACT == KS_ACT_TANH) return tanhf(x);
  if (ACT == KS_ACT_GELU) {  // tanh form (jax.nn.gelu's default): 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))
    const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
    // tanh(u) = 1 - 2 / (exp(2u) + 1); the hardware exponential is exact enough when the result is rounded to bf16
    const float t = FAST ? 1.f - 2.f / (__expf(2.f * u) + 1.f) : tanhf(u);
    return 0.5f * x * (1.f + t);
  }
  return x;
}

__device__ __forceinline__ __bf16 to_bf16(float x) { return (__bf16)x; }


// First layer: VEC consecutive fp32 inputs of row m starting at column k (zero beyond the real width or batch),
// converted to T and packed into one 16-byte register vector.
template <typename T, int VEC>
__device__ __forceinline__ u32x4 load_first(const float* __restrict__ x, int64_t m, int64_t M, int64_t ldx, int k,
                                            int Kreal) {
  float f[VEC];
  if (m < M && (ldx & 3) == 0 && k + VEC <= Kreal) {  // whole vector inside a 16-byte aligned row: wide loads
    const float4* p4 = reinterpret_cast<const float4*>(x + m * ldx + k);
#pragma unroll
    for (int e = 0; e < VEC / 4; ++e) {
      const float4 t = p4[e];
      f[4 * e] = t.x; f[4 * e + 1] = t.y; f[4 * e + 2] = t.z; f[4 * e + 3] = t.w;
    }
  } else {
#pragma unroll
    for (int e = 0; e < VEC; ++e) f[e] = (m < M && k + e < Kreal) ? x[m * ldx + k + e] : 0.f;
  }
  u32x4 out;
  if constexpr (sizeof(T) == 2) {
    unsigned w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const unsigned lo = __builtin_bit_cast(unsigned short, (__bf16)f[2 * e]);
      const unsigned hi = __builtin_bit_cast(unsigned short, (__bf16)f[2 * e + 1]);
      w[e] = lo | (hi << 16);
    }
    out = u32x4{w[0], w[1], w[2], w[3]};
  } else {
    out = u32x4{__builtin_bit_cast(unsigned, f[0]), __builtin_bit_cast(unsigned, f[1]),
                __builtin_bit_cast(unsigned, f[2]), __builtin_bit_cast(unsigned, f[3])};
  }
  return out;
}

// T = math/storage type of activations and weights (__bf16 or float).
// FIRST: x is the caller's unpadded fp32 input (row stride ldx = in_dim).
// LAST: y is the caller's unpadded fp32 output (row stride ldy = out_dim).
// BM: rows per workgroup (128, or 64 for small batches so that the grid still covers every CU twice).
// The K loop is software-pipelined: the global loads of slice k+1 are issued into registers before the MFMAs
// of slice k run out of LDS, so HBM/L2 latency overlaps the matrix-core work.
template <typename T, bool FIRST, bool LAST, int ACT, int BM, int BN, int WAVES_M, int WAVES_N, int KMUL = 1>
__global__ __launch_bounds__(64 * WAVES_M * WAVES_N) void mlp_layer_kernel(int64_t M, int K /*padded to BK*/, int Kreal, int Nreal,
                                                        const void* __restrict__ xin, int64_t ldx,
                                                        const T* __restrict__ W /*(Np, K)*/,
                                                        const float* __restrict__ bias /*(Np)*/,
                                                        void* __restrict__ yout, int64_t ldy) {
  constexpr bool BF = sizeof(T) == 2;
  constexpr int BK = (BF ? 64 : 32) * KMUL;  // elements of K per slice (KMUL 2: half the barriers per flop, twice the LDS)
  constexpr int PAD = BF ? 8 : 4;        // keeps 16-byte row alignment and spreads LDS banks
  constexpr int VEC = 16 / sizeof(T);    // elements per 16-byte load
  constexpr int NT = 64 * WAVES_M * WAVES_N;    // threads per workgroup
  constexpr int A_VECS = BM * BK / VEC / NT;    // 16-byte loads per thread for the A slice
  constexpr int B_VECS = BN * BK / VEC / NT;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // output block of one wavefront
  constexpr int MI = WM / 32, NI = WN / 32;     // 32 x 32 MFMA tiles per wavefront
  static_assert(A_VECS >= 1 && B_VECS >= 1 && MI >= 1 && NI >= 1, "tile too small for the workgroup");
  extern __shared__ __attribute__((aligned(16))) unsigned char mlp_lds[];
  T (*As)[BK + PAD] = reinterpret_cast<T (*)[BK + PAD]>(mlp_lds);
  T (*Bs)[BK + PAD] = reinterpret_cast<T (*)[BK + PAD]>(mlp_lds + sizeof(T) * BM * (BK + PAD));
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int64_t m0 = (int64_t)blockIdx.x * BM;
  const int n0 = blockIdx.y * BN;
  f32x16 acc[MI][NI];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  constexpr int VPR = BK / VEC;  // 16-byte vectors per tile row
  u32x4 ra[A_VECS], rb[B_VECS];
  // global -> registers for the K slice starting at KS_K0 (kept as a macro so the register arrays never have
  // their address taken)
#define KS_FETCH(KS_K0)                                                                                        \
  {                                                                                                            \
    _Pragma("unroll") for (int c = 0; c < A_VECS; ++c) {                                                       \
      const int v = tid + NT * c, row = v / VPR, col = (v % VPR) * VEC;                                        \
      const int64_t m = m0 + row;                                                                              \
      if constexpr (FIRST) {                                                                                   \
        ra[c] = load_first<T, VEC>((const float*)xin, m, M, ldx, (KS_K0) + col, Kreal);                        \
      } else {                                                                                                 \
        ra[c] = (m < M) ? *reinterpret_cast<const u32x4*>((const T*)xin + m * ldx + (KS_K0) + col)             \
                        : u32x4{0u, 0u, 0u, 0u};                                                              \
      }                                                                                                        \
    }                                                                                                          \
    _Pragma("unroll") for (int c = 0; c < B_VECS; ++c) {                                                       \
      const int v = tid + NT * c, row = v / VPR, col = (v % VPR) * VEC;                                        \
      rb[c] = *reinterpret_cast<const u32x4*>(W + (int64_t)(n0 + row) * K + (KS_K0) + col);                    \
    }                                                                                                          \
  }

  // gridDim.z > 1: this workgroup reduces only its slice of K and writes partial sums to its own copy of the
  // output (LAST outputs only; the caller adds the copies up in a fixed order)
  const int kslice = K / (int)gridDim.z;
  const int kbeg = (int)blockIdx.z * kslice, kend = kbeg + kslice;
  KS_FETCH(kbeg)
  for (int k0 = kbeg; k0 < kend; k0 += BK) {
#pragma unroll
    for (int c = 0; c < A_VECS; ++c) {
      const int v = tid + NT * c, row = v / VPR, col = (v % VPR) * VEC;
      *reinterpret_cast<u32x4*>(&As[row][col]) = ra[c];
    }
#pragma unroll
    for (int c = 0; c < B_VECS; ++c) {
      const int v = tid + NT * c, row = v / VPR, col = (v % VPR) * VEC;
      *reinterpret_cast<u32x4*>(&Bs[row][col]) = rb[c];
    }
    __syncthreads();
    // Next slice in flight while the matrix cores work on this one.  The fetch is unconditional (the last pass
    // re-reads its own slice) so that the register arrays are plain loop-carried values.
    const int kn = k0 + BK < kend ? k0 + BK : k0;
    KS_FETCH(kn)
    if constexpr (BF) {
#pragma unroll
      for (int kk = 0; kk < BK; kk += 16) {
        bf16x8 af[MI], bfr[NI];
#pragma unroll
        for (int i = 0; i < MI; ++i) af[i] = *(const bf16x8*)&As[wm * WM + i * 32 + (lane & 31)][kk + (lane >> 5) * 8];
#pragma unroll
        for (int j = 0; j < NI; ++j) bfr[j] = *(const bf16x8*)&Bs[wn * WN + j * 32 + (lane & 31)][kk + (lane >> 5) * 8];
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
          for (int j = 0; j < NI; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int kk = 0; kk < BK; kk += 2) {
        float af[MI], bfr[NI];
#pragma unroll
        for (int i = 0; i < MI; ++i) af[i] = (float)As[wm * WM + i * 32 + (lane & 31)][kk + (lane >> 5)];
#pragma unroll
        for (int j = 0; j < NI; ++j) bfr[j] = (float)Bs[wn * WN + j * 32 + (lane & 31)][kk + (lane >> 5)];
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
          for (int j = 0; j < NI; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bfr[j], acc[i][j], 0, 0, 0);
      }
    }
    __syncthreads();
  }
#undef KS_FETCH
  // ---- epilogue: bias + activation + store
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j) {
      const int col = n0 + wn * WN + j * 32 + (lane & 31);
      const float b = blockIdx.z == 0 ? bias[col] : 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t row = m0 + wm * WM + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
        if (row >= M) continue;
        const float v = acc[i][j][r] + b;
        if (LAST) {
          if (col < Nreal) ((float*)yout)[(int64_t)blockIdx.z * M * ldy + row * ldy + col] = v;
        } else {
          const float h = activate<ACT, BF>(v);
          ((T*)yout)[row * ldy + col] = BF ? (T)to_bf16(h) : (T)h;
        }
      }
    }
}


// ---------------------------------------------------------------- matrix-core yardstick
// Nothing but 32x32x16 bf16 MFMAs on register operands: eight independent accumulator tiles per wavefront (the fused
// kernel's own count), no loads, no LDS, no epilogue.  What this loop reaches is the most any kernel built on that
// instruction can reach on this part at the clock it sustains under matrix load.  Per workgroup: stamps[2 b] = shader
// clock cycles of the loop, stamps[2 b + 1] = the same interval on the constant 100 MHz counter.
__global__ __launch_bounds__(256) void mfma_yardstick_kernel(int iters, float* __restrict__ out, long long* __restrict__ stamps) {
  f32x16 acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
  bf16x8 a, b;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    // operands that differ between lanes and are neither zero nor all equal
    const unsigned h = (threadIdx.x * 8u + e + blockIdx.x * 977u) * 2654435761u;
    a[e] = (__bf16)(((float)(h >> 8) / 8388608.0f) - 1.0f);
    b[e] = (__bf16)(((float)((h * 40503u) >> 8) / 8388608.0f) - 1.0f);
  }
  const long long c0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[i], 0, 0, 0);
  }
  const long long c1 = clock64(), w1 = wall_clock64();
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) sum += acc[i][r];
  out[(int64_t)blockIdx.x * 256 + threadIdx.x] = sum;
  if (stamps && threadIdx.x == 0) {
    stamps[2 * (int64_t)blockIdx.x] = c1 - c0;
    stamps[2 * (int64_t)blockIdx.x + 1] = w1 - w0;
  }
}

// ---------------------------------------------------------------- whole network in one kernel (bf16)
// A 512-thread workgroup keeps a BM-row tile of activations in LDS as bf16 for the whole network and walks the
// layers in place; only the network input and output touch HBM.  The product is computed transposed,
// C^T = W * A^T: the weights are the MFMA "A" operand (32 output features x 16 k), the activations the "B"
// operand (16 k x 32 batch rows), so that a lane's accumulators hold 4 consecutive features of one batch row
// and the epilogue writes them back with one 8-byte LDS store.  Wavefront w owns output tiles w and w + 8 and
// all BM rows; its weight fragments stream from global memory (L2-resident, pre-ordered so that a fragment is
// one contiguous 1 KB read) through a register ring kPF steps deep; activation fragments come from LDS.
constexpr int kFusedMaxWidth = 512;
constexpr int kFusedWaves = 8;
// ring depth: 4 steps, 2 for the 64-row tile (two workgroups per CU, 128 registers each)
constexpr int kPF = 4;

struct FusedArgs {
  int64_t M;
  int n_layers, in_dim, out_dim, lda;
  int fk[KS_MAX_LAYERS], fn[KS_MAX_LAYERS];
  const u32x4* Wp[KS_MAX_LAYERS];
  const float* bp[KS_MAX_LAYERS];
  const float* x;
  float* y;
  long long* prof;  // phase time stamps of wavefront 0, written only by -DKS_PROFILE builds
  // training forward: hidden layer l's activations also go to save[l], (M, save_ld[l]) bf16 row-major, for the backward pass
  __bf16* save[KS_MAX_LAYERS];
  int save_ld[KS_MAX_LAYERS];
  // training forward for the whole-network backward kernel: hidden layer l's activations transposed, keep_t[l]: (width, ldt).
  // The weight-gradient product takes them as they are, and the backward kernel's epilogue reads its f'(Y) from them.
  __bf16* keep_t[KS_MAX_LAYERS];
  __bf16* keep_t_in;  // the network input, transposed: (in_t_width, ldt), zero beyond the real inputs
  int in_t_width;
  int64_t ldt;
};

#ifdef KS_PROFILE
#define KS_MLP_STAMP(k) if (a.prof && tid == 0) a.prof[(int64_t)blockIdx.x * 32 + (k)] = wall_clock64();
#define KS_MLP_STAMP2(k) if (a.prof && threadIdx.x == 0) a.prof[(int64_t)blockIdx.x * 32 + (k)] = wall_clock64();
#else
#define KS_MLP_STAMP(k)
#define KS_MLP_STAMP2(k)
#endif

typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

__device__ __forceinline__ unsigned pack_bf16(float lo, float hi) {
  return __builtin_bit_cast(unsigned, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
}

// One layer's MFMA work of one wavefront: NT output tiles (weights w[t]) times MI row tiles.  `arow` points at
// this lane's activation fragment of K step 0 (row lane % 32 of the first row tile, k half lane / 32).
// Weight fragments sit in a register ring kPF steps ahead; activation fragments are read one step ahead.
template <int NT, int MI, int kPF>
__device__ __forceinline__ void fused_layer_mma(f32x16 (&acc)[2][MI], const u32x4* __restrict__ w0,
                                                const u32x4* __restrict__ w1, int nk, const __bf16* __restrict__ arow,
                                                int lda) {
  static_assert(kPF % 2 == 0, "the activation double buffer relies on an even ring depth");
  u32x4 rw[kPF][NT];
#pragma unroll
  for (int u = 0; u < kPF; ++u) {
    const int st = u < nk ? u : nk - 1;
    rw[u][0] = w0[st * 64];
    if (NT > 1) rw[u][NT - 1] = w1[st * 64];
  }
  bf16x8 bq[2][MI];
#pragma unroll
  for (int i = 0; i < MI; ++i) bq[0][i] = *(const bf16x8*)(arow + i * 32 * lda);
  int s = 0;
  for (; s + kPF <= nk; s += kPF) {
#pragma unroll
    for (int u = 0; u < kPF; ++u) {
      const int step = s + u;
      const int nstep = step + 1 < nk ? step + 1 : step;
#pragma unroll
      for (int i = 0; i < MI; ++i) bq[(u + 1) & 1][i] = *(const bf16x8*)(arow + i * 32 * lda + nstep * 16);
      bf16x8 wf[NT];
#pragma unroll
      for (int t = 0; t < NT; ++t) wf[t] = __builtin_bit_cast(bf16x8, rw[u][t]);
      const int nx = step + kPF < nk ? step + kPF : nk - 1;
      rw[u][0] = w0[nx * 64];
      if (NT > 1) rw[u][NT - 1] = w1[nx * 64];
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int i = 0; i < MI; ++i)
          acc[t][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[t], bq[u & 1][i], acc[t][i], 0, 0, 0);
    }
  }
#pragma unroll
  for (int u = 0; u < kPF - 1; ++u) {
    if (s + u < nk) {
      const int step = s + u;
      const int nstep = step + 1 < nk ? step + 1 : step;
#pragma unroll
      for (int i = 0; i < MI; ++i) bq[(u + 1) & 1][i] = *(const bf16x8*)(arow + i * 32 * lda + nstep * 16);
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int i = 0; i < MI; ++i)
          acc[t][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, rw[u][t]), bq[u & 1][i],
                                                              acc[t][i], 0, 0, 0);
    }
  }
}

// Accumulator tile layout: lane l, register r -> feature 32 j + 8 (r / 4) + 4 (l / 32) + r % 4 of batch row l % 32.
__device__ __forceinline__ void fused_bias_init(f32x16& acc, const float* __restrict__ bias, int j, int lane) {
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const float4 b = *reinterpret_cast<const float4*>(bias + j * 32 + 8 * g + 4 * (lane >> 5));
    acc[4 * g] = b.x; acc[4 * g + 1] = b.y; acc[4 * g + 2] = b.z; acc[4 * g + 3] = b.w;
  }
}

// Hidden layer: activation, round to bf16, back into the tile (4 consecutive features = one 8-byte LDS store).
// `keep_t` (nullable) points at the transposed copy's entry (feature 0, this lane's row): across the 32 lanes of a half the
// same register holds 32 consecutive rows of one feature, so a 2-byte store per lane writes two whole 64-byte runs.
template <int ACT>
__device__ __forceinline__ void fused_store_hidden(const f32x16& acc, __bf16* __restrict__ act, int lda, int j,
                                                   int row, int lane, __bf16* __restrict__ keep_t = nullptr, int64_t ldt = 0) {
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int f0 = j * 32 + 8 * g + 4 * (lane >> 5);
    const uint2 packed = {pack_bf16(activate<ACT, true>(acc[4 * g]), activate<ACT, true>(acc[4 * g + 1])),
                          pack_bf16(activate<ACT, true>(acc[4 * g + 2]), activate<ACT, true>(acc[4 * g + 3]))};
    *reinterpret_cast<uint2*>(act + row * lda + f0) = packed;
    if (keep_t) {
      unsigned short* o = reinterpret_cast<unsigned short*>(keep_t) + (int64_t)f0 * ldt;
      o[0] = (unsigned short)packed.x; o[ldt] = (unsigned short)(packed.x >> 16);
      o[2 * ldt] = (unsigned short)packed.y; o[3 * ldt] = (unsigned short)(packed.y >> 16);
    }
  }
}

// The finished 128-row tile, transposed, to dst (width, ld): thread p takes the columns 2 p and 2 p + 1 of the tile (one
// 4-byte LDS read per row), 8 rows per 16-byte store (a run of 256 bytes per column and tile), and returns the columns' sums.
__device__ __forceinline__ f32x2 tile_transposed_out(const __bf16* __restrict__ act, int lda, int p, __bf16* __restrict__ dst, int64_t ld,
                                                     int64_t m0) {
  f32x2 s = {0.f, 0.f};
  __bf16* out0 = dst + (int64_t)(2 * p) * ld + m0;
  __bf16* out1 = out0 + ld;
#pragma unroll 2
  for (int r0 = 0; r0 < 128; r0 += 8) {
    bf16x2 v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = *reinterpret_cast<const bf16x2*>(act + (r0 + k) * lda + 2 * p);
    __bf16 a[8], b[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      a[k] = v[k][0]; b[k] = v[k][1];
      s[0] += (float)a[k]; s[1] += (float)b[k];
    }
    *reinterpret_cast<uint4*>(out0 + r0) = *reinterpret_cast<const uint4*>(a);
    *reinterpret_cast<uint4*>(out1 + r0) = *reinterpret_cast<const uint4*>(b);
  }
  return s;
}

// Output layer: fp32 rows of the caller's (M, out_dim) matrix.
__device__ __forceinline__ void fused_store_output(const f32x16& acc, float* __restrict__ y, int64_t M, int out_dim,
                                                   int j, int64_t m, int lane) {
  if (m >= M) return;
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    const int f0 = j * 32 + 8 * g + 4 * (lane >> 5);
    float* dst = y + m * out_dim + f0;
    if ((out_dim & 3) == 0 && f0 + 4 <= out_dim) {
      *reinterpret_cast<float4*>(dst) = float4{acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (f0 + e < out_dim) dst[e] = acc[4 * g + e];
    }
  }
}

// One layer of the whole-network kernel for one wavefront: MFMA work, barrier, epilogue, barrier.
template <int ACT, int MI, bool LAST, bool KEEP>
__device__ __forceinline__ void fused_layer(const FusedArgs& a, int l, __bf16* __restrict__ act, int64_t m0, int lane,
                                            int wave, int64_t tile) {
  const int nk = a.fk[l], nt = a.fn[l], lda = a.lda;
  const __bf16* arow = act + (lane & 31) * lda + (lane >> 5) * 8;
  const int row = lane & 31;
  if (nt * MI <= kFusedWaves) {  // few tiles: one (feature tile, row tile) pair per wavefront
    const bool busy = wave < nt * MI;
    const int j = busy ? wave / MI : 0, i = busy ? wave % MI : 0;
    f32x16 acc[2][1];
    fused_bias_init(acc[0][0], a.bp[l], j, lane);
    acc[1][0] = acc[0][0];
    const u32x4* w0 = a.Wp[l] + (int64_t)j * nk * 64 + lane;
    if (busy) fused_layer_mma<1, 1, (MI == 2 ? 2 : kPF)>(acc, w0, w0, nk, arow + i * 32 * lda, lda);
    KS_MLP_STAMP2(2 + 3 * l)
    __syncthreads();  // every wavefront has read this layer's input; the tile can be overwritten
    KS_MLP_STAMP2(3 + 3 * l)
    if (busy) {
      if (LAST) fused_store_output(acc[0][0], a.y, a.M, a.out_dim, j, m0 + i * 32 + row, lane);
      else fused_store_hidden<ACT>(acc[0][0], act, lda, j, i * 32 + row, lane);
    }
  } else {
    const int mine = wave < nt ? (wave + kFusedWaves < nt ? 2 : 1) : 0;
    const int j0 = wave < nt ? wave : 0, j1 = wave + kFusedWaves < nt ? wave + kFusedWaves : j0;
    f32x16 acc[2][MI];
    fused_bias_init(acc[0][0], a.bp[l], j0, lane);
    fused_bias_init(acc[1][0], a.bp[l], j1, lane);
#pragma unroll
    for (int i = 1; i < MI; ++i) {
      acc[0][i] = acc[0][0];
      acc[1][i] = acc[1][0];
    }
    const u32x4* w0 = a.Wp[l] + (int64_t)j0 * nk * 64 + lane;
    const u32x4* w1 = a.Wp[l] + (int64_t)j1 * nk * 64 + lane;
    if (mine == 2) fused_layer_mma<2, MI, (MI == 2 ? 2 : kPF)>(acc, w0, w1, nk, arow, lda);
    else if (mine == 1) fused_layer_mma<1, MI, (MI == 2 ? 2 : kPF)>(acc, w0, w0, nk, arow, lda);
    KS_MLP_STAMP2(2 + 3 * l)
    __syncthreads();
    KS_MLP_STAMP2(3 + 3 * l)
#pragma unroll
    for (int t = 0; t < 2; ++t)
      if (t < mine) {
        const int j = t == 0 ? j0 : j1;
#pragma unroll
        for (int i = 0; i < MI; ++i) {
          if (LAST) fused_store_output(acc[t][i], a.y, a.M, a.out_dim, j, m0 + i * 32 + row, lane);
          else fused_store_hidden<ACT>(acc[t][i], act, lda, j, i * 32 + row, lane,
                                       (KEEP && MI == 4) ? a.keep_t[l] + m0 + i * 32 + row : nullptr, a.ldt);
        }
      }
  }
  __syncthreads();
  KS_MLP_STAMP2(4 + 3 * l)
  if (!LAST && a.save[l]) {
    // the finished tile, 16 bytes per thread and pass, rows as contiguous runs; the next layer only reads the tile until every
    // wavefront (this copy included, which sits before its matrix work in program order) has passed the next barrier
    const int w8 = nt * 4;  // 16-byte pieces per row (32 features = 4 pieces)
    __bf16* dst = a.save[l];
    const int ld = a.save_ld[l];
    for (int idx = threadIdx.x; idx < MI * 32 * w8; idx += 64 * kFusedWaves) {
      const int r = idx / w8, c8 = idx - r * w8;
      if (m0 + r < a.M) *reinterpret_cast<uint4*>(dst + (m0 + r) * ld + c8 * 8) = *reinterpret_cast<const uint4*>(act + r * lda + c8 * 8);
    }
  }
}

template <int ACT, int BM, bool KEEP = false>
__device__ __forceinline__ void mlp_fused_body(const FusedArgs& a, int64_t tile) {
  constexpr int MI = BM / 32;
  constexpr int NTHR = 64 * kFusedWaves;
  extern __shared__ __attribute__((aligned(16))) unsigned char mlp_lds[];
  __bf16* act = reinterpret_cast<__bf16*>(mlp_lds);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t m0 = tile * BM;
  const int lda = a.lda;
  KS_MLP_STAMP(0)
  {  // network input -> bf16 tile; zero beyond the batch and in the K padding of the first layer
    const int in_dim = a.in_dim;
    const int K0 = (KEEP && a.in_t_width > a.fk[0] * 16) ? a.in_t_width : a.fk[0] * 16;  // the transposed copy is padded further
    const int64_t rows_left = a.M - m0;
    const int rows = rows_left < BM ? (int)rows_left : BM;
    const float* src = a.x + m0 * in_dim;
    const int padw = K0 - in_dim;
    for (int idx = tid; idx < BM * padw; idx += NTHR) {
      const int r = idx / padw, c = idx - r * padw;
      act[r * lda + in_dim + c] = (__bf16)0.0f;
    }
    for (int idx = rows * in_dim + tid; idx < BM * in_dim; idx += NTHR) {
      const int r = idx / in_dim, c = idx - r * in_dim;
      act[r * lda + c] = (__bf16)0.0f;
    }
    if ((in_dim & 3) == 0) {  // rows are 16-byte aligned: four wide loads in flight per thread
      const float4* src4 = reinterpret_cast<const float4*>(src);
      const int total4 = rows * in_dim / 4;
      for (int base = tid; base < total4; base += NTHR * 4) {
        float4 v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int idx = base + q * NTHR;
          v[q] = idx < total4 ? src4[idx] : float4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int idx = base + q * NTHR;
          if (idx < total4) {
            const int r = idx * 4 / in_dim, c = idx * 4 - r * in_dim;
            *reinterpret_cast<uint2*>(act + r * lda + c) = uint2{pack_bf16(v[q].x, v[q].y), pack_bf16(v[q].z, v[q].w)};
          }
        }
      }
    } else {
      const int total = rows * in_dim;
      for (int base = tid; base < total; base += NTHR * 4) {
        float v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int idx = base + q * NTHR;
          v[q] = idx < total ? src[idx] : 0.f;
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int idx = base + q * NTHR;
          if (idx < total) {
            const int r = idx / in_dim, c = idx - r * in_dim;
            act[r * lda + c] = (__bf16)v[q];
          }
        }
      }
    }
  }
  __syncthreads();
  KS_MLP_STAMP(1)
  if (KEEP && BM == 128 && a.keep_t_in && tid < a.in_t_width / 2)  // the first layer overwrites the tile only after its barrier
    (void)tile_transposed_out(act, lda, tid, a.keep_t_in, a.ldt, m0);
  for (int l = 0; l + 1 < a.n_layers; ++l) {
    fused_layer<ACT, MI, false, KEEP>(a, l, act, m0, lane, wave, tile);
  }
  fused_layer<ACT, MI, true, KEEP>(a, a.n_layers - 1, act, m0, lane, wave, tile);
}

// KEEP: the training forward that also stores every hidden layer's activations and the network input transposed
// (FusedArgs::keep_t, keep_t_in; 128-row tiles only)
template <int ACT, int BM, bool KEEP = false>
__global__ __launch_bounds__(64 * kFusedWaves) __attribute__((amdgpu_waves_per_eu(BM <= 64 ? 4 : 2, BM <= 64 ? 4 : 2)))
void mlp_fused_kernel(const FusedArgs a) {
  mlp_fused_body<ACT, BM, KEEP>(a, blockIdx.x);
}

// Two networks over the same rows in one launch (actor and critic of a control step): blockIdx.y picks the network, so
// the second network's workgroups fill the CUs next to the first one's instead of waiting for their launch to drain.
template <int ACT, int BM>
__global__ __launch_bounds__(64 * kFusedWaves) __attribute__((amdgpu_waves_per_eu(BM <= 64 ? 4 : 2, BM <= 64 ? 4 : 2)))
void mlp_fused_pair_kernel(const FusedArgs a, const FusedArgs b) {
  // Workgroup L of the launch runs on XCD L % 8.  XCDs 0-3 take the first network and 4-7 the second, so that an XCD's L2
  // fetches one network's weights, not both (the weights are cold at every control step: the physics launch in between
  // sweeps the L2s).
  const int64_t L = blockIdx.x + (int64_t)blockIdx.y * gridDim.x;
  int net = blockIdx.y;
  int64_t tile = blockIdx.x;
  if (gridDim.x % 4 == 0) {
    net = (int)(L % 8) / 4;
    tile = (L / 8) * 4 + (L % 8) % 4;
  }
  if (net == 0) mlp_fused_body<ACT, BM>(a, tile);
  else mlp_fused_body<ACT, BM>(b, tile);
}

// ---------------------------------------------------------------- whole-network backward pass of the hidden layers
// dZ_{l-1} = (dZ_l W_l) * f'(Y_{l-1}) for l = L-1 .. 1 in one launch, a 128-row tile per workgroup that never leaves LDS: the
// product is the forward kernel's K loop over the fragment-ordered transposed weights, its epilogue reads f'(Y) from the
// transposed activations the training forward stored (FusedArgs::keep_t) and writes the new tile both into LDS and, transposed,
// to memory (the operand of the weight-gradient product: in the accumulator layout the 32 lanes of a half hold 32 consecutive
// rows of one feature, so 2-byte loads and stores per lane move whole 64-byte runs), and the tile's column sums follow (the
// bias gradient, one partial row per tile).
struct FusedBwdArgs {
  int64_t M;
  int n_layers, lda;
  int fk[KS_MAX_LAYERS], fn[KS_MAX_LAYERS];   // the forward kernel's K steps and output tiles per layer
  const u32x4* WtP[KS_MAX_LAYERS];            // l >= 1: W_l^T in fragment order, [input tile][step over outputs][lane] x 16 bytes
  const float* dy;                            // (M, out_dim): gradient of the network output, in the caller's layout
  int out_dim, np_last;                       // np_last: rows of dzT[L-1] (the output width padded for the weight-gradient product)
  const __bf16* yT[KS_MAX_LAYERS];            // hidden layer l's activations, transposed (width, ldt), as the training forward left them
  __bf16* dzT[KS_MAX_LAYERS];                 // out, every layer: dZ_l^T (width, ldt)
  float* bias_part[KS_MAX_LAYERS];            // out, every layer: (tiles, width) column sums of dZ_l per tile
  int64_t ldt;
};

template <int ACT>
__global__ __launch_bounds__(64 * kFusedWaves) __attribute__((amdgpu_waves_per_eu(2, 2)))
void mlp_fused_bwd_kernel(const FusedBwdArgs a) {
  constexpr int MI = 4, BM = 128, NTHR = 64 * kFusedWaves;
  extern __shared__ __attribute__((aligned(16))) unsigned char mlp_lds[];
  __bf16* act = reinterpret_cast<__bf16*>(mlp_lds);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t tile = blockIdx.x, m0 = tile * BM;
  const int lda = a.lda, L = a.n_layers;
  {  // the last layer's gradient tile from the caller's fp32 rows; zero in the padding columns and beyond the batch (such rows
     // stay zero through every layer)
    const int np = a.np_last, od = a.out_dim;
    for (int idx = tid; idx < BM * np; idx += NTHR) {
      const int r = idx / np, c = idx - r * np;
      act[r * lda + c] = (__bf16)((c < od && m0 + r < a.M) ? a.dy[(m0 + r) * od + c] : 0.f);
    }
  }
  __syncthreads();
  if (tid < a.np_last / 2) {  // its transpose and column sums; the first K loop below only reads the tile
    const f32x2 cs = tile_transposed_out(act, lda, tid, a.dzT[L - 1], a.ldt, m0);
    float* part = a.bias_part[L - 1] + tile * a.np_last + 2 * tid;
    part[0] = cs[0];
    part[1] = cs[1];
  }
  const __bf16* arow = act + (lane & 31) * lda + (lane >> 5) * 8;
  const int row = lane & 31;
  for (int l = L - 1; l >= 1; --l) {
    const int nk = a.fn[l] * 2;  // K steps over layer l's outputs
    const int nt = a.fk[l] / 2;  // 32-wide tiles over layer l - 1's outputs
    const int mine = wave < nt ? (wave + kFusedWaves < nt ? 2 : 1) : 0;
    const int j0 = wave < nt ? wave : 0, j1 = wave + kFusedWaves < nt ? wave + kFusedWaves : j0;
    f32x16 acc[2][MI];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[t][i][r] = 0.f;
    const u32x4* w0 = a.WtP[l] + (int64_t)j0 * nk * 64 + lane;
    const u32x4* w1 = a.WtP[l] + (int64_t)j1 * nk * 64 + lane;
    if (mine == 2) fused_layer_mma<2, MI, kPF>(acc, w0, w1, nk, arow, lda);
    else if (mine == 1) fused_layer_mma<1, MI, kPF>(acc, w0, w0, nk, arow, lda);
    __syncthreads();  // every wavefront has read dZ_l; the tile can take dZ_{l-1}
    // Epilogue in blocks of one (feature tile, row tile) pair = 16 accumulator registers.  A block's 16 activations Y_{l-1} come
    // from the transposed copy (per feature, 32 lanes read 32 consecutive rows); the next block's loads are issued before this
    // block is worked on, so their latency hides behind it instead of adding up 32 times per layer.
    auto y_block = [&](int blk, unsigned short (&yv)[16]) {
      const int t = blk >> 2, i = blk & 3;
      const int j = t == 0 ? j0 : j1;
      const unsigned short* y = reinterpret_cast<const unsigned short*>(a.yT[l - 1]) + m0 + i * 32 + row;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const unsigned short* yg = y + (int64_t)(j * 32 + 8 * g + 4 * (lane >> 5)) * a.ldt;
#pragma unroll
        for (int e = 0; e < 4; ++e) yv[4 * g + e] = yg[e * a.ldt];
      }
    };
    unsigned short ya[16], yb[16];
    const int nblk = mine * MI;
    if (nblk > 0) y_block(0, ya);
#pragma unroll
    for (int blk = 0; blk < 2 * MI; ++blk) {
      if (blk < nblk) {
        unsigned short (&cur)[16] = (blk & 1) ? yb : ya;
        unsigned short (&nxt)[16] = (blk & 1) ? ya : yb;
        if (blk + 1 < nblk) y_block(blk + 1, nxt);
        const int t = blk >> 2, i = blk & 3;
        const int j = t == 0 ? j0 : j1;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          float d[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float yv = __builtin_bit_cast(float, (unsigned)cur[4 * g + e] << 16);
            d[e] = 1.f;
            if (ACT == KS_ACT_ELU) d[e] = yv > 0.f ? 1.f : yv + 1.f;
            if (ACT == KS_ACT_RELU) d[e] = yv > 0.f ? 1.f : 0.f;
            if (ACT == KS_ACT_TANH) d[e] = 1.f - yv * yv;
            d[e] *= acc[t][i][4 * g + e];
          }
          const int f0 = j * 32 + 8 * g + 4 * (lane >> 5);
          const uint2 packed = {pack_bf16(d[0], d[1]), pack_bf16(d[2], d[3])};
          *reinterpret_cast<uint2*>(act + (i * 32 + row) * lda + f0) = packed;
          // transposed, straight from the registers: 32 lanes hold 32 consecutive rows of one feature
          unsigned short* o = reinterpret_cast<unsigned short*>(a.dzT[l - 1]) + (int64_t)f0 * a.ldt + m0 + i * 32 + row;
          o[0] = (unsigned short)packed.x; o[a.ldt] = (unsigned short)(packed.x >> 16);
          o[2 * a.ldt] = (unsigned short)packed.y; o[3 * a.ldt] = (unsigned short)(packed.y >> 16);
        }
      }
    }
    __syncthreads();
    if (tid < nt * 16) {  // column sums of the new tile (the bias gradient's share); the next K loop only reads the tile, as this does
      f32x2 cs = {0.f, 0.f};
#pragma unroll 8
      for (int r = 0; r < BM; ++r) {
        const bf16x2 v = *reinterpret_cast<const bf16x2*>(act + r * lda + 2 * tid);
        cs[0] += (float)v[0]; cs[1] += (float)v[1];
      }
      float* part = a.bias_part[l - 1] + tile * (nt * 32) + 2 * tid;
      part[0] = cs[0];
      part[1] = cs[1];
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
  // whole-network kernel (bf16, every padded width <= kFusedMaxWidth): weights re-ordered into MFMA fragments
  int fused;                    // 1 when the tables below are valid
  int fk[KS_MAX_LAYERS];        // K steps of 16 per layer
  int fn[KS_MAX_LAYERS];        // 32-wide output tiles per layer
  int lda;                      // LDS row stride of the activation tile, in bf16 elements
  void* Wp[KS_MAX_LAYERS];      // [tile][k step][lane] x 16 bytes
  float* bp[KS_MAX_LAYERS];     // bias padded to 32 * fn
  // training state (ks_mlp_train_init): fp32 master weights in the padded (npad, kpad) layout, their gradients
  // and Adam moments, and the transposed working copy that the input-gradient GEMM reads
  int train;
  float *mW[KS_MAX_LAYERS], *mb[KS_MAX_LAYERS];
  float *gW[KS_MAX_LAYERS], *gb[KS_MAX_LAYERS];
  float *m1W[KS_MAX_LAYERS], *m2W[KS_MAX_LAYERS], *m1b[KS_MAX_LAYERS], *m2b[KS_MAX_LAYERS];
  void* Wt[KS_MAX_LAYERS];      // (kpad, npad) working-precision transpose
  void* WtP[KS_MAX_LAYERS];     // l >= 1, whole-network kernel only: W_l^T in fragment order, for the whole-network backward pass
  int chain_saved;              // the last training forward kept the activations in the whole-network backward pass's formats
  int bias_frozen[KS_MAX_LAYERS];  // leading bias entries of the layer that the optimiser leaves alone
  float* zero_bias;             // zeros, as wide as the widest GEMM output
  double* sq_part;              // kSqBlocks partial sums of squares per gradient tensor (weights and biases of every layer)
};


// ---------------------------------------------------------------- training: the small kernels around the GEMMs
// The three matrix products of a layer's backward pass reuse mlp_layer_kernel (Y = X W^T):
//   input gradient   dY_prev = dZ W        : X = dZ (M, npad),      "W" = W^T (kpad, npad)
//   weight gradient  dW = dZ^T Y_prev      : X = dZ^T (npad, Mp),   "W" = Y_prev^T (kpad, Mp), fp32 output
// so what is left are transposes, the activation derivative, column sums and the optimiser.
template <typename T>
__device__ __forceinline__ float to_f32(T v) { return (float)v; }
template <typename T>
__device__ __forceinline__ T from_f32(float v) { return (T)v; }

// fp32 (M, n) -> T (M, ld), zero in the padding columns
template <typename T>
__global__ __launch_bounds__(256) void cast_pad_kernel(int64_t M, int n, int ld, const float* __restrict__ src, T* __restrict__ dst) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= M * ld) return;
  const int64_t m = idx / ld;
  const int c = (int)(idx - m * ld);
  dst[idx] = from_f32<T>(c < n ? src[m * n + c] : 0.f);
}

// T (M, ld) -> fp32 (M, n): the input gradient in the caller's layout; optionally added to what is there, and rows
// flagged in zero_rows come out as zero (an episode boundary stops the gradient)
template <typename T>
__global__ __launch_bounds__(256) void unpad_cast_kernel(int64_t M, int n, int ld, const T* __restrict__ src, float* __restrict__ dst,
                                                         int accumulate, const uint8_t* __restrict__ zero_rows) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= M * n) return;
  const int64_t m = idx / n;
  const int c = (int)(idx - m * n);
  if (zero_rows && zero_rows[m]) { dst[idx] = 0.f; return; }
  const float v = to_f32(src[m * ld + c]);
  dst[idx] = accumulate ? dst[idx] + v : v;
}

// (M, ld_src) with C meaningful columns -> (Cpad, Mp) transposed, zero outside (C, M).  S is float or T.
template <typename S, typename T>
__global__ __launch_bounds__(256) void transpose_kernel(int64_t M, int C, int64_t ld_src, const S* __restrict__ src, int Cpad, int64_t Mp,
                                                        T* __restrict__ dst) {
  __shared__ float tile[32][33];
  const int64_t m0 = (int64_t)blockIdx.x * 32;
  const int c0 = blockIdx.y * 32;
  const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
  for (int r = ty; r < 32; r += 8) {
    const int64_t m = m0 + r;
    const int c = c0 + tx;
    tile[r][tx] = (m < M && c < C) ? (float)src[m * ld_src + c] : 0.f;
  }
  __syncthreads();
  for (int r = ty; r < 32; r += 8) {
    const int c = c0 + r;
    const int64_t m = m0 + tx;
    if (c < Cpad && m < Mp) dst[(int64_t)c * Mp + m] = from_f32<T>(tile[tx][r]);
  }
}

// y = gelu(z), tanh form, over a whole (M, ld) buffer
template <typename T>
__global__ __launch_bounds__(256) void gelu_forward_kernel(int64_t n, const T* __restrict__ z, T* __restrict__ y) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n) return;
  const float x = to_f32(z[idx]);
  y[idx] = from_f32<T>(0.5f * x * (1.f + tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x))));
}

// dZ = dY * gelu'(Z) from the stored pre-activation, written over dY
template <typename T>
__global__ __launch_bounds__(256) void gelu_backward_kernel(int64_t n, const T* __restrict__ z, T* __restrict__ dy) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n) return;
  const float x = to_f32(z[idx]);
  const float t = tanhf(0.7978845608028654f * (x + 0.044715f * x * x * x));
  const float d = 0.5f * (1.f + t) + 0.5f * x * (1.f - t * t) * 0.7978845608028654f * (1.f + 3.f * 0.044715f * x * x);
  dy[idx] = from_f32<T>(to_f32(dy[idx]) * d);
}

// dZ = dY * act'(Z), written over dY; act' is expressed through the stored activation output Y.
template <typename T, int ACT>
__global__ __launch_bounds__(256) void act_backward_kernel(int64_t n, const T* __restrict__ y, T* __restrict__ dy) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n) return;
  const float yv = to_f32(y[idx]);
  float d = 1.f;
  if (ACT == KS_ACT_ELU) d = yv > 0.f ? 1.f : yv + 1.f;  // elu'(z) = exp(z) = elu(z) + 1 for z <= 0
  if (ACT == KS_ACT_RELU) d = yv > 0.f ? 1.f : 0.f;
  if (ACT == KS_ACT_TANH) d = 1.f - yv * yv;
  dy[idx] = from_f32<T>(to_f32(dy[idx]) * d);
}

// One pass over the gradient that a layer hands down, fusing what the backward step of the layer below needs:
//   dZ = dY * act'(Y) (in place), its transpose (for the weight-gradient product), the transpose of the stored
//   activation Y (the other operand of the weight-gradient product of the layer above) and the column sums of dZ
//   (the bias gradient, as kColsumSlices partial rows that sum_parts_kernel adds in a fixed order).
// A workgroup owns 64 columns and every kColsumSlices-th tile of 64 rows; tiles go through LDS so that both the
// row-major and the transposed accesses are 16-byte vectors.  Needs C % 64 == 0 and Mp % 64 == 0.
template <typename T, int ACT>
__global__ __launch_bounds__(256) void bwd_prep_kernel(int64_t M, int64_t Mp, int C, const T* __restrict__ y, T* __restrict__ dy,
                                                       T* __restrict__ dzT, T* __restrict__ yT, float* __restrict__ part) {
  constexpr int kPad = sizeof(T) == 2 ? 2 : 1;
  constexpr int kVec = 16 / sizeof(T);        // elements per 16-byte vector
  constexpr int kNv = 16 / kVec;              // vectors per thread and tile (16 elements)
  __shared__ T sdz[64][64 + kPad];
  __shared__ T sy[64][64 + kPad];
  const int t = threadIdx.x;
  const int c0 = blockIdx.x * 64;
  const int r = t >> 2, seg = (t & 3) * 16;
  float acc = 0.f;
  for (int64_t tile = blockIdx.y; tile < Mp / 64; tile += gridDim.y) {
    const int64_t m0 = tile * 64, m = m0 + r;
    T vy[16], vd[16];
    if (m < M) {
#pragma unroll
      for (int k = 0; k < kNv; ++k) {
        reinterpret_cast<uint4*>(vy)[k] = reinterpret_cast<const uint4*>(y + m * C + c0 + seg)[k];
        reinterpret_cast<uint4*>(vd)[k] = reinterpret_cast<const uint4*>(dy + m * C + c0 + seg)[k];
      }
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        const float yv = to_f32(vy[k]);
        float d = 1.f;
        if (ACT == KS_ACT_ELU) d = yv > 0.f ? 1.f : yv + 1.f;
        if (ACT == KS_ACT_RELU) d = yv > 0.f ? 1.f : 0.f;
        if (ACT == KS_ACT_TANH) d = 1.f - yv * yv;
        vd[k] = from_f32<T>(to_f32(vd[k]) * d);
      }
#pragma unroll
      for (int k = 0; k < kNv; ++k) reinterpret_cast<uint4*>(dy + m * C + c0 + seg)[k] = reinterpret_cast<uint4*>(vd)[k];
    } else {
#pragma unroll
      for (int k = 0; k < 16; ++k) { vy[k] = from_f32<T>(0.f); vd[k] = from_f32<T>(0.f); }
    }
    __syncthreads();  // the previous tile's readers are done
#pragma unroll
    for (int k = 0; k < 16; ++k) { sdz[r][seg + k] = vd[k]; sy[r][seg + k] = vy[k]; }
    __syncthreads();
    if (t < 64) {
      float s0 = 0.f;
      for (int rr = 0; rr < 64; ++rr) s0 += to_f32(sdz[rr][t]);
      acc += s0;
    }
    // transposed: this thread writes 16 consecutive rows of column c0 + r
    T od[16], oy[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) { od[k] = sdz[seg + k][r]; oy[k] = sy[seg + k][r]; }
#pragma unroll
    for (int k = 0; k < kNv; ++k) {
      reinterpret_cast<uint4*>(dzT + (int64_t)(c0 + r) * Mp + m0 + seg)[k] = reinterpret_cast<uint4*>(od)[k];
      reinterpret_cast<uint4*>(yT + (int64_t)(c0 + r) * Mp + m0 + seg)[k] = reinterpret_cast<uint4*>(oy)[k];
    }
  }
  if (t < 64) part[(int64_t)blockIdx.y * C + c0 + t] = acc;
}

// column sums of a (M, ld) matrix in two deterministic stages: gridDim.y row slices write partial sums, which
// sum_parts_kernel adds up in a fixed order
constexpr int kColsumSlices = 64;
template <typename T>
__global__ __launch_bounds__(256) void colsum_kernel(int64_t M, int ld, const T* __restrict__ a, float* __restrict__ part) {
  __shared__ float red[4][64];
  const int c = blockIdx.x * 64 + (threadIdx.x & 63), g = threadIdx.x >> 6;
  float s = 0.f;
  if (c < ld)
    for (int64_t m = (int64_t)blockIdx.y * 4 + g; m < M; m += 4 * (int64_t)gridDim.y) s += to_f32(a[m * ld + c]);
  red[g][threadIdx.x & 63] = s;
  __syncthreads();
  if (g == 0 && c < ld)
    part[(int64_t)blockIdx.y * ld + c] = (red[0][threadIdx.x] + red[1][threadIdx.x]) + (red[2][threadIdx.x] + red[3][threadIdx.x]);
}

// out[c] = sum over z of part[z][c] for the few columns of a bias gradient: a workgroup of 64 threads per column adds its nz
// partial sums with a fixed tree (one thread walking them one after the other pays nz dependent load latencies)
__global__ __launch_bounds__(64) void sum_parts_tree_kernel(int64_t n, int nz, const float* __restrict__ part, float* __restrict__ out) {
  __shared__ float red[64];
  const int64_t c = blockIdx.x;
  float s = 0.f;
  for (int z = threadIdx.x; z < nz; z += 64) s += part[(int64_t)z * n + c];
  red[threadIdx.x] = s;
  __syncthreads();
  for (int w = 32; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) out[c] = red[0];
}

// out[i] = sum over z of part[z][i], z ascending
__global__ __launch_bounds__(256) void sum_parts_kernel(int64_t n, int nz, const float* __restrict__ part, float* __restrict__ out) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float s = 0.f;
  for (int z0 = 0; z0 < nz; z0 += 8) {  // eight slices' loads in flight, added in slice order
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = z0 + k < nz ? part[(int64_t)(z0 + k) * n + i] : 0.f;
#pragma unroll
    for (int k = 0; k < 8; ++k)
      if (z0 + k < nz) s += v[k];
  }
  out[i] = s;
}

// Every gradient of a network from its partial sums, in one launch (the whole-network backward pass): weight gradient l =
// the sum of its nz[l] row slices, z ascending as in sum_parts_kernel; bias gradient l = the sum over the row tiles of the
// per-tile column sums, four columns per workgroup with one wavefront each and the fixed tree of sum_parts_tree_kernel.
struct GradFinishArgs {
  int n_layers, tiles;
  int nz[KS_MAX_LAYERS], nb[KS_MAX_LAYERS];
  int64_t nW[KS_MAX_LAYERS];
  int first_w[KS_MAX_LAYERS + 1], first_b[KS_MAX_LAYERS + 1];  // workgroups of the weights, then of the biases, per layer
  const float *wpart[KS_MAX_LAYERS], *bpart[KS_MAX_LAYERS];
  float *gW[KS_MAX_LAYERS], *gb[KS_MAX_LAYERS];
};
__global__ __launch_bounds__(256) void grad_finish_kernel(GradFinishArgs a) {
  const int b = blockIdx.x;
  if (b < a.first_w[a.n_layers]) {
    int l = 0;
    while (l + 1 < a.n_layers && b >= a.first_w[l + 1]) ++l;
    const int64_t i = (int64_t)(b - a.first_w[l]) * 256 + threadIdx.x, n = a.nW[l];
    if (i >= n) return;
    float s = 0.f;
    const float* part = a.wpart[l];
    const int nz = a.nz[l];
    for (int z0 = 0; z0 < nz; z0 += 8) {  // eight slices' loads in flight, added in slice order
      float v[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) v[k] = z0 + k < nz ? part[(int64_t)(z0 + k) * n + i] : 0.f;
#pragma unroll
      for (int k = 0; k < 8; ++k)
        if (z0 + k < nz) s += v[k];
    }
    a.gW[l][i] = s;
    return;
  }
  const int bb = b - a.first_w[a.n_layers];
  int l = 0;
  while (l + 1 < a.n_layers && bb >= a.first_b[l + 1]) ++l;
  const int c = (bb - a.first_b[l]) * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63, n = a.nb[l];
  if (c >= n) return;
  float s = 0.f;
  for (int z = lane; z < a.tiles; z += 64) s += a.bpart[l][(int64_t)z * n + c];
  for (int w = 32; w > 0; w >>= 1) s += __shfl_down(s, w);  // lane k adds lane k + w: the same tree for every column
  if (lane == 0) a.gb[l][c] = s;
}


// Sum of squares of gradient buffers, NaNs counted as zero (the optimiser zeroes them first), added to *acc in double.
// Every addition happens in a fixed order (a strided pass per lane, a tree over the lanes, then the partial sums one after
// the other), so the clip factor, and with it a whole update, is the same bits on every run.
constexpr int kSqBlocks = 64;
struct SqTensors {
  const float* g[2 * KS_MAX_LAYERS];
  int64_t n[2 * KS_MAX_LAYERS];
};

__device__ __forceinline__ double block_sqsum(const float* __restrict__ g, int64_t n, int first, int stride, double* red) {
  double s = 0.0;
  for (int64_t i = first; i < n; i += stride) {
    const float v = g[i];
    if (v == v) s += (double)v * (double)v;
  }
  red[threadIdx.x] = s;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
    __syncthreads();
  }
  return red[0];
}

// grid (kSqBlocks, tensors): part[tensor][block] = this block's share of the tensor
__global__ __launch_bounds__(256) void sqnorm_parts_kernel(SqTensors t, double* __restrict__ part) {
  __shared__ double red[256];
  const double v = block_sqsum(t.g[blockIdx.y], t.n[blockIdx.y], (int)(blockIdx.x * 256 + threadIdx.x), kSqBlocks * 256, red);
  if (threadIdx.x == 0) part[blockIdx.y * kSqBlocks + blockIdx.x] = v;
}

// one workgroup: *acc += the partial sums, in index order
__global__ __launch_bounds__(256) void sqnorm_finish_kernel(int n, const double* __restrict__ part, double* __restrict__ acc) {
  __shared__ double red[256];
  double s = 0.0;
  for (int i = threadIdx.x; i < n; i += 256) s += part[i];
  red[threadIdx.x] = s;
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) *acc += red[0];
}

// one workgroup over a whole buffer (small tensors that belong to no network: log standard deviations, head parameters)
__global__ __launch_bounds__(256) void sqnorm_kernel(int64_t n, const float* __restrict__ g, double* __restrict__ acc) {
  __shared__ double red[256];
  const double v = block_sqsum(g, n, (int)threadIdx.x, 256, red);
  if (threadIdx.x == 0) *acc += v;
}

// optax.chain(zero_nans, clip_by_global_norm, add_decayed_weights, scale_by_adam, scale(lr), scale(-1)) on one tensor
__global__ __launch_bounds__(256) void adam_kernel(int64_t n, float* __restrict__ p, const float* __restrict__ g,
                                                  float* __restrict__ m1, float* __restrict__ m2, KsAdamParams a,
                                                  const double* __restrict__ sqnorm) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  float gv = g[i];
  if (!(gv == gv)) gv = 0.f;                                       // zero_nans
  if (a.max_grad_norm > 0.f && sqnorm) {                           // clip_by_global_norm
    const float norm = (float)sqrt(*sqnorm);
    if (norm > a.max_grad_norm) gv = gv / norm * a.max_grad_norm;
  }
  gv += a.weight_decay * p[i];                                     // add_decayed_weights
  const float nm1 = a.b1 * m1[i] + (1.f - a.b1) * gv;              // scale_by_adam
  const float nm2 = a.b2 * m2[i] + (1.f - a.b2) * gv * gv;
  m1[i] = nm1;
  m2[i] = nm2;
  const float mhat = nm1 / (1.f - powf(a.b1, (float)a.step));
  const float vhat = nm2 / (1.f - powf(a.b2, (float)a.step));
  p[i] -= a.lr * mhat / (sqrtf(vhat) + a.eps);
}

// fp32 master (npad, kpad) -> working copies: W (npad, kpad), W^T (kpad, npad) and, for the whole-network kernel,
// the fragment-ordered copy [tile][k step][lane][8]
template <typename T>
__global__ __launch_bounds__(256) void refresh_kernel(int npad, int kpad, const float* __restrict__ mW, T* __restrict__ W,
                                                      T* __restrict__ Wt, __bf16* __restrict__ Wp, int fk, int fn,
                                                      __bf16* __restrict__ WtP) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx < (int64_t)npad * kpad) {
    const int o = (int)(idx / kpad), i = (int)(idx - (int64_t)o * kpad);
    const float v = mW[idx];
    W[idx] = from_f32<T>(v);
    if (Wt) Wt[(int64_t)i * npad + o] = from_f32<T>(v);
  }
  if (Wp && idx < (int64_t)fn * fk * 64 * 8) {
    const int e = (int)(idx & 7), lane = (int)((idx >> 3) & 63);
    const int64_t js = idx >> 9;
    const int st = (int)(js % fk), j = (int)(js / fk);
    const int o = j * 32 + (lane & 31), i = st * 16 + (lane >> 5) * 8 + e;
    Wp[idx] = (__bf16)((o < npad && i < kpad) ? mW[(int64_t)o * kpad + i] : 0.f);
  }
  if (WtP && idx < (int64_t)fn * fk * 64 * 8) {  // the transposed roles: tiles over the inputs, 2 fn steps over the outputs
    const int e = (int)(idx & 7), lane = (int)((idx >> 3) & 63);
    const int64_t js = idx >> 9;
    const int st = (int)(js % (2 * fn)), j = (int)(js / (2 * fn));
    const int i = j * 32 + (lane & 31), o = st * 16 + (lane >> 5) * 8 + e;
    WtP[idx] = (__bf16)((o < npad && i < kpad) ? mW[(int64_t)o * kpad + i] : 0.f);
  }
}

// One optimiser step of a whole network in one launch: every weight and bias element goes through the chain of adam_kernel,
// and the thread that updates a master weight also writes its working copies (W, W^T, the fragment-ordered copy of the
// whole-network kernel), as refresh_kernel does; the thread of a layer's element o < npad updates bias o as well.  The same
// arithmetic per element as the per-tensor launches, which it replaces (two dozen launches and copies per network).
struct AdamNetArgs {
  int n_layers;
  int npad[KS_MAX_LAYERS], kpad[KS_MAX_LAYERS], fk[KS_MAX_LAYERS], fn[KS_MAX_LAYERS], frozen[KS_MAX_LAYERS];
  int first_block[KS_MAX_LAYERS + 1];  // workgroups [first_block[l], first_block[l + 1]) belong to layer l
  float *mW[KS_MAX_LAYERS], *m1W[KS_MAX_LAYERS], *m2W[KS_MAX_LAYERS], *mb[KS_MAX_LAYERS], *m1b[KS_MAX_LAYERS], *m2b[KS_MAX_LAYERS];
  const float *gW[KS_MAX_LAYERS], *gb[KS_MAX_LAYERS];
  void *W[KS_MAX_LAYERS], *Wt[KS_MAX_LAYERS];
  __bf16 *Wp[KS_MAX_LAYERS], *WtP[KS_MAX_LAYERS];
  float *b[KS_MAX_LAYERS], *bp[KS_MAX_LAYERS];
};

__device__ __forceinline__ float adam_element(float p, float g, float& m1, float& m2, const KsAdamParams& a, const double* sqnorm) {
  float gv = g;
  if (!(gv == gv)) gv = 0.f;                                       // zero_nans
  if (a.max_grad_norm > 0.f && sqnorm) {                           // clip_by_global_norm
    const float norm = (float)sqrt(*sqnorm);
    if (norm > a.max_grad_norm) gv = gv / norm * a.max_grad_norm;
  }
  gv += a.weight_decay * p;                                        // add_decayed_weights
  m1 = a.b1 * m1 + (1.f - a.b1) * gv;                              // scale_by_adam
  m2 = a.b2 * m2 + (1.f - a.b2) * gv * gv;
  const float mhat = m1 / (1.f - powf(a.b1, (float)a.step));
  const float vhat = m2 / (1.f - powf(a.b2, (float)a.step));
  return p - a.lr * mhat / (sqrtf(vhat) + a.eps);
}

template <typename T>
__global__ __launch_bounds__(256) void adam_net_kernel(AdamNetArgs n, KsAdamParams a, const double* __restrict__ sqnorm) {
  int l = 0;
  while (l + 1 < n.n_layers && (int)blockIdx.x >= n.first_block[l + 1]) ++l;
  const int npad = n.npad[l], kpad = n.kpad[l];
  const int64_t idx = (int64_t)(blockIdx.x - n.first_block[l]) * 256 + threadIdx.x;
  if (idx < (int64_t)npad * kpad) {
    float m1 = n.m1W[l][idx], m2 = n.m2W[l][idx];
    const float v = adam_element(n.mW[l][idx], n.gW[l][idx], m1, m2, a, sqnorm);
    n.m1W[l][idx] = m1; n.m2W[l][idx] = m2; n.mW[l][idx] = v;
    const int o = (int)(idx / kpad), i = (int)(idx - (int64_t)o * kpad);
    reinterpret_cast<T*>(n.W[l])[idx] = from_f32<T>(v);
    if (n.Wt[l]) reinterpret_cast<T*>(n.Wt[l])[(int64_t)i * npad + o] = from_f32<T>(v);
    // [tile o / 32][k step i / 16][lane (o % 32) + 32 ((i % 16) / 8)][i % 8].  The fragment copy is padded to 32 outputs and 16
    // inputs, the master to the coarser tiles of the per-layer kernel: master entries beyond the fragment copy are padding
    // (zero weights with zero gradients) and have no place in it.
    if (n.Wp[l] && o < n.fn[l] * 32 && i < n.fk[l] * 16) {
      const int64_t at = ((((int64_t)(o >> 5) * n.fk[l] + (i >> 4)) * 64 + (o & 31) + 32 * ((i >> 3) & 1)) << 3) + (i & 7);
      n.Wp[l][at] = (__bf16)v;
      if (n.WtP[l]) {  // the same entry with the roles of input and output exchanged
        const int64_t att = ((((int64_t)(i >> 5) * (2 * n.fn[l]) + (o >> 4)) * 64 + (i & 31) + 32 * ((o >> 3) & 1)) << 3) + (o & 7);
        n.WtP[l][att] = (__bf16)v;
      }
    }
  }
  if (idx < npad) {
    float v = n.mb[l][idx];
    if (idx >= n.frozen[l]) {
      float m1 = n.m1b[l][idx], m2 = n.m2b[l][idx];
      v = adam_element(v, n.gb[l][idx], m1, m2, a, sqnorm);
      n.m1b[l][idx] = m1; n.m2b[l][idx] = m2; n.mb[l][idx] = v;
    }
    n.b[l][idx] = v;
    if (n.bp[l] && idx < n.fn[l] * 32) n.bp[l][idx] = v;
  }
}

static inline int round_up(int x, int m) { return (x + m - 1) / m * m; }

static uint16_t f32_to_bf16_rne(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);  // NaN
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

template <typename T, bool FIRST, bool LAST, int BM, int BN, int WAVES_M, int WAVES_N, int KMUL = 1>
static int launch_layer_tile(int act, hipStream_t s, int64_t M, int npad, int K, int Kreal, int Nreal, const void* x,
                             int64_t ldx, const void* W, const float* b, void* y, int64_t ldy, int ksplit = 1) {
  constexpr int BK = (sizeof(T) == 2 ? 64 : 32) * KMUL, PAD = sizeof(T) == 2 ? 8 : 4;
  constexpr int lds = (int)sizeof(T) * (BM + BN) * (BK + PAD);
  const dim3 grid((unsigned)((M + BM - 1) / BM), (unsigned)(npad / BN), (unsigned)ksplit);
  const dim3 block(64 * WAVES_M * WAVES_N);
#define KS_LAUNCH(A)                                                                                           \
  {                                                                                                            \
    auto kfn = mlp_layer_kernel<T, FIRST, LAST, A, BM, BN, WAVES_M, WAVES_N, KMUL>;                            \
    if (lds > 64 * 1024 &&                                                                                     \
        hipFuncSetAttribute((const void*)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)  \
      return fail(KS_ELAUNCH, "ks_mlp_forward: cannot raise the LDS limit to %d bytes", lds);                  \
    hipLaunchKernelGGL(kfn, grid, block, lds, s, M, K, Kreal, Nreal, x, ldx, (const T*)W, b, y, ldy);          \
  }
  if (LAST) { KS_LAUNCH(KS_ACT_NONE) return KS_OK; }
  switch (act) {
    case KS_ACT_ELU: KS_LAUNCH(KS_ACT_ELU) break;
    case KS_ACT_RELU: KS_LAUNCH(KS_ACT_RELU) break;
    case KS_ACT_TANH: KS_LAUNCH(KS_ACT_TANH) break;
    case KS_ACT_GELU: KS_LAUNCH(KS_ACT_GELU) break;
    default: KS_LAUNCH(KS_ACT_NONE) break;
  }
#undef KS_LAUNCH
  return KS_OK;
}

// Tile choice.  Large batches take the whole layer width per workgroup (BN = 512 or 256) so that the activations
// are read from HBM once per layer; small (rollout-sized) batches take 64 x 128 tiles so that the grid still
// covers the 256 CUs more than once.
template <typename T, bool FIRST, bool LAST>
static int launch_layer(int act, hipStream_t s, int64_t M, int npad, int K, int Kreal, int Nreal, const void* x,
                        int64_t ldx, const void* W, const float* b, void* y, int64_t ldy) {
#define KS_ARGS act, s, M, npad, K, Kreal, Nreal, x, ldx, W, b, y, ldy
  if (M >= 32768 && npad % 512 == 0 && sizeof(T) == 2) return launch_layer_tile<T, FIRST, LAST, 128, 512, 2, 4>(KS_ARGS);
  if (M >= 32768 && npad % 256 == 0) return launch_layer_tile<T, FIRST, LAST, 128, 256, 2, 2>(KS_ARGS);
  if (M * (npad / kBN) <= 128 * 512) return launch_layer_tile<T, FIRST, LAST, 64, 128, 2, 2>(KS_ARGS);
  return launch_layer_tile<T, FIRST, LAST, 128, 128, 2, 2>(KS_ARGS);
#undef KS_ARGS
}

}  // namespace ks

using namespace ks;

struct KsMlp {
  DevMlp m;
  std::vector<float> host_w[KS_MAX_LAYERS], host_b[KS_MAX_LAYERS];  // the caller's fp32 parameters, for ks_mlp_train_init
};

extern "C" int ks_mlp_create(const KsMlpDesc* d, KsMlp** out) {
  if (!d || !out) return fail(KS_EINVAL, "ks_mlp_create: null argument");
  if (d->n_layers < 1 || d->n_layers > KS_MAX_LAYERS) return fail(KS_ELIMIT, "ks_mlp_create: %d layers (1..%d)", d->n_layers, KS_MAX_LAYERS);
  if (d->dtype != KS_MLP_F32 && d->dtype != KS_MLP_BF16) return fail(KS_EINVAL, "ks_mlp_create: unknown dtype");
  if (d->activation < KS_ACT_NONE || d->activation > KS_ACT_GELU) return fail(KS_EINVAL, "ks_mlp_create: unknown activation");
  for (int l = 0; l <= d->n_layers; ++l)
    if (d->dims[l] < 1 || d->dims[l] > 65536) return fail(KS_EINVAL, "ks_mlp_create: bad width %d", d->dims[l]);
  KsMlp* h = new KsMlp();
  DevMlp& m = h->m;
  std::memset(&m, 0, sizeof(m));
  m.n_layers = d->n_layers; m.activation = d->activation; m.dtype = d->dtype;
  const int bk = d->dtype == KS_MLP_BF16 ? 64 : 32;
  const size_t esz = d->dtype == KS_MLP_BF16 ? 2 : 4;
  for (int l = 0; l <= d->n_layers; ++l) m.dims[l] = d->dims[l];
  for (int l = 0; l < d->n_layers; ++l) {
    if (!d->weights[l] || !d->biases[l]) { ks_mlp_destroy(h); return fail(KS_EINVAL, "ks_mlp_create: layer %d has no weights", l); }
    h->host_w[l].assign(d->weights[l], d->weights[l] + (size_t)d->dims[l + 1] * d->dims[l]);
    h->host_b[l].assign(d->biases[l], d->biases[l] + d->dims[l + 1]);
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
  // fragment-ordered copy for the whole-network kernel
  bool fusable = d->dtype == KS_MLP_BF16;
  for (int l = 0; l <= d->n_layers && fusable; ++l)
    if (round_up(d->dims[l], 32) > kFusedMaxWidth) fusable = false;
  if (fusable) {
    int kmax = 0;
    for (int l = 0; l < d->n_layers; ++l) {
      m.fn[l] = round_up(d->dims[l + 1], 32) / 32;
      m.fk[l] = (l == 0 ? round_up(d->dims[0], 16) : m.fn[l - 1] * 32) / 16;
      kmax = m.fk[l] * 16 > kmax ? m.fk[l] * 16 : kmax;
      if (l + 1 < d->n_layers && m.fn[l] * 32 > kmax) kmax = m.fn[l] * 32;
      const size_t n = (size_t)m.fn[l] * m.fk[l] * 64 * 8;
      std::vector<uint16_t> w(n, 0);
      for (int j = 0; j < m.fn[l]; ++j)
        for (int st = 0; st < m.fk[l]; ++st)
          for (int lane = 0; lane < 64; ++lane)
            for (int e = 0; e < 8; ++e) {
              const int o = j * 32 + (lane & 31), i = st * 16 + (lane >> 5) * 8 + e;
              if (o < d->dims[l + 1] && i < d->dims[l])
                w[(((size_t)j * m.fk[l] + st) * 64 + lane) * 8 + e] = f32_to_bf16_rne(d->weights[l][(size_t)o * d->dims[l] + i]);
            }
      std::vector<float> b(m.fn[l] * 32, 0.f);
      for (int o = 0; o < d->dims[l + 1]; ++o) b[o] = d->biases[l][o];
      if (hipMalloc(&m.Wp[l], n * 2) != hipSuccess || hipMalloc((void**)&m.bp[l], b.size() * 4) != hipSuccess ||
          hipMemcpy(m.Wp[l], w.data(), n * 2, hipMemcpyHostToDevice) != hipSuccess ||
          hipMemcpy(m.bp[l], b.data(), b.size() * 4, hipMemcpyHostToDevice) != hipSuccess) {
        ks_mlp_destroy(h);
        return fail(KS_ELAUNCH, "ks_mlp_create: upload of layer %d failed", l);
      }
    }
    m.lda = kmax + 8;  // +16 bytes per row: 16-byte aligned rows that start 4 banks apart
    m.fused = 1;
  }
  *out = h;
  return KS_OK;
}

namespace ks {
// For the recurrent sequence kernels, which multiply by a one-layer network's weights themselves: the live working-precision
// weight matrix of layer l, (npad, kpad) row-major, and, once ks_mlp_train_init has run, its transpose (kpad, npad).  The
// optimiser step rewrites both in place, so the pointers stay valid for the life of the handle.
int mlp_peek_layer(const KsMlp* h, int l, const void** W, const void** Wt, int* npad, int* kpad, int* dtype) {
  if (!h || l < 0 || l >= h->m.n_layers) return fail(KS_EINVAL, "mlp_peek_layer: no such layer");
  *W = h->m.W[l]; *Wt = h->m.train ? h->m.Wt[l] : nullptr;
  *npad = h->m.npad[l]; *kpad = h->m.kpad[l]; *dtype = h->m.dtype;
  return KS_OK;
}
}  // namespace ks

extern "C" int ks_mlp_destroy(KsMlp* h) {
  if (!h) return KS_OK;
  for (int l = 0; l < KS_MAX_LAYERS; ++l) {
    if (h->m.W[l]) (void)hipFree(h->m.W[l]);
    if (h->m.b[l]) (void)hipFree(h->m.b[l]);
    if (h->m.Wp[l]) (void)hipFree(h->m.Wp[l]);
    if (h->m.bp[l]) (void)hipFree(h->m.bp[l]);
    float* t[] = {h->m.mW[l], h->m.mb[l], h->m.gW[l], h->m.gb[l], h->m.m1W[l], h->m.m2W[l], h->m.m1b[l], h->m.m2b[l]};
    for (float* q : t)
      if (q) (void)hipFree(q);
    if (h->m.Wt[l]) (void)hipFree(h->m.Wt[l]);
    if (h->m.WtP[l]) (void)hipFree(h->m.WtP[l]);
  }
  if (h->m.zero_bias) (void)hipFree(h->m.zero_bias);
  if (h->m.sq_part) (void)hipFree(h->m.sq_part);
  delete h;
  return KS_OK;
}

static FusedArgs fused_args(const DevMlp& m, int64_t M, const float* x, float* y) {
  FusedArgs a;
  std::memset(&a, 0, sizeof(a));
  a.M = M; a.n_layers = m.n_layers; a.in_dim = m.dims[0]; a.out_dim = m.dims[m.n_layers]; a.lda = m.lda;
  for (int l = 0; l < m.n_layers; ++l) {
    a.fk[l] = m.fk[l]; a.fn[l] = m.fn[l];
    a.Wp[l] = (const u32x4*)m.Wp[l]; a.bp[l] = m.bp[l];
  }
  a.x = x; a.y = y;
  return a;
}

struct TrainWs;
static void keep_args(FusedArgs& a, const DevMlp& m, const TrainWs* ws);

template <int BM>
static int launch_fused_tile(const DevMlp& m, hipStream_t s, int64_t M, const float* x, float* y, char* const* save,
                             const TrainWs* keep = nullptr) {
  FusedArgs a = fused_args(m, M, x, y);
  if (save)
    for (int l = 0; l + 1 < m.n_layers; ++l) {
      a.save[l] = (__bf16*)save[l];
      a.save_ld[l] = m.npad[l];
    }
  if (keep) keep_args(a, m, keep);
#ifdef KS_PROFILE
  if (const char* e = getenv("KS_MLP_PROF_PTR")) a.prof = (long long*)strtoull(e, nullptr, 16);
#endif
  const int lds = BM * m.lda * 2;
  const int64_t blocks = (M + BM - 1) / BM;
  if (blocks > 0x7fffffff) return fail(KS_ELIMIT, "ks_mlp_forward: too many rows");
#define KS_LAUNCH(A)                                                                                           \
  {                                                                                                            \
    auto kfn = (keep && BM == 128) ? mlp_fused_kernel<A, BM, BM == 128> : mlp_fused_kernel<A, BM, false>;      \
    if (lds > 64 * 1024 &&                                                                                     \
        hipFuncSetAttribute((const void*)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)  \
      return fail(KS_ELAUNCH, "ks_mlp_forward: cannot raise the LDS limit to %d bytes", lds);                  \
    hipLaunchKernelGGL(kfn, dim3((unsigned)blocks), dim3(64 * kFusedWaves), lds, s, a);                        \
  }
  switch (m.activation) {
    case KS_ACT_ELU: KS_LAUNCH(KS_ACT_ELU) break;
    case KS_ACT_RELU: KS_LAUNCH(KS_ACT_RELU) break;
    case KS_ACT_TANH: KS_LAUNCH(KS_ACT_TANH) break;
    case KS_ACT_GELU: KS_LAUNCH(KS_ACT_GELU) break;
    default: KS_LAUNCH(KS_ACT_NONE) break;
  }
#undef KS_LAUNCH
  return check_launch("ks_mlp_forward");
}

// Row tile: 128 rows amortise each weight fragment over four MFMAs; smaller batches take smaller tiles so that
// the grid still reaches every CU.
static int launch_fused(const DevMlp& m, hipStream_t s, int64_t M, const float* x, float* y, char* const* save = nullptr) {
#ifdef KS_PROFILE
  if (const char* e = getenv("KS_MLP_BM")) {
    const int bm = atoi(e);
    if (bm == 128) return launch_fused_tile<128>(m, s, M, x, y, save);
    if (bm == 64) return launch_fused_tile<64>(m, s, M, x, y, save);
    if (bm == 32) return launch_fused_tile<32>(m, s, M, x, y, save);
  }
#endif
  if (M >= 128 * 256) return launch_fused_tile<128>(m, s, M, x, y, save);
  if (M >= 64 * 256) return launch_fused_tile<64>(m, s, M, x, y, save);
  return launch_fused_tile<32>(m, s, M, x, y, save);
}

template <int BM>
static int launch_fused_pair_tile(const DevMlp& m0, const DevMlp& m1, hipStream_t s, int64_t M, const float* x0, float* y0,
                                  const float* x1, float* y1) {
  const FusedArgs a = fused_args(m0, M, x0, y0), b = fused_args(m1, M, x1, y1);
  const int lds = BM * (m0.lda > m1.lda ? m0.lda : m1.lda) * 2;
  const int64_t blocks = (M + BM - 1) / BM;
  if (blocks > 0x7fffffff) return fail(KS_ELIMIT, "ks_mlp_forward_pair: too many rows");
#define KS_LAUNCH(A)                                                                                           \
  {                                                                                                            \
    auto kfn = mlp_fused_pair_kernel<A, BM>;                                                                   \
    if (lds > 64 * 1024 &&                                                                                     \
        hipFuncSetAttribute((const void*)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)  \
      return fail(KS_ELAUNCH, "ks_mlp_forward_pair: cannot raise the LDS limit to %d bytes", lds);             \
    hipLaunchKernelGGL(kfn, dim3((unsigned)blocks, 2), dim3(64 * kFusedWaves), lds, s, a, b);                  \
  }
  switch (m0.activation) {
    case KS_ACT_ELU: KS_LAUNCH(KS_ACT_ELU) break;
    case KS_ACT_RELU: KS_LAUNCH(KS_ACT_RELU) break;
    case KS_ACT_TANH: KS_LAUNCH(KS_ACT_TANH) break;
    case KS_ACT_GELU: KS_LAUNCH(KS_ACT_GELU) break;
    default: KS_LAUNCH(KS_ACT_NONE) break;
  }
#undef KS_LAUNCH
  return check_launch("ks_mlp_forward_pair");
}

extern "C" int ks_mlp_forward_pair(const KsMlp* h0, const KsMlp* h1, ks_stream_t stream, int64_t M, const float* x0,
                                   float* y0, const float* x1, float* y1, void* workspace0, void* workspace1) {
  if (!h0 || !h1) return fail(KS_EINVAL, "ks_mlp_forward_pair: null handle");
  if (M < 0) return fail(KS_EINVAL, "ks_mlp_forward_pair: negative row count");
  if (M == 0) return KS_OK;
  if (!x0 || !y0 || !x1 || !y1) return fail(KS_EINVAL, "ks_mlp_forward_pair: null pointer");
  if (y0 == y1) return fail(KS_EINVAL, "ks_mlp_forward_pair: the two outputs must differ");
  hipStream_t s = (hipStream_t)stream;
  // one launch when both networks run as whole-network kernels with the same activation and row tile; else one each
  if (h0->m.fused && h1->m.fused && h0->m.activation == h1->m.activation && M < 64 * 256)
    return launch_fused_pair_tile<32>(h0->m, h1->m, s, M, x0, y0, x1, y1);
  const int rc = ks_mlp_forward(h0, stream, M, x0, y0, workspace0);
  if (rc != KS_OK) return rc;
  return ks_mlp_forward(h1, stream, M, x1, y1, workspace1);
}

extern "C" int ks_mfma_yardstick(ks_stream_t stream, int32_t workgroups, int32_t iters, float* out, int64_t* stamps) {
  if (workgroups < 1 || iters < 1) return fail(KS_EINVAL, "ks_mfma_yardstick: workgroups and iterations must be positive");
  if (!out) return fail(KS_EINVAL, "ks_mfma_yardstick: null output");
  hipLaunchKernelGGL(mfma_yardstick_kernel, dim3((unsigned)workgroups), dim3(256), 0, (hipStream_t)stream, iters, out,
                     reinterpret_cast<long long*>(stamps));
  return check_launch("ks_mfma_yardstick");
}

extern "C" int64_t ks_mlp_workspace_bytes(const KsMlp* h, int64_t M) {
  if (!h || M < 0) return 0;
  if (h->m.fused) return 0;
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
  if (m.fused) return launch_fused(m, (hipStream_t)stream, M, x, y);
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
#define KS_GO(T)                                                                                                      \
  if (first && last) rc = launch_layer<T, true, true>(m.activation, s, M, m.npad[l], m.kpad[l], m.dims[l], m.dims[l + 1], in, ldin, m.W[l], m.b[l], outp, ldo); \
  else if (first) rc = launch_layer<T, true, false>(m.activation, s, M, m.npad[l], m.kpad[l], m.dims[l], m.dims[l + 1], in, ldin, m.W[l], m.b[l], outp, ldo);   \
  else if (last) rc = launch_layer<T, false, true>(m.activation, s, M, m.npad[l], m.kpad[l], m.dims[l], m.dims[l + 1], in, ldin, m.W[l], m.b[l], outp, ldo);    \
  else rc = launch_layer<T, false, false>(m.activation, s, M, m.npad[l], m.kpad[l], m.dims[l], m.dims[l + 1], in, ldin, m.W[l], m.b[l], outp, ldo);
    int rc = KS_OK;
    if (m.dtype == KS_MLP_BF16) { KS_GO(__bf16) } else { KS_GO(float) }
#undef KS_GO
    if (rc != KS_OK) return rc;
    in = outp;
    ldin = ldo;
  }
  return check_launch("ks_mlp_forward");
}

// ---------------------------------------------------------------------------------------------
// training entry points
// ---------------------------------------------------------------------------------------------
static int widest_pad(const DevMlp& m) {
  int w = 0;
  for (int l = 0; l < m.n_layers; ++l) {
    w = m.npad[l] > w ? m.npad[l] : w;
    w = round_up(m.kpad[l], kBN) > w ? round_up(m.kpad[l], kBN) : w;
  }
  return w;
}

template <typename T>
static void refresh_layers(DevMlp& m, hipStream_t s);

extern "C" int ks_mlp_train_init(KsMlp* h) {
  if (!h) return fail(KS_EINVAL, "ks_mlp_train_init: null handle");
  DevMlp& m = h->m;
  if (m.train) return KS_OK;
  // a failure part way leaves nothing behind: what was allocated so far is released and the handle stays untrained
  auto give_up = [&](const char* what) {
    for (int l = 0; l < KS_MAX_LAYERS; ++l) {
      float** t[] = {&m.mW[l], &m.mb[l], &m.gW[l], &m.gb[l], &m.m1W[l], &m.m2W[l], &m.m1b[l], &m.m2b[l]};
      for (float** q : t) {
        if (*q) (void)hipFree(*q);
        *q = nullptr;
      }
      if (m.Wt[l]) (void)hipFree(m.Wt[l]);
      m.Wt[l] = nullptr;
      if (m.WtP[l]) (void)hipFree(m.WtP[l]);
      m.WtP[l] = nullptr;
    }
    if (m.zero_bias) (void)hipFree(m.zero_bias);
    if (m.sq_part) (void)hipFree(m.sq_part);
    m.zero_bias = nullptr;
    m.sq_part = nullptr;
    m.train = 0;
    return fail(KS_ELAUNCH, "ks_mlp_train_init: %s failed", what);
  };
  const size_t esz = m.dtype == KS_MLP_BF16 ? 2 : 4;
  for (int l = 0; l < m.n_layers; ++l) {
    const size_t n = (size_t)m.npad[l] * m.kpad[l], nb = m.npad[l];
    std::vector<float> w(n, 0.f), b(nb, 0.f);
    for (int o = 0; o < m.dims[l + 1]; ++o) {
      for (int i = 0; i < m.dims[l]; ++i) w[(size_t)o * m.kpad[l] + i] = h->host_w[l][(size_t)o * m.dims[l] + i];
      b[o] = h->host_b[l][o];
    }
    float** wbufs[] = {&m.mW[l], &m.gW[l], &m.m1W[l], &m.m2W[l]};
    float** bbufs[] = {&m.mb[l], &m.gb[l], &m.m1b[l], &m.m2b[l]};
    for (float** q : wbufs)
      if (hipMalloc((void**)q, n * 4) != hipSuccess || hipMemset(*q, 0, n * 4) != hipSuccess) return give_up("allocation");
    for (float** q : bbufs)
      if (hipMalloc((void**)q, nb * 4) != hipSuccess || hipMemset(*q, 0, nb * 4) != hipSuccess) return give_up("allocation");
    if (hipMemcpy(m.mW[l], w.data(), n * 4, hipMemcpyHostToDevice) != hipSuccess ||
        hipMemcpy(m.mb[l], b.data(), nb * 4, hipMemcpyHostToDevice) != hipSuccess)
      return give_up("upload");
    // the first layer's transpose is padded to whole output tiles of the input-gradient product; the padding stays zero
    const size_t nt = l == 0 ? (size_t)round_up(m.kpad[0], kBN) * m.npad[0] : n;
    if (hipMalloc(&m.Wt[l], nt * esz) != hipSuccess || hipMemset(m.Wt[l], 0, nt * esz) != hipSuccess)
      return give_up("allocation");
    if (m.fused && l >= 1) {  // as many fragments as the forward copy: (fk / 2) tiles of inputs x (2 fn) steps over outputs
      const size_t np = (size_t)m.fn[l] * m.fk[l] * 512 * 2;
      if (hipMalloc(&m.WtP[l], np) != hipSuccess || hipMemset(m.WtP[l], 0, np) != hipSuccess) return give_up("allocation");
    }
  }
  const int wz = widest_pad(m);
  if (hipMalloc((void**)&m.zero_bias, (size_t)wz * 4) != hipSuccess || hipMemset(m.zero_bias, 0, (size_t)wz * 4) != hipSuccess)
    return give_up("allocation");
  if (hipMalloc((void**)&m.sq_part, sizeof(double) * kSqBlocks * 2 * KS_MAX_LAYERS) != hipSuccess)
    return give_up("allocation");
  m.train = 1;
  // working copies (among them the transposes, which did not exist yet) from the master weights
  if (m.dtype == KS_MLP_BF16) refresh_layers<__bf16>(m, (hipStream_t)0);
  else refresh_layers<float>(m, (hipStream_t)0);
  if (hipStreamSynchronize((hipStream_t)0) != hipSuccess) return give_up("refresh");
  return KS_OK;
}

template <typename T>
static void refresh_layers(DevMlp& m, hipStream_t s) {
  for (int l = 0; l < m.n_layers; ++l) {
    const int64_t n = (int64_t)m.npad[l] * m.kpad[l];
    const int64_t np = m.fused ? (int64_t)m.fn[l] * m.fk[l] * 512 : 0;
    const int64_t tot = n > np ? n : np;
    hipLaunchKernelGGL(refresh_kernel<T>, dim3((unsigned)((tot + 255) / 256)), dim3(256), 0, s, m.npad[l], m.kpad[l], m.mW[l],
                       (T*)m.W[l], (T*)m.Wt[l], m.fused ? (__bf16*)m.Wp[l] : (__bf16*)nullptr, m.fk[l], m.fn[l], (__bf16*)m.WtP[l]);
    (void)hipMemcpyAsync(m.b[l], m.mb[l], (size_t)m.npad[l] * 4, hipMemcpyDeviceToDevice, s);
    if (m.fused) (void)hipMemcpyAsync(m.bp[l], m.mb[l], (size_t)m.fn[l] * 32 * 4, hipMemcpyDeviceToDevice, s);
  }
}

constexpr int kDwSplit = 32;  // most slices the weight-gradient reduction over the rows is cut into
constexpr int kDiscMaxSlices = 64;  // most slices a long row reduction of the fp32 products (sgemm below) is cut into

// workspace: hidden activations of every layer, two (M, widest) gradient buffers, two transposes (widest, Mp)
struct TrainWs {
  char* act[KS_MAX_LAYERS];
  char* pre[KS_MAX_LAYERS];  // pre-activations of the hidden layers, kept only for GELU (not recoverable from its output)
  char *d0, *d1, *t0, *t1, *t2;
  float* part;  // partial sums of the split reductions
  int64_t Mp;
  // whole-network backward pass (chain_ok): per hidden layer the activations transposed, per layer dZ^T and one row of bias
  // partial sums per 128-row tile; all transposes have the row stride Mp128
  char *yT[KS_MAX_LAYERS], *dzT[KS_MAX_LAYERS];
  float *bpart[KS_MAX_LAYERS], *wpart[KS_MAX_LAYERS];  // wpart: the row slices of each layer's weight-gradient product
  int64_t Mp128;
};

// Whether a batch of M rows goes through the whole-network backward pass: bf16 networks that run the whole-network forward
// kernel on 128-row tiles, with hidden layers wide enough that every wavefront owns whole feature tiles of all four row tiles
// (the accumulator-order copy of the activations is laid out for that split).
static bool chain_ok(const DevMlp& m, int64_t M) {
  if (!m.fused || m.dtype != KS_MLP_BF16 || m.activation == KS_ACT_GELU || m.n_layers < 2 || M < 128 * 256) return false;
  for (int l = 0; l + 1 < m.n_layers; ++l)
    if (m.npad[l] != m.fn[l] * 32 || m.fn[l] * 4 <= kFusedWaves || !m.WtP[l + 1]) return false;
  // the transposed copies of the input and of the output gradient are cut from the LDS tile at their padded widths
  if (round_up(m.kpad[0], kBN) + 8 > m.lda || m.npad[m.n_layers - 1] + 8 > m.lda) return false;
  return true;
}
static int64_t carve_train(const DevMlp& m, int64_t M, char* base, TrainWs* ws) {
  const int64_t esz = m.dtype == KS_MLP_BF16 ? 2 : 4;
  const int64_t Mp = (M + 63) / 64 * 64;
  const int wz = widest_pad(m);
  int64_t off = 0;
  auto take = [&](int64_t bytes) {
    char* p = base ? base + off : nullptr;
    off += (bytes + 255) / 256 * 256;
    return p;
  };
  TrainWs w;
  std::memset(&w, 0, sizeof(w));
  for (int l = 0; l + 1 < m.n_layers; ++l) w.act[l] = take(M * m.npad[l] * esz);
  if (m.activation == KS_ACT_GELU)
    for (int l = 0; l + 1 < m.n_layers; ++l) w.pre[l] = take(M * m.npad[l] * esz);
  w.d0 = take(M * wz * esz);
  w.d1 = take(M * wz * esz);
  w.t0 = take((int64_t)wz * Mp * esz);
  w.t1 = take((int64_t)wz * Mp * esz);
  w.t2 = take((int64_t)wz * Mp * esz);
  int64_t maxw = 0;
  for (int l = 0; l < m.n_layers; ++l) maxw = (int64_t)m.npad[l] * m.kpad[l] > maxw ? (int64_t)m.npad[l] * m.kpad[l] : maxw;
  int64_t nparts = kDwSplit * maxw > (int64_t)4 * kColsumSlices * wz ? kDwSplit * maxw : (int64_t)4 * kColsumSlices * wz;
  if (m.n_layers == 1 && esz == 4)  // the one-pass weight and bias gradient of a single fp32 layer: slices of both
    nparts = nparts > (int64_t)kDiscMaxSlices * (maxw + wz) ? nparts : (int64_t)kDiscMaxSlices * (maxw + wz);
  w.part = (float*)take(nparts * 4);
  w.Mp = Mp;
  w.Mp128 = (M + 127) / 128 * 128;
  if (chain_ok(m, M)) {
    const int64_t tiles = w.Mp128 / 128;
    for (int l = 0; l + 1 < m.n_layers; ++l) {
      w.yT[l] = take((int64_t)m.npad[l] * w.Mp128 * esz);
      w.bpart[l] = (float*)take(tiles * m.npad[l] * 4);
    }
    for (int l = 0; l < m.n_layers; ++l) w.dzT[l] = take((int64_t)m.npad[l] * w.Mp128 * esz);
    w.bpart[m.n_layers - 1] = (float*)take(tiles * m.npad[m.n_layers - 1] * 4);
    for (int l = 0; l < m.n_layers; ++l) w.wpart[l] = (float*)take((int64_t)kDwSplit * m.npad[l] * m.kpad[l] * 4);
    w.yT[m.n_layers - 1] = take((int64_t)round_up(m.kpad[0], kBN) * w.Mp128 * esz);  // the network input, transposed
  }
  if (ws) *ws = w;
  return off;
}

static void keep_args(FusedArgs& a, const DevMlp& m, const TrainWs* ws) {
  for (int l = 0; l + 1 < m.n_layers; ++l) {
    a.keep_t[l] = (__bf16*)ws->yT[l];
  }
  a.keep_t_in = (__bf16*)ws->yT[m.n_layers - 1];
  a.in_t_width = round_up(m.kpad[0], kBN);
  a.ldt = ws->Mp128;
}

extern "C" int64_t ks_mlp_train_workspace_bytes(const KsMlp* h, int64_t M) {
  if (!h || M < 0) return 0;
  return carve_train(h->m, M, nullptr, nullptr) + 256;
}

template <typename T>
static int train_forward(DevMlp& m, hipStream_t s, int64_t M, const float* x, float* y, const TrainWs& ws) {
  // bf16 networks that fit the whole-network kernel run it, with every hidden layer's activations written out for the backward
  // pass as well; the stored rows must have the width the backward pass expects (its padding is in units of 64, the kernel's 32)
  bool whole = m.fused && m.dtype == KS_MLP_BF16 && m.activation != KS_ACT_GELU;
  for (int l = 0; whole && l + 1 < m.n_layers; ++l) whole = m.npad[l] == m.fn[l] * 32;
  m.chain_saved = 0;
  if (whole && chain_ok(m, M)) {  // activations in the formats of the whole-network backward pass, not row-major
    m.chain_saved = 1;
    return launch_fused_tile<128>(m, s, M, x, y, nullptr, &ws);
  }
  if (whole) return launch_fused(m, s, M, x, y, ws.act);
  const void* in = x;
  int64_t ldin = m.dims[0];
  for (int l = 0; l < m.n_layers; ++l) {
    const bool first = l == 0, last = l == m.n_layers - 1;
    const bool split_act = !last && m.activation == KS_ACT_GELU;  // keep the pre-activation, then apply GELU
    void* outp = last ? (void*)y : (split_act ? (void*)ws.pre[l] : (void*)ws.act[l]);
    const int64_t ldo = last ? m.dims[l + 1] : m.npad[l];
    const int act_l = split_act ? KS_ACT_NONE : m.activation;
    int rc;
    if (first && last) rc = launch_layer<T, true, true>(act_l, s, M, m.npad[l], m.kpad[l], m.dims[l], m.dims[l + 1], in, ldin, m.W[l], m.b[l], outp, ldo);
    else if (first) rc = launch_layer<T, true, false>(act_l, s, M, m.npad[l], m.kpad[l], m.dims[l], m.dims[l + 1], in, ldin, m.W[l], m.b[l], outp, ldo);
    else if (last) rc = launch_layer<T, false, true>(act_l, s, M, m.npad[l], m.kpad[l], m.dims[l], m.dims[l + 1], in, ldin, m.W[l], m.b[l], outp, ldo);
    else rc = launch_layer<T, false, false>(act_l, s, M, m.npad[l], m.kpad[l], m.dims[l], m.dims[l + 1], in, ldin, m.W[l], m.b[l], outp, ldo);
    if (rc != KS_OK) return rc;
    if (split_act) {
      const int64_t n = M * m.npad[l];
      hipLaunchKernelGGL(gelu_forward_kernel<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, n, (const T*)ws.pre[l], (T*)ws.act[l]);
      outp = ws.act[l];
    }
    in = outp;
    ldin = ldo;
  }
  return KS_OK;
}

extern "C" int ks_mlp_train_forward(KsMlp* h, ks_stream_t stream, int64_t M, const float* x, float* y, void* workspace) {
  if (!h || !h->m.train) return fail(KS_EINVAL, "ks_mlp_train_forward: call ks_mlp_train_init first");
  if (M <= 0 || !x || !y || !workspace) return fail(KS_EINVAL, "ks_mlp_train_forward: bad argument");
  if ((M + kBM - 1) / kBM > 0x7fffffff) return fail(KS_ELIMIT, "ks_mlp_train_forward: too many rows");
  TrainWs ws;
  carve_train(h->m, M, (char*)workspace, &ws);
  const int rc = h->m.dtype == KS_MLP_BF16 ? train_forward<__bf16>(h->m, (hipStream_t)stream, M, x, y, ws)
                                           : train_forward<float>(h->m, (hipStream_t)stream, M, x, y, ws);
  return rc != KS_OK ? rc : check_launch("ks_mlp_train_forward");
}

// The backward pass of a network whose forward kept the whole-network formats (chain_ok): the last layer's gradient by the small
// kernels, every hidden layer's in one launch of mlp_fused_bwd_kernel, then one weight-gradient product per layer.
template <typename T>
static int train_backward_chain(DevMlp& m, hipStream_t s, int64_t M, const float* x, const float* dy, const TrainWs& ws) {
  const int L = m.n_layers;
  const int64_t Mp = ws.Mp128, tiles = Mp / 128;
  const int npl = m.npad[L - 1];
  {
    FusedBwdArgs a;
    std::memset(&a, 0, sizeof(a));
    a.M = M; a.n_layers = L; a.lda = m.lda; a.ldt = Mp;
    a.dy = dy; a.out_dim = m.dims[L]; a.np_last = npl;
    for (int l = 0; l < L; ++l) {
      a.fk[l] = m.fk[l]; a.fn[l] = m.fn[l];
      a.WtP[l] = (const u32x4*)m.WtP[l];
      if (l + 1 < L) a.yT[l] = (const __bf16*)ws.yT[l];
      a.dzT[l] = (__bf16*)ws.dzT[l];
      a.bias_part[l] = ws.bpart[l];
    }
    const int lds = 128 * m.lda * 2;
#define KS_LAUNCH(A)                                                                                           \
  {                                                                                                            \
    auto kfn = mlp_fused_bwd_kernel<A>;                                                                        \
    if (lds > 64 * 1024 &&                                                                                     \
        hipFuncSetAttribute((const void*)kfn, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)  \
      return fail(KS_ELAUNCH, "ks_mlp_train_backward: cannot raise the LDS limit to %d bytes", lds);           \
    hipLaunchKernelGGL(kfn, dim3((unsigned)tiles), dim3(64 * kFusedWaves), lds, s, a);                         \
  }
    switch (m.activation) {
      case KS_ACT_ELU: KS_LAUNCH(KS_ACT_ELU) break;
      case KS_ACT_RELU: KS_LAUNCH(KS_ACT_RELU) break;
      case KS_ACT_TANH: KS_LAUNCH(KS_ACT_TANH) break;
      default: KS_LAUNCH(KS_ACT_NONE) break;
    }
#undef KS_LAUNCH
  }
  (void)x;  // the training forward left its transpose behind
  const T* xT = (const T*)ws.yT[L - 1];
  GradFinishArgs g;
  std::memset(&g, 0, sizeof(g));
  g.n_layers = L; g.tiles = (int)tiles;
  int wblocks = 0, bblocks = 0;
  for (int l = L - 1; l >= 0; --l) {
    const int np = m.npad[l], kp = m.kpad[l], kp128 = round_up(kp, kBN);
    const T* dzT = (const T*)ws.dzT[l];
    const T* yT = l > 0 ? (const T*)ws.yT[l - 1] : xT;
    const bool wide = np % 128 == 0;
    int ksplit = wide ? kDwSplit : kDwSplit / 2;
    while (ksplit > 1 && (Mp / 128) % ksplit != 0) ksplit >>= 1;  // K slices of 128 rows per pass
    int rc;
    if (wide)
      rc = launch_layer_tile<T, false, true, 128, 128, 2, 2, 2>(KS_ACT_NONE, s, np, kp128, (int)Mp, (int)Mp, kp, dzT, Mp, yT, m.zero_bias,
                                                                 (void*)ws.wpart[l], kp, ksplit);
    else
      rc = launch_layer_tile<T, false, true, 64, 128, 2, 2>(KS_ACT_NONE, s, np, kp128, (int)Mp, (int)Mp, kp, dzT, Mp, yT, m.zero_bias,
                                                             (void*)ws.wpart[l], kp, ksplit);
    if (rc != KS_OK) return rc;
    g.nz[l] = ksplit; g.nW[l] = (int64_t)np * kp; g.nb[l] = np;
    g.wpart[l] = ws.wpart[l]; g.bpart[l] = ws.bpart[l]; g.gW[l] = m.gW[l]; g.gb[l] = m.gb[l];
  }
  for (int l = 0; l < L; ++l) {
    g.first_w[l] = wblocks; g.first_b[l] = bblocks;
    wblocks += (int)((g.nW[l] + 255) / 256);
    bblocks += (g.nb[l] + 3) / 4;
  }
  g.first_w[L] = wblocks; g.first_b[L] = bblocks;
  hipLaunchKernelGGL(grad_finish_kernel, dim3((unsigned)(wblocks + bblocks)), dim3(256), 0, s, g);
  return KS_OK;
}

template <bool A_KC, bool B_KC>
static void sgemm(hipStream_t s, int64_t M, int N, int64_t K, const float* A, int64_t lda, const float* B, int64_t ldb, float* C,
                  int64_t ldc, const float* bias, int act, bool accumulate, float* part, float* colsum = nullptr, float* colpart = nullptr);

template <typename T>
static int train_backward(DevMlp& m, hipStream_t s, int64_t M, const float* x, const float* dy, const TrainWs& ws,
                          float* dx = nullptr, bool want_w = true, bool accumulate_dx = false, const uint8_t* zero_rows = nullptr) {
  const int L = m.n_layers;
  const int64_t Mp = ws.Mp;
  if (m.chain_saved && sizeof(T) == 2) {
    if (want_w && !dx) return train_backward_chain<T>(m, s, M, x, dy, ws);
    // the layer-by-layer pass below reads row-major activations: rebuild them from the transposed copies
    for (int l = 0; l + 1 < L; ++l)
      hipLaunchKernelGGL((transpose_kernel<T, T>), dim3((unsigned)((m.npad[l] + 31) / 32), (unsigned)((M + 31) / 32)), dim3(256), 0, s,
                         (int64_t)m.npad[l], (int)M, ws.Mp128, (const T*)ws.yT[l], (int)M, (int64_t)m.npad[l], (T*)ws.act[l]);
    m.chain_saved = 0;
  }
  T* dz = (T*)ws.d0;
  T* dnext = (T*)ws.d1;
  if (L == 1 && sizeof(T) == 4 && m.dims[1] == m.npad[0]) {
    // a single fp32 layer whose width needs no padding (the projections of the recurrent cells): the caller's gradient is
    // already the operand, and with one layer nothing below writes into this buffer
    dz = (T*)const_cast<float*>(dy);
  } else {  // the output gradient in working precision, padded to the last layer's width
    const int64_t n = M * m.npad[L - 1];
    hipLaunchKernelGGL(cast_pad_kernel<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, M, m.dims[L], m.npad[L - 1], dy, dz);
  }
  // The layer-l step needs dZ_l (row-major, for the input gradient), dZ_l^T and Y_{l-1}^T (for the weight gradient) and
  // the column sums of dZ_l.  For hidden layers of a width that is a multiple of 64 one fused pass (bwd_prep_kernel)
  // turns the input gradient of the layer above into all four; otherwise separate kernels do.
  T* dzT = (T*)ws.t0;    // dZ_l^T
  T* dzT_next = (T*)ws.t2;
  bool have_dzT = false, have_bias = false;
  for (int l = L - 1; l >= 0; --l) {
    const int np = m.npad[l], kp = m.kpad[l], kp128 = round_up(kp, kBN);
    if (l == 0 && dx) {  // gradient with respect to the network input
      // an fp32 network whose input width needs no padding: the product writes the caller's buffer itself
      const bool direct = sizeof(T) == 4 && m.dims[0] == kp128 && !accumulate_dx && !zero_rows;
      const int rc0 = launch_layer<T, false, false>(KS_ACT_NONE, s, M, kp128, np, np, kp128, dz, np, m.Wt[0], m.zero_bias,
                                                    direct ? (T*)dx : dnext, kp128);
      if (rc0 != KS_OK) return rc0;
      if (!direct) {
        const int64_t n = M * m.dims[0];
        hipLaunchKernelGGL(unpad_cast_kernel<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, M, m.dims[0], kp128, (const T*)dnext, dx,
                           accumulate_dx ? 1 : 0, zero_rows);
      }
    }
    if (!want_w && l == 0) break;
    if (L == 1 && sizeof(T) == 4 && np >= 128) {
      // A single fp32 layer (the projections of the recurrent cells, over all the (step, env) rows of a trajectory slice): the
      // weight gradient dZ^T X and the bias gradient, the column sums of dZ, in one pass over the row-major operands as they
      // are, on the 128 x 128 tiles of the long-reduction product; no transposed copies.
      float* colpart = ws.part + (int64_t)kDiscMaxSlices * np * kp;
      sgemm<false, false>(s, np, m.dims[0], M, (const float*)dz, np, x, m.dims[0], m.gW[0], kp, nullptr, KS_ACT_NONE, false, ws.part,
                          m.gb[0], colpart);
      break;
    }
    if (want_w && !have_bias) {
      const int nz = M >= 32768 ? 4 * kColsumSlices : kColsumSlices;  // narrow layers: more row slices fill the chip
      hipLaunchKernelGGL(colsum_kernel<T>, dim3((unsigned)((np + 63) / 64), nz), dim3(256), 0, s, M, np, dz, ws.part);
      hipLaunchKernelGGL(sum_parts_tree_kernel, dim3((unsigned)np), dim3(64), 0, s, (int64_t)np, nz, ws.part, m.gb[l]);
    }
    if (want_w && !have_dzT)
      hipLaunchKernelGGL((transpose_kernel<T, T>), dim3((unsigned)((Mp + 31) / 32), (unsigned)((np + 31) / 32)), dim3(256), 0, s, M, np,
                         (int64_t)np, dz, np, Mp, dzT);
    have_dzT = have_bias = false;
    bool have_yT = false;
    int rc;
    if (l > 0) {
      // input gradient, then through the activation of the layer below
      rc = launch_layer<T, false, false>(KS_ACT_NONE, s, M, kp, np, np, kp, dz, np, m.Wt[l], m.zero_bias, dnext, kp);
      if (rc != KS_OK) return rc;
      const bool fused = want_w && m.activation != KS_ACT_GELU && kp % 64 == 0 && kp == kp128 && kp == m.npad[l - 1];
      if (fused) {
#define KS_PREP(A) hipLaunchKernelGGL((bwd_prep_kernel<T, A>), dim3((unsigned)(kp / 64), kColsumSlices), dim3(256), 0, s, M, Mp, kp, \
                                      (const T*)ws.act[l - 1], dnext, dzT_next, (T*)ws.t1, ws.part)
        switch (m.activation) {
          case KS_ACT_ELU: KS_PREP(KS_ACT_ELU); break;
          case KS_ACT_RELU: KS_PREP(KS_ACT_RELU); break;
          case KS_ACT_TANH: KS_PREP(KS_ACT_TANH); break;
          default: KS_PREP(KS_ACT_NONE); break;
        }
#undef KS_PREP
        hipLaunchKernelGGL(sum_parts_tree_kernel, dim3((unsigned)kp), dim3(64), 0, s, (int64_t)kp, kColsumSlices, ws.part, m.gb[l - 1]);
        have_yT = have_dzT = have_bias = true;
      } else {
        const int64_t n = M * kp;
#define KS_ACTB(A) hipLaunchKernelGGL((act_backward_kernel<T, A>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, n, (const T*)ws.act[l - 1], dnext)
        switch (m.activation) {
          case KS_ACT_ELU: KS_ACTB(KS_ACT_ELU); break;
          case KS_ACT_RELU: KS_ACTB(KS_ACT_RELU); break;
          case KS_ACT_TANH: KS_ACTB(KS_ACT_TANH); break;
          case KS_ACT_GELU:
            hipLaunchKernelGGL(gelu_backward_kernel<T>, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, n, (const T*)ws.pre[l - 1], dnext);
            break;
          default: break;
        }
#undef KS_ACTB
      }
    }
    if (!want_w) {
      T* tmp = dz; dz = dnext; dnext = tmp;
      continue;
    }
    // weight gradient: dZ^T (np, Mp) times Y_prev^T (kp128, Mp)^T
    if (!have_yT) {
      if (l == 0)
        hipLaunchKernelGGL((transpose_kernel<float, T>), dim3((unsigned)((Mp + 31) / 32), (unsigned)((kp128 + 31) / 32)), dim3(256), 0, s, M,
                           m.dims[0], (int64_t)m.dims[0], x, kp128, Mp, (T*)ws.t1);
      else
        hipLaunchKernelGGL((transpose_kernel<T, T>), dim3((unsigned)((Mp + 31) / 32), (unsigned)((kp128 + 31) / 32)), dim3(256), 0, s, M,
                           m.npad[l - 1], (int64_t)m.npad[l - 1], (const T*)ws.act[l - 1], kp128, Mp, (T*)ws.t1);
    }
    // the reduction runs over the rows: cut it into slices so that the grid covers the chip, then add the slices up
    // wide layers over many rows: 128 x 128 output tiles halve the operand traffic per flop, twice the slices keep the grid
    const bool wide = Mp >= 32768 && np % 128 == 0;
    int ksplit = wide ? kDwSplit : kDwSplit / 2;
    while (ksplit > 1 && (Mp / 64) % ksplit != 0) ksplit >>= 1;
    if (wide)
      rc = launch_layer_tile<T, false, true, 128, 128, 2, 2>(KS_ACT_NONE, s, np, kp128, (int)Mp, (int)Mp, kp, dzT, Mp, ws.t1,
                                                              m.zero_bias, ksplit > 1 ? (void*)ws.part : (void*)m.gW[l], kp, ksplit);
    else
      rc = launch_layer_tile<T, false, true, 64, 128, 2, 2>(KS_ACT_NONE, s, np, kp128, (int)Mp, (int)Mp, kp, dzT, Mp, ws.t1,
                                                             m.zero_bias, ksplit > 1 ? (void*)ws.part : (void*)m.gW[l], kp, ksplit);
    if (rc != KS_OK) return rc;
    if (ksplit > 1) {
      const int64_t n = (int64_t)np * kp;
      hipLaunchKernelGGL(sum_parts_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, n, ksplit, ws.part, m.gW[l]);
    }
    if (l == 0) break;
    T* tmp = dz; dz = dnext; dnext = tmp;
    tmp = dzT; dzT = dzT_next; dzT_next = tmp;
  }
  return KS_OK;
}

extern "C" int ks_mlp_train_backward(KsMlp* h, ks_stream_t stream, int64_t M, const float* x, const float* dy, void* workspace) {
  if (!h || !h->m.train) return fail(KS_EINVAL, "ks_mlp_train_backward: call ks_mlp_train_init first");
  if (M <= 0 || !x || !dy || !workspace) return fail(KS_EINVAL, "ks_mlp_train_backward: bad argument");
  if (M > (1 << 30)) return fail(KS_ELIMIT, "ks_mlp_train_backward: too many rows");
  TrainWs ws;
  carve_train(h->m, M, (char*)workspace, &ws);
  const int rc = h->m.dtype == KS_MLP_BF16 ? train_backward<__bf16>(h->m, (hipStream_t)stream, M, x, dy, ws)
                                           : train_backward<float>(h->m, (hipStream_t)stream, M, x, dy, ws);
  return rc != KS_OK ? rc : check_launch("ks_mlp_train_backward");
}

extern "C" int ks_mlp_train_backward_dx(KsMlp* h, ks_stream_t stream, int64_t M, const float* x, const float* dy, float* dx,
                                        int32_t weight_gradients, int32_t accumulate_dx, const uint8_t* zero_rows, void* workspace) {
  if (!h || !h->m.train) return fail(KS_EINVAL, "ks_mlp_train_backward_dx: call ks_mlp_train_init first");
  if (M <= 0 || !dy || !dx || !workspace || (weight_gradients && !x)) return fail(KS_EINVAL, "ks_mlp_train_backward_dx: bad argument");
  if (M > (1 << 30)) return fail(KS_ELIMIT, "ks_mlp_train_backward_dx: too many rows");
  TrainWs ws;
  carve_train(h->m, M, (char*)workspace, &ws);
  const bool w = weight_gradients != 0, acc = accumulate_dx != 0;
  const int rc = h->m.dtype == KS_MLP_BF16 ? train_backward<__bf16>(h->m, (hipStream_t)stream, M, x, dy, ws, dx, w, acc, zero_rows)
                                           : train_backward<float>(h->m, (hipStream_t)stream, M, x, dy, ws, dx, w, acc, zero_rows);
  return rc != KS_OK ? rc : check_launch("ks_mlp_train_backward_dx");
}

extern "C" int ks_mlp_freeze_bias_prefix(KsMlp* h, int32_t layer, int32_t count) {
  if (!h) return fail(KS_EINVAL, "ks_mlp_freeze_bias_prefix: null handle");
  if (layer < 0 || layer >= h->m.n_layers || count < 0 || count > h->m.dims[layer + 1])
    return fail(KS_EINVAL, "ks_mlp_freeze_bias_prefix: layer %d, count %d out of range", layer, count);
  h->m.bias_frozen[layer] = count;
  return KS_OK;
}

extern "C" int ks_grad_sqnorm(ks_stream_t stream, int64_t n, const float* g, double* acc) {
  if (n < 0 || !acc || (n > 0 && !g)) return fail(KS_EINVAL, "ks_grad_sqnorm: bad argument");
  if (n == 0) return KS_OK;
  hipLaunchKernelGGL(sqnorm_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, n, g, acc);
  return check_launch("ks_grad_sqnorm");
}

extern "C" int ks_mlp_grad_sqnorm(const KsMlp* h, ks_stream_t stream, double* acc) {
  if (!h || !h->m.train || !acc) return fail(KS_EINVAL, "ks_mlp_grad_sqnorm: bad argument");
  SqTensors t;
  int nt = 0;
  for (int l = 0; l < h->m.n_layers; ++l) {
    t.g[nt] = h->m.gW[l];
    t.n[nt++] = (int64_t)h->m.npad[l] * h->m.kpad[l];
    const int fz = h->m.bias_frozen[l];
    if (h->m.npad[l] > fz) {
      t.g[nt] = h->m.gb[l] + fz;
      t.n[nt++] = (int64_t)h->m.npad[l] - fz;
    }
  }
  hipLaunchKernelGGL(sqnorm_parts_kernel, dim3(kSqBlocks, (unsigned)nt), dim3(256), 0, (hipStream_t)stream, t, h->m.sq_part);
  hipLaunchKernelGGL(sqnorm_finish_kernel, dim3(1), dim3(256), 0, (hipStream_t)stream, nt * kSqBlocks, h->m.sq_part, acc);
  return check_launch("ks_mlp_grad_sqnorm");
}

static int check_adam(const KsAdamParams* p, const char* who) {
  if (!p) return fail(KS_EINVAL, "%s: null parameters", who);
  if (p->step < 1) return fail(KS_EINVAL, "%s: step starts at 1", who);
  if (!(p->b1 >= 0.f && p->b1 < 1.f && p->b2 >= 0.f && p->b2 < 1.f)) return fail(KS_EINVAL, "%s: betas must be in [0, 1)", who);
  return KS_OK;
}

extern "C" int ks_adam_step(ks_stream_t stream, int64_t n, float* param, const float* grad, float* m1, float* m2,
                            const KsAdamParams* p, const double* sqnorm) {
  const int rc = check_adam(p, "ks_adam_step");
  if (rc != KS_OK) return rc;
  if (n < 0 || (n > 0 && (!param || !grad || !m1 || !m2))) return fail(KS_EINVAL, "ks_adam_step: bad argument");
  if (n == 0) return KS_OK;
  hipLaunchKernelGGL(adam_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, n, param, grad, m1, m2, *p, sqnorm);
  return check_launch("ks_adam_step");
}

extern "C" int ks_mlp_adam_step(KsMlp* h, ks_stream_t stream, const KsAdamParams* p, const double* sqnorm) {
  if (!h || !h->m.train) return fail(KS_EINVAL, "ks_mlp_adam_step: call ks_mlp_train_init first");
  const int rc = check_adam(p, "ks_mlp_adam_step");
  if (rc != KS_OK) return rc;
  DevMlp& m = h->m;
  hipStream_t s = (hipStream_t)stream;
  AdamNetArgs n{};
  n.n_layers = m.n_layers;
  int blocks = 0;
  for (int l = 0; l < m.n_layers; ++l) {
    n.npad[l] = m.npad[l]; n.kpad[l] = m.kpad[l]; n.fk[l] = m.fk[l]; n.fn[l] = m.fn[l]; n.frozen[l] = m.bias_frozen[l];
    n.first_block[l] = blocks;
    blocks += (int)(((int64_t)m.npad[l] * m.kpad[l] + 255) / 256);  // npad * kpad >= npad: the bias rides on the first threads
    n.mW[l] = m.mW[l]; n.m1W[l] = m.m1W[l]; n.m2W[l] = m.m2W[l]; n.gW[l] = m.gW[l];
    n.mb[l] = m.mb[l]; n.m1b[l] = m.m1b[l]; n.m2b[l] = m.m2b[l]; n.gb[l] = m.gb[l];
    n.W[l] = m.W[l]; n.Wt[l] = m.Wt[l]; n.Wp[l] = m.fused ? (__bf16*)m.Wp[l] : nullptr; n.WtP[l] = (__bf16*)m.WtP[l];
    n.b[l] = m.b[l]; n.bp[l] = m.fused ? m.bp[l] : nullptr;
  }
  n.first_block[m.n_layers] = blocks;
  if (m.dtype == KS_MLP_BF16) hipLaunchKernelGGL(adam_net_kernel<__bf16>, dim3((unsigned)blocks), dim3(256), 0, s, n, *p, sqnorm);
  else hipLaunchKernelGGL(adam_net_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, s, n, *p, sqnorm);
  return check_launch("ks_mlp_adam_step");
}

// ---------------------------------------------------------------- discriminator update (ksim/task/amp.py:360-438)
// Gradient of   0.5 sum (D(real) - 1)^2 + 0.5 sum (D(sim) + 1)^2 + coef / 2 * mean_b sum_t |grad_x D(real[b, t])|^2
// with respect to every weight and bias of an MLP D with one output, applied frame by frame.  The last term differentiates
// the network twice.  With z_l = W_l y_{l-1} + b_l, y_l = f(z_l), the input gradient is g = W_1^T d_1 with d_L = 1,
// d_l = f'(z_l) * (W_{l+1}^T d_{l+1}) =: f'(z_l) * a_l.  The gradient of P(g) walks that computation backwards, which is a
// forward sweep through the layers: with v_0 = dP/dg,
//   dP/dW_l += d_l^T v_{l-1},   u_l = v_{l-1} W_l^T,   v_l = u_l * f'(z_l),   r_l = u_l * a_l * f''(z_l),
// and r_l, the part that reaches z_l through f', joins the ordinary backward pass of the squared-error terms as an extra
// gradient of z_l on the real rows.  The discriminator is small next to the policy, so everything here runs in fp32 on the
// master weights, the products on the fp32 matrix-core instruction.
namespace ks {

// C(i, j) (+)= sum_k A(i, k) B(k, j) in fp32 on the matrix cores: 64 x 64 tile per workgroup, 16-deep slices through LDS,
// each of the four wavefronts accumulating one 32 x 32 quadrant with v_mfma_f32_32x32x2_f32 (lane c + 32 h feeds
// A(c, 2 s + h) and B(2 s + h, c) of step s and ends up with C(8 g + 4 h + e, c) in accumulator register 4 g + e).
// A_KC: A is stored (i, k) with k contiguous, otherwise (k, i); B_KC: B is stored (j, k) with k contiguous, otherwise (k, j).
// gridDim.z cuts the k range into slices of kslice; with more than one slice, slice z writes its partial product (M, N)
// densely to C + z * M * N and sum_slices_kernel adds them up in a fixed order.
template <bool A_KC, bool B_KC>
__global__ __launch_bounds__(256) void sgemm_kernel(int M, int N, int K, const float* __restrict__ A, int64_t lda,
                                                    const float* __restrict__ B, int64_t ldb, float* __restrict__ C, int64_t ldc,
                                                    int kslice, const float* __restrict__ bias, int act, int accumulate) {
  __shared__ float As[16][68];
  __shared__ float Bs[16][68];
  const int t = threadIdx.x, i0 = blockIdx.y * 64, j0 = blockIdx.x * 64;
  const int kbeg = blockIdx.z * kslice, kend = min(K, kbeg + kslice);
  const int wave = t >> 6, lane = t & 63, c = lane & 31, h = lane >> 5;
  const int wi = (wave >> 1) * 32, wj = (wave & 1) * 32;
  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  for (int k0 = kbeg; k0 < kend; k0 += 16) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int ka = A_KC ? t % 16 : t / 64 + 4 * r, ia = A_KC ? t / 16 + 16 * r : t % 64;
      const int gi = i0 + ia, gka = k0 + ka;
      As[ka][ia] = (gi < M && gka < kend) ? (A_KC ? A[(int64_t)gi * lda + gka] : A[(int64_t)gka * lda + gi]) : 0.f;
      const int kb = B_KC ? t % 16 : t / 64 + 4 * r, jb = B_KC ? t / 16 + 16 * r : t % 64;
      const int gj = j0 + jb, gkb = k0 + kb;
      Bs[kb][jb] = (gj < N && gkb < kend) ? (B_KC ? B[(int64_t)gj * ldb + gkb] : B[(int64_t)gkb * ldb + gj]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int s = 0; s < 8; ++s)
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(As[2 * s + h][wi + c], Bs[2 * s + h][wj + c], acc, 0, 0, 0);
    __syncthreads();
  }
  const bool sliced = gridDim.z > 1;
  float* out = sliced ? C + (int64_t)blockIdx.z * M * N : C;
  const int64_t ld = sliced ? N : ldc;
  const int gj = j0 + wj + c;
  if (gj >= N) return;
  const float bj = (!sliced && bias) ? bias[gj] : 0.f;
#pragma unroll
  for (int g = 0; g < 4; ++g)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int gi = i0 + wi + 8 * g + 4 * h + e;
      if (gi >= M) continue;
      float v = acc[4 * g + e];
      if (!sliced) {
        v += bj;
        if (act == KS_ACT_ELU) v = v > 0.f ? v : expm1f(v);
        else if (act == KS_ACT_RELU) v = fmaxf(v, 0.f);
        else if (act == KS_ACT_TANH) v = tanhf(v);
        if (accumulate) v += out[(int64_t)gi * ld + gj];
      }
      out[(int64_t)gi * ld + gj] = v;
    }
}

// The same product for the weight and bias gradients of wide layers, C(i, j) (+)= sum_k A(k, i) B(k, j) with both operands
// stored (k, .) and a long reduction over the rows: a 128 x 128 tile per workgroup (each wavefront a 64 x 64 block = 2 x 2 MFMA tiles, so a value read
// from LDS feeds two matrix instructions), 16-byte global loads (vec_a / vec_b: the operand's rows are 16-byte aligned) whose
// next slice is in flight while the matrix cores work on this one.  A narrow B (71 columns, or the single column of ones that
// makes the product a column sum) wastes matrix work, not memory traffic, which is what bounds these products.  `colsum`
// (nullable) also receives sum_k A(k, i), the bias gradient that goes with a weight gradient, from the tiles that pass through
// LDS anyway.  Slices and partial outputs as in sgemm_kernel.
__global__ __launch_bounds__(256) void sgemm_tn128_kernel(int M, int N, int K, const float* __restrict__ A, int64_t lda,
                                                          const float* __restrict__ B, int64_t ldb, float* __restrict__ C, int64_t ldc,
                                                          int kslice, int accumulate, int vec_a, int vec_b,
                                                          float* __restrict__ colsum) {
  __shared__ __attribute__((aligned(16))) float As[16][132];
  __shared__ __attribute__((aligned(16))) float Bs[16][132];
  const int t = threadIdx.x, i0 = blockIdx.y * 128, j0 = blockIdx.x * 128;
  const int kbeg = blockIdx.z * kslice, kend = min(K, kbeg + kslice);
  const int wave = t >> 6, lane = t & 63, c = lane & 31, h = lane >> 5;
  const int wi = (wave >> 1) * 64, wj = (wave & 1) * 64;
  f32x16 acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;
  float4 ra[2], rb[2];
  float cs = 0.f;  // colsum: this thread's column of A, summed over the slice
  // thread t loads rows k = t / 32 and 8 + t / 32 of the slice, four consecutive columns from 4 (t % 32)
  const int lk = t >> 5, l4 = (t & 31) * 4;
#define KS_TN_FETCH(K0)                                                                                           \
  _Pragma("unroll") for (int r = 0; r < 2; ++r) {                                                                 \
    const int k = (K0) + lk + 8 * r;                                                                              \
    const int gi = i0 + l4, gj = j0 + l4;                                                                         \
    ra[r] = float4{0.f, 0.f, 0.f, 0.f};                                                                           \
    rb[r] = float4{0.f, 0.f, 0.f, 0.f};                                                                           \
    if (k < kend) {                                                                                               \
      if (gi + 3 < M && vec_a) ra[r] = *reinterpret_cast<const float4*>(A + (int64_t)k * lda + gi);               \
      else if (gi < M) {                                                                                          \
        const float* q = A + (int64_t)k * lda + gi;                                                               \
        ra[r].x = q[0]; if (gi + 1 < M) ra[r].y = q[1]; if (gi + 2 < M) ra[r].z = q[2]; if (gi + 3 < M) ra[r].w = q[3]; \
      }                                                                                                           \
      if (gj + 3 < N && vec_b) rb[r] = *reinterpret_cast<const float4*>(B + (int64_t)k * ldb + gj);               \
      else if (gj < N) {                                                                                          \
        const float* q = B + (int64_t)k * ldb + gj;                                                               \
        rb[r].x = q[0]; if (gj + 1 < N) rb[r].y = q[1]; if (gj + 2 < N) rb[r].z = q[2]; if (gj + 3 < N) rb[r].w = q[3]; \
      }                                                                                                           \
    }                                                                                                             \
  }
  KS_TN_FETCH(kbeg)
  for (int k0 = kbeg; k0 < kend; k0 += 16) {
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      *reinterpret_cast<float4*>(&As[lk + 8 * r][l4]) = ra[r];
      *reinterpret_cast<float4*>(&Bs[lk + 8 * r][l4]) = rb[r];
    }
    __syncthreads();
    KS_TN_FETCH(k0 + 16)  // beyond the slice: zeros that are never stored
    if (colsum && blockIdx.x == 0 && t < 128) {  // sum_k A(k, i) on the side: the tile is in LDS anyway
#pragma unroll
      for (int k = 0; k < 16; ++k) cs += As[k][t];
    }
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const float a0 = As[2 * s + h][wi + c], a1 = As[2 * s + h][wi + 32 + c];
      const float b0 = Bs[2 * s + h][wj + c], b1 = Bs[2 * s + h][wj + 32 + c];
      acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
      acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
      acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
      acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
    }
    __syncthreads();
  }
#undef KS_TN_FETCH
  const bool sliced = gridDim.z > 1;
  float* out = sliced ? C + (int64_t)blockIdx.z * M * N : C;
  const int64_t ld = sliced ? N : ldc;
  if (colsum && blockIdx.x == 0 && t < 128 && i0 + t < M) {  // sliced: partial row z of (slices, M); else the sums themselves
    float* q = colsum + (sliced ? (int64_t)blockIdx.z * M : 0) + i0 + t;
    *q = (!sliced && accumulate) ? *q + cs : cs;
  }
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int gj = j0 + wj + 32 * b + c;
      if (gj >= N) continue;
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int gi = i0 + wi + 32 * a + 8 * g + 4 * h + e;
          if (gi >= M) continue;
          float v = acc[a][b][4 * g + e];
          if (!sliced && accumulate) v += out[(int64_t)gi * ld + gj];
          out[(int64_t)gi * ld + gj] = v;
        }
    }
}

__global__ __launch_bounds__(256) void sum_slices_kernel(int M, int N, int nz, const float* __restrict__ part, float* __restrict__ C,
                                                         int64_t ldc, int accumulate) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)M * N) return;
  float s = 0.f;
  const int64_t mn = (int64_t)M * N;
  for (int z0 = 0; z0 < nz; z0 += 8) {  // eight slices' loads in flight, added in slice order as before
    float v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = z0 + k < nz ? part[(int64_t)(z0 + k) * mn + idx] : 0.f;
#pragma unroll
    for (int k = 0; k < 8; ++k)
      if (z0 + k < nz) s += v[k];
  }
  const int i = (int)(idx / N), j = (int)(idx - (int64_t)i * N);
  C[(int64_t)i * ldc + j] = accumulate ? C[(int64_t)i * ldc + j] + s : s;
}

__global__ __launch_bounds__(256) void fill_kernel(int64_t n, float v, float* __restrict__ p) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx < n) p[idx] = v;
}

// first and second derivative of the activation from its output y = f(z)
__device__ __forceinline__ void act_derivatives(int act, float y, float& d1, float& d2) {
  d1 = 1.f; d2 = 0.f;
  if (act == KS_ACT_ELU) { if (y <= 0.f) { d1 = y + 1.f; d2 = y + 1.f; } }  // exp(z) = elu(z) + 1 for z <= 0
  else if (act == KS_ACT_RELU) d1 = y > 0.f ? 1.f : 0.f;
  else if (act == KS_ACT_TANH) { d1 = 1.f - y * y; d2 = -2.f * y * d1; }
}

// dz = out - target (target +1 on the first n_real rows, -1 on the rest) and the two squared-error sums (one workgroup)
__global__ __launch_bounds__(1024) void disc_signal_kernel(int64_t n_real, int64_t n, const float* __restrict__ out, float* __restrict__ dz,
                                                           float* __restrict__ losses) {
  __shared__ double sh[2][1024];
  double a = 0.0, b = 0.0;
  for (int64_t i = threadIdx.x; i < n; i += 1024) {
    const float e = out[i] - (i < n_real ? 1.f : -1.f);
    dz[i] = e;
    if (i < n_real) a += 0.5 * (double)e * e; else b += 0.5 * (double)e * e;
  }
  sh[0][threadIdx.x] = a; sh[1][threadIdx.x] = b;
  __syncthreads();
  for (int w = 512; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) { sh[0][threadIdx.x] += sh[0][threadIdx.x + w]; sh[1][threadIdx.x] += sh[1][threadIdx.x + w]; }
    __syncthreads();
  }
  if (threadIdx.x == 0) { losses[0] = (float)sh[0][0]; losses[1] = (float)sh[1][0]; }
}

// penalty value coef / 2 * sum g^2 / n_motions and, in place, its gradient v = coef / n_motions * g (one workgroup)
__global__ __launch_bounds__(1024) void disc_penalty_kernel(int64_t n, float coef, float inv_motions, float* __restrict__ g,
                                                            float* __restrict__ loss) {
  __shared__ double sh[1024];
  double a = 0.0;
  for (int64_t i = threadIdx.x; i < n; i += 1024) {
    const float v = g[i];
    a += (double)v * v;
    g[i] = coef * inv_motions * v;
  }
  sh[threadIdx.x] = a;
  __syncthreads();
  for (int w = 512; w > 0; w >>= 1) {
    if ((int)threadIdx.x < w) sh[threadIdx.x] += sh[threadIdx.x + w];
    __syncthreads();
  }
  if (threadIdx.x == 0) *loss = (float)(0.5 * coef * inv_motions * sh[0]);
}

// d = f'(y) * a
__global__ __launch_bounds__(256) void disc_delta_kernel(int64_t n, int act, const float* __restrict__ y, const float* __restrict__ a,
                                                         float* __restrict__ d) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n) return;
  float d1, d2;
  act_derivatives(act, y[idx], d1, d2);
  d[idx] = d1 * a[idx];
}

// v = u * f'(y), r = u * a * f''(y)
__global__ __launch_bounds__(256) void disc_tangent_kernel(int64_t n, int act, const float* __restrict__ y, const float* __restrict__ a,
                                                           const float* __restrict__ u, float* __restrict__ v, float* __restrict__ r) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n) return;
  float d1, d2;
  act_derivatives(act, y[idx], d1, d2);
  const float uu = u[idx];
  v[idx] = uu * d1;
  r[idx] = uu * a[idx] * d2;
}

// dz = dy * f'(y) (+ r on the first n_extra elements)
__global__ __launch_bounds__(256) void disc_dz_kernel(int64_t n, int64_t n_extra, int act, const float* __restrict__ y,
                                                      const float* __restrict__ r, float* __restrict__ dz) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= n) return;
  float d1, d2;
  act_derivatives(act, y[idx], d1, d2);
  float v = dz[idx] * d1;
  if (idx < n_extra) v += r[idx];
  dz[idx] = v;
}

}  // namespace ks

// kDiscMaxSlices is defined beside kDwSplit: the training backward pass of single fp32 layers shares these products

struct DiscWs {
  float* y[KS_MAX_LAYERS];      // hidden outputs, all rows
  float* a[KS_MAX_LAYERS];      // real rows: W_{l+1}^T d_{l+1}
  float* d[KS_MAX_LAYERS];      // real rows: d_l
  float* r[KS_MAX_LAYERS];      // real rows: extra gradient of z_l
  float *out, *dz0, *dz1, *g, *u, *v, *ones, *part, *colpart;
};

static int64_t carve_disc(const DevMlp& m, int64_t R, int64_t M, char* base, DiscWs* ws) {
  int64_t off = 0;
  auto take = [&](int64_t floats) {
    char* p = base ? base + off : nullptr;
    off += (floats * 4 + 255) / 256 * 256;
    return (float*)p;
  };
  DiscWs w;
  std::memset(&w, 0, sizeof(w));
  int wmax = 1;
  int64_t maxw = 1;
  for (int l = 0; l <= m.n_layers; ++l) wmax = m.dims[l] > wmax ? m.dims[l] : wmax;
  for (int l = 0; l < m.n_layers; ++l) maxw = (int64_t)m.dims[l] * m.dims[l + 1] > maxw ? (int64_t)m.dims[l] * m.dims[l + 1] : maxw;
  for (int l = 0; l + 1 < m.n_layers; ++l) {
    w.y[l] = take(M * m.dims[l + 1]);
    w.a[l] = take(R * m.dims[l + 1]);
    w.d[l] = take(R * m.dims[l + 1]);
    w.r[l] = take(R * m.dims[l + 1]);
  }
  w.out = take(M);
  w.dz0 = take(M * wmax);
  w.dz1 = take(M * wmax);
  w.g = take(R * m.dims[0]);
  w.u = take(R * wmax);
  w.v = take(R * wmax);
  w.ones = take(M);
  w.part = take(kDiscMaxSlices * maxw);
  w.colpart = take((int64_t)kDiscMaxSlices * wmax);
  if (ws) *ws = w;
  return off;
}

// launches one product; cuts the k range when the output alone would leave most of the chip idle
// colsum / colpart (wide row reductions only): colsum (M) += sum_k A(k, i) from the same pass, colpart its (slices, M) partials
template <bool A_KC, bool B_KC>
static void sgemm(hipStream_t s, int64_t M, int N, int64_t K, const float* A, int64_t lda, const float* B, int64_t ldb, float* C,
                  int64_t ldc, const float* bias, int act, bool accumulate, float* part, float* colsum, float* colpart) {
  if (M <= 0 || N <= 0 || K <= 0) return;  // every caller with an empty sum adds into its output
  if (!A_KC && !B_KC && M == 1 && N >= 128 && !bias && act == KS_ACT_NONE) {
    // one output row: the same numbers as the (N, 1) product with the operands exchanged, which takes the wide path below
    sgemm<false, false>(s, N, 1, K, B, ldb, A, lda, C, 1, nullptr, KS_ACT_NONE, accumulate, part);
    return;
  }
  if (!A_KC && !B_KC && M >= 128 && !bias && act == KS_ACT_NONE) {  // gradients of wide layers: long reductions over the rows
    const int vec_a = lda % 4 == 0 && ((uintptr_t)A & 15) == 0, vec_b = ldb % 4 == 0 && ((uintptr_t)B & 15) == 0;
    const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
    int slices = 1;
    if (part && K >= 2048) {
      slices = (int)((512 + tiles - 1) / tiles);
      if (slices > kDiscMaxSlices) slices = kDiscMaxSlices;
      if ((int64_t)slices * 256 > K) slices = (int)(K / 256);
    }
    int kslice = (int)((K + slices - 1) / slices);
    kslice = (kslice + 15) / 16 * 16;
    slices = (int)((K + kslice - 1) / kslice);
    hipLaunchKernelGGL(sgemm_tn128_kernel, dim3((unsigned)((N + 127) / 128), (unsigned)((M + 127) / 128), (unsigned)slices), dim3(256), 0, s,
                       (int)M, N, (int)K, A, lda, B, ldb, slices > 1 ? part : C, ldc, kslice, accumulate ? 1 : 0, vec_a, vec_b,
                       colsum ? (slices > 1 ? colpart : colsum) : (float*)nullptr);
    if (slices > 1) {
      const int64_t n = M * N;
      hipLaunchKernelGGL(sum_slices_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (int)M, N, slices, part, C, ldc, accumulate ? 1 : 0);
      if (colsum)
        hipLaunchKernelGGL(sum_slices_kernel, dim3((unsigned)((M + 255) / 256)), dim3(256), 0, s, (int)M, 1, slices, colpart, colsum, (int64_t)1,
                           accumulate ? 1 : 0);
    }
    return;
  }
  const int64_t tiles = ((M + 63) / 64) * ((N + 63) / 64);
  int slices = 1;
  if (part && tiles < 128 && K >= 2048) {
    slices = (int)((K + 511) / 512);
    const int64_t want = (512 + tiles - 1) / tiles;
    if (slices > want) slices = (int)want;
    if (slices > kDiscMaxSlices) slices = kDiscMaxSlices;
  }
  int kslice = (int)((K + slices - 1) / slices);
  kslice = (kslice + 15) / 16 * 16;
  slices = (int)((K + kslice - 1) / kslice);
  if (slices < 1) slices = 1;
  hipLaunchKernelGGL((sgemm_kernel<A_KC, B_KC>), dim3((unsigned)((N + 63) / 64), (unsigned)((M + 63) / 64), (unsigned)slices), dim3(256), 0, s,
                     (int)M, N, (int)K, A, lda, B, ldb, slices > 1 ? part : C, ldc, kslice, bias, act, accumulate ? 1 : 0);
  if (slices > 1) {
    const int64_t n = M * N;
    hipLaunchKernelGGL(sum_slices_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (int)M, N, slices, part, C, ldc, accumulate ? 1 : 0);
  }
}

extern "C" int64_t ks_mlp_disc_workspace_bytes(const KsMlp* h, int64_t n_real, int64_t n_sim) {
  if (!h || n_real < 0 || n_sim < 0) return 0;
  return carve_disc(h->m, n_real, n_real + n_sim, nullptr, nullptr) + 256;
}

extern "C" int ks_mlp_disc_loss_grad(KsMlp* h, ks_stream_t stream, int64_t n_real, const float* real, int64_t n_sim, const float* sim,
                                     float grad_penalty_coef, int64_t n_motions, float* losses, void* workspace) {
  if (!h || !h->m.train) return fail(KS_EINVAL, "ks_mlp_disc_loss_grad: call ks_mlp_train_init first");
  DevMlp& m = h->m;
  const int L = m.n_layers, act = m.activation;
  const int64_t R = n_real, M = n_real + n_sim;
  if (m.dims[L] != 1) return fail(KS_EINVAL, "ks_mlp_disc_loss_grad: the discriminator must have one output, not %d", m.dims[L]);
  if (act == KS_ACT_GELU) return fail(KS_EINVAL, "ks_mlp_disc_loss_grad: GELU is not supported here (ELU, ReLU, tanh or none)");
  if (n_real < 0 || n_sim < 0 || M <= 0 || (n_real > 0 && !real) || (n_sim > 0 && !sim) || !losses || !workspace)
    return fail(KS_EINVAL, "ks_mlp_disc_loss_grad: bad argument");
  if (M > 4000000) return fail(KS_ELIMIT, "ks_mlp_disc_loss_grad: %lld rows exceed the limit of 4000000", (long long)M);
  const bool penalty = grad_penalty_coef != 0.f && R > 0;
  if (penalty && (n_motions <= 0 || n_real % n_motions != 0))
    return fail(KS_EINVAL, "ks_mlp_disc_loss_grad: %lld real frames do not divide into %lld motions", (long long)n_real, (long long)n_motions);
  hipStream_t s = (hipStream_t)stream;
  DiscWs ws;
  carve_disc(m, R, M, (char*)workspace, &ws);
  auto blocks = [](int64_t n) { return dim3((unsigned)((n + 255) / 256)); };
  for (int l = 0; l < L; ++l) {  // everything below adds into the gradient buffers
    const int64_t nw = (int64_t)m.npad[l] * m.kpad[l];
    hipLaunchKernelGGL(fill_kernel, blocks(nw), dim3(256), 0, s, nw, 0.f, m.gW[l]);
    hipLaunchKernelGGL(fill_kernel, blocks(m.npad[l]), dim3(256), 0, s, (int64_t)m.npad[l], 0.f, m.gb[l]);
  }
  hipLaunchKernelGGL(fill_kernel, blocks(M), dim3(256), 0, s, M, 1.f, ws.ones);
  hipLaunchKernelGGL(fill_kernel, dim3(1), dim3(256), 0, s, (int64_t)3, 0.f, losses);

  // forward over the real rows, then the simulated ones
  for (int l = 0; l < L; ++l) {
    const bool last = l == L - 1;
    float* outp = last ? ws.out : ws.y[l];
    const int n = m.dims[l + 1], k = m.dims[l];
    const int a_l = last ? KS_ACT_NONE : act;
    if (l == 0) {
      sgemm<true, true>(s, R, n, k, real, k, m.mW[0], m.kpad[0], outp, n, m.mb[0], a_l, false, nullptr);
      sgemm<true, true>(s, n_sim, n, k, sim, k, m.mW[0], m.kpad[0], outp + R * n, n, m.mb[0], a_l, false, nullptr);
    } else {
      sgemm<true, true>(s, M, n, k, ws.y[l - 1], k, m.mW[l], m.kpad[l], outp, n, m.mb[l], a_l, false, nullptr);
    }
  }
  hipLaunchKernelGGL(disc_signal_kernel, dim3(1), dim3(1024), 0, s, R, M, ws.out, ws.dz0, losses);

  if (penalty) {
    // input gradient on the real rows: d_L = 1, down to g = d_1 W_1
    const float* dnext = ws.ones;
    for (int l = L - 1; l >= 1; --l) {  // hidden layer l (its output is y[l - 1])
      const int n = m.dims[l], k = m.dims[l + 1];
      sgemm<true, false>(s, R, n, k, dnext, k, m.mW[l], m.kpad[l], ws.a[l - 1], n, nullptr, KS_ACT_NONE, false, nullptr);
      hipLaunchKernelGGL(disc_delta_kernel, blocks(R * n), dim3(256), 0, s, R * n, act, ws.y[l - 1], ws.a[l - 1], ws.d[l - 1]);
      dnext = ws.d[l - 1];
    }
    sgemm<true, false>(s, R, m.dims[0], m.dims[1], dnext, m.dims[1], m.mW[0], m.kpad[0], ws.g, m.dims[0], nullptr, KS_ACT_NONE, false, nullptr);
    hipLaunchKernelGGL(disc_penalty_kernel, dim3(1), dim3(1024), 0, s, R * m.dims[0], grad_penalty_coef, 1.f / (float)n_motions, ws.g,
                       losses + 2);
    // the sweep back through that computation, first layer to last
    const float* prev = ws.g;
    float *u = ws.u, *v = ws.v;
    for (int l = 1; l <= L; ++l) {
      const int n = m.dims[l], k = m.dims[l - 1];
      const float* dl = l == L ? ws.ones : ws.d[l - 1];
      sgemm<false, false>(s, n, k, R, dl, n, prev, k, m.gW[l - 1], m.kpad[l - 1], nullptr, KS_ACT_NONE, true, ws.part);
      if (l == L) break;
      sgemm<true, true>(s, R, n, k, prev, k, m.mW[l - 1], m.kpad[l - 1], u, n, nullptr, KS_ACT_NONE, false, nullptr);
      hipLaunchKernelGGL(disc_tangent_kernel, blocks(R * n), dim3(256), 0, s, R * n, act, ws.y[l - 1], ws.a[l - 1], u, v, ws.r[l - 1]);
      prev = v;  // the next layer's products read v and write u; only then does its elementwise pass overwrite v
    }
  }

  // ordinary backward pass of the squared-error terms over all rows, with r_l added on the real rows
  float *dz = ws.dz0, *dnx = ws.dz1;
  for (int l = L; l >= 1; --l) {
    const int n = m.dims[l], k = m.dims[l - 1];
    // wide layers: the bias gradient (the column sums of dz) rides on the weight gradient's pass over dz
    const bool with_bias = n >= 128;
    float* gb = with_bias ? m.gb[l - 1] : nullptr;
    if (l == 1) {
      sgemm<false, false>(s, n, k, R, dz, n, real, k, m.gW[0], m.kpad[0], nullptr, KS_ACT_NONE, true, ws.part, gb, ws.colpart);
      sgemm<false, false>(s, n, k, n_sim, dz + R * n, n, sim, k, m.gW[0], m.kpad[0], nullptr, KS_ACT_NONE, true, ws.part, gb, ws.colpart);
    } else {
      sgemm<false, false>(s, n, k, M, dz, n, ws.y[l - 2], k, m.gW[l - 1], m.kpad[l - 1], nullptr, KS_ACT_NONE, true, ws.part, gb, ws.colpart);
    }
    if (!with_bias) sgemm<false, false>(s, n, 1, M, dz, n, ws.ones, 1, m.gb[l - 1], 1, nullptr, KS_ACT_NONE, true, ws.part);
    if (l == 1) break;
    sgemm<true, false>(s, M, k, n, dz, n, m.mW[l - 1], m.kpad[l - 1], dnx, k, nullptr, KS_ACT_NONE, false, nullptr);
    hipLaunchKernelGGL(disc_dz_kernel, blocks(M * k), dim3(256), 0, s, M * k, penalty ? R * k : (int64_t)0, act, ws.y[l - 2], ws.r[l - 2], dnx);
    float* tmp = dz; dz = dnx; dnx = tmp;
  }
  return check_launch("ks_mlp_disc_loss_grad");
}

// strided copy of the meaningful (out, in) block of a padded (npad, kpad) matrix
__global__ __launch_bounds__(256) void unpad_kernel(int rows, int cols, int ld, const float* __restrict__ src, float* __restrict__ dst) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)rows * cols) return;
  const int r = (int)(idx / cols), c = (int)(idx - (int64_t)r * cols);
  dst[idx] = src[(int64_t)r * ld + c];
}

extern "C" int ks_mlp_get_params(const KsMlp* h, ks_stream_t stream, int32_t l, float* weight, float* bias, int32_t gradients) {
  if (!h || !h->m.train) return fail(KS_EINVAL, "ks_mlp_get_params: call ks_mlp_train_init first");
  const DevMlp& m = h->m;
  if (l < 0 || l >= m.n_layers) return fail(KS_EINVAL, "ks_mlp_get_params: layer %d out of range", l);
  const int out = m.dims[l + 1], in = m.dims[l];
  if (weight)
    hipLaunchKernelGGL(unpad_kernel, dim3((unsigned)(((int64_t)out * in + 255) / 256)), dim3(256), 0, (hipStream_t)stream, out, in,
                       m.kpad[l], gradients ? m.gW[l] : m.mW[l], weight);
  if (bias)
    hipLaunchKernelGGL(unpad_kernel, dim3((unsigned)((out + 255) / 256)), dim3(256), 0, (hipStream_t)stream, 1, out, out,
                       gradients ? m.gb[l] : m.mb[l], bias);
  return check_launch("ks_mlp_get_params");
}
