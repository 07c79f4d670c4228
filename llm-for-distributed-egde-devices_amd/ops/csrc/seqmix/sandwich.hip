// Kernels of the layer-spec layers that carry a norm on both sides of every sublayer (ops/seqmix.py):
// the RMS norm in groups of fp32 rows (a sublayer's input), the same norm with a multiplier added into
// the fp32 stream (a sublayer's output, with a mixture's expert outputs summed in the same pass), the
// silu gated-linear activation of rows whose input carried a router weight, and what a gated delta rule
// with one decay per head reads (unit-length q / k, decays, beta).
//
// Storage is fp32 or bf16 (template T); the norms, the router weights, decays and beta are fp32 in both.
#include "common.h"
#include "seqmix/seqmix_common.h"

namespace {

// Sum of squares of each of `groups` equal consecutive parts of the row in row_s [W]: a part is cut into
// `split` strided shares (4 / groups of them while there are fewer parts than waves), one wave per share;
// the shares of a part are added in a fixed order.  Leaves 1 / sqrt(mean + eps) per part in inv_s [groups].
__device__ __forceinline__ void group_inv_rms(const float* row_s, float* part_s, float* inv_s, int W, int groups,
                                              float eps) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, gs = W / groups;
  const int split = groups >= NT / 64 ? 1 : (NT / 64) / groups;
  for (int u = wave; u < groups * split; u += NT / 64) {
    const int g = u / split, sh = u % split;
    float ss = 0.f;
    for (int c = sh * 64 + lane; c < gs; c += split * 64) { const float v = row_s[g * gs + c]; ss += v * v; }
    ss = wave_sum(ss);
    if (lane == 0) part_s[u] = ss;
  }
  __syncthreads();
  for (int g = tid; g < groups; g += NT) {
    float ss = 0.f;
    for (int sh = 0; sh < split; ++sh) ss += part_s[g * split + sh];
    inv_s[g] = 1.f / sqrtf(ss / (float)gs + eps);
  }
  __syncthreads();
}

// LDS: row [W] | shares [max(groups, NT / 64)] | inverse rms [groups].  VEC (W % 8 == 0): 8 coordinates per
// thread and pass, 16- / 32-byte accesses.
template <typename T, bool VEC>
__global__ void __launch_bounds__(NT) group_norm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                        T* __restrict__ y, int W, int groups, float eps) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  float* row_s = smem;
  float* part_s = row_s + W;
  float* inv_s = part_s + max(groups, NT / 64);
  const size_t t = blockIdx.x;
  const int gs = W / groups;
  if constexpr (VEC) {
    for (int c = threadIdx.x * 8; c < W; c += NT * 8) {
      float v[8];
      load8<float>(x + t * W + c, v);
      store8<float>(row_s + c, v);
    }
  } else {
    for (int c = threadIdx.x; c < W; c += NT) row_s[c] = x[t * W + c];
  }
  __syncthreads();
  group_inv_rms(row_s, part_s, inv_s, W, groups, eps);
  if constexpr (VEC) {
    for (int c = threadIdx.x * 8; c < W; c += NT * 8) {
      float v[8], wv[8];
      load8<float>(row_s + c, v);
      load8<float>(w + c, wv);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] *= inv_s[(c + e) / gs] * wv[e];
      store8<T>(y + t * W + c, v);
    }
  } else {
    for (int c = threadIdx.x; c < W; c += NT) stf<T>(y + t * W + c, row_s[c] * inv_s[c / gs] * w[c]);
  }
}

// x += mult * group-norm(y + sum_k pw[k] parts[k]) w   (y null: the parts alone; pw null: ones)
template <typename T, bool VEC>
__global__ void __launch_bounds__(NT) group_norm_residual_kernel(float* __restrict__ x, const T* __restrict__ y,
                                                                 const T* __restrict__ parts, const float* __restrict__ pw,
                                                                 int K, const float* __restrict__ w, int W, int groups,
                                                                 float eps, float mult) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  float* row_s = smem;
  float* part_s = row_s + W;
  float* inv_s = part_s + max(groups, NT / 64);
  const size_t t = blockIdx.x;
  const int gs = W / groups;
  if constexpr (VEC) {
    for (int c = threadIdx.x * 8; c < W; c += NT * 8) {
      float v[8];
      if (y) load8<T>(y + t * W + c, v);
      else {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = 0.f;
      }
      for (int k = 0; k < K; ++k) {
        float p[8];
        load8<T>(parts + (t * K + k) * W + c, p);
        const float pk = pw ? pw[t * K + k] : 1.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += pw ? pk * p[e] : p[e];
      }
      store8<float>(row_s + c, v);
    }
  } else {
    for (int c = threadIdx.x; c < W; c += NT) {
      float v = y ? ldf<T>(y + t * W + c) : 0.f;
      for (int k = 0; k < K; ++k) {
        const float p = ldf<T>(parts + (t * K + k) * W + c);
        v += pw ? pw[t * K + k] * p : p;
      }
      row_s[c] = v;
    }
  }
  __syncthreads();
  group_inv_rms(row_s, part_s, inv_s, W, groups, eps);
  if constexpr (VEC) {
    for (int c = threadIdx.x * 8; c < W; c += NT * 8) {
      float v[8], wv[8], xv[8];
      load8<float>(row_s + c, v);
      load8<float>(w + c, wv);
      load8<float>(x + t * W + c, xv);
#pragma unroll
      for (int e = 0; e < 8; ++e) xv[e] += mult * (v[e] * inv_s[(c + e) / gs] * wv[e]);
      store8<float>(x + t * W + c, xv);
    }
  } else {
    for (int c = threadIdx.x; c < W; c += NT) x[t * W + c] += mult * (row_s[c] * inv_s[c / gs] * w[c]);
  }
}

// silu(rw gate) (rw up), rw = the row's router weight (null: 1); u row = gate [ff] | up [ff]
template <typename T>
__global__ void __launch_bounds__(NT) glu_silu_kernel(const T* __restrict__ u, int ld, T* __restrict__ y, int ff,
                                                      const float* __restrict__ row_w) {
  const size_t t = blockIdx.x;
  const float rw = row_w ? row_w[t] : 1.f;
  for (int c = blockIdx.y * NT + threadIdx.x; c < ff; c += NT * gridDim.y)
    stf<T>(y + t * ff + c, siluf_(rw * ldf<T>(u + t * ld + c)) * (rw * ldf<T>(u + t * ld + ff + c)));
}

// prep row = q [G, N] | k [G, N] | decay [H] | beta [H], all fp32; the decay and beta inputs are columns
// [a0, a0 + H) and [b0, b0 + H) of u
template <typename T>
__global__ void __launch_bounds__(NT) delta_prep_head_kernel(const T* __restrict__ qkv, int Cq, const T* __restrict__ u,
                                                             int ld, int b0, int a0, const float* __restrict__ dt_bias,
                                                             const float* __restrict__ A_log, float* __restrict__ prep,
                                                             int H, int G, int N) {
  const size_t t = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, GN = G * N;
  float* pr = prep + t * (2 * GN + 2 * H);
  const float qs = 1.f / sqrtf((float)N);
  for (int unit = wave; unit < 2 * G; unit += NT / 64) {     // unit = (q | k, kv head): one wave each
    const T* src = qkv + t * Cq + (size_t)unit * N;
    float ss = 0.f;
    for (int n = lane; n < N; n += 64) { const float v = ldf<T>(src + n); ss += v * v; }
    const float r = 1.f / sqrtf(wave_sum(ss) + 1e-6f) * (unit < G ? qs : 1.f);
    for (int n = lane; n < N; n += 64) pr[(size_t)unit * N + n] = ldf<T>(src + n) * r;
  }
  for (int e = tid; e < H; e += NT) {
    const float raw = ldf<T>(u + t * ld + a0 + e) + dt_bias[e];
    const float sp = raw > 20.f ? raw : log1pf(expf(raw));
    pr[2 * GN + e] = expf(-expf(A_log[e]) * sp);
    pr[2 * GN + H + e] = sigmoidf_(ldf<T>(u + t * ld + b0 + e));
  }
}

}  // namespace

#define SM_T(f32, ...)                                  \
  do {                                                  \
    if (f32) { using T = float; __VA_ARGS__; }          \
    else { using T = bf16_t; __VA_ARGS__; }             \
  } while (0)

extern "C" {

static size_t group_norm_lds(int W, int groups) {
  return sizeof(float) * ((size_t)W + (groups > NT / 64 ? groups : NT / 64) + groups);
}

int edge_sm_group_norm(const float* x, const float* w, void* y, int rows, int W, int groups, float eps, int f32,
                       hipStream_t st) {
  if (rows == 0) return 0;
  if (groups < 1 || W % groups) return -2;
  if (group_norm_lds(W, groups) > 64 * 1024) return -3;
  if (W % 8 == 0 && (((uintptr_t)x | (uintptr_t)w | (uintptr_t)y) & 31) == 0)
    SM_T(f32, hipLaunchKernelGGL((group_norm_kernel<T, true>), dim3(rows), dim3(NT), group_norm_lds(W, groups), st, x, w,
                                 (T*)y, W, groups, eps));
  else
    SM_T(f32, hipLaunchKernelGGL((group_norm_kernel<T, false>), dim3(rows), dim3(NT), group_norm_lds(W, groups), st, x, w,
                                 (T*)y, W, groups, eps));
  return (int)hipGetLastError();
}

int edge_sm_group_norm_residual(float* x, const void* y, const void* parts, const float* pw, int K, const float* w,
                                int rows, int W, int groups, float eps, float mult, int f32, hipStream_t st) {
  if (rows == 0) return 0;
  if (groups < 1 || W % groups || (!y && K == 0)) return -2;
  if (group_norm_lds(W, groups) > 64 * 1024) return -3;
  if (W % 8 == 0 && (((uintptr_t)x | (uintptr_t)w | (uintptr_t)y | (uintptr_t)parts) & 31) == 0)
    SM_T(f32, hipLaunchKernelGGL((group_norm_residual_kernel<T, true>), dim3(rows), dim3(NT), group_norm_lds(W, groups), st,
                                 x, (const T*)y, (const T*)parts, pw, K, w, W, groups, eps, mult));
  else
    SM_T(f32, hipLaunchKernelGGL((group_norm_residual_kernel<T, false>), dim3(rows), dim3(NT), group_norm_lds(W, groups),
                                 st, x, (const T*)y, (const T*)parts, pw, K, w, W, groups, eps, mult));
  return (int)hipGetLastError();
}

int edge_sm_glu_silu(const void* u, int ld, void* y, const float* row_w, int rows, int ff, int f32, hipStream_t st) {
  if (rows == 0 || ff == 0) return 0;
  const int gy = (ff + NT * 4 - 1) / (NT * 4);
  SM_T(f32, hipLaunchKernelGGL(glu_silu_kernel<T>, dim3(rows, gy), dim3(NT), 0, st, (const T*)u, ld, (T*)y, ff, row_w));
  return (int)hipGetLastError();
}

int edge_sm_delta_prep_head(const void* qkv, int Cq, const void* u, int ld, int b0, int a0, const float* dt_bias,
                            const float* A_log, float* prep, int rows, int H, int G, int N, int f32, hipStream_t st) {
  if (rows == 0) return 0;
  if (G <= 0 || H % G) return -2;
  SM_T(f32, hipLaunchKernelGGL(delta_prep_head_kernel<T>, dim3(rows), dim3(NT), 0, st, (const T*)qkv, Cq, (const T*)u, ld,
                               b0, a0, dt_bias, A_log, prep, H, G, N));
  return (int)hipGetLastError();
}

}  // extern "C"
