// Kernels of the layer-spec layers that keep several residual streams (ops/seqmix.py): the RMS norm of a
// weighted sum of the streams (a sublayer's input), the rebuild of every stream from all of them plus the
// sublayer's output (with a mixture's expert outputs summed in the same pass), the PolyNorm activation, and
// the two ends of gated attention with rotated values: per-head RMS norm + pair rotation + temperature on
// q / k with the page-table scatter of the keys and the rotated values, and the turn back of each head's
// output with the element-wise sigmoid gate.
//
// Storage is fp32 or bf16 (template T); the streams, norms, angles and stream weights are fp32 in both.
#include "common.h"
#include "seqmix/seqmix_common.h"

namespace {

constexpr int MAXS = 16;                                     // residual streams

// X [rows, S, W] fp32; u = sum_s in_w[s] X[t, s] (in_w null: the plain sum); y = u / sqrt(mean(u^2) + eps) * w.
// LDS: u [W].  VEC (W % 4 == 0): four coordinates per thread and pass.
template <typename T, bool VEC>
__global__ void __launch_bounds__(NT) hyper_read_norm_kernel(const float* __restrict__ X, const float* __restrict__ in_w,
                                                             const float* __restrict__ w, T* __restrict__ y, int S, int W,
                                                             float eps) {
  extern __shared__ __attribute__((aligned(16))) float u_s[];
  __shared__ float red[NT / 64];
  const size_t t = blockIdx.x;
  const float* xr = X + t * S * W;
  float a[MAXS];
#pragma unroll
  for (int s = 0; s < MAXS; ++s) a[s] = s < S ? (in_w ? in_w[s] : 1.f) : 0.f;
  float ss = 0.f;
  if constexpr (VEC) {
    for (int c = threadIdx.x * 4; c < W; c += NT * 4) {
      float4 u = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
      for (int s = 0; s < MAXS; ++s) {
        if (s < S) {
          const float4 v = *reinterpret_cast<const float4*>(xr + (size_t)s * W + c);
          u.x += a[s] * v.x; u.y += a[s] * v.y; u.z += a[s] * v.z; u.w += a[s] * v.w;
        }
      }
      *reinterpret_cast<float4*>(u_s + c) = u;
      ss += u.x * u.x + u.y * u.y + u.z * u.z + u.w * u.w;
    }
  } else {
    for (int c = threadIdx.x; c < W; c += NT) {
      float u = 0.f;
#pragma unroll
      for (int s = 0; s < MAXS; ++s)
        if (s < S) u += a[s] * xr[(size_t)s * W + c];
      u_s[c] = u;
      ss += u * u;
    }
  }
  const float r = 1.f / sqrtf(block_sum<NT>(ss, red) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += NT) stf<T>(y + t * W + c, u_s[c] * r * w[c]);
}

// X [rows, S, W] fp32 in place: X[t, r] <- sum_s mix[s, r] X[t, s] + out_w[r] v, v = y[t] + sum_k pw[t, k] parts[t, k]
// (fp32, k order; y / parts / pw may be null; pw null with parts: ones).  mix null: X[t, r] += v.
template <typename T>
__global__ void __launch_bounds__(NT) hyper_update_kernel(float* __restrict__ X, const float* __restrict__ mix,
                                                          const float* __restrict__ out_w, const T* __restrict__ y,
                                                          const T* __restrict__ parts, const float* __restrict__ pw, int K,
                                                          int S, int W) {
  __shared__ float m_s[MAXS * MAXS + MAXS];
  const size_t t = blockIdx.x;
  if (mix) {
    for (int e = threadIdx.x; e < S * S + S; e += NT) m_s[e] = e < S * S ? mix[e] : out_w[e - S * S];
    __syncthreads();
  }
  float* xr = X + t * S * W;
  for (int c = blockIdx.y * NT + threadIdx.x; c < W; c += gridDim.y * NT) {
    float v = y ? ldf<T>(y + t * W + c) : 0.f;
    for (int k = 0; k < K; ++k) {
      const float p = ldf<T>(parts + (t * K + k) * W + c);
      v += pw ? pw[t * K + k] * p : p;
    }
    float xs[MAXS];
#pragma unroll
    for (int s = 0; s < MAXS; ++s) xs[s] = s < S ? xr[(size_t)s * W + c] : 0.f;
#pragma unroll
    for (int r = 0; r < MAXS; ++r) {
      if (r < S) {
        float n;
        if (mix) {
          n = 0.f;
#pragma unroll
          for (int s = 0; s < MAXS; ++s)
            if (s < S) n += m_s[s * S + r] * xs[s];
          n += m_s[S * S + r] * v;
        } else {
          n = xs[r] + v;
        }
        xr[(size_t)r * W + c] = n;
      }
    }
  }
}

// z [rows, F] -> a N(z) + b N(z^2) + c N(z^3) + e, N(v) = v / sqrt(mean(v^2) + eps) over the row.  LDS: z [F] fp32.
template <typename T>
__global__ void __launch_bounds__(NT) poly_norm_kernel(const T* __restrict__ z, int ld, const float* __restrict__ coef,
                                                       T* __restrict__ y, int F, float eps) {
  extern __shared__ __attribute__((aligned(16))) float z_s[];
  __shared__ float red[NT / 64];
  const size_t t = blockIdx.x;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int c = threadIdx.x; c < F; c += NT) {
    const float v = ldf<T>(z + t * ld + c), v2 = v * v;
    z_s[c] = v;
    s2 += v2;
    s4 += v2 * v2;
    s6 += v2 * v2 * v2;
  }
  const float inv = 1.f / (float)F;
  const float r1 = coef[0] / sqrtf(block_sum<NT>(s2, red) * inv + eps);
  const float r2 = coef[1] / sqrtf(block_sum<NT>(s4, red) * inv + eps);
  const float r3 = coef[2] / sqrtf(block_sum<NT>(s6, red) * inv + eps);
  const float e = coef[3];
  for (int c = threadIdx.x; c < F; c += NT) {
    const float v = z_s[c];
    stf<T>(y + t * F + c, v * r1 + v * v * r2 + v * v * v * r3 + e);
  }
}

// proj row = q [H, D] | k [G, D] | v [G, Dv] | ...  One wave per head at a time.  q / k: divided by the head's
// root mean square times qw / kw (null: no norm), pairs (2i, 2i + 1), i < rot / 2, turned by cs[pos, i] =
// (cos, sin), q times temp[h] (null: 1).  v: pairs over all Dv turned by vcs[pos, m] (null: copied).  q goes
// to q_out [rows, H, D], k and v to the token's page row.
template <typename T>
__global__ void __launch_bounds__(NT) qk_norm_rope_write_kernel(
    const T* __restrict__ proj, int ld, const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
    const int* __restrict__ seq_slot, const int* __restrict__ ptab, int ptab_ld, const float* __restrict__ qw,
    const float* __restrict__ kw, float eps, const float* __restrict__ cs, const float* __restrict__ vcs,
    const float* __restrict__ temp, T* __restrict__ q_out, T* __restrict__ kp, T* __restrict__ vp, int H, int G, int D,
    int Dv, int rot, int page) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int pos = tok_pos[t], slot = seq_slot[tok_seq[t]];
  const size_t prow = (size_t)ptab[(size_t)slot * ptab_ld + pos / page] * page + pos % page;
  const T* row = proj + (size_t)t * ld;
  const float* c = cs ? cs + (size_t)pos * rot : nullptr;
  const float* cv = vcs ? vcs + (size_t)pos * Dv : nullptr;  // Dv / 2 pairs of (cos, sin)
  for (int unit = wave; unit < H + 2 * G; unit += NT / 64) {
    if (unit < H + G) {
      const bool isq = unit < H;
      const T* src = row + (size_t)unit * D;
      const float* w = isq ? qw : kw;
      float r = 1.f;
      if (w) {
        float ss = 0.f;
        for (int d = lane; d < D; d += 64) { const float v = ldf<T>(src + d); ss += v * v; }
        r = 1.f / sqrtf(wave_sum(ss) / (float)D + eps);
      }
      const float mul = (isq && temp) ? temp[unit] : 1.f;
      T* dst = isq ? q_out + ((size_t)t * H + unit) * D : kp + (prow * G + (unit - H)) * D;
      for (int d = lane; d < D; d += 64) {
        float v = ldf<T>(src + d) * r * (w ? w[d] : 1.f);
        if (c && d < rot) {
          const float o = ldf<T>(src + (d ^ 1)) * r * (w ? w[d ^ 1] : 1.f);
          const float co = c[d & ~1], si = c[(d & ~1) + 1];
          v = (d & 1) ? v * co + o * si : v * co - o * si;
        }
        stf<T>(dst + d, v * mul);
      }
    } else {
      const int g = unit - H - G;
      const T* src = row + (size_t)(H + G) * D + (size_t)g * Dv;
      T* dst = vp + (prow * G + g) * Dv;
      for (int d = lane; d < Dv; d += 64) {
        float v = ldf<T>(src + d);
        if (cv) {
          const float o = ldf<T>(src + (d ^ 1)), co = cv[d & ~1], si = cv[(d & ~1) + 1];
          v = (d & 1) ? v * co + o * si : v * co - o * si;
        }
        stf<T>(dst + d, v);
      }
    }
  }
}

// a [rows, H * Dv]: every head's pairs (2m, 2m + 1) turned by -pos (vcs[pos, m] = (cos, sin); null: as it is), then
// times sigmoid(gate[t, e]) (null: 1).
template <typename T>
__global__ void __launch_bounds__(NT) unrotate_gate_kernel(const T* __restrict__ a, const T* __restrict__ gate, int gate_ld,
                                                           const int* __restrict__ tok_pos, const float* __restrict__ vcs,
                                                           T* __restrict__ out, int HD, int Dv) {
  const size_t t = blockIdx.x;
  const float* cv = vcs ? vcs + (size_t)tok_pos[t] * Dv : nullptr;
  for (int e = blockIdx.y * NT + threadIdx.x; e < HD; e += gridDim.y * NT) {
    float v = ldf<T>(a + t * HD + e);
    if (cv) {
      const int d = e % Dv;
      const float o = ldf<T>(a + t * HD + (e ^ 1)), co = cv[d & ~1], si = cv[(d & ~1) + 1];
      v = (d & 1) ? v * co - o * si : v * co + o * si;
    }
    if (gate) v *= sigmoidf_(ldf<T>(gate + t * gate_ld + e));
    stf<T>(out + t * HD + e, v);
  }
}

}  // namespace

#define SM_T(f32, ...)                                  \
  do {                                                  \
    if (f32) { using T = float; __VA_ARGS__; }          \
    else { using T = bf16_t; __VA_ARGS__; }             \
  } while (0)

extern "C" {

int edge_sm_hyper_read_norm(const float* X, const float* in_w, const float* w, void* y, int rows, int S, int W, float eps,
                            int f32, hipStream_t st) {
  if (rows == 0) return 0;
  if (S < 1 || S > MAXS) return -2;
  if ((size_t)W * 4 > 60 * 1024) return -3;
  if (W % 4 == 0 && ((uintptr_t)X & 15) == 0)
    SM_T(f32, hipLaunchKernelGGL((hyper_read_norm_kernel<T, true>), dim3(rows), dim3(NT), (size_t)W * 4, st, X, in_w, w,
                                 (T*)y, S, W, eps));
  else
    SM_T(f32, hipLaunchKernelGGL((hyper_read_norm_kernel<T, false>), dim3(rows), dim3(NT), (size_t)W * 4, st, X, in_w, w,
                                 (T*)y, S, W, eps));
  return (int)hipGetLastError();
}

int edge_sm_hyper_update(float* X, const float* mix, const float* out_w, const void* y, const void* parts, const float* pw,
                         int K, int rows, int S, int W, int f32, hipStream_t st) {
  if (rows == 0) return 0;
  if (S < 1 || S > MAXS || (!y && K == 0) || (mix && !out_w)) return -2;
  const int gy = rows >= 1024 ? 1 : (W + NT - 1) / NT < 8 ? (W + NT - 1) / NT : 8;
  SM_T(f32, hipLaunchKernelGGL(hyper_update_kernel<T>, dim3(rows, gy), dim3(NT), 0, st, X, mix, out_w, (const T*)y,
                               (const T*)parts, pw, K, S, W));
  return (int)hipGetLastError();
}

int edge_sm_poly_norm(const void* z, int ld, const float* coef, void* y, int rows, int F, float eps, int f32,
                      hipStream_t st) {
  if (rows == 0 || F == 0) return 0;
  if ((size_t)F * 4 > 60 * 1024) return -3;
  SM_T(f32, hipLaunchKernelGGL(poly_norm_kernel<T>, dim3(rows), dim3(NT), (size_t)F * 4, st, (const T*)z, ld, coef, (T*)y,
                               F, eps));
  return (int)hipGetLastError();
}

int edge_sm_qk_norm_rope_write(const void* proj, int ld, const int* tok_seq, const int* tok_pos, const int* seq_slot,
                               const int* ptab, int ptab_ld, const float* qw, const float* kw, float eps, const float* cs,
                               const float* vcs, const float* temp, void* q_out, void* kp, void* vp, int rows, int H, int G,
                               int D, int Dv, int rot, int page, int f32, hipStream_t st) {
  if (rows == 0) return 0;
  if (rot % 2 || rot > D || (rot > 0 && !cs) || (vcs && Dv % 2)) return -2;
  SM_T(f32, hipLaunchKernelGGL(qk_norm_rope_write_kernel<T>, dim3(rows), dim3(NT), 0, st, (const T*)proj, ld, tok_seq,
                               tok_pos, seq_slot, ptab, ptab_ld, qw, kw, eps, rot > 0 ? cs : nullptr, vcs, temp, (T*)q_out,
                               (T*)kp, (T*)vp, H, G, D, Dv, rot, page));
  return (int)hipGetLastError();
}

int edge_sm_unrotate_gate(const void* a, const void* gate, int gate_ld, const int* tok_pos, const float* vcs, void* out,
                          int rows, int HD, int Dv, int f32, hipStream_t st) {
  if (rows == 0 || HD == 0) return 0;
  if (vcs && (Dv % 2 || HD % Dv)) return -2;
  const int gy = (HD + NT - 1) / NT < 8 ? (HD + NT - 1) / NT : 8;
  SM_T(f32, hipLaunchKernelGGL(unrotate_gate_kernel<T>, dim3(rows, gy), dim3(NT), 0, st, (const T*)a, (const T*)gate,
                               gate_ld, tok_pos, vcs, (T*)out, HD, Dv));
  return (int)hipGetLastError();
}

}  // extern "C"
