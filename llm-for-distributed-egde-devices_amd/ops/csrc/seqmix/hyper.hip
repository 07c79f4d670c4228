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
// C = columns per thread and pass (4 with 16-byte stream accesses when W % 4 == 0, else 1).
// NEXT: the next sublayer's read and norm in the same pass (one workgroup per token, dynamic LDS u [W]):
// h[t] = u / sqrt(mean(u^2) + eps) * w2 with u = sum_r in2[r] X_new[t, r] (in2 null: the plain sum).
template <typename T, int C, bool NEXT>
__global__ void __launch_bounds__(NT) hyper_update_kernel(float* __restrict__ X, const float* __restrict__ mix,
                                                          const float* __restrict__ out_w, const T* __restrict__ y,
                                                          const T* __restrict__ parts, const float* __restrict__ pw, int K,
                                                          int S, int W, const float* __restrict__ in2,
                                                          const float* __restrict__ w2, T* __restrict__ h, float eps) {
  extern __shared__ __attribute__((aligned(16))) float u_s[];
  __shared__ float m_s[MAXS * MAXS + MAXS];
  __shared__ float red[NT / 64];
  const size_t t = blockIdx.x;
  float a2[MAXS];
  float ss = 0.f;
#pragma unroll
  for (int s = 0; s < MAXS; ++s) a2[s] = (NEXT && s < S) ? (in2 ? in2[s] : 1.f) : 0.f;
  if (mix) {
    for (int e = threadIdx.x; e < S * S + S; e += NT) m_s[e] = e < S * S ? mix[e] : out_w[e - S * S];
    __syncthreads();
  }
  float* xr = X + t * S * W;
  auto ld4 = [&](const T* p, float* f) {                     // C consecutive activations
    if constexpr (C == 1) f[0] = ldf<T>(p);
    else if constexpr (sizeof(T) == 4) {
      const float4 a = *reinterpret_cast<const float4*>(p);
      f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w;
    } else {
      const uint2 a = *reinterpret_cast<const uint2*>(p);
      f[0] = __uint_as_float(a.x << 16); f[1] = __uint_as_float(a.x & 0xffff0000u);
      f[2] = __uint_as_float(a.y << 16); f[3] = __uint_as_float(a.y & 0xffff0000u);
    }
  };
  for (int c = (blockIdx.y * NT + threadIdx.x) * C; c < W; c += gridDim.y * NT * C) {
    float v[C];
#pragma unroll
    for (int i = 0; i < C; ++i) v[i] = 0.f;
    if (y) ld4(y + t * W + c, v);
    for (int k = 0; k < K; ++k) {
      float p[C];
      ld4(parts + (t * K + k) * W + c, p);
      const float wk = pw ? pw[t * K + k] : 1.f;
#pragma unroll
      for (int i = 0; i < C; ++i) v[i] += wk * p[i];
    }
    float xs[MAXS][C];
#pragma unroll
    for (int s = 0; s < MAXS; ++s) {
      if (s < S) {
        if constexpr (C == 4) {
          const float4 a = *reinterpret_cast<const float4*>(xr + (size_t)s * W + c);
          xs[s][0] = a.x; xs[s][1] = a.y; xs[s][2] = a.z; xs[s][3] = a.w;
        } else {
          xs[s][0] = xr[(size_t)s * W + c];
        }
      } else {
#pragma unroll
        for (int i = 0; i < C; ++i) xs[s][i] = 0.f;
      }
    }
    float u[C];
#pragma unroll
    for (int i = 0; i < C; ++i) u[i] = 0.f;
#pragma unroll
    for (int r = 0; r < MAXS; ++r) {
      if (r < S) {
        float n[C];
#pragma unroll
        for (int i = 0; i < C; ++i) {
          if (mix) {
            float a = 0.f;
#pragma unroll
            for (int s = 0; s < MAXS; ++s)
              if (s < S) a += m_s[s * S + r] * xs[s][i];
            n[i] = a + m_s[S * S + r] * v[i];
          } else {
            n[i] = xs[r][i] + v[i];
          }
          if constexpr (NEXT) u[i] += a2[r] * n[i];
        }
        if constexpr (C == 4) *reinterpret_cast<float4*>(xr + (size_t)r * W + c) = make_float4(n[0], n[1], n[2], n[3]);
        else xr[(size_t)r * W + c] = n[0];
      }
    }
    if constexpr (NEXT) {
#pragma unroll
      for (int i = 0; i < C; ++i) { u_s[c + i] = u[i]; ss += u[i] * u[i]; }
    }
  }
  if constexpr (NEXT) {
    const float r = 1.f / sqrtf(block_sum<NT>(ss, red) / (float)W + eps);
    for (int c = threadIdx.x; c < W; c += NT) stf<T>(h + t * W + c, u_s[c] * r * w2[c]);
  }
}

// z [rows, F] -> a N(z) + b N(z^2) + c N(z^3) + e, N(v) = v / sqrt(mean(v^2) + eps) over the row.  LDS: z [F] fp32.
// VEC (F, ld % 8 == 0, 32-byte aligned rows): 8 coordinates per thread and pass.
template <typename T, bool VEC>
__global__ void __launch_bounds__(NT) poly_norm_kernel(const T* __restrict__ z, int ld, const float* __restrict__ coef,
                                                       T* __restrict__ y, int F, float eps) {
  extern __shared__ __attribute__((aligned(16))) float z_s[];
  __shared__ float red[NT / 64];
  const size_t t = blockIdx.x;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  if constexpr (VEC) {
    for (int c = threadIdx.x * 8; c < F; c += NT * 8) {
      float v[8];
      load8<T>(z + t * ld + c, v);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float v2 = v[i] * v[i];
        z_s[c + i] = v[i];
        s2 += v2;
        s4 += v2 * v2;
        s6 += v2 * v2 * v2;
      }
    }
  } else {
    for (int c = threadIdx.x; c < F; c += NT) {
      const float v = ldf<T>(z + t * ld + c), v2 = v * v;
      z_s[c] = v;
      s2 += v2;
      s4 += v2 * v2;
      s6 += v2 * v2 * v2;
    }
  }
  const float inv = 1.f / (float)F;
  const float r1 = coef[0] / sqrtf(block_sum<NT>(s2, red) * inv + eps);
  const float r2 = coef[1] / sqrtf(block_sum<NT>(s4, red) * inv + eps);
  const float r3 = coef[2] / sqrtf(block_sum<NT>(s6, red) * inv + eps);
  const float e = coef[3];
  if constexpr (VEC) {
    for (int c = threadIdx.x * 8; c < F; c += NT * 8) {      // every thread reads back the chunk it wrote
      float o[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float v = z_s[c + i];
        o[i] = v * r1 + v * v * r2 + v * v * v * r3 + e;
      }
      store8<T>(y + t * F + c, o);
    }
  } else {
    for (int c = threadIdx.x; c < F; c += NT) {
      const float v = z_s[c];
      stf<T>(y + t * F + c, v * r1 + v * v * r2 + v * v * v * r3 + e);
    }
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

// The same with 8 coordinates per thread (D, Dv, ld % 8 == 0, 32-byte aligned rows): a head (q, k or v) is held
// by LPH = max(D, Dv) / 8 neighbouring threads, NT / LPH heads per workgroup (blockIdx.y walks the rest); one 16- /
// 32-byte load per thread, the head's sum of squares from the threads' shares through LDS, then norm, turn (a
// rotation pair never leaves its chunk), temperature and one 16- / 32-byte store.
template <typename T>
__global__ void __launch_bounds__(NT) qk_norm_rope_write_vec_kernel(
    const T* __restrict__ proj, int ld, const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
    const int* __restrict__ seq_slot, const int* __restrict__ ptab, int ptab_ld, const float* __restrict__ qw,
    const float* __restrict__ kw, float eps, const float* __restrict__ cs, const float* __restrict__ vcs,
    const float* __restrict__ temp, T* __restrict__ q_out, T* __restrict__ kp, T* __restrict__ vp, int H, int G, int D,
    int Dv, int rot, int page, int LPH) {
  __shared__ float part_s[NT];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int unit = blockIdx.y * (NT / LPH) + tid / LPH, d = (tid % LPH) * 8;
  const bool isv = unit >= H + G, isq = unit < H;
  const int size = isv ? Dv : D;
  const bool live = tid / LPH < NT / LPH && unit < H + 2 * G && d < size;
  const float* w = isv ? nullptr : (isq ? qw : kw);
  float v[8];
  float ss = 0.f;
  if (live) {
    load8<T>(proj + (size_t)t * ld + (isv ? (size_t)(H + G) * D + (size_t)(unit - H - G) * Dv : (size_t)unit * D) + d, v);
    if (w) {
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += v[i] * v[i];
    }
  }
  part_s[tid] = ss;
  __syncthreads();
  if (!live) return;
  const int pos = tok_pos[t], slot = seq_slot[tok_seq[t]];
  const size_t prow = (size_t)ptab[(size_t)slot * ptab_ld + pos / page] * page + pos % page;
  if (w) {
    float tot = 0.f;
    const int first = (tid / LPH) * LPH;
    for (int i = 0; i < D / 8; ++i) tot += part_s[first + i];
    const float r = 1.f / sqrtf(tot / (float)D + eps);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] *= r * w[d + i];
  }
  const float* c = isv ? (vcs ? vcs + (size_t)pos * Dv : nullptr) : ((cs && d < rot) ? cs + (size_t)pos * rot : nullptr);
  if (c) {
    const int lim = isv ? Dv : rot;
#pragma unroll
    for (int i = 0; i < 8; i += 2) {
      if (d + i < lim) {
        const float co = c[d + i], si = c[d + i + 1], a = v[i], b = v[i + 1];
        v[i] = a * co - b * si;
        v[i + 1] = b * co + a * si;
      }
    }
  }
  if (isq && temp) {
    const float mul = temp[unit];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] *= mul;
  }
  T* dst = isq ? q_out + ((size_t)t * H + unit) * D : isv ? vp + (prow * G + (unit - H - G)) * Dv : kp + (prow * G + (unit - H)) * D;
  store8<T>(dst + d, v);
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

// w2 given: the next sublayer's input h [rows, W] = norm(sum_r in2[r] X_new[:, r]) w2 is written in the same pass
int edge_sm_hyper_update(float* X, const float* mix, const float* out_w, const void* y, const void* parts, const float* pw,
                         int K, int rows, int S, int W, const float* in2, const float* w2, void* h, float eps, int f32,
                         hipStream_t st) {
  if (rows == 0) return 0;
  if (S < 1 || S > MAXS || (!y && K == 0) || (mix && !out_w) || (w2 && !h)) return -2;
  const bool vec = W % 4 == 0 && (((uintptr_t)X | (uintptr_t)y | (uintptr_t)parts) & 15) == 0;
  if (w2) {
    if ((size_t)W * 4 > 60 * 1024) return -3;
    if (vec)
      SM_T(f32, hipLaunchKernelGGL((hyper_update_kernel<T, 4, true>), dim3(rows), dim3(NT), (size_t)W * 4, st, X, mix, out_w,
                                   (const T*)y, (const T*)parts, pw, K, S, W, in2, w2, (T*)h, eps));
    else
      SM_T(f32, hipLaunchKernelGGL((hyper_update_kernel<T, 1, true>), dim3(rows), dim3(NT), (size_t)W * 4, st, X, mix, out_w,
                                   (const T*)y, (const T*)parts, pw, K, S, W, in2, w2, (T*)h, eps));
    return (int)hipGetLastError();
  }
  const int per = NT * (vec ? 4 : 1);
  const int gy = rows >= 1024 ? 1 : (W + per - 1) / per < 8 ? (W + per - 1) / per : 8;
  if (vec)
    SM_T(f32, hipLaunchKernelGGL((hyper_update_kernel<T, 4, false>), dim3(rows, gy), dim3(NT), 0, st, X, mix, out_w,
                                 (const T*)y, (const T*)parts, pw, K, S, W, nullptr, nullptr, (T*)nullptr, 0.f));
  else
    SM_T(f32, hipLaunchKernelGGL((hyper_update_kernel<T, 1, false>), dim3(rows, gy), dim3(NT), 0, st, X, mix, out_w,
                                 (const T*)y, (const T*)parts, pw, K, S, W, nullptr, nullptr, (T*)nullptr, 0.f));
  return (int)hipGetLastError();
}

int edge_sm_poly_norm(const void* z, int ld, const float* coef, void* y, int rows, int F, float eps, int f32,
                      hipStream_t st) {
  if (rows == 0 || F == 0) return 0;
  if ((size_t)F * 4 > 60 * 1024) return -3;
  if (F % 8 == 0 && ld % 8 == 0 && (((uintptr_t)z | (uintptr_t)y) & 31) == 0)
    SM_T(f32, hipLaunchKernelGGL((poly_norm_kernel<T, true>), dim3(rows), dim3(NT), (size_t)F * 4, st, (const T*)z, ld, coef,
                                 (T*)y, F, eps));
  else
    SM_T(f32, hipLaunchKernelGGL((poly_norm_kernel<T, false>), dim3(rows), dim3(NT), (size_t)F * 4, st, (const T*)z, ld, coef,
                                 (T*)y, F, eps));
  return (int)hipGetLastError();
}

int edge_sm_qk_norm_rope_write(const void* proj, int ld, const int* tok_seq, const int* tok_pos, const int* seq_slot,
                               const int* ptab, int ptab_ld, const float* qw, const float* kw, float eps, const float* cs,
                               const float* vcs, const float* temp, void* q_out, void* kp, void* vp, int rows, int H, int G,
                               int D, int Dv, int rot, int page, int f32, hipStream_t st) {
  if (rows == 0) return 0;
  if (rot % 2 || rot > D || (rot > 0 && !cs) || (vcs && Dv % 2)) return -2;
  const int lph = (D > Dv ? D : Dv) / 8;                      // threads per head
  if (D % 8 == 0 && Dv % 8 == 0 && ld % 8 == 0 && lph >= 1 && lph <= NT &&
      (((uintptr_t)proj | (uintptr_t)q_out | (uintptr_t)kp | (uintptr_t)vp) & 31) == 0)
    SM_T(f32, hipLaunchKernelGGL(qk_norm_rope_write_vec_kernel<T>, dim3(rows, (H + 2 * G + NT / lph - 1) / (NT / lph)), dim3(NT),
                                 0, st, (const T*)proj, ld, tok_seq, tok_pos, seq_slot, ptab, ptab_ld, qw, kw, eps,
                                 rot > 0 ? cs : nullptr, vcs, temp, (T*)q_out, (T*)kp, (T*)vp, H, G, D, Dv, rot, page, lph));
  else
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
