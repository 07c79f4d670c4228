// Kernels of the post-norm layer-spec layers (ops/seqmix.py): embedding with a hashed (previous token,
// token) row, the sublayers' input convolution over the fp32 stream, LayerNorm of fp32 rows and the
// LayerNorm + residual add on a sublayer's output (with a mixture's weighted expert sum), RMS norm of a
// column slice, the cached and the query side of latent attention (RMS norm, neighbour-pair rotation,
// page-table scatter), the gated delta rule (unit-length q / k, decays, the token-by-token recurrence
// over a [N, P] fp32 state per head, per-head norm with a sigmoid gate), the clamped gated-linear
// activation, and the mixture of experts' router and decode-sized expert products.
//
// Storage is fp32 or bf16 (template T); norms, scores' inputs that the design keeps in 32-bit, decays,
// the router and the recurrent state are fp32 in both.  A token is addressed by (sequence of the step,
// position); recurrent rows live per state slot and are taken as zero by a portion that starts at
// position 0, so a freed slot needs no clearing.
#include "common.h"
#include "seqmix/seqmix_common.h"

namespace {

// ---------------------------------------------------------------------------------- embedding
template <typename T>
__global__ void __launch_bounds__(NT) embed_bigram_kernel(const int64_t* __restrict__ ids, const T* __restrict__ table,
                                                          const T* __restrict__ bigram, const int64_t* __restrict__ prev_tok,
                                                          const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                                                          const int* __restrict__ seq_slot, const int* __restrict__ seq_start,
                                                          float* __restrict__ out, int W, int V, long buckets, long mul_prev,
                                                          long mul_cur) {
  const int t = blockIdx.x, s = tok_seq[t], pos = tok_pos[t];
  auto clampv = [V](int64_t id) { return id < 0 ? (int64_t)0 : (id >= V ? (int64_t)V - 1 : id); };
  const int64_t id = clampv(ids[t]);
  int64_t row = buckets;                                     // a sequence's first token
  if (pos > 0) {
    const int64_t prev = pos > seq_start[s] ? clampv(ids[t - 1]) : clampv(prev_tok[seq_slot[s]]);
    row = (prev * mul_prev + id * mul_cur) % buckets;
  }
  for (int c = threadIdx.x; c < W; c += NT)
    out[(size_t)t * W + c] = ldf<T>(table + (size_t)id * W + c) + ldf<T>(bigram + (size_t)row * W + c);
}

// runs after the embedding of the same step: every sequence's last token becomes its slot's previous token
__global__ void prev_token_kernel(const int64_t* __restrict__ ids, int64_t* __restrict__ prev_tok,
                                  const int* __restrict__ seq_slot, const int* __restrict__ seq_len,
                                  const int* __restrict__ seq_off, int n) {
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s < n) prev_tok[seq_slot[s]] = ids[seq_off[s] + seq_len[s] - 1];
}

// ---------------------------------------------------------------------------------- input convolution
// out = x + sum_k w[:, k] x_(pos - taps + 1 + k) over the fp32 stream; inputs before the portion come from
// the slot's tail (zeros before the sequence's start).  state_w: steps in which every sequence brings one
// token shift the tail in the same launch (the thread of (token, channel) is that channel's only reader).
// VEC: four channels per thread through 16-byte loads of the stream (W a multiple of 4)
template <typename T, bool VEC>
__global__ void __launch_bounds__(NT) canon_kernel(const float* __restrict__ x, int W, const float* __restrict__ w,
                                                   const float* state, const int* __restrict__ tok_seq,
                                                   const int* __restrict__ tok_pos, const int* __restrict__ seq_slot,
                                                   const int* __restrict__ seq_start, const int* __restrict__ seq_off,
                                                   T* __restrict__ out, int taps, float* state_w) {
  const int t = blockIdx.x, s = tok_seq[t], pos = tok_pos[t], start = seq_start[s], off = seq_off[s];
  const float* st = state + (size_t)seq_slot[s] * (taps - 1) * W;
  float* stw = state_w ? state_w + (size_t)seq_slot[s] * (taps - 1) * W : nullptr;
  if constexpr (VEC) {
    for (int c = (blockIdx.y * NT + threadIdx.x) * 4; c < W; c += NT * gridDim.y * 4) {
      float acc[4] = {0.f, 0.f, 0.f, 0.f};
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      for (int k = 0; k < taps; ++k) {
        const int p = pos - (taps - 1) + k;
        v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (p >= start) v = *reinterpret_cast<const float4*>(x + (size_t)(off + p - start) * W + c);
        else if (p >= 0) v = *reinterpret_cast<const float4*>(st + (size_t)(p - (start - (taps - 1))) * W + c);
        acc[0] += w[c * taps + k] * v.x;
        acc[1] += w[(c + 1) * taps + k] * v.y;
        acc[2] += w[(c + 2) * taps + k] * v.z;
        acc[3] += w[(c + 3) * taps + k] * v.w;
        if (stw && k >= 1) *reinterpret_cast<float4*>(stw + (size_t)(k - 1) * W + c) = v;
      }
      stf<T>(out + (size_t)t * W + c, v.x + acc[0]);
      stf<T>(out + (size_t)t * W + c + 1, v.y + acc[1]);
      stf<T>(out + (size_t)t * W + c + 2, v.z + acc[2]);
      stf<T>(out + (size_t)t * W + c + 3, v.w + acc[3]);
    }
    return;
  }
  for (int c = blockIdx.y * NT + threadIdx.x; c < W; c += NT * gridDim.y) {
    float acc = 0.f, cur = 0.f;
    for (int k = 0; k < taps; ++k) {
      const int p = pos - (taps - 1) + k;
      float v = 0.f;
      if (p >= start) v = x[(size_t)(off + p - start) * W + c];
      else if (p >= 0) v = st[(size_t)(p - (start - (taps - 1))) * W + c];
      acc += w[c * taps + k] * v;
      if (stw && k >= 1) stw[(size_t)(k - 1) * W + c] = v;
      cur = v;
    }
    stf<T>(out + (size_t)t * W + c, cur + acc);
  }
}

// the inputs of each sequence's last taps - 1 positions, in position order
__global__ void __launch_bounds__(NT) canon_state_kernel(const float* __restrict__ x, int W, float* __restrict__ state,
                                                         const int* __restrict__ seq_slot, const int* __restrict__ seq_start,
                                                         const int* __restrict__ seq_len, const int* __restrict__ seq_off,
                                                         int taps) {
  constexpr int MAXT = 16;
  const int s = blockIdx.x;
  const int start = seq_start[s], end = start + seq_len[s], off = seq_off[s];
  float* st = state + (size_t)seq_slot[s] * (taps - 1) * W;
  for (int c = blockIdx.y * NT + threadIdx.x; c < W; c += NT * gridDim.y) {
    float keep[MAXT];
#pragma unroll
    for (int k = 0; k < MAXT; ++k) {
      if (k < taps - 1) {
        const int p = end - (taps - 1) + k;
        float v = 0.f;
        if (p >= start) v = x[(size_t)(off + p - start) * W + c];
        else if (p >= 0) v = st[(size_t)(p - (start - (taps - 1))) * W + c];
        keep[k] = v;
      }
    }
#pragma unroll
    for (int k = 0; k < MAXT; ++k)
      if (k < taps - 1) st[(size_t)k * W + c] = keep[k];
  }
}

// ---------------------------------------------------------------------------------- norms
template <typename T>
__global__ void __launch_bounds__(NT) layer_norm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                        const float* __restrict__ b, T* __restrict__ y, int W, float eps) {
  __shared__ float red[NT / 64];
  const float* xr = x + (size_t)blockIdx.x * W;
  float sum = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) sum += xr[c];
  const float mean = block_sum<NT>(sum, red) / (float)W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) { const float d = xr[c] - mean; ss += d * d; }
  const float r = 1.f / sqrtf(block_sum<NT>(ss, red) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += NT) stf<T>(y + (size_t)blockIdx.x * W + c, (xr[c] - mean) * r * w[c] + b[c]);
}

// x += LayerNorm(y + sum_k pw[k] parts[k]) w + b; the summed row is kept in LDS (W floats)
template <typename T>
__global__ void __launch_bounds__(NT) ln_residual_kernel(float* __restrict__ x, const T* __restrict__ y,
                                                         const T* __restrict__ parts, const float* __restrict__ pw, int K,
                                                         const float* __restrict__ w, const float* __restrict__ b, int W,
                                                         float eps) {
  extern __shared__ __attribute__((aligned(16))) float row_s[];
  __shared__ float red[NT / 64];
  const size_t t = blockIdx.x;
  float sum = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) {
    float v = y ? ldf<T>(y + t * W + c) : 0.f;
    for (int k = 0; k < K; ++k) v += pw[t * K + k] * ldf<T>(parts + (t * K + k) * W + c);
    row_s[c] = v;
    sum += v;
  }
  const float mean = block_sum<NT>(sum, red) / (float)W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) { const float d = row_s[c] - mean; ss += d * d; }
  const float r = 1.f / sqrtf(block_sum<NT>(ss, red) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += NT) x[t * W + c] += (row_s[c] - mean) * r * w[c] + b[c];
}

template <typename T>
__global__ void __launch_bounds__(NT) rms_cols_kernel(const T* __restrict__ u, int ld, int c0, int C,
                                                      const float* __restrict__ w, T* __restrict__ y, float eps) {
  __shared__ float red[NT / 64];
  const T* ur = u + (size_t)blockIdx.x * ld + c0;
  float ss = 0.f;
  for (int c = threadIdx.x; c < C; c += NT) { const float v = ldf<T>(ur + c); ss += v * v; }
  const float r = 1.f / sqrtf(block_sum<NT>(ss, red) / (float)C + eps);
  for (int c = threadIdx.x; c < C; c += NT) stf<T>(y + (size_t)blockIdx.x * C + c, ldf<T>(ur + c) * r * w[c]);
}

// per head: y / rms(y) * w (one weight vector for all heads) * sigmoid(z)  (silu: * z sigmoid(z))
template <typename T>
__global__ void __launch_bounds__(64) head_norm_gate_kernel(const float* __restrict__ y, const T* __restrict__ z, int z_ld,
                                                            const float* __restrict__ w, T* __restrict__ out, int H, int P,
                                                            float eps, int silu) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* yr = y + ((size_t)t * H + h) * P;
  float ss = 0.f;
  for (int c = lane; c < P; c += 64) ss += yr[c] * yr[c];
  const float r = 1.f / sqrtf(wave_sum(ss) / (float)P + eps);
  for (int c = lane; c < P; c += 64) {
    const float zv = ldf<T>(z + (size_t)t * z_ld + h * P + c);
    stf<T>(out + ((size_t)t * H + h) * P + c, yr[c] * r * w[c] * (silu ? siluf_(zv) : sigmoidf_(zv)));
  }
}

// g sigmoid(1.702 g) (up + 1), g = min(gate, limit), up clamped to +-limit; u row = gate [ff] | up [ff]
__device__ __forceinline__ float glu_clamp_f(float g, float up, float limit) {
  g = fminf(g, limit);
  up = fminf(fmaxf(up, -limit), limit);
  return g * sigmoidf_(1.702f * g) * (up + 1.f);
}

template <typename T>
__global__ void __launch_bounds__(NT) glu_clamp_kernel(const T* __restrict__ u, int ld, T* __restrict__ y, int ff,
                                                       float limit) {
  const size_t t = blockIdx.x;
  for (int c = blockIdx.y * NT + threadIdx.x; c < ff; c += NT * gridDim.y)
    stf<T>(y + t * ff + c, glu_clamp_f(ldf<T>(u + t * ld + c), ldf<T>(u + t * ld + ff + c), limit));
}

// ---------------------------------------------------------------------------------- latent attention
// Cached side (u given): row = rms(u[c0 : c0 + kvr]) w | rotate(u[c0 + kvr : c0 + kvr + R]) to the token's
// page row.  Query side: qc[t, h] = q_lat[t, h] | rotate(q[t, h, D : D + R]).  Rotation turns the pairs
// (2i, 2i + 1), i < rot / 2, by cs[pos, i] = (cos, sin).
template <typename T>
__global__ void __launch_bounds__(NT) latent_write_kernel(const T* __restrict__ u, int ld, int c0, const float* __restrict__ w,
                                                          float eps, const T* __restrict__ q, const T* __restrict__ q_lat,
                                                          long ql_t, long ql_h, const int* __restrict__ tok_seq,
                                                          const int* __restrict__ tok_pos, const int* __restrict__ seq_slot,
                                                          const int* __restrict__ ptab, int ptab_ld,
                                                          const float* __restrict__ cs, T* __restrict__ pages,
                                                          T* __restrict__ qc, int H, int D, int R, int kvr, int rot, int page) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x, pos = tok_pos[t], tid = threadIdx.x;
  const float* c = cs ? cs + (size_t)pos * rot : nullptr;    // rot / 2 pairs of (cos, sin)
  auto turned = [&](const T* v, int d) {                     // coordinate d of the rotated R-vector v
    const float a = ldf<T>(v + d);
    if (d >= rot || !c) return a;
    const float o = ldf<T>(v + (d ^ 1)), co = c[d & ~1], si = c[(d & ~1) + 1];
    return (d & 1) ? a * co + o * si : a * co - o * si;
  };
  if (u) {
    const T* ur = u + (size_t)t * ld + c0;
    float ss = 0.f;
    for (int e = tid; e < kvr; e += NT) { const float v = ldf<T>(ur + e); ss += v * v; }
    const float r = 1.f / sqrtf(block_sum<NT>(ss, red) / (float)kvr + eps);
    const int slot = seq_slot[tok_seq[t]];
    T* row = pages + ((size_t)ptab[(size_t)slot * ptab_ld + pos / page] * page + pos % page) * (kvr + R);
    for (int e = tid; e < kvr; e += NT) stf<T>(row + e, ldf<T>(ur + e) * r * w[e]);
    for (int e = tid; e < R; e += NT) stf<T>(row + kvr + e, turned(ur + kvr, e));
  }
  const int DC = kvr + R;
  for (int e = tid; e < H * DC; e += NT) {
    const int h = e / DC, d = e % DC;
    const float v = d < kvr ? ldf<T>(q_lat + (size_t)t * ql_t + (size_t)h * ql_h + d)
                            : turned(q + ((size_t)t * H + h) * (D + R) + D, d - kvr);
    stf<T>(qc + (size_t)t * H * DC + e, v);
  }
}

// ---------------------------------------------------------------------------------- gated delta rule
// prep row = q [G, N] | k [G, N] | decay [H, N] | beta [H], all fp32
template <typename T>
__global__ void __launch_bounds__(NT) delta_prep_kernel(const T* __restrict__ qkv, int Cq, const T* __restrict__ u, int ld,
                                                        int b0, const float* __restrict__ a, const float* __restrict__ dt_bias,
                                                        const float* __restrict__ A_log, float* __restrict__ prep, int H, int G,
                                                        int N) {
  const size_t t = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, GN = G * N, HN = H * N;
  float* pr = prep + t * (2 * GN + HN + H);
  const float qs = 1.f / sqrtf((float)N);
  for (int unit = wave; unit < 2 * G; unit += NT / 64) {     // unit = (q | k, kv head): one wave each
    const T* src = qkv + t * Cq + (size_t)unit * N;
    float ss = 0.f;
    for (int n = lane; n < N; n += 64) { const float v = ldf<T>(src + n); ss += v * v; }
    const float r = 1.f / sqrtf(wave_sum(ss) + 1e-6f) * (unit < G ? qs : 1.f);
    for (int n = lane; n < N; n += 64) pr[(size_t)unit * N + n] = ldf<T>(src + n) * r;
  }
  for (int e = tid; e < HN; e += NT) {
    const float raw = a[t * HN + e] + dt_bias[e];
    const float sp = raw > 20.f ? raw : log1pf(expf(raw));
    pr[2 * GN + e] = expf(-expf(A_log[e / N]) * sp);
  }
  for (int e = tid; e < H; e += NT) pr[2 * GN + HN + e] = sigmoidf_(ldf<T>(u + t * ld + b0 + e));
}

// sum over the 16 lanes of a DPP row (quad swaps, then row rotations by 4 and 8); every lane gets the sum
__device__ __forceinline__ float row16_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xF, 0xF, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xF, 0xF, false));
  return v;
}

// GD = decay numbers per head in a prep row: N (one per key channel) or 1 (one for the head's whole state).
// One workgroup per (sequence, head, 16 value columns): wave w owns columns 4 w .. 4 w + 3; the 16 lanes of
// a DPP row share one column, lane rg of the row keeping state rows rg * NR .. rg * NR + NR - 1 in
// registers (NR = ceil(N / 16) rounded up to 4), so the two sums over rows per token (S^T k and S^T q) are
// NR FMAs and four in-row DPP adds.  Tokens are staged TC at a time (q, k, decay rows, beta, the 16 values);
// the next chunk's rows travel global -> registers while the current one is stepped, registers -> the
// other LDS buffer after it (one barrier per chunk).
template <typename T, int NR>
__global__ void __launch_bounds__(NT) delta_scan_kernel(const float* __restrict__ prep, int prep_ld, const T* __restrict__ qkv,
                                                        int Cq, float* __restrict__ state, const int* __restrict__ seq_slot,
                                                        const int* __restrict__ seq_start, const int* __restrict__ seq_len,
                                                        const int* __restrict__ seq_off, float* __restrict__ y, int H, int G,
                                                        int N, int P, int GD) {
  constexpr int NP = 16 * NR, TC = NR >= 16 ? 4 : (NR >= 8 ? 8 : 16), EL = TC * 3 * NP / NT;   // EL = 12
  constexpr int CW = 16;                                     // value columns per workgroup
  __shared__ __attribute__((aligned(16))) float rows_s[2][TC][3][NP];   // q | k | decay
  __shared__ float v_s[2][TC][CW], b_s[2][TC];
  const int s = blockIdx.x, h = blockIdx.y, p0 = blockIdx.z * CW, tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6, rg = lane & 15, col = wave * 4 + (lane >> 4), p = p0 + col;
  const int start = seq_start[s], len = seq_len[s], off = seq_off[s];
  const int g = h / (H / G), GN = G * N, HN = H * GD;
  float* st = state + ((size_t)seq_slot[s] * H + h) * N * P;
  float S[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int n = rg * NR + i;
    S[i] = (start > 0 && n < N && p < P) ? st[(size_t)n * P + p] : 0.f;
  }
  float pre[EL], pre_v = 0.f, pre_b = 0.f;
  auto fetch = [&](int t0) {                                 // rows of tokens t0 .. t0 + TC - 1 into registers
    const int tc = min(TC, len - t0);
#pragma unroll
    for (int i = 0; i < EL; ++i) {
      const int e = tid + i * NT, tt = e / (3 * NP), r = e % (3 * NP), which = r / NP, n = r % NP;
      float v = which == 2 ? 1.f : 0.f;                      // rows past N: no decay, no key, no query
      if (tt < tc && n < N) {
        const float* pr = prep + (size_t)(off + t0 + tt) * prep_ld;
        v = which == 0 ? pr[g * N + n] : (which == 1 ? pr[GN + g * N + n] : pr[2 * GN + h * GD + (GD == 1 ? 0 : n)]);
      }
      pre[i] = v;
    }
    {
      const int tt = tid / CW, c = tid % CW;
      pre_v = (tid < TC * CW && tt < tc && p0 + c < P) ? ldf<T>(qkv + (size_t)(off + t0 + tt) * Cq + 2 * GN + h * P + p0 + c) : 0.f;
      pre_b = tid < tc ? prep[(size_t)(off + t0 + tid) * prep_ld + 2 * GN + HN + h] : 0.f;
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < EL; ++i) {
      const int e = tid + i * NT;
      (&rows_s[buf][0][0][0])[e] = pre[i];
    }
    if (tid < TC * CW) v_s[buf][tid / CW][tid % CW] = pre_v;
    if (tid < TC) b_s[buf][tid] = pre_b;
  };
  static_assert(TC * CW <= NT && TC * 3 * NP % NT == 0, "staging shape");
  fetch(0);
  stash(0);
  __syncthreads();
  int buf = 0;
  for (int t0 = 0; t0 < len; t0 += TC, buf ^= 1) {
    const int tc = min(TC, len - t0);
    const bool more = t0 + TC < len;
    if (more) fetch(t0 + TC);
    for (int tt = 0; tt < tc; ++tt) {
      const float4* qq = reinterpret_cast<const float4*>(&rows_s[buf][tt][0][rg * NR]);
      const float4* kq = reinterpret_cast<const float4*>(&rows_s[buf][tt][1][rg * NR]);
      const float4* gq = reinterpret_cast<const float4*>(&rows_s[buf][tt][2][rg * NR]);
      float4 kk[NR / 4];
      float kv = 0.f;
#pragma unroll
      for (int i = 0; i < NR / 4; ++i) {
        const float4 gv = gq[i];
        kk[i] = kq[i];
        S[4 * i] *= gv.x; S[4 * i + 1] *= gv.y; S[4 * i + 2] *= gv.z; S[4 * i + 3] *= gv.w;
        kv += S[4 * i] * kk[i].x + S[4 * i + 1] * kk[i].y + S[4 * i + 2] * kk[i].z + S[4 * i + 3] * kk[i].w;
      }
      kv = row16_sum(kv);
      const float w = b_s[buf][tt] * (v_s[buf][tt][col] - kv);
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < NR / 4; ++i) {
        const float4 qv = qq[i];
        S[4 * i] += kk[i].x * w; S[4 * i + 1] += kk[i].y * w; S[4 * i + 2] += kk[i].z * w; S[4 * i + 3] += kk[i].w * w;
        o += S[4 * i] * qv.x + S[4 * i + 1] * qv.y + S[4 * i + 2] * qv.z + S[4 * i + 3] * qv.w;
      }
      o = row16_sum(o);
      if (rg == 0 && p < P) y[(size_t)(off + t0 + tt) * H * P + h * P + p] = o;
    }
    if (more) stash(buf ^ 1);
    __syncthreads();
  }
  if (p < P) {
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int n = rg * NR + i;
      if (n < N) st[(size_t)n * P + p] = S[i];
    }
  }
}

// ---------------------------------------------------------------------------------- mixture of experts
// Router scores: one wave per (token, expert), fp32 dot product over the width with 8-element loads.
template <typename T>
__global__ void __launch_bounds__(NT) moe_logits_kernel(const T* __restrict__ h, int W, const float* __restrict__ router,
                                                        int E, float* __restrict__ z, const float* __restrict__ bias) {
  const size_t t = blockIdx.x;
  const int lane = threadIdx.x & 63, e = blockIdx.y * (NT / 64) + (threadIdx.x >> 6);
  if (e >= E) return;
  const T* hr = h + t * W;
  const float* rr = router + (size_t)e * W;
  float acc = 0.f;
  if (W % 8 == 0) {
    for (int c = lane * 8; c < W; c += 64 * 8) {
      float a[8], r[8];
      load8<T>(hr + c, a);
      load8<float>(rr + c, r);
#pragma unroll
      for (int k = 0; k < 8; ++k) acc += a[k] * r[k];
    }
  } else {
    for (int c = lane; c < W; c += 64) acc += ldf<T>(hr + c) * rr[c];
  }
  acc = wave_sum(acc);
  if (lane == 0) z[t * E + e] = acc + (bias ? bias[e] : 0.f);
}

// One wave per token: softmax over the experts' scores, then the `top` largest (lowest index on a tie),
// divided by their sum (+ 1e-20) and multiplied by scale.  sigm: the scores are sigmoid(z) and the `top`
// largest keep their own value (times scale); they are picked by z itself (the same order), so scores that
// round to 1 do not tie.  sigm == 2: the `top` largest logits, softmax over those alone (times scale).
__global__ void __launch_bounds__(64) moe_topk_kernel(const float* __restrict__ z, int E, int top, float scale,
                                                      int* __restrict__ idx, float* __restrict__ wts, int sigm) {
  extern __shared__ __attribute__((aligned(16))) float z_s[];   // [E]
  const size_t t = blockIdx.x;
  const int lane = threadIdx.x;
  float mx = -INFINITY;
  for (int e = lane; e < E; e += 64) { z_s[e] = z[t * E + e]; mx = fmaxf(mx, z_s[e]); }
  mx = wave_max(mx);
  if (!sigm) {
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) sum += expf(z_s[e] - mx);
    sum = wave_sum(sum);
    for (int e = lane; e < E; e += 64) z_s[e] = expf(z_s[e] - mx) / sum;
  }
  float tot = 0.f, my_w = 0.f;
  int my_i = 0;                                              // lane k keeps the k-th choice
  const float gone = sigm ? -INFINITY : -2.f;                // what a taken entry becomes (below every live one)
  for (int k = 0; k < top; ++k) {
    float best = sigm ? -INFINITY : -1.f;
    int bi = E;
    for (int e = lane; e < E; e += 64)
      if (z_s[e] > best) { best = z_s[e]; bi = e; }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
    }
    if (bi >= E) {                                           // scores that compare with nothing (NaN): keep the ids in range
      bi = k;
      best = 0.f;
    }
    if (lane == k) { my_w = best; my_i = bi; }
    if (lane == 0) z_s[bi] = gone;                           // LDS accesses of one wave keep their order
    tot += best;
  }
  float soft = 0.f;
  if (sigm == 2) {                                           // the first choice holds the largest logit
    const float ex = lane < top ? expf(my_w - __shfl(my_w, 0, 64)) : 0.f;
    soft = ex / wave_sum(ex);
  }
  if (lane < top) {
    idx[t * top + lane] = my_i;
    wts[t * top + lane] = sigm == 2 ? soft * scale : sigm ? sigmoidf_(my_w) * scale : my_w / (tot + 1e-20f) * scale;
  }
}

// decode-sized steps: out row r of pair (token, choice) = act(gate_r . h, up_r . h); one wave per row at a time,
// lanes stride the width with 8-element loads, the token's row sits in LDS as fp32.  silu: the activation is
// silu(w gate) (w up) with w = in_w[pair] (null: 1), the unit of an input scaled by the router's weight.
template <typename T>
__global__ void __launch_bounds__(NT) moe_gate_up_kernel(const T* __restrict__ h, int W, const int* __restrict__ idx, int top,
                                                         const T* __restrict__ w_gu, int ff, float limit, T* __restrict__ y,
                                                         int rows_per_wg, int E, int silu, const float* __restrict__ in_w) {
  extern __shared__ __attribute__((aligned(16))) float h_s[];   // [W]
  const size_t pair = blockIdx.x, t = pair / top;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int c = tid; c < W; c += NT) h_s[c] = ldf<T>(h + t * W + c);
  __syncthreads();
  const T* wg = w_gu + (size_t)min(max(idx[pair], 0), E - 1) * 2 * ff * W;
  const int r1 = min(ff, (int)(blockIdx.y + 1) * rows_per_wg);
  for (int r = blockIdx.y * rows_per_wg + wave; r < r1; r += NT / 64) {
    float ag = 0.f, au = 0.f;
    if (W % 8 == 0) {
      for (int c = lane * 8; c < W; c += 64 * 8) {
        float a[8], b[8];
        load8<T>(wg + (size_t)r * W + c, a);
        load8<T>(wg + (size_t)(ff + r) * W + c, b);
#pragma unroll
        for (int e = 0; e < 8; ++e) { ag += a[e] * h_s[c + e]; au += b[e] * h_s[c + e]; }
      }
    } else {
      for (int c = lane; c < W; c += 64) {
        ag += ldf<T>(wg + (size_t)r * W + c) * h_s[c];
        au += ldf<T>(wg + (size_t)(ff + r) * W + c) * h_s[c];
      }
    }
    ag = wave_sum(ag);
    au = wave_sum(au);
    if (lane == 0) {
      const float rw = in_w ? in_w[pair] : 1.f;
      stf<T>(y + pair * ff + r, silu ? siluf_(rw * ag) * (rw * au) : glu_clamp_f(ag, au, limit));
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(NT) moe_down_kernel(const T* __restrict__ y, int ff, const int* __restrict__ idx,
                                                      const T* __restrict__ w_down, int W, T* __restrict__ out,
                                                      int rows_per_wg, int E) {
  extern __shared__ __attribute__((aligned(16))) float y_s[];   // [ff]
  const size_t pair = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int c = tid; c < ff; c += NT) y_s[c] = ldf<T>(y + pair * ff + c);
  __syncthreads();
  const T* wd = w_down + (size_t)min(max(idx[pair], 0), E - 1) * W * ff;
  const int r1 = min(W, (int)(blockIdx.y + 1) * rows_per_wg);
  for (int r = blockIdx.y * rows_per_wg + wave; r < r1; r += NT / 64) {
    float acc = 0.f;
    if (ff % 8 == 0) {
      for (int c = lane * 8; c < ff; c += 64 * 8) {
        float a[8];
        load8<T>(wd + (size_t)r * ff + c, a);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc += a[e] * y_s[c + e];
      }
    } else {
      for (int c = lane; c < ff; c += 64) acc += ldf<T>(wd + (size_t)r * ff + c) * y_s[c];
    }
    acc = wave_sum(acc);
    if (lane == 0) stf<T>(out + pair * W + r, acc);
  }
}

}  // namespace

#define SM_T(f32, ...)                                  \
  do {                                                  \
    if (f32) { using T = float; __VA_ARGS__; }          \
    else { using T = bf16_t; __VA_ARGS__; }             \
  } while (0)

extern "C" {

int edge_sm_embed_bigram(const int64_t* ids, const void* table, const void* bigram, int64_t* prev_tok, const int* tok_seq,
                         const int* tok_pos, const int* seq_slot, const int* seq_start, const int* seq_len,
                         const int* seq_off, float* out, int rows, int n, int W, int V, long buckets, long mul_prev,
                         long mul_cur, int f32, hipStream_t st) {
  if (rows == 0) return 0;
  if (buckets <= 0) return -2;
  SM_T(f32, hipLaunchKernelGGL(embed_bigram_kernel<T>, dim3(rows), dim3(NT), 0, st, ids, (const T*)table, (const T*)bigram,
                               prev_tok, tok_seq, tok_pos, seq_slot, seq_start, out, W, V, buckets, mul_prev, mul_cur));
  hipLaunchKernelGGL(prev_token_kernel, dim3((n + 63) / 64), dim3(64), 0, st, ids, prev_tok, seq_slot, seq_len, seq_off, n);
  return (int)hipGetLastError();
}

int edge_sm_canon(const float* x, int W, const float* w, float* state, const int* tok_seq, const int* tok_pos,
                  const int* seq_slot, const int* seq_start, const int* seq_len, const int* seq_off, void* out, int rows,
                  int n, int taps, int max_len, int f32, hipStream_t st) {
  if (rows == 0) return 0;
  if (taps < 1 || taps > 16) return -2;
  const bool one = max_len == 1 && taps > 1;                 // every sequence brings one token
  const int gy = (W + NT * 4 - 1) / (NT * 4);
  if (W % 4 == 0)
    SM_T(f32, hipLaunchKernelGGL((canon_kernel<T, true>), dim3(rows, gy), dim3(NT), 0, st, x, W, w, (const float*)state,
                                 tok_seq, tok_pos, seq_slot, seq_start, seq_off, (T*)out, taps,
                                 one ? state : (float*)nullptr));
  else
    SM_T(f32, hipLaunchKernelGGL((canon_kernel<T, false>), dim3(rows, gy), dim3(NT), 0, st, x, W, w, (const float*)state,
                                 tok_seq, tok_pos, seq_slot, seq_start, seq_off, (T*)out, taps,
                                 one ? state : (float*)nullptr));
  if (taps > 1 && !one)
    hipLaunchKernelGGL(canon_state_kernel, dim3(n, gy), dim3(NT), 0, st, x, W, state, seq_slot, seq_start, seq_len, seq_off,
                       taps);
  return (int)hipGetLastError();
}

int edge_sm_layer_norm(const float* x, const float* w, const float* b, void* y, int rows, int W, float eps, int f32,
                       hipStream_t st) {
  if (rows == 0) return 0;
  SM_T(f32, hipLaunchKernelGGL(layer_norm_kernel<T>, dim3(rows), dim3(NT), 0, st, x, w, b, (T*)y, W, eps));
  return (int)hipGetLastError();
}

int edge_sm_ln_residual(float* x, const void* y, const void* parts, const float* pw, int K, const float* w, const float* b,
                        int rows, int W, float eps, int f32, hipStream_t st) {
  if (rows == 0) return 0;
  if ((size_t)W * 4 > 60 * 1024) return -3;
  SM_T(f32, hipLaunchKernelGGL(ln_residual_kernel<T>, dim3(rows), dim3(NT), (size_t)W * 4, st, x, (const T*)y,
                               (const T*)parts, pw, K, w, b, W, eps));
  return (int)hipGetLastError();
}

int edge_sm_rms_cols(const void* u, int ld, int c0, int C, const float* w, void* y, int rows, float eps, int f32,
                     hipStream_t st) {
  if (rows == 0) return 0;
  SM_T(f32, hipLaunchKernelGGL(rms_cols_kernel<T>, dim3(rows), dim3(NT), 0, st, (const T*)u, ld, c0, C, w, (T*)y, eps));
  return (int)hipGetLastError();
}

int edge_sm_head_norm_gate(const float* y, const void* z, int z_ld, const float* w, void* out, int rows, int H, int P,
                           float eps, int silu, int f32, hipStream_t st) {
  if (rows == 0) return 0;
  SM_T(f32, hipLaunchKernelGGL(head_norm_gate_kernel<T>, dim3(rows, H), dim3(64), 0, st, y, (const T*)z, z_ld, w, (T*)out, H,
                               P, eps, silu));
  return (int)hipGetLastError();
}

int edge_sm_glu_clamp(const void* u, int ld, void* y, int rows, int ff, float limit, int f32, hipStream_t st) {
  if (rows == 0 || ff == 0) return 0;
  const int gy = (ff + NT * 4 - 1) / (NT * 4);
  SM_T(f32, hipLaunchKernelGGL(glu_clamp_kernel<T>, dim3(rows, gy), dim3(NT), 0, st, (const T*)u, ld, (T*)y, ff, limit));
  return (int)hipGetLastError();
}

int edge_sm_latent_write(const void* u, int ld, int c0, const float* w, float eps, const void* q, const void* q_lat,
                         long ql_t, long ql_h, const int* tok_seq, const int* tok_pos, const int* seq_slot, const int* ptab,
                         int ptab_ld, const float* cs, void* pages, void* qc, int rows, int H, int D, int R, int kvr, int rot,
                         int page, int f32, hipStream_t st) {
  if (rows == 0) return 0;
  if (rot % 2 || rot > R || (rot > 0 && !cs) || (u && !w)) return -2;
  SM_T(f32, hipLaunchKernelGGL(latent_write_kernel<T>, dim3(rows), dim3(NT), 0, st, (const T*)u, ld, c0, w, eps, (const T*)q,
                               (const T*)q_lat, ql_t, ql_h, tok_seq, tok_pos, seq_slot, ptab, ptab_ld, cs, (T*)pages, (T*)qc,
                               H, D, R, kvr, rot, page));
  return (int)hipGetLastError();
}

int edge_sm_delta_prep(const void* qkv, int Cq, const void* u, int ld, int b0, const float* a, const float* dt_bias,
                       const float* A_log, float* prep, int rows, int H, int G, int N, int f32, hipStream_t st) {
  if (rows == 0) return 0;
  if (G <= 0 || H % G) return -2;
  SM_T(f32, hipLaunchKernelGGL(delta_prep_kernel<T>, dim3(rows), dim3(NT), 0, st, (const T*)qkv, Cq, (const T*)u, ld, b0, a,
                               dt_bias, A_log, prep, H, G, N));
  return (int)hipGetLastError();
}

int edge_sm_delta_scan(const float* prep, int prep_ld, const void* qkv, int Cq, float* state, const int* seq_slot,
                       const int* seq_start, const int* seq_len, const int* seq_off, float* y, int n, int H, int G, int N,
                       int P, int GD, int f32, hipStream_t st) {
  if (n == 0) return 0;
  if (G <= 0 || H % G || N > 256 || (GD != N && GD != 1)) return -2;
  const dim3 grid(n, H, (P + 15) / 16);
#define SM_DS(NR)                                                                                                  \
  SM_T(f32, hipLaunchKernelGGL((delta_scan_kernel<T, NR>), grid, dim3(NT), 0, st, prep, prep_ld, (const T*)qkv, Cq, \
                               state, seq_slot, seq_start, seq_len, seq_off, y, H, G, N, P, GD))
  if (N <= 64) SM_DS(4);
  else if (N <= 128) SM_DS(8);
  else SM_DS(16);
#undef SM_DS
  return (int)hipGetLastError();
}

// z: fp32 scratch [rows, E] (the experts' scores)
int edge_sm_moe_route(const void* h, int W, const float* router, const float* bias, int E, int top, float scale, float* z,
                      int* idx, float* wts, int rows, int sigm, int f32, hipStream_t st) {
  if (rows == 0) return 0;
  if (top < 1 || top > E || top > 64 || E > 8192) return -2;
  SM_T(f32, hipLaunchKernelGGL(moe_logits_kernel<T>, dim3(rows, (E + NT / 64 - 1) / (NT / 64)), dim3(NT), 0, st, (const T*)h,
                               W, router, E, z, bias));
  hipLaunchKernelGGL(moe_topk_kernel, dim3(rows), dim3(64), (size_t)E * 4, st, (const float*)z, E, top, scale, idx, wts, sigm);
  return (int)hipGetLastError();
}

// y: scratch [rows * top, ff]; out [rows * top, W]
int edge_sm_moe_experts(const void* h, int W, const int* idx, int top, const void* w_gu, const void* w_down, int ff,
                        float limit, int silu, const float* in_w, void* y, void* out, int rows, int E, int f32,
                        hipStream_t st) {
  if (rows == 0) return 0;
  if ((size_t)W * 4 > 60 * 1024 || (size_t)ff * 4 > 60 * 1024) return -3;
  const int rpw = 16;
  SM_T(f32, hipLaunchKernelGGL(moe_gate_up_kernel<T>, dim3(rows * top, (ff + rpw - 1) / rpw), dim3(NT), (size_t)W * 4, st,
                               (const T*)h, W, idx, top, (const T*)w_gu, ff, limit, (T*)y, rpw, E, silu, in_w));
  SM_T(f32, hipLaunchKernelGGL(moe_down_kernel<T>, dim3(rows * top, (W + rpw - 1) / rpw), dim3(NT), (size_t)ff * 4, st,
                               (const T*)y, ff, idx, (const T*)w_down, W, (T*)out, rpw, E));
  return (int)hipGetLastError();
}

}  // extern "C"
