// Kernels of the ragged-step sequence mixers (ops/seqmix.py): scalar-gain RMS norm, squared ReLU,
// rotary + paged key / value write, block pooling, windowed attention with pooled blocks over a
// paged cache, causal convolution with a per-slot tail, the Mamba-2 recurrence, the gated group
// norm and the two-branch combine with the residual add.
//
// Every kernel is instantiated for fp32 and bf16 storage (template T); scores, softmax, norms,
// decays and the recurrent state are fp32 in both.  A token is addressed by (sequence of the step,
// position) and its key / value row by the sequence's page-table row, so a result does not depend
// on how a prompt was cut into steps or on what else is in the batch: each query's visible keys are
// walked in the same order from the same first key, each block mean sums its rows in position
// order, and the recurrence steps token by token.
#include "common.h"
#include "seqmix/seqmix_common.h"

namespace {

// ---------------------------------------------------------------------------------- rows
template <typename T>
__global__ void __launch_bounds__(NT) embed_kernel(const int64_t* __restrict__ ids, const T* __restrict__ table,
                                                   float* __restrict__ out, int W, int V, float scale) {
  const int t = blockIdx.x;
  int64_t id = ids[t];
  id = id < 0 ? 0 : (id >= V ? V - 1 : id);
  for (int c = threadIdx.x; c < W; c += NT) out[(size_t)t * W + c] = ldf<T>(table + (size_t)id * W + c) * scale;
}

template <typename T>
__global__ void __launch_bounds__(NT) scalar_norm_kernel(const float* __restrict__ x, const float* __restrict__ gain,
                                                         T* __restrict__ y, int W, float eps) {
  __shared__ float red[NT / 64];
  const float* xr = x + (size_t)blockIdx.x * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) { const float v = xr[c]; ss += v * v; }
  ss = block_sum<NT>(ss, red);
  const float r = 1.f / sqrtf(ss / (float)W + eps) * gain[0];
  for (int c = threadIdx.x; c < W; c += NT) stf<T>(y + (size_t)blockIdx.x * W + c, xr[c] * r);
}

// VEC: eight columns per thread through 16-byte accesses (ld, c0, C multiples of 8)
template <typename T, bool VEC>
__global__ void __launch_bounds__(NT) relu2_kernel(const T* __restrict__ u, int ld, int c0, T* __restrict__ y, int C) {
  const int t = blockIdx.x;
  if constexpr (VEC) {
    for (int c = (blockIdx.y * NT + threadIdx.x) * 8; c < C; c += NT * gridDim.y * 8) {
      float f[8];
      load8<T>(u + (size_t)t * ld + c0 + c, f);
#pragma unroll
      for (int e = 0; e < 8; ++e) { const float v = fmaxf(f[e], 0.f); f[e] = v * v; }
      store8<T>(y + (size_t)t * C + c, f);
    }
  } else {
    for (int c = blockIdx.y * NT + threadIdx.x; c < C; c += NT * gridDim.y) {
      const float v = fmaxf(ldf<T>(u + (size_t)t * ld + c0 + c), 0.f);
      stf<T>(y + (size_t)t * C + c, v * v);
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(NT) cat_cast_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                      T* __restrict__ y, int W) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < 2 * W; c += NT)
    stf<T>(y + (size_t)t * 2 * W + c, c < W ? a[(size_t)t * W + c] : b[(size_t)t * W + c - W]);
}

// x += 0.5 (l / rms(l) * wl + r / rms(r) * wr) + extra
template <typename T>
__global__ void __launch_bounds__(NT) combine_kernel(float* __restrict__ x, const T* __restrict__ l,
                                                     const T* __restrict__ r, const float* __restrict__ wl,
                                                     const float* __restrict__ wr, const T* __restrict__ extra, int W,
                                                     float eps) {
  __shared__ float red[NT / 64];
  const size_t row = (size_t)blockIdx.x * W;
  float sl = 0.f, sr = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) {
    const float a = ldf<T>(l + row + c), b = ldf<T>(r + row + c);
    sl += a * a;
    sr += b * b;
  }
  sl = block_sum<NT>(sl, red);
  sr = block_sum<NT>(sr, red);
  const float rl = 1.f / sqrtf(sl / (float)W + eps), rr = 1.f / sqrtf(sr / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += NT) {
    float v = 0.5f * (ldf<T>(l + row + c) * rl * wl[c] + ldf<T>(r + row + c) * rr * wr[c]);
    if (extra) v += ldf<T>(extra + row + c);
    x[row + c] += v;
  }
}

// out = (y silu(z)) / rms over each of `groups` equal parts * w
template <typename T>
__global__ void __launch_bounds__(NT) gated_norm_kernel(const float* __restrict__ y, const T* __restrict__ z, int z_ld,
                                                        const float* __restrict__ w, T* __restrict__ out, int C,
                                                        int groups, float eps) {
  __shared__ float red[NT / 64];
  const int t = blockIdx.x, g = blockIdx.y, gs = C / groups;
  const float* yr = y + (size_t)t * C + g * gs;
  const T* zr = z + (size_t)t * z_ld + g * gs;
  float ss = 0.f;
  for (int c = threadIdx.x; c < gs; c += NT) {
    const float v = yr[c] * siluf_(ldf<T>(zr + c));
    ss += v * v;
  }
  ss = block_sum<NT>(ss, red);
  const float r = 1.f / sqrtf(ss / (float)gs + eps);
  for (int c = threadIdx.x; c < gs; c += NT)
    stf<T>(out + (size_t)t * C + g * gs + c, yr[c] * siluf_(ldf<T>(zr + c)) * r * w[g * gs + c]);
}

// ---------------------------------------------------------------------------------- rotary + paged write
// proj row = q [H, D] | k [G, D] | v [G, Dv]; cs [positions, rot / 2, 2]
template <typename T, bool VEC>
__global__ void __launch_bounds__(NT) rope_write_kernel(const T* __restrict__ proj, int ld, const int* __restrict__ tok_seq,
                                                        const int* __restrict__ tok_pos, const int* __restrict__ seq_slot,
                                                        const int* __restrict__ ptab, int ptab_ld,
                                                        const float* __restrict__ cs, T* __restrict__ q_out,
                                                        T* __restrict__ kp, T* __restrict__ vp, int H, int G, int D, int Dv,
                                                        int rot, int page) {
  const int t = blockIdx.x;
  const int pos = tok_pos[t], slot = seq_slot[tok_seq[t]];
  const size_t prow = (size_t)ptab[(size_t)slot * ptab_ld + pos / page] * page + pos % page;
  const T* row = proj + (size_t)t * ld;
  const int half = rot >> 1, nqk = (H + G) * D;
  const float* c = cs ? cs + (size_t)pos * rot : nullptr;          // rot / 2 pairs of (cos, sin)
  if constexpr (VEC) {                                       // 8 coordinates per thread (D, Dv, rot / 2, ld: multiples of 8)
    for (int e = threadIdx.x * 8; e < nqk; e += NT * 8) {
      const int hh = e / D, d = e % D;
      float v[8];
      load8<T>(row + e, v);
      if (d < rot) {
        const int i = d < half ? d : d - half;
        float o[8], tab[16];
        load8<T>(row + (d < half ? e + half : e - half), o);
        load8<float>(c + 2 * i, tab);
        load8<float>(c + 2 * i + 8, tab + 8);
#pragma unroll
        for (int k = 0; k < 8; ++k)
          v[k] = d < half ? v[k] * tab[2 * k] - o[k] * tab[2 * k + 1] : v[k] * tab[2 * k] + o[k] * tab[2 * k + 1];
      }
      if (hh < H) store8<T>(q_out + (size_t)t * H * D + e, v);
      else store8<T>(kp + (prow * G + (hh - H)) * D + d, v);
    }
    if (!vp) return;                                         // the values are the keys: nothing more to cache
    for (int e = threadIdx.x * 8; e < G * Dv; e += NT * 8)
      *reinterpret_cast<uint4*>(vp + prow * G * Dv + e) = *reinterpret_cast<const uint4*>(row + nqk + e);
    if constexpr (sizeof(T) == 4)                            // fp32 rows: the second 16 bytes of each chunk
      for (int e = threadIdx.x * 8; e < G * Dv; e += NT * 8)
        *reinterpret_cast<uint4*>(vp + prow * G * Dv + e + 4) = *reinterpret_cast<const uint4*>(row + nqk + e + 4);
    return;
  }
  for (int e = threadIdx.x; e < nqk; e += NT) {
    const int hh = e / D, d = e % D;
    float v = ldf<T>(row + e);
    if (d < rot) {
      const int i = d < half ? d : d - half;
      const float co = c[2 * i], si = c[2 * i + 1];
      const float o = ldf<T>(row + (d < half ? e + half : e - half));
      v = d < half ? v * co - o * si : v * co + o * si;
    }
    if (hh < H) stf<T>(q_out + (size_t)t * H * D + e, v);
    else stf<T>(kp + (prow * G + (hh - H)) * D + d, v);
  }
  if (!vp) return;
  for (int e = threadIdx.x; e < G * Dv; e += NT) vp[prow * G * Dv + e] = row[nqk + e];
}

// mean over the rows of each block whose last token lies in [start, start + len)
template <typename T>
__global__ void __launch_bounds__(NT) pool_kernel(const T* __restrict__ kp, const T* __restrict__ vp,
                                                  float* __restrict__ kb, float* __restrict__ vb,
                                                  const int* __restrict__ seq_slot, const int* __restrict__ seq_start,
                                                  const int* __restrict__ seq_len, const int* __restrict__ ptab,
                                                  int ptab_ld, int G, int D, int Dv, int page, int PB, int pool) {
  const int s = blockIdx.x;
  const int start = seq_start[s], end = start + seq_len[s];
  const int b = start / pool + blockIdx.y;
  if (b * pool + pool - 1 >= end) return;
  const int* pt = ptab + (size_t)seq_slot[s] * ptab_ld;
  const int p0 = b * pool;
  const size_t dst = (size_t)pt[p0 / page] * PB + (p0 % page) / pool;
  const float inv = 1.f / (float)pool;
  const int nk = G * D, nv = G * Dv;
  for (int e = threadIdx.x; e < nk + nv; e += NT) {
    float acc = 0.f;
    for (int j = 0; j < pool; ++j) {
      const int p = p0 + j;
      const size_t r = (size_t)pt[p / page] * page + p % page;
      acc += e < nk ? ldf<T>(kp + r * nk + e) : ldf<T>(vp + r * nv + (e - nk));
    }
    if (e < nk) kb[dst * nk + e] = acc * inv;
    else vb[dst * nv + (e - nk)] = acc * inv;
  }
}

// ---------------------------------------------------------------------------------- attention
// One workgroup per (token, kv head): its R = H / G query heads share every key / value row read.
// Keys are walked in chunks of KC: (A) thread j scores key j against the R queries (q in LDS,
// broadcast reads), (B) wave w keeps the running max / sum of heads w, w + 4, .. and turns the
// chunk's scores into weights, (C) wave w accumulates weight x value over its quarter of the
// chunk with lane = value coordinate (coalesced row reads).  Tokens of the window first, then the
// pooled blocks (fp32 rows): one softmax over both.  A score may be capped (cap tanh(s / cap), cap > 0) and
// lose slope[head] * dist, dist = the query's distance to this thread's key.
constexpr int KC = 256;

template <typename KT, int RMAX, int DVL, bool VEC>
__device__ __forceinline__ void attn_chunk(const KT* __restrict__ kbase, const KT* __restrict__ vbase, int cnt, int g,
                                           int kld, int vld, int D, int Dv, int R, const float* q_s, float* s_s, int* row_s,
                                           float* m_s, float* l_s, float* a_s, int rowidx, float (&acc)[RMAX][VEC ? 8 : DVL],
                                           float cap = 0.f, const float* sl_s = nullptr, int dist = 0) {
  constexpr int AW = VEC ? 8 : DVL;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // (A) scores
  {
    float a[RMAX];
#pragma unroll
    for (int r = 0; r < RMAX; ++r) a[r] = 0.f;
    if (tid < cnt) {
      const KT* kr = kbase + (size_t)rowidx * kld + g * D;
      if constexpr (VEC) {                                  // rows are 16-byte aligned: D % 8 == 0
        for (int d = 0; d < D; d += 8) {
          float kv[8];
          load8<KT>(kr + d, kv);
#pragma unroll
          for (int e = 0; e < 8; ++e)
#pragma unroll
            for (int r = 0; r < RMAX; ++r) a[r] += q_s[r * D + d + e] * kv[e];
        }
      } else {
        for (int d = 0; d < D; ++d) {
          const float kv = ldf<KT>(kr + d);
#pragma unroll
          for (int r = 0; r < RMAX; ++r) a[r] += q_s[r * D + d] * kv;
        }
      }
    }
    if (cap > 0.f) {
#pragma unroll
      for (int r = 0; r < RMAX; ++r) a[r] = cap * tanhf(a[r] / cap);
    }
    if (sl_s) {
#pragma unroll
      for (int r = 0; r < RMAX; ++r) a[r] -= sl_s[r] * (float)dist;
    }
#pragma unroll
    for (int r = 0; r < RMAX; ++r) s_s[r * KC + tid] = tid < cnt ? a[r] : -INFINITY;
    row_s[tid] = rowidx;
  }
  __syncthreads();
  // (B) running softmax statistics, one head per wave at a time
  for (int r = wave; r < R; r += NT / 64) {
    float v[KC / 64], cm = -INFINITY;
#pragma unroll
    for (int k = 0; k < KC / 64; ++k) { v[k] = s_s[r * KC + lane + 64 * k]; cm = fmaxf(cm, v[k]); }
    cm = wave_max(cm);
    const float mo = m_s[r], mn = fmaxf(mo, cm);
    float ls = 0.f;
#pragma unroll
    for (int k = 0; k < KC / 64; ++k) {
      const float p = expf(v[k] - mn);
      s_s[r * KC + lane + 64 * k] = p;
      ls += p;
    }
    ls = wave_sum(ls);
    if (lane == 0) {
      const float al = expf(mo - mn);                      // mo = -inf on the first chunk: 0
      m_s[r] = mn;
      l_s[r] = l_s[r] * al + ls;
      a_s[r] = al;
    }
  }
  __syncthreads();
  // (C) weights x values
#pragma unroll
  for (int r = 0; r < RMAX; ++r) {
    const float al = r < R ? a_s[r] : 1.f;
#pragma unroll
    for (int dl = 0; dl < AW; ++dl) acc[r][dl] *= al;
  }
  // eight rows' loads are issued before their products (the walk is latency-bound otherwise)
  const int j1 = min(cnt, 64 * (wave + 1));
  constexpr int UN = 8;
  if constexpr (VEC) {
    // lane = (key of the round, 8 value coordinates): LPK lanes cover a row with one 16-byte (bf16) or
    // two (fp32) loads each, 64 / LPK rows per round, UN rounds in flight; the lanes' partial sums over
    // their keys are added up once, after the last chunk
    constexpr int LPK = 8 * DVL, KPR = 64 / LPK;
    const int dpart = lane % LPK, ksub = lane / LPK;
    const bool live = dpart * 8 < Dv;
    for (int j = 64 * wave; j < j1; j += UN * KPR) {
      float vv[UN][8];
#pragma unroll
      for (int k = 0; k < UN; ++k) {
        const int jk = j + k * KPR + ksub;
        if (live && jk < j1) load8<KT>(vbase + (size_t)row_s[jk] * vld + g * Dv + dpart * 8, vv[k]);
        else {
#pragma unroll
          for (int e = 0; e < 8; ++e) vv[k][e] = 0.f;
        }
      }
#pragma unroll
      for (int k = 0; k < UN; ++k) {
        const int jk = min(j + k * KPR + ksub, j1 - 1);     // rows past the end were loaded as zeros
#pragma unroll
        for (int r = 0; r < RMAX; ++r) {
          const float p = s_s[r * KC + jk];
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[r][e] += p * vv[k][e];
        }
      }
    }
  } else {
    for (int j = 64 * wave; j < j1; j += UN) {
      float vv[UN][DVL];
#pragma unroll
      for (int k = 0; k < UN; ++k) {
        const KT* vr = vbase + (size_t)row_s[min(j + k, j1 - 1)] * vld + g * Dv;
#pragma unroll
        for (int dl = 0; dl < DVL; ++dl) vv[k][dl] = lane + 64 * dl < Dv ? ldf<KT>(vr + lane + 64 * dl) : 0.f;
      }
#pragma unroll
      for (int k = 0; k < UN; ++k) {
        if (j + k < j1) {
#pragma unroll
          for (int r = 0; r < RMAX; ++r) {
            const float p = s_s[r * KC + j + k];
#pragma unroll
            for (int dl = 0; dl < DVL; ++dl) acc[r][dl] += p * vv[k][dl];
          }
        }
      }
    }
  }
  __syncthreads();
}

template <typename T, int RMAX, int DVL, bool VEC>
__global__ void __launch_bounds__(NT) attn_kernel(const T* __restrict__ q, const T* __restrict__ gate, int gate_ld,
                                                  const T* __restrict__ kp, const T* __restrict__ vp,
                                                  const float* __restrict__ kb, const float* __restrict__ vb,
                                                  const int* __restrict__ tok_seq, const int* __restrict__ tok_pos,
                                                  const int* __restrict__ seq_slot, const int* __restrict__ ptab,
                                                  int ptab_ld, T* __restrict__ out, int H, int G, int D, int Dv,
                                                  int page, int PB, float scale, int window, int pool, int nsp, int nsplit,
                                                  float* __restrict__ part, int kld, int vld, int chunked, float cap,
                                                  const float* __restrict__ slopes, const float* __restrict__ sink,
                                                  int gate_elem, int keep_first) {
  // keep_first: the tokens j < keep_first stay visible behind a sliding window
  // chunked: `window` is a chunk size (query i sees floor(i / window) * window .. i); cap / slopes: see attn_chunk;
  // sink: a number per query head that joins the softmax denominator (it enters as the first key split's
  // starting maximum with sum 1 and no value); gate_elem: the gate is [T, H * Dv], one per output coordinate
  // kld / vld: elements between consecutive cached rows of kp / vp (G * D and G * Dv for separate key
  // and value pages; a latent cache whose value is a slice of the key row passes the same stride twice)
  extern __shared__ __attribute__((aligned(16))) float smem[];
  // more than RMAX query heads per kv head: nsp workgroups share the kv head, RMAX heads each
  const int t = blockIdx.x, g = blockIdx.y / nsp, r0 = (blockIdx.y % nsp) * RMAX;
  const int R = min(RMAX, H / G - r0), hq0 = g * (H / G) + r0;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float* q_s = smem;                         // [RMAX][D]
  float* s_s = q_s + RMAX * D;               // [RMAX][KC]
  float* red = s_s + RMAX * KC;              // [RMAX][Dv]
  float* m_s = red + RMAX * Dv;              // [RMAX] x 3
  float* l_s = m_s + RMAX;
  float* a_s = l_s + RMAX;
  float* sl_s = a_s + RMAX;                  // [RMAX] slopes of this workgroup's heads
  int* row_s = reinterpret_cast<int*>(sl_s + RMAX);  // [KC]
  const int i = tok_pos[t];
  const int* pt = ptab + (size_t)seq_slot[tok_seq[t]] * ptab_ld;
  for (int e = tid; e < RMAX * D; e += NT) {
    const int r = e / D, d = e % D;
    q_s[e] = r < R ? ldf<T>(q + ((size_t)t * H + hq0 + r) * D + d) * scale : 0.f;
  }
  for (int e = tid; e < RMAX * Dv; e += NT) red[e] = 0.f;
  if (tid < RMAX) {
    const bool sk = sink && blockIdx.z == 0 && tid < R;
    m_s[tid] = sk ? sink[hq0 + tid] : -INFINITY;
    l_s[tid] = sk ? 1.f : 0.f;
    a_s[tid] = 1.f;
    sl_s[tid] = (slopes && tid < R) ? slopes[hq0 + tid] : 0.f;
  }
  constexpr int AW = VEC ? 8 : DVL;
  float acc[RMAX][AW];
#pragma unroll
  for (int r = 0; r < RMAX; ++r)
#pragma unroll
    for (int dl = 0; dl < AW; ++dl) acc[r][dl] = 0.f;
  __syncthreads();
  const int jlo = window > 0 ? (chunked ? (i / window) * window : max(0, i - window + 1)) : 0;
  const int nt = i - jlo + 1;
  const int nb = (!chunked && window > 0 && pool > 0 && i - window + 1 > 0) ? (i - window + 1) / pool : 0;
  const int kf = (!chunked && window > 0) ? min(keep_first, jlo) : 0;   // kept first tokens that lie before the window
  // key chunks [ci0, ci1) of this query belong to this workgroup (blockIdx.z of nsplit; 1: all of them)
  const int nchunks = (kf + KC - 1) / KC + (nt + KC - 1) / KC + (nb + KC - 1) / KC, cps = (nchunks + nsplit - 1) / nsplit;
  const int ci0 = blockIdx.z * cps, ci1 = min(nchunks, ci0 + cps);
  int ci = 0;
  for (int c0 = 0; c0 < kf; c0 += KC, ++ci) {
    if (ci < ci0 || ci >= ci1) continue;
    const int j = c0 + tid;
    const int rowidx = j < kf ? pt[j / page] * page + j % page : 0;
    attn_chunk<T, RMAX, DVL, VEC>(kp, vp, min(KC, kf - c0), g, kld, vld, D, Dv, R, q_s, s_s, row_s, m_s, l_s, a_s, rowidx, acc,
                                  cap, slopes ? sl_s : nullptr, i - j);
  }
  for (int c0 = 0; c0 < nt; c0 += KC, ++ci) {
    if (ci < ci0 || ci >= ci1) continue;
    const int j = jlo + c0 + tid;
    const int rowidx = c0 + tid < nt ? pt[j / page] * page + j % page : 0;
    attn_chunk<T, RMAX, DVL, VEC>(kp, vp, min(KC, nt - c0), g, kld, vld, D, Dv, R, q_s, s_s, row_s, m_s, l_s, a_s, rowidx, acc,
                                  cap, slopes ? sl_s : nullptr, i - j);
  }
  for (int c0 = 0; c0 < nb; c0 += KC, ++ci) {
    if (ci < ci0 || ci >= ci1) continue;
    const int p0 = (c0 + tid) * pool;
    const int rowidx = c0 + tid < nb ? pt[p0 / page] * PB + (p0 % page) / pool : 0;
    attn_chunk<float, RMAX, DVL, VEC>(kb, vb, min(KC, nb - c0), g, G * D, G * Dv, D, Dv, R, q_s, s_s, row_s, m_s, l_s, a_s, rowidx, acc);
  }
  // sum the four waves' partial outputs, normalise, gate
  if constexpr (VEC) {                                       // add up the lanes that walked different keys
    constexpr int LPK = 8 * DVL;
#pragma unroll
    for (int r = 0; r < RMAX; ++r)
#pragma unroll
      for (int e = 0; e < 8; ++e)
#pragma unroll
        for (int o = LPK; o < 64; o <<= 1) acc[r][e] += __shfl_xor(acc[r][e], o, 64);
  }
  for (int w = 0; w < NT / 64; ++w) {
    if (wave == w) {
      if constexpr (VEC) {
        constexpr int LPK = 8 * DVL;
        if (lane < LPK && lane * 8 < Dv) {
#pragma unroll
          for (int r = 0; r < RMAX; ++r)
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (r < R) red[r * Dv + lane * 8 + e] += acc[r][e];
        }
      } else {
#pragma unroll
        for (int r = 0; r < RMAX; ++r)
#pragma unroll
          for (int dl = 0; dl < DVL; ++dl)
            if (r < R && lane + 64 * dl < Dv) red[r * Dv + lane + 64 * dl] += acc[r][dl];
      }
    }
    __syncthreads();
  }
  if (nsplit > 1) {                                          // unnormalised sums, running max and sum per head
    float* dst = part + (((size_t)t * gridDim.y + blockIdx.y) * nsplit + blockIdx.z) * (RMAX * (Dv + 2));
    for (int e = tid; e < R * Dv; e += NT) dst[e] = red[e];
    if (tid < R) { dst[RMAX * Dv + tid] = m_s[tid]; dst[RMAX * Dv + RMAX + tid] = l_s[tid]; }
    return;
  }
  for (int e = tid; e < R * Dv; e += NT) {
    const int r = e / Dv, h = hq0 + r;
    float o = red[e] / l_s[r];
    if (gate) o *= sigmoidf_(ldf<T>(gate + (size_t)t * gate_ld + (gate_elem ? h * Dv + e % Dv : h)));
    stf<T>(out + ((size_t)t * H + h) * Dv + e % Dv, o);
  }
}


// sums the key-split partial results of attn_kernel: out = sum_z e^{m_z - M} acc_z / sum_z e^{m_z - M} l_z
template <typename T>
__global__ void __launch_bounds__(NT) attn_merge_kernel(const float* __restrict__ part, const T* __restrict__ gate,
                                                        int gate_ld, T* __restrict__ out, int H, int G, int Dv, int nsp,
                                                        int nsplit, int rmax, int gate_elem) {
  const int t = blockIdx.x, g = blockIdx.y / nsp, r0 = (blockIdx.y % nsp) * rmax;
  const int R = min(rmax, H / G - r0), hq0 = g * (H / G) + r0, stride = rmax * (Dv + 2);
  const float* src = part + ((size_t)t * gridDim.y + blockIdx.y) * nsplit * stride;
  for (int e = threadIdx.x; e < R * Dv; e += NT) {
    const int r = e / Dv;
    float M = -INFINITY;
    for (int z = 0; z < nsplit; ++z) M = fmaxf(M, src[z * stride + rmax * Dv + r]);
    float acc = 0.f, l = 0.f;
    for (int z = 0; z < nsplit; ++z) {
      const float mz = src[z * stride + rmax * Dv + r];
      const float wz = mz == -INFINITY ? 0.f : expf(mz - M);
      acc += wz * src[z * stride + e];
      l += wz * src[z * stride + rmax * Dv + rmax + r];
    }
    float o = acc / l;
    if (gate) o *= sigmoidf_(ldf<T>(gate + (size_t)t * gate_ld + (gate_elem ? (hq0 + r) * Dv + e % Dv : hq0 + r)));
    stf<T>(out + ((size_t)t * H + hq0 + r) * Dv + e % Dv, o);
  }
}

// ---------------------------------------------------------------------------------- attention, bf16 MFMA
// Prompt portions in bf16: 64 query rows of one (sequence, head) per workgroup, 16 per wave, on
// v_mfma_f32_16x16x32_bf16.  A key tile is one page of the sequence (64 tokens, rows G * D apart) or
// 64 pooled blocks (fp32 rows rounded to bf16 while staging); per tile S = Q K^T from a padded-row
// LDS image of K, the mask (window / block-complete rule) and the online softmax in fp32 in the
// log2 domain, P to per-wave LDS as bf16, O += P V with V fragments read transposed from the
// row-major V tile.  Tiles wholly outside a workgroup's window are never visited.
constexpr int MQ = 64, MK = 64;

// RH query heads of one kv head per workgroup: a staged key / value tile serves all of them
// (second launch bound: workgroups per CU the register budget must allow - four for 64-wide heads, so the
// 1024 workgroups of a 4096-token, 16-head prompt are resident at once)
// KVS: the value of a cached row is its first Dv numbers (a latent cache, or values that are the keys): the
// staged key tile serves as the value tile, nothing is loaded twice
// EXT: scores are capped (cap tanh(s / cap), cap > 0) and lose slopes[head] * distance; chunked: `window` is a
// chunk size (a query sees its own chunk's start .. itself), else a sliding window beside the sequence's first
// keep_first tokens; sink[head] joins the softmax denominator; the gate is [T, H * Dv], one per output coordinate
struct AttnExt {
  float scale, cap;
  const float* slopes;
  const float* sink;
  int chunked, keep_first;
};

template <int DK, int DV, int RH, bool KVS, bool EXT = false>
__global__ void __launch_bounds__(NT, (DV * RH <= 4 ? 4 : (DV * RH <= 8 ? 2 : 1))) attn_mfma_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ gate, int gate_ld, const bf16_t* __restrict__ kp,
    const bf16_t* __restrict__ vp, const float* __restrict__ kb, const float* __restrict__ vb,
    const int* __restrict__ seq_slot, const int* __restrict__ seq_start, const int* __restrict__ seq_len,
    const int* __restrict__ seq_off, const int* __restrict__ ptab, int ptab_ld, bf16_t* __restrict__ out, int n, int H,
    int G, int PB, float scale_log2, int window, int pool, int kld, int vld, AttnExt ext = AttnExt{}) {
  constexpr int D = 32 * DK, Dv = 16 * DV;
  constexpr float LOG2E = 1.4426950408889634f;
  constexpr int KS = D * 2 + 16, VS = KVS ? KS : Dv * 2 + 16, PS = MK * 2 + 16;      // LDS row strides in bytes
  static_assert(!KVS || Dv <= D, "a value slice lies inside the key row");
  __shared__ __attribute__((aligned(16))) char k_lds[MK * KS];
  __shared__ __attribute__((aligned(16))) char v_own[KVS ? 16 : MK * VS];
  char* const v_lds = KVS ? k_lds : v_own;
  __shared__ __attribute__((aligned(16))) char p_all[4 * 16 * PS];
  constexpr int NPID = 1024;
  __shared__ int pid_s[NPID];                                // the sequence's first page ids (one global hop per tile less)
  typedef __attribute__((address_space(3))) v4s lds_v4s;
  int qt = blockIdx.x, s = 0;
  for (; s < n; ++s) {
    const int nq = (seq_len[s] + MQ - 1) / MQ;
    if (qt < nq) break;
    qt -= nq;
  }
  if (s == n) return;
  const int h0 = blockIdx.y * RH, g = h0 / (H / G);
  const int start = seq_start[s], len = seq_len[s], off = seq_off[s];
  const int* pt = ptab + (size_t)seq_slot[s] * ptab_ld;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g4 = lane >> 4, c16 = lane & 15;
  char* p_lds = p_all + wave * 16 * PS;
  const int wq0 = qt * MQ + wave * 16;                       // this wave's first row inside the portion
  v8s qf[RH][DK];
  {
    const int t = wq0 + c16;
#pragma unroll
    for (int r = 0; r < RH; ++r)
#pragma unroll
      for (int kk = 0; kk < DK; ++kk)
        qf[r][kk] = t < len ? *reinterpret_cast<const v8s*>(q + ((size_t)(off + t) * H + h0 + r) * D + kk * 32 + 8 * g4)
                            : v8s{0, 0, 0, 0, 0, 0, 0, 0};
  }
  v4f o[RH][DV];
  float m_i[RH][4], l_i[RH][4];
#pragma unroll
  for (int r = 0; r < RH; ++r) {
#pragma unroll
    for (int i = 0; i < DV; ++i) o[r][i] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 4; ++i) { m_i[r][i] = -INFINITY; l_i[r][i] = 0.f; }
  }
  // EXT: a score in the log2 domain is c1 - c2 / (2^(xs s) + 1) - sl2 (i - j)  (cap tanh(x / cap) written with one
  // exp2 and one rcp; no cap: s scale_log2 - sl2 (i - j)); clo = first position of each row's chunk
  float sl2[RH];
  int clo[4];
  const float c1 = ext.cap * LOG2E, c2 = 2.f * ext.cap * LOG2E, xs = ext.cap > 0.f ? ext.scale * 2.f * LOG2E / ext.cap : 0.f;
#pragma unroll
  for (int r = 0; r < RH; ++r) sl2[r] = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) clo[i] = 0;
  if constexpr (EXT) {
    if (window > 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int qpos = start + wq0 + 4 * g4 + i;
        clo[i] = ext.chunked ? (qpos / window) * window : max(0, qpos - window + 1);
      }
    }
#pragma unroll
    for (int r = 0; r < RH; ++r) {
      if (ext.slopes) sl2[r] = ext.slopes[h0 + r] * LOG2E;
      if (ext.sink) {                                        // the sink: a starting maximum with sum 1 and no value
#pragma unroll
        for (int i = 0; i < 4; ++i) { m_i[r][i] = ext.sink[h0 + r] * LOG2E; l_i[r][i] = 1.f; }
      }
    }
  }
  const int imin = start + qt * MQ, imax = start + min(len, qt * MQ + MQ) - 1;
  const int jlo = window > 0 ? ((EXT && ext.chunked) ? (imin / window) * window : max(0, imin - window + 1)) : 0;
  const int nbmax = (window > 0 && pool > 0 && imax - window + 1 > 0) ? (imax - window + 1) / pool : 0;
  // the tiles that hold kept first tokens and lie wholly before the window's first tile come first
  const int nfirst = (EXT && window > 0 && !ext.chunked) ? min((ext.keep_first + MK - 1) / MK, jlo / MK) : 0;
  const int tok_tiles = nfirst + imax / MK - jlo / MK + 1, ntiles = tok_tiles + (nbmax + MK - 1) / MK;
  auto tile_base = [&](int tile) {                           // first position (token tiles) / block (pooled tiles) of a tile
    return tile < nfirst ? tile * MK : tile < tok_tiles ? (jlo / MK + tile - nfirst) * MK : (tile - tok_tiles) * MK;
  };
  for (int i = tid; i < min(imax / MK + 1, NPID); i += NT) pid_s[i] = pt[i];
  __syncthreads();
  auto page_of = [&](int idx) { return idx < NPID ? pid_s[idx] : pt[idx]; };

  // a tile's rows travel global -> registers while the tile before it computes, registers -> LDS
  // between the two barriers
  static_assert(DV % 2 == 0, "value chunks per thread");
  constexpr int KL = DK, VL = KVS ? 0 : DV / 2;              // 16-byte chunks per thread per tile
  uint4 kreg[KL], vreg[VL > 0 ? VL : 1];
  auto load_tile = [&](int tile) {
    const bool tok = tile < tok_tiles;
    const int base = tile_base(tile);
    const size_t prow = tok ? (size_t)page_of(base / MK) * MK : 0;
#pragma unroll
    for (int i = 0; i < KL + VL; ++i) {
      const bool isk = i < KL;
      const int e = tid + (isk ? i : i - KL) * NT, cpr = isk ? D / 8 : Dv / 8;
      const int r = e / cpr, c = e % cpr;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (tok) {
        v = isk ? *reinterpret_cast<const uint4*>(kp + (prow + r) * kld + g * D + c * 8)
                : *reinterpret_cast<const uint4*>(vp + (prow + r) * vld + g * Dv + c * 8);
      } else if (base + r < nbmax) {
        const int p0 = (base + r) * pool;
        const size_t row = ((size_t)page_of(p0 / MK) * PB + (p0 % MK) / pool) * G + g;
        float f[8];
        load8<float>(isk ? kb + row * D + c * 8 : vb + row * Dv + c * 8, f);
        v = pack8(f);
      }
      if (isk) kreg[i] = v;
      else vreg[VL > 0 ? i - KL : 0] = v;
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < KL; ++i) {
      const int e = tid + i * NT;
      *reinterpret_cast<uint4*>(k_lds + (e / (D / 8)) * KS + (e % (D / 8)) * 16) = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < VL; ++i) {
      const int e = tid + i * NT;
      *reinterpret_cast<uint4*>(v_lds + (e / (Dv / 8)) * VS + (e % (Dv / 8)) * 16) = vreg[i];
    }
  };
  if (ntiles > 0) load_tile(0);
  for (int tile = 0; tile < ntiles; ++tile) {
    const bool tok = tile < tok_tiles;
    const int base = tile_base(tile);
    __syncthreads();                                         // every wave is done with the previous tile
    store_tile();
    __syncthreads();
    if (tile + 1 < ntiles) load_tile(tile + 1);
#pragma unroll
    for (int r = 0; r < RH; ++r) {
    v4f sc[4];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt) {
      sc[nt] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kk = 0; kk < DK; ++kk) {
        const v8s kf = *reinterpret_cast<const v8s*>(k_lds + (nt * 16 + c16) * KS + (kk * 32 + 8 * g4) * 2);
        sc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[r][kk], kf, sc[nt], 0, 0, 0);
      }
    }
    // lane holds S[row = 4 g4 + i][key = 16 nt + c16]
    float alpha[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int qpos = start + wq0 + 4 * g4 + i;
      const int seen = (window > 0 && pool > 0 && qpos - window + 1 > 0) ? (qpos - window + 1) / pool : 0;
      float mx = -INFINITY;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const int key = base + nt * 16 + c16;
        bool vis;
        float v;
        if constexpr (EXT) {
          vis = key <= qpos && (key >= clo[i] || key < ext.keep_first);
          const float bias = sl2[r] * (float)(qpos - key);
          if (ext.cap > 0.f)                                 // 2^(xs s) = inf gives the cap itself, 0 gives -cap
            v = c1 - c2 * __builtin_amdgcn_rcpf(__builtin_amdgcn_exp2f(sc[nt][i] * xs) + 1.f) - bias;
          else
            v = sc[nt][i] * scale_log2 - bias;
          v = vis ? v : -INFINITY;
        } else {
          vis = tok ? (key <= qpos && (window <= 0 || qpos - key < window)) : key < seen;
          v = vis ? sc[nt][i] * scale_log2 : -INFINITY;
        }
        sc[nt][i] = v;
        mx = fmaxf(mx, v);
      }
#pragma unroll
      for (int o_ = 1; o_ < 16; o_ <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o_, 64));
      const float mnew = fmaxf(m_i[r][i], mx);
      const float msafe = (mnew == -INFINITY) ? 0.f : mnew;
      alpha[i] = __builtin_amdgcn_exp2f(m_i[r][i] - msafe);
      float rs = 0.f;
#pragma unroll
      for (int nt = 0; nt < 4; ++nt) {
        const float p = __builtin_amdgcn_exp2f(sc[nt][i] - msafe);
        sc[nt][i] = p;
        rs += p;
      }
#pragma unroll
      for (int o_ = 1; o_ < 16; o_ <<= 1) rs += __shfl_xor(rs, o_, 64);
      l_i[r][i] = l_i[r][i] * alpha[i] + rs;
      m_i[r][i] = mnew;
    }
#pragma unroll
    for (int dt = 0; dt < DV; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) o[r][dt][i] *= alpha[i];
#pragma unroll
    for (int nt = 0; nt < 4; ++nt)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        *reinterpret_cast<bf16_t*>(p_lds + (4 * g4 + i) * PS + (nt * 16 + c16) * 2) = f2bf(sc[nt][i]);
    __builtin_amdgcn_s_waitcnt(0xC07F);                      // lgkmcnt(0): this wave's P rows are in LDS
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const v8s pf = *reinterpret_cast<const v8s*>(p_lds + c16 * PS + (ks * 32 + 8 * g4) * 2);
      const int key0 = ks * 32 + 8 * g4, qq = c16 >> 2, pp = c16 & 3;
#pragma unroll
      for (int dt = 0; dt < DV; ++dt) {
        const char* a0 = v_lds + (key0 + qq) * VS + (dt * 16 + 4 * pp) * 2;
        const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)(a0));
        const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)(a0 + 4 * VS));
        const v8s vf = v8s{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        o[r][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vf, o[r][dt], 0, 0, 0);
      }
    }
      __builtin_amdgcn_wave_barrier();                     // this wave's P reads precede the next head's P writes
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int t = wq0 + 4 * g4 + i;
    if (t < len) {
#pragma unroll
      for (int r = 0; r < RH; ++r) {
        float inv = l_i[r][i] > 0.f ? 1.f / l_i[r][i] : 0.f;
        if constexpr (!EXT) {
          if (gate) inv *= sigmoidf_(bf2f(gate[(size_t)(off + t) * gate_ld + h0 + r]));
        }
#pragma unroll
        for (int dt = 0; dt < DV; ++dt) {
          float ov = o[r][dt][i] * inv;
          if constexpr (EXT) {
            if (gate) ov *= sigmoidf_(bf2f(gate[(size_t)(off + t) * gate_ld + (h0 + r) * Dv + dt * 16 + c16]));
          }
          out[((size_t)(off + t) * H + h0 + r) * Dv + dt * 16 + c16] = f2bf(ov);
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------- convolution
constexpr int MAX_TAPS = 16;

constexpr int TOKB = 16;                                     // tokens per workgroup on prompt-sized steps: weights are read once for all of them

template <typename T, bool VEC>
__global__ void __launch_bounds__(NT) conv_kernel(const T* __restrict__ u, int ld, int c0, int C,
                                                  const float* __restrict__ w, const float* __restrict__ bias,
                                                  const T* state, const int* __restrict__ tok_seq,
                                                  const int* __restrict__ tok_pos, const int* __restrict__ seq_slot,
                                                  const int* __restrict__ seq_start, const int* __restrict__ seq_off,
                                                  T* __restrict__ out, int taps, T* state_w, int rows, int tokb) {
  // state_w (steps in which every sequence brings one token: the thread of (token, channel) is the only
  // reader of that channel's tail): the tail is shifted here and no second launch follows
  const int t0 = blockIdx.x * tokb, t1 = min(rows, t0 + tokb);
  if constexpr (VEC) {                                       // eight channels per thread (ld, c0, C multiples of 8)
    for (int c = (blockIdx.y * NT + threadIdx.x) * 8; c < C; c += NT * gridDim.y * 8) {
      float br[8], wr[8][4];                                 // up to four taps stay in registers
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        br[e] = bias[c + e];
#pragma unroll
        for (int k = 0; k < 4; ++k) wr[e][k] = k < taps ? w[(c + e) * taps + k] : 0.f;
      }
      for (int t = t0; t < t1; ++t) {
        const int s = tok_seq[t], pos = tok_pos[t], start = seq_start[s], off = seq_off[s];
        const T* st = state + (size_t)seq_slot[s] * (taps - 1) * C;
        T* stw = state_w ? state_w + (size_t)seq_slot[s] * (taps - 1) * C : nullptr;
        float acc[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = br[e];
        for (int k0 = 0; k0 < taps; k0 += 4) {               // four taps' rows in flight
          float x[4][8];
#pragma unroll
          for (int kk = 0; kk < 4; ++kk) {
            const int k = k0 + kk, p = pos - (taps - 1) + k;
            if (k < taps && p >= start) load8<T>(u + (size_t)(off + p - start) * ld + c0 + c, x[kk]);
            else if (k < taps && p >= 0) load8<T>(st + (size_t)(p - (start - (taps - 1))) * C + c, x[kk]);
            else {
#pragma unroll
              for (int e = 0; e < 8; ++e) x[kk][e] = 0.f;
            }
          }
#pragma unroll
          for (int kk = 0; kk < 4; ++kk) {
            if (k0 + kk < taps) {
#pragma unroll
              for (int e = 0; e < 8; ++e)
                acc[e] += (k0 == 0 ? wr[e][kk] : w[(c + e) * taps + k0 + kk]) * x[kk][e];
              // the new tail = inputs of positions pos - (taps - 2) .. pos = taps 1 .. taps - 1 of this window
              if (stw && k0 + kk >= 1) store8<T>(stw + (size_t)(k0 + kk - 1) * C + c, x[kk]);
            }
          }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] = siluf_(acc[e]);
        store8<T>(out + (size_t)t * C + c, acc);
      }
    }
  } else {
    for (int t = t0; t < t1; ++t) {
      const int s = tok_seq[t], pos = tok_pos[t], start = seq_start[s], off = seq_off[s];
      const T* st = state + (size_t)seq_slot[s] * (taps - 1) * C;
      T* stw = state_w ? state_w + (size_t)seq_slot[s] * (taps - 1) * C : nullptr;
      for (int c = blockIdx.y * NT + threadIdx.x; c < C; c += NT * gridDim.y) {
        float acc = bias[c];
        for (int k = 0; k < taps; ++k) {
          const int p = pos - (taps - 1) + k;
          float x = 0.f;
          if (p >= start) x = ldf<T>(u + (size_t)(off + p - start) * ld + c0 + c);
          else if (p >= 0) x = ldf<T>(st + (size_t)(p - (start - (taps - 1))) * C + c);
          acc += w[c * taps + k] * x;
          if (stw && k >= 1) stf<T>(stw + (size_t)(k - 1) * C + c, x);
        }
        stf<T>(out + (size_t)t * C + c, siluf_(acc));
      }
    }
  }
}

// the inputs of each sequence's last taps - 1 positions, in position order
template <typename T>
__global__ void __launch_bounds__(NT) conv_state_kernel(const T* __restrict__ u, int ld, int c0, int C,
                                                        T* __restrict__ state, const int* __restrict__ seq_slot,
                                                        const int* __restrict__ seq_start,
                                                        const int* __restrict__ seq_len, const int* __restrict__ seq_off,
                                                        int taps) {
  const int s = blockIdx.x;
  const int start = seq_start[s], end = start + seq_len[s], off = seq_off[s];
  T* st = state + (size_t)seq_slot[s] * (taps - 1) * C;
  for (int c = blockIdx.y * NT + threadIdx.x; c < C; c += NT * gridDim.y) {
    T keep[MAX_TAPS];
#pragma unroll
    for (int k = 0; k < MAX_TAPS; ++k) {
      if (k < taps - 1) {
        const int p = end - (taps - 1) + k;
        T v = T(0);                                       // bit pattern 0 = 0.0 in both storage types
        if (p >= start) v = u[(size_t)(off + p - start) * ld + c0 + c];
        else if (p >= 0) v = st[(size_t)(p - (start - (taps - 1))) * C + c];
        keep[k] = v;
      }
    }
#pragma unroll
    for (int k = 0; k < MAX_TAPS; ++k)
      if (k < taps - 1) st[(size_t)k * C + c] = keep[k];
  }
}

// ---------------------------------------------------------------------------------- state-space recurrence
// One wave per (sequence, head, 64 value columns); lane = column p holds S[0..N)[p] in registers.
// Tokens are staged TC at a time (B, C rows, step size and decay in LDS), then stepped in order.
constexpr int TC = 16;

template <typename T, int NMAX>
__global__ void __launch_bounds__(64) ssd_kernel(const T* __restrict__ xbc, int Cx, const T* __restrict__ u, int ld,
                                                 int dt0, const float* __restrict__ dt_bias,
                                                 const float* __restrict__ A_log, const float* __restrict__ Dp,
                                                 float* __restrict__ state, const int* __restrict__ seq_slot,
                                                 const int* __restrict__ seq_start, const int* __restrict__ seq_len,
                                                 const int* __restrict__ seq_off, float* __restrict__ y, int Hs, int P,
                                                 int N, int groups) {
  __shared__ float B_s[TC][NMAX], C_s[TC][NMAX], dt_s[TC], dec_s[TC];
  const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, p = blockIdx.z * 64 + tid;
  const int start = seq_start[s], len = seq_len[s], off = seq_off[s];
  const int g = h / (Hs / groups), inner = Hs * P;
  float* st = state + ((size_t)seq_slot[s] * Hs + h) * N * P;
  float S[NMAX];
#pragma unroll
  for (int n = 0; n < NMAX; ++n) S[n] = (start > 0 && n < N && p < P) ? st[(size_t)n * P + p] : 0.f;
  const float a = expf(A_log[h]), Dh = Dp[h], bias = dt_bias[h];
  if (len == 1) {
    // one token (decode): no staging; B, C, x, the step size and the state rows are independent loads
    if (p < P) {
      const size_t row = (size_t)off;
      const float raw = ldf<T>(u + row * ld + dt0 + h) + bias;
      const float dt = raw > 20.f ? raw : log1pf(expf(raw));
      const float dec = expf(-a * dt), xv = ldf<T>(xbc + row * Cx + h * P + p), dx = dt * xv;
      const T* bc = xbc + row * Cx + inner + g * N;
      float yv = 0.f;
#pragma unroll
      for (int n = 0; n < NMAX; ++n) {
        if (n < N) {
          const float Sn = dec * S[n] + ldf<T>(bc + n) * dx;
          yv += Sn * ldf<T>(bc + groups * N + n);
          st[(size_t)n * P + p] = Sn;
        }
      }
      y[row * inner + h * P + p] = yv + Dh * xv;
    }
    return;
  }
  for (int t0 = 0; t0 < len; t0 += TC) {
    const int tc = min(TC, len - t0);
    __syncthreads();
    for (int e = tid; e < tc * NMAX; e += 64) {
      const int tt = e / NMAX, n = e % NMAX;
      const T* row = xbc + (size_t)(off + t0 + tt) * Cx + inner + g * N;
      B_s[tt][n] = n < N ? ldf<T>(row + n) : 0.f;
      C_s[tt][n] = n < N ? ldf<T>(row + groups * N + n) : 0.f;
    }
    if (tid < tc) {
      const float raw = ldf<T>(u + (size_t)(off + t0 + tid) * ld + dt0 + h) + bias;
      const float dt = raw > 20.f ? raw : log1pf(expf(raw));
      dt_s[tid] = dt;
      dec_s[tid] = expf(-a * dt);
    }
    __syncthreads();
    if (p < P) {
      for (int tt = 0; tt < tc; ++tt) {
        const size_t row = (size_t)(off + t0 + tt);
        const float xv = ldf<T>(xbc + row * Cx + h * P + p);
        const float dx = dt_s[tt] * xv, dec = dec_s[tt];
        float yv = 0.f;
#pragma unroll
        for (int n = 0; n < NMAX; ++n) {
          S[n] = dec * S[n] + B_s[tt][n] * dx;
          yv += S[n] * C_s[tt][n];
        }
        y[row * inner + h * P + p] = yv + Dh * xv;
      }
    }
  }
  if (p < P) {
#pragma unroll
    for (int n = 0; n < NMAX; ++n)
      if (n < N) st[(size_t)n * P + p] = S[n];
  }
}


// ---------------------------------------------------------------------------------- chunked recurrence
// The same recurrence for long portions, in chunks of CL tokens (state-space duality): with
// la_t = -exp(A_log) * (dt_1 + .. + dt_t) inside a chunk,
//   S_t = e^{la_t} S_in + sum_{s<=t} e^{la_t - la_s} dt_s B_s x_s^T
//   y_t = e^{la_t} C_t^T S_in + sum_{s<=t} (C_t . B_s) e^{la_t - la_s} dt_s x_s + D x_t
// (1) every chunk's own contribution to its end state, all chunks in parallel; (2) the states at
// the chunk borders, one short pass per sequence; (3) every chunk's outputs, all chunks in parallel.
// All fp32 FMAs; every exponent is <= 0.
constexpr int CL = 64;

__device__ __forceinline__ int chunk_base(const int* __restrict__ seq_len, int s) {
  int b = 0;
  for (int i = 0; i < s; ++i) b += (seq_len[i] + CL - 1) / CL;
  return b;
}

// step sizes and inclusive log-decay of one chunk into LDS (first wave; tc <= 64 tokens)
template <typename T>
__device__ __forceinline__ void chunk_steps(const T* __restrict__ u, int ld, int dt0, int h, float bias, float a,
                                            size_t row0, int tc, float* dt_s, float* la_s) {
  if (threadIdx.x < 64) {
    const int t = threadIdx.x;
    float dt = 0.f;
    if (t < tc) {
      const float raw = ldf<T>(u + (row0 + t) * ld + dt0 + h) + bias;
      dt = raw > 20.f ? raw : log1pf(expf(raw));
    }
    float v = -a * dt;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const float w = __shfl_up(v, o, 64);
      if (t >= o) v += w;
    }
    dt_s[t] = dt;
    la_s[t] = v;
  }
}

// (1) Sloc[n][p] = sum_s e^{la_end - la_s} dt_s B_s[n] x_s[p] for one 64 x 64 tile of (n, p)
template <typename T>
__global__ void __launch_bounds__(NT) ssd_chunk_state_kernel(
    const T* __restrict__ xbc, int Cx, const T* __restrict__ u, int ld, int dt0, const float* __restrict__ dt_bias,
    const float* __restrict__ A_log, const int* __restrict__ seq_len, const int* __restrict__ seq_off,
    float* __restrict__ sloc, float* __restrict__ cdec, int Hs, int P, int N, int groups, int ntn, int ntp) {
  __shared__ float dt_s[CL], la_s[CL], B_s[CL][CL + 1], X_s[CL][CL + 1];
  const int tile = blockIdx.x % (ntn * ntp), c = blockIdx.x / (ntn * ntp), s = blockIdx.y, h = blockIdx.z;
  const int len = seq_len[s];
  if (c * CL >= len) return;
  const int tc = min(CL, len - c * CL), n0 = (tile / ntp) * CL, p0 = (tile % ntp) * CL;
  const size_t row0 = (size_t)seq_off[s] + (size_t)c * CL;
  const int g = h / (Hs / groups), inner = Hs * P, tid = threadIdx.x;
  chunk_steps<T>(u, ld, dt0, h, dt_bias[h], expf(A_log[h]), row0, tc, dt_s, la_s);
  __syncthreads();
  const float la_end = la_s[tc - 1];
  for (int e = tid; e < CL * CL; e += NT) {
    const int t = e / CL, j = e % CL;
    const bool ok = t < tc;
    B_s[t][j] = ok && n0 + j < N ? ldf<T>(xbc + (row0 + t) * Cx + inner + g * N + n0 + j) : 0.f;
    X_s[t][j] = ok && p0 + j < P ? ldf<T>(xbc + (row0 + t) * Cx + h * P + p0 + j) * (expf(la_end - la_s[t]) * dt_s[t]) : 0.f;
  }
  __syncthreads();
  const int ty = tid / 16, tx = tid % 16;
  float acc[4][4] = {};
  for (int t = 0; t < tc; ++t) {
    float b[4], x[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) { b[i] = B_s[t][ty * 4 + i]; x[i] = X_s[t][tx * 4 + i]; }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] += b[i] * x[j];
  }
  const size_t cb = (size_t)chunk_base(seq_len, s) + c;
  float* dst = sloc + (cb * Hs + h) * (size_t)N * P;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + ty * 4 + i, p = p0 + tx * 4 + j;
      if (n < N && p < P) dst[(size_t)n * P + p] = acc[i][j];
    }
  if (tile == 0 && tid == 0) cdec[cb * Hs + h] = expf(la_end);
}

// (2) the state entering every chunk (written over that chunk's own contribution) and the final state
__global__ void __launch_bounds__(NT) ssd_chunk_scan_kernel(float* __restrict__ sloc, const float* __restrict__ cdec,
                                                            float* __restrict__ state,
                                                            const int* __restrict__ seq_slot,
                                                            const int* __restrict__ seq_start,
                                                            const int* __restrict__ seq_len, int Hs, int NP) {
  const int s = blockIdx.x, h = blockIdx.y, e = blockIdx.z * NT + threadIdx.x;
  if (e >= NP) return;
  const int nc = (seq_len[s] + CL - 1) / CL;
  const size_t cb = chunk_base(seq_len, s);
  float* st = state + ((size_t)seq_slot[s] * Hs + h) * NP + e;
  float S = seq_start[s] > 0 ? *st : 0.f;
  for (int c = 0; c < nc; ++c) {
    float* q = sloc + ((cb + c) * Hs + h) * (size_t)NP + e;
    const float own = *q;
    *q = S;
    S = cdec[(cb + c) * Hs + h] * S + own;
  }
  *st = S;
}

// (3) y for one chunk and 64 value columns
template <typename T>
__global__ void __launch_bounds__(NT) ssd_chunk_out_kernel(
    const T* __restrict__ xbc, int Cx, const T* __restrict__ u, int ld, int dt0, const float* __restrict__ dt_bias,
    const float* __restrict__ A_log, const float* __restrict__ Dp, const int* __restrict__ seq_len,
    const int* __restrict__ seq_off, const float* __restrict__ sin_, float* __restrict__ y, int Hs, int P, int N,
    int groups, int ntp) {
  constexpr int NK = 32;
  __shared__ float dt_s[CL], la_s[CL], M_s[CL][CL + 1];
  __shared__ float buf[2 * CL * (NK + 1) + NK * CL];          // C tile | B tile | S_in tile; later the x tile
  float(*C_s)[NK + 1] = reinterpret_cast<float(*)[NK + 1]>(buf);
  float(*B_s)[NK + 1] = reinterpret_cast<float(*)[NK + 1]>(buf + CL * (NK + 1));
  float(*S_s)[CL] = reinterpret_cast<float(*)[CL]>(buf + 2 * CL * (NK + 1));
  float(*X_s)[CL + 1] = reinterpret_cast<float(*)[CL + 1]>(buf);
  static_assert(CL * (CL + 1) <= 2 * CL * (NK + 1) + NK * CL, "x tile fits the staging buffer");
  const int pt = blockIdx.x % ntp, c = blockIdx.x / ntp, s = blockIdx.y, h = blockIdx.z;
  const int len = seq_len[s];
  if (c * CL >= len) return;
  const int tc = min(CL, len - c * CL), p0 = pt * CL;
  const size_t row0 = (size_t)seq_off[s] + (size_t)c * CL;
  const int g = h / (Hs / groups), inner = Hs * P, tid = threadIdx.x, ty = tid / 16, tx = tid % 16;
  chunk_steps<T>(u, ld, dt0, h, dt_bias[h], expf(A_log[h]), row0, tc, dt_s, la_s);
  const float* sin_c = sin_ + (((size_t)chunk_base(seq_len, s) + c) * Hs + h) * (size_t)N * P;
  float accm[4][4] = {}, acci[4][4] = {};
  for (int n0 = 0; n0 < N; n0 += NK) {
    __syncthreads();
    for (int e = tid; e < CL * NK; e += NT) {
      const int t = e / NK, j = e % NK;
      const bool ok = t < tc && n0 + j < N;
      const T* row = xbc + (row0 + t) * Cx + inner + g * N + n0 + j;
      B_s[t][j] = ok ? ldf<T>(row) : 0.f;
      C_s[t][j] = ok ? ldf<T>(row + groups * N) : 0.f;
    }
    for (int e = tid; e < NK * CL; e += NT) {
      const int j = e / CL, p = e % CL;
      S_s[j][p] = n0 + j < N && p0 + p < P ? sin_c[(size_t)(n0 + j) * P + p0 + p] : 0.f;
    }
    __syncthreads();
#pragma unroll 4
    for (int k = 0; k < NK; ++k) {
      float cv[4], bv[4], sv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) { cv[i] = C_s[ty * 4 + i][k]; bv[i] = B_s[tx * 4 + i][k]; sv[i] = S_s[k][tx * 4 + i]; }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) { accm[i][j] += cv[i] * bv[j]; acci[i][j] += cv[i] * sv[j]; }
    }
  }
  // M[t][s'] = (C_t . B_s') e^{la_t - la_s'} dt_s' for s' <= t
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int t = ty * 4 + i, sp = tx * 4 + j;
      M_s[t][sp] = (sp <= t && t < tc) ? accm[i][j] * expf(la_s[t] - la_s[sp]) * dt_s[sp] : 0.f;
    }
  __syncthreads();                                            // every wave is done with the C / B / S_in tiles
  for (int e = tid; e < CL * CL; e += NT) {
    const int t = e / CL, p = e % CL;
    X_s[t][p] = t < tc && p0 + p < P ? ldf<T>(xbc + (row0 + t) * Cx + h * P + p0 + p) : 0.f;
  }
  __syncthreads();
  float out[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float el = expf(la_s[ty * 4 + i]);
#pragma unroll
    for (int j = 0; j < 4; ++j) out[i][j] = el * acci[i][j];
  }
  for (int sp = 0; sp < tc; ++sp) {
    float mv[4], xv[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) { mv[i] = M_s[ty * 4 + i][sp]; xv[i] = X_s[sp][tx * 4 + i]; }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) out[i][j] += mv[i] * xv[j];
  }
  const float Dh = Dp[h];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int t = ty * 4 + i, p = p0 + tx * 4 + j;
      if (t < tc && p < P) y[(row0 + t) * inner + h * P + p] = out[i][j] + Dh * X_s[t][tx * 4 + j];
    }
}

}  // namespace

#define SM_T(f32, ...)                                  \
  do {                                                  \
    if (f32) { using T = float; __VA_ARGS__; }          \
    else { using T = bf16_t; __VA_ARGS__; }             \
  } while (0)

extern "C" {

int edge_sm_embed(const int64_t* ids, const void* table, float* out, int rows, int W, int V, float scale, int f32,
                  hipStream_t st) {
  if (rows == 0) return 0;
  SM_T(f32, hipLaunchKernelGGL(embed_kernel<T>, dim3(rows), dim3(NT), 0, st, ids, (const T*)table, out, W, V, scale));
  return (int)hipGetLastError();
}

int edge_sm_scalar_norm(const float* x, const float* gain, void* y, int rows, int W, float eps, int f32,
                        hipStream_t st) {
  if (rows == 0) return 0;
  SM_T(f32, hipLaunchKernelGGL(scalar_norm_kernel<T>, dim3(rows), dim3(NT), 0, st, x, gain, (T*)y, W, eps));
  return (int)hipGetLastError();
}

int edge_sm_relu2(const void* u, int ld, int c0, void* y, int rows, int C, int f32, hipStream_t st) {
  if (rows == 0 || C == 0) return 0;
  if (ld % 8 == 0 && c0 % 8 == 0 && C % 8 == 0) {
    const int gy = (C / 8 + NT - 1) / NT;
    SM_T(f32, hipLaunchKernelGGL((relu2_kernel<T, true>), dim3(rows, gy), dim3(NT), 0, st, (const T*)u, ld, c0, (T*)y, C));
  } else {
    const int gy = (C + NT * 4 - 1) / (NT * 4);
    SM_T(f32, hipLaunchKernelGGL((relu2_kernel<T, false>), dim3(rows, gy), dim3(NT), 0, st, (const T*)u, ld, c0, (T*)y, C));
  }
  return (int)hipGetLastError();
}

int edge_sm_cat_cast(const float* a, const float* b, void* y, int rows, int W, int f32, hipStream_t st) {
  if (rows == 0) return 0;
  SM_T(f32, hipLaunchKernelGGL(cat_cast_kernel<T>, dim3(rows), dim3(NT), 0, st, a, b, (T*)y, W));
  return (int)hipGetLastError();
}

int edge_sm_combine(float* x, const void* l, const void* r, const float* wl, const float* wr, const void* extra,
                    int rows, int W, float eps, int f32, hipStream_t st) {
  if (rows == 0) return 0;
  SM_T(f32, hipLaunchKernelGGL(combine_kernel<T>, dim3(rows), dim3(NT), 0, st, x, (const T*)l, (const T*)r, wl, wr,
                               (const T*)extra, W, eps));
  return (int)hipGetLastError();
}

int edge_sm_gated_norm(const float* y, const void* z, int z_ld, const float* w, void* out, int rows, int C, int groups,
                       float eps, int f32, hipStream_t st) {
  if (rows == 0) return 0;
  if (groups <= 0 || C % groups) return -2;
  SM_T(f32, hipLaunchKernelGGL(gated_norm_kernel<T>, dim3(rows, groups), dim3(NT), 0, st, y, (const T*)z, z_ld, w,
                               (T*)out, C, groups, eps));
  return (int)hipGetLastError();
}

int edge_sm_rope_write(const void* proj, int ld, const int* tok_seq, const int* tok_pos, const int* seq_slot,
                       const int* ptab, int ptab_ld, const float* cs, void* q_out, void* kp, void* vp, int rows,
                       int H, int G, int D, int Dv, int rot, int page, int f32, hipStream_t st) {
  if (rows == 0) return 0;
  if (rot % 2 || rot > D || (rot > 0 && !cs)) return -2;
  if (D % 8 == 0 && Dv % 8 == 0 && rot % 16 == 0 && ld % 8 == 0 && ((uintptr_t)proj & 31) == 0)
    SM_T(f32, hipLaunchKernelGGL((rope_write_kernel<T, true>), dim3(rows), dim3(NT), 0, st, (const T*)proj, ld, tok_seq,
                                 tok_pos, seq_slot, ptab, ptab_ld, cs, (T*)q_out, (T*)kp, (T*)vp, H, G, D, Dv, rot, page));
  else
    SM_T(f32, hipLaunchKernelGGL((rope_write_kernel<T, false>), dim3(rows), dim3(NT), 0, st, (const T*)proj, ld, tok_seq,
                                 tok_pos, seq_slot, ptab, ptab_ld, cs, (T*)q_out, (T*)kp, (T*)vp, H, G, D, Dv, rot, page));
  return (int)hipGetLastError();
}

int edge_sm_pool_blocks(const void* kp, const void* vp, float* kb, float* vb, const int* seq_slot,
                        const int* seq_start, const int* seq_len, const int* ptab, int ptab_ld, int n, int max_blocks,
                        int G, int D, int Dv, int page, int PB, int pool, int f32, hipStream_t st) {
  if (n == 0 || max_blocks <= 0) return 0;
  SM_T(f32, hipLaunchKernelGGL(pool_kernel<T>, dim3(n, max_blocks), dim3(NT), 0, st, (const T*)kp, (const T*)vp, kb, vb,
                               seq_slot, seq_start, seq_len, ptab, ptab_ld, G, D, Dv, page, PB, pool));
  return (int)hipGetLastError();
}

// nsplit > 1: the keys of every query are walked by nsplit workgroups (decode steps: few queries, long
// windows); part = fp32 scratch [rows, G * nsp, nsplit, rmax * (Dv + 2)] (edge_sm_attention_part_floats)
static size_t attn_lds_bytes(int rmax, int D, int Dv) {
  return sizeof(float) * ((size_t)rmax * D + (size_t)rmax * KC + (size_t)rmax * Dv + 4 * rmax) + sizeof(int) * KC;
}

// query heads of one kv head that share a workgroup: the whole group up to 16, fewer while their rows
// (queries, scores, partial outputs) would not fit 64 KB of LDS, and down to 4 while a step of few
// queries over few kv heads (decode steps over one latent head) would leave most CUs without a
// workgroup; 0: not even one head fits
int edge_sm_attention_rmax(int rows, int H, int G, int D, int Dv) {
  const int R = H / G;
  int rmax = R <= 1 ? 1 : R <= 2 ? 2 : R <= 4 ? 4 : R <= 8 ? 8 : 16;
  while (rmax > 1 && attn_lds_bytes(rmax, D, Dv) > 64 * 1024) rmax >>= 1;
  while (rmax > 4 && (long)rows * G * ((R + rmax - 1) / rmax) < 64) rmax >>= 1;
  return attn_lds_bytes(rmax, D, Dv) > 64 * 1024 ? 0 : rmax;
}

size_t edge_sm_attention_part_floats(int rows, int H, int G, int D, int Dv, int nsplit) {
  const int R = H / G, rmax = max(1, edge_sm_attention_rmax(rows, H, G, D, Dv)), nsp = (R + rmax - 1) / rmax;
  return (size_t)rows * G * nsp * nsplit * rmax * (Dv + 2);
}

int edge_sm_attention(const void* q, const void* gate, int gate_ld, const void* kp, const void* vp, const float* kb,
                      const float* vb, const int* tok_seq, const int* tok_pos, const int* seq_slot, const int* ptab,
                      int ptab_ld, void* out, int rows, int H, int G, int D, int Dv, int page, int PB, float scale,
                      int window, int pool, int f32, int nsplit, float* part, int kld, int vld, int chunked, float cap,
                      const float* slopes, const float* sink, int gate_elem, int keep_first, hipStream_t st) {
  if (rows == 0) return 0;
  if (G <= 0 || H % G || Dv > 512 || (chunked && pool > 0) || keep_first < 0) return -2;
  const int R = H / G;
  const int rmax = edge_sm_attention_rmax(rows, H, G, D, Dv);
  if (rmax == 0) return -3;
  const int nsp = (R + rmax - 1) / rmax;
  if (nsplit < 1 || (nsplit > 1 && !part)) return -2;
  const size_t lds = attn_lds_bytes(rmax, D, Dv);
  const bool vec = D % 8 == 0 && Dv % 8 == 0 && kld % 8 == 0 && vld % 8 == 0;
#define SM_ATT_V(RM, DL, V)                                                                                         \
  SM_T(f32, hipLaunchKernelGGL((attn_kernel<T, RM, DL, V>), dim3(rows, G * nsp, nsplit), dim3(NT), lds, st, (const T*)q,         \
                               (const T*)gate, gate_ld, (const T*)kp, (const T*)vp, kb, vb, tok_seq, tok_pos,       \
                               seq_slot, ptab, ptab_ld, (T*)out, H, G, D, Dv, page, PB, scale, window, pool, nsp, nsplit, part, \
                               kld, vld, chunked, cap, slopes, sink, gate_elem, keep_first))
#define SM_ATT(RM, DL)               \
  do {                               \
    if (vec) SM_ATT_V(RM, DL, true); \
    else SM_ATT_V(RM, DL, false);    \
  } while (0)
#define SM_ATT_R(DL)                 \
  switch (rmax) {                    \
    case 1: SM_ATT(1, DL); break;    \
    case 2: SM_ATT(2, DL); break;    \
    case 4: SM_ATT(4, DL); break;    \
    case 8: SM_ATT(8, DL); break;    \
    default: SM_ATT(16, DL); break;  \
  }
  if (Dv <= 64) { SM_ATT_R(1); }
  else if (Dv <= 128) { SM_ATT_R(2); }
  else if (Dv <= 256) { SM_ATT_R(4); }
  else { SM_ATT_R(8); }
#undef SM_ATT_R
#undef SM_ATT
#undef SM_ATT_V
  if (nsplit > 1)
    SM_T(f32, hipLaunchKernelGGL(attn_merge_kernel<T>, dim3(rows, G * nsp), dim3(NT), 0, st, part, (const T*)gate, gate_ld,
                                 (T*)out, H, G, Dv, nsp, nsplit, rmax, gate_elem));
  return (int)hipGetLastError();
}

int edge_sm_conv_silu(const void* u, int ld, int c0, int C, const float* w, const float* bias, void* state,
                      const int* tok_seq, const int* tok_pos, const int* seq_slot, const int* seq_start,
                      const int* seq_len, const int* seq_off, void* out, int rows, int n, int taps, int f32,
                      int max_len, hipStream_t st) {
  if (rows == 0) return 0;
  if (taps < 1 || taps > MAX_TAPS) return -2;
  const bool one = max_len == 1 && taps > 1;                 // every sequence brings one token
  const int tokb = rows >= 64 * TOKB ? TOKB : 1;             // decode-sized steps: one token per workgroup
  const int gy = (C + NT - 1) / NT;
  if (ld % 8 == 0 && c0 % 8 == 0 && C % 8 == 0)
    SM_T(f32, hipLaunchKernelGGL((conv_kernel<T, true>), dim3((rows + tokb - 1) / tokb, (C / 8 + NT - 1) / NT), dim3(NT),
                                 0, st, (const T*)u, ld, c0, C, w, bias, (const T*)state, tok_seq, tok_pos, seq_slot,
                                 seq_start, seq_off, (T*)out, taps, one ? (T*)state : (T*)nullptr, rows, tokb));
  else
    SM_T(f32, hipLaunchKernelGGL((conv_kernel<T, false>), dim3((rows + tokb - 1) / tokb, gy), dim3(NT), 0, st,
                                 (const T*)u, ld, c0, C, w, bias, (const T*)state, tok_seq, tok_pos, seq_slot, seq_start,
                                 seq_off, (T*)out, taps, one ? (T*)state : (T*)nullptr, rows, tokb));
  if (taps > 1 && !one)
    SM_T(f32, hipLaunchKernelGGL(conv_state_kernel<T>, dim3(n, gy), dim3(NT), 0, st, (const T*)u, ld, c0, C, (T*)state,
                                 seq_slot, seq_start, seq_len, seq_off, taps));
  return (int)hipGetLastError();
}

int edge_sm_ssd_scan(const void* xbc, int Cx, const void* u, int ld, int dt0, const float* dt_bias, const float* A_log,
                     const float* Dp, float* state, const int* seq_slot, const int* seq_start, const int* seq_len,
                     const int* seq_off, float* y, int n, int Hs, int P, int N, int groups, int f32, hipStream_t st) {
  if (n == 0) return 0;
  if (N > 256 || groups <= 0 || Hs % groups) return -2;
  const dim3 grid(n, Hs, (P + 63) / 64);
#define SM_SSD(NM)                                                                                                  \
  SM_T(f32, hipLaunchKernelGGL((ssd_kernel<T, NM>), grid, dim3(64), 0, st, (const T*)xbc, Cx, (const T*)u, ld, dt0, \
                               dt_bias, A_log, Dp, state, seq_slot, seq_start, seq_len, seq_off, y, Hs, P, N, groups))
  if (N <= 16) SM_SSD(16);
  else if (N <= 32) SM_SSD(32);
  else if (N <= 64) SM_SSD(64);
  else if (N <= 128) SM_SSD(128);
  else SM_SSD(256);
#undef SM_SSD
  return (int)hipGetLastError();
}

// chunked form for long portions: scratch sloc [chunks, Hs, N, P] and cdec [chunks, Hs] (fp32);
// chunks = sum over sequences of ceil(len / 64), max_chunks = the largest of them
int edge_sm_ssd_chunked(const void* xbc, int Cx, const void* u, int ld, int dt0, const float* dt_bias,
                        const float* A_log, const float* Dp, float* state, const int* seq_slot, const int* seq_start,
                        const int* seq_len, const int* seq_off, float* y, float* sloc, float* cdec, int n,
                        int max_chunks, int Hs, int P, int N, int groups, int f32, hipStream_t st) {
  if (n == 0 || max_chunks <= 0) return 0;
  if (groups <= 0 || Hs % groups) return -2;
  const int ntn = (N + CL - 1) / CL, ntp = (P + CL - 1) / CL;
  SM_T(f32, hipLaunchKernelGGL(ssd_chunk_state_kernel<T>, dim3(max_chunks * ntn * ntp, n, Hs), dim3(NT), 0, st,
                               (const T*)xbc, Cx, (const T*)u, ld, dt0, dt_bias, A_log, seq_len, seq_off, sloc, cdec, Hs,
                               P, N, groups, ntn, ntp));
  hipLaunchKernelGGL(ssd_chunk_scan_kernel, dim3(n, Hs, (N * P + NT - 1) / NT), dim3(NT), 0, st, sloc, cdec, state,
                     seq_slot, seq_start, seq_len, Hs, N * P);
  SM_T(f32, hipLaunchKernelGGL(ssd_chunk_out_kernel<T>, dim3(max_chunks * ntp, n, Hs), dim3(NT), 0, st, (const T*)xbc,
                               Cx, (const T*)u, ld, dt0, dt_bias, A_log, Dp, seq_len, seq_off, sloc, y, Hs, P, N, groups,
                               ntp));
  return (int)hipGetLastError();
}

// bf16 prompt portions on the matrix cores; returns 1 when no instantiation takes (D, Dv): the caller
// then runs the general kernel
int edge_sm_attention_mfma(const void* q, const void* gate, int gate_ld, const void* kp, const void* vp,
                           const float* kb, const float* vb, const int* seq_slot, const int* seq_start,
                           const int* seq_len, const int* seq_off, const int* ptab, int ptab_ld, void* out, int n,
                           int qtiles, int H, int G, int D, int Dv, int page, int PB, float scale, int window,
                           int pool, int kld, int vld, int chunked, float cap, const float* slopes, const float* sink,
                           int gate_elem, int keep_first, hipStream_t st) {
  if (page != MK || G <= 0 || H % G || kld % 8 || vld % 8) return 1;
  const bool extras = chunked || cap > 0.f || slopes || sink || gate_elem || keep_first > 0;
  if (n == 0 || qtiles == 0) return 0;
  const float sl2 = scale * 1.4426950408889634f;
  // query heads per workgroup: a staged tile can serve 4 or 2 heads of a kv group, but the kernel is
  // bound by each wave's MFMA -> softmax -> LDS -> MFMA chain and needs ~4 waves per SIMD to hide it
  // (4096-token prompt, 16 heads: 111 us with one head per workgroup, 190 us with four), so heads are
  // grouped only while >= 1024 workgroups remain
  const int R = H / G;
  int rh = 1;
  if (R % 4 == 0 && (long)qtiles * (H / 4) >= 1024) rh = 4;
  else if (R % 2 == 0 && (long)qtiles * (H / 2) >= 1024) rh = 2;
  const bool kvs = kp == vp && kld == vld;
  if (kvs && pool > 0) return 1;                             // pooled entries keep separate key / value rows
  if (extras) {
    // the capped / biased / chunked / sink / kept-first-tokens form: an element-wise gate or none, no pooled blocks
    if ((kvs && D != Dv) || pool > 0 || (gate && !gate_elem)) return 1;
    const AttnExt ext{scale, cap, slopes, sink, chunked, (chunked || window <= 0) ? 0 : keep_first};
#define SM_MFX_R(DK, DV, RH) SM_MFX_RK(DK, DV, RH, true)
#define SM_MFX_RK(DK, DV, RH, KVS)                                                                                   \
  hipLaunchKernelGGL((attn_mfma_kernel<DK, DV, RH, KVS, true>), dim3(qtiles, H / RH), dim3(NT), 0, st,               \
                     (const bf16_t*)q, (const bf16_t*)gate, gate_ld, (const bf16_t*)kp, (const bf16_t*)vp, kb, vb,   \
                     seq_slot, seq_start, seq_len, seq_off, ptab, ptab_ld, (bf16_t*)out, n, H, G, PB, sl2, window,   \
                     pool, kld, vld, ext)
#define SM_MFX(DK, DV)                    \
  do {                                    \
    if (rh == 4) SM_MFX_R(DK, DV, 4);     \
    else if (rh == 2) SM_MFX_R(DK, DV, 2);\
    else SM_MFX_R(DK, DV, 1);             \
  } while (0)
#define SM_MFXS(DK, DV)                          \
  do {                                           \
    if (rh == 4) SM_MFX_RK(DK, DV, 4, false);    \
    else if (rh == 2) SM_MFX_RK(DK, DV, 2, false);\
    else SM_MFX_RK(DK, DV, 1, false);            \
  } while (0)
    if (kvs) {
      if (D == 32) SM_MFX(1, 2);
      else if (D == 64) SM_MFX(2, 4);
      else if (D == 96) SM_MFX(3, 6);
      else if (D == 128) SM_MFX(4, 8);
      else if (D == 256) SM_MFX_R(8, 16, 1);
      else return 1;
    }
    else if (D == 64 && Dv == 64) SM_MFXS(2, 4);             // separate key and value pages
    else if (D == 96 && Dv == 96) SM_MFXS(3, 6);
    else if (D == 128 && Dv == 128) SM_MFXS(4, 8);
    else if (D == 128 && Dv == 64) SM_MFXS(4, 4);
    else if (D == 64 && Dv == 128) SM_MFXS(2, 8);
    else if (D == 32 && Dv == 32) SM_MFXS(1, 2);
    else return 1;
#undef SM_MFXS
#undef SM_MFX
#undef SM_MFX_RK
#undef SM_MFX_R
    return (int)hipGetLastError();
  }
#define SM_MF_ARGS                                                                                                  \
  dim3(NT), 0, st, (const bf16_t*)q, (const bf16_t*)gate, gate_ld, (const bf16_t*)kp, (const bf16_t*)vp, kb, vb,     \
      seq_slot, seq_start, seq_len, seq_off, ptab, ptab_ld, (bf16_t*)out, n, H, G, PB, sl2, window, pool, kld, vld
#define SM_MF_R(DK, DV, RH, KVS) \
  hipLaunchKernelGGL((attn_mfma_kernel<DK, DV, RH, KVS>), dim3(qtiles, H / RH), SM_MF_ARGS)
#define SM_MF(DK, DV)                             \
  do {                                            \
    if (rh == 4) SM_MF_R(DK, DV, 4, false);       \
    else if (rh == 2) SM_MF_R(DK, DV, 2, false);  \
    else SM_MF_R(DK, DV, 1, false);               \
  } while (0)
#define SM_MFK(DK, DV)                            \
  do {                                            \
    if (rh == 4) SM_MF_R(DK, DV, 4, true);        \
    else if (rh == 2) SM_MF_R(DK, DV, 2, true);   \
    else SM_MF_R(DK, DV, 1, true);                \
  } while (0)
  if (kvs) {                                                 // latent rows: latent | shared key part, value = the latent
    if (D == 128 && Dv == 96) SM_MFK(4, 6);
    else if (D == 160 && Dv == 128) SM_MFK(5, 8);
    else if (D == 192 && Dv == 128) SM_MFK(6, 8);
    else if (D == 320 && Dv == 256) SM_MF_R(10, 16, 1, true);   // one head per workgroup: its output tile fills the registers
    else return 1;
  }
  else if (D == 64 && Dv == 64) SM_MF(2, 4);
  else if (D == 96 && Dv == 96) SM_MF(3, 6);
  else if (D == 128 && Dv == 128) SM_MF(4, 8);
  else if (D == 128 && Dv == 64) SM_MF(4, 4);
  else if (D == 64 && Dv == 128) SM_MF(2, 8);
  else if (D == 32 && Dv == 32) SM_MF(1, 2);
  else return 1;
#undef SM_MF
#undef SM_MFK
#undef SM_MF_R
#undef SM_MF_ARGS
  return (int)hipGetLastError();
}

}  // extern "C"
