// Per-slot sequence state beside the KV cache (gfx950): pooled-block caches,
// short causal convolutions and three linear recurrences.
//
//   kv_pool_update    block means of the cached keys/values for the blocks a
//                     step completes (read by attn_mod's pooled entries)
//   causal_conv_silu  per-channel causal convolution + SiLU; the last taps-1
//                     inputs of every slot are its state
//   ssd_scan          S <- exp(-exp(A_h) dt) S + dt B x^T ; y = S^T C + D x
//   delta_scan        S <- diag(w) S - (a u)(u^T S) + k v^T ; o = S^T r
//   gated_delta_scan  S <- g S ; S <- S + k (beta (v - S^T k))^T ; o = S^T q
//
// Geometry is the cache's: token (b,t) = row b*T+t sits at position pos[b]+t
// of slot slots[b] (default b); tokens t >= lens[b] are padding. Every state
// is taken as zero at position 0 and is written back only by rows with real
// tokens, so a reused slot needs no reset and idle rows keep their state.
// Decays, step sizes, gates and states are fp32 whatever the activation
// dtype ("short" stands for bf16 bits).
//
// The scans share one layout: a workgroup owns one head (or a slice of
// its value columns) of one batch row and walks the tokens in order. The
// state matrix [rows x columns] is spread as: thread (column j, slice s)
// keeps rows [R s, R s + R) of column j in registers (R = 32, 16 or 8); the slices of a
// column are neighbouring lanes, so the two per-token reductions over rows
// are in-register sums plus a few lane shuffles. Per-token vectors (B, C /
// r, k, w, ...) are staged through LDS in chunks of tokens, with all their
// transcendental functions evaluated once per element at staging time.
#include "common.h"

namespace dnet {

namespace {

template <typename T> __device__ __forceinline__ float lds(const T* p);
template <> __device__ __forceinline__ float lds<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float lds<short>(const short* p) { return bits2f(*p); }
template <typename T> __device__ __forceinline__ void sts(T* p, float v);
template <> __device__ __forceinline__ void sts<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void sts<short>(short* p, float v) { *p = f2bits(v); }

// State rows per thread R is 32, 16 or 8 (fewer rows = more lanes per column =
// more waves in flight when batch x heads is small). LDS pitch of one R-row
// slice: 4 spare floats shift neighbouring slices by four banks, so the 16 B
// reads of the slices of a column never collide.
template <int R> __host__ __device__ inline int padded(int r) {
  return (r / R) * (R + 4) + (r % R);
}

struct Geo {
  const int* pos;
  const int* lens;
  const int* slots;
  int T, Bc;
};

__device__ __forceinline__ bool row_geo(const Geo& g, int b, int& p0, int& n,
                                        int& slot) {
  n = g.lens ? min(g.lens[b], g.T) : g.T;
  slot = g.slots ? g.slots[b] : b;
  p0 = g.pos[b];
  return n > 0 && slot >= 0 && slot < g.Bc && p0 >= 0;
}

__device__ __forceinline__ float sigmoid_a(float x) {
  return 1.0f / (1.0f + expf(-x));
}
__device__ __forceinline__ float softplus_a(float x) {
  return x > 20.f ? x : log1pf(expf(x));
}

// ---- pooled blocks ---------------------------------------------------------
// grid (candidate blocks, Hkv, B): block c0 + blockIdx.x of row b, c0 = the
// first block whose last position is >= pos[b].
template <typename T>
__global__ __launch_bounds__(128) void kv_pool_kernel(
    const T* __restrict__ kc, const T* __restrict__ vc, T* __restrict__ pk,
    T* __restrict__ pv, const Geo g, const int Hkv, const int Smax,
    const int Sp, const int D, const int DV, const int pool) {
  int p0, n, slot;
  if (!row_geo(g, blockIdx.z, p0, n, slot)) return;
  const int c = p0 / pool + blockIdx.x;
  const int last = c * pool + pool - 1;
  if (last >= p0 + n || last >= Smax || c >= Sp) return;
  const int hk = blockIdx.y;
  const float inv = 1.0f / (float)pool;
  const T* ks = kc + (((int64_t)slot * Hkv + hk) * Smax + (int64_t)c * pool) * D;
  const T* vs = vc + (((int64_t)slot * Hkv + hk) * Smax + (int64_t)c * pool) * DV;
  for (int e = threadIdx.x; e < D; e += blockDim.x) {
    float s = 0.f;
    for (int j = 0; j < pool; ++j) s += lds<T>(ks + (int64_t)j * D + e);
    sts<T>(pk + (((int64_t)slot * Hkv + hk) * Sp + c) * D + e, s * inv);
  }
  for (int e = threadIdx.x; e < DV; e += blockDim.x) {
    float s = 0.f;
    for (int j = 0; j < pool; ++j) s += lds<T>(vs + (int64_t)j * DV + e);
    sts<T>(pv + (((int64_t)slot * Hkv + hk) * Sp + c) * DV + e, s * inv);
  }
}

// ---- causal convolution ----------------------------------------------------
// grid (channel tiles, B*T), CW channels per thread (4 when the row stride,
// the first column and C are multiples of 4: 8 B / 16 B accesses). state
// [Bc, taps-1, C]: entry j of a slot holds the input at position
// pos - (taps-1) + j (positions < 0 count as zero).
template <typename T, int CW>
__global__ __launch_bounds__(256) void conv_silu_kernel(
    const T* __restrict__ x, const int64_t ld, const int col0,
    const float* __restrict__ w, const float* __restrict__ bias,
    const T* __restrict__ state, float* __restrict__ y, const Geo g,
    const int C, const int taps) {
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * CW;
  if (c >= C) return;
  const int64_t row = blockIdx.y;
  const int b = (int)(row / g.T), t = (int)(row % g.T);
  int p0, n, slot;
  float acc[CW];
  const bool on = row_geo(g, b, p0, n, slot) && t < n;
#pragma unroll
  for (int e = 0; e < CW; ++e) acc[e] = on ? bias[c + e] : 0.f;
  if (on) {
    for (int j = 0; j < taps; ++j) {
      const int tt = t - (taps - 1) + j;
      const T* src = nullptr;
      if (tt >= 0) {
        src = x + ((int64_t)b * g.T + tt) * ld + col0 + c;
      } else if (p0 + tt >= 0) {
        src = state + ((int64_t)slot * (taps - 1) + (taps - 1 + tt)) * C + c;
      }
      if (src == nullptr) continue;
      float v[CW];
      if constexpr (CW == 4 && sizeof(T) == 2) {
        const short4v q = *reinterpret_cast<const short4v*>(src);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = bits2f(q.x[e]);
      } else if constexpr (CW == 4) {
        const float4 q = *reinterpret_cast<const float4*>(src);
        v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
      } else {
        v[0] = lds<T>(src);
      }
#pragma unroll
      for (int e = 0; e < CW; ++e)
        acc[e] = fmaf(w[(c + e) * taps + j], v[e], acc[e]);
    }
#pragma unroll
    for (int e = 0; e < CW; ++e) acc[e] = acc[e] * sigmoid_a(acc[e]);
  }
  if constexpr (CW == 4) {
    *reinterpret_cast<float4*>(y + row * C + c) =
        make_float4(acc[0], acc[1], acc[2], acc[3]);
  } else {
    y[row * C + c] = acc[0];
  }
}

// Token-tiled variant for taps <= 4: grid (channel tiles, B * token tiles).
// A thread walks kConvTile consecutive tokens of its CW channels with the
// taps and the sliding window of inputs in registers, so every input is read
// once and the weights once per tile.
constexpr int kConvTile = 16;

template <typename T, int CW>
__device__ __forceinline__ void conv_load(const T* src, float (&v)[CW]) {
  if constexpr (CW == 4 && sizeof(T) == 2) {
    const short4v q = *reinterpret_cast<const short4v*>(src);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = bits2f(q.x[e]);
  } else if constexpr (CW == 4) {
    const float4 q = *reinterpret_cast<const float4*>(src);
    v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
  } else {
    v[0] = lds<T>(src);
  }
}

template <typename T, int CW, int TAPS>
__global__ __launch_bounds__(256) void conv_silu_tile_kernel(
    const T* __restrict__ x, const int64_t ld, const int col0,
    const float* __restrict__ w, const float* __restrict__ bias,
    const T* __restrict__ state, float* __restrict__ y, const Geo g,
    const int C) {
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) * CW;
  if (c >= C) return;
  const int ntile = (g.T + kConvTile - 1) / kConvTile;
  const int b = blockIdx.y / ntile;
  const int t0 = (blockIdx.y % ntile) * kConvTile;
  const int t1 = min(t0 + kConvTile, g.T);
  int p0, n, slot;
  const bool valid = row_geo(g, b, p0, n, slot);
  float wr[TAPS][CW], br[CW], win[TAPS][CW];
#pragma unroll
  for (int e = 0; e < CW; ++e) {
    br[e] = bias[c + e];
#pragma unroll
    for (int j = 0; j < TAPS; ++j) wr[j][e] = w[(c + e) * TAPS + j];
  }
  // inputs at t0-(TAPS-1) .. t0-1: earlier rows of this step, the slot's
  // tail, or zero before position 0
#pragma unroll
  for (int j = 0; j < TAPS - 1; ++j) {
    const int tt = t0 - (TAPS - 1) + j;
#pragma unroll
    for (int e = 0; e < CW; ++e) win[j][e] = 0.f;
    if (!valid || t0 >= n) continue;
    if (tt >= 0)
      conv_load<T, CW>(x + ((int64_t)b * g.T + tt) * ld + col0 + c, win[j]);
    else if (p0 + tt >= 0)
      conv_load<T, CW>(
          state + ((int64_t)slot * (TAPS - 1) + (TAPS - 1 + tt)) * C + c,
          win[j]);
  }
#pragma unroll 4
  for (int t = t0; t < t1; ++t) {
    const int64_t row = (int64_t)b * g.T + t;
    float acc[CW];
    if (valid && t < n) {
      conv_load<T, CW>(x + row * ld + col0 + c, win[TAPS - 1]);
#pragma unroll
      for (int e = 0; e < CW; ++e) {
        float a = br[e];
#pragma unroll
        for (int j = 0; j < TAPS; ++j) a = fmaf(wr[j][e], win[j][e], a);
        acc[e] = a * sigmoid_a(a);
      }
#pragma unroll
      for (int j = 0; j < TAPS - 1; ++j)
#pragma unroll
        for (int e = 0; e < CW; ++e) win[j][e] = win[j + 1][e];
    } else {
#pragma unroll
      for (int e = 0; e < CW; ++e) acc[e] = 0.f;
    }
    if constexpr (CW == 4) {
      *reinterpret_cast<float4*>(y + row * C + c) =
          make_float4(acc[0], acc[1], acc[2], acc[3]);
    } else {
      y[row * C + c] = acc[0];
    }
  }
}

// grid (channel tiles, B): shift the slot's tail by its n new inputs
template <typename T>
__global__ __launch_bounds__(256) void conv_state_kernel(
    const T* __restrict__ x, const int64_t ld, const int col0,
    T* __restrict__ state, const Geo g, const int C, const int taps) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int b = blockIdx.y;
  int p0, n, slot;
  if (!row_geo(g, b, p0, n, slot)) return;
  T* st = state + (int64_t)slot * (taps - 1) * C + c;
  for (int s = 0; s < taps - 1; ++s) {          // ascending: reads run ahead
    const int q = n - (taps - 1) + s;           // index among the new tokens
    T v = (T)0;
    if (q >= 0) v = x[((int64_t)b * g.T + q) * ld + col0 + c];
    else if (p0 + q >= 0) v = st[(int64_t)(s + n) * C];
    st[(int64_t)s * C] = v;
  }
}

// ---- state-space recurrence ------------------------------------------------
// grid (heads * column tiles, B), block = JB columns x NS slices.
// LDS per token of a chunk: B [NP], C [NP], x [JB], dt, decay.
template <typename TD, int R>
__global__ __launch_bounds__(256) void ssd_scan_kernel(
    const float* __restrict__ xbc, const TD* __restrict__ dt_src,
    const int64_t dld, const int dcol0, const float* __restrict__ dt_bias,
    const float* __restrict__ a_log, const float* __restrict__ dskip,
    float* __restrict__ state, float* __restrict__ y, const Geo g,
    const int heads, const int P, const int N, const int G, const int JB,
    const int NS, const int TC) {
  const int ntile = (P + JB - 1) / JB;
  const int h = blockIdx.x / ntile;
  const int j0 = (blockIdx.x % ntile) * JB;
  const int b = blockIdx.y;
  int p0, n, slot;
  if (!row_geo(g, b, p0, n, slot)) return;
  const int grp = h / (heads / G);
  const int inner = heads * P, C = inner + 2 * G * N;
  const int NR = NS * R;                    // state rows incl. padding
  const int NP = NS * (R + 4);                   // LDS pitch of one token
  const int jl = threadIdx.x / NS, sl = threadIdx.x % NS;
  const int j = j0 + jl;
  const bool col_ok = j < P;

  extern __shared__ __attribute__((aligned(16))) float sm[];
  float* sB = sm;                               // [TC][NP]
  float* sC = sB + TC * NP;                     // [TC][NP]
  float* sX = sC + TC * NP;                     // [TC][JB]
  float* sDt = sX + TC * JB;                    // [TC]
  float* sDec = sDt + TC;                       // [TC]

  float S[R];
  float* sp = state + (((int64_t)slot * heads + h) * N) * P;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int row = sl * R + r;
    S[r] = (p0 > 0 && col_ok && row < N) ? sp[(int64_t)row * P + j] : 0.f;
  }
  const float a_h = expf(a_log[h]), d_h = dskip[h], bias_h = dt_bias[h];

  for (int t0 = 0; t0 < n; t0 += TC) {
    const int tc = min(TC, n - t0);
    __syncthreads();                            // previous chunk consumed
    for (int idx = threadIdx.x; idx < tc * NR; idx += blockDim.x) {
      const int tt = idx / NR, r = idx % NR;
      const float* src = xbc + ((int64_t)b * g.T + t0 + tt) * C + inner;
      sB[tt * NP + padded<R>(r)] = r < N ? src[grp * N + r] : 0.f;
      sC[tt * NP + padded<R>(r)] = r < N ? src[G * N + grp * N + r] : 0.f;
    }
    for (int idx = threadIdx.x; idx < tc * JB; idx += blockDim.x) {
      const int tt = idx / JB, c = idx % JB;
      sX[idx] = (j0 + c < P)
                    ? xbc[((int64_t)b * g.T + t0 + tt) * C + h * P + j0 + c]
                    : 0.f;
    }
    for (int tt = threadIdx.x; tt < tc; tt += blockDim.x) {
      const float raw =
          lds<TD>(dt_src + ((int64_t)b * g.T + t0 + tt) * dld + dcol0 + h);
      const float dt = softplus_a(raw + bias_h);
      sDt[tt] = dt;
      sDec[tt] = expf(-a_h * dt);
    }
    __syncthreads();
    for (int tt = 0; tt < tc; ++tt) {
      const float xj = sX[tt * JB + jl];
      const float dec = sDec[tt], dtx = sDt[tt] * xj;
      const float4* bp = reinterpret_cast<const float4*>(sB + tt * NP + sl * (R + 4));
      const float4* cp = reinterpret_cast<const float4*>(sC + tt * NP + sl * (R + 4));
      float acc = 0.f;
#pragma unroll
      for (int r4 = 0; r4 < R / 4; ++r4) {
        const float4 bv = bp[r4], cv = cp[r4];
        S[4 * r4 + 0] = fmaf(dec, S[4 * r4 + 0], dtx * bv.x);
        S[4 * r4 + 1] = fmaf(dec, S[4 * r4 + 1], dtx * bv.y);
        S[4 * r4 + 2] = fmaf(dec, S[4 * r4 + 2], dtx * bv.z);
        S[4 * r4 + 3] = fmaf(dec, S[4 * r4 + 3], dtx * bv.w);
        acc = fmaf(S[4 * r4 + 0], cv.x, acc);
        acc = fmaf(S[4 * r4 + 1], cv.y, acc);
        acc = fmaf(S[4 * r4 + 2], cv.z, acc);
        acc = fmaf(S[4 * r4 + 3], cv.w, acc);
      }
      for (int off = NS >> 1; off > 0; off >>= 1)
        acc += __shfl_xor(acc, off, 64);
      if (sl == 0 && col_ok)
        y[((int64_t)b * g.T + t0 + tt) * inner + h * P + j] =
            fmaf(d_h, xj, acc);
    }
  }
  if (col_ok) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int row = sl * R + r;
      if (row < N) sp[(int64_t)row * P + j] = S[r];
    }
  }
}

// ---- generalized delta rule ------------------------------------------------
// grid (H * column tiles, B), block = JB value columns x NS key slices.
// LDS per token of a chunk: r, k, w, a*k [DP each], v [JB], 1/(|k|^2+eps).
template <typename T, int R>
__global__ __launch_bounds__(256) void delta_scan_kernel(
    const T* __restrict__ src, const int64_t ld, const int r0, const int k0,
    const int v0, const int a0, const T* __restrict__ wl,
    const float* __restrict__ w0, const float* __restrict__ ab,
    float* __restrict__ state, float* __restrict__ o, const Geo g,
    const int H, const int d, const int JB, const int NS, const int TC,
    const float decay_scale, const float unit_eps) {
  const int ntile = (d + JB - 1) / JB;
  const int h = blockIdx.x / ntile;
  const int j0 = (blockIdx.x % ntile) * JB;
  const int b = blockIdx.y;
  int p0, n, slot;
  if (!row_geo(g, b, p0, n, slot)) return;
  const int DR = NS * R;                    // key rows incl. padding
  const int DP = NS * (R + 4);                   // LDS pitch of one token
  const int jl = threadIdx.x / NS, sl = threadIdx.x % NS;
  const int j = j0 + jl;
  const bool col_ok = j < d;
  const int wid = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const int nw = (blockDim.x + kWave - 1) / kWave;

  extern __shared__ __attribute__((aligned(16))) float sm[];
  float* sR = sm;                               // [TC][DP]
  float* sK = sR + TC * DP;
  float* sW = sK + TC * DP;
  float* sAK = sW + TC * DP;                    // a * k
  float* sV = sAK + TC * DP;                    // [TC][JB]
  float* sRn = sV + TC * JB;                    // [TC] 1 / (sum k^2 + eps)

  float S[R];
  float* sp = state + (((int64_t)slot * H + h) * d) * d;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int row = sl * R + r;
    S[r] = (p0 > 0 && col_ok && row < d) ? sp[(int64_t)row * d + j] : 0.f;
  }
  const int hd = h * d;

  for (int t0 = 0; t0 < n; t0 += TC) {
    const int tc = min(TC, n - t0);
    __syncthreads();                            // previous chunk consumed
    // element-wise staging: every load of the chunk is in flight at once
    for (int idx = threadIdx.x; idx < tc * DR; idx += blockDim.x) {
      const int tt = idx / DR, i = idx % DR;
      const int64_t row = (int64_t)b * g.T + t0 + tt;
      const T* sr = src + row * ld;
      float rv = 0.f, kv = 0.f, wv = 0.f, av = 0.f;
      if (i < d) {
        rv = lds<T>(sr + r0 + hd + i);
        kv = lds<T>(sr + k0 + hd + i);
        wv = expf(-decay_scale *
                  sigmoid_a(lds<T>(wl + row * (int64_t)(H * d) + hd + i) +
                            w0[hd + i]));
        av = sigmoid_a(lds<T>(sr + a0 + hd + i) + ab[hd + i]);
      }
      const int at = tt * DP + padded<R>(i);
      sR[at] = rv;
      sK[at] = kv;
      sW[at] = wv;
      sAK[at] = av * kv;
    }
    for (int idx = threadIdx.x; idx < tc * JB; idx += blockDim.x) {
      const int tt = idx / JB, c = idx % JB;
      sV[idx] = (j0 + c < d)
                    ? lds<T>(src + ((int64_t)b * g.T + t0 + tt) * ld + v0 +
                             hd + j0 + c)
                    : 0.f;
    }
    __syncthreads();
    // unit key: u = k * rsqrt(sum k^2 + eps); the update needs u u^T only,
    // so one scalar 1 / (sum k^2 + eps) per token is enough
    for (int tt = wid; tt < tc; tt += nw) {
      float ss = 0.f;
      for (int i = lane; i < d; i += kWave) {
        const float kv = sK[tt * DP + padded<R>(i)];
        ss += kv * kv;
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
      if (lane == 0) sRn[tt] = 1.0f / (ss + unit_eps);
    }
    __syncthreads();
    for (int tt = 0; tt < tc; ++tt) {
      const int base = tt * DP + sl * (R + 4);
      const float4* kp = reinterpret_cast<const float4*>(sK + base);
      float ks = 0.f;                           // (k^T S)_j over my rows
#pragma unroll
      for (int r4 = 0; r4 < R / 4; ++r4) {
        const float4 kv = kp[r4];
        ks = fmaf(kv.x, S[4 * r4 + 0], ks);
        ks = fmaf(kv.y, S[4 * r4 + 1], ks);
        ks = fmaf(kv.z, S[4 * r4 + 2], ks);
        ks = fmaf(kv.w, S[4 * r4 + 3], ks);
      }
      for (int off = NS >> 1; off > 0; off >>= 1)
        ks += __shfl_xor(ks, off, 64);
      const float us = ks * sRn[tt];            // (a u)(u^T S) = a k * us
      const float vj = sV[tt * JB + jl];
      const float4* wp = reinterpret_cast<const float4*>(sW + base);
      const float4* ap = reinterpret_cast<const float4*>(sAK + base);
      const float4* rp = reinterpret_cast<const float4*>(sR + base);
      float acc = 0.f;
#pragma unroll
      for (int r4 = 0; r4 < R / 4; ++r4) {
        const float4 wv = wp[r4], av = ap[r4], kv = kp[r4], rv = rp[r4];
        S[4 * r4 + 0] = fmaf(wv.x, S[4 * r4 + 0], fmaf(kv.x, vj, -av.x * us));
        S[4 * r4 + 1] = fmaf(wv.y, S[4 * r4 + 1], fmaf(kv.y, vj, -av.y * us));
        S[4 * r4 + 2] = fmaf(wv.z, S[4 * r4 + 2], fmaf(kv.z, vj, -av.z * us));
        S[4 * r4 + 3] = fmaf(wv.w, S[4 * r4 + 3], fmaf(kv.w, vj, -av.w * us));
        acc = fmaf(S[4 * r4 + 0], rv.x, acc);
        acc = fmaf(S[4 * r4 + 1], rv.y, acc);
        acc = fmaf(S[4 * r4 + 2], rv.z, acc);
        acc = fmaf(S[4 * r4 + 3], rv.w, acc);
      }
      for (int off = NS >> 1; off > 0; off >>= 1)
        acc += __shfl_xor(acc, off, 64);
      if (sl == 0 && col_ok)
        o[((int64_t)b * g.T + t0 + tt) * (int64_t)(H * d) + hd + j] = acc;
    }
  }
  if (col_ok) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int row = sl * R + r;
      if (row < d) sp[(int64_t)row * d + j] = S[r];
    }
  }
}

// ---- gated delta rule --------------------------------------------------------
// S <- g S ; u = beta (v - S^T k) ; S <- S + k u^T ; o = S^T q, state [d x dv]
// per value head, q/k heads shared by groups of value heads. grid (H * column
// tiles, B), block = JB value columns x NS key slices. LDS per token of a
// chunk: unit q (times d^-1/2), unit k [DP each], v [JB], beta, g. q, k, v
// come from the convolution's fp32 output; the raw write-strength and decay
// projections from columns of `gates` (activation dtype).
template <typename T, int R>
__global__ __launch_bounds__(256) void gated_delta_scan_kernel(
    const float* __restrict__ qkv, const T* __restrict__ gates,
    const int64_t gld, const int b0, const int a0,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias,
    float* __restrict__ state, float* __restrict__ o, const Geo g,
    const int H, const int KH, const int d, const int dv, const int JB,
    const int NS, const int TC, const float unit_eps) {
  const int ntile = (dv + JB - 1) / JB;
  const int h = blockIdx.x / ntile;
  const int j0 = (blockIdx.x % ntile) * JB;
  const int b = blockIdx.y;
  int p0, n, slot;
  if (!row_geo(g, b, p0, n, slot)) return;
  const int kh = h / (H / KH);
  const int C = 2 * KH * d + H * dv;
  const int DR = NS * R;                    // key rows incl. padding
  const int DP = NS * (R + 4);              // LDS pitch of one token
  const int jl = threadIdx.x / NS, sl = threadIdx.x % NS;
  const int j = j0 + jl;
  const bool col_ok = j < dv;
  const int wid = threadIdx.x / kWave, lane = threadIdx.x & (kWave - 1);
  const int nw = (blockDim.x + kWave - 1) / kWave;

  extern __shared__ __attribute__((aligned(16))) float sm[];
  float* sQ = sm;                               // [TC][DP]
  float* sK = sQ + TC * DP;
  float* sV = sK + TC * DP;                     // [TC][JB]
  float* sBeta = sV + TC * JB;                  // [TC]
  float* sG = sBeta + TC;                       // [TC]

  float S[R];
  float* sp = state + (((int64_t)slot * H + h) * d) * dv;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int row = sl * R + r;
    S[r] = (p0 > 0 && col_ok && row < d) ? sp[(int64_t)row * dv + j] : 0.f;
  }
  const float a_h = expf(a_log[h]), bias_h = dt_bias[h];
  const float qscale = 1.0f / sqrtf((float)d);

  for (int t0 = 0; t0 < n; t0 += TC) {
    const int tc = min(TC, n - t0);
    __syncthreads();                            // previous chunk consumed
    for (int idx = threadIdx.x; idx < tc * DR; idx += blockDim.x) {
      const int tt = idx / DR, i = idx % DR;
      const float* sr = qkv + ((int64_t)b * g.T + t0 + tt) * C;
      const int at = tt * DP + padded<R>(i);
      sQ[at] = i < d ? sr[kh * d + i] : 0.f;
      sK[at] = i < d ? sr[KH * d + kh * d + i] : 0.f;
    }
    for (int idx = threadIdx.x; idx < tc * JB; idx += blockDim.x) {
      const int tt = idx / JB, c = idx % JB;
      sV[idx] = (j0 + c < dv)
                    ? qkv[((int64_t)b * g.T + t0 + tt) * C + 2 * KH * d +
                          h * dv + j0 + c]
                    : 0.f;
    }
    for (int tt = threadIdx.x; tt < tc; tt += blockDim.x) {
      const T* gr = gates + ((int64_t)b * g.T + t0 + tt) * gld;
      sBeta[tt] = sigmoid_a(lds<T>(gr + b0 + h));
      sG[tt] = expf(-a_h * softplus_a(lds<T>(gr + a0 + h) + bias_h));
    }
    __syncthreads();
    // unit vectors: x / sqrt(sum x^2 + eps), q also times d^-1/2
    for (int tt = wid; tt < tc; tt += nw) {
      float sq = 0.f, sk = 0.f;
      for (int i = lane; i < d; i += kWave) {
        const float qv = sQ[tt * DP + padded<R>(i)];
        const float kv = sK[tt * DP + padded<R>(i)];
        sq = fmaf(qv, qv, sq);
        sk = fmaf(kv, kv, sk);
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        sq += __shfl_xor(sq, off, 64);
        sk += __shfl_xor(sk, off, 64);
      }
      const float rq = qscale / sqrtf(sq + unit_eps);
      const float rk = 1.0f / sqrtf(sk + unit_eps);
      for (int i = lane; i < d; i += kWave) {
        sQ[tt * DP + padded<R>(i)] *= rq;
        sK[tt * DP + padded<R>(i)] *= rk;
      }
    }
    __syncthreads();
    for (int tt = 0; tt < tc; ++tt) {
      const int base = tt * DP + sl * (R + 4);
      const float4* kp = reinterpret_cast<const float4*>(sK + base);
      const float4* qp = reinterpret_cast<const float4*>(sQ + base);
      const float gt = sG[tt];
      float ks = 0.f;                           // (S^T k)_j over my rows
#pragma unroll
      for (int r4 = 0; r4 < R / 4; ++r4) {
        const float4 kv = kp[r4];
        S[4 * r4 + 0] *= gt;
        S[4 * r4 + 1] *= gt;
        S[4 * r4 + 2] *= gt;
        S[4 * r4 + 3] *= gt;
        ks = fmaf(kv.x, S[4 * r4 + 0], ks);
        ks = fmaf(kv.y, S[4 * r4 + 1], ks);
        ks = fmaf(kv.z, S[4 * r4 + 2], ks);
        ks = fmaf(kv.w, S[4 * r4 + 3], ks);
      }
      for (int off = NS >> 1; off > 0; off >>= 1)
        ks += __shfl_xor(ks, off, 64);
      const float uj = sBeta[tt] * (sV[tt * JB + jl] - ks);
      float acc = 0.f;
#pragma unroll
      for (int r4 = 0; r4 < R / 4; ++r4) {
        const float4 kv = kp[r4], qv = qp[r4];
        S[4 * r4 + 0] = fmaf(kv.x, uj, S[4 * r4 + 0]);
        S[4 * r4 + 1] = fmaf(kv.y, uj, S[4 * r4 + 1]);
        S[4 * r4 + 2] = fmaf(kv.z, uj, S[4 * r4 + 2]);
        S[4 * r4 + 3] = fmaf(kv.w, uj, S[4 * r4 + 3]);
        acc = fmaf(S[4 * r4 + 0], qv.x, acc);
        acc = fmaf(S[4 * r4 + 1], qv.y, acc);
        acc = fmaf(S[4 * r4 + 2], qv.z, acc);
        acc = fmaf(S[4 * r4 + 3], qv.w, acc);
      }
      for (int off = NS >> 1; off > 0; off >>= 1)
        acc += __shfl_xor(acc, off, 64);
      if (sl == 0 && col_ok)
        o[((int64_t)b * g.T + t0 + tt) * (int64_t)(H * dv) + h * dv + j] = acc;
    }
  }
  if (col_ok) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int row = sl * R + r;
      if (row < d) sp[(int64_t)row * dv + j] = S[r];
    }
  }
}

bool is_bf16(const torch::Tensor& t) { return t.scalar_type() == torch::kBFloat16; }
bool is_f32(const torch::Tensor& t) { return t.scalar_type() == torch::kFloat32; }

Geo make_geo(const torch::Tensor& pos, const c10::optional<torch::Tensor>& lens,
             const c10::optional<torch::Tensor>& slots, int64_t B, int64_t T,
             int64_t Bc) {
  auto chk = [&](const torch::Tensor& t) {
    DNET_CHECK(t.scalar_type() == torch::kInt32 && t.is_contiguous() &&
                   t.numel() >= B, "int32 index tensor [B]");
    return t.data_ptr<int>();
  };
  Geo g;
  g.pos = chk(pos);
  g.lens = lens.has_value() ? chk(*lens) : nullptr;
  g.slots = slots.has_value() ? chk(*slots) : nullptr;
  if (!slots.has_value()) DNET_CHECK(B <= Bc, "more rows than state slots");
  g.T = (int)T;
  g.Bc = (int)Bc;
  return g;
}

// Shape of a scan block: R state rows per thread, NS = slices per column (a
// power of two so lane shuffles pair them up), JB columns so that the block
// has at most 256 threads and at least one whole wave (spare columns idle).
// R shrinks from 32 while the launch would leave most SIMDs with one wave.
void scan_shape(int rows, int cols, int64_t heads_x_batch, int min_r, int& R,
                int& NS, int& JB) {
  R = 32;
  while (R > 8 && R / 2 >= rows) R /= 2;      // no more rows than the state has
  min_r = min_r < R ? min_r : R;
  for (;; R /= 2) {
    NS = 1;
    while (NS * R < rows) NS *= 2;
    JB = 1;
    while (JB < cols && JB * 2 * NS <= 256) JB *= 2;
    while (JB * NS < kWave) JB *= 2;
    const int64_t waves =
        heads_x_batch * ((cols + JB - 1) / JB) * (JB * NS / kWave);
    if (R <= min_r || waves >= 4096) break;
  }
}

}  // namespace

void kv_pool_update(torch::Tensor kcache, torch::Tensor vcache,
                    torch::Tensor pool_k, torch::Tensor pool_v,
                    torch::Tensor pos, c10::optional<torch::Tensor> lens,
                    c10::optional<torch::Tensor> slots, int64_t T,
                    int64_t pool) {
  DNET_CHECK(kcache.dim() == 4 && vcache.dim() == 4 && pool_k.dim() == 4 &&
                 pool_v.dim() == 4 && kcache.is_contiguous() &&
                 vcache.is_contiguous() && pool_k.is_contiguous() &&
                 pool_v.is_contiguous(), "caches [Bc, Hkv, S, D]");
  const int Bc = kcache.size(0), Hkv = kcache.size(1), Smax = kcache.size(2);
  const int D = kcache.size(3), DV = vcache.size(3), Sp = pool_k.size(2);
  DNET_CHECK(vcache.size(0) == Bc && vcache.size(1) == Hkv &&
                 vcache.size(2) == Smax && pool_k.size(0) == Bc &&
                 pool_k.size(1) == Hkv && pool_k.size(3) == D &&
                 pool_v.size(0) == Bc && pool_v.size(1) == Hkv &&
                 pool_v.size(2) == Sp && pool_v.size(3) == DV, "cache shapes");
  DNET_CHECK(pool_k.scalar_type() == kcache.scalar_type() &&
                 pool_v.scalar_type() == kcache.scalar_type() &&
                 vcache.scalar_type() == kcache.scalar_type(), "dtypes");
  DNET_CHECK(pool >= 1 && T >= 1, "pool, T");
  const int64_t B = pos.numel();
  if (B == 0) return;
  const Geo g = make_geo(pos, lens, slots, B, T, Bc);
  const dim3 grid((unsigned)((T + pool - 1) / pool + 1), (unsigned)Hkv,
                  (unsigned)B);
  auto st = current_stream();
  if (is_bf16(kcache))
    hipLaunchKernelGGL((kv_pool_kernel<short>), grid, dim3(128), 0, st,
                       (const short*)kcache.data_ptr(),
                       (const short*)vcache.data_ptr(),
                       (short*)pool_k.data_ptr(), (short*)pool_v.data_ptr(), g,
                       Hkv, Smax, Sp, D, DV, (int)pool);
  else if (is_f32(kcache))
    hipLaunchKernelGGL((kv_pool_kernel<float>), grid, dim3(128), 0, st,
                       (const float*)kcache.data_ptr(),
                       (const float*)vcache.data_ptr(),
                       (float*)pool_k.data_ptr(), (float*)pool_v.data_ptr(), g,
                       Hkv, Smax, Sp, D, DV, (int)pool);
  else DNET_CHECK(false, "kv_pool_update: dtype");
}

void causal_conv_silu(torch::Tensor x, int64_t col0, torch::Tensor w,
                      torch::Tensor bias, torch::Tensor state, torch::Tensor y,
                      torch::Tensor pos, c10::optional<torch::Tensor> lens,
                      c10::optional<torch::Tensor> slots, int64_t T) {
  DNET_CHECK(x.dim() == 2 && x.is_contiguous(), "x [B*T, ld]");
  DNET_CHECK(w.dim() == 2 && is_f32(w) && w.is_contiguous(), "w fp32 [C, taps]");
  const int C = w.size(0), taps = w.size(1);
  const int64_t M = x.size(0);
  DNET_CHECK(T > 0 && M % T == 0, "rows = B*T");
  const int64_t B = M / T;
  DNET_CHECK(taps >= 1 && col0 >= 0 && col0 + C <= x.size(1), "columns");
  DNET_CHECK(is_f32(bias) && bias.is_contiguous() && bias.numel() == C, "bias");
  DNET_CHECK(state.dim() == 3 && state.is_contiguous() &&
                 state.size(1) == taps - 1 && state.size(2) == C &&
                 state.scalar_type() == x.scalar_type(),
             "state [Bc, taps-1, C] in x's dtype");
  DNET_CHECK(is_f32(y) && y.is_contiguous() && y.size(0) == M &&
                 y.size(1) == C, "y fp32 [B*T, C]");
  if (M == 0) return;
  const Geo g = make_geo(pos, lens, slots, B, T, state.size(0));
  auto st = current_stream();
  const bool v4 = C % 4 == 0 && col0 % 4 == 0 && x.size(1) % 4 == 0;
  const int cpt = v4 ? 4 : 1;                 // channels per thread
  const dim3 grid((unsigned)((C + 256 * cpt - 1) / (256 * cpt)), (unsigned)M);
  const dim3 sgrid((unsigned)((C + 255) / 256), (unsigned)B);
  const int ntile = (int)((T + kConvTile - 1) / kConvTile);
  const dim3 tgrid(grid.x, (unsigned)(B * ntile));
#define CVT(TT, WW, TP)                                                     \
  hipLaunchKernelGGL((conv_silu_tile_kernel<TT, WW, TP>), tgrid, dim3(256), \
                     0, st, (const TT*)x.data_ptr(), x.size(1), (int)col0,  \
                     w.data_ptr<float>(), bias.data_ptr<float>(),           \
                     (const TT*)state.data_ptr(), y.data_ptr<float>(), g, C)
#define CV(TT, WW)                                                          \
  do {                                                                      \
    if (taps == 4) CVT(TT, WW, 4);                                          \
    else if (taps == 3) CVT(TT, WW, 3);                                     \
    else if (taps == 2) CVT(TT, WW, 2);                                     \
    else                                                                    \
      hipLaunchKernelGGL((conv_silu_kernel<TT, WW>), grid, dim3(256), 0,    \
                         st, (const TT*)x.data_ptr(), x.size(1), (int)col0, \
                         w.data_ptr<float>(), bias.data_ptr<float>(),       \
                         (const TT*)state.data_ptr(), y.data_ptr<float>(),  \
                         g, C, taps);                                       \
    if (taps > 1)                                                           \
      hipLaunchKernelGGL((conv_state_kernel<TT>), sgrid, dim3(256), 0, st,  \
                         (const TT*)x.data_ptr(), x.size(1), (int)col0,     \
                         (TT*)state.data_ptr(), g, C, taps);                \
  } while (0)
  if (is_bf16(x)) { if (v4) CV(short, 4); else CV(short, 1); }
  else if (is_f32(x)) { if (v4) CV(float, 4); else CV(float, 1); }
  else DNET_CHECK(false, "causal_conv_silu: dtype");
#undef CVT
#undef CV
}

void ssd_scan(torch::Tensor xbc, torch::Tensor dt_src, int64_t dt_col0,
              torch::Tensor dt_bias, torch::Tensor a_log, torch::Tensor dskip,
              torch::Tensor state, torch::Tensor y, torch::Tensor pos,
              c10::optional<torch::Tensor> lens,
              c10::optional<torch::Tensor> slots, int64_t T, int64_t heads,
              int64_t P, int64_t N, int64_t G) {
  const int64_t M = xbc.size(0);
  DNET_CHECK(T > 0 && M % T == 0, "rows = B*T");
  const int64_t B = M / T;
  DNET_CHECK(heads > 0 && G > 0 && heads % G == 0 && P > 0 && N > 0, "sizes");
  DNET_CHECK(N <= 256, "state size <= 256");
  const int64_t inner = heads * P;
  DNET_CHECK(xbc.dim() == 2 && is_f32(xbc) && xbc.is_contiguous() &&
                 xbc.size(1) == inner + 2 * G * N, "xbc fp32 [B*T, x|B|C]");
  DNET_CHECK(dt_src.dim() == 2 && dt_src.is_contiguous() &&
                 dt_src.size(0) == M && dt_col0 >= 0 &&
                 dt_col0 + heads <= dt_src.size(1), "dt columns");
  for (const torch::Tensor* t : {&dt_bias, &a_log, &dskip})
    DNET_CHECK(is_f32(*t) && t->is_contiguous() && t->numel() == heads,
               "per-head fp32 parameters");
  DNET_CHECK(state.dim() == 4 && is_f32(state) && state.is_contiguous() &&
                 state.size(1) == heads && state.size(2) == N &&
                 state.size(3) == P, "state fp32 [Bc, heads, N, P]");
  DNET_CHECK(is_f32(y) && y.is_contiguous() && y.size(0) == M &&
                 y.size(1) == inner, "y fp32 [B*T, heads*P]");
  if (M == 0) return;
  const Geo g = make_geo(pos, lens, slots, B, T, state.size(0));
  int R, NS, JB;
  // 32 rows per thread: narrower slices multiply the per-token LDS reads of
  // B and C, which the columns of a wave share (measured slower)
  scan_shape((int)N, (int)P, heads * B, 32, R, NS, JB);
  const int NP = NS * (R + 4);
  int TC = 32;
  while (TC > 1 && (size_t)TC * (2 * NP + JB + 2) * 4 > 48 * 1024) TC /= 2;
  const size_t lds_bytes = (size_t)TC * (2 * NP + JB + 2) * sizeof(float);
  const dim3 grid((unsigned)(heads * ((P + JB - 1) / JB)), (unsigned)B);
  auto st = current_stream();
#define SS(TD, RR)                                                           \
  hipLaunchKernelGGL((ssd_scan_kernel<TD, RR>), grid, dim3(JB * NS),         \
                     lds_bytes, st, xbc.data_ptr<float>(),                   \
                     (const TD*)dt_src.data_ptr(), dt_src.size(1),           \
                     (int)dt_col0, dt_bias.data_ptr<float>(),                \
                     a_log.data_ptr<float>(), dskip.data_ptr<float>(),       \
                     state.data_ptr<float>(), y.data_ptr<float>(), g,        \
                     (int)heads, (int)P, (int)N, (int)G, JB, NS, TC)
#define SS_R(TD)                          \
  do {                                    \
    if (R == 32) SS(TD, 32);              \
    else if (R == 16) SS(TD, 16);         \
    else SS(TD, 8);                       \
  } while (0)
  if (is_bf16(dt_src)) SS_R(short);
  else if (is_f32(dt_src)) SS_R(float);
  else DNET_CHECK(false, "ssd_scan: dt dtype");
#undef SS_R
#undef SS
}

void delta_scan(torch::Tensor src, int64_t r0, int64_t k0, int64_t v0,
                int64_t a0, torch::Tensor wl, torch::Tensor w0,
                torch::Tensor ab, torch::Tensor state, torch::Tensor o,
                torch::Tensor pos, c10::optional<torch::Tensor> lens,
                c10::optional<torch::Tensor> slots, int64_t T, int64_t H,
                int64_t d, double decay_scale, double unit_eps) {
  const int64_t M = src.size(0);
  DNET_CHECK(T > 0 && M % T == 0, "rows = B*T");
  const int64_t B = M / T;
  DNET_CHECK(H > 0 && d > 0 && d <= 256, "head size <= 256");
  const int64_t n = H * d;
  DNET_CHECK(src.dim() == 2 && src.is_contiguous(), "src [B*T, ld]");
  for (int64_t c0 : {r0, k0, v0, a0})
    DNET_CHECK(c0 >= 0 && c0 + n <= src.size(1), "column ranges");
  DNET_CHECK(wl.dim() == 2 && wl.is_contiguous() && wl.size(0) == M &&
                 wl.size(1) == n && wl.scalar_type() == src.scalar_type(),
             "wl [B*T, H*d]");
  DNET_CHECK(is_f32(w0) && w0.is_contiguous() && w0.numel() == n &&
                 is_f32(ab) && ab.is_contiguous() && ab.numel() == n,
             "w0 / ab fp32 [H*d]");
  DNET_CHECK(state.dim() == 4 && is_f32(state) && state.is_contiguous() &&
                 state.size(1) == H && state.size(2) == d &&
                 state.size(3) == d, "state fp32 [Bc, H, d, d]");
  DNET_CHECK(is_f32(o) && o.is_contiguous() && o.size(0) == M &&
                 o.size(1) == n, "o fp32 [B*T, H*d]");
  if (M == 0) return;
  const Geo g = make_geo(pos, lens, slots, B, T, state.size(0));
  int R, NS, JB;
  scan_shape((int)d, (int)d, H * B, 8, R, NS, JB);
  const int DP = NS * (R + 4);
  int TC = 32;
  while (TC > 1 && (size_t)TC * (4 * DP + JB + 1) * 4 > 48 * 1024) TC /= 2;
  const size_t lds_bytes = (size_t)TC * (4 * DP + JB + 1) * sizeof(float);
  const dim3 grid((unsigned)(H * ((d + JB - 1) / JB)), (unsigned)B);
  auto st = current_stream();
#define DS(TT, RR)                                                           \
  hipLaunchKernelGGL((delta_scan_kernel<TT, RR>), grid, dim3(JB * NS),       \
                     lds_bytes, st, (const TT*)src.data_ptr(), src.size(1),  \
                     (int)r0, (int)k0, (int)v0, (int)a0,                     \
                     (const TT*)wl.data_ptr(), w0.data_ptr<float>(),         \
                     ab.data_ptr<float>(), state.data_ptr<float>(),          \
                     o.data_ptr<float>(), g, (int)H, (int)d, JB, NS, TC,     \
                     (float)decay_scale, (float)unit_eps)
#define DS_R(TT)                          \
  do {                                    \
    if (R == 32) DS(TT, 32);              \
    else if (R == 16) DS(TT, 16);         \
    else DS(TT, 8);                       \
  } while (0)
  if (is_bf16(src)) DS_R(short);
  else if (is_f32(src)) DS_R(float);
  else DNET_CHECK(false, "delta_scan: dtype");
#undef DS_R
#undef DS
}

void gated_delta_scan(torch::Tensor qkv, torch::Tensor gates, int64_t b_col0,
                      int64_t a_col0, torch::Tensor a_log,
                      torch::Tensor dt_bias, torch::Tensor state,
                      torch::Tensor o, torch::Tensor pos,
                      c10::optional<torch::Tensor> lens,
                      c10::optional<torch::Tensor> slots, int64_t T,
                      int64_t H, int64_t KH, int64_t d, int64_t dv,
                      double unit_eps) {
  const int64_t M = qkv.size(0);
  DNET_CHECK(T > 0 && M % T == 0, "rows = B*T");
  const int64_t B = M / T;
  DNET_CHECK(H > 0 && KH > 0 && H % KH == 0 && d > 0 && d <= 256 && dv > 0,
             "heads / key heads / key size <= 256");
  DNET_CHECK(qkv.dim() == 2 && is_f32(qkv) && qkv.is_contiguous() &&
                 qkv.size(1) == 2 * KH * d + H * dv, "qkv fp32 [B*T, q|k|v]");
  DNET_CHECK(gates.dim() == 2 && gates.is_contiguous() &&
                 gates.size(0) == M, "gates [B*T, ld]");
  for (int64_t c0 : {b_col0, a_col0})
    DNET_CHECK(c0 >= 0 && c0 + H <= gates.size(1), "gate columns");
  DNET_CHECK(is_f32(a_log) && a_log.is_contiguous() && a_log.numel() == H &&
                 is_f32(dt_bias) && dt_bias.is_contiguous() &&
                 dt_bias.numel() == H, "per-head fp32 parameters");
  DNET_CHECK(state.dim() == 4 && is_f32(state) && state.is_contiguous() &&
                 state.size(1) == H && state.size(2) == d &&
                 state.size(3) == dv, "state fp32 [Bc, H, d, dv]");
  DNET_CHECK(is_f32(o) && o.is_contiguous() && o.size(0) == M &&
                 o.size(1) == H * dv, "o fp32 [B*T, H*dv]");
  if (M == 0) return;
  const Geo g = make_geo(pos, lens, slots, B, T, state.size(0));
  int R, NS, JB;
  scan_shape((int)d, (int)dv, H * B, 8, R, NS, JB);
  const int DP = NS * (R + 4);
  int TC = 32;
  while (TC > 1 && (size_t)TC * (2 * DP + JB + 2) * 4 > 48 * 1024) TC /= 2;
  const size_t lds_bytes = (size_t)TC * (2 * DP + JB + 2) * sizeof(float);
  const dim3 grid((unsigned)(H * ((dv + JB - 1) / JB)), (unsigned)B);
  auto st = current_stream();
#define GD(TT, RR)                                                           \
  hipLaunchKernelGGL((gated_delta_scan_kernel<TT, RR>), grid,                \
                     dim3(JB * NS), lds_bytes, st, qkv.data_ptr<float>(),    \
                     (const TT*)gates.data_ptr(), gates.size(1),             \
                     (int)b_col0, (int)a_col0, a_log.data_ptr<float>(),      \
                     dt_bias.data_ptr<float>(), state.data_ptr<float>(),     \
                     o.data_ptr<float>(), g, (int)H, (int)KH, (int)d,        \
                     (int)dv, JB, NS, TC, (float)unit_eps)
#define GD_R(TT)                          \
  do {                                    \
    if (R == 32) GD(TT, 32);              \
    else if (R == 16) GD(TT, 16);         \
    else GD(TT, 8);                       \
  } while (0)
  if (is_bf16(gates)) GD_R(short);
  else if (is_f32(gates)) GD_R(float);
  else DNET_CHECK(false, "gated_delta_scan: gates dtype");
#undef GD_R
#undef GD
}

}  // namespace dnet
