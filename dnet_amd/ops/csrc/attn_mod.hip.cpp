// Score-modified causal attention against the KV cache (gfx950), for decode
// (T = 1) and ragged batched prefill (T = padded length, lens = real ones)
// through one entry point, any head sizes (D != DV allowed), bf16 or fp32.
//
//   s_ij  = (q_i . k_j) * scale * temp[h]
//   s_ij  = cap * tanh(s_ij / cap)                    (cap > 0)
//   s_ij -= r1[h] * ln(1 + r2[h] * (i - j))           (r1/r2 given)
//   p_ij  = exp(s_ij) / (sum_{j<=i} exp(s_ij) + exp(sink[h]))
//
// Every score, weight and accumulator is fp32. Query (b,t) = row b*T+t sits
// at position pos[b]+t of cache row slots[b] and sees keys j <= i (and
// j > i - window when window > 0). The sequence geometry lives in device
// tensors, so a captured decode graph replays across steps.
//
// Pooled blocks (pool > 0, needs window > 0): beside the window's tokens a
// query at position i sees entry c of the pooled caches pk/pv [Bc, Hkv, Sp, D]
// (block means written by kv_pool_update) for every c < (i - window + 1) /
// pool, in the same softmax and without a distance penalty.
//
// Chunked visibility (chunk > 0): a query sees key j only inside its own block
// of `chunk` positions, j >= (i / chunk) * chunk, blocks counted from position
// 0. Sigmoid weights (sbias given): no softmax; a visible key weighs
// sigmoid(s_ij + sbias[h]) and the weights are not normalized over the keys
// (rows and prefill kernels; no sink, no pooled entries).
//
// Three kernels:
//  * attn_mod_rows<T>: flash-decode layout. One workgroup per (q tile, kv
//    head, batch row): K/V chunks of 64 positions are staged through LDS once
//    and shared by up to 16 query rows (tokens x grouped heads); score phase =
//    one key per lane, accumulate phase = output dims across lanes with the
//    weight broadcast from a per-wave LDS slab. Used for decode, for fp32,
//    and for head sizes the MFMA kernel does not cover.
//  * attn_mod_mfma<DC,NV>: bf16 prefill on v_mfma_f32_16x16x32_bf16 — QK^T
//    and PV on the matrix cores, modifiers + online softmax in the fp32 C
//    fragments. Head sizes are zero-padded in LDS to DC*32 / NV*16.
//  * attn_mod_mfma_heads<DC,NV>: bf16 decode with >= 16 query heads per kv
//    head (latent attention's one shared row): the grouped heads are the rows
//    of the MFMA tile, split over the keys.
#include "common.h"

namespace dnet {

using bf16x8 = __attribute__((ext_vector_type(8))) __bf16;
using bf16x2 = __attribute__((ext_vector_type(2))) __bf16;
using f32x4 = __attribute__((ext_vector_type(4))) float;

namespace {

template <typename T> __device__ __forceinline__ float ldv(const T* p);
template <> __device__ __forceinline__ float ldv<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldv<short>(const short* p) { return bits2f(*p); }
template <typename T> __device__ __forceinline__ void stv(T* p, float v);
template <> __device__ __forceinline__ void stv<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stv<short>(short* p, float v) { *p = f2bits(v); }

__device__ __forceinline__ float wave_all_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float wave_all_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

// dot of two LDS rows of n elements
__device__ __forceinline__ float dot_lds(const float* a, const float* b, int n) {
  float s = 0.f;
  for (int e = 0; e < n; ++e) s = fmaf(a[e], b[e], s);
  return s;
}
__device__ __forceinline__ float dot_lds(const short* a, const short* b, int n) {
  float s = 0.f;
  if ((n & 3) == 0) {      // rows are 8 B aligned (pitch is a multiple of 4)
    for (int e = 0; e < n; e += 4) {
      const short4v ka = *reinterpret_cast<const short4v*>(a + e);
      const short4v qb = *reinterpret_cast<const short4v*>(b + e);
      s = __builtin_amdgcn_fdot2_f32_bf16(
          *reinterpret_cast<const bf16x2*>(&ka.x[0]),
          *reinterpret_cast<const bf16x2*>(&qb.x[0]), s, false);
      s = __builtin_amdgcn_fdot2_f32_bf16(
          *reinterpret_cast<const bf16x2*>(&ka.x[2]),
          *reinterpret_cast<const bf16x2*>(&qb.x[2]), s, false);
    }
  } else {
    for (int e = 0; e < n; ++e) s = fmaf(bits2f(a[e]), bits2f(b[e]), s);
  }
  return s;
}

constexpr int kChunkR = 64;   // keys per staged chunk (one per lane)
constexpr int kRowsMax = 16;  // query rows per workgroup (4 per wave)
constexpr int kHeadsMfmaMinGroup = 16;  // decode: heads per kv head from which
                                        // the matrix-core heads kernel runs

__host__ __device__ inline int pitch_of(int n, int elem) {
  // fp32: odd dword pitch; bf16: 8 B aligned rows with a 2-dword skew
  if (elem == 4) return n | 1;
  return ((n + 3) & ~3) + 4;
}

struct ModParams {
  const int* pos;
  const int* lens;
  const int* slots;
  const float* temp;
  const float* r1;
  const float* r2;
  const float* sinks;
  const void* pk;      // pooled caches (same dtype as the cache) or null
  const void* pv;
  const float* sbias;  // per-head bias of the sigmoid weights, or null
  int T, Bc, Hq, Hkv, Smax, D, DV, QT, window, pool, Sp, chunk;
  // VS: elements between consecutive value rows of the cache. vshare: the
  // values are the first DV entries of the key rows (latent attention), the
  // value pointer is the key pointer and VS = D.
  int VS, vshare;
  float scale, softcap;
};

// pooled entries visible to a query at position i
__device__ __forceinline__ int pool_count(int i, int window, int pool, int Sp) {
  if (pool <= 0 || i < 0) return 0;
  return min(Sp, max(0, (i - window + 1) / pool));
}

// transcendental flavours: fp32 models use the accurate library functions,
// bf16 models the hardware approximations (error far below bf16 rounding)
template <bool FAST> __device__ __forceinline__ float m_exp(float x) {
  return FAST ? __expf(x) : expf(x);
}
template <bool FAST> __device__ __forceinline__ float m_tanh(float x) {
  return FAST ? 1.f - 2.f * __builtin_amdgcn_rcpf(__expf(2.f * x) + 1.f)
              : tanhf(x);
}
template <bool FAST> __device__ __forceinline__ float m_sigmoid(float x) {
  return FAST ? __builtin_amdgcn_rcpf(1.f + __expf(-x))
              : 1.f / (1.f + expf(-x));
}
template <bool FAST> __device__ __forceinline__ float m_log1p(float x) {
  return FAST ? __logf(1.f + x) : log1pf(x);
}

// 16 B global -> LDS row copies (rows are 8 B aligned for bf16, 4 B for fp32)
__device__ __forceinline__ void stage16(short* dst, const short* src, bool on) {
  short8 z;
#pragma unroll
  for (int j = 0; j < 8; ++j) z.x[j] = 0;
  if (on) z = *reinterpret_cast<const short8*>(src);
  *reinterpret_cast<short4v*>(dst) = *reinterpret_cast<short4v*>(&z.x[0]);
  *reinterpret_cast<short4v*>(dst + 4) = *reinterpret_cast<short4v*>(&z.x[4]);
}
__device__ __forceinline__ void stage16(float* dst, const float* src, bool on) {
  float4 z = {0.f, 0.f, 0.f, 0.f};
  if (on) z = *reinterpret_cast<const float4*>(src);
  dst[0] = z.x; dst[1] = z.y; dst[2] = z.z; dst[3] = z.w;
}

// VEC: head sizes are multiples of 16 B -> vector staging; for bf16 the
// accumulate phase then owns output dims in pairs (one 4 B LDS read per key).
// splits > 1 (decode only): blockIdx.x is the split; chunks are dealt round
// robin and unnormalized (acc, m, l) go to `partial` [B, Hq, splits, DV+2].
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void attn_mod_rows(
    const T* __restrict__ q, const T* __restrict__ kc_tok,
    const T* __restrict__ vc_tok, T* __restrict__ out,
    float* __restrict__ partial, const int splits, const ModParams P) {
  constexpr bool FAST = sizeof(T) == 2;
  constexpr bool PAIR = VEC && sizeof(T) == 2;
  constexpr int EV = 16 / sizeof(T);
  const int b = blockIdx.z;
  const int G = P.Hq / P.Hkv;
  const int GS = (G + kRowsMax - 1) / kRowsMax;     // head-group splits
  const int hkv = blockIdx.y / GS;
  const int g0 = (blockIdx.y % GS) * kRowsMax;
  const int Gb = min(kRowsMax, G - g0);
  const int split = splits > 1 ? blockIdx.x : 0;
  const int t0 = splits > 1 ? 0 : blockIdx.x * P.QT;
  const int n = P.lens ? min(P.lens[b], P.T) : P.T;
  if (t0 >= n) return;
  const int slot = P.slots ? P.slots[b] : b;
  if (slot < 0 || slot >= P.Bc) return;
  const int p0 = P.pos[b];
  const int nt = min(P.QT, n - t0);
  const int rows = nt * Gb;
  const int D = P.D, DV = P.DV;
  const bool vshare = P.vshare != 0;
  const int PK = pitch_of(D, sizeof(T));
  const int PV = vshare ? PK : pitch_of(DV, sizeof(T));
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63;

  extern __shared__ __attribute__((aligned(16))) char smem[];
  T* k_lds = reinterpret_cast<T*>(smem);                 // [64][PK]
  // shared values: the staged key rows are read again as value rows
  T* v_lds = vshare ? k_lds : k_lds + kChunkR * PK;      // [64][PV]
  T* q_lds = k_lds + kChunkR * PK +
             (vshare ? 0 : kChunkR * PV);                // [16][PK]
  float* p_lds = reinterpret_cast<float*>(q_lds + kRowsMax * PK);  // [4][64]

  const int64_t qstride = (int64_t)P.Hq * D;
  for (int idx = threadIdx.x; idx < rows * D; idx += blockDim.x) {
    const int r = idx / D, e = idx % D;
    const int t = t0 + r / Gb, g = g0 + r % Gb;
    q_lds[r * PK + e] =
        q[((int64_t)b * P.T + t) * qstride + (int64_t)(hkv * G + g) * D + e];
  }

  // per-wave query rows r = wid + 4*rr
  float m[4], l[4], acc[4][4], tmp[4], r1[4], r2[4], sb[4];
  int qi[4], cb[4];
  const bool sig = P.sbias != nullptr;
#pragma unroll
  for (int rr = 0; rr < 4; ++rr) {
    const int r = wid + 4 * rr;
    const int rc = min(r, rows - 1);
    const int h = hkv * G + g0 + rc % Gb;
    qi[rr] = (r < rows) ? p0 + t0 + rc / Gb : -1;
    tmp[rr] = P.scale * (P.temp ? P.temp[h] : 1.f);
    r1[rr] = P.r1 ? P.r1[h] : 0.f;
    r2[rr] = P.r1 ? P.r2[h] : 0.f;
    sb[rr] = sig ? P.sbias[h] : 0.f;
    // first position of the query's block (chunked visibility)
    cb[rr] = (P.chunk > 0 && qi[rr] >= 0) ? (qi[rr] / P.chunk) * P.chunk : 0;
    m[rr] = sig ? 0.f : -1e30f;
    l[rr] = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[rr][j] = 0.f;
  }
  const float cap = P.softcap, inv_cap = cap > 0.f ? 1.f / cap : 0.f;

  const int kv_end = min(p0 + t0 + nt, P.Smax);          // exclusive
  int kv_begin = P.window > 0 ? max(0, p0 + t0 - P.window + 1) : 0;
  if (P.chunk > 0) kv_begin = max(kv_begin, ((p0 + t0) / P.chunk) * P.chunk);
  const int64_t kbase = ((int64_t)slot * P.Hkv + hkv) * P.Smax * D;
  const int64_t vbase = ((int64_t)slot * P.Hkv + hkv) * P.Smax * P.VS;
  const int VS = P.VS;

  // chunk list: pooled entries first, then the token range
  const int np_max = pool_count(p0 + t0 + nt - 1, P.window, P.pool, P.Sp);
  const int n_pc = (np_max + kChunkR - 1) / kChunkR;
  const int tok0 = kv_begin & ~(kChunkR - 1);
  const int n_tc = kv_end > tok0 ? (kv_end - tok0 + kChunkR - 1) / kChunkR : 0;
  const int64_t pkbase = ((int64_t)slot * P.Hkv + hkv) * P.Sp * D;
  const int64_t pvbase = ((int64_t)slot * P.Hkv + hkv) * P.Sp * DV;

  for (int c = split; c < n_pc + n_tc; c += splits) {
    const bool pooled = c < n_pc;
    const int s0 = pooled ? c * kChunkR : tok0 + (c - n_pc) * kChunkR;
    const int valid = min(kChunkR, (pooled ? np_max : kv_end) - s0);
    const T* kc = pooled ? reinterpret_cast<const T*>(P.pk) + pkbase
                         : kc_tok + kbase;
    const T* vc = pooled ? reinterpret_cast<const T*>(P.pv) + pvbase
                         : vc_tok + vbase;   // (pooled entries: VS == DV)
    __syncthreads();          // previous chunk consumed (and q staged)
    if (VEC) {
      const int dk = D / EV, dvv = DV / EV;
      for (int idx = threadIdx.x; idx < kChunkR * dk; idx += blockDim.x) {
        const int r = idx / dk, e = (idx % dk) * EV;
        stage16(&k_lds[r * PK + e], &kc[(int64_t)(s0 + r) * D + e],
                r < valid);
      }
      if (!vshare)
        for (int idx = threadIdx.x; idx < kChunkR * dvv; idx += blockDim.x) {
          const int r = idx / dvv, e = (idx % dvv) * EV;
          stage16(&v_lds[r * PV + e], &vc[(int64_t)(s0 + r) * VS + e],
                  r < valid);
        }
    } else {
      for (int idx = threadIdx.x; idx < kChunkR * D; idx += blockDim.x) {
        const int r = idx / D, e = idx % D;
        k_lds[r * PK + e] =
            r < valid ? kc[(int64_t)(s0 + r) * D + e] : (T)0;
      }
      if (!vshare)
        for (int idx = threadIdx.x; idx < kChunkR * DV; idx += blockDim.x) {
          const int r = idx / DV, e = idx % DV;
          v_lds[r * PV + e] =
              r < valid ? vc[(int64_t)(s0 + r) * VS + e] : (T)0;
        }
    }
    __syncthreads();
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
      const int i = qi[rr];
      // entries of this chunk's source that row i may see: [0, lim)
      const int lim = pooled ? pool_count(i, P.window, P.pool, P.Sp) : i + 1;
      if (lim <= s0) continue;              // wave-uniform: nothing visible
      const int r = wid + 4 * rr;
      const int j = s0 + lane;
      bool live = lane < valid && j < lim;
      if (!pooled && P.window > 0) live = live && (j > i - P.window);
      if (P.chunk > 0) live = live && (j >= cb[rr]);
      float s = dot_lds(&k_lds[lane * PK], &q_lds[r * PK], D) * tmp[rr];
      if (cap > 0.f) s = cap * m_tanh<FAST>(s * inv_cap);
      if (P.r1 && !pooled)
        s -= r1[rr] * m_log1p<FAST>(r2[rr] * (float)max(i - j, 0));
      float alpha, p;
      if (sig) {                            // wave-uniform
        alpha = 1.f;
        p = live ? m_sigmoid<FAST>(s + sb[rr]) : 0.f;
      } else {
        if (!live) s = -INFINITY;
        const float mn = fmaxf(m[rr], wave_all_max(s));
        alpha = m_exp<FAST>(m[rr] - mn);
        p = live ? m_exp<FAST>(s - mn) : 0.f;
        l[rr] = l[rr] * alpha + wave_all_sum(p);
        m[rr] = mn;
      }
      p_lds[wid * kChunkR + lane] = p;
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // wave-local slab
      const int vis = min(valid, lim - s0);
      const float* pw = &p_lds[wid * kChunkR];
      if (PAIR) {
        // lane owns dims (2*lane, 2*lane+1) + 128*jj
#pragma unroll
        for (int jj = 0; jj < 2; ++jj) {
          const int dv = 2 * lane + 128 * jj;
          if (dv < DV) {
            float a0 = acc[rr][2 * jj] * alpha, a1 = acc[rr][2 * jj + 1] * alpha;
            const short* vcol = reinterpret_cast<const short*>(v_lds) + dv;
#pragma unroll 4
            for (int s2 = 0; s2 < vis; ++s2) {
              const unsigned pr =
                  *reinterpret_cast<const unsigned*>(vcol + s2 * PV);
              const float ps = pw[s2];
              union { unsigned u; float f; } lo, hi;
              lo.u = pr << 16;
              hi.u = pr & 0xffff0000u;
              a0 = fmaf(ps, lo.f, a0);
              a1 = fmaf(ps, hi.f, a1);
            }
            acc[rr][2 * jj] = a0;
            acc[rr][2 * jj + 1] = a1;
          }
        }
      } else {
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const int dv = lane + 64 * jj;
          if (dv < DV) {
            float a = acc[rr][jj] * alpha;
#pragma unroll 4
            for (int s2 = 0; s2 < vis; ++s2)
              a = fmaf(pw[s2], ldv<T>(&v_lds[s2 * PV + dv]), a);
            acc[rr][jj] = a;
          }
        }
      }
    }
  }

#pragma unroll
  for (int rr = 0; rr < 4; ++rr) {
    const int r = wid + 4 * rr;
    if (r >= rows) continue;
    const int t = t0 + r / Gb, h = hkv * G + g0 + r % Gb;
    if (splits > 1) {
      float* pp = partial +
                  (((int64_t)b * P.Hq + h) * splits + split) * (DV + 2);
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        if (PAIR) {
          const int dv = 2 * lane + 128 * (jj >> 1) + (jj & 1);
          if (dv < DV) pp[dv] = acc[rr][jj];
        } else {
          const int dv = lane + 64 * jj;
          if (dv < DV) pp[dv] = acc[rr][jj];
        }
      }
      if (lane == 0) {
        pp[DV] = m[rr];
        pp[DV + 1] = l[rr];
      }
      continue;
    }
    float c = 1.f;
    if (P.sinks) {
      const float sk = P.sinks[h];
      const float m2 = fmaxf(m[rr], sk);
      c = m_exp<FAST>(m[rr] - m2);
      l[rr] = l[rr] * c + m_exp<FAST>(sk - m2);
    }
    const float inv = sig ? 1.f : (l[rr] > 0.f ? c / l[rr] : 0.f);
    T* op = out + ((int64_t)b * P.T + t) * P.Hq * DV + (int64_t)h * DV;
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      if (PAIR) {
        const int dv = 2 * lane + 128 * (jj >> 1) + (jj & 1);
        if (dv < DV) stv<T>(op + dv, acc[rr][jj] * inv);
      } else {
        const int dv = lane + 64 * jj;
        if (dv < DV) stv<T>(op + dv, acc[rr][jj] * inv);
      }
    }
  }
}

// merge the splits of one (batch row, head): one wave per output row
template <typename T>
__global__ __launch_bounds__(64) void attn_mod_combine(
    const float* __restrict__ partial, T* __restrict__ out,
    const float* __restrict__ sinks, const int* __restrict__ pos,
    const int* __restrict__ slots, const int Hq, const int DV,
    const int splits, const int Bc, const int plain_sum) {
  const int b = blockIdx.x / Hq, h = blockIdx.x % Hq;
  const float* pp = partial + (int64_t)blockIdx.x * splits * (DV + 2);
  if (plain_sum) {             // unnormalized weights: the splits just add
    for (int dv = threadIdx.x; dv < DV; dv += 64) {
      float a = 0.f;
      for (int s = 0; s < splits; ++s) a += pp[s * (DV + 2) + dv];
      stv<T>(out + (int64_t)blockIdx.x * DV + dv, a);
    }
    return;
  }
  float M = -1e30f;
  for (int s = 0; s < splits; ++s) M = fmaxf(M, pp[s * (DV + 2) + DV]);
  if (sinks) M = fmaxf(M, sinks[h]);
  float L = sinks ? expf(sinks[h] - M) : 0.f;
  for (int s = 0; s < splits; ++s)
    L += pp[s * (DV + 2) + DV + 1] * expf(pp[s * (DV + 2) + DV] - M);
  const float inv = L > 0.f ? 1.f / L : 0.f;
  for (int dv = threadIdx.x; dv < DV; dv += 64) {
    float a = 0.f;
    for (int s = 0; s < splits; ++s)
      a += pp[s * (DV + 2) + dv] * expf(pp[s * (DV + 2) + DV] - M);
    stv<T>(out + (int64_t)blockIdx.x * DV + dv, a * inv);
  }
}

// ---- bf16 prefill on the matrix cores -------------------------------------
// Block = 4 waves, each owning 16 query tokens of a 64-token tile of one
// head (grid = token tiles x Hq x batch rows). Per 32-key tile the waves
// stage K [32][DC*32] and V transposed [NV*16][32] in LDS (head sizes
// zero-padded), QK^T = 2 x DC MFMAs into fp32 C fragments (lane holds
// q = hi*4+r, key = lane&15), modifiers + online softmax on the fragments,
// P relayed through a per-wave LDS slab as the A operand of NV PV MFMAs.
__device__ __forceinline__ float fast_tanh(float x) {
  // 1 - 2/(e^{2x}+1): saturates cleanly (e^{2x} -> inf or 0)
  return 1.f - 2.f * __builtin_amdgcn_rcpf(__expf(2.f * x) + 1.f);
}

template <int DC, int NV>
__global__ __launch_bounds__(256) void attn_mod_mfma(
    const short* __restrict__ q, const short* __restrict__ kc,
    const short* __restrict__ vc, short* __restrict__ out,
    const ModParams P) {
  constexpr int ST = 32;
  constexpr int DP = DC * 32, DVP = NV * 16;
  constexpr int KP = DP + 8, SP = ST + 8;
  __shared__ short k_lds[ST * KP];
  __shared__ short vt_lds[DVP * SP];
  __shared__ short p_lds[4][16 * SP];

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int h = blockIdx.y, b = blockIdx.z;
  const int hk = h / (P.Hq / P.Hkv);
  const int D = P.D, DV = P.DV;
  const int n = P.lens ? min(P.lens[b], P.T) : P.T;
  const int tile0 = blockIdx.x * 64;
  if (tile0 >= n) return;
  const int slot = P.slots ? P.slots[b] : b;
  if (slot < 0 || slot >= P.Bc) return;
  const int p0 = P.pos[b];
  const int qt = tile0 + wave * 16;
  const int row = lane & 15, hi = lane >> 4;
  const int qrow = min(qt + row, n - 1);
  const short* qp = q + ((int64_t)b * P.T + qrow) * P.Hq * D + (int64_t)h * D;
  const short* kp = kc + ((int64_t)slot * P.Hkv + hk) * P.Smax * D;
  const int VS = P.VS;
  const short* vp = vc + ((int64_t)slot * P.Hkv + hk) * P.Smax * VS;

  bf16x8 qf[DC];
#pragma unroll
  for (int c = 0; c < DC; ++c) {
    const int e0 = c * 32 + hi * 8;
    short8 z;
#pragma unroll
    for (int j = 0; j < 8; ++j) z.x[j] = 0;
    if (e0 < D) z = *reinterpret_cast<const short8*>(&qp[e0]);
    qf[c] = *reinterpret_cast<const bf16x8*>(&z);
  }
  f32x4 acc[NV];
#pragma unroll
  for (int nn = 0; nn < NV; ++nn) acc[nn] = {0.f, 0.f, 0.f, 0.f};
  float m_run[4], l_run[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    m_run[r] = -1e30f;
    l_run[r] = 0.f;
  }
  const float sc_t = P.scale * (P.temp ? P.temp[h] : 1.f);
  const float cap = P.softcap, inv_cap = cap > 0.f ? 1.f / cap : 0.f;
  const float r1 = P.r1 ? P.r1[h] : 0.f, r2 = P.r1 ? P.r2[h] : 0.f;
  const bool sig = P.sbias != nullptr;
  const float sbias = sig ? P.sbias[h] : 0.f;

  const int q_hi = min(tile0 + 63, n - 1);
  const short* kp_tok = kp;
  const short* vp_tok = vp;

  // phase 0: pooled entries (block means before the window); phase 1: tokens
  for (int ph = P.pool > 0 ? 0 : 1; ph < 2; ++ph) {
  const bool pooled = ph == 0;
  const int Sdim = pooled ? P.Sp : P.Smax;
  const int s_end = pooled ? pool_count(p0 + q_hi, P.window, P.pool, P.Sp)
                           : min(P.Smax, p0 + q_hi + 1);
  int s_begin = 0;
  if (!pooled && P.window > 0)
    s_begin = max(0, p0 + tile0 - P.window + 1) & ~(ST - 1);
  if (!pooled && P.chunk > 0)
    s_begin = max(s_begin, (((p0 + tile0) / P.chunk) * P.chunk) & ~(ST - 1));
  kp = pooled ? reinterpret_cast<const short*>(P.pk) +
                    ((int64_t)slot * P.Hkv + hk) * P.Sp * D
              : kp_tok;
  vp = pooled ? reinterpret_cast<const short*>(P.pv) +
                    ((int64_t)slot * P.Hkv + hk) * P.Sp * DV
              : vp_tok;

  for (int s0 = s_begin; s0 < s_end; s0 += ST) {
    __syncthreads();
    for (int idx = threadIdx.x; idx < ST * (DP / 8); idx += 256) {
      const int sr = idx / (DP / 8), dc = (idx % (DP / 8)) * 8;
      const int sg = min(s0 + sr, Sdim - 1);
      short8 z;
#pragma unroll
      for (int j = 0; j < 8; ++j) z.x[j] = 0;
      if (dc < D) z = *reinterpret_cast<const short8*>(&kp[(int64_t)sg * D + dc]);
      *reinterpret_cast<short8*>(&k_lds[sr * KP + dc]) = z;
    }
    for (int idx = threadIdx.x; idx < ST * (DVP / 2); idx += 256) {
      const int sr = idx / (DVP / 2), dc = (idx % (DVP / 2)) * 2;
      const int sg = min(s0 + sr, Sdim - 1);
      short v0 = 0, v1 = 0;
      if (dc < DV) {              // DV is even (multiple of 8)
        v0 = vp[(int64_t)sg * VS + dc];
        v1 = vp[(int64_t)sg * VS + dc + 1];
      }
      vt_lds[dc * SP + sr] = v0;
      vt_lds[(dc + 1) * SP + sr] = v1;
    }
    __syncthreads();

    float p_val[2][4], m_new[4];
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      f32x4 sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(
            &k_lds[(sub * 16 + row) * KP + c * 32 + hi * 8]);
        sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[c], kf, sc, 0, 0, 0);
      }
      const int j = s0 + sub * 16 + row;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int qq = qt + hi * 4 + r;
        const int i = p0 + qq;
        float val = sc[r] * sc_t;
        if (cap > 0.f) val = cap * fast_tanh(val * inv_cap);
        bool dead;
        if (pooled) {
          dead = (qq >= n) || (j >= pool_count(i, P.window, P.pool, P.Sp));
        } else {
          if (P.r1) val -= r1 * __logf(1.f + r2 * (float)max(i - j, 0));
          dead = (j > i) || (qq >= n) || (j >= P.Smax);
          if (P.window > 0) dead |= (j <= i - P.window);
          if (P.chunk > 0) dead |= (j < (i / P.chunk) * P.chunk);
        }
        if (sig)
          p_val[sub][r] =
              dead ? 0.f : __builtin_amdgcn_rcpf(1.f + __expf(-(val + sbias)));
        else
          p_val[sub][r] = dead ? -INFINITY : val;
      }
    }
    if (!sig)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float mx = fmaxf(p_val[0][r], p_val[1][r]);
#pragma unroll
      for (int off = 8; off > 0; off >>= 1)
        mx = fmaxf(mx, __shfl_xor(mx, off, 16));
      m_new[r] = fmaxf(m_run[r], mx);
      const float corr = __expf(m_run[r] - m_new[r]);
      float ls = 0.f;
#pragma unroll
      for (int sub = 0; sub < 2; ++sub) {
        p_val[sub][r] = __expf(p_val[sub][r] - m_new[r]);
        ls += p_val[sub][r];
      }
#pragma unroll
      for (int off = 8; off > 0; off >>= 1) ls += __shfl_xor(ls, off, 16);
      l_run[r] = l_run[r] * corr + ls;
      m_run[r] = m_new[r];
#pragma unroll
      for (int nn = 0; nn < NV; ++nn) acc[nn][r] *= corr;
    }
#pragma unroll
    for (int sub = 0; sub < 2; ++sub)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        p_lds[wave][(hi * 4 + r) * SP + sub * 16 + row] =
            f2bits(p_val[sub][r]);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // wave-local slab
    const bf16x8 pf =
        *reinterpret_cast<const bf16x8*>(&p_lds[wave][row * SP + hi * 8]);
#pragma unroll
    for (int nn = 0; nn < NV; ++nn) {
      const bf16x8 vf = *reinterpret_cast<const bf16x8*>(
          &vt_lds[(nn * 16 + row) * SP + hi * 8]);
      acc[nn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vf, acc[nn], 0,
                                                        0, 0);
    }
  }
  }  // phases

#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int qq = qt + hi * 4 + r;
    if (qq >= n) continue;
    float c = 1.f;
    if (P.sinks) {
      const float sk = P.sinks[h];
      const float m2 = fmaxf(m_run[r], sk);
      c = __expf(m_run[r] - m2);
      l_run[r] = l_run[r] * c + __expf(sk - m2);
    }
    const float inv = sig ? 1.f : (l_run[r] > 0.f ? c / l_run[r] : 0.f);
    short* op = out + ((int64_t)b * P.T + qq) * P.Hq * DV + (int64_t)h * DV;
#pragma unroll
    for (int nn = 0; nn < NV; ++nn) {
      const int dv = nn * 16 + row;
      if (dv < DV) op[dv] = f2bits(acc[nn][r] * inv);
    }
  }
}

// ---- bf16 decode of grouped heads on the matrix cores ----------------------
// One token per batch row (T = 1) and many query heads per kv head (latent
// attention: every head reads the one shared row): the G grouped heads are
// the 16 rows of a wave's MFMA tile (4 waves = 64 heads per block), so a
// staged 32-key K/V tile is used by all of them. grid (splits, Hkv * head
// tiles, B); key tiles are dealt round robin to the splits and unnormalized
// (acc, m, l) go to `partial` [B, Hq, splits, DV+2] for attn_mod_combine
// (which also adds the sink). No pooled entries.
template <int DC, int NV>
__global__ __launch_bounds__(256) void attn_mod_mfma_heads(
    const short* __restrict__ q, const short* __restrict__ kc,
    const short* __restrict__ vc, float* __restrict__ partial,
    const int splits, const ModParams P) {
  constexpr int ST = 32;
  constexpr int DP = DC * 32, DVP = NV * 16;
  constexpr int KP = DP + 8, SP = ST + 8;
  __shared__ short k_lds[ST * KP];
  __shared__ short vt_lds[DVP * SP];
  __shared__ short p_lds[4][16 * SP];

  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int split = blockIdx.x, b = blockIdx.z;
  const int G = P.Hq / P.Hkv;
  const int GT = (G + 63) / 64;
  const int hk = blockIdx.y / GT;
  const int gw = (blockIdx.y % GT) * 64 + wave * 16;   // wave's first head
  const int D = P.D, DV = P.DV, VS = P.VS;
  if (P.lens && P.lens[b] <= 0) return;                // idle row
  const int slot = P.slots ? P.slots[b] : b;
  if (slot < 0 || slot >= P.Bc) return;
  const int i = P.pos[b];                              // the query's position
  const int row = lane & 15, hi = lane >> 4;
  const int hrow = hk * G + min(gw + row, G - 1);
  const short* qp = q + ((int64_t)b * P.Hq + hrow) * D;
  const short* kp = kc + ((int64_t)slot * P.Hkv + hk) * P.Smax * D;
  const short* vp = vc + ((int64_t)slot * P.Hkv + hk) * P.Smax * VS;

  bf16x8 qf[DC];
#pragma unroll
  for (int c = 0; c < DC; ++c) {
    const int e0 = c * 32 + hi * 8;
    short8 z;
#pragma unroll
    for (int j = 0; j < 8; ++j) z.x[j] = 0;
    if (e0 < D) z = *reinterpret_cast<const short8*>(&qp[e0]);
    qf[c] = *reinterpret_cast<const bf16x8*>(&z);
  }
  f32x4 acc[NV];
#pragma unroll
  for (int nn = 0; nn < NV; ++nn) acc[nn] = {0.f, 0.f, 0.f, 0.f};
  float m_run[4], l_run[4], sc_t[4], r1[4], r2[4];
  bool alive[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int g = gw + hi * 4 + r;
    alive[r] = g < G;
    const int h = hk * G + min(g, G - 1);
    sc_t[r] = P.scale * (P.temp ? P.temp[h] : 1.f);
    r1[r] = P.r1 ? P.r1[h] : 0.f;
    r2[r] = P.r1 ? P.r2[h] : 0.f;
    m_run[r] = -1e30f;
    l_run[r] = 0.f;
  }
  const float cap = P.softcap, inv_cap = cap > 0.f ? 1.f / cap : 0.f;

  const int s_end = min(P.Smax, i + 1);
  const int s_begin = P.window > 0 ? (max(0, i - P.window + 1) & ~(ST - 1)) : 0;
  const int tiles = s_end > s_begin ? (s_end - s_begin + ST - 1) / ST : 0;

  // the next tile's key rows travel from memory into registers while the
  // current tile is worked on
  constexpr int KV = ST * (DP / 8) / 256;       // 16 B pieces per thread
  short8 kreg[KV];
  auto load_tile = [&](const int s0) {
#pragma unroll
    for (int v = 0; v < KV; ++v) {
      const int idx = threadIdx.x + v * 256;
      const int sr = idx / (DP / 8), dc = (idx % (DP / 8)) * 8;
      const int sg = min(s0 + sr, P.Smax - 1);
      short8 z;
#pragma unroll
      for (int j = 0; j < 8; ++j) z.x[j] = 0;
      if (dc < D) z = *reinterpret_cast<const short8*>(&kp[(int64_t)sg * D + dc]);
      kreg[v] = z;
    }
  };
  if (split < tiles) load_tile(s_begin + split * ST);

  for (int tile = split; tile < tiles; tile += splits) {
    const int s0 = s_begin + tile * ST;
    __syncthreads();
#pragma unroll
    for (int v = 0; v < KV; ++v) {
      const int idx = threadIdx.x + v * 256;
      const int sr = idx / (DP / 8), dc = (idx % (DP / 8)) * 8;
      *reinterpret_cast<short8*>(&k_lds[sr * KP + dc]) = kreg[v];
    }
    if (tile + splits < tiles) load_tile(s0 + splits * ST);
    if (P.vshare) {
      // the staged key rows are the values: transpose them inside LDS, the
      // 32 keys of a value dimension across neighbouring lanes (consecutive
      // writes, key rows 4 banks apart for the reads)
      __syncthreads();
      for (int idx = threadIdx.x; idx < ST * (DVP / 2); idx += 256) {
        const int sr = idx % ST, dc = (idx / ST) * 2;
        unsigned pr = 0;
        if (dc < DV)              // DV is even (multiple of 8)
          pr = *reinterpret_cast<const unsigned*>(&k_lds[sr * KP + dc]);
        vt_lds[dc * SP + sr] = (short)(pr & 0xffffu);
        vt_lds[(dc + 1) * SP + sr] = (short)(pr >> 16);
      }
    } else {
      for (int idx = threadIdx.x; idx < ST * (DVP / 2); idx += 256) {
        const int sr = idx / (DVP / 2), dc = (idx % (DVP / 2)) * 2;
        const int sg = min(s0 + sr, P.Smax - 1);
        short v0 = 0, v1 = 0;
        if (dc < DV) {            // DV is even (multiple of 8)
          v0 = vp[(int64_t)sg * VS + dc];
          v1 = vp[(int64_t)sg * VS + dc + 1];
        }
        vt_lds[dc * SP + sr] = v0;
        vt_lds[(dc + 1) * SP + sr] = v1;
      }
    }
    __syncthreads();

    float p_val[2][4], m_new[4];
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      f32x4 sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < DC; ++c) {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(
            &k_lds[(sub * 16 + row) * KP + c * 32 + hi * 8]);
        sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[c], kf, sc, 0, 0, 0);
      }
      const int j = s0 + sub * 16 + row;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float val = sc[r] * sc_t[r];
        if (cap > 0.f) val = cap * fast_tanh(val * inv_cap);
        if (P.r1) val -= r1[r] * __logf(1.f + r2[r] * (float)max(i - j, 0));
        bool dead = (j > i) || (j >= P.Smax) || !alive[r];
        if (P.window > 0) dead |= (j <= i - P.window);
        p_val[sub][r] = dead ? -INFINITY : val;
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float mx = fmaxf(p_val[0][r], p_val[1][r]);
#pragma unroll
      for (int off = 8; off > 0; off >>= 1)
        mx = fmaxf(mx, __shfl_xor(mx, off, 16));
      m_new[r] = fmaxf(m_run[r], mx);
      const float corr = __expf(m_run[r] - m_new[r]);
      float ls = 0.f;
#pragma unroll
      for (int sub = 0; sub < 2; ++sub) {
        p_val[sub][r] = __expf(p_val[sub][r] - m_new[r]);
        ls += p_val[sub][r];
      }
#pragma unroll
      for (int off = 8; off > 0; off >>= 1) ls += __shfl_xor(ls, off, 16);
      l_run[r] = l_run[r] * corr + ls;
      m_run[r] = m_new[r];
#pragma unroll
      for (int nn = 0; nn < NV; ++nn) acc[nn][r] *= corr;
    }
#pragma unroll
    for (int sub = 0; sub < 2; ++sub)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        p_lds[wave][(hi * 4 + r) * SP + sub * 16 + row] =
            f2bits(p_val[sub][r]);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // wave-local slab
    const bf16x8 pf =
        *reinterpret_cast<const bf16x8*>(&p_lds[wave][row * SP + hi * 8]);
#pragma unroll
    for (int nn = 0; nn < NV; ++nn) {
      const bf16x8 vf = *reinterpret_cast<const bf16x8*>(
          &vt_lds[(nn * 16 + row) * SP + hi * 8]);
      acc[nn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vf, acc[nn], 0,
                                                        0, 0);
    }
  }

  // a split without tiles still reports its neutral (0, -1e30, 0)
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    if (!alive[r]) continue;
    const int h = hk * G + gw + hi * 4 + r;
    float* pp = partial + (((int64_t)b * P.Hq + h) * splits + split) * (DV + 2);
#pragma unroll
    for (int nn = 0; nn < NV; ++nn) {
      const int dv = nn * 16 + row;
      if (dv < DV) pp[dv] = acc[nn][r];
    }
    if (row == 0) {
      pp[DV] = m_run[r];
      pp[DV + 1] = l_run[r];
    }
  }
}

}  // namespace

static const float* opt_f32(const c10::optional<torch::Tensor>& t, int64_t n,
                            const char* what) {
  if (!t.has_value()) return nullptr;
  DNET_CHECK(t->scalar_type() == torch::kFloat32 && t->is_contiguous() &&
                 t->numel() == n, what);
  return t->data_ptr<float>();
}
static const int* opt_i32(const c10::optional<torch::Tensor>& t, int64_t n,
                          const char* what) {
  if (!t.has_value()) return nullptr;
  DNET_CHECK(t->scalar_type() == torch::kInt32 && t->is_contiguous() &&
                 t->numel() >= n, what);
  return t->data_ptr<int>();
}

void attn_mod(torch::Tensor q, torch::Tensor kcache,
              c10::optional<torch::Tensor> vcache_opt,
              torch::Tensor pos, c10::optional<torch::Tensor> lens,
              c10::optional<torch::Tensor> slots, torch::Tensor out,
              int64_t T, double scale, c10::optional<torch::Tensor> temp,
              double softcap, c10::optional<torch::Tensor> dist_r1,
              c10::optional<torch::Tensor> dist_r2,
              c10::optional<torch::Tensor> sinks, int64_t window,
              c10::optional<torch::Tensor> partials, int64_t splits,
              c10::optional<torch::Tensor> pool_k,
              c10::optional<torch::Tensor> pool_v, int64_t pool,
              int64_t v_dim, int64_t chunk,
              c10::optional<torch::Tensor> sig_bias) {
  // no value cache: values = the first v_dim entries of the key rows
  const bool vshare = !vcache_opt.has_value();
  const torch::Tensor& vcache = vshare ? kcache : *vcache_opt;
  DNET_CHECK(kcache.dim() == 4 && vcache.dim() == 4 &&
                 kcache.is_contiguous() && vcache.is_contiguous(), "cache");
  const int Bc = kcache.size(0), Hkv = kcache.size(1), Smax = kcache.size(2);
  const int D = kcache.size(3);
  const int DV = vshare ? (int)v_dim : (int)vcache.size(3);
  DNET_CHECK(vcache.size(0) == Bc && vcache.size(1) == Hkv &&
                 vcache.size(2) == Smax, "k/v cache shapes differ");
  DNET_CHECK(!vshare || (DV >= 1 && DV <= D && pool == 0),
             "shared values: 1 <= v_dim <= key size, no pooled blocks");
  const int64_t M = q.size(0);
  DNET_CHECK(T > 0 && M % T == 0, "rows = B*T");
  const int64_t B = M / T;
  DNET_CHECK(q.dim() == 2 && q.is_contiguous() && q.size(1) % D == 0,
             "q [B*T, Hq*D]");
  const int Hq = q.size(1) / D;
  DNET_CHECK(Hq % Hkv == 0, "grouped heads");
  DNET_CHECK(out.is_contiguous() && out.size(0) == M &&
                 out.size(1) == (int64_t)Hq * DV, "out [B*T, Hq*DV]");
  DNET_CHECK(q.scalar_type() == kcache.scalar_type() &&
                 q.scalar_type() == vcache.scalar_type() &&
                 q.scalar_type() == out.scalar_type(), "dtypes");
  DNET_CHECK(D >= 1 && D <= 256 && DV >= 1 && DV <= 256, "head sizes <= 256");
  DNET_CHECK(dist_r1.has_value() == dist_r2.has_value(), "r1 and r2");
  if (!slots.has_value()) DNET_CHECK(B <= Bc, "more rows than cache slots");
  if (M == 0) return;
  ModParams P;
  P.pos = opt_i32(pos, B, "pos int32 [B]");
  P.lens = opt_i32(lens, B, "lens int32 [B]");
  P.slots = opt_i32(slots, B, "slots int32 [B]");
  P.temp = opt_f32(temp, Hq, "temp fp32 [Hq]");
  P.r1 = opt_f32(dist_r1, Hq, "r1 fp32 [Hq]");
  P.r2 = opt_f32(dist_r2, Hq, "r2 fp32 [Hq]");
  P.sinks = opt_f32(sinks, Hq, "sinks fp32 [Hq]");
  P.sbias = opt_f32(sig_bias, Hq, "sig_bias fp32 [Hq]");
  P.chunk = (int)std::max<int64_t>(0, chunk);
  const bool sig = P.sbias != nullptr;
  DNET_CHECK(!sig || (!sinks.has_value() && pool == 0),
             "sigmoid weights take no sink and no pooled entries");
  DNET_CHECK(P.chunk == 0 || pool == 0, "chunks take no pooled entries");
  P.T = (int)T; P.Bc = Bc; P.Hq = Hq; P.Hkv = Hkv; P.Smax = Smax;
  P.D = D; P.DV = DV; P.window = (int)window;
  P.VS = vshare ? D : DV; P.vshare = vshare ? 1 : 0;
  P.scale = (float)scale; P.softcap = (float)softcap;
  P.pk = P.pv = nullptr;
  P.pool = 0; P.Sp = 0;
  if (pool > 0) {
    DNET_CHECK(window > 0, "pooled blocks need a window");
    DNET_CHECK(pool_k.has_value() && pool_v.has_value(), "pooled caches");
    DNET_CHECK(pool_k->dim() == 4 && pool_k->is_contiguous() &&
                   pool_v->dim() == 4 && pool_v->is_contiguous() &&
                   pool_k->size(0) == Bc && pool_k->size(1) == Hkv &&
                   pool_k->size(3) == D && pool_v->size(0) == Bc &&
                   pool_v->size(1) == Hkv && pool_v->size(3) == DV &&
                   pool_v->size(2) == pool_k->size(2) &&
                   pool_k->scalar_type() == kcache.scalar_type() &&
                   pool_v->scalar_type() == kcache.scalar_type(),
               "pooled caches [Bc, Hkv, Sp, D|DV] in the cache dtype");
    P.pk = pool_k->data_ptr();
    P.pv = pool_v->data_ptr();
    P.pool = (int)pool;
    P.Sp = (int)pool_k->size(2);
  }
  const int G = Hq / Hkv;
  const int GS = (G + kRowsMax - 1) / kRowsMax;
  P.QT = std::max(1, kRowsMax / std::min(G, kRowsMax));
  auto stream = current_stream();
  const bool f32 = q.scalar_type() == torch::kFloat32;
  DNET_CHECK(f32 || q.scalar_type() == torch::kBFloat16, "bf16 or fp32");
  const int es = f32 ? 4 : 2;
  const int PK = pitch_of(D, es), PV = pitch_of(DV, es);
  const size_t lds = (size_t)es * (kChunkR * PK + (vshare ? 0 : kChunkR * PV) +
                                   kRowsMax * PK) + sizeof(float) * 4 * kChunkR;
  DNET_CHECK(lds <= 160 * 1024, "attn_mod: head sizes exceed LDS");
  const dim3 grid((unsigned)((T + P.QT - 1) / P.QT), (unsigned)(Hkv * GS),
                  (unsigned)B);
  // bf16 decode with many heads per kv head: the grouped heads are the rows
  // of the matrix-core tile (the Python side sizes `partials` by the same
  // rule: attn_mod_heads_on_mfma)
  if (!f32 && T == 1 && G >= kHeadsMfmaMinGroup && pool == 0 && !sig &&
      P.chunk == 0 && D % 8 == 0 && DV % 8 == 0) {
    const int ns = (int)std::max<int64_t>(1, splits);
    DNET_CHECK(partials.has_value() &&
                   partials->scalar_type() == torch::kFloat32 &&
                   partials->is_contiguous() &&
                   partials->numel() >= B * Hq * ns * (int64_t)(DV + 2),
               "partials fp32 [B, Hq, splits, DV+2]");
    float* part = partials->data_ptr<float>();
    const int GT = (G + 63) / 64;
    const dim3 hgrid((unsigned)ns, (unsigned)(Hkv * GT), (unsigned)B);
#define AH(DCC, NVV)                                                         \
  hipLaunchKernelGGL((attn_mod_mfma_heads<DCC, NVV>), hgrid, dim3(256), 0,   \
                     stream, (const short*)q.data_ptr(),                     \
                     (const short*)kcache.data_ptr(),                        \
                     (const short*)vcache.data_ptr(), part, ns, P)
#define AH_V(DCC)                          \
  do {                                     \
    if (DV <= 64) AH(DCC, 4);              \
    else if (DV <= 128) AH(DCC, 8);        \
    else if (DV <= 192) AH(DCC, 12);       \
    else AH(DCC, 16);                      \
  } while (0)
    if (D <= 64) AH_V(2);
    else if (D <= 128) AH_V(4);
    else if (D <= 192) AH_V(6);
    else AH_V(8);
#undef AH_V
#undef AH
    hipLaunchKernelGGL((attn_mod_combine<short>), dim3((unsigned)(B * Hq)),
                       dim3(64), 0, stream, part, (short*)out.data_ptr(),
                       P.sinks, P.pos, P.slots, Hq, DV, ns, Bc, 0);
    return;
  }
  // bf16 prompts: matrix-core kernel (head sizes padded to its tile classes)
  if (!f32 && T >= 16 && D % 8 == 0 && DV % 8 == 0) {
    const dim3 mgrid((unsigned)((T + 63) / 64), (unsigned)Hq, (unsigned)B);
#define AM(DCC, NVV)                                                         \
  hipLaunchKernelGGL((attn_mod_mfma<DCC, NVV>), mgrid, dim3(256), 0, stream, \
                     (const short*)q.data_ptr(),                             \
                     (const short*)kcache.data_ptr(),                        \
                     (const short*)vcache.data_ptr(), (short*)out.data_ptr(), \
                     P)
#define AM_V(DCC)                          \
  do {                                     \
    if (DV <= 64) AM(DCC, 4);              \
    else if (DV <= 128) AM(DCC, 8);        \
    else if (DV <= 192) AM(DCC, 12);       \
    else AM(DCC, 16);                      \
  } while (0)
    if (D <= 64) AM_V(2);
    else if (D <= 128) AM_V(4);
    else if (D <= 192) AM_V(6);
    else AM_V(8);
#undef AM_V
#undef AM
    return;
  }
  // split-KV (decode only): more workgroups when batch x kv heads is small
  int ns = (int)std::max<int64_t>(1, splits);
  float* part = nullptr;
  if (T != 1) ns = 1;
  if (ns > 1) {
    DNET_CHECK(partials.has_value() &&
                   partials->scalar_type() == torch::kFloat32 &&
                   partials->is_contiguous() &&
                   partials->numel() >= B * Hq * ns * (int64_t)(DV + 2),
               "partials fp32 [B, Hq, splits, DV+2]");
    part = partials->data_ptr<float>();
  }
  const dim3 rgrid(ns > 1 ? (unsigned)ns : grid.x, grid.y, grid.z);
  const bool vec = (D * es) % 16 == 0 && (DV * es) % 16 == 0;
#define AR(TT, VV)                                                          \
  do {                                                                      \
    if (lds > 64 * 1024)                                                    \
      DNET_CHECK_HIP(hipFuncSetAttribute(                                   \
          (const void*)attn_mod_rows<TT, VV>,                               \
          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));           \
    hipLaunchKernelGGL((attn_mod_rows<TT, VV>), rgrid, dim3(256), lds,      \
                       stream, (const TT*)q.data_ptr(),                     \
                       (const TT*)kcache.data_ptr(),                        \
                       (const TT*)vcache.data_ptr(), (TT*)out.data_ptr(),   \
                       part, ns, P);                                        \
    if (ns > 1)                                                             \
      hipLaunchKernelGGL((attn_mod_combine<TT>), dim3((unsigned)(B * Hq)),  \
                         dim3(64), 0, stream, part, (TT*)out.data_ptr(),    \
                         P.sinks, P.pos, P.slots, Hq, DV, ns, Bc,           \
                         sig ? 1 : 0);                                      \
  } while (0)
  if (f32) {
    if (vec) AR(float, true); else AR(float, false);
  } else {
    if (vec) AR(short, true); else AR(short, false);
  }
#undef AR
}

}  // namespace dnet
