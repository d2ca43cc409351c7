// Token-mixing steps around the matrix products of a layer that normalizes
// its sublayers' outputs (gfx950):
//
//   pair_hash_embed       embed[token] + table[hash(previous, token)] -> fp32
//                         residual rows; the slot's last token is its state
//   causal_conv_residual  y = x + conv(x): per-channel causal convolution of
//                         the fp32 residual, no bias, no activation; the last
//                         taps-1 inputs of every slot are its state (fp32)
//   decay_scan            S <- decay_h S + k v^T ; o = S^T q over SiLU(q),
//                         SiLU(k), SiLU(v): linear attention with a constant
//                         decay per head
//   qknorm_half_append    RMS norm of q and k over the whole projection,
//                         half-split rotation (channel i with i + n), keys
//                         and raw-key values appended to the cache
//   mul_sigmoid           a * sigmoid(gate columns)
//   silu_mul_halves       silu(gate half) * up half, any dtype and width
//
// Geometry is the cache's: token (b,t) = row b*T+t sits at position pos[b]+t
// of slot slots[b] (default b); tokens t >= lens[b] are padding. State is
// taken as zero at position 0 and written only by rows with real tokens.
// Sums, statistics, angles, decays and states are fp32 whatever the
// activation dtype ("short" stands for bf16 bits).
#include "common.h"

namespace dnet {

namespace {

template <typename T> __device__ __forceinline__ float ldx(const T* p);
template <> __device__ __forceinline__ float ldx<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldx<short>(const short* p) { return bits2f(*p); }
template <typename T> __device__ __forceinline__ void stx(T* p, float v);
template <> __device__ __forceinline__ void stx<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stx<short>(short* p, float v) { *p = f2bits(v); }

__device__ __forceinline__ float sigmoid_x(float x) {
  return 1.0f / (1.0f + expf(-x));
}

struct Rows {
  const int* pos;
  const int* lens;
  const int* slots;
  int T, Bc;
};

__device__ __forceinline__ bool row_of(const Rows& g, int b, int& p0, int& n,
                                       int& slot) {
  n = g.lens ? min(g.lens[b], g.T) : g.T;
  slot = g.slots ? g.slots[b] : b;
  p0 = g.pos[b];
  return n > 0 && slot >= 0 && slot < g.Bc && p0 >= 0;
}

const int* i32_or_null(const c10::optional<torch::Tensor>& t, int64_t n) {
  if (!t.has_value()) return nullptr;
  DNET_CHECK(t->scalar_type() == torch::kInt32 && t->is_contiguous() &&
                 t->numel() >= n, "int32 index tensor [B]");
  return t->data_ptr<int>();
}

Rows make_rows(const torch::Tensor& pos,
               const c10::optional<torch::Tensor>& lens,
               const c10::optional<torch::Tensor>& slots, int64_t B, int64_t T,
               int64_t Bc) {
  DNET_CHECK(pos.scalar_type() == torch::kInt32 && pos.is_contiguous() &&
                 pos.numel() >= B, "pos int32 [B]");
  if (!slots.has_value()) DNET_CHECK(B <= Bc, "more rows than cache slots");
  Rows g;
  g.pos = pos.data_ptr<int>();
  g.lens = i32_or_null(lens, B);
  g.slots = i32_or_null(slots, B);
  g.T = (int)T;
  g.Bc = (int)Bc;
  return g;
}

bool is_bf16(const torch::Tensor& t) { return t.scalar_type() == torch::kBFloat16; }
bool is_f32(const torch::Tensor& t) { return t.scalar_type() == torch::kFloat32; }

// ---- hashed pair embedding ---------------------------------------------------
// grid (B*T), one workgroup per token. Padding rows get the plain embedding
// (their output is never used).
template <typename T> __device__ __forceinline__ void ld4(const T* p, float (&v)[4]);
template <> __device__ __forceinline__ void ld4<float>(const float* p, float (&v)[4]) {
  const float4 q = *reinterpret_cast<const float4*>(p);
  v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
}
template <> __device__ __forceinline__ void ld4<short>(const short* p, float (&v)[4]) {
  const short4v q = *reinterpret_cast<const short4v*>(p);
#pragma unroll
  for (int e = 0; e < 4; ++e) v[e] = bits2f(q.x[e]);
}

template <typename T, bool V4>
__global__ __launch_bounds__(256) void pair_hash_embed_kernel(
    const int64_t* __restrict__ tokens, const T* __restrict__ embed,
    const T* __restrict__ table, const int* prev,
    float* __restrict__ out, const Rows g, const int W, const int vocab,
    const int buckets, const int64_t mul_prev, const int64_t mul_cur,
    int* prev_out) {
  const int64_t row = blockIdx.x;
  const int b = (int)(row / g.T), t = (int)(row % g.T);
  int p0, n, slot;
  const bool on = row_of(g, b, p0, n, slot) && t < n;
  int64_t tok = tokens[row];
  tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
  int64_t pr = -1;                     // table row, -1: none
  if (on) {
    if (p0 + t == 0) {
      pr = buckets;
    } else {
      const int64_t last = t > 0 ? tokens[row - 1] : (int64_t)prev[slot];
      pr = (last * mul_prev + tok * mul_cur) % buckets;
      if (pr < 0) pr += buckets;
    }
  }
  if (prev_out != nullptr) {
    // one token per row (decode): this workgroup alone reads the slot's last
    // token, so it also moves it on, once every thread has read it
    __syncthreads();
    if (on && threadIdx.x == 0) prev_out[slot] = (int)tokens[row];
  }
  const T* er = embed + tok * W;
  const T* tr = pr >= 0 ? table + pr * W : nullptr;
  float* orow = out + row * W;
  if constexpr (V4) {          // W % 4 == 0: 8 B / 16 B loads, 16 B stores
    for (int i = threadIdx.x * 4; i < W; i += blockDim.x * 4) {
      float v[4], u[4] = {0.f, 0.f, 0.f, 0.f};
      ld4<T>(er + i, v);
      if (tr) ld4<T>(tr + i, u);
      *reinterpret_cast<float4*>(orow + i) =
          make_float4(v[0] + u[0], v[1] + u[1], v[2] + u[2], v[3] + u[3]);
    }
  } else {
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      float v = ldx<T>(er + i);
      if (tr) v += ldx<T>(tr + i);
      orow[i] = v;
    }
  }
}

// grid (B), prompts only: after the rows are embedded, the slot's last token
// moves on. A separate launch: every row of the embed kernel reads the old
// value.
__global__ void pair_hash_state_kernel(const int64_t* __restrict__ tokens,
                                       int* __restrict__ prev, const Rows g,
                                       const int B) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= B) return;
  int p0, n, slot;
  if (!row_of(g, b, p0, n, slot)) return;
  prev[slot] = (int)tokens[(int64_t)b * g.T + n - 1];
}

// ---- residual convolution ----------------------------------------------------
// grid (channel tiles, B * token tiles): a thread walks kTile consecutive
// tokens of one channel with the sliding window of inputs in registers.
constexpr int kTile = 16;
constexpr int kMaxTaps = 16;

// TAIL (a row's tokens fit one tile, decode steps above all): the thread that
// walked the row also writes the slot's new tail, which is what its window
// registers hold at the end; otherwise conv_tail_kernel does, in a launch of
// its own, after every tile has read the old tail.
template <typename TO, bool TAIL>
__global__ __launch_bounds__(256) void conv_residual_kernel(
    const float* __restrict__ x, const float* __restrict__ w, float* state,
    TO* __restrict__ y, const Rows g, const int C, const int taps) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int ntile = (g.T + kTile - 1) / kTile;
  const int b = blockIdx.y / ntile;
  const int t0 = (blockIdx.y % ntile) * kTile;
  const int t1 = min(t0 + kTile, g.T);
  int p0, n, slot;
  const bool valid = row_of(g, b, p0, n, slot);
  float wr[kMaxTaps], win[kMaxTaps];
#pragma unroll
  for (int j = 0; j < kMaxTaps; ++j) {
    wr[j] = j < taps ? w[c * taps + j] : 0.f;
    win[j] = 0.f;
  }
  // inputs at t0-(taps-1) .. t0-1: earlier rows of this step, the slot's
  // tail, or zero before position 0
  if (valid && t0 < n) {
#pragma unroll
    for (int j = 0; j < kMaxTaps - 1; ++j) {
      if (j >= taps - 1) break;
      const int tt = t0 - (taps - 1) + j;
      if (tt >= 0)
        win[j] = x[((int64_t)b * g.T + tt) * C + c];
      else if (p0 + tt >= 0)
        win[j] = state[((int64_t)slot * (taps - 1) + (taps - 1 + tt)) * C + c];
    }
  }
  for (int t = t0; t < t1; ++t) {
    const int64_t row = (int64_t)b * g.T + t;
    float acc = 0.f;
    if (valid && t < n) {
      const float cur = x[row * C + c];
      acc = cur;
#pragma unroll
      for (int j = 0; j < kMaxTaps; ++j) {
        if (j >= taps) break;
        const float v = (j == taps - 1) ? cur : win[j];
        acc = fmaf(wr[j], v, acc);
      }
#pragma unroll
      for (int j = 0; j < kMaxTaps - 1; ++j) {
        if (j >= taps - 1) break;
        win[j] = (j == taps - 2) ? cur : win[j + 1];
      }
    }
    stx<TO>(y + row * C + c, acc);
  }
  if constexpr (TAIL) {
    if (valid) {
#pragma unroll
      for (int j = 0; j < kMaxTaps - 1; ++j) {
        if (j >= taps - 1) break;
        state[((int64_t)slot * (taps - 1) + j) * C + c] = win[j];
      }
    }
  }
}

// grid (channel tiles, B): shift the slot's tail by its n new inputs
__global__ __launch_bounds__(256) void conv_tail_kernel(
    const float* __restrict__ x, float* __restrict__ state, const Rows g,
    const int C, const int taps) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int b = blockIdx.y;
  int p0, n, slot;
  if (!row_of(g, b, p0, n, slot)) return;
  float* st = state + (int64_t)slot * (taps - 1) * C + c;
  for (int s = 0; s < taps - 1; ++s) {          // ascending: reads run ahead
    const int q = n - (taps - 1) + s;           // index among the new tokens
    float v = 0.f;
    if (q >= 0) v = x[((int64_t)b * g.T + q) * C + c];
    else if (p0 + q >= 0) v = st[(int64_t)(s + n) * C];
    st[(int64_t)s * C] = v;
  }
}

// ---- constant-decay linear attention -----------------------------------------
// grid (H * column tiles, B), block = JB value columns x NS key slices: thread
// (column j, slice s) keeps rows [R s, R s + R) of column j of the head's
// state [d x dv] in registers and walks the tokens in order. Per token of a
// staged chunk LDS holds silu(q), silu(k) [DP each] and silu(v) [JB]; the
// product over the rows of a column is an in-register sum plus lane shuffles
// over the NS neighbouring lanes.
template <int R> __host__ __device__ inline int padded_row(int r) {
  return (r / R) * (R + 4) + (r % R);
}

template <typename T, int R>
__global__ __launch_bounds__(256) void decay_scan_kernel(
    const T* __restrict__ src, const int64_t ld, const int q0, const int k0,
    const int v0, const float* __restrict__ decay, float* __restrict__ state,
    float* __restrict__ o, const Rows g, const int H, const int d,
    const int dv, const int JB, const int NS, const int TC) {
  const int ntile = (dv + JB - 1) / JB;
  const int h = blockIdx.x / ntile;
  const int j0 = (blockIdx.x % ntile) * JB;
  const int b = blockIdx.y;
  int p0, n, slot;
  if (!row_of(g, b, p0, n, slot)) return;
  const int DR = NS * R;                    // key rows incl. padding
  const int DP = NS * (R + 4);              // LDS pitch of one token
  const int jl = threadIdx.x / NS, sl = threadIdx.x % NS;
  const int j = j0 + jl;
  const bool col_ok = j < dv;

  extern __shared__ __attribute__((aligned(16))) float sm[];
  float* sQ = sm;                               // [TC][DP]
  float* sK = sQ + TC * DP;
  float* sV = sK + TC * DP;                     // [TC][JB]

  float S[R];
  float* sp = state + (((int64_t)slot * H + h) * d) * dv;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int row = sl * R + r;
    S[r] = (p0 > 0 && col_ok && row < d) ? sp[(int64_t)row * dv + j] : 0.f;
  }
  const float gh = decay[h];

  for (int t0 = 0; t0 < n; t0 += TC) {
    const int tc = min(TC, n - t0);
    __syncthreads();                            // previous chunk consumed
    for (int idx = threadIdx.x; idx < tc * DR; idx += blockDim.x) {
      const int tt = idx / DR, i = idx % DR;
      const T* sr = src + ((int64_t)b * g.T + t0 + tt) * ld;
      const int at = tt * DP + padded_row<R>(i);
      float qv = 0.f, kv = 0.f;
      if (i < d) {
        qv = ldx<T>(sr + q0 + h * d + i);
        kv = ldx<T>(sr + k0 + h * d + i);
        qv = qv * sigmoid_x(qv);
        kv = kv * sigmoid_x(kv);
      }
      sQ[at] = qv;
      sK[at] = kv;
    }
    for (int idx = threadIdx.x; idx < tc * JB; idx += blockDim.x) {
      const int tt = idx / JB, c = idx % JB;
      float vv = 0.f;
      if (j0 + c < dv) {
        vv = ldx<T>(src + ((int64_t)b * g.T + t0 + tt) * ld + v0 + h * dv +
                    j0 + c);
        vv = vv * sigmoid_x(vv);
      }
      sV[idx] = vv;
    }
    __syncthreads();
    for (int tt = 0; tt < tc; ++tt) {
      const int base = tt * DP + sl * (R + 4);
      const float4* kp = reinterpret_cast<const float4*>(sK + base);
      const float4* qp = reinterpret_cast<const float4*>(sQ + base);
      const float vj = sV[tt * JB + jl];
      float acc = 0.f;
#pragma unroll
      for (int r4 = 0; r4 < R / 4; ++r4) {
        const float4 kv = kp[r4], qv = qp[r4];
        S[4 * r4 + 0] = fmaf(kv.x, vj, gh * S[4 * r4 + 0]);
        S[4 * r4 + 1] = fmaf(kv.y, vj, gh * S[4 * r4 + 1]);
        S[4 * r4 + 2] = fmaf(kv.z, vj, gh * S[4 * r4 + 2]);
        S[4 * r4 + 3] = fmaf(kv.w, vj, gh * S[4 * r4 + 3]);
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

// ---- whole-projection q/k norm, half-split rotation, cache append -----------
// grid (B*T), one workgroup per token. qk row = [q (nq*d) | k (nkv*d)].
constexpr int kMaxHalfRot = 128;

template <typename T>
__global__ __launch_bounds__(256) void qknorm_half_append_kernel(
    const T* __restrict__ qk, const float* __restrict__ qw,
    const float* __restrict__ kw, T* __restrict__ qout, T* __restrict__ kc,
    T* __restrict__ vc, const Rows g, const float eps, const int nq,
    const int nkv, const int d, const int Smax,
    const float* __restrict__ freq, const int nrot) {
  __shared__ float red[8];
  __shared__ float rot_c[kMaxHalfRot], rot_s[kMaxHalfRot];
  const int64_t row = blockIdx.x;
  const int b = (int)(row / g.T), t = (int)(row % g.T);
  const int NQ = nq * d, NK = nkv * d;
  const T* src = qk + row * (int64_t)(NQ + NK);
  const int p = g.pos[b] + t;
  const int slot = g.slots ? g.slots[b] : b;
  const bool keep = (!g.lens || t < g.lens[b]) && p >= 0 && p < Smax &&
                    slot >= 0 && slot < g.Bc;
  for (int i = threadIdx.x; i < nrot; i += blockDim.x)
    sincosf((float)p * freq[i], &rot_s[i], &rot_c[i]);
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < NQ; i += blockDim.x) {
    const float v = ldx<T>(src + i);
    sq = fmaf(v, v, sq);
  }
  for (int i = threadIdx.x; i < NK; i += blockDim.x) {
    const float v = ldx<T>(src + NQ + i);
    sk = fmaf(v, v, sk);
  }
  sq = block_reduce_sum(sq, red);          // (also orders the sincos writes)
  sk = block_reduce_sum(sk, red);
  const float rq = 1.0f / sqrtf(sq / (float)NQ + eps);
  const float rk = 1.0f / sqrtf(sk / (float)NK + eps);
  T* qo = qout + row * (int64_t)NQ;
  // per head: nrot turning pairs (i, i + nrot), then d - 2 nrot plain channels
  const int per = d - nrot;                // work items of one head
  for (int idx = threadIdx.x; idx < (nq + nkv) * per; idx += blockDim.x) {
    const int hh = idx / per, i = idx % per;
    const bool isq = hh < nq;
    if (!isq && !keep) continue;
    const int hb = isq ? hh * d : (hh - nq) * d;     // head's first channel
    const T* hs = src + (isq ? 0 : NQ) + hb;
    const float* wv = (isq ? qw : kw) + hb;
    const float r = isq ? rq : rk;
    T* dst = isq ? qo + hb
                 : kc + (((int64_t)slot * nkv + (hh - nq)) * Smax + p) * d;
    if (i < nrot) {
      const float u = ldx<T>(hs + i) * r * wv[i];
      const float v = ldx<T>(hs + i + nrot) * r * wv[i + nrot];
      stx<T>(dst + i, u * rot_c[i] - v * rot_s[i]);
      stx<T>(dst + i + nrot, v * rot_c[i] + u * rot_s[i]);
    } else {
      const int e = i + nrot;
      stx<T>(dst + e, ldx<T>(hs + e) * r * wv[e]);
    }
  }
  // the values: the key projections as they came
  if (keep)
    for (int i = threadIdx.x; i < NK; i += blockDim.x) {
      const int hk = i / d, e = i % d;
      vc[(((int64_t)slot * nkv + hk) * Smax + p) * d + e] = src[NQ + i];
    }
}

// ---- small element-wise steps -------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void mul_sigmoid_kernel(
    const T* __restrict__ a, const T* __restrict__ gate, const int64_t ld,
    const int col0, T* __restrict__ y, const int N, const int64_t total) {
  for (int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
       idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t row = idx / N;
    const int c = (int)(idx % N);
    stx<T>(y + idx, ldx<T>(a + idx) * sigmoid_x(ldx<T>(gate + row * ld + col0 + c)));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void silu_mul_halves_kernel(
    const T* __restrict__ gu, T* __restrict__ y, const int I,
    const int64_t total) {
  for (int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x;
       idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t row = idx / I;
    const int c = (int)(idx % I);
    const float gv = ldx<T>(gu + row * 2 * I + c);
    const float uv = ldx<T>(gu + row * 2 * I + I + c);
    stx<T>(y + idx, gv * sigmoid_x(gv) * uv);
  }
}

}  // namespace

void pair_hash_embed(torch::Tensor tokens, torch::Tensor embed,
                     torch::Tensor table, torch::Tensor prev,
                     torch::Tensor out, torch::Tensor pos,
                     c10::optional<torch::Tensor> lens,
                     c10::optional<torch::Tensor> slots, int64_t buckets,
                     int64_t mul_prev, int64_t mul_cur) {
  DNET_CHECK(tokens.dim() == 2 && tokens.is_contiguous() &&
                 tokens.scalar_type() == torch::kInt64, "tokens int64 [B, T]");
  const int64_t B = tokens.size(0), T = tokens.size(1);
  const int W = embed.size(1);
  DNET_CHECK(embed.dim() == 2 && embed.is_contiguous() && table.dim() == 2 &&
                 table.is_contiguous() && table.size(1) == W &&
                 table.size(0) == buckets + 1 && buckets > 0 &&
                 table.scalar_type() == embed.scalar_type(),
             "embed [V, W], table [buckets+1, W]");
  DNET_CHECK(prev.scalar_type() == torch::kInt32 && prev.is_contiguous() &&
                 prev.dim() == 1, "prev int32 [Bc]");
  DNET_CHECK(is_f32(out) && out.is_contiguous() && out.numel() == B * T * W,
             "out fp32 [B, T, W]");
  if (B * T == 0) return;
  const Rows g = make_rows(pos, lens, slots, B, T, prev.size(0));
  auto st = current_stream();
#define PE(TT, VV)                                                             \
  hipLaunchKernelGGL((pair_hash_embed_kernel<TT, VV>),                         \
                     dim3((unsigned)(B * T)), dim3(256), 0, st,                \
                     tokens.data_ptr<int64_t>(), (const TT*)embed.data_ptr(),  \
                     (const TT*)table.data_ptr(), prev.data_ptr<int>(),        \
                     out.data_ptr<float>(), g, W, (int)embed.size(0),          \
                     (int)buckets, mul_prev, mul_cur,                          \
                     T == 1 ? prev.data_ptr<int>() : nullptr)
  const bool v4 = W % 4 == 0;
  if (is_bf16(embed)) { if (v4) PE(short, true); else PE(short, false); }
  else if (is_f32(embed)) { if (v4) PE(float, true); else PE(float, false); }
  else DNET_CHECK(false, "pair_hash_embed: dtype");
#undef PE
  if (T > 1)
    hipLaunchKernelGGL(pair_hash_state_kernel, dim3((unsigned)((B + 63) / 64)),
                     dim3(64), 0, st, tokens.data_ptr<int64_t>(),
                     prev.data_ptr<int>(), g, (int)B);
}

void causal_conv_residual(torch::Tensor x, torch::Tensor w, torch::Tensor state,
                          torch::Tensor y, torch::Tensor pos,
                          c10::optional<torch::Tensor> lens,
                          c10::optional<torch::Tensor> slots, int64_t T) {
  DNET_CHECK(x.dim() == 2 && x.is_contiguous() && is_f32(x), "x fp32 [B*T, C]");
  DNET_CHECK(w.dim() == 2 && is_f32(w) && w.is_contiguous() &&
                 w.size(0) == x.size(1), "w fp32 [C, taps]");
  const int C = w.size(0), taps = w.size(1);
  DNET_CHECK(taps >= 1 && taps <= kMaxTaps, "1 <= taps <= 16");
  const int64_t M = x.size(0);
  DNET_CHECK(T > 0 && M % T == 0, "rows = B*T");
  const int64_t B = M / T;
  DNET_CHECK(state.dim() == 3 && state.is_contiguous() && is_f32(state) &&
                 state.size(1) == taps - 1 && state.size(2) == C,
             "state fp32 [Bc, taps-1, C]");
  DNET_CHECK(y.is_contiguous() && y.size(0) == M && y.size(1) == C,
             "y [B*T, C]");
  if (M == 0) return;
  const Rows g = make_rows(pos, lens, slots, B, T, state.size(0));
  auto st = current_stream();
  const int ntile = (int)((T + kTile - 1) / kTile);
  const dim3 grid((unsigned)((C + 255) / 256), (unsigned)(B * ntile));
  const bool fused = ntile == 1;        // the walking thread writes the tail
#define CR(TT, FF)                                                            \
  hipLaunchKernelGGL((conv_residual_kernel<TT, FF>), grid, dim3(256), 0, st,  \
                     x.data_ptr<float>(), w.data_ptr<float>(),                \
                     state.data_ptr<float>(), (TT*)y.data_ptr(), g, C, taps)
  if (is_bf16(y)) { if (fused) CR(short, true); else CR(short, false); }
  else if (is_f32(y)) { if (fused) CR(float, true); else CR(float, false); }
  else DNET_CHECK(false, "causal_conv_residual: output dtype");
#undef CR
  if (taps > 1 && !fused)
    hipLaunchKernelGGL(conv_tail_kernel,
                       dim3((unsigned)((C + 255) / 256), (unsigned)B),
                       dim3(256), 0, st, x.data_ptr<float>(),
                       state.data_ptr<float>(), g, C, taps);
}

void decay_scan(torch::Tensor src, int64_t q0, int64_t k0, int64_t v0,
                torch::Tensor decay, torch::Tensor state, torch::Tensor o,
                torch::Tensor pos, c10::optional<torch::Tensor> lens,
                c10::optional<torch::Tensor> slots, int64_t T, int64_t H,
                int64_t d, int64_t dv) {
  const int64_t M = src.size(0);
  DNET_CHECK(T > 0 && M % T == 0, "rows = B*T");
  const int64_t B = M / T;
  DNET_CHECK(src.dim() == 2 && src.is_contiguous(), "src [B*T, ld]");
  const int64_t ld = src.size(1);
  DNET_CHECK(q0 >= 0 && k0 >= 0 && v0 >= 0 && q0 + H * d <= ld &&
                 k0 + H * d <= ld && v0 + H * dv <= ld, "src columns");
  DNET_CHECK(is_f32(decay) && decay.is_contiguous() && decay.numel() == H,
             "decay fp32 [H]");
  DNET_CHECK(is_f32(state) && state.is_contiguous() && state.dim() == 4 &&
                 state.size(1) == H && state.size(2) == d &&
                 state.size(3) == dv, "state fp32 [Bc, H, d, dv]");
  DNET_CHECK(is_f32(o) && o.is_contiguous() && o.size(0) == M &&
                 o.size(1) == H * dv, "o fp32 [B*T, H*dv]");
  DNET_CHECK(d >= 1 && d <= 1024, "1 <= dim <= 1024");
  if (M == 0) return;
  const Rows g = make_rows(pos, lens, slots, B, T, state.size(0));
  // rows per thread: few rows = more lanes per column = more waves when
  // batch x heads is small; slices of a column stay inside one wave
  int R = 32;
  if (d <= 64) R = 8;
  else if (d <= 256) R = 16;
  int NS = 1;
  while (NS * R < d) NS *= 2;               // power of two, <= 64
  DNET_CHECK(NS <= 64, "decay_scan: head size");
  const int JB = std::max(1, std::min<int>(256 / NS, (int)dv));
  const int threads = JB * NS;
  const int DP = NS * (R + 4);
  int TC = 16;
  while (TC > 1 && (size_t)TC * (2 * DP + JB) * sizeof(float) > 48 * 1024)
    TC >>= 1;
  const size_t lds = (size_t)TC * (2 * DP + JB) * sizeof(float);
  const int ntile = (int)((dv + JB - 1) / JB);
  const dim3 grid((unsigned)(H * ntile), (unsigned)B);
  auto st = current_stream();
#define DS(TT, RR)                                                            \
  hipLaunchKernelGGL((decay_scan_kernel<TT, RR>), grid, dim3(threads), lds,   \
                     st, (const TT*)src.data_ptr(), ld, (int)q0, (int)k0,     \
                     (int)v0, decay.data_ptr<float>(),                        \
                     state.data_ptr<float>(), o.data_ptr<float>(), g, (int)H, \
                     (int)d, (int)dv, JB, NS, TC)
#define DS_R(TT)                   \
  do {                             \
    if (R == 8) DS(TT, 8);         \
    else if (R == 16) DS(TT, 16);  \
    else DS(TT, 32);               \
  } while (0)
  if (is_bf16(src)) DS_R(short);
  else if (is_f32(src)) DS_R(float);
  else DNET_CHECK(false, "decay_scan: dtype");
#undef DS_R
#undef DS
}

void qknorm_half_append(torch::Tensor qk, torch::Tensor qw, torch::Tensor kw,
                        torch::Tensor qout, torch::Tensor kcache,
                        torch::Tensor vcache, torch::Tensor pos,
                        c10::optional<torch::Tensor> lens,
                        c10::optional<torch::Tensor> slots, double eps,
                        int64_t nq, int64_t nkv, int64_t d, int64_t T,
                        c10::optional<torch::Tensor> rot_freq) {
  const int64_t M = qk.size(0);
  DNET_CHECK(T > 0 && M % T == 0, "rows = B*T");
  const int64_t B = M / T;
  int nrot = 0;
  if (rot_freq.has_value()) {
    DNET_CHECK(is_f32(*rot_freq) && rot_freq->is_contiguous() &&
                   rot_freq->numel() * 2 <= d &&
                   rot_freq->numel() <= kMaxHalfRot, "rot_freq fp32 [<= d/2]");
    nrot = (int)rot_freq->numel();
  }
  DNET_CHECK(qk.dim() == 2 && qk.is_contiguous() &&
                 qk.size(1) == (nq + nkv) * d, "qk [M, nq*d + nkv*d]");
  DNET_CHECK(qout.is_contiguous() && qout.size(0) == M &&
                 qout.size(1) == nq * d, "qout shape");
  DNET_CHECK(kcache.dim() == 4 && vcache.dim() == 4 &&
                 kcache.is_contiguous() && vcache.is_contiguous(), "cache");
  const int Bc = kcache.size(0), Smax = kcache.size(2);
  DNET_CHECK(kcache.size(1) == nkv && kcache.size(3) == d &&
                 vcache.sizes() == kcache.sizes(), "cache dims");
  DNET_CHECK(qout.scalar_type() == qk.scalar_type() &&
                 kcache.scalar_type() == qk.scalar_type() &&
                 vcache.scalar_type() == qk.scalar_type(), "dtypes");
  DNET_CHECK(is_f32(qw) && is_f32(kw) && qw.is_contiguous() &&
                 kw.is_contiguous() && qw.numel() == nq * d &&
                 kw.numel() == nkv * d, "norm weights");
  if (M == 0) return;
  const Rows g = make_rows(pos, lens, slots, B, T, Bc);
  auto st = current_stream();
#define QH(TT)                                                                \
  hipLaunchKernelGGL((qknorm_half_append_kernel<TT>), dim3((unsigned)M),      \
                     dim3(256), 0, st, (const TT*)qk.data_ptr(),              \
                     qw.data_ptr<float>(), kw.data_ptr<float>(),              \
                     (TT*)qout.data_ptr(), (TT*)kcache.data_ptr(),            \
                     (TT*)vcache.data_ptr(), g, (float)eps, (int)nq,          \
                     (int)nkv, (int)d, Smax,                                  \
                     nrot ? rot_freq->data_ptr<float>() : nullptr, nrot)
  if (is_bf16(qk)) QH(short);
  else if (is_f32(qk)) QH(float);
  else DNET_CHECK(false, "qknorm_half_append: dtype");
#undef QH
}

void mul_sigmoid(torch::Tensor a, torch::Tensor gate_src, int64_t col0,
                 torch::Tensor y) {
  DNET_CHECK(a.dim() == 2 && a.is_contiguous() && y.is_contiguous() &&
                 y.sizes() == a.sizes() && y.scalar_type() == a.scalar_type(),
             "a, y [M, N]");
  const int64_t M = a.size(0), N = a.size(1);
  DNET_CHECK(gate_src.dim() == 2 && gate_src.is_contiguous() &&
                 gate_src.size(0) == M && col0 >= 0 &&
                 col0 + N <= gate_src.size(1) &&
                 gate_src.scalar_type() == a.scalar_type(), "gate columns");
  const int64_t total = M * N;
  if (total == 0) return;
  const unsigned blocks = (unsigned)std::min<int64_t>((total + 255) / 256, 8192);
  auto st = current_stream();
  if (is_bf16(a))
    hipLaunchKernelGGL((mul_sigmoid_kernel<short>), dim3(blocks), dim3(256), 0,
                       st, (const short*)a.data_ptr(),
                       (const short*)gate_src.data_ptr(), gate_src.size(1),
                       (int)col0, (short*)y.data_ptr(), (int)N, total);
  else if (is_f32(a))
    hipLaunchKernelGGL((mul_sigmoid_kernel<float>), dim3(blocks), dim3(256), 0,
                       st, (const float*)a.data_ptr(),
                       (const float*)gate_src.data_ptr(), gate_src.size(1),
                       (int)col0, (float*)y.data_ptr(), (int)N, total);
  else DNET_CHECK(false, "mul_sigmoid: dtype");
}

void silu_mul_halves(torch::Tensor gu, torch::Tensor y) {
  DNET_CHECK(gu.dim() == 2 && gu.is_contiguous() && y.is_contiguous() &&
                 y.dim() == 2 && y.size(0) == gu.size(0) &&
                 gu.size(1) == 2 * y.size(1) &&
                 y.scalar_type() == gu.scalar_type(), "gu [M, 2I], y [M, I]");
  const int64_t total = y.numel();
  if (total == 0) return;
  const unsigned blocks = (unsigned)std::min<int64_t>((total + 255) / 256, 8192);
  auto st = current_stream();
  if (is_bf16(gu))
    hipLaunchKernelGGL((silu_mul_halves_kernel<short>), dim3(blocks),
                       dim3(256), 0, st, (const short*)gu.data_ptr(),
                       (short*)y.data_ptr(), (int)y.size(1), total);
  else if (is_f32(gu))
    hipLaunchKernelGGL((silu_mul_halves_kernel<float>), dim3(blocks),
                       dim3(256), 0, st, (const float*)gu.data_ptr(),
                       (float*)y.data_ptr(), (int)y.size(1), total);
  else DNET_CHECK(false, "silu_mul_halves: dtype");
}

}  // namespace dnet
