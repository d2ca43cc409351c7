// Latent attention: the shared key/value row and the queries that meet it
// (gfx950).
//
// One cache row per token serves every head as key and as value:
//   [ rmsnorm(c) * w  (R entries) | rotated key part (rd entries) ]
// latent_append builds it from the down-projection's output and writes it at
// position pos[b]+t of cache row slots[b]; latent_q_pack lays the queries out
// the same way, per head [query carried into the latent space (R) | rotated
// query part (rd)], so that one dot product over R + rd entries is the score.
// The rotation pairs entries (2i, 2i+1) and turns them by position * f_i;
// statistics, angles and the rotation itself are fp32 with the accurate
// sincosf, whatever the activation dtype ("short" stands for bf16 bits).
#include "common.h"

namespace dnet {
namespace {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<short>(const short* p) { return bits2f(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<short>(short* p, float v) { *p = f2bits(v); }

constexpr int kMaxPairs = 128;      // rotated entries <= 256

// grid (B*T); one workgroup per token
template <typename T>
__global__ __launch_bounds__(256) void latent_append_kernel(
    const T* __restrict__ src, const int64_t ld, const int col0,
    const float* __restrict__ wn, const float eps, const int R, const int np,
    const float* __restrict__ freq, T* __restrict__ kcache,
    const int* __restrict__ pos, const int* __restrict__ lens,
    const int* __restrict__ slots, const int Tn, const int Bc,
    const int Smax) {
  __shared__ float red[8];
  const int64_t row = blockIdx.x;
  const int b = (int)(row / Tn), t = (int)(row % Tn);
  const int n = lens ? min(lens[b], Tn) : Tn;
  if (t >= n) return;                              // padding: not appended
  const int slot = slots ? slots[b] : b;
  const int p = pos[b] + t;
  if (slot < 0 || slot >= Bc || p < 0 || p >= Smax) return;
  const T* sr = src + row * ld + col0;
  const int D = R + 2 * np;
  T* dst = kcache + ((int64_t)slot * Smax + p) * D;
  float ss = 0.f;
  for (int i = threadIdx.x; i < R; i += blockDim.x) {
    const float v = ldf<T>(sr + i);
    ss = fmaf(v, v, ss);
  }
  ss = block_reduce_sum(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)R + eps);
  for (int i = threadIdx.x; i < R; i += blockDim.x)
    stf<T>(dst + i, ldf<T>(sr + i) * r * wn[i]);
  for (int i = threadIdx.x; i < np; i += blockDim.x) {
    float sn, cs;
    sincosf((float)p * freq[i], &sn, &cs);
    const float u = ldf<T>(sr + R + 2 * i), v = ldf<T>(sr + R + 2 * i + 1);
    stf<T>(dst + R + 2 * i, u * cs - v * sn);
    stf<T>(dst + R + 2 * i + 1, v * cs + u * sn);
  }
}

// grid (B*T); q [M, H*(d+rd)], qabs [H, M, R] -> out [M, H*(R+rd)]
template <typename T>
__global__ __launch_bounds__(256) void latent_q_pack_kernel(
    const T* __restrict__ q, const T* __restrict__ qabs,
    const float* __restrict__ freq, const int* __restrict__ pos,
    T* __restrict__ out, const int Tn, const int64_t M, const int H,
    const int d, const int np, const int R) {
  __shared__ float cs_s[kMaxPairs], sn_s[kMaxPairs];
  const int64_t row = blockIdx.x;
  const int b = (int)(row / Tn), t = (int)(row % Tn);
  const float p = (float)(pos[b] + t);
  for (int i = threadIdx.x; i < np; i += blockDim.x)
    sincosf(p * freq[i], &sn_s[i], &cs_s[i]);
  __syncthreads();
  const int rd = 2 * np, D = R + rd;
  const T* qr = q + row * (int64_t)H * (d + rd);
  T* orow = out + row * (int64_t)H * D;
  for (int idx = threadIdx.x; idx < H * R; idx += blockDim.x) {
    const int h = idx / R, i = idx % R;
    orow[(int64_t)h * D + i] = qabs[((int64_t)h * M + row) * R + i];
  }
  for (int idx = threadIdx.x; idx < H * np; idx += blockDim.x) {
    const int h = idx / np, i = idx % np;
    const T* qp = qr + (int64_t)h * (d + rd) + d + 2 * i;
    const float u = ldf<T>(qp), v = ldf<T>(qp + 1);
    stf<T>(orow + (int64_t)h * D + R + 2 * i, u * cs_s[i] - v * sn_s[i]);
    stf<T>(orow + (int64_t)h * D + R + 2 * i + 1, v * cs_s[i] + u * sn_s[i]);
  }
}

const int* idx_ptr(const c10::optional<torch::Tensor>& t, int64_t n) {
  if (!t.has_value()) return nullptr;
  DNET_CHECK(t->scalar_type() == torch::kInt32 && t->is_contiguous() &&
                 t->numel() >= n, "int32 index tensor [B]");
  return t->data_ptr<int>();
}

}  // namespace

void latent_append(torch::Tensor src, int64_t col0, torch::Tensor wn,
                   double eps, int64_t R, torch::Tensor rot_freq,
                   torch::Tensor kcache, torch::Tensor pos,
                   c10::optional<torch::Tensor> lens,
                   c10::optional<torch::Tensor> slots, int64_t T) {
  const int64_t M = src.size(0);
  DNET_CHECK(T > 0 && M % T == 0, "rows = B*T");
  const int64_t B = M / T;
  const int64_t np = rot_freq.numel();
  DNET_CHECK(src.dim() == 2 && src.is_contiguous() && col0 >= 0 && R > 0 &&
                 col0 + R + 2 * np <= src.size(1), "src columns");
  DNET_CHECK(wn.scalar_type() == torch::kFloat32 && wn.is_contiguous() &&
                 wn.numel() == R, "wn fp32 [R]");
  DNET_CHECK(rot_freq.scalar_type() == torch::kFloat32 &&
                 rot_freq.is_contiguous(), "rot_freq fp32");
  DNET_CHECK(kcache.dim() == 4 && kcache.is_contiguous() &&
                 kcache.size(1) == 1 && kcache.size(3) == R + 2 * np &&
                 kcache.scalar_type() == src.scalar_type(),
             "cache [Bc, 1, Smax, R+rd] in the activation dtype");
  DNET_CHECK(pos.scalar_type() == torch::kInt32 && pos.is_contiguous() &&
                 pos.numel() >= B, "pos int32 [B]");
  if (!slots.has_value())
    DNET_CHECK(B <= kcache.size(0), "more rows than cache slots");
  if (M == 0) return;
  auto st = current_stream();
#define LA(TT)                                                               \
  hipLaunchKernelGGL((latent_append_kernel<TT>), dim3((unsigned)M),          \
                     dim3(256), 0, st, (const TT*)src.data_ptr(),            \
                     src.size(1), (int)col0, wn.data_ptr<float>(),           \
                     (float)eps, (int)R, (int)np,                            \
                     rot_freq.data_ptr<float>(), (TT*)kcache.data_ptr(),     \
                     pos.data_ptr<int>(), idx_ptr(lens, B),                  \
                     idx_ptr(slots, B), (int)T, (int)kcache.size(0),         \
                     (int)kcache.size(2))
  if (src.scalar_type() == torch::kBFloat16) LA(short);
  else if (src.scalar_type() == torch::kFloat32) LA(float);
  else DNET_CHECK(false, "latent_append: dtype");
#undef LA
}

void latent_q_pack(torch::Tensor q, torch::Tensor qabs, torch::Tensor rot_freq,
                   torch::Tensor pos, torch::Tensor out, int64_t T, int64_t H,
                   int64_t d) {
  const int64_t M = q.size(0);
  DNET_CHECK(T > 0 && M % T == 0, "rows = B*T");
  const int64_t np = rot_freq.numel();
  DNET_CHECK(np <= kMaxPairs, "rotated size <= 256");
  DNET_CHECK(q.dim() == 2 && q.is_contiguous() &&
                 q.size(1) == H * (d + 2 * np), "q [B*T, H*(d+rd)]");
  DNET_CHECK(qabs.dim() == 3 && qabs.is_contiguous() && qabs.size(0) == H &&
                 qabs.size(1) == M && qabs.scalar_type() == q.scalar_type(),
             "qabs [H, B*T, R]");
  const int64_t R = qabs.size(2);
  DNET_CHECK(out.is_contiguous() && out.size(0) == M &&
                 out.size(1) == H * (R + 2 * np) &&
                 out.scalar_type() == q.scalar_type(), "out [B*T, H*(R+rd)]");
  DNET_CHECK(rot_freq.scalar_type() == torch::kFloat32 &&
                 rot_freq.is_contiguous(), "rot_freq fp32");
  DNET_CHECK(pos.scalar_type() == torch::kInt32 && pos.is_contiguous() &&
                 pos.numel() >= M / T, "pos int32 [B]");
  if (M == 0) return;
  auto st = current_stream();
#define LQ(TT)                                                               \
  hipLaunchKernelGGL((latent_q_pack_kernel<TT>), dim3((unsigned)M),          \
                     dim3(256), 0, st, (const TT*)q.data_ptr(),              \
                     (const TT*)qabs.data_ptr(),                             \
                     rot_freq.data_ptr<float>(), pos.data_ptr<int>(),        \
                     (TT*)out.data_ptr(), (int)T, M, (int)H, (int)d,         \
                     (int)np, (int)R)
  if (q.scalar_type() == torch::kBFloat16) LQ(short);
  else if (q.scalar_type() == torch::kFloat32) LQ(float);
  else DNET_CHECK(false, "latent_q_pack: dtype");
#undef LQ
}

}  // namespace dnet
