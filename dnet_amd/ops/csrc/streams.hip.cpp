// Residual streams (hyper-connections) on an fp32 residual (gfx950).
//
// A row of xs [M, S*W] holds S streams of width W side by side. One kernel
// per sublayer boundary does, for its row,
//
//   write:  x_t <- sum_s mix[s, t] x_s + w_out[t] * y      (all t at once)
//   read:   u = sum_t next_in[t] x_t ;  out = u / sqrt(mean(u^2) + eps) * wn
//
// with either half optional (y == null: read only; next_in == null: write
// only). Every sum and the norm statistics are fp32; y comes in the
// activation dtype (or fp32), out leaves in the activation dtype.
// One workgroup per row; 16 B accesses when W is a multiple of 4.
#include "common.h"

namespace dnet {
namespace {

constexpr int kMaxStreams = 8;

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<short>(const short* p) { return bits2f(*p); }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<short>(short* p, float v) { *p = f2bits(v); }

struct StreamW {
  float mix[kMaxStreams * kMaxStreams];   // [from][to]
  float out[kMaxStreams];
  float in[kMaxStreams];
};

// VW elements per thread and step (4 or 1)
template <typename TY, typename TO, int VW>
__global__ __launch_bounds__(256) void hc_write_read_kernel(
    float* __restrict__ xs, const TY* __restrict__ y,
    const float* __restrict__ mix, const float* __restrict__ w_out,
    const float* __restrict__ next_in, const float* __restrict__ wn,
    TO* __restrict__ out, const int S, const int W, const float eps) {
  __shared__ float red[8];
  __shared__ StreamW sw;
  if (threadIdx.x < S * S && mix)
    sw.mix[(threadIdx.x / S) * kMaxStreams + threadIdx.x % S] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    sw.out[threadIdx.x] = w_out ? w_out[threadIdx.x] : 0.f;
    sw.in[threadIdx.x] = next_in ? next_in[threadIdx.x] : 0.f;
  }
  __syncthreads();
  const int64_t row = blockIdx.x;
  float* xr = xs + row * (int64_t)S * W;
  const TY* yr = y ? y + row * (int64_t)W : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x * VW; i < W; i += blockDim.x * VW) {
    float x[kMaxStreams][VW];
#pragma unroll
    for (int s = 0; s < kMaxStreams; ++s)
      if (s < S) {
        if constexpr (VW == 4) {
          const float4 v = *reinterpret_cast<const float4*>(xr + (int64_t)s * W + i);
          x[s][0] = v.x; x[s][1] = v.y; x[s][2] = v.z; x[s][3] = v.w;
        } else {
          x[s][0] = xr[(int64_t)s * W + i];
        }
      }
    float u[VW];
#pragma unroll
    for (int j = 0; j < VW; ++j) u[j] = 0.f;
    if (yr) {
      float yv[VW];
      if constexpr (VW == 4 && sizeof(TY) == 4) {
        const float4 v = *reinterpret_cast<const float4*>(yr + i);
        yv[0] = v.x; yv[1] = v.y; yv[2] = v.z; yv[3] = v.w;
      } else if constexpr (VW == 4) {
        const short4v v = *reinterpret_cast<const short4v*>(yr + i);
#pragma unroll
        for (int j = 0; j < 4; ++j) yv[j] = bits2f(v.x[j]);
      } else {
        yv[0] = ldf<TY>(yr + i);
      }
#pragma unroll
      for (int t = 0; t < kMaxStreams; ++t)
        if (t < S) {
          float nv[VW];
#pragma unroll
          for (int j = 0; j < VW; ++j) nv[j] = 0.f;
#pragma unroll
          for (int s = 0; s < kMaxStreams; ++s)
            if (s < S) {
              const float c = sw.mix[s * kMaxStreams + t];
#pragma unroll
              for (int j = 0; j < VW; ++j) nv[j] = fmaf(c, x[s][j], nv[j]);
            }
          const float co = sw.out[t], ci = sw.in[t];
#pragma unroll
          for (int j = 0; j < VW; ++j) {
            nv[j] = fmaf(co, yv[j], nv[j]);
            u[j] = fmaf(ci, nv[j], u[j]);
          }
          if constexpr (VW == 4)
            *reinterpret_cast<float4*>(xr + (int64_t)t * W + i) =
                make_float4(nv[0], nv[1], nv[2], nv[3]);
          else
            xr[(int64_t)t * W + i] = nv[0];
        }
    } else {
#pragma unroll
      for (int t = 0; t < kMaxStreams; ++t)
        if (t < S) {
          const float ci = sw.in[t];
#pragma unroll
          for (int j = 0; j < VW; ++j) u[j] = fmaf(ci, x[t][j], u[j]);
        }
    }
#pragma unroll
    for (int j = 0; j < VW; ++j) ss = fmaf(u[j], u[j], ss);
  }
  if (!out) return;                      // uniform: write only
  ss = block_reduce_sum(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)W + eps);
  TO* orow = out + row * (int64_t)W;
  // each thread re-reads exactly the elements it wrote above
  for (int i = threadIdx.x * VW; i < W; i += blockDim.x * VW) {
    float u[VW];
#pragma unroll
    for (int j = 0; j < VW; ++j) u[j] = 0.f;
#pragma unroll
    for (int t = 0; t < kMaxStreams; ++t)
      if (t < S) {
        const float ci = sw.in[t];
        if constexpr (VW == 4) {
          const float4 v =
              *reinterpret_cast<const float4*>(xr + (int64_t)t * W + i);
          u[0] = fmaf(ci, v.x, u[0]);
          u[1] = fmaf(ci, v.y, u[1]);
          u[2] = fmaf(ci, v.z, u[2]);
          u[3] = fmaf(ci, v.w, u[3]);
        } else {
          u[0] = fmaf(ci, xr[(int64_t)t * W + i], u[0]);
        }
      }
    if constexpr (VW == 4) {
      const float4 g = *reinterpret_cast<const float4*>(wn + i);
      const float o0 = u[0] * r * g.x, o1 = u[1] * r * g.y;
      const float o2 = u[2] * r * g.z, o3 = u[3] * r * g.w;
      if constexpr (sizeof(TO) == 4) {
        *reinterpret_cast<float4*>(orow + i) = make_float4(o0, o1, o2, o3);
      } else {
        short4v pk;
        pk.x[0] = f2bits(o0); pk.x[1] = f2bits(o1);
        pk.x[2] = f2bits(o2); pk.x[3] = f2bits(o3);
        *reinterpret_cast<short4v*>(orow + i) = pk;
      }
    } else {
      stf<TO>(orow + i, u[0] * r * wn[i]);
    }
  }
}

bool f32c(const torch::Tensor& t, int64_t n) {
  return t.scalar_type() == torch::kFloat32 && t.is_contiguous() &&
         t.numel() == n;
}

}  // namespace

void hc_write_read(torch::Tensor xs, c10::optional<torch::Tensor> y,
                   c10::optional<torch::Tensor> mix,
                   c10::optional<torch::Tensor> w_out,
                   c10::optional<torch::Tensor> next_in,
                   c10::optional<torch::Tensor> next_wn,
                   c10::optional<torch::Tensor> out, double eps) {
  DNET_CHECK(xs.dim() == 2 && xs.scalar_type() == torch::kFloat32 &&
                 xs.is_contiguous(), "xs fp32 [M, S*W]");
  const int64_t M = xs.size(0);
  int64_t S = 0;
  if (w_out.has_value()) S = w_out->numel();
  else if (next_in.has_value()) S = next_in->numel();
  DNET_CHECK(S >= 1 && S <= kMaxStreams && xs.size(1) % S == 0,
             "1..8 streams of equal width");
  const int64_t W = xs.size(1) / S;
  DNET_CHECK(y.has_value() == mix.has_value() &&
                 y.has_value() == w_out.has_value(), "write: y, mix, w_out");
  DNET_CHECK(next_in.has_value() == next_wn.has_value() &&
                 next_in.has_value() == out.has_value(),
             "read: next_in, next_wn, out");
  DNET_CHECK(y.has_value() || out.has_value(), "nothing to do");
  if (y.has_value()) {
    DNET_CHECK(y->dim() == 2 && y->is_contiguous() && y->size(0) == M &&
                   y->size(1) == W, "y [M, W]");
    DNET_CHECK(f32c(*mix, S * S) && f32c(*w_out, S), "mix [S,S], w_out [S]");
  }
  if (out.has_value()) {
    DNET_CHECK(f32c(*next_in, S) && f32c(*next_wn, W), "next_in [S], wn [W]");
    DNET_CHECK(out->is_contiguous() && out->size(0) == M &&
                   out->size(1) == W, "out [M, W]");
  }
  if (M == 0) return;
  auto st = current_stream();
  const bool yf = y.has_value() && y->scalar_type() == torch::kFloat32;
  const bool of = out.has_value() && out->scalar_type() == torch::kFloat32;
  DNET_CHECK(!y.has_value() || yf || y->scalar_type() == torch::kBFloat16,
             "y bf16 or fp32");
  DNET_CHECK(!out.has_value() || of ||
                 out->scalar_type() == torch::kBFloat16, "out bf16 or fp32");
#define HC(TY, TO, VW)                                                       \
  hipLaunchKernelGGL(                                                        \
      (hc_write_read_kernel<TY, TO, VW>), dim3((unsigned)M), dim3(256), 0,   \
      st, xs.data_ptr<float>(),                                              \
      y.has_value() ? (const TY*)y->data_ptr() : nullptr,                    \
      mix.has_value() ? mix->data_ptr<float>() : nullptr,                    \
      w_out.has_value() ? w_out->data_ptr<float>() : nullptr,                \
      next_in.has_value() ? next_in->data_ptr<float>() : nullptr,            \
      next_wn.has_value() ? next_wn->data_ptr<float>() : nullptr,            \
      out.has_value() ? (TO*)out->data_ptr() : nullptr, (int)S, (int)W,      \
      (float)eps)
#define HC_V(TY, TO)                \
  do {                              \
    if (W % 4 == 0) HC(TY, TO, 4);  \
    else HC(TY, TO, 1);             \
  } while (0)
  if (yf && of) HC_V(float, float);
  else if (yf) HC_V(float, short);
  else if (of) HC_V(short, float);
  else HC_V(short, short);
#undef HC_V
#undef HC
}

}  // namespace dnet
