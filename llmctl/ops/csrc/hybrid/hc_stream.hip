// Several fp32 residual streams per token (hyper-connections) and the small passes of layers built on them:
//   hc_embed_norm     every stream starts as the embedding row; the first sublayer's input
//                     norm(sum_s c_in[s] x_s) * g (an RMS norm with a single weight g)
//   hc_update_norm_   x_t <- sum_s mix[s, t] x_s + mult c_out[t] (s1 y1 + s2 y2) for all streams at once from the old
//                     ones, and the next sublayer's input norm(sum_t c_in[t] x_t) * g in the same pass over the row
//   gated_add_f32_    out += y * sigmoid(g), one gate logit per row
//   tanh_act          elementwise tanh
//   softcap_          x <- cap tanh(x / cap) in place
// All arithmetic fp32; y and the sublayer inputs in the activation dtype or fp32.
#include "hybrid_common.h"

namespace llmctl_hybrid {

namespace {
constexpr int NT = 256;
constexpr int NW = NT / 64;
constexpr int KEEP = 8;    // a thread's first KEEP columns stay in registers (rows up to KEEP * NT wide are read once)
constexpr int MAXS = 8;    // streams

struct HcCoef {
  float mix[MAXS * MAXS];  // [from, to]
  float out[MAXS];         // mult * c_out
  float in[MAXS];
};

template <typename T>
__global__ __launch_bounds__(NT) void hc_embed_norm_kernel(const int64_t* __restrict__ ids, const T* __restrict__ table,
                                                           const float* __restrict__ c_in, const float* __restrict__ g,
                                                           float* __restrict__ X, T* __restrict__ h, int S, int W, float eps) {
  __shared__ float red[NW];
  const int64_t row = blockIdx.x;
  const T* e = table + ids[row] * (int64_t)W;
  float cs = 0.f;
  for (int s = 0; s < S; ++s) cs += c_in[s];
  float q = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) {
    const float v = ldf(e + c);
    for (int s = 0; s < S; ++s) X[(row * S + s) * W + c] = v;
    const float u = v * cs;
    q += u * u;
  }
  const float f = cs * g[0] / sqrtf(block_sum<NW>(q, red) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += NT) stf(h + row * W + c, ldf(e + c) * f);
}

// S: streams (compile time, so that a column's streams live in registers)
template <typename TY, typename TH, int S>
__global__ __launch_bounds__(NT) void hc_update_norm_kernel(float* __restrict__ X, const TY* __restrict__ y1, int64_t y1_st, float s1,
                                                            const TY* __restrict__ y2, int64_t y2_st, float s2,
                                                            const float* __restrict__ mix, const float* __restrict__ c_out, float mult,
                                                            const float* __restrict__ c_in, const float* __restrict__ g,
                                                            TH* __restrict__ h, int W, float eps) {
  __shared__ float red[NW];
  __shared__ HcCoef co;
  if (threadIdx.x < S * S) co.mix[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) {
    co.out[threadIdx.x] = mult * c_out[threadIdx.x];
    co.in[threadIdx.x] = c_in != nullptr ? c_in[threadIdx.x] : 0.f;
  }
  __syncthreads();
  const int64_t row = blockIdx.x;
  float* xr = X + row * S * (int64_t)W;
  float u[KEEP];
  float q = 0.f;
  auto column = [&](int c) -> float {
    float old[S];
#pragma unroll
    for (int s = 0; s < S; ++s) old[s] = xr[(int64_t)s * W + c];
    float y = ldf(y1 + row * y1_st + c) * s1;
    if (y2 != nullptr) y += ldf(y2 + row * y2_st + c) * s2;
    float uu = 0.f;
#pragma unroll
    for (int t = 0; t < S; ++t) {
      float v = co.out[t] * y;
#pragma unroll
      for (int s = 0; s < S; ++s) v += co.mix[s * S + t] * old[s];
      xr[(int64_t)t * W + c] = v;
      uu += co.in[t] * v;
    }
    return uu;
  };
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int c = threadIdx.x + i * NT;
    u[i] = c < W ? column(c) : 0.f;
    q += u[i] * u[i];
  }
  for (int c = threadIdx.x + KEEP * NT; c < W; c += NT) {
    const float v = column(c);
    q += v * v;
  }
  if (h == nullptr) return;
  const float f = g[0] / sqrtf(block_sum<NW>(q, red) / (float)W + eps);
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int c = threadIdx.x + i * NT;
    if (c < W) stf(h + row * W + c, u[i] * f);
  }
  for (int c = threadIdx.x + KEEP * NT; c < W; c += NT) {  // the thread's own stores
    float uu = 0.f;
#pragma unroll
    for (int t = 0; t < S; ++t) uu += co.in[t] * xr[(int64_t)t * W + c];
    stf(h + row * W + c, uu * f);
  }
}

template <typename TY>
__global__ __launch_bounds__(NT) void gated_add_kernel(float* __restrict__ out, const TY* __restrict__ y, int64_t y_st,
                                                       const TY* __restrict__ g, int64_t g_st, int W) {
  const int64_t row = blockIdx.x;
  const float gate = 1.0f / (1.0f + expf(-ldf(g + row * g_st)));
  for (int c = threadIdx.x; c < W; c += NT) out[row * W + c] += ldf(y + row * y_st + c) * gate;
}

template <typename T>
__global__ __launch_bounds__(NT) void tanh_kernel(const T* __restrict__ x, T* __restrict__ y, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x;
  if (i < n) stf(y + i, tanhf(ldf(x + i)));
}

__global__ __launch_bounds__(NT) void softcap_kernel(float* __restrict__ x, int64_t n, float cap, float inv) {
  const int64_t i = (int64_t)blockIdx.x * NT + threadIdx.x;
  if (i < n) x[i] = cap * tanhf(x[i] * inv);
}

bool f32c(const at::Tensor& t, int64_t n) { return t.is_cuda() && t.is_contiguous() && t.scalar_type() == at::kFloat && t.numel() == n; }
}  // namespace

std::tuple<at::Tensor, at::Tensor> hc_embed_norm(const at::Tensor& ids, const at::Tensor& table, int64_t streams, const at::Tensor& c_in,
                                                 const at::Tensor& g, double eps, bool out_bf16) {
  HYB_CHECK(table.is_cuda() && table.is_contiguous() && table.dim() == 2, "table: contiguous [vocab, W]");
  HYB_CHECK(ids.is_cuda() && ids.is_contiguous() && ids.scalar_type() == at::kLong && ids.dim() == 1, "ids: int64 [T]");
  HYB_CHECK(streams >= 1 && streams <= MAXS && f32c(c_in, streams) && f32c(g, 1), "1 .. 8 streams, c_in fp32 [streams], g fp32 [1]");
  HYB_CHECK((table.scalar_type() == at::kBFloat16) == out_bf16, "the sublayer input takes the table's dtype");
  const int64_t T = ids.numel(), W = table.size(1);
  c10::DeviceGuard guard(table.device());
  at::Tensor X = at::empty({T, streams, W}, table.options().dtype(at::kFloat));
  at::Tensor h = at::empty({T, W}, table.options());
  if (T == 0) return {X, h};
  dispatch_act(table, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    hc_embed_norm_kernel<Tt><<<dim3((unsigned)T), NT, 0, cur_stream()>>>(ids.data_ptr<int64_t>(), (const Tt*)table.data_ptr(), c_in.data_ptr<float>(),
                                                                       g.data_ptr<float>(), X.data_ptr<float>(), (Tt*)h.data_ptr(), (int)streams,
                                                                       (int)W, (float)eps);
  });
  return {X, h};
}

at::Tensor hc_update_norm_(at::Tensor X, const at::Tensor& y1, double s1, const c10::optional<at::Tensor>& y2, double s2, const at::Tensor& mix,
                           const at::Tensor& c_out, double mult, const c10::optional<at::Tensor>& c_in, const c10::optional<at::Tensor>& g,
                           double eps, bool out_bf16) {
  HYB_CHECK(X.is_cuda() && X.is_contiguous() && X.scalar_type() == at::kFloat && X.dim() == 3, "streams: contiguous fp32 [T, S, W]");
  const int64_t T = X.size(0), S = X.size(1), W = X.size(2);
  HYB_CHECK(S >= 1 && S <= MAXS && f32c(mix, S * S) && f32c(c_out, S), "1 .. 8 streams, mix fp32 [S, S], c_out fp32 [S]");
  check_rows(y1, "y1");
  HYB_CHECK(y1.size(0) == T && y1.size(1) == W, "y1: [T, W]");
  if (y2.has_value()) {
    check_rows(*y2, "y2");
    HYB_CHECK(y2->size(0) == T && y2->size(1) == W && y2->scalar_type() == y1.scalar_type(), "y2: [T, W] of y1's dtype");
  }
  HYB_CHECK(c_in.has_value() == g.has_value(), "the next input takes c_in and g together");
  if (c_in.has_value()) HYB_CHECK(f32c(*c_in, S) && f32c(*g, 1), "c_in fp32 [S], g fp32 [1]");
  c10::DeviceGuard guard(X.device());
  const bool want = c_in.has_value();
  at::Tensor h = want ? at::empty({T, W}, X.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat)) : at::empty({0}, X.options());
  if (T == 0) return h;
  hipStream_t st = cur_stream();
  auto go = [&](auto* ty, auto* th) {
    using TY = std::remove_pointer_t<decltype(ty)>;
    using TH = std::remove_pointer_t<decltype(th)>;
    auto launch = [&](auto kern) {
      kern<<<dim3((unsigned)T), NT, 0, st>>>(X.data_ptr<float>(), (const TY*)y1.data_ptr(), y1.stride(0), (float)s1,
                                             y2.has_value() ? (const TY*)y2->data_ptr() : nullptr, y2.has_value() ? y2->stride(0) : 0, (float)s2,
                                             mix.data_ptr<float>(), c_out.data_ptr<float>(), (float)mult, want ? c_in->data_ptr<float>() : nullptr,
                                             want ? g->data_ptr<float>() : nullptr, want ? (TH*)h.data_ptr() : nullptr, (int)W, (float)eps);
    };
    switch (S) {
      case 1: launch(hc_update_norm_kernel<TY, TH, 1>); break;
      case 2: launch(hc_update_norm_kernel<TY, TH, 2>); break;
      case 3: launch(hc_update_norm_kernel<TY, TH, 3>); break;
      case 4: launch(hc_update_norm_kernel<TY, TH, 4>); break;
      case 5: launch(hc_update_norm_kernel<TY, TH, 5>); break;
      case 6: launch(hc_update_norm_kernel<TY, TH, 6>); break;
      case 7: launch(hc_update_norm_kernel<TY, TH, 7>); break;
      default: launch(hc_update_norm_kernel<TY, TH, 8>); break;
    }
  };
  dispatch_act(y1, [&](auto* ty) {
    if (out_bf16) go(ty, (bf16_t*)nullptr);
    else go(ty, (float*)nullptr);
  });
  return h;
}

void gated_add_f32_(at::Tensor out, const at::Tensor& y, const at::Tensor& g) {
  HYB_CHECK(out.is_cuda() && out.is_contiguous() && out.scalar_type() == at::kFloat && out.dim() == 2, "out: contiguous fp32 [T, W]");
  check_rows(y, "y");
  HYB_CHECK(y.size(0) == out.size(0) && y.size(1) == out.size(1), "y: [T, W]");
  HYB_CHECK(g.is_cuda() && g.dim() == 2 && g.size(0) == out.size(0) && g.size(1) == 1 && g.scalar_type() == y.scalar_type(), "g: [T, 1] of y's dtype");
  if (out.size(0) == 0) return;
  c10::DeviceGuard guard(out.device());
  dispatch_act(y, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    gated_add_kernel<Tt><<<dim3((unsigned)out.size(0)), NT, 0, cur_stream()>>>(out.data_ptr<float>(), (const Tt*)y.data_ptr(), y.stride(0),
                                                                             (const Tt*)g.data_ptr(), g.stride(0), (int)out.size(1));
  });
}

at::Tensor tanh_act(const at::Tensor& x) {
  HYB_CHECK(x.is_cuda() && x.is_contiguous(), "x: contiguous GPU tensor");
  c10::DeviceGuard guard(x.device());
  at::Tensor y = at::empty_like(x);
  const int64_t n = x.numel();
  if (n == 0) return y;
  dispatch_act(x, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    tanh_kernel<Tt><<<dim3((unsigned)((n + NT - 1) / NT)), NT, 0, cur_stream()>>>((const Tt*)x.data_ptr(), (Tt*)y.data_ptr(), n);
  });
  return y;
}

void softcap_(at::Tensor x, double cap) {
  HYB_CHECK(x.is_cuda() && x.is_contiguous() && x.scalar_type() == at::kFloat && cap > 0.0, "x: contiguous fp32 GPU tensor; cap > 0");
  const int64_t n = x.numel();
  if (n == 0) return;
  c10::DeviceGuard guard(x.device());
  softcap_kernel<<<dim3((unsigned)((n + NT - 1) / NT)), NT, 0, cur_stream()>>>(x.data_ptr<float>(), n, (float)cap, (float)(1.0 / cap));
}

}  // namespace llmctl_hybrid
