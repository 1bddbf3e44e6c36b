// The fp32 residual stream of parallel layers and the small row-wise passes around the mixers:
// LayerNorm (two-pass mean / variance), residual update fused with the next LayerNorm, RMS norm of a
// column range, sigmoid gating, SwiGLU, per-head unit-RMS with weight and gate.
#include "hybrid_common.h"

namespace llmctl_hybrid {

constexpr int NT = 256;
constexpr int NW = NT / 64;

// x [T, W] fp32 (updated in place when a != nullptr: x += a + b), h = LayerNorm(x) * w + bias.
template <typename T>
__global__ __launch_bounds__(NT) void add_layernorm_kernel(float* __restrict__ x, const T* __restrict__ a, int64_t a_stride,
                                                           const float* __restrict__ b, const float* __restrict__ w,
                                                           const float* __restrict__ bias, T* __restrict__ h, int W,
                                                           float eps) {
  __shared__ float red[NW];
  const int64_t r = blockIdx.x;
  float* xr = x + r * W;
  float s = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) {
    float v = xr[c];
    if (a != nullptr) {
      v += ldf(a + r * a_stride + c);
      if (b != nullptr) v += b[r * W + c];
      xr[c] = v;
    }
    s += v;
  }
  if (h == nullptr) return;
  const float mean = block_sum<NW>(s, red) / (float)W;
  float q = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) {
    const float d = xr[c] - mean;
    q += d * d;
  }
  const float rstd = 1.0f / sqrtf(block_sum<NW>(q, red) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += NT) stf(h + r * W + c, (xr[c] - mean) * rstd * w[c] + bias[c]);
}

// x [T, W] fp32 (updated in place when a != nullptr: x += a + b), then up to two RMS norms of the same
// x (one statistic): h_k = x / sqrt(mean(x^2) + eps) * (plus + w_k); ``plus`` = 1 for weights stored
// around zero.  A parallel layer's residual update and the two norms its branches read, in one pass.
template <typename T>
__global__ __launch_bounds__(NT) void add_rmsnorm2_kernel(float* __restrict__ x, const T* __restrict__ a, int64_t a_stride,
                                                          const T* __restrict__ b, int64_t b_stride, const float* __restrict__ w1,
                                                          const float* __restrict__ w2, T* __restrict__ h1, T* __restrict__ h2, int W,
                                                          float eps, float plus) {
  __shared__ float red[NW];
  constexpr int KEEP = 16;  // a thread's first KEEP values stay in registers (rows up to KEEP * NT wide are read once)
  const int64_t r = blockIdx.x;
  float* xr = x + r * W;
  float keep[KEEP];
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int c = threadIdx.x + i * NT;
    float v = 0.f;
    if (c < W) {
      v = xr[c];
      if (a != nullptr) {
        float d = ldf(a + r * a_stride + c);
        if (b != nullptr) d += ldf(b + r * b_stride + c);
        v += d;
        xr[c] = v;
      }
    }
    keep[i] = v;
    q += v * v;
  }
  for (int c = threadIdx.x + KEEP * NT; c < W; c += NT) {
    float v = xr[c];
    if (a != nullptr) {
      float d = ldf(a + r * a_stride + c);
      if (b != nullptr) d += ldf(b + r * b_stride + c);
      v += d;
      xr[c] = v;
    }
    q += v * v;
  }
  if (h1 == nullptr) return;
  const float rstd = 1.0f / sqrtf(block_sum<NW>(q, red) / (float)W + eps);
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int c = threadIdx.x + i * NT;
    if (c < W) {
      const float v = keep[i] * rstd;
      stf(h1 + r * W + c, v * (plus + w1[c]));
      if (h2 != nullptr) stf(h2 + r * W + c, v * (plus + w2[c]));
    }
  }
  for (int c = threadIdx.x + KEEP * NT; c < W; c += NT) {
    const float v = xr[c] * rstd;
    stf(h1 + r * W + c, v * (plus + w1[c]));
    if (h2 != nullptr) stf(h2 + r * W + c, v * (plus + w2[c]));
  }
}

// gu [rows, 2F] = [gate | up] -> g' = min(gate, limit), u' = clamp(up, -limit, limit),
// y = g' * sigmoid(alpha * g') * (u' + 1)
template <typename T>
__global__ void clamped_glu_kernel(const T* __restrict__ gu, T* __restrict__ y, int64_t rows, int F, float limit, float alpha) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * F) return;
  const int64_t r = i / F;
  const int c = (int)(i - r * F);
  const float g = fminf(ldf(gu + r * 2 * F + c), limit);
  const float u = fminf(fmaxf(ldf(gu + r * 2 * F + F + c), -limit), limit);
  stf(y + i, g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
}

// the same with 16-byte accesses (F a multiple of 8, aligned rows): one thread per 8 bf16 / 4 fp32 outputs
template <typename T>
__global__ void clamped_glu_vec_kernel(const T* __restrict__ gu, T* __restrict__ y, int64_t rows, int F, float limit, float alpha) {
  constexpr int N = Vec16<T>::N;
  const int per = F / N;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * per) return;
  const int64_t r = i / per;
  const int c = (int)(i - r * per) * N;
  float g[N], u[N], o[N];
  Vec16<T>::load(gu + r * 2 * F + c, g);
  Vec16<T>::load(gu + r * 2 * F + F + c, u);
#pragma unroll
  for (int k = 0; k < N; ++k) {
    const float gk = fminf(g[k], limit), uk = fminf(fmaxf(u[k], -limit), limit);
    o[k] = gk / (1.0f + expf(-alpha * gk)) * (uk + 1.0f);
  }
  Vec16<T>::store(y + r * F + c, o);
}

template <typename T>
__global__ __launch_bounds__(NT) void rmsnorm_cols_kernel(const T* __restrict__ x, int64_t x_stride, const float* __restrict__ w,
                                                          T* __restrict__ y, int n, float eps) {
  __shared__ float red[NW];
  const int64_t r = blockIdx.x;
  float q = 0.f;
  for (int c = threadIdx.x; c < n; c += NT) {
    const float v = ldf(x + r * x_stride + c);
    q += v * v;
  }
  const float rstd = 1.0f / sqrtf(block_sum<NW>(q, red) / (float)n + eps);
  for (int c = threadIdx.x; c < n; c += NT) stf(y + r * n + c, ldf(x + r * x_stride + c) * rstd * w[c]);
}

template <typename TO, typename TG>
__global__ void gate_mul_kernel(const TO* __restrict__ o, const TG* __restrict__ g, int64_t g_stride, TG* __restrict__ y,
                                int64_t rows, int N, int per) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * N) return;
  const int64_t r = i / N;
  const int c = (int)(i - r * N);
  const float gv = ldf(g + r * g_stride + c / per);  // one gate per ``per`` neighbouring columns
  stf(y + i, ldf(o + i) * (1.0f / (1.0f + expf(-gv))));
}

template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ y, int64_t rows, int F) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * F) return;
  const int64_t r = i / F;
  const int c = (int)(i - r * F);
  const float g = ldf(gu + r * 2 * F + c), u = ldf(gu + r * 2 * F + F + c);
  stf(y + i, g / (1.0f + expf(-g)) * u);
}

// o [T, H, dv] fp32 -> y [T, H*dv]: o / rms(o over dv) * w * sigmoid(g) (silu: * g sigmoid(g)); one wave per (token, head).
template <typename T>
__global__ __launch_bounds__(NT) void headnorm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                           const T* __restrict__ g, int64_t g_stride, T* __restrict__ y,
                                                           int64_t pairs, int H, int dv, float eps, int silu) {
  const int64_t p = (int64_t)blockIdx.x * NW + (threadIdx.x >> 6);
  if (p >= pairs) return;
  const int lane = threadIdx.x & 63;
  const int64_t t = p / H;
  const int hd = (int)(p - t * H);
  const float* op = o + p * dv;
  float q = 0.f;
  for (int c = lane; c < dv; c += 64) q += op[c] * op[c];
  const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)dv + eps);
  for (int c = lane; c < dv; c += 64) {
    const float gv = ldf(g + t * g_stride + hd * dv + c);
    const float gate = 1.0f / (1.0f + expf(-gv));
    stf(y + p * dv + c, op[c] * rstd * w[hd * dv + c] * (silu ? gv * gate : gate));
  }
}

// ------------------------------------------------------------------------------------------ host
static at::Tensor out_like(const at::Tensor& ref, at::IntArrayRef shape, bool bf16) {
  return at::empty(shape, ref.options().dtype(bf16 ? at::kBFloat16 : at::kFloat));
}

at::Tensor layernorm_f32(const at::Tensor& x, const at::Tensor& w, const at::Tensor& b, double eps, bool out_bf16) {
  HYB_CHECK(x.is_cuda() && x.dim() == 2 && x.is_contiguous() && x.scalar_type() == at::kFloat, "x: contiguous fp32 [T, W]");
  const int W = (int)x.size(1);
  HYB_CHECK(w.scalar_type() == at::kFloat && b.scalar_type() == at::kFloat && w.numel() == W && b.numel() == W && w.is_contiguous() && b.is_contiguous(), "norm weight / bias: fp32 [W]");
  c10::DeviceGuard guard(x.device());
  at::Tensor h = out_like(x, x.sizes(), out_bf16);
  if (x.size(0) == 0) return h;
  dispatch_act(h, [&](auto* tag) {
    using T = std::remove_pointer_t<decltype(tag)>;
    add_layernorm_kernel<T><<<dim3((unsigned)x.size(0)), NT, 0, cur_stream()>>>(
        x.data_ptr<float>(), (const T*)nullptr, 0, nullptr, w.data_ptr<float>(), b.data_ptr<float>(), (T*)h.data_ptr(), W, (float)eps);
  });
  return h;
}

static void check_add(const at::Tensor& x, const at::Tensor& a, const c10::optional<at::Tensor>& b) {
  HYB_CHECK(x.is_cuda() && x.dim() == 2 && x.is_contiguous() && x.scalar_type() == at::kFloat, "x: contiguous fp32 [T, W]");
  check_rows(a, "a");
  HYB_CHECK(a.size(0) == x.size(0) && a.size(1) == x.size(1), "a must have x's shape");
  if (b.has_value()) HYB_CHECK(b->is_cuda() && b->is_contiguous() && b->scalar_type() == at::kFloat && b->sizes() == x.sizes(), "b: contiguous fp32 of x's shape");
}

void residual_add_(at::Tensor x, const at::Tensor& a, const c10::optional<at::Tensor>& b) {
  check_add(x, a, b);
  if (x.size(0) == 0) return;
  c10::DeviceGuard guard(x.device());
  dispatch_act(a, [&](auto* tag) {
    using T = std::remove_pointer_t<decltype(tag)>;
    add_layernorm_kernel<T><<<dim3((unsigned)x.size(0)), NT, 0, cur_stream()>>>(
        x.data_ptr<float>(), (const T*)a.data_ptr(), a.stride(0), b.has_value() ? b->data_ptr<float>() : nullptr, nullptr, nullptr,
        (T*)nullptr, (int)x.size(1), 0.f);
  });
}

at::Tensor add_layernorm_f32_(at::Tensor x, const at::Tensor& a, const c10::optional<at::Tensor>& b, const at::Tensor& w,
                              const at::Tensor& bias, double eps, bool out_bf16) {
  check_add(x, a, b);
  const int W = (int)x.size(1);
  HYB_CHECK(w.scalar_type() == at::kFloat && bias.scalar_type() == at::kFloat && w.numel() == W && bias.numel() == W && w.is_contiguous() && bias.is_contiguous(), "norm weight / bias: fp32 [W]");
  HYB_CHECK((a.scalar_type() == at::kBFloat16) == out_bf16, "the output has a's dtype");
  c10::DeviceGuard guard(x.device());
  at::Tensor h = out_like(x, x.sizes(), out_bf16);
  if (x.size(0) == 0) return h;
  dispatch_act(a, [&](auto* tag) {
    using T = std::remove_pointer_t<decltype(tag)>;
    add_layernorm_kernel<T><<<dim3((unsigned)x.size(0)), NT, 0, cur_stream()>>>(
        x.data_ptr<float>(), (const T*)a.data_ptr(), a.stride(0), b.has_value() ? b->data_ptr<float>() : nullptr, w.data_ptr<float>(),
        bias.data_ptr<float>(), (T*)h.data_ptr(), W, (float)eps);
  });
  return h;
}

at::Tensor rmsnorm_cols(const at::Tensor& x, const at::Tensor& w, double eps, int64_t n, bool out_bf16) {
  check_rows(x, "x");
  HYB_CHECK(n >= 1 && n <= x.size(1) && w.numel() == n && w.scalar_type() == at::kFloat && w.is_contiguous(), "w: fp32 [n], n <= columns");
  HYB_CHECK((x.scalar_type() == at::kBFloat16) == out_bf16, "the output has x's dtype");
  c10::DeviceGuard guard(x.device());
  at::Tensor y = out_like(x, {x.size(0), n}, out_bf16);
  if (x.size(0) == 0) return y;
  dispatch_act(x, [&](auto* tag) {
    using T = std::remove_pointer_t<decltype(tag)>;
    rmsnorm_cols_kernel<T><<<dim3((unsigned)x.size(0)), NT, 0, cur_stream()>>>((const T*)x.data_ptr(), x.stride(0), w.data_ptr<float>(),
                                                                            (T*)y.data_ptr(), (int)n, (float)eps);
  });
  return y;
}

at::Tensor sigmoid_gate_mul(const at::Tensor& o, const at::Tensor& g) {
  check_rows(g, "g");
  HYB_CHECK(o.is_cuda() && o.is_contiguous() && o.dim() == 2 && o.size(0) == g.size(0) && g.size(1) >= 1 && o.size(1) % g.size(1) == 0,
            "o: contiguous [T, C]; g [T, C] or [T, H] with H dividing C");
  HYB_CHECK(o.scalar_type() == g.scalar_type(), "o and g share a dtype");
  c10::DeviceGuard guard(g.device());
  at::Tensor y = at::empty(o.sizes(), g.options());
  const int64_t n = o.numel();
  if (n == 0) return y;
  dispatch_act(g, [&](auto* tag) {
    using T = std::remove_pointer_t<decltype(tag)>;
    gate_mul_kernel<T, T><<<dim3((unsigned)((n + 255) / 256)), 256, 0, cur_stream()>>>((const T*)o.data_ptr(), (const T*)g.data_ptr(),
                                                                                     g.stride(0), (T*)y.data_ptr(), o.size(0), (int)o.size(1), (int)(o.size(1) / g.size(1)));
  });
  return y;
}

at::Tensor swiglu_any(const at::Tensor& gu) {
  HYB_CHECK(gu.is_cuda() && gu.is_contiguous() && gu.dim() == 2 && gu.size(1) % 2 == 0, "gu: contiguous [T, 2F]");
  c10::DeviceGuard guard(gu.device());
  const int F = (int)(gu.size(1) / 2);
  at::Tensor y = at::empty({gu.size(0), F}, gu.options());
  const int64_t n = y.numel();
  if (n == 0) return y;
  dispatch_act(gu, [&](auto* tag) {
    using T = std::remove_pointer_t<decltype(tag)>;
    swiglu_kernel<T><<<dim3((unsigned)((n + 255) / 256)), 256, 0, cur_stream()>>>((const T*)gu.data_ptr(), (T*)y.data_ptr(), gu.size(0), F);
  });
  return y;
}

std::tuple<at::Tensor, at::Tensor> add_rmsnorm2_f32_(at::Tensor x, const c10::optional<at::Tensor>& a, const c10::optional<at::Tensor>& b,
                                                     const at::Tensor& w1, const c10::optional<at::Tensor>& w2, double eps, bool one_plus,
                                                     bool out_bf16) {
  HYB_CHECK(x.is_cuda() && x.dim() == 2 && x.is_contiguous() && x.scalar_type() == at::kFloat, "x: contiguous fp32 [T, W]");
  const int W = (int)x.size(1);
  auto okw = [&](const at::Tensor& w) { return w.is_cuda() && w.scalar_type() == at::kFloat && w.numel() == W && w.is_contiguous(); };
  HYB_CHECK(okw(w1) && (!w2.has_value() || okw(*w2)), "norm weights: fp32 [W]");
  const at::ScalarType act = out_bf16 ? at::kBFloat16 : at::kFloat;
  if (a.has_value()) {
    check_rows(*a, "a");
    HYB_CHECK(a->sizes() == x.sizes() && a->scalar_type() == act, "a: x's shape, the output dtype");
    if (b.has_value()) {
      check_rows(*b, "b");
      HYB_CHECK(b->sizes() == x.sizes() && b->scalar_type() == act, "b: x's shape, the output dtype");
    }
  } else {
    HYB_CHECK(!b.has_value(), "b without a");
  }
  c10::DeviceGuard guard(x.device());
  at::Tensor h1 = out_like(x, x.sizes(), out_bf16);
  at::Tensor h2 = w2.has_value() ? out_like(x, x.sizes(), out_bf16) : at::Tensor();
  if (x.size(0) == 0) return {h1, w2.has_value() ? h2 : h1};
  dispatch_act(h1, [&](auto* tag) {
    using T = std::remove_pointer_t<decltype(tag)>;
    add_rmsnorm2_kernel<T><<<dim3((unsigned)x.size(0)), NT, 0, cur_stream()>>>(
        x.data_ptr<float>(), a.has_value() ? (const T*)a->data_ptr() : nullptr, a.has_value() ? a->stride(0) : 0,
        b.has_value() ? (const T*)b->data_ptr() : nullptr, b.has_value() ? b->stride(0) : 0, w1.data_ptr<float>(),
        w2.has_value() ? w2->data_ptr<float>() : nullptr, (T*)h1.data_ptr(), w2.has_value() ? (T*)h2.data_ptr() : nullptr, W, (float)eps,
        one_plus ? 1.0f : 0.0f);
  });
  return {h1, w2.has_value() ? h2 : h1};
}

void residual_add_act_(at::Tensor x, const at::Tensor& a, const c10::optional<at::Tensor>& b) {
  HYB_CHECK(x.is_cuda() && x.dim() == 2 && x.is_contiguous() && x.scalar_type() == at::kFloat, "x: contiguous fp32 [T, W]");
  check_rows(a, "a");
  HYB_CHECK(a.sizes() == x.sizes(), "a must have x's shape");
  if (b.has_value()) {
    check_rows(*b, "b");
    HYB_CHECK(b->sizes() == x.sizes() && b->scalar_type() == a.scalar_type(), "b: x's shape, a's dtype");
  }
  if (x.size(0) == 0) return;
  c10::DeviceGuard guard(x.device());
  dispatch_act(a, [&](auto* tag) {
    using T = std::remove_pointer_t<decltype(tag)>;
    add_rmsnorm2_kernel<T><<<dim3((unsigned)x.size(0)), NT, 0, cur_stream()>>>(
        x.data_ptr<float>(), (const T*)a.data_ptr(), a.stride(0), b.has_value() ? (const T*)b->data_ptr() : nullptr,
        b.has_value() ? b->stride(0) : 0, nullptr, nullptr, (T*)nullptr, (T*)nullptr, (int)x.size(1), 0.f, 0.f);
  });
}

at::Tensor clamped_glu(const at::Tensor& gu, double limit, double alpha) {
  HYB_CHECK(gu.is_cuda() && gu.is_contiguous() && gu.dim() == 2 && gu.size(1) % 2 == 0, "gu: contiguous [T, 2F]");
  c10::DeviceGuard guard(gu.device());
  const int F = (int)(gu.size(1) / 2);
  at::Tensor y = at::empty({gu.size(0), F}, gu.options());
  const int64_t n = y.numel();
  if (n == 0) return y;
  dispatch_act(gu, [&](auto* tag) {
    using T = std::remove_pointer_t<decltype(tag)>;
    if (F % 8 == 0 && aligned16<T>(gu)) {
      const int64_t nv = n / Vec16<T>::N;
      clamped_glu_vec_kernel<T><<<dim3((unsigned)((nv + 255) / 256)), 256, 0, cur_stream()>>>((const T*)gu.data_ptr(), (T*)y.data_ptr(), gu.size(0),
                                                                                            F, (float)limit, (float)alpha);
    } else {
      clamped_glu_kernel<T><<<dim3((unsigned)((n + 255) / 256)), 256, 0, cur_stream()>>>((const T*)gu.data_ptr(), (T*)y.data_ptr(), gu.size(0), F,
                                                                                       (float)limit, (float)alpha);
    }
  });
  return y;
}

at::Tensor headnorm_gate(const at::Tensor& o, const at::Tensor& w, const at::Tensor& g, double eps, bool out_bf16, bool silu) {
  HYB_CHECK(o.is_cuda() && o.is_contiguous() && o.dim() == 3 && o.scalar_type() == at::kFloat, "o: contiguous fp32 [T, H, dv]");
  check_rows(g, "g");
  const int64_t T = o.size(0);
  const int H = (int)o.size(1), dv = (int)o.size(2);
  HYB_CHECK(g.size(0) == T && g.size(1) == (int64_t)H * dv && w.numel() == (int64_t)H * dv && w.scalar_type() == at::kFloat && w.is_contiguous(), "g [T, H*dv], w fp32 [H*dv]");
  HYB_CHECK((g.scalar_type() == at::kBFloat16) == out_bf16, "the output has g's dtype");
  c10::DeviceGuard guard(o.device());
  at::Tensor y = out_like(o, {T, (int64_t)H * dv}, out_bf16);
  if (T == 0) return y;
  const int64_t pairs = T * H;
  dispatch_act(g, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    headnorm_gate_kernel<Tt><<<dim3((unsigned)((pairs + NW - 1) / NW)), NT, 0, cur_stream()>>>(
        o.data_ptr<float>(), w.data_ptr<float>(), (const Tt*)g.data_ptr(), g.stride(0), (Tt*)y.data_ptr(), pairs, H, dv, (float)eps, silu ? 1 : 0);
  });
  return y;
}

}  // namespace llmctl_hybrid
