// The fp32 residual stream of sequential layers with norms on both sides of a sublayer and a gated
// residual, and the small passes around them:
//   gated_norm_add_norm_f32_  g = y sigmoid(r); x += g / rms(g) * w_post; h = x / rms(x) * w_next, one pass per row
//   embed_rmsnorm_f32         x = table[id] + pos_table[position] as the fp32 stream, and its first RMS norm
//   act_any                   relu(x)^2 or the exact (erf) GELU on a column range of a wider row
// All arithmetic fp32; y, r, h in the activation dtype or fp32.
#include "hybrid_common.h"

namespace llmctl_hybrid {

namespace {
constexpr int NT = 256;
constexpr int NW = NT / 64;
constexpr int KEEP = 8;  // a thread's first KEEP values stay in registers (rows up to KEEP * NT wide are read once)

__device__ __forceinline__ float sigmoidf_(float v) { return 1.0f / (1.0f + expf(-v)); }

template <typename TY, typename TR, typename TH>
__global__ __launch_bounds__(NT) void gated_norm_add_norm_kernel(float* __restrict__ x, const TY* __restrict__ y, int64_t y_st,
                                                                 const TR* __restrict__ r, int64_t r_st, const float* __restrict__ wp,
                                                                 const float* __restrict__ wn, TH* __restrict__ h, int W, float eps) {
  __shared__ float red[NW];
  const int64_t row = blockIdx.x;
  float* xr = x + row * W;
  const TY* yr = y + row * y_st;
  const TR* rr = r + row * r_st;
  float g[KEEP];
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int c = threadIdx.x + i * NT;
    g[i] = c < W ? ldf(yr + c) * sigmoidf_(ldf(rr + c)) : 0.f;
    q += g[i] * g[i];
  }
  for (int c = threadIdx.x + KEEP * NT; c < W; c += NT) {
    const float v = ldf(yr + c) * sigmoidf_(ldf(rr + c));
    q += v * v;
  }
  const float rstd = 1.0f / sqrtf(block_sum<NW>(q, red) / (float)W + eps);
  float q2 = 0.f;
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int c = threadIdx.x + i * NT;
    if (c < W) {
      g[i] = xr[c] + g[i] * rstd * wp[c];
      xr[c] = g[i];
      q2 += g[i] * g[i];
    }
  }
  for (int c = threadIdx.x + KEEP * NT; c < W; c += NT) {
    const float v = xr[c] + ldf(yr + c) * sigmoidf_(ldf(rr + c)) * rstd * wp[c];
    xr[c] = v;
    q2 += v * v;
  }
  if (h == nullptr) return;
  const float rstd2 = 1.0f / sqrtf(block_sum<NW>(q2, red) / (float)W + eps);
#pragma unroll
  for (int i = 0; i < KEEP; ++i) {
    const int c = threadIdx.x + i * NT;
    if (c < W) stf(h + row * W + c, g[i] * rstd2 * wn[c]);
  }
  for (int c = threadIdx.x + KEEP * NT; c < W; c += NT) stf(h + row * W + c, xr[c] * rstd2 * wn[c]);
}

template <typename T>
__global__ __launch_bounds__(NT) void embed_rmsnorm_kernel(const int64_t* __restrict__ ids, const int* __restrict__ pos,
                                                           const T* __restrict__ table, const T* __restrict__ ptable, const float* __restrict__ w,
                                                           float* __restrict__ x, T* __restrict__ h, int W, float eps) {
  __shared__ float red[NW];
  const int64_t row = blockIdx.x;
  const T* e = table + ids[row] * (int64_t)W;
  const T* p = ptable + (int64_t)pos[row] * W;
  float q = 0.f;
  for (int c = threadIdx.x; c < W; c += NT) {
    const float v = ldf(e + c) + ldf(p + c);
    x[row * W + c] = v;
    q += v * v;
  }
  const float rstd = 1.0f / sqrtf(block_sum<NW>(q, red) / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += NT) stf(h + row * W + c, x[row * W + c] * rstd * w[c]);  // the thread's own stores
}

template <int KIND>
__device__ __forceinline__ float act_one(float v) {
  if constexpr (KIND == 0) {
    const float r = fmaxf(v, 0.f);
    return r * r;
  } else {
    return 0.5f * v * (1.0f + erff(v * 0.70710678118654752f));
  }
}

template <typename T, int KIND>
__global__ void act_kernel(const T* __restrict__ x, int64_t x_st, T* __restrict__ y, int64_t rows, int F) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * F) return;
  const int64_t r = i / F;
  const int c = (int)(i - r * F);
  stf(y + i, act_one<KIND>(ldf(x + r * x_st + c)));
}

template <typename T, int KIND>
__global__ void act_vec_kernel(const T* __restrict__ x, int64_t x_st, T* __restrict__ y, int64_t rows, int F) {
  constexpr int N = Vec16<T>::N;
  const int per = F / N;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= rows * per) return;
  const int64_t r = i / per;
  const int c = (int)(i - r * per) * N;
  float v[N];
  Vec16<T>::load(x + r * x_st + c, v);
#pragma unroll
  for (int k = 0; k < N; ++k) v[k] = act_one<KIND>(v[k]);
  Vec16<T>::store(y + r * F + c, v);
}

// z [T, >= H*dk + G*dk + G*dv] = [q | k | v | ...]: unit RMS over all of q and over all of k, times the weights;
// q times the position's temperature; [v | k] per kv group to the token's cache row.  One block per token.
template <typename T>
__global__ __launch_bounds__(NT) void qk_fullnorm_prep_kernel(const T* __restrict__ z, int64_t z_st, const float* __restrict__ wq,
                                                              const float* __restrict__ wk, const int* __restrict__ pos, T* __restrict__ q,
                                                              T* __restrict__ cache, const int64_t* __restrict__ slots, int H, int G, int dk,
                                                              int dv, float eps, float coef, int every) {
  __shared__ float red[NW];
  const int64_t t = blockIdx.x;
  const T* zr = z + t * z_st;
  const int nq = H * dk, nk = G * dk, nv = G * dv;
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x; c < nq; c += NT) {
    const float v = ldf(zr + c);
    sq += v * v;
  }
  for (int c = threadIdx.x; c < nk; c += NT) {
    const float v = ldf(zr + nq + c);
    sk += v * v;
  }
  const float rq = 1.0f / sqrtf(block_sum<NW>(sq, red) / (float)nq + eps);
  const float rk = 1.0f / sqrtf(block_sum<NW>(sk, red) / (float)nk + eps);
  float temp = 1.0f;
  if (coef != 0.f) temp = 1.0f + coef * logf((float)((pos[t] + 1) / every) + 1.0f);
  for (int c = threadIdx.x; c < nq; c += NT) stf(q + t * nq + c, ldf(zr + c) * rq * wq[c] * temp);
  const int64_t slot = slots[t];
  if (slot < 0) return;
  T* row = cache + slot * (int64_t)(nk + nv);
  for (int c = threadIdx.x; c < nk; c += NT) {
    const int g = c / dk, d = c - g * dk;
    stf(row + g * (dv + dk) + dv + d, ldf(zr + nq + c) * rk * wk[c]);
  }
  for (int c = threadIdx.x; c < nv; c += NT) {
    const int g = c / dv, d = c - g * dv;
    row[g * (dv + dk) + d] = zr[nq + nk + c];
  }
}

bool f32w(const at::Tensor& w, int64_t n) { return w.is_cuda() && w.scalar_type() == at::kFloat && w.is_contiguous() && w.numel() == n; }
}  // namespace

at::Tensor gated_norm_add_norm_f32_(at::Tensor x, const at::Tensor& y, const at::Tensor& r, const at::Tensor& w_post,
                                    const c10::optional<at::Tensor>& w_next, double eps, bool out_bf16) {
  HYB_CHECK(x.is_cuda() && x.dim() == 2 && x.is_contiguous() && x.scalar_type() == at::kFloat, "x: contiguous fp32 [T, W]");
  check_rows(y, "y");
  check_rows(r, "r");
  const int64_t T = x.size(0), W = x.size(1);
  HYB_CHECK(y.sizes() == x.sizes() && r.sizes() == x.sizes(), "y and r must have x's shape");
  HYB_CHECK(f32w(w_post, W) && (!w_next.has_value() || f32w(*w_next, W)), "norm weights: fp32 [W]");
  c10::DeviceGuard guard(x.device());
  at::Tensor h = w_next.has_value() ? at::empty({T, W}, x.options().dtype(out_bf16 ? at::kBFloat16 : at::kFloat)) : at::empty({0}, x.options());
  if (T == 0) return h;
  const float* wn = w_next.has_value() ? w_next->data_ptr<float>() : nullptr;
  hipStream_t st = cur_stream();
  auto go = [&](auto* ty, auto* tr, auto* th) {
    using TY = std::remove_pointer_t<decltype(ty)>;
    using TR = std::remove_pointer_t<decltype(tr)>;
    using TH = std::remove_pointer_t<decltype(th)>;
    gated_norm_add_norm_kernel<TY, TR, TH><<<dim3((unsigned)T), NT, 0, st>>>(x.data_ptr<float>(), (const TY*)y.data_ptr(), y.stride(0),
                                                                           (const TR*)r.data_ptr(), r.stride(0), w_post.data_ptr<float>(), wn,
                                                                           wn != nullptr ? (TH*)h.data_ptr() : (TH*)nullptr, (int)W, (float)eps);
  };
  dispatch_act(y, [&](auto* ty) {
    dispatch_act(r, [&](auto* tr) {
      if (out_bf16) go(ty, tr, (bf16_t*)nullptr);
      else go(ty, tr, (float*)nullptr);
    });
  });
  return h;
}

std::tuple<at::Tensor, at::Tensor> embed_rmsnorm_f32(const at::Tensor& ids, const at::Tensor& pos, const at::Tensor& table,
                                                     const at::Tensor& pos_table, const at::Tensor& w, double eps, bool out_bf16) {
  HYB_CHECK(table.is_cuda() && table.dim() == 2 && table.is_contiguous() && pos_table.is_cuda() && pos_table.dim() == 2 && pos_table.is_contiguous() &&
                pos_table.size(1) == table.size(1) && pos_table.scalar_type() == table.scalar_type(),
            "embedding and position tables: contiguous [rows, W] of one dtype");
  const int64_t T = ids.numel(), W = table.size(1);
  HYB_CHECK(ids.is_cuda() && ids.is_contiguous() && ids.scalar_type() == at::kLong && pos.is_cuda() && pos.is_contiguous() && pos.scalar_type() == at::kInt && pos.numel() == T,
            "ids int64 [T], pos int32 [T]");
  HYB_CHECK(f32w(w, W), "norm weight: fp32 [W]");
  HYB_CHECK((table.scalar_type() == at::kBFloat16) == out_bf16, "the output has the tables' dtype");
  c10::DeviceGuard guard(table.device());
  at::Tensor x = at::empty({T, W}, table.options().dtype(at::kFloat));
  at::Tensor h = at::empty({T, W}, table.options());
  if (T == 0) return {x, h};
  dispatch_act(table, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    embed_rmsnorm_kernel<Tt><<<dim3((unsigned)T), NT, 0, cur_stream()>>>(ids.data_ptr<int64_t>(), pos.data_ptr<int>(), (const Tt*)table.data_ptr(),
                                                                        (const Tt*)pos_table.data_ptr(), w.data_ptr<float>(), x.data_ptr<float>(),
                                                                        (Tt*)h.data_ptr(), (int)W, (float)eps);
  });
  return {x, h};
}

at::Tensor act_any(const at::Tensor& x, int64_t kind) {
  check_rows(x, "x");
  HYB_CHECK(kind == 0 || kind == 1, "activation kind: 0 = squared relu, 1 = erf gelu");
  c10::DeviceGuard guard(x.device());
  const int64_t rows = x.size(0);
  const int F = (int)x.size(1);
  at::Tensor y = at::empty({rows, F}, x.options());
  const int64_t n = y.numel();
  if (n == 0) return y;
  hipStream_t st = cur_stream();
  dispatch_act(x, [&](auto* tag) {
    using T = std::remove_pointer_t<decltype(tag)>;
    const bool vec = F % Vec16<T>::N == 0 && aligned16<T>(x);
    const int64_t nv = vec ? n / Vec16<T>::N : n;
    const dim3 grid((unsigned)((nv + 255) / 256));
    if (vec) {
      if (kind == 0) act_vec_kernel<T, 0><<<grid, 256, 0, st>>>((const T*)x.data_ptr(), x.stride(0), (T*)y.data_ptr(), rows, F);
      else act_vec_kernel<T, 1><<<grid, 256, 0, st>>>((const T*)x.data_ptr(), x.stride(0), (T*)y.data_ptr(), rows, F);
    } else {
      if (kind == 0) act_kernel<T, 0><<<grid, 256, 0, st>>>((const T*)x.data_ptr(), x.stride(0), (T*)y.data_ptr(), rows, F);
      else act_kernel<T, 1><<<grid, 256, 0, st>>>((const T*)x.data_ptr(), x.stride(0), (T*)y.data_ptr(), rows, F);
    }
  });
  return y;
}

at::Tensor qk_fullnorm_prep(const at::Tensor& z, int64_t H, int64_t G, int64_t dk, int64_t dv, const at::Tensor& q_norm, const at::Tensor& k_norm,
                            double eps, const at::Tensor& pos, double temp_coef, int64_t temp_every, at::Tensor cache, const at::Tensor& slots) {
  check_rows(z, "z");
  const int64_t T = z.size(0);
  HYB_CHECK(H >= 1 && G >= 1 && H % G == 0 && dk >= 1 && dv >= 1 && z.size(1) >= (H + G) * dk + G * dv, "z: [T, >= H*dk + G*dk + G*dv]");
  HYB_CHECK(f32w(q_norm, H * dk) && f32w(k_norm, G * dk), "norm weights: fp32 [H*dk], [G*dk]");
  HYB_CHECK(cache.is_cuda() && cache.is_contiguous() && cache.dim() == 3 && cache.size(2) == G * (dv + dk) && cache.scalar_type() == z.scalar_type(),
            "cache: contiguous [blocks, block_size, G * (dv + dk)] of z's dtype");
  HYB_CHECK(pos.is_cuda() && pos.is_contiguous() && pos.scalar_type() == at::kInt && pos.numel() == T && slots.is_cuda() && slots.is_contiguous() &&
                slots.scalar_type() == at::kLong && slots.numel() == T,
            "pos int32 [T], slots int64 [T]");
  HYB_CHECK(temp_every >= 1, "temperature period >= 1");
  c10::DeviceGuard guard(z.device());
  at::Tensor q = at::empty({T, H, dk}, z.options());
  if (T == 0) return q;
  dispatch_act(z, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    qk_fullnorm_prep_kernel<Tt><<<dim3((unsigned)T), NT, 0, cur_stream()>>>((const Tt*)z.data_ptr(), z.stride(0), q_norm.data_ptr<float>(),
                                                                           k_norm.data_ptr<float>(), pos.data_ptr<int>(), (Tt*)q.data_ptr(),
                                                                           (Tt*)cache.data_ptr(), slots.data_ptr<int64_t>(), (int)H, (int)G, (int)dk,
                                                                           (int)dv, (float)eps, (float)temp_coef, (int)temp_every);
  });
  return q;
}

}  // namespace llmctl_hybrid
