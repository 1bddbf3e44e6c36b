// Helpers of the hybrid-mixer kernels (latent attention, mLSTM, group-limited router, fp32 residual
// stream).  Every kernel is generic over its sizes (read from the tensors) and templated on the
// activation element T = float or bf16; all arithmetic is fp32.  Wave size 64.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <ATen/ATen.h>
#include <ATen/hip/HIPContext.h>
#include <c10/core/DeviceGuard.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/library.h>

#include <cstdint>

#define HYB_CHECK(cond, ...) TORCH_CHECK(cond, "llmctl hybrid: ", __VA_ARGS__)

namespace llmctl_hybrid {

using bf16_t = unsigned short;

__device__ __forceinline__ float ldf(const float* p) { return *p; }
__device__ __forceinline__ float ldf(const bf16_t* p) { return __uint_as_float(((unsigned)*p) << 16); }
__device__ __forceinline__ void stf(float* p, float v) { *p = v; }
__device__ __forceinline__ void stf(bf16_t* p, float v) { *p = __bfloat16_as_ushort(__float2bfloat16(v)); }

// 16-byte accesses: 8 bf16 or 4 fp32 consecutive elements <-> floats (the pointer must be 16-byte aligned)
template <typename T>
struct Vec16;
template <>
struct Vec16<bf16_t> {
  static constexpr int N = 8;
  __device__ __forceinline__ static void load(const bf16_t* p, float* v) {
    const uint4 r = *reinterpret_cast<const uint4*>(p);
    const unsigned w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(w[i] << 16);
      v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
  __device__ __forceinline__ static void store(bf16_t* p, const float* v) {
    unsigned w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      w[i] = (unsigned)__bfloat16_as_ushort(__float2bfloat16(v[2 * i])) | ((unsigned)__bfloat16_as_ushort(__float2bfloat16(v[2 * i + 1])) << 16);
    *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
  }
};
template <>
struct Vec16<float> {
  static constexpr int N = 4;
  __device__ __forceinline__ static void load(const float* p, float* v) {
    const float4 r = *reinterpret_cast<const float4*>(p);
    v[0] = r.x, v[1] = r.y, v[2] = r.z, v[3] = r.w;
  }
  __device__ __forceinline__ static void store(float* p, const float* v) { *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]); }
};

template <typename T>
inline bool aligned16(const at::Tensor& t) {
  return reinterpret_cast<uintptr_t>(t.data_ptr()) % 16 == 0 && (t.dim() < 2 || (t.stride(0) * sizeof(T)) % 16 == 0);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Sum over a block of NW waves; every thread gets the result.  ``red`` holds NW floats; two barriers.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();  // red may still be read from a previous call
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NW; ++i) s += red[i];
  return s;
}

inline hipStream_t cur_stream() { return at::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

template <typename F>
inline void dispatch_act(const at::Tensor& t, F&& f) {
  if (t.scalar_type() == at::kFloat) {
    f((float*)nullptr);
  } else {
    HYB_CHECK(t.scalar_type() == at::kBFloat16, "activations must be fp32 or bf16");
    f((bf16_t*)nullptr);
  }
}

inline void check_rows(const at::Tensor& t, const char* name) {
  HYB_CHECK(t.is_cuda() && t.dim() == 2 && (t.size(1) == 1 || t.stride(1) == 1), name, ": 2-D GPU tensor with unit column stride");
}

// Optional parts of attention over a paged row cache (latent_attn*.hip).  A cache row of a token holds
// ``groups`` sub-rows of equal width; a sub-row's first ``rk`` entries are the value and the entries
// from ``koff`` on the key.  Query head h reads sub-row h / (H / groups).
struct RowAttnOpts {
  int64_t groups = 1;
  int64_t koff = 0;
  int64_t chunk = (int64_t)1 << 30;  // position i sees j only if i / chunk == j / chunk
  const float* hscale = nullptr;      // [H] a factor on every head's scores
  const float* ofreq = nullptr;       // [rk / 2] turn the output's neighbour pairs back by -position * ofreq
  int64_t max_ctx = 0;                // the longest context of the step, if the host knows it (sizes decode splits)
  const float* dist_a = nullptr;      // [H], with dist_b [H]: dist_a ln(1 + dist_b (i - j)) is taken off the scaled score
  const float* dist_b = nullptr;
  const float* sig_bias = nullptr;    // [H]: no softmax; a visible key weighs sigmoid(score + sig_bias), nothing is normalised
  double softcap = 0.0;               // c > 0: the scaled score becomes c tanh(score / c)
  int64_t keep_first = 0;             // the window does not hide the keys at positions below this
};

}  // namespace llmctl_hybrid
