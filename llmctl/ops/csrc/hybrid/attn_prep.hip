// Query / key / value preparation of grouped-query attention over a paged row cache.
//
// Input z [T, H*dk + G*dk + G*dv] = [q | k | v] of a step's packed tokens.  Per token:
//   q, k   per-head RMS norm over dk (weight shared by the heads), then rotary on the first rot_dims
//          entries of every head: pairs are neighbours (2i, 2i+1) or halves (i, i + rot_dims/2),
//          angle = position * freq[i] in fp32, cos and sin times ``amp``;
//   v      optionally turned the same way over all of dv by position * vfreq[m] (the attention
//          kernel turns the head's weighted sum back by the query's position);
//   k, v   written to the token's cache row of kv head g: [v (dv) | k (dk)]; q returned [T, H, dk].
// Options: no norm (null weights); the value of a token is the output of its key projection, ahead of norm and rotary (z holds
// no v columns); v <- (1 - lambda) v + lambda v_first, with v_first [T, G*dv] rows of another layer's values of the
// same tokens and lambda one number in device memory.
// One workgroup per token (up to 16 waves), one wave per head slot in turn; all arithmetic fp32.  The token's cos / sin
// (they depend on the position and the pair only) are computed once into LDS and shared by its heads.
#include "hybrid_common.h"

namespace llmctl_hybrid {

// element index of pair p's two members
__device__ __forceinline__ void pair_idx(int p, int dims, bool inter, int& i0, int& i1) {
  if (inter) {
    i0 = 2 * p;
    i1 = 2 * p + 1;
  } else {
    i0 = p;
    i1 = p + dims / 2;
  }
}

template <typename T>
__global__ __launch_bounds__(1024) void attn_qkv_prep_kernel(const T* __restrict__ z, int64_t z_stride, const float* __restrict__ qn,
                                                            const float* __restrict__ kn, const int* __restrict__ pos,
                                                            const float* __restrict__ freq, const float* __restrict__ vfreq,
                                                            T* __restrict__ q_out, T* __restrict__ cache,
                                                            const int64_t* __restrict__ slots, int H, int G, int dk, int dv,
                                                            int rot_dims, int inter, float amp, float eps, int v_from_k,
                                                            const T* __restrict__ v_first, int64_t vf_stride,
                                                            const float* __restrict__ v_lambda) {
  extern __shared__ float cs_tab[];  // [rot_dims / 2][2] cos, sin (times amp), then [dv / 2][2] for the values
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float lam = v_first != nullptr ? v_lambda[0] : 0.f;
  const float p = (float)pos[t];
  const int nrot = rot_dims / 2, nv = vfreq != nullptr ? dv / 2 : 0;
  for (int i = threadIdx.x; i < nrot + nv; i += blockDim.x) {
    float s, c;
    if (i < nrot) {
      sincosf(p * freq[i], &s, &c);
      s *= amp;
      c *= amp;
    } else {
      sincosf(p * vfreq[i - nrot], &s, &c);
    }
    cs_tab[2 * i] = c;
    cs_tab[2 * i + 1] = s;
  }
  __syncthreads();
  const int64_t slot = slots[t];
  const int rs = dv + dk;
  const T* zr = z + t * z_stride;
  for (int hs = wave; hs < H + 2 * G; hs += (int)(blockDim.x >> 6)) {
    if (hs < H + G) {  // a query or key head: norm, rotary
      const bool is_q = hs < H;
      const T* x = zr + (int64_t)hs * dk;  // k heads follow the q heads at the same pitch
      const float* nw = is_q ? qn : kn;
      T* out;
      if (is_q) out = q_out + (t * H + hs) * dk;
      else if (slot >= 0) out = cache + (slot * G + (hs - H)) * rs + dv;
      else continue;
      float rstd = 1.0f;
      if (nw != nullptr) {
        float ss = 0.f;
        for (int c = lane; c < dk; c += 64) {
          const float v = ldf(x + c);
          ss += v * v;
        }
        rstd = 1.0f / sqrtf(wave_sum(ss) / (float)dk + eps);
      }
      for (int pr = lane; pr < rot_dims / 2; pr += 64) {
        int i0, i1;
        pair_idx(pr, rot_dims, inter, i0, i1);
        const float c = cs_tab[2 * pr], s = cs_tab[2 * pr + 1];
        const float a = ldf(x + i0) * rstd * (nw != nullptr ? nw[i0] : 1.f), b = ldf(x + i1) * rstd * (nw != nullptr ? nw[i1] : 1.f);
        stf(out + i0, a * c - b * s);
        stf(out + i1, b * c + a * s);
      }
      for (int c = rot_dims + lane; c < dk; c += 64) stf(out + c, ldf(x + c) * rstd * (nw != nullptr ? nw[c] : 1.f));
    } else {  // a value head
      if (slot < 0) continue;
      const int g = hs - H - G;
      const T* x = v_from_k ? zr + (int64_t)(H + g) * dk : zr + (int64_t)(H + G) * dk + (int64_t)g * dv;
      T* out = cache + (slot * G + g) * rs;
      if (v_first != nullptr) {  // (not combined with a turn of the values)
        const T* f = v_first + t * vf_stride + (int64_t)g * dv;
        for (int c = lane; c < dv; c += 64) stf(out + c, (1.0f - lam) * ldf(x + c) + lam * ldf(f + c));
        continue;
      }
      if (vfreq != nullptr) {
        for (int pr = lane; pr < dv / 2; pr += 64) {
          int i0, i1;
          pair_idx(pr, dv, inter, i0, i1);
          const float c = cs_tab[2 * (nrot + pr)], s = cs_tab[2 * (nrot + pr) + 1];
          const float a = ldf(x + i0), b = ldf(x + i1);
          stf(out + i0, a * c - b * s);
          stf(out + i1, b * c + a * s);
        }
      } else {
        for (int c = lane; c < dv; c += 64) stf(out + c, ldf(x + c));
      }
    }
  }
}

// Two neighbours at once: one 4-byte (bf16) or 8-byte (fp32) access
template <typename T>
struct Pair;
template <>
struct Pair<bf16_t> {
  __device__ __forceinline__ static void ld(const bf16_t* p, float& a, float& b) {
    const unsigned w = *reinterpret_cast<const unsigned*>(p);
    a = __uint_as_float(w << 16);
    b = __uint_as_float(w & 0xffff0000u);
  }
  __device__ __forceinline__ static void st(bf16_t* p, float a, float b) {
    *reinterpret_cast<unsigned*>(p) =
        (unsigned)__bfloat16_as_ushort(__float2bfloat16(a)) | ((unsigned)__bfloat16_as_ushort(__float2bfloat16(b)) << 16);
  }
};
template <>
struct Pair<float> {
  __device__ __forceinline__ static void ld(const float* p, float& a, float& b) {
    const float2 w = *reinterpret_cast<const float2*>(p);
    a = w.x;
    b = w.y;
  }
  __device__ __forceinline__ static void st(float* p, float a, float b) { *reinterpret_cast<float2*>(p) = make_float2(a, b); }
};

// The form for many tokens, neighbour pairs and heads of at most 128: lane p owns pair (2p, 2p+1) of a head, a wave first
// requests the pairs of up to eight head slots (so that eight loads per lane are in flight), then norms, turns
// and stores them.  Same arithmetic as the kernel above.
template <typename T>
__global__ __launch_bounds__(256) void attn_qkv_prep_pairs_kernel(const T* __restrict__ z, int64_t z_stride, const float* __restrict__ qn,
                                                                  const float* __restrict__ kn, const int* __restrict__ pos,
                                                                  const float* __restrict__ freq, const float* __restrict__ vfreq,
                                                                  T* __restrict__ q_out, T* __restrict__ cache,
                                                                  const int64_t* __restrict__ slots, int H, int G, int dk, int dv,
                                                                  int rot_dims, float amp, float eps, int v_from_k,
                                                                  const T* __restrict__ v_first, int64_t vf_stride,
                                                                  const float* __restrict__ v_lambda) {
  extern __shared__ float cs_tab[];
  constexpr int MAXS = 8;
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float lam = v_first != nullptr ? v_lambda[0] : 0.f;
  const float p = (float)pos[t];
  const int nrot = rot_dims / 2, nv = vfreq != nullptr ? dv / 2 : 0;
  for (int i = threadIdx.x; i < nrot + nv; i += 256) {
    float s, c;
    if (i < nrot) {
      sincosf(p * freq[i], &s, &c);
      s *= amp;
      c *= amp;
    } else {
      sincosf(p * vfreq[i - nrot], &s, &c);
    }
    cs_tab[2 * i] = c;
    cs_tab[2 * i + 1] = s;
  }
  __syncthreads();
  const int64_t slot = slots[t];
  const int rs = dv + dk, nslots = H + 2 * G;
  const T* zr = z + t * z_stride;
  for (int base = 0; base < nslots; base += 4 * MAXS) {
    float xa[MAXS], xb[MAXS];
#pragma unroll
    for (int k = 0; k < MAXS; ++k) {
      const int hs = base + wave + 4 * k;
      xa[k] = 0.f;
      xb[k] = 0.f;
      if (hs < nslots) {
        const bool qk = hs < H + G;
        const T* x = qk ? zr + (int64_t)hs * dk
                        : (v_from_k ? zr + (int64_t)(hs - G) * dk : zr + (int64_t)(H + G) * dk + (int64_t)(hs - H - G) * dv);
        if (2 * lane < (qk ? dk : dv)) Pair<T>::ld(x + 2 * lane, xa[k], xb[k]);
      }
    }
#pragma unroll
    for (int k = 0; k < MAXS; ++k) {
      const int hs = base + wave + 4 * k;  // the same for every lane of the wave
      if (hs >= nslots) continue;
      float a = xa[k], b = xb[k];
      if (hs < H + G) {
        const bool is_q = hs < H;
        const float* nw = is_q ? qn : kn;
        const float rstd = nw != nullptr ? 1.0f / sqrtf(wave_sum(a * a + b * b) / (float)dk + eps) : 1.0f;
        if (2 * lane >= dk || (!is_q && slot < 0)) continue;
        if (nw != nullptr) {
          a *= rstd * nw[2 * lane];
          b *= rstd * nw[2 * lane + 1];
        }
        if (lane < nrot) {
          const float c = cs_tab[2 * lane], sn = cs_tab[2 * lane + 1];
          const float ra = a * c - b * sn, rb = b * c + a * sn;
          a = ra;
          b = rb;
        }
        T* out = is_q ? q_out + (t * H + hs) * dk : cache + (slot * G + (hs - H)) * rs + dv;
        Pair<T>::st(out + 2 * lane, a, b);
      } else {
        if (2 * lane >= dv || slot < 0) continue;
        if (v_first != nullptr) {
          float fa, fb;
          Pair<T>::ld(v_first + t * vf_stride + (int64_t)(hs - H - G) * dv + 2 * lane, fa, fb);
          a = (1.0f - lam) * a + lam * fa;
          b = (1.0f - lam) * b + lam * fb;
        }
        if (vfreq != nullptr) {
          const float c = cs_tab[2 * (nrot + lane)], sn = cs_tab[2 * (nrot + lane) + 1];
          const float ra = a * c - b * sn, rb = b * c + a * sn;
          a = ra;
          b = rb;
        }
        Pair<T>::st(cache + (slot * G + (hs - H - G)) * rs + 2 * lane, a, b);
      }
    }
  }
}

at::Tensor attn_qkv_prep(const at::Tensor& z, int64_t H, int64_t G, int64_t dk, int64_t dv, const c10::optional<at::Tensor>& q_norm,
                         const c10::optional<at::Tensor>& k_norm, double eps, const at::Tensor& pos, const at::Tensor& freq, int64_t rot_dims,
                         bool interleaved, double amp, const c10::optional<at::Tensor>& vfreq, at::Tensor cache, const at::Tensor& slots,
                         bool v_from_k, const c10::optional<at::Tensor>& v_first, const c10::optional<at::Tensor>& v_lambda) {
  check_rows(z, "z");
  const int64_t T = z.size(0);
  HYB_CHECK(H >= 1 && G >= 1 && H % G == 0 && dk >= 1 && dv >= 1 && z.size(1) >= (H + G) * dk + (v_from_k ? 0 : G * dv),
            "z: [T, >= H*dk + G*dk + G*dv]");
  auto f32v = [](const at::Tensor& t, int64_t n) { return t.is_cuda() && t.is_contiguous() && t.scalar_type() == at::kFloat && t.numel() == n; };
  HYB_CHECK(q_norm.has_value() == k_norm.has_value(), "q and k are normed together or not at all");
  if (q_norm.has_value()) HYB_CHECK(f32v(*q_norm, dk) && f32v(*k_norm, dk), "q / k norm weights: fp32 [dk]");
  HYB_CHECK(!v_from_k || (dv == dk && !vfreq.has_value() && !v_first.has_value()), "values that are the keys: dv == dk, neither turned nor mixed");
  HYB_CHECK(v_first.has_value() == v_lambda.has_value(), "the value mix takes its rows and its factor together");
  if (v_first.has_value()) {
    check_rows(*v_first, "v_first");
    HYB_CHECK(v_first->size(0) == T && v_first->size(1) == G * dv && v_first->scalar_type() == z.scalar_type() && f32v(*v_lambda, 1) && !vfreq.has_value(),
              "v_first: [T, G*dv] of z's dtype, v_lambda fp32 [1], no turn of the values");
  }
  const float* qn_p = q_norm.has_value() ? q_norm->data_ptr<float>() : nullptr;
  const float* kn_p = k_norm.has_value() ? k_norm->data_ptr<float>() : nullptr;
  const void* vf_p = v_first.has_value() ? v_first->data_ptr() : nullptr;
  const int64_t vf_st = v_first.has_value() ? v_first->stride(0) : 0;
  const float* lam_p = v_lambda.has_value() ? v_lambda->data_ptr<float>() : nullptr;
  HYB_CHECK(rot_dims % 2 == 0 && rot_dims >= 0 && rot_dims <= dk && f32v(freq, rot_dims / 2), "rotary: even dims <= dk, fp32 frequencies [dims/2]");
  if (vfreq.has_value()) HYB_CHECK(dv % 2 == 0 && f32v(*vfreq, dv / 2), "value rotation: even dv, fp32 frequencies [dv/2]");
  HYB_CHECK(cache.is_cuda() && cache.is_contiguous() && cache.dim() == 3 && cache.size(2) == G * (dv + dk) && cache.scalar_type() == z.scalar_type(),
            "cache: contiguous [blocks, block_size, G * (dv + dk)] of the activation dtype");
  HYB_CHECK(pos.is_cuda() && pos.is_contiguous() && pos.scalar_type() == at::kInt && pos.numel() == T && slots.is_cuda() && slots.is_contiguous() &&
                slots.scalar_type() == at::kLong && slots.numel() == T, "pos int32 [T], slots int64 [T]");
  c10::DeviceGuard guard(z.device());
  at::Tensor q = at::empty({T, H, dk}, z.options());
  if (T == 0) return q;
  dispatch_act(z, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    const bool vf_ok = !v_first.has_value() || (vf_st % 2 == 0 && reinterpret_cast<uintptr_t>(vf_p) % 8 == 0);
    if (T >= 256 && interleaved && dk % 2 == 0 && dv % 2 == 0 && dk <= 128 && dv <= 128 && z.stride(0) % 2 == 0 &&
        reinterpret_cast<uintptr_t>(z.data_ptr()) % 8 == 0 && vf_ok) {
      attn_qkv_prep_pairs_kernel<Tt><<<dim3((unsigned)T), 256, (size_t)(rot_dims + dv) * sizeof(float), cur_stream()>>>(
          (const Tt*)z.data_ptr(), z.stride(0), qn_p, kn_p, pos.data_ptr<int>(), freq.data_ptr<float>(),
          vfreq.has_value() ? vfreq->data_ptr<float>() : nullptr, (Tt*)q.data_ptr(), (Tt*)cache.data_ptr(), slots.data_ptr<int64_t>(), (int)H,
          (int)G, (int)dk, (int)dv, (int)rot_dims, (float)amp, (float)eps, v_from_k ? 1 : 0, (const Tt*)vf_p, vf_st, lam_p);
      return;
    }
    // few tokens (decode steps): one wave per head slot, up to 16; many tokens: 4 waves per token fill the chip
    const unsigned nthreads = T >= 256 ? 256u : (unsigned)std::min<int64_t>(16, std::max<int64_t>(4, H + 2 * G)) * 64;
    attn_qkv_prep_kernel<Tt><<<dim3((unsigned)T), nthreads, (size_t)(rot_dims + dv) * sizeof(float), cur_stream()>>>(
        (const Tt*)z.data_ptr(), z.stride(0), qn_p, kn_p, pos.data_ptr<int>(), freq.data_ptr<float>(),
        vfreq.has_value() ? vfreq->data_ptr<float>() : nullptr, (Tt*)q.data_ptr(), (Tt*)cache.data_ptr(), slots.data_ptr<int64_t>(), (int)H,
        (int)G, (int)dk, (int)dv, (int)rot_dims, interleaved ? 1 : 0, (float)amp, (float)eps, v_from_k ? 1 : 0, (const Tt*)vf_p, vf_st, lam_p);
  });
  return q;
}

}  // namespace llmctl_hybrid
