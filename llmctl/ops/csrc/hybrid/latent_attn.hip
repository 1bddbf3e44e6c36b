// Latent attention over a paged cache of rows [latent (rank) | rotary key part (rot)], one row per
// token shared by all heads.  Queries arrive in the same layout (the unrotated query part already
// carried into the latent space), so a score is one dot product of width R = rank + rot and the value
// of a key is the first ``rank`` entries of its row.  Sliding window (key j visible to query i when
// 0 <= i - j < window) and a per-head softmax sink (exp(sink) in the denominator, no value).
//
//   latent_kv_write     RMS norm of the latent, rotary of the key part, write the cache row
//   latent_q_assemble   [q_lat | rotary(q_rot)] per head
//   latent_attn_prefill prompt portions: one query per lane, keys streamed as wave-uniform rows
//   latent_attn_decode  one query per sequence: one key per lane for the scores, lanes over the
//                       value entries for the weighted sum
// Scores, softmax and the accumulators are fp32; angles are fp32 (position * inverse frequency).
#include "hybrid_common.h"

namespace llmctl_hybrid {

template <typename T>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(const T* __restrict__ x, int64_t x_stride, const float* __restrict__ w,
                                                              const int* __restrict__ pos, const float* __restrict__ inv_freq,
                                                              T* __restrict__ cache, const int64_t* __restrict__ slots, int rk,
                                                              int dr, int rot_dims, float eps, int inter, float amp) {
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const int64_t slot = slots[t];
  if (slot < 0) return;
  const T* xr = x + t * x_stride;
  T* out = cache + slot * (int64_t)(rk + dr);
  float q = 0.f;
  for (int c = threadIdx.x; c < rk; c += 256) {
    const float v = ldf(xr + c);
    q += v * v;
  }
  const float rstd = 1.0f / sqrtf(block_sum<4>(q, red) / (float)rk + eps);
  for (int c = threadIdx.x; c < rk; c += 256) stf(out + c, ldf(xr + c) * rstd * w[c]);
  const int half = rot_dims / 2;
  const float p = (float)pos[t];
  for (int i = threadIdx.x; i < half; i += 256) {
    float s, c;
    sincosf(p * inv_freq[i], &s, &c);
    s *= amp;
    c *= amp;
    const int i0 = inter ? 2 * i : i, i1 = inter ? 2 * i + 1 : i + half;  // neighbours or halves
    const float u = ldf(xr + rk + i0), v = ldf(xr + rk + i1);
    stf(out + rk + i0, u * c - v * s);
    stf(out + rk + i1, v * c + u * s);
  }
  for (int i = rot_dims + threadIdx.x; i < dr; i += 256) stf(out + rk + i, ldf(xr + rk + i));
}

template <typename T>
__global__ __launch_bounds__(256) void latent_q_assemble_kernel(const T* __restrict__ ql, int64_t ql_st, int64_t ql_sh,
                                                                const T* __restrict__ q, int64_t q_st, const int* __restrict__ pos,
                                                                const float* __restrict__ inv_freq, T* __restrict__ qa, int H,
                                                                int rk, int dn, int dr, int rot_dims, int inter, float amp) {
  extern __shared__ float cs_tab[];  // the token's [rot_dims / 2][2] cos, sin (times amp), shared by its heads
  const int64_t t = blockIdx.x;
  const int R = rk + dr, half = rot_dims / 2;
  const float p = (float)pos[t];
  for (int i = threadIdx.x; i < half; i += 256) {
    float s, co;
    sincosf(p * inv_freq[i], &s, &co);
    cs_tab[2 * i] = co * amp;
    cs_tab[2 * i + 1] = s * amp;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < H * rk; i += 256) {
    const int h = i / rk, c = i - h * rk;
    qa[(t * H + h) * R + c] = ql[t * ql_st + h * ql_sh + c];
  }
  for (int i = threadIdx.x; i < H * half; i += 256) {
    const int h = i / half, c = i - h * half;
    const float co = cs_tab[2 * c], s = cs_tab[2 * c + 1];
    const T* qr = q + t * q_st + h * (int64_t)(dn + dr) + dn;
    const int i0 = inter ? 2 * c : c, i1 = inter ? 2 * c + 1 : c + half;
    const float u = ldf(qr + i0), v = ldf(qr + i1);
    stf(qa + (t * H + h) * R + rk + i0, u * co - v * s);
    stf(qa + (t * H + h) * R + rk + i1, v * co + u * s);
  }
  const int rest = dr - rot_dims;
  for (int i = threadIdx.x; i < H * rest; i += 256) {
    const int h = i / rest, c = rot_dims + (i - h * rest);
    qa[(t * H + h) * R + rk + c] = q[t * q_st + h * (int64_t)(dn + dr) + dn + c];
  }
}

// ---------------------------------------------------------------------------------------- prefill
// Attention over a paged row cache in its general form (RowAttnOpts): the token's cache row holds G
// sub-rows of width rs, one per kv group; a sub-row's entries [koff, koff + R) are the key and its
// first rk entries the value (latent attention: G = 1, koff = 0, R = rs).
struct GenArgs {
  const int* bt;
  const int* ctx;
  const float* sink;    // nullptr: none
  const float* hscale;  // nullptr: 1
  const float* ofreq;   // nullptr: the output is not turned back
  const float* dist_a;  // nullptr: no distance penalty
  const float* dist_b;
  const float* sig_bias;  // SIG forms: the head's bias inside the sigmoid
  int bt_stride, H, R, rk, bs, window, chunk, G, rs, koff, keep;  // keep: the window spares the keys at positions below it
  float scale, cap, inv_cap;                                       // cap > 0: the scaled score becomes cap tanh(score / cap)
};

__device__ __forceinline__ int first_visible(int p, int window, int chunk) { return max(max(p - window + 1, (p / chunk) * chunk), 0); }

// grid (q tiles of 64, sequences, heads * value tiles); one wave per block, lane = query.
// SIG: a visible key weighs sigmoid(score + bias) and nothing is normalised (no running maximum, no sink).
template <typename T, int VT, bool SIG>
__global__ __launch_bounds__(64) void latent_attn_prefill_kernel(const T* __restrict__ qa, const T* __restrict__ cache, const int* __restrict__ cu,
                                                                 T* __restrict__ out, GenArgs g, int nvt) {
  extern __shared__ float qT[];  // [R][64]
  const int n = blockIdx.y;
  const int h = blockIdx.z / nvt, v0 = (blockIdx.z % nvt) * VT;
  const int H = g.H, R = g.R, rk = g.rk, bs = g.bs;
  const int a = cu[n], qlen = cu[n + 1] - a;
  const int q0 = blockIdx.x * 64;
  if (q0 >= qlen) return;
  const int lane = threadIdx.x;
  const int p0 = g.ctx[n] - qlen;  // position of the sequence's first query row
  const bool live = q0 + lane < qlen;
  const int qp = p0 + q0 + lane;
  const int64_t qrow = ((int64_t)(a + q0 + (live ? lane : 0)) * H + h) * R;
  for (int d = 0; d < R; ++d) qT[d * 64 + lane] = live ? ldf(qa + qrow + d) : 0.f;
  const int last = p0 + min(q0 + 63, qlen - 1);
  const int j0 = first_visible(p0 + q0, g.window, g.chunk);
  const int lo = first_visible(qp, g.window, g.chunk);
  // keys that the window spares: positions [c0, min(keep, j0)) of the chunk of the tile's first query (a tile that
  // spans two chunks starts the second one inside [j0, last], where the chunk test below applies)
  const int c0 = ((p0 + q0) / g.chunk) * g.chunk;
  const int kept = max(min(g.keep, j0) - c0, 0);
  const int cq = (qp / g.chunk) * g.chunk;  // first position of this query's chunk
  const float scale = g.scale * (g.hscale != nullptr ? g.hscale[h] : 1.0f);
  const bool pen = g.dist_a != nullptr;
  const float da = pen ? g.dist_a[h] : 0.f, db = pen ? g.dist_b[h] : 0.f;
  const float sb = SIG ? g.sig_bias[h] : 0.f;
  float m = -INFINITY, l = 0.f;
  if (g.sink != nullptr) {  // the sink: exp(sink - m) with m = sink
    m = g.sink[h];
    l = 1.0f;
  }
  float acc[VT];
#pragma unroll
  for (int i = 0; i < VT; ++i) acc[i] = 0.f;
  const int* btn = g.bt + (int64_t)n * g.bt_stride;
  const int grp = h / (H / g.G);
  for (int jj = -kept; jj <= last - j0; ++jj) {
    const int j = jj < 0 ? c0 + kept + jj : j0 + jj;
    const T* row = cache + (((int64_t)btn[j / bs] * bs + j % bs) * g.G + grp) * g.rs;
    const T* key = row + g.koff;
    float s = 0.f;
    for (int d = 0; d < R; ++d) s += qT[d * 64 + lane] * ldf(key + d);
    s *= scale;
    if (g.cap > 0.f) s = g.cap * tanhf(s * g.inv_cap);
    if (live && j <= qp && (j >= lo || (j < g.keep && j >= cq))) {
      if (pen) s -= da * log1pf(db * (float)(qp - j));
      if constexpr (SIG) {
        const float p = 1.0f / (1.0f + expf(-(s + sb)));
#pragma unroll
        for (int i = 0; i < VT; ++i) acc[i] += p * ldf(row + min(v0 + i, rk - 1));
      } else {
        const float mn = fmaxf(m, s);
        const float corr = expf(m - mn), p = expf(s - mn);  // m = -inf before the first key: corr = 0
        l = l * corr + p;
#pragma unroll
        for (int i = 0; i < VT; ++i) acc[i] = acc[i] * corr + p * ldf(row + min(v0 + i, rk - 1));
        m = mn;
      }
    }
  }
  if (!live) return;
  const float inv = SIG ? 1.0f : 1.0f / l;
  if (g.ofreq != nullptr) {  // neighbour pairs (2m, 2m + 1) turned back by the query's position
#pragma unroll
    for (int i = 0; i < VT; i += 2)
      if (v0 + i + 1 < rk) {
        float sn, cs;
        sincosf((float)qp * g.ofreq[(v0 + i) >> 1], &sn, &cs);
        const float u = acc[i], w = acc[i + 1];
        acc[i] = u * cs + w * sn;
        acc[i + 1] = w * cs - u * sn;
      }
  }
  T* o = out + ((int64_t)(a + q0 + lane) * H + h) * rk;
#pragma unroll
  for (int i = 0; i < VT; ++i)
    if (v0 + i < rk) stf(o + v0 + i, acc[i] * inv);
}

// ----------------------------------------------------------------------------------------- decode
// grid (sequences, heads); 4 waves, each takes chunks of 64 keys (one key per lane for the score).
template <typename T, int NA, bool SIG>
__global__ __launch_bounds__(256) void latent_attn_decode_kernel(const T* __restrict__ qa, const T* __restrict__ cache, T* __restrict__ out,
                                                                 GenArgs g) {
  extern __shared__ float sm[];
  const int H = g.H, R = g.R, rk = g.rk, bs = g.bs;
  float* qs = sm;                                   // [R]
  float* pw = qs + R + (R & 1);                     // [4][64]; the padding keeps ro 8-byte aligned
  int64_t* ro = reinterpret_cast<int64_t*>(pw + 256);  // [4][64]
  float* ml = reinterpret_cast<float*>(ro + 256);   // [4][2]
  float* ac = ml + 8;                               // [4][rk]
  const int n = blockIdx.x, h = blockIdx.y;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int len = g.ctx[n];
  const int lo = first_visible(len - 1, g.window, g.chunk);
  const int c0 = ((len - 1) / g.chunk) * g.chunk;
  const int kept = max(min(g.keep, lo) - c0, 0);  // keys before the window that it spares: [c0, c0 + kept)
  const int nk = kept + len - lo;
  const T* qr = qa + ((int64_t)n * H + h) * R;
  for (int d = threadIdx.x; d < R; d += 256) qs[d] = ldf(qr + d);
  __syncthreads();
  const int* btn = g.bt + (int64_t)n * g.bt_stride;
  const int grp = h / (H / g.G);
  const float scale = g.scale * (g.hscale != nullptr ? g.hscale[h] : 1.0f);
  const bool pen = g.dist_a != nullptr;
  const float da = pen ? g.dist_a[h] : 0.f, db = pen ? g.dist_b[h] : 0.f;
  const float sb = SIG ? g.sig_bias[h] : 0.f;
  float m = SIG ? 0.f : -INFINITY, l = 0.f;
  float acc[NA];
#pragma unroll
  for (int i = 0; i < NA; ++i) acc[i] = 0.f;
  for (int c = wave * 64; c < nk; c += 256) {
    const int ci = c + lane;
    const int j = ci < kept ? c0 + ci : lo + ci - kept;
    const bool ok = ci < nk;
    int64_t slot = 0;
    float s = -INFINITY;
    if (ok) {
      slot = ((int64_t)btn[j / bs] * bs + j % bs) * g.G + grp;
      const T* key = cache + slot * g.rs + g.koff;
      float d0 = 0.f;
      for (int d = 0; d < R; ++d) d0 += qs[d] * ldf(key + d);
      s = d0 * scale;
      if (g.cap > 0.f) s = g.cap * tanhf(s * g.inv_cap);
      if (pen) s -= da * log1pf(db * (float)(len - 1 - j));
    }
    float p, corr;
    if constexpr (SIG) {
      p = ok ? 1.0f / (1.0f + expf(-(s + sb))) : 0.f;
      corr = 1.0f;
      l = 1.0f;  // the waves' parts are summed as they are
    } else {
      const float mn = fmaxf(m, wave_max(s));  // at least one key of the chunk is valid: finite
      p = ok ? expf(s - mn) : 0.f;
      corr = expf(m - mn);                     // m = -inf on the first chunk: 0
      l = l * corr + wave_sum(p);
      m = mn;
    }
    pw[wave * 64 + lane] = p;
    ro[wave * 64 + lane] = slot;
    __builtin_amdgcn_wave_barrier();
    const int cnt = min(64, nk - c);
#pragma unroll
    for (int i = 0; i < NA; ++i) acc[i] *= corr;
    for (int jj = 0; jj < cnt; ++jj) {
      const float pj = pw[wave * 64 + jj];
      const T* row = cache + ro[wave * 64 + jj] * g.rs;
#pragma unroll
      for (int i = 0; i < NA; ++i) {
        const int d = lane + 64 * i;
        if (d < rk) acc[i] += pj * ldf(row + d);
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (lane == 0) {
    ml[wave * 2] = m;
    ml[wave * 2 + 1] = l;
  }
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    const int d = lane + 64 * i;
    if (d < rk) ac[wave * rk + d] = acc[i];
  }
  __syncthreads();
  float M = g.sink != nullptr ? g.sink[h] : -INFINITY;
#pragma unroll
  for (int w = 0; w < 4; ++w) M = fmaxf(M, ml[w * 2]);
  float L = g.sink != nullptr ? expf(g.sink[h] - M) : 0.f;
  float f[4];
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    f[w] = ml[w * 2 + 1] > 0.f ? expf(ml[w * 2] - M) : 0.f;
    L += ml[w * 2 + 1] * f[w];
  }
  if constexpr (SIG) {
#pragma unroll
    for (int w = 0; w < 4; ++w) f[w] = 1.0f;  // (a wave that saw no key holds zeros)
    L = 1.0f;
  }
  T* o = out + ((int64_t)n * H + h) * rk;
  for (int d = threadIdx.x; d < rk; d += 256) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) v += ac[w * rk + d] * f[w];
    if (g.ofreq != nullptr && (d ^ 1) < rk) {  // turned back together with its pair partner d ^ 1
      float u = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) u += ac[w * rk + (d ^ 1)] * f[w];
      float sn, cs;
      sincosf((float)(len - 1) * g.ofreq[d >> 1], &sn, &cs);
      v = (d & 1) ? v * cs - u * sn : v * cs + u * sn;
    }
    stf(o + d, v / L);
  }
}

// latent_attn_mfma.hip: the matrix-core form for bf16 shapes that fit it
bool latent_attn_mfma_ok(const at::Tensor& qa, int64_t rk, int64_t rs, int64_t koff, bool turn_back);
// capped scores are built into the plain softmax form only, for keys up to 256 wide
static bool mfma_cap_ok(const RowAttnOpts& x, int64_t R) {
  return x.softcap == 0.0 || (x.ofreq == nullptr && x.sig_bias == nullptr && x.hscale == nullptr && R <= 256);
}
void latent_attn_mfma(const at::Tensor& qa, const at::Tensor& cache, const at::Tensor& bt, const at::Tensor* cu, const at::Tensor& ctx,
                      int64_t window, const float* sink, double scale, int64_t rk, int64_t max_q, at::Tensor& out, const RowAttnOpts& x);

// ------------------------------------------------------------------------------------------ host
static void check_cache(const at::Tensor& cache, const at::Tensor& like, int64_t R) {
  HYB_CHECK(cache.is_cuda() && cache.is_contiguous() && cache.dim() == 3 && cache.size(2) == R && cache.scalar_type() == like.scalar_type(),
            "cache: contiguous [blocks, block_size, row width] of the activation dtype");
}

static void check_i32(const at::Tensor& t, const char* name) {
  HYB_CHECK(t.is_cuda() && t.is_contiguous() && t.scalar_type() == at::kInt, name, ": contiguous int32 GPU tensor");
}

static bool f32_vec(const at::Tensor& t, int64_t n) {
  return t.is_cuda() && t.scalar_type() == at::kFloat && t.is_contiguous() && t.numel() == n;
}

void latent_kv_write(const at::Tensor& dkv, const at::Tensor& norm_w, double eps, const at::Tensor& pos, const at::Tensor& inv_freq,
                     int64_t rot_dims, at::Tensor cache, const at::Tensor& slots, bool interleaved, double amp) {
  check_rows(dkv, "dkv");
  const int64_t T = dkv.size(0), R = dkv.size(1), rk = norm_w.numel();
  HYB_CHECK(rk >= 1 && rk <= R && norm_w.scalar_type() == at::kFloat && norm_w.is_contiguous(), "norm weight: fp32 [rank]");
  const int64_t dr = R - rk;
  HYB_CHECK(rot_dims % 2 == 0 && rot_dims <= dr && f32_vec(inv_freq, rot_dims / 2), "rotary: even dims <= rot part, fp32 inverse frequencies [dims/2]");
  check_cache(cache, dkv, R);
  check_i32(pos, "pos");
  HYB_CHECK(pos.numel() == T && slots.is_cuda() && slots.is_contiguous() && slots.scalar_type() == at::kLong && slots.numel() == T, "pos int32 [T], slots int64 [T]");
  if (T == 0) return;
  c10::DeviceGuard guard(dkv.device());
  dispatch_act(dkv, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    latent_kv_write_kernel<Tt><<<dim3((unsigned)T), 256, 0, cur_stream()>>>(
        (const Tt*)dkv.data_ptr(), dkv.stride(0), norm_w.data_ptr<float>(), pos.data_ptr<int>(), inv_freq.data_ptr<float>(),
        (Tt*)cache.data_ptr(), slots.data_ptr<int64_t>(), (int)rk, (int)dr, (int)rot_dims, (float)eps, interleaved ? 1 : 0, (float)amp);
  });
}

at::Tensor latent_q_assemble(const at::Tensor& q_lat, const at::Tensor& q, const at::Tensor& pos, const at::Tensor& inv_freq,
                             int64_t rot_dims, int64_t dn, bool interleaved, double amp) {
  HYB_CHECK(q.is_cuda() && q.dim() == 3 && (q.size(2) == 1 || q.stride(2) == 1) && q.stride(1) == q.size(2), "q: [T, H, dn + rot], heads back to back");
  const int64_t T = q.size(0), H = q.size(1), dr = q.size(2) - dn;
  HYB_CHECK(q_lat.is_cuda() && q_lat.dim() == 3 && q_lat.size(0) == T && q_lat.size(1) == H && (q_lat.size(2) == 1 || q_lat.stride(2) == 1) && q_lat.scalar_type() == q.scalar_type(), "q_lat: [T, H, rank], unit last stride, q's dtype");
  const int64_t rk = q_lat.size(2);
  HYB_CHECK(dr >= 0 && rot_dims % 2 == 0 && rot_dims <= dr && f32_vec(inv_freq, rot_dims / 2), "rotary: even dims <= rot part");
  check_i32(pos, "pos");
  HYB_CHECK(pos.numel() == T, "pos: int32 [T]");
  c10::DeviceGuard guard(q.device());
  at::Tensor qa = at::empty({T, H, rk + dr}, q.options());
  if (T == 0) return qa;
  dispatch_act(q, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    latent_q_assemble_kernel<Tt><<<dim3((unsigned)T), 256, (size_t)rot_dims * sizeof(float), cur_stream()>>>(
        (const Tt*)q_lat.data_ptr(), q_lat.stride(0), q_lat.stride(1), (const Tt*)q.data_ptr(), q.stride(0), pos.data_ptr<int>(),
        inv_freq.data_ptr<float>(), (Tt*)qa.data_ptr(), (int)H, (int)rk, (int)dn, (int)dr, (int)rot_dims, interleaved ? 1 : 0, (float)amp);
  });
  return qa;
}

// The optional tensors of the general form, checked; returns the kernels' view of them.
static RowAttnOpts row_opts(const at::Tensor& qa, const at::Tensor& cache, int64_t rk, const c10::optional<at::Tensor>& sink, int64_t groups,
                            int64_t koff, int64_t chunk, const c10::optional<at::Tensor>& hscale, const c10::optional<at::Tensor>& ofreq,
                            int64_t max_ctx, const float** sink_p, const c10::optional<at::Tensor>& sig_bias = c10::nullopt,
                            const c10::optional<at::Tensor>& dist_a = c10::nullopt, const c10::optional<at::Tensor>& dist_b = c10::nullopt,
                            double softcap = 0.0, int64_t keep_first = 0) {
  const int64_t H = qa.size(1), R = qa.size(2);
  HYB_CHECK(groups >= 1 && H % groups == 0 && cache.size(2) % groups == 0, "kv groups must divide the heads and the cache row");
  const int64_t rs = cache.size(2) / groups;
  HYB_CHECK(koff >= 0 && koff + R <= rs && rk >= 1 && rk <= rs, "key [koff, koff + R) and value [0, rk) must lie inside a sub-row");
  HYB_CHECK(chunk >= 1, "chunk >= 1");
  if (sink.has_value()) HYB_CHECK(f32_vec(*sink, H), "sink: fp32 [H]");
  if (hscale.has_value()) HYB_CHECK(f32_vec(*hscale, H), "head scale: fp32 [H]");
  if (ofreq.has_value()) HYB_CHECK(rk % 2 == 0 && f32_vec(*ofreq, rk / 2), "output turn: even value width, fp32 frequencies [rk / 2]");
  *sink_p = sink.has_value() ? sink->data_ptr<float>() : nullptr;
  RowAttnOpts x;
  x.groups = groups;
  x.koff = koff;
  x.chunk = std::min<int64_t>(chunk, (int64_t)1 << 30);
  x.hscale = hscale.has_value() ? hscale->data_ptr<float>() : nullptr;
  x.ofreq = ofreq.has_value() ? ofreq->data_ptr<float>() : nullptr;
  x.max_ctx = max_ctx;
  HYB_CHECK(dist_a.has_value() == dist_b.has_value(), "the distance penalty takes both of its vectors");
  if (dist_a.has_value()) HYB_CHECK(f32_vec(*dist_a, H) && f32_vec(*dist_b, H), "distance penalty: fp32 [H] twice");
  if (sig_bias.has_value()) HYB_CHECK(f32_vec(*sig_bias, H) && !sink.has_value() && !ofreq.has_value(), "sigmoid weights: fp32 bias [H], no sink, no output turn");
  x.dist_a = dist_a.has_value() ? dist_a->data_ptr<float>() : nullptr;
  x.dist_b = dist_b.has_value() ? dist_b->data_ptr<float>() : nullptr;
  x.sig_bias = sig_bias.has_value() ? sig_bias->data_ptr<float>() : nullptr;
  HYB_CHECK(softcap >= 0.0 && keep_first >= 0, "softcap >= 0, keep_first >= 0");
  x.softcap = softcap;
  x.keep_first = std::min<int64_t>(keep_first, (int64_t)1 << 30);
  return x;
}

static GenArgs gen_args(const at::Tensor& qa, const at::Tensor& cache, const at::Tensor& bt, const at::Tensor& ctx, const float* sink,
                        int64_t window, double scale, int64_t rk, const RowAttnOpts& x) {
  GenArgs g;
  g.bt = bt.data_ptr<int>();
  g.ctx = ctx.data_ptr<int>();
  g.sink = sink;
  g.hscale = x.hscale;
  g.ofreq = x.ofreq;
  g.dist_a = x.dist_a;
  g.dist_b = x.dist_b;
  g.sig_bias = x.sig_bias;
  g.bt_stride = (int)bt.size(1);
  g.H = (int)qa.size(1);
  g.R = (int)qa.size(2);
  g.rk = (int)rk;
  g.bs = (int)cache.size(1);
  g.window = (int)window;
  g.chunk = (int)x.chunk;
  g.G = (int)x.groups;
  g.rs = (int)(cache.size(2) / x.groups);
  g.koff = (int)x.koff;
  g.keep = (int)x.keep_first;
  g.scale = (float)scale;
  g.cap = (float)x.softcap;
  g.inv_cap = x.softcap > 0.0 ? (float)(1.0 / x.softcap) : 0.f;
  return g;
}

at::Tensor latent_attn_prefill(const at::Tensor& qa, const at::Tensor& cache, const at::Tensor& bt, const at::Tensor& cu,
                               const at::Tensor& ctx, int64_t window, const c10::optional<at::Tensor>& sink, double scale, int64_t rk,
                               int64_t max_q, bool mfma, int64_t groups, int64_t koff, int64_t chunk,
                               const c10::optional<at::Tensor>& hscale, const c10::optional<at::Tensor>& ofreq,
                               const c10::optional<at::Tensor>& sig_bias, const c10::optional<at::Tensor>& dist_a,
                               const c10::optional<at::Tensor>& dist_b, double softcap, int64_t keep_first) {
  HYB_CHECK(qa.is_cuda() && qa.is_contiguous() && qa.dim() == 3, "qa: contiguous [T, H, R]");
  const int64_t T = qa.size(0), H = qa.size(1), R = qa.size(2);
  check_cache(cache, qa, cache.size(2));
  check_i32(bt, "block tables");
  check_i32(cu, "cu");
  check_i32(ctx, "ctx");
  const int64_t ns = ctx.numel();
  HYB_CHECK(bt.dim() == 2 && bt.size(0) == ns && cu.numel() == ns + 1, "block tables [n, max_blocks], cu [n + 1], ctx [n]");
  HYB_CHECK(window >= 1 && max_q >= 1, "window >= 1, max_q >= 1");
  window = std::min<int64_t>(window, (int64_t)1 << 30);
  const float* sink_p;
  const RowAttnOpts x = row_opts(qa, cache, rk, sink, groups, koff, chunk, hscale, ofreq, 0, &sink_p, sig_bias, dist_a, dist_b, softcap, keep_first);
  HYB_CHECK((size_t)R * 64 * sizeof(float) <= 160 * 1024, "key too wide for the query tile in LDS");
  c10::DeviceGuard guard(qa.device());
  at::Tensor out = at::empty({T, H, rk}, qa.options());
  if (T == 0 || ns == 0) return out;
  if (mfma && mfma_cap_ok(x, R) && (x.dist_a == nullptr || x.sig_bias != nullptr) && latent_attn_mfma_ok(qa, rk, cache.size(2) / groups, koff, x.ofreq != nullptr || x.sig_bias != nullptr)) {
    latent_attn_mfma(qa, cache, bt, &cu, ctx, window, sink_p, scale, rk, max_q, out, x);
    return out;
  }
  const int VT = rk <= 32 ? 32 : (rk <= 64 ? 64 : 128);
  const int nvt = (int)((rk + VT - 1) / VT);
  HYB_CHECK(H * nvt <= 65535 && ns <= 65535, "grid too large");
  dim3 grid((unsigned)((max_q + 63) / 64), (unsigned)ns, (unsigned)(H * nvt));
  const size_t lds = (size_t)R * 64 * sizeof(float);
  const GenArgs g = gen_args(qa, cache, bt, ctx, sink_p, window, scale, rk, x);
  dispatch_act(qa, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    auto launch = [&](auto kern) {
      if (lds > 64 * 1024) HYB_CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess, "LDS size");
      kern<<<grid, 64, lds, cur_stream()>>>((const Tt*)qa.data_ptr(), (const Tt*)cache.data_ptr(), cu.data_ptr<int>(), (Tt*)out.data_ptr(), g, nvt);
    };
    if (x.sig_bias != nullptr) {
      if (VT == 32) launch(latent_attn_prefill_kernel<Tt, 32, true>);
      else if (VT == 64) launch(latent_attn_prefill_kernel<Tt, 64, true>);
      else launch(latent_attn_prefill_kernel<Tt, 128, true>);
    } else {
      if (VT == 32) launch(latent_attn_prefill_kernel<Tt, 32, false>);
      else if (VT == 64) launch(latent_attn_prefill_kernel<Tt, 64, false>);
      else launch(latent_attn_prefill_kernel<Tt, 128, false>);
    }
  });
  return out;
}

at::Tensor latent_attn_decode(const at::Tensor& qa, const at::Tensor& cache, const at::Tensor& bt, const at::Tensor& ctx,
                              int64_t window, const c10::optional<at::Tensor>& sink, double scale, int64_t rk, bool mfma, int64_t groups,
                              int64_t koff, int64_t chunk, const c10::optional<at::Tensor>& hscale, const c10::optional<at::Tensor>& ofreq,
                              int64_t max_ctx, const c10::optional<at::Tensor>& sig_bias, const c10::optional<at::Tensor>& dist_a,
                              const c10::optional<at::Tensor>& dist_b, double softcap, int64_t keep_first) {
  HYB_CHECK(qa.is_cuda() && qa.is_contiguous() && qa.dim() == 3, "qa: contiguous [n, H, R]");
  const int64_t ns = qa.size(0), H = qa.size(1), R = qa.size(2);
  check_cache(cache, qa, cache.size(2));
  check_i32(bt, "block tables");
  check_i32(ctx, "ctx");
  HYB_CHECK(bt.dim() == 2 && bt.size(0) == ns && ctx.numel() == ns, "block tables [n, max_blocks], ctx [n]");
  HYB_CHECK(window >= 1, "window >= 1");
  window = std::min<int64_t>(window, (int64_t)1 << 30);
  const float* sink_p;
  const RowAttnOpts x = row_opts(qa, cache, rk, sink, groups, koff, chunk, hscale, ofreq, max_ctx, &sink_p, sig_bias, dist_a, dist_b, softcap, keep_first);
  c10::DeviceGuard guard(qa.device());
  at::Tensor out = at::empty({ns, H, rk}, qa.options());
  if (ns == 0) return out;
  if (mfma && mfma_cap_ok(x, R) && (x.dist_a == nullptr || x.sig_bias != nullptr) && latent_attn_mfma_ok(qa, rk, cache.size(2) / groups, koff, x.ofreq != nullptr || x.sig_bias != nullptr)) {
    latent_attn_mfma(qa, cache, bt, nullptr, ctx, window, sink_p, scale, rk, 1, out, x);
    return out;
  }
  HYB_CHECK(rk <= 512, "generic decode kernel: value width <= 512");
  const int64_t Rp = R + (R & 1);  // keeps the int64 array 8-byte aligned
  const size_t lds = (size_t)(Rp + 256) * 4 + 256 * 8 + 8 * 4 + (size_t)4 * rk * 4;
  HYB_CHECK(lds <= 64 * 1024 && H <= 65535, "key / value too wide");
  dim3 grid((unsigned)ns, (unsigned)H);
  const GenArgs g = gen_args(qa, cache, bt, ctx, sink_p, window, scale, rk, x);
  dispatch_act(qa, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    auto launch = [&](auto kern) { kern<<<grid, 256, lds, cur_stream()>>>((const Tt*)qa.data_ptr(), (const Tt*)cache.data_ptr(), (Tt*)out.data_ptr(), g); };
    if (x.sig_bias != nullptr) {
      if (rk <= 128) launch(latent_attn_decode_kernel<Tt, 2, true>);
      else launch(latent_attn_decode_kernel<Tt, 8, true>);
    } else {
      if (rk <= 128) launch(latent_attn_decode_kernel<Tt, 2, false>);
      else launch(latent_attn_decode_kernel<Tt, 8, false>);
    }
  });
  return out;
}

}  // namespace llmctl_hybrid
