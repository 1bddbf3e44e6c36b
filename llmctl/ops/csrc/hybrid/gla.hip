// Gated linear attention: per (sequence, head) a memory S [dk, dv] (fp32) whose key rows decay by a
// data-dependent factor, S_t = diag(a_t) S_(t-1) + k_t v_t^T, read out as o_t = S_t^T q_t.
//
//   gla_scan           token by token; one wave per (sequence, head, 64 value columns): a lane owns one
//                      value column and keeps its dk state entries in registers, so update and read-out are
//                      lane-local; a_t, k_t, q_t reach all lanes through a wave-private LDS line.  The decay
//                      a_t = sigmoid(z_t + bias)^(1/tau) is computed here as exp(log_sigmoid / tau) in fp32.
//   gla_chunk_combine  the memory at the first token of every chunk of a portion from the chunks' own
//                      contributions and total decays (S_end = diag(D) S_begin + S_loc), and the sequence's
//                      new carried memory.
#include "hybrid_common.h"

namespace llmctl_hybrid {

namespace {
constexpr int TB = 8;  // tokens fetched ahead as one batch

struct GlaArgs {
  const void* q;
  const void* k;
  const void* v;
  int64_t q_st, q_sh, k_st, k_sh, v_st, v_sh;  // token and head strides (elements)
  const float* z;                              // [T, H * dk] decay logits
  int64_t z_st;
  const float* zb;  // [H * dk]
  float inv_tau, qscale;
  float* S;  // [slots, H, dk, dv]
  const int* slots;
  const int* cu;
  const int* start;
  float* logd;  // nullptr, or [sequences, H, dk]: the sum of log a_t over the sequence's tokens of this step
  float* out;   // nullptr, or [T, H, dv]
  int H, dk, dv, write_state;
};

__device__ __forceinline__ float log_sigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

template <typename T, int KT>
__global__ __launch_bounds__(64) void gla_scan_kernel(GlaArgs a) {
  constexpr int NR = (KT + 63) / 64;
  __shared__ __attribute__((aligned(16))) float line[2][3 * KT];  // [decay | k | q * qscale], two tokens in flight
  const int sq = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int t_a = a.cu[sq], t_b = a.cu[sq + 1];
  if (t_a == t_b) return;
  const int H = a.H, dk = a.dk, dv = a.dv;
  const int col = blockIdx.z * 64 + lane;
  const bool cok = col < dv;
  const int colc = cok ? col : dv - 1;
  const int64_t slot = a.slots[sq];
  float* Sb = a.S + (slot * H + h) * (int64_t)dk * dv;
  float S[KT];
  const bool fresh = a.start[sq] == 0;
#pragma unroll
  for (int d = 0; d < KT; ++d) S[d] = (!fresh && d < dk) ? Sb[(int64_t)d * dv + colc] : 0.f;
  const T* qp = reinterpret_cast<const T*>(a.q) + (int64_t)h * a.q_sh;
  const T* kp = reinterpret_cast<const T*>(a.k) + (int64_t)h * a.k_sh;
  const T* vp = reinterpret_cast<const T*>(a.v) + (int64_t)h * a.v_sh + colc;
  const float* zp = a.z + (int64_t)h * dk;
  float zbias[NR], ld[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int c = lane + 64 * i;
    zbias[i] = c < dk ? a.zb[h * dk + c] : 0.f;
    ld[i] = 0.f;
  }
  float kn[TB][NR], qn[TB][NR], zn[TB][NR], vn[TB];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int j = 0; j < TB; ++j) {
      const int64_t t = min(t0 + j, t_b - 1);
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        const int c = lane + 64 * i;
        const bool ok = c < dk;
        kn[j][i] = ok ? ldf(kp + t * a.k_st + c) : 0.f;
        qn[j][i] = ok ? ldf(qp + t * a.q_st + c) : 0.f;
        zn[j][i] = ok ? zp[t * a.z_st + c] : 0.f;
      }
      vn[j] = ldf(vp + t * a.v_st);
    }
  };
  fetch(t_a);
  for (int t0 = t_a; t0 < t_b; t0 += TB) {
    float kc[TB][NR], qc[TB][NR], zc[TB][NR], vc[TB];
#pragma unroll
    for (int j = 0; j < TB; ++j) {
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        kc[j][i] = kn[j][i];
        qc[j][i] = qn[j][i];
        zc[j][i] = zn[j][i];
      }
      vc[j] = vn[j];
    }
    if (t0 + TB < t_b) fetch(t0 + TB);
#pragma unroll
    for (int j = 0; j < TB; ++j) {
      const int t = t0 + j;
      if (t < t_b) {
        float* ln = line[j & 1];
#pragma unroll
        for (int i = 0; i < NR; ++i) {
          const int c = lane + 64 * i;
          if (c < KT) {
            float al = 1.f;  // channels past dk: their state entries stay zero
            if (c < dk) {
              const float la = log_sigmoid(zc[j][i] + zbias[i]) * a.inv_tau;
              ld[i] += la;
              al = expf(la);
            }
            ln[c] = al;
            ln[KT + c] = kc[j][i];
            ln[2 * KT + c] = qc[j][i] * a.qscale;
          }
        }
        __builtin_amdgcn_wave_barrier();
        const float vv = vc[j];
        float num[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int d = 0; d < KT; d += 4) {
          const float4 a4 = *reinterpret_cast<const float4*>(ln + d);
          const float4 k4 = *reinterpret_cast<const float4*>(ln + KT + d);
          const float4 q4 = *reinterpret_cast<const float4*>(ln + 2 * KT + d);
          S[d] = a4.x * S[d] + k4.x * vv;
          S[d + 1] = a4.y * S[d + 1] + k4.y * vv;
          S[d + 2] = a4.z * S[d + 2] + k4.z * vv;
          S[d + 3] = a4.w * S[d + 3] + k4.w * vv;
          num[0] += S[d] * q4.x;
          num[1] += S[d + 1] * q4.y;
          num[2] += S[d + 2] * q4.z;
          num[3] += S[d + 3] * q4.w;
        }
        if (cok && a.out != nullptr) a.out[((int64_t)t * H + h) * dv + col] = (num[0] + num[1]) + (num[2] + num[3]);
        __builtin_amdgcn_wave_barrier();
      }
    }
  }
  if (a.write_state && cok) {
#pragma unroll
    for (int d = 0; d < KT; ++d)
      if (d < dk) Sb[(int64_t)d * dv + col] = S[d];
  }
  if (a.logd != nullptr && blockIdx.z == 0) {
#pragma unroll
    for (int i = 0; i < NR; ++i)
      if (lane + 64 * i < dk) a.logd[((int64_t)sq * H + h) * dk + lane + 64 * i] = ld[i];
  }
}

// Sequence s has chunks [base[s], base[s+1]); chunk p run from zeros left (loc, logd)[p].  For every chunk
// the memory at its first token goes to init[p]: the sequence's carried memory (zeros at position 0) for its
// first chunk, then S' = exp(logd) S + loc; what follows the last chunk is the sequence's new carried memory.
// One thread per memory entry, chunks in order.
__global__ void gla_chunk_combine_kernel(float* __restrict__ Sp, const int* __restrict__ slots, const int* __restrict__ start,
                                         const int* __restrict__ base, const float* __restrict__ loc, const float* __restrict__ logd,
                                         float* __restrict__ init, int H, int dk, int dv) {
  const int s = blockIdx.x, h = blockIdx.y;
  const int64_t per = (int64_t)dk * dv;
  const int64_t e = (int64_t)blockIdx.z * blockDim.x + threadIdx.x;
  if (e >= per || base[s] == base[s + 1]) return;
  const int d = (int)(e / dv);
  float* real = Sp + ((int64_t)slots[s] * H + h) * per + e;
  float val = start[s] == 0 ? 0.f : *real;
  for (int p = base[s]; p < base[s + 1]; ++p) {
    init[((int64_t)p * H + h) * per + e] = val;
    val = expf(logd[((int64_t)p * H + h) * dk + d]) * val + loc[((int64_t)p * H + h) * per + e];
  }
  *real = val;
}

static void head_view(const at::Tensor& t, const char* name, int64_t T, int64_t H, at::ScalarType dt) {
  HYB_CHECK(t.is_cuda() && t.dim() == 3 && t.size(0) == T && t.size(1) == H && (t.size(2) == 1 || t.stride(2) == 1) && t.scalar_type() == dt,
            name, ": [T, H, d] with unit last stride, one dtype for q, k, v");
}
}  // namespace

at::Tensor gla_scan(const at::Tensor& q, const at::Tensor& k, const at::Tensor& v, const at::Tensor& z, const at::Tensor& z_bias,
                    double tau, double qscale, at::Tensor S, const at::Tensor& slots, const at::Tensor& cu, const at::Tensor& start,
                    const c10::optional<at::Tensor>& logd, bool write_out, bool write_state) {
  HYB_CHECK(q.dim() == 3, "q: [T, H, dk]");
  const int64_t T = q.size(0), H = q.size(1), dk = q.size(2), dv = v.dim() == 3 ? v.size(2) : 0;
  head_view(q, "q", T, H, q.scalar_type());
  head_view(k, "k", T, H, q.scalar_type());
  head_view(v, "v", T, H, q.scalar_type());
  HYB_CHECK(k.size(2) == dk && dk >= 1 && dk <= 256 && dv >= 1, "key size 1 .. 256, value size >= 1");
  HYB_CHECK(z.is_cuda() && z.dim() == 2 && z.size(0) == T && z.size(1) == H * dk && z.scalar_type() == at::kFloat && (z.size(1) == 1 || z.stride(1) == 1),
            "decay logits: fp32 [T, H * dk]");
  HYB_CHECK(z_bias.is_cuda() && z_bias.scalar_type() == at::kFloat && z_bias.is_contiguous() && z_bias.numel() == H * dk, "decay bias: fp32 [H * dk]");
  HYB_CHECK(S.is_cuda() && S.is_contiguous() && S.scalar_type() == at::kFloat && S.dim() == 4 && S.size(1) == H && S.size(2) == dk && S.size(3) == dv,
            "state: contiguous fp32 [slots, H, dk, dv]");
  auto i32 = [](const at::Tensor& t) { return t.is_cuda() && t.is_contiguous() && t.scalar_type() == at::kInt; };
  HYB_CHECK(i32(slots) && i32(cu) && i32(start), "slots, cu, start: contiguous int32 GPU tensors");
  const int64_t ns = slots.numel();
  HYB_CHECK(cu.numel() == ns + 1 && start.numel() == ns, "cu [n + 1], start [n], slots [n]");
  HYB_CHECK(tau > 0.0, "tau > 0");
  if (logd.has_value())
    HYB_CHECK(logd->is_cuda() && logd->is_contiguous() && logd->scalar_type() == at::kFloat && logd->numel() == ns * H * dk, "log decay sums: fp32 [n, H, dk]");
  c10::DeviceGuard guard(q.device());
  at::Tensor out = write_out ? at::empty({T, H, dv}, q.options().dtype(at::kFloat)) : at::Tensor();
  if (T == 0 || ns == 0) return write_out ? out : at::empty({0}, q.options().dtype(at::kFloat));
  HYB_CHECK(H <= 65535 && (dv + 63) / 64 <= 65535, "grid too large");
  GlaArgs a;
  a.q = q.data_ptr(), a.k = k.data_ptr(), a.v = v.data_ptr();
  a.q_st = q.stride(0), a.q_sh = q.stride(1), a.k_st = k.stride(0), a.k_sh = k.stride(1), a.v_st = v.stride(0), a.v_sh = v.stride(1);
  a.z = z.data_ptr<float>(), a.z_st = z.stride(0), a.zb = z_bias.data_ptr<float>();
  a.inv_tau = (float)(1.0 / tau), a.qscale = (float)qscale;
  a.S = S.data_ptr<float>(), a.slots = slots.data_ptr<int>(), a.cu = cu.data_ptr<int>(), a.start = start.data_ptr<int>();
  a.logd = logd.has_value() ? logd->data_ptr<float>() : nullptr;
  a.out = write_out ? out.data_ptr<float>() : nullptr;
  a.H = (int)H, a.dk = (int)dk, a.dv = (int)dv;
  a.write_state = write_state ? 1 : 0;  // off for chunks re-run from their true memory: the combine pass has stored the new one
  dim3 grid((unsigned)ns, (unsigned)H, (unsigned)((dv + 63) / 64));
  hipStream_t st = cur_stream();
  dispatch_act(q, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    if (dk <= 16) gla_scan_kernel<Tt, 16><<<grid, 64, 0, st>>>(a);
    else if (dk <= 32) gla_scan_kernel<Tt, 32><<<grid, 64, 0, st>>>(a);
    else if (dk <= 48) gla_scan_kernel<Tt, 48><<<grid, 64, 0, st>>>(a);
    else if (dk <= 64) gla_scan_kernel<Tt, 64><<<grid, 64, 0, st>>>(a);
    else if (dk <= 96) gla_scan_kernel<Tt, 96><<<grid, 64, 0, st>>>(a);
    else if (dk <= 128) gla_scan_kernel<Tt, 128><<<grid, 64, 0, st>>>(a);
    else if (dk <= 192) gla_scan_kernel<Tt, 192><<<grid, 64, 0, st>>>(a);
    else gla_scan_kernel<Tt, 256><<<grid, 64, 0, st>>>(a);
  });
  return write_out ? out : at::empty({0}, q.options().dtype(at::kFloat));
}

void gla_chunk_combine(at::Tensor S, const at::Tensor& slots, const at::Tensor& start, const at::Tensor& base, const at::Tensor& loc,
                       const at::Tensor& logd, at::Tensor init) {
  HYB_CHECK(S.is_cuda() && S.is_contiguous() && S.scalar_type() == at::kFloat && S.dim() == 4, "state: contiguous fp32 [slots, H, dk, dv]");
  const int64_t H = S.size(1), dk = S.size(2), dv = S.size(3);
  auto f32 = [](const at::Tensor& t) { return t.is_cuda() && t.is_contiguous() && t.scalar_type() == at::kFloat; };
  auto i32 = [](const at::Tensor& t) { return t.is_cuda() && t.is_contiguous() && t.scalar_type() == at::kInt; };
  HYB_CHECK(f32(loc) && f32(logd) && f32(init) && loc.dim() == 4 && loc.sizes() == init.sizes() && loc.size(1) == H && loc.size(2) == dk && loc.size(3) == dv,
            "chunk contributions and chunk-start memories: fp32 [chunks, H, dk, dv]");
  const int64_t P = loc.size(0);
  HYB_CHECK(logd.numel() == P * H * dk, "log decay sums: fp32 [chunks, H, dk]");
  HYB_CHECK(i32(slots) && i32(start) && i32(base) && start.numel() == slots.numel() && base.numel() == slots.numel() + 1, "slots [n], start [n], base [n + 1]: int32");
  const int64_t ns = slots.numel();
  if (ns == 0 || P == 0) return;
  c10::DeviceGuard guard(S.device());
  const int64_t per = dk * dv;
  HYB_CHECK(H <= 65535 && (per + 255) / 256 <= 65535, "grid too large");
  gla_chunk_combine_kernel<<<dim3((unsigned)ns, (unsigned)H, (unsigned)((per + 255) / 256)), 256, 0, cur_stream()>>>(
      S.data_ptr<float>(), slots.data_ptr<int>(), start.data_ptr<int>(), base.data_ptr<int>(), loc.data_ptr<float>(), logd.data_ptr<float>(),
      init.data_ptr<float>(), (int)H, (int)dk, (int)dv);
}

}  // namespace llmctl_hybrid
