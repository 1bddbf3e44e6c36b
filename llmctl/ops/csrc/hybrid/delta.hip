// The generalized delta rule: per (sequence, head) a memory S [dk, dv] (fp32),
//   S_t = diag(w_t) S_(t-1) - (a_t u_t) (u_t^T S_(t-1)) + k_t v_t^T   (both terms read the old memory),   o_t = S_t^T r_t,
// with the decay w = exp(-coef sigmoid(zw + w0)), the removal rate a = sigmoid(za + ab) per key channel and the
// unit key u = k / sqrt(sum k^2 + key_eps) of the head, all computed here in fp32.
//
//   delta_scan           token by token; one wave per (sequence, head, 64 value columns): a lane owns one value column
//                        and keeps its dk memory entries in registers, so u^T S, the update and the read-out are
//                        lane-local; w, a u, u, k, r of a token reach all lanes through a wave-private LDS line.
//                        With ``P`` given, further waves run the same recurrence on the columns of the identity and
//                        without the k v^T term: that is the product of the tokens' transition matrices
//                        A_t = diag(w_t) - (a_t u_t) u_t^T, which carries a memory across the sequence's tokens.
//   delta_chunk_combine  the memory at the first token of every chunk of a portion from the chunks' own contributions
//                        and transition products (S_end = P S_begin + S_loc), and the sequence's new carried memory
//                        (a small matrix product per chunk, register-tiled out of LDS).
#include "hybrid_common.h"

namespace llmctl_hybrid {

namespace {
constexpr int TB = 8;  // tokens fetched ahead as one batch

struct DeltaArgs {
  const void* r;
  const void* k;
  const void* v;
  const void* za;
  int64_t r_st, r_sh, k_st, k_sh, v_st, v_sh, za_st;  // token and head strides (elements)
  const float* zw;                                     // [T, H * dk] decay logits
  int64_t zw_st;
  const float* w0;  // [H * dk]
  const float* ab;  // [H * dk]
  float coef, keps;
  float* S;  // [slots, H, dk, dv]
  const int* slots;
  const int* cu;
  const int* start;
  float* P;    // nullptr, or [sequences, H, dk, dk]: the product of the transition matrices of the sequence's tokens, transposed
  float* out;  // nullptr, or [T, H, dv]
  int H, dk, dv, write_state;
};

__device__ __forceinline__ float sigm(float x) { return 1.0f / (1.0f + expf(-x)); }

template <typename T, int KT>
__global__ __launch_bounds__(64) void delta_scan_kernel(DeltaArgs a) {
  constexpr int NR = (KT + 63) / 64;
  __shared__ __attribute__((aligned(16))) float line[2][5 * KT];  // [w | a u | u | k | r], two tokens in flight
  const int sq = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int t_a = a.cu[sq], t_b = a.cu[sq + 1];
  if (t_a == t_b) return;
  const int H = a.H, dk = a.dk, dv = a.dv;
  const int nvt = (dv + 63) / 64;
  const bool ident = (int)blockIdx.z >= nvt;  // a tile of the transition product (only launched when a.P is given)
  const int ncol = ident ? dk : dv;
  const int col = (ident ? (int)blockIdx.z - nvt : (int)blockIdx.z) * 64 + lane;
  const bool cok = col < ncol;
  const int colc = cok ? col : ncol - 1;
  const int64_t slot = a.slots[sq];
  float* Sb = a.S + (slot * H + h) * (int64_t)dk * dv;
  float S[KT];
  const bool fresh = a.start[sq] == 0;
#pragma unroll
  for (int d = 0; d < KT; ++d) {
    if (ident) S[d] = d == colc ? 1.f : 0.f;
    else S[d] = (!fresh && d < dk) ? Sb[(int64_t)d * dv + colc] : 0.f;
  }
  const T* rp = reinterpret_cast<const T*>(a.r) + (int64_t)h * a.r_sh;
  const T* kp = reinterpret_cast<const T*>(a.k) + (int64_t)h * a.k_sh;
  const T* vp = reinterpret_cast<const T*>(a.v) + (int64_t)h * a.v_sh + (ident ? 0 : colc);
  const T* ap = reinterpret_cast<const T*>(a.za) + (int64_t)h * dk;
  const float* zp = a.zw + (int64_t)h * dk;
  float w0[NR], ab[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int c = lane + 64 * i;
    w0[i] = c < dk ? a.w0[h * dk + c] : 0.f;
    ab[i] = c < dk ? a.ab[h * dk + c] : 0.f;
  }
  float kn[TB][NR], rn[TB][NR], zn[TB][NR], an[TB][NR], vn[TB];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int j = 0; j < TB; ++j) {
      const int64_t t = min(t0 + j, t_b - 1);
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        const int c = lane + 64 * i;
        const bool ok = c < dk;
        kn[j][i] = ok ? ldf(kp + t * a.k_st + c) : 0.f;
        rn[j][i] = ok ? ldf(rp + t * a.r_st + c) : 0.f;
        an[j][i] = ok ? ldf(ap + t * a.za_st + c) : 0.f;
        zn[j][i] = ok ? zp[t * a.zw_st + c] : 0.f;
      }
      vn[j] = ident ? 0.f : ldf(vp + t * a.v_st);
    }
  };
  fetch(t_a);
  for (int t0 = t_a; t0 < t_b; t0 += TB) {
    float kc[TB][NR], rc[TB][NR], wc[TB][NR], ac[TB][NR], vc[TB], inv[TB];
#pragma unroll
    for (int j = 0; j < TB; ++j) {
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        kc[j][i] = kn[j][i];
        rc[j][i] = rn[j][i];
        wc[j][i] = expf(-a.coef * sigm(zn[j][i] + w0[i]));
        ac[j][i] = sigm(an[j][i] + ab[i]);
        ss += kc[j][i] * kc[j][i];
      }
      vc[j] = vn[j];
      inv[j] = 1.0f / sqrtf(wave_sum(ss) + a.keps);  // eight independent reductions: off the token loop's path
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
            const bool ok = c < dk;  // channels past dk: their memory entries stay zero
            const float u = kc[j][i] * inv[j];
            ln[c] = ok ? wc[j][i] : 1.f;
            ln[KT + c] = ok ? ac[j][i] * u : 0.f;
            ln[2 * KT + c] = ok ? u : 0.f;
            ln[3 * KT + c] = kc[j][i];
            ln[4 * KT + c] = rc[j][i];
          }
        }
        __builtin_amdgcn_wave_barrier();
        const float vv = vc[j];
        float us[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int d = 0; d < KT; d += 4) {
          const float4 u4 = *reinterpret_cast<const float4*>(ln + 2 * KT + d);
          us[0] += u4.x * S[d];
          us[1] += u4.y * S[d + 1];
          us[2] += u4.z * S[d + 2];
          us[3] += u4.w * S[d + 3];
        }
        const float uS = (us[0] + us[1]) + (us[2] + us[3]);
        float num[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int d = 0; d < KT; d += 4) {
          const float4 w4 = *reinterpret_cast<const float4*>(ln + d);
          const float4 a4 = *reinterpret_cast<const float4*>(ln + KT + d);
          const float4 k4 = *reinterpret_cast<const float4*>(ln + 3 * KT + d);
          const float4 r4 = *reinterpret_cast<const float4*>(ln + 4 * KT + d);
          S[d] = w4.x * S[d] - a4.x * uS + k4.x * vv;
          S[d + 1] = w4.y * S[d + 1] - a4.y * uS + k4.y * vv;
          S[d + 2] = w4.z * S[d + 2] - a4.z * uS + k4.z * vv;
          S[d + 3] = w4.w * S[d + 3] - a4.w * uS + k4.w * vv;
          num[0] += S[d] * r4.x;
          num[1] += S[d + 1] * r4.y;
          num[2] += S[d + 2] * r4.z;
          num[3] += S[d + 3] * r4.w;
        }
        if (!ident && cok && a.out != nullptr) a.out[((int64_t)t * H + h) * dv + col] = (num[0] + num[1]) + (num[2] + num[3]);
        __builtin_amdgcn_wave_barrier();
      }
    }
  }
  if (ident) {
    if (cok) {
      float* Pb = a.P + ((int64_t)sq * H + h) * dk * dk;
#pragma unroll
      for (int d = 0; d < KT; ++d)
        if (d < dk) Pb[(int64_t)col * dk + d] = S[d];  // transposed: the combine pass reads rows of P^T
    }
  } else if (a.write_state && cok) {
#pragma unroll
    for (int d = 0; d < KT; ++d)
      if (d < dk) Sb[(int64_t)d * dv + col] = S[d];
  }
}

// Sequence s has chunks [base[s], base[s+1]); chunk p run from zeros left loc[p] and its transition product, stored
// transposed: Pt[p][j][d] = P[d][j].  For every chunk the memory at its first token goes to init[p]: the sequence's
// carried memory (zeros at position 0) for its first chunk, then S' = P S + loc; what follows the last chunk is the
// sequence's new carried memory.  The columns of a memory are independent under P, so a workgroup owns (sequence,
// head, ``cpb`` value columns) and walks the chunks in order: its columns of the running memory [dk, cpb] and the
// chunk's Pt live in LDS, a thread owns a 4 x 4 tile of the product (both operands read as 16-byte rows) over a
// ``JG``-th of the sum, the parts are added through LDS, and the next chunk's Pt and loc are fetched into registers
// while this chunk's product runs.  dk, dv and cpb are multiples of 4.
constexpr int CB_NT = 256;
constexpr int CB_PRE = 48;   // Pt entries a thread fetches ahead: dk * dk <= CB_PRE * CB_NT
constexpr int CB_TILES = 2;  // 4 x 4 tiles per thread when one thread sums all of j: dk * cpb <= 16 * CB_TILES * CB_NT

__global__ __launch_bounds__(CB_NT) void delta_chunk_combine_kernel(float* __restrict__ Sp, const int* __restrict__ slots,
                                                                    const int* __restrict__ start, const int* __restrict__ base,
                                                                    const float* __restrict__ loc, const float* __restrict__ Pt,
                                                                    float* __restrict__ init, int H, int dk, int dv, int cpb, int JG) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int s = blockIdx.x, h = blockIdx.y, cb = blockIdx.z * cpb, tid = threadIdx.x;
  const int p_lo = base[s], p_hi = base[s + 1];
  if (p_lo == p_hi) return;
  const int per = dk * dv, pp = dk * dk, mine = dk * cpb;
  const int tcols = cpb / 4, ntiles = (dk / 4) * tcols;
  float* val = lds;             // [dk][cpb]
  float* pt = lds + mine;       // [dk][dk], pt[j][d]
  float* red = pt + pp;         // [JG - 1][ntiles][16]
  // this thread's tiles and its part of the sum
  const int g = JG > 1 ? tid / ntiles : 0;
  int tile[CB_TILES];
#pragma unroll
  for (int k = 0; k < CB_TILES; ++k) {
    if (JG > 1) tile[k] = (k == 0 && g < JG) ? tid % ntiles : -1;
    else tile[k] = tid + k * CB_NT < ntiles ? tid + k * CB_NT : -1;
  }
  const int jlen = (dk + JG - 1) / JG;
  const int j_lo = min(g * jlen, dk), j_hi = min(j_lo + jlen, dk);
  float* real = Sp + ((int64_t)slots[s] * H + h) * per;
  const bool fresh = start[s] == 0;
  for (int e = tid; e < mine; e += CB_NT) val[e] = fresh ? 0.f : real[(e / cpb) * dv + cb + e % cpb];
  float pre[CB_PRE];
  auto fetch = [&](int p) {
    const float* src = Pt + ((int64_t)p * H + h) * pp;
#pragma unroll
    for (int i = 0; i < CB_PRE; ++i) {
      const int e = tid + i * CB_NT;
      pre[i] = e < pp ? src[e] : 0.f;
    }
  };
  // the chunk's own contribution, fetched a chunk ahead like its Pt (by the threads that finish the sums)
  float nl[CB_TILES][4][4];
  auto fetch_loc = [&](int p) {
    const float* lp = loc + ((int64_t)p * H + h) * per + cb;
#pragma unroll
    for (int k = 0; k < CB_TILES; ++k) {
      if (tile[k] >= 0 && g == 0) {
        const int d0 = (tile[k] / tcols) * 4, c0 = (tile[k] % tcols) * 4;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float4 l4 = *reinterpret_cast<const float4*>(lp + (d0 + r) * dv + c0);
          nl[k][r][0] = l4.x, nl[k][r][1] = l4.y, nl[k][r][2] = l4.z, nl[k][r][3] = l4.w;
        }
      }
    }
  };
#pragma unroll
  for (int k = 0; k < CB_TILES; ++k)
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
      for (int c = 0; c < 4; ++c) nl[k][r][c] = 0.f;
  fetch(p_lo);
  fetch_loc(p_lo);
  for (int p = p_lo; p < p_hi; ++p) {
#pragma unroll
    for (int i = 0; i < CB_PRE; ++i) {
      const int e = tid + i * CB_NT;
      if (e < pp) pt[e] = pre[i];
    }
    __syncthreads();  // this chunk's Pt and the memory before it are in LDS
    float* ip = init + ((int64_t)p * H + h) * per + cb;
    for (int e = tid; e < mine; e += CB_NT) ip[(e / cpb) * dv + e % cpb] = val[e];
    float acc[CB_TILES][4][4];
#pragma unroll
    for (int k = 0; k < CB_TILES; ++k)
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[k][r][c] = nl[k][r][c];
    if (p + 1 < p_hi) {
      fetch(p + 1);
      fetch_loc(p + 1);
    }
#pragma unroll
    for (int k = 0; k < CB_TILES; ++k) {
      if (tile[k] >= 0) {
        const int d0 = (tile[k] / tcols) * 4, c0 = (tile[k] % tcols) * 4;
#pragma unroll 4
        for (int j = j_lo; j < j_hi; ++j) {
          const float4 a4 = *reinterpret_cast<const float4*>(pt + j * dk + d0);
          const float4 b4 = *reinterpret_cast<const float4*>(val + j * cpb + c0);
          const float a[4] = {a4.x, a4.y, a4.z, a4.w}, b[4] = {b4.x, b4.y, b4.z, b4.w};
#pragma unroll
          for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[k][r][c] += a[r] * b[c];
        }
      }
    }
    if (JG > 1 && g > 0 && tile[0] >= 0) {
      float* rp = red + ((g - 1) * ntiles + tile[0]) * 16;
#pragma unroll
      for (int r = 0; r < 4; ++r) *reinterpret_cast<float4*>(rp + 4 * r) = make_float4(acc[0][r][0], acc[0][r][1], acc[0][r][2], acc[0][r][3]);
    }
    __syncthreads();  // every read of this chunk's memory and Pt is done; the parts of the sums are in LDS
    if (g == 0) {
#pragma unroll
      for (int k = 0; k < CB_TILES; ++k) {
        if (tile[k] >= 0) {
          const int d0 = (tile[k] / tcols) * 4, c0 = (tile[k] % tcols) * 4;
          if (k == 0)
            for (int gg = 1; gg < JG; ++gg) {
              const float* rp = red + ((gg - 1) * ntiles + tile[0]) * 16;
#pragma unroll
              for (int r = 0; r < 4; ++r) {
                const float4 x4 = *reinterpret_cast<const float4*>(rp + 4 * r);
                acc[0][r][0] += x4.x, acc[0][r][1] += x4.y, acc[0][r][2] += x4.z, acc[0][r][3] += x4.w;
              }
            }
#pragma unroll
          for (int r = 0; r < 4; ++r)
            *reinterpret_cast<float4*>(val + (d0 + r) * cpb + c0) = make_float4(acc[k][r][0], acc[k][r][1], acc[k][r][2], acc[k][r][3]);
        }
      }
    }
  }
  __syncthreads();
  for (int e = tid; e < mine; e += CB_NT) real[(e / cpb) * dv + cb + e % cpb] = val[e];
}

static void head_view(const at::Tensor& t, const char* name, int64_t T, int64_t H, at::ScalarType dt) {
  HYB_CHECK(t.is_cuda() && t.dim() == 3 && t.size(0) == T && t.size(1) == H && (t.size(2) == 1 || t.stride(2) == 1) && t.scalar_type() == dt,
            name, ": [T, H, d] with unit last stride, one dtype for r, k, v");
}
}  // namespace

at::Tensor delta_scan(const at::Tensor& r, const at::Tensor& k, const at::Tensor& v, const at::Tensor& zw, const at::Tensor& w0,
                      const at::Tensor& za, const at::Tensor& ab, double decay_coef, double key_eps, at::Tensor S, const at::Tensor& slots,
                      const at::Tensor& cu, const at::Tensor& start, const c10::optional<at::Tensor>& P, bool write_out, bool write_state) {
  HYB_CHECK(r.dim() == 3, "r: [T, H, dk]");
  const int64_t T = r.size(0), H = r.size(1), dk = r.size(2), dv = v.dim() == 3 ? v.size(2) : 0;
  head_view(r, "r", T, H, r.scalar_type());
  head_view(k, "k", T, H, r.scalar_type());
  head_view(v, "v", T, H, r.scalar_type());
  HYB_CHECK(k.size(2) == dk && dk >= 1 && dk <= 256 && dv >= 1, "key size 1 .. 256, value size >= 1");
  HYB_CHECK(zw.is_cuda() && zw.dim() == 2 && zw.size(0) == T && zw.size(1) == H * dk && zw.scalar_type() == at::kFloat && (zw.size(1) == 1 || zw.stride(1) == 1),
            "decay logits: fp32 [T, H * dk]");
  HYB_CHECK(za.is_cuda() && za.dim() == 2 && za.size(0) == T && za.size(1) == H * dk && za.scalar_type() == r.scalar_type() && (za.size(1) == 1 || za.stride(1) == 1),
            "removal logits: [T, H * dk] of r's dtype");
  auto f32 = [](const at::Tensor& t, int64_t n) { return t.is_cuda() && t.scalar_type() == at::kFloat && t.is_contiguous() && t.numel() == n; };
  HYB_CHECK(f32(w0, H * dk) && f32(ab, H * dk), "decay and removal biases: fp32 [H * dk]");
  HYB_CHECK(S.is_cuda() && S.is_contiguous() && S.scalar_type() == at::kFloat && S.dim() == 4 && S.size(1) == H && S.size(2) == dk && S.size(3) == dv,
            "state: contiguous fp32 [slots, H, dk, dv]");
  auto i32 = [](const at::Tensor& t) { return t.is_cuda() && t.is_contiguous() && t.scalar_type() == at::kInt; };
  HYB_CHECK(i32(slots) && i32(cu) && i32(start), "slots, cu, start: contiguous int32 GPU tensors");
  const int64_t ns = slots.numel();
  HYB_CHECK(cu.numel() == ns + 1 && start.numel() == ns, "cu [n + 1], start [n], slots [n]");
  if (P.has_value()) HYB_CHECK(f32(*P, ns * H * dk * dk), "transition products: fp32 [n, H, dk, dk]");
  c10::DeviceGuard guard(r.device());
  at::Tensor out = write_out ? at::empty({T, H, dv}, r.options().dtype(at::kFloat)) : at::Tensor();
  if (T == 0 || ns == 0) return write_out ? out : at::empty({0}, r.options().dtype(at::kFloat));
  const int64_t tiles = (dv + 63) / 64 + (P.has_value() ? (dk + 63) / 64 : 0);
  HYB_CHECK(H <= 65535 && tiles <= 65535, "grid too large");
  DeltaArgs a;
  a.r = r.data_ptr(), a.k = k.data_ptr(), a.v = v.data_ptr(), a.za = za.data_ptr();
  a.r_st = r.stride(0), a.r_sh = r.stride(1), a.k_st = k.stride(0), a.k_sh = k.stride(1), a.v_st = v.stride(0), a.v_sh = v.stride(1);
  a.za_st = za.stride(0);
  a.zw = zw.data_ptr<float>(), a.zw_st = zw.stride(0), a.w0 = w0.data_ptr<float>(), a.ab = ab.data_ptr<float>();
  a.coef = (float)decay_coef, a.keps = (float)key_eps;
  a.S = S.data_ptr<float>(), a.slots = slots.data_ptr<int>(), a.cu = cu.data_ptr<int>(), a.start = start.data_ptr<int>();
  a.P = P.has_value() ? P->data_ptr<float>() : nullptr;
  a.out = write_out ? out.data_ptr<float>() : nullptr;
  a.H = (int)H, a.dk = (int)dk, a.dv = (int)dv;
  a.write_state = write_state ? 1 : 0;  // off for chunks re-run from their true memory: the combine pass has stored the new one
  dim3 grid((unsigned)ns, (unsigned)H, (unsigned)tiles);
  hipStream_t st = cur_stream();
  dispatch_act(r, [&](auto* tag) {
    using Tt = std::remove_pointer_t<decltype(tag)>;
    if (dk <= 16) delta_scan_kernel<Tt, 16><<<grid, 64, 0, st>>>(a);
    else if (dk <= 32) delta_scan_kernel<Tt, 32><<<grid, 64, 0, st>>>(a);
    else if (dk <= 48) delta_scan_kernel<Tt, 48><<<grid, 64, 0, st>>>(a);
    else if (dk <= 64) delta_scan_kernel<Tt, 64><<<grid, 64, 0, st>>>(a);
    else if (dk <= 96) delta_scan_kernel<Tt, 96><<<grid, 64, 0, st>>>(a);
    else if (dk <= 128) delta_scan_kernel<Tt, 128><<<grid, 64, 0, st>>>(a);
    else if (dk <= 192) delta_scan_kernel<Tt, 192><<<grid, 64, 0, st>>>(a);
    else delta_scan_kernel<Tt, 256><<<grid, 64, 0, st>>>(a);
  });
  return write_out ? out : at::empty({0}, r.options().dtype(at::kFloat));
}

void delta_chunk_combine(at::Tensor S, const at::Tensor& slots, const at::Tensor& start, const at::Tensor& base, const at::Tensor& loc,
                         const at::Tensor& P, at::Tensor init) {
  HYB_CHECK(S.is_cuda() && S.is_contiguous() && S.scalar_type() == at::kFloat && S.dim() == 4, "state: contiguous fp32 [slots, H, dk, dv]");
  const int64_t H = S.size(1), dk = S.size(2), dv = S.size(3);
  auto f32 = [](const at::Tensor& t) { return t.is_cuda() && t.is_contiguous() && t.scalar_type() == at::kFloat; };
  auto i32 = [](const at::Tensor& t) { return t.is_cuda() && t.is_contiguous() && t.scalar_type() == at::kInt; };
  HYB_CHECK(f32(loc) && f32(P) && f32(init) && loc.dim() == 4 && loc.sizes() == init.sizes() && loc.size(1) == H && loc.size(2) == dk && loc.size(3) == dv,
            "chunk contributions and chunk-start memories: fp32 [chunks, H, dk, dv]");
  const int64_t Pn = loc.size(0);
  HYB_CHECK(P.numel() == Pn * H * dk * dk, "transition products: fp32 [chunks, H, dk, dk]");
  HYB_CHECK(i32(slots) && i32(start) && i32(base) && start.numel() == slots.numel() && base.numel() == slots.numel() + 1, "slots [n], start [n], base [n + 1]: int32");
  const int64_t ns = slots.numel();
  if (ns == 0 || Pn == 0) return;
  HYB_CHECK(dk % 4 == 0 && dv % 4 == 0 && dk * dk <= CB_PRE * CB_NT, "combine pass: dk and dv multiples of 4, dk * dk <= 12288");
  // value columns per workgroup; parts of the sum per tile when a workgroup has fewer tiles than threads
  const int64_t cpb = (dv % 16 == 0 && dv > 16) ? 16 : dv;
  const int64_t ntiles = (dk / 4) * (cpb / 4);
  const int64_t JG = ntiles >= CB_NT ? 1 : std::min<int64_t>(4, CB_NT / ntiles);
  HYB_CHECK(ntiles <= CB_TILES * CB_NT, "combine pass: dk * dv too large");
  const size_t lds = (size_t)(dk * cpb + dk * dk + (JG - 1) * ntiles * 16) * sizeof(float);
  HYB_CHECK(lds <= 64 * 1024 && H <= 65535, "memory too large for the combine pass");
  c10::DeviceGuard guard(S.device());
  delta_chunk_combine_kernel<<<dim3((unsigned)ns, (unsigned)H, (unsigned)(dv / cpb)), CB_NT, lds, cur_stream()>>>(
      S.data_ptr<float>(), slots.data_ptr<int>(), start.data_ptr<int>(), base.data_ptr<int>(), loc.data_ptr<float>(), P.data_ptr<float>(),
      init.data_ptr<float>(), (int)H, (int)dk, (int)dv, (int)cpb, (int)JG);
}

}  // namespace llmctl_hybrid
