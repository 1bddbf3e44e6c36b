// Latent attention on the matrix cores (bf16; MFMA 32x32x16), prompt portions and decode rows alike.
//
// The cache row [latent | rotary key] of width R is key and, in its first ``rank`` entries, value; the
// queries come in the same layout (see latent_attn.hip).  This is the flash-attention forward of the
// framework's paged prefill kernel re-cut for that layout:
//   * a workgroup (4 waves) owns 128 query rows = TB tokens x HB heads of one sequence (HB = 1 for
//     long portions, = the head count for decode rows and short portions, where the heads of a token
//     fill the tile and share every key row);
//   * tiles of 64 keys, gathered through the block table into LDS once per workgroup: a "row image"
//     of all of R (in column blocks of 128) for S^T = K Q^T, and a "transposed-read image" of the
//     column blocks that hold this workgroup's value columns for O^T += V^T P^T;
//   * Q fragments stay in registers for the whole key loop; softmax is lane-local (query on the lane),
//     exp2 domain, deferred rescale; the sink starts the running maximum and the denominator;
//   * the key loop runs only over the tiles that the rows' windows touch.
// Value columns beyond 256 go to further workgroups (blockIdx.z), which recompute the scores.
// Shapes it takes: R and rank multiples of 8, R <= 640; anything else runs the generic kernels.
#include "attn_common.h"
#include "hybrid_common.h"

namespace llmctl_hybrid {
using namespace llmctl::attn;

namespace {
constexpr int LKB = 64;         // keys per tile
constexpr int LROWB = 256;      // bytes of one row of a 128-column block image
constexpr int LIMG = LKB * LROWB;
constexpr float kRescaleTh = 8.f;
constexpr float kLog2e = 1.4426950408889634f;

struct LArgs {
  const unsigned short* qa;
  const unsigned short* cache;
  unsigned short* out;
  const int* bt;
  const int* cu;   // nullptr: one query row per sequence (decode)
  const int* ctx;
  const float* sink;    // nullptr: no sink
  const float* hscale;  // nullptr or a factor on every head's scores
  const float* ofreq;   // nullptr, or [rk / 2]: the output's neighbour pairs are turned back by -position * ofreq
  const float* dist_a;  // SIG forms: [H] each; dist_a ln(1 + dist_b (i - j)) is taken off the scaled score and a visible
  const float* dist_b;  // key weighs sigmoid(score + sig_bias); dist_a may be nullptr (no penalty)
  const float* sig_bias;
  int H, R, rk, bs, maxb, window, HB, nvt;
  int G, rs, koff, chunk, hpg;  // kv groups, row width, key's first column, chunk mask size, head tiles per group
  int keep;                     // the window spares the keys at positions below this
  float scale_log2;
  float cap_log2, cap_inv2;     // CAP forms: x (log2 domain) = cap_log2 * tanh(s * scale); cap_inv2 = 2 log2(e) scale / cap
  // decode rows with the key range split over blockIdx.x (few sequences would otherwise leave the chip
  // idle): each split writes its unnormalised fp32 output and (running maximum, denominator) here
  int nsplit;
  float* ws_o;   // [rows, nsplit, rk]
  float* ws_ml;  // [rows, nsplit, 2]
};

// ROT: the output's neighbour pairs are turned back by the query's position (a.ofreq); a template flag
// so that the forms without it keep their register budget.  SIG: the weights are sigmoids of the scores
// (after the distance penalty), not a softmax: no running maximum, no rescale, no denominator; the splits
// of decode rows are merged as a plain sum (m = 0 everywhere, l = 1 in the first split only).  CAP: the scaled score
// s becomes cap tanh(s / cap) before masks and softmax (tanh y = 1 - 2 / (1 + e^(2y))).
template <int NCB, int NDB, bool ROT, bool SIG = false, bool CAP = false>
__global__ __launch_bounds__(256, 1) void latent_attn_mfma_kernel(LArgs a) {
  constexpr int NKS = NCB * 8;
  constexpr int NTB = (NDB + 3) / 4;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  // the tile images: one set, or two (the fill of tile t + 1 then runs beside the products of tile t)
  // where two fit LDS
  constexpr int BUFB = (NCB + NTB) * LIMG;
  constexpr bool DB = 2 * BUFB + 1024 <= 160 * 1024;

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int r = lane & 31, hh = lane >> 5;
  const int n = blockIdx.y;
  const int hg = blockIdx.z / a.nvt, v0 = (blockIdx.z % a.nvt) * (NDB * 32);
  const int P = a.H / a.G;                       // query heads per kv group
  const int grp = hg / a.hpg, hsub = (hg % a.hpg) * a.HB;  // this workgroup's kv group, its first head inside it
  const int q_begin = a.cu ? a.cu[n] : n;
  const int qlen = a.cu ? a.cu[n + 1] - q_begin : 1;
  const int HB = a.HB, TB = 128 / HB;
  const int split = a.nsplit > 1 ? blockIdx.x : 0;
  // prompt portions: the last query blocks of a sequence see the most keys; they are dispatched first
  const int tok0 = a.nsplit > 1 ? 0 : (int)(gridDim.x - 1 - blockIdx.x) * TB;
  if (tok0 >= qlen) return;
  const int ctx = a.ctx[n];
  const int pos0 = ctx - qlen;
  const int row = wave * 32 + r;
  const int my_tok = tok0 + row / HB, my_head = grp * P + hsub + row % HB;
  const bool valid = my_tok < qlen && hsub + row % HB < P;
  const int tokc = min(my_tok, qlen - 1), headc = grp * P + min(hsub + row % HB, P - 1);
  const int my_pos = pos0 + tokc;
  const int* btn = a.bt + (long)n * a.maxb;

  bf16x8_t qf[NKS];
  {
    const unsigned short* Qp = a.qa + ((long)(q_begin + tokc) * a.H + headc) * a.R;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      const int col = ks * 16 + 8 * hh;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (col < a.R) v = gload16(Qp + col);
      qf[ks] = __builtin_bit_cast(bf16x8_t, v);
    }
  }
  f32x16 o[NDB];
#pragma unroll
  for (int d = 0; d < NDB; ++d)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[d][i] = 0.f;
  float m_i = -INFINITY, l_i = 0.f;
  if (a.sink != nullptr) {  // the sink: one unit of mass at its own logit
    m_i = a.sink[headc] * kLog2e;
    l_i = 1.0f;
  }
  const float my_scale = a.scale_log2 * (a.hscale != nullptr ? a.hscale[headc] : 1.0f);
  if (split > 0) {                                 // (the sink is counted by the first split only)
    m_i = -INFINITY;
    l_i = 0.f;
  }
  float pen_a = 0.f, pen_b = 0.f, sig_b2 = 0.f;
  if constexpr (SIG) {
    m_i = 0.f;
    l_i = split == 0 ? 1.f : 0.f;
    if (a.dist_a != nullptr) pen_a = a.dist_a[headc], pen_b = a.dist_b[headc];
    sig_b2 = a.sig_bias[headc] * kLog2e;
  }

  const int first_pos = pos0 + tok0, last_pos = pos0 + min(tok0 + TB, qlen) - 1;
  // the first key a query at position p may see: inside its window and inside its chunk
  auto first_key = [&](int p) { return max(max(p - a.window + 1, (p / a.chunk) * a.chunk), 0); };
  const int t_first = first_key(first_pos) / LKB, t_end = last_pos / LKB + 1;
  // tiles before the window whose first keys it spares (those of the chunk of the block's first row; a block that
  // spans two chunks meets the second one inside the window's tiles): the key loop runs over them first.  Loop
  // index i in [t_lo, t_hi) stands for tile i < n_kept ? kept0 + i : t_first + i - n_kept.
  const int kept0 = ((first_pos / a.chunk) * a.chunk) / LKB;
  const int n_kept = a.keep > 0 ? max(min((a.keep + LKB - 1) / LKB, t_first) - kept0, 0) : 0;
  auto tile_of = [&](int i) { return i < n_kept ? kept0 + i : t_first + i - n_kept; };
  int t_lo = 0, t_hi = n_kept + t_end - t_first;
  if (a.nsplit > 1) {
    const int per = (t_hi - t_lo + a.nsplit - 1) / a.nsplit;
    t_lo += split * per;
    t_hi = min(t_hi, t_lo + per);
  }
  // this wave's rows: positions [w_first, w_last]
  const int w_first = pos0 + min(tok0 + (wave * 32) / HB, qlen - 1);
  const int w_last = pos0 + min(tok0 + (wave * 32 + 31) / HB, qlen - 1);
  const bool wave_live = tok0 + (wave * 32) / HB < qlen && hsub + (HB >= 32 ? (wave * 32) % HB : 0) < P;
  const int w_lo = first_key(w_first), my_lo = first_key(my_pos);
  const int my_c0 = (my_pos / a.chunk) * a.chunk;  // first position of this row's chunk
  const int w_lo_last = first_key(w_last);  // first_key never decreases with the position
  // lane-only parts of the LDS read addresses, so that the key loop adds constants to them
  int tr_lo[4], tr_hi[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) tr_frag_offs<128>(c * 32, lane, tr_lo[c], tr_hi[c]);
  // K fragment of k-step ks, rows kb * 32 + r: chunk (2 ks + hh) ^ (r & 15) = (2 ks) ^ (hh ^ (r & 15))
  const int k_row = r * LROWB, k_x = (hh ^ (r & 15)) << 4;

  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const unsigned lds_base = lds_addr(smem);
  // cache slots of a tile's 64 keys, looked up in the block table one tile ahead (double-buffered)
  int* slot_lds = reinterpret_cast<int*>(smem + (DB ? 2 : 1) * BUFB);
  auto load_slots = [&](int t, int buf) {
    if (tid < LKB) {
      const int key = min(t * LKB + tid, ctx - 1);
      slot_lds[buf * LKB + tid] = btn[key / a.bs] * a.bs + key % a.bs;
    }
  };
  // LDS-DMA fill: every wave instruction moves 4 key rows x 256 B of one image straight from the cache
  // to LDS (no registers, all pieces of the tile in flight at once); the images' swizzles are applied
  // to the source chunk.  Keys past the context and columns past the row read a valid neighbour instead
  // (finite data): such keys are masked below and such columns meet zero Q entries or are never stored.
  auto fill = [&](int sbuf, int ibuf) {
#pragma unroll 4
    for (int g = wave_u; g < 16 * (NCB + NTB); g += 4) {
      const int img = g >> 4, rg = g & 15;
      const int krow = rg * 4 + (lane >> 4), chp = lane & 15;
      const long slot = slot_lds[sbuf * LKB + krow];
      int col;
      if (img < NCB) {
        col = a.koff + (img * 16 + (chp ^ swz_row<128>(krow))) * 8;
      } else {
        col = ((v0 / 128 + (img - NCB)) * 16 + (chp ^ swz_tr<128>(krow))) * 8;
      }
      col = min(col, a.rs - 8);
      dma16(a.cache + (slot * a.G + grp) * a.rs + col, lds_base + (unsigned)(ibuf * BUFB + img * LIMG + rg * 1024));
    }
  };
  // double-buffered form: the slots of tile t + 2 are requested BEFORE the fill of tile t + 1 is issued and
  // stored to LDS at the top of the next iteration, so that no wave waits on its own fill in between (a
  // wave's memory operations complete in order)
  auto slot_of = [&](int t) {
    const int key = min(t * LKB + tid, ctx - 1);
    return btn[key / a.bs] * a.bs + key % a.bs;
  };
  int pend = 0;
  if (t_lo < t_hi) load_slots(tile_of(t_lo), 0);
  if constexpr (DB) {
    if (t_lo < t_hi) {
      __syncthreads();
      if (t_lo + 1 < t_hi && tid < LKB) pend = slot_of(tile_of(t_lo + 1));
      fill(0, 0);
    }
  }
  for (int t = t_lo; t < t_hi; ++t) {
    const int sbuf = (t - t_lo) & 1;
    const unsigned char* Ks = smem + (DB ? sbuf * BUFB : 0);
    const unsigned char* Vs = Ks + NCB * LIMG;
    if constexpr (DB) {
      // tile t was requested one iteration ago.  After the barrier every wave's pieces of it have landed,
      // every wave is done with tile t - 1 (its images may be overwritten) and the slots of t + 1 are visible
      if (t + 1 < t_hi && tid < LKB) slot_lds[(sbuf ^ 1) * LKB + tid] = pend;
      vm_wait<0>();
      __syncthreads();
      if (t + 2 < t_hi && tid < LKB) pend = slot_of(tile_of(t + 2));
      if (t + 1 < t_hi) fill(sbuf ^ 1, sbuf ^ 1);
    } else {
      __syncthreads();
      fill(sbuf, 0);
      if (t + 1 < t_hi) load_slots(tile_of(t + 1), sbuf ^ 1);
      vm_wait<0>();
      __syncthreads();
    }
    const int kv0 = tile_of(t) * LKB;
    if (!wave_live || kv0 > w_last || (kv0 + LKB - 1 < w_lo && kv0 >= a.keep)) continue;

    f32x16 s[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int i = 0; i < 16; ++i) s[kb][i] = 0.f;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const bf16x8_t kf = lds_read_b128(Ks + (ks >> 3) * LIMG + kb * 32 * LROWB, k_row + (k_x ^ (((2 * ks) & 15) << 4)));
        s[kb] = mfma32(kf, qf[ks], s[kb]);
      }
    }
    bf16x8_t pb[2][2];
    if constexpr (SIG) {
      // x (log2 domain) = s * scale - a log2(1 + b (i - j)) + bias; weight = 1 / (1 + 2^-x); hidden keys weigh 0
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        float p[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = kv0 + kb * 32 + acc_row(i, hh);
          const float dist = (float)max(my_pos - key, 0);
          const float x = s[kb][i] * my_scale - pen_a * __log2f(1.0f + pen_b * dist) + sig_b2;
          const float w = __builtin_amdgcn_rcpf(1.0f + fast_exp2(-x));
          p[i] = (!valid || key > my_pos || (key < my_lo && (key >= a.keep || key < my_c0)) || key >= ctx) ? 0.f : w;
        }
        pb[kb][0] = to_bf16x8(p);
        pb[kb][1] = to_bf16x8(p + 8);
      }
    } else {
      float mx = -INFINITY;
      if (kv0 + LKB - 1 <= w_first && kv0 >= w_lo_last && kv0 + LKB - 1 < ctx) {
        // every key of the tile is visible to every row of this wave: no mask (rows past the portion's end
        // carry finite scores of a repeated row and are never stored)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            if constexpr (CAP) s[kb][i] = a.cap_log2 * (1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + fast_exp2(s[kb][i] * a.cap_inv2)));
            else s[kb][i] *= my_scale;
            mx = fmaxf(mx, s[kb][i]);
          }
        if (!valid) mx = -INFINITY;  // such a row must not trigger the wave's rescale
      } else {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            float x;
            if constexpr (CAP) x = a.cap_log2 * (1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + fast_exp2(s[kb][i] * a.cap_inv2)));
            else x = s[kb][i] * my_scale;
            const int key = kv0 + kb * 32 + acc_row(i, hh);
            if (!valid || key > my_pos || (key < my_lo && (key >= a.keep || key < my_c0)) || key >= ctx) x = -INFINITY;
            s[kb][i] = x;
            mx = fmaxf(mx, x);
          }
      }
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      const bool grow = __builtin_amdgcn_ballot_w64(mx > m_i + kRescaleTh) != 0;
      const float m_raw = grow ? fmaxf(m_i, mx) : m_i;
      const float m_new = m_raw == -INFINITY ? 0.f : m_raw;  // nothing seen yet (a later split, all keys masked)
      float rs = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        float p[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          p[i] = fast_exp2(s[kb][i] - m_new);
          rs += p[i];
        }
        pb[kb][0] = to_bf16x8(p);
        pb[kb][1] = to_bf16x8(p + 8);
      }
      rs += __shfl_xor(rs, 32);
      if (grow) {
        const float alpha = fast_exp2(m_i - m_new);
        l_i *= alpha;
#pragma unroll
        for (int d = 0; d < NDB; ++d)
#pragma unroll
          for (int i = 0; i < 16; ++i) o[d][i] *= alpha;
      }
      l_i += rs;
      m_i = m_raw;
    }
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int d = 0; d < NDB; ++d) {
          const bf16x8_t vf = tr_frag_at<128>(Vs + (d >> 2) * LIMG, kb * 32 + 16 * st, tr_lo[d & 3], tr_hi[d & 3]);
          o[d] = mfma32(vf, pb[kb][st], o[d]);
        }
  }

  if (valid && a.nsplit > 1) {
    const long rowi = (long)(q_begin + my_tok) * a.H + my_head;
    float* Wp = a.ws_o + (rowi * a.nsplit + split) * a.rk;
#pragma unroll
    for (int d = 0; d < NDB; ++d)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int col = v0 + d * 32 + 8 * g + 4 * hh;
        if (col < a.rk) *reinterpret_cast<float4*>(Wp + col) = make_float4(o[d][4 * g], o[d][4 * g + 1], o[d][4 * g + 2], o[d][4 * g + 3]);
      }
    if (v0 == 0 && hh == 0) {
      a.ws_ml[(rowi * a.nsplit + split) * 2] = m_i;
      a.ws_ml[(rowi * a.nsplit + split) * 2 + 1] = l_i;
    }
  } else if (valid) {
    const float inv = 1.f / l_i;
    unsigned short* Op = a.out + ((long)(q_begin + my_tok) * a.H + my_head) * a.rk;
#pragma unroll
    for (int d = 0; d < NDB; ++d)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int col = v0 + d * 32 + 8 * g + 4 * hh;
        if (col < a.rk) {
          if constexpr (ROT) {  // turn the neighbour pairs (col, col + 1), (col + 2, col + 3) back
#pragma unroll
            for (int j = 0; j < 4; j += 2) {
              float sn, cs;
              sincosf((float)my_pos * a.ofreq[(col + j) >> 1], &sn, &cs);
              const float u = o[d][4 * g + j], w = o[d][4 * g + j + 1];
              o[d][4 * g + j] = u * cs + w * sn;
              o[d][4 * g + j + 1] = w * cs - u * sn;
            }
          }
          unsigned short w4[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) w4[j] = __bfloat16_as_ushort(__float2bfloat16(o[d][4 * g + j] * inv));
          *reinterpret_cast<uint2*>(Op + col) =
              make_uint2((unsigned)w4[0] | ((unsigned)w4[1] << 16), (unsigned)w4[2] | ((unsigned)w4[3] << 16));
        }
      }
  }
}

// out[row] = sum_s o_s 2^(m_s - M) / sum_s l_s 2^(m_s - M), M = max_s m_s (splits that saw nothing: m = -inf, l = 0)
__global__ void latent_split_merge_kernel(const float* __restrict__ ws_o, const float* __restrict__ ws_ml, unsigned short* __restrict__ out,
                                          int nsplit, int rk, const float* __restrict__ ofreq, const int* __restrict__ ctx, int H) {
  const long row = blockIdx.x;
  const float pos = ofreq != nullptr ? (float)(ctx[row / H] - 1) : 0.f;  // one row per sequence: its last position
  const float* ml = ws_ml + row * nsplit * 2;
  float M = -INFINITY;
  for (int s = 0; s < nsplit; ++s) M = fmaxf(M, ml[2 * s]);
  float L = 0.f;
  for (int s = 0; s < nsplit; ++s) L += ml[2 * s + 1] * (ml[2 * s] == -INFINITY ? 0.f : fast_exp2(ml[2 * s] - M));
  const float inv = 1.f / L;
  for (int c = threadIdx.x; c < rk; c += blockDim.x) {
    float v = 0.f, w = 0.f;  // column c and, for the turn back, its pair partner c ^ 1
    for (int s = 0; s < nsplit; ++s)
      if (ml[2 * s] != -INFINITY) {
        const float f = fast_exp2(ml[2 * s] - M);
        v += ws_o[(row * nsplit + s) * rk + c] * f;
        if (ofreq != nullptr) w += ws_o[(row * nsplit + s) * rk + (c ^ 1)] * f;
      }
    if (ofreq != nullptr) {
      float sn, cs;
      sincosf(pos * ofreq[c >> 1], &sn, &cs);
      v = (c & 1) ? v * cs - w * sn : v * cs + w * sn;
    }
    out[row * rk + c] = __bfloat16_as_ushort(__float2bfloat16(v * inv));
  }
}

template <int NCB, bool ROT, bool SIG = false, bool CAP = false>
void launch_ncb(const LArgs& a, int ndb, dim3 grid, hipStream_t st) {
  auto go = [&](auto kern, int NDBv) {
    const size_t one = (size_t)(NCB + (NDBv + 3) / 4) * LIMG;
    const size_t lds = (2 * one + 1024 <= 160 * 1024 ? 2 * one : one) + 2 * LKB * sizeof(int);
    HYB_CHECK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) == hipSuccess, "LDS size");
    kern<<<grid, 256, lds, st>>>(a);
  };
  if (ndb == 2) go(latent_attn_mfma_kernel<NCB, 2, ROT, SIG, CAP>, 2);
  else if (ndb == 4) go(latent_attn_mfma_kernel<NCB, 4, ROT, SIG, CAP>, 4);
  else go(latent_attn_mfma_kernel<NCB, 8, ROT, SIG, CAP>, 8);
}
}  // namespace

// turn_back: the output is to be turned back (RowAttnOpts::ofreq) or the weights are sigmoids
// (RowAttnOpts::sig_bias); those forms are built for keys up to 256 wide
bool latent_attn_mfma_ok(const at::Tensor& qa, int64_t rk, int64_t rs, int64_t koff, bool turn_back) {
  const int64_t R = qa.size(2);
  return qa.scalar_type() == at::kBFloat16 && R % 8 == 0 && rk % 8 == 0 && rs % 8 == 0 && koff % 8 == 0 && R <= (turn_back ? 256 : 640) && qa.size(1) >= 1;
}

// cu == nullptr: one query row per sequence.  ``x`` carries the optional parts (see RowAttnOpts).
void latent_attn_mfma(const at::Tensor& qa, const at::Tensor& cache, const at::Tensor& bt, const at::Tensor* cu, const at::Tensor& ctx,
                      int64_t window, const float* sink, double scale, int64_t rk, int64_t max_q, at::Tensor& out, const RowAttnOpts& x) {
  const int64_t H = qa.size(1), R = qa.size(2), ns = ctx.numel();
  const int64_t G = x.groups, P = H / G, rs = cache.size(2) / G;
  const int ncb = (int)((R + 127) / 128);
  const int ndb = rk <= 64 ? 2 : (rk <= 128 ? 4 : 8);
  const int nvt = (int)((rk + ndb * 32 - 1) / (ndb * 32));
  int HB = 1;
  if (max_q < 64) {
    while (HB < P && HB < 128) HB *= 2;
  }
  const int TB = 128 / HB;
  const int hpg = (int)((P + HB - 1) / HB);  // head tiles per kv group
  const int hgroups = (int)G * hpg;
  HYB_CHECK(ns <= 65535 && hgroups * nvt <= 65535, "grid too large");
  // decode rows: split the visible key tiles over workgroups until the launch has a few hundred of them
  int nsplit = 1;
  at::Tensor ws_o, ws_ml;
  if (cu == nullptr && rk % 4 == 0) {
    const int64_t span = std::min<int64_t>(std::min<int64_t>(window, x.chunk), x.max_ctx > 0 ? x.max_ctx : (int64_t)1 << 30);
    const int tiles = (int)std::min<int64_t>((span + LKB - 1) / LKB + 1 + (x.keep_first + LKB - 1) / LKB, 1 << 20);
    const long blocks = (long)ns * hgroups * nvt;
    while (nsplit < tiles && nsplit < 32 && blocks * nsplit < 512) nsplit *= 2;
    if (nsplit > 1) {
      ws_o = at::empty({ns * H, nsplit, rk}, qa.options().dtype(at::kFloat));
      ws_ml = at::empty({ns * H, nsplit, 2}, qa.options().dtype(at::kFloat));
    }
  }
  LArgs a{reinterpret_cast<const unsigned short*>(qa.data_ptr()), reinterpret_cast<const unsigned short*>(cache.data_ptr()),
          reinterpret_cast<unsigned short*>(out.data_ptr()), bt.data_ptr<int>(), cu ? cu->data_ptr<int>() : nullptr, ctx.data_ptr<int>(),
          sink, x.hscale, x.ofreq, x.dist_a, x.dist_b, x.sig_bias, (int)H, (int)R, (int)rk, (int)cache.size(1), (int)bt.size(1), (int)window, HB, nvt,
          (int)G, (int)rs, (int)x.koff, (int)x.chunk, hpg, (int)x.keep_first,
          (float)(scale * 1.4426950408889634), (float)(x.softcap * 1.4426950408889634),
          x.softcap > 0.0 ? (float)(2.0 * 1.4426950408889634 * scale / x.softcap) : 0.f, nsplit, nsplit > 1 ? ws_o.data_ptr<float>() : nullptr,
          nsplit > 1 ? ws_ml.data_ptr<float>() : nullptr};
  dim3 grid(nsplit > 1 ? (unsigned)nsplit : (unsigned)((max_q + TB - 1) / TB), (unsigned)ns, (unsigned)(hgroups * nvt));
  hipStream_t st = cur_stream();
  if (x.softcap > 0.0) {  // built for keys up to 256 wide, plain softmax form (the caller checks)
    HYB_CHECK(x.hscale == nullptr && ncb <= 2, "capped scores: no per-head factor, keys up to 256 wide");
    if (ncb == 1) launch_ncb<1, false, false, true>(a, ndb, grid, st);
    else launch_ncb<2, false, false, true>(a, ndb, grid, st);
  } else if (x.sig_bias != nullptr) {  // built for keys up to 256 wide (latent_attn_mfma_ok)
    if (ncb == 1) launch_ncb<1, false, true>(a, ndb, grid, st);
    else launch_ncb<2, false, true>(a, ndb, grid, st);
  } else if (x.ofreq != nullptr) {
    if (ncb == 1) launch_ncb<1, true>(a, ndb, grid, st);
    else launch_ncb<2, true>(a, ndb, grid, st);
  } else {
    switch (ncb) {
      case 1: launch_ncb<1, false>(a, ndb, grid, st); break;
      case 2: launch_ncb<2, false>(a, ndb, grid, st); break;
      case 3: launch_ncb<3, false>(a, ndb, grid, st); break;
      case 4: launch_ncb<4, false>(a, ndb, grid, st); break;
      default: launch_ncb<5, false>(a, ndb, grid, st); break;
    }
  }
  if (nsplit > 1)
    latent_split_merge_kernel<<<dim3((unsigned)(ns * H)), 128, 0, st>>>(ws_o.data_ptr<float>(), ws_ml.data_ptr<float>(),
                                                                        reinterpret_cast<unsigned short*>(out.data_ptr()), nsplit, (int)rk,
                                                                        x.ofreq, ctx.data_ptr<int>(), (int)H);
}

}  // namespace llmctl_hybrid
