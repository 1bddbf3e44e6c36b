// Group-limited sigmoid router: scores s = sigmoid(logits) (fp32); the E experts form G equal groups of
// neighbours; a group's score is the sum of its two largest s; only experts of the ``keep`` best
// groups are eligible; the ``top`` largest eligible scores are chosen (ties: the lower index) and are
// the routing weights as they are.  One thread per token.
#include "hybrid_common.h"

namespace llmctl_hybrid {

constexpr int MAXPICK = 64;

__global__ void group_topk_router_kernel(const float* __restrict__ logits, int64_t* __restrict__ idx, float* __restrict__ wgt, int64_t T,
                                         int E, int top, int G, int keep) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const float* z = logits + t * E;
  const int per = E / G;
  int gsel[MAXPICK];
  for (int kk = 0; kk < keep; ++kk) {
    float best = -1.f;
    int bi = -1;
    for (int g = 0; g < G; ++g) {
      bool used = false;
      for (int u = 0; u < kk; ++u) used |= gsel[u] == g;
      if (used) continue;
      float a = -1.f, b = -1.f;  // the two largest scores of the group
      for (int e = g * per; e < (g + 1) * per; ++e) {
        const float s = 1.0f / (1.0f + expf(-z[e]));
        if (s > a) {
          b = a;
          a = s;
        } else if (s > b) {
          b = s;
        }
      }
      const float gs = a + (per > 1 ? b : 0.f);
      if (gs > best) {
        best = gs;
        bi = g;
      }
    }
    gsel[kk] = bi;
  }
  int esel[MAXPICK];
  for (int kk = 0; kk < top; ++kk) {
    float best = -1.f;
    int bi = -1;
    for (int u = 0; u < keep; ++u) {
      const int g = gsel[u];
      for (int e = g * per; e < (g + 1) * per; ++e) {
        bool used = false;
        for (int w = 0; w < kk; ++w) used |= esel[w] == e;
        if (used) continue;
        const float s = 1.0f / (1.0f + expf(-z[e]));
        if (s > best || (s == best && e < bi)) {
          best = s;
          bi = e;
        }
      }
    }
    esel[kk] = bi;
    idx[t * top + kk] = bi;
    wgt[t * top + kk] = best;
  }
}

std::tuple<at::Tensor, at::Tensor> group_topk_router(const at::Tensor& logits, int64_t top, int64_t groups, int64_t keep) {
  HYB_CHECK(logits.is_cuda() && logits.is_contiguous() && logits.dim() == 2 && logits.scalar_type() == at::kFloat, "logits: contiguous fp32 [T, E]");
  const int64_t T = logits.size(0), E = logits.size(1);
  HYB_CHECK(groups >= 1 && E % groups == 0 && keep >= 1 && keep <= groups && top >= 1 && top <= keep * (E / groups) && top <= MAXPICK && keep <= MAXPICK,
            "experts split into equal groups; top fits the kept groups; top, keep <= 64");
  c10::DeviceGuard guard(logits.device());
  at::Tensor idx = at::empty({T, top}, logits.options().dtype(at::kLong));
  at::Tensor wgt = at::empty({T, top}, logits.options());
  if (T == 0) return {idx, wgt};
  group_topk_router_kernel<<<dim3((unsigned)((T + 127) / 128)), 128, 0, cur_stream()>>>(logits.data_ptr<float>(), idx.data_ptr<int64_t>(),
                                                                                       wgt.data_ptr<float>(), T, (int)E, (int)top, (int)groups, (int)keep);
  return {idx, wgt};
}

// Softmax router with a selection bias: s = softmax(logits) (fp32); the ``top`` experts with the largest
// choice score s + bias are chosen (ties: the lower index).  With G > 1 groups the experts form G equal groups of
// neighbours, a group's score is its largest choice score, and only experts of the ``keep`` best groups (ties:
// the lower index) can be chosen.  The weights are the chosen experts' own s, over their sum (+ 1e-20) when
// ``renorm``.  One thread per token.
__global__ void bias_topk_router_kernel(const float* __restrict__ logits, const float* __restrict__ bias, int64_t* __restrict__ idx,
                                        float* __restrict__ wgt, int64_t T, int E, int top, int G, int keep, int renorm) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const float* z = logits + t * E;
  float mx = -INFINITY;
  for (int e = 0; e < E; ++e) mx = fmaxf(mx, z[e]);
  float den = 0.f;
  for (int e = 0; e < E; ++e) den += expf(z[e] - mx);
  const float inv = 1.0f / den;
  const int per = E / G;
  int gsel[MAXPICK];
  if (G > 1) {
    for (int kk = 0; kk < keep; ++kk) {
      float best = -INFINITY;
      int bi = -1;
      for (int g = 0; g < G; ++g) {
        bool used = false;
        for (int u = 0; u < kk; ++u) used |= gsel[u] == g;
        if (used) continue;
        float gs = -INFINITY;
        for (int e = g * per; e < (g + 1) * per; ++e) gs = fmaxf(gs, expf(z[e] - mx) * inv + (bias != nullptr ? bias[e] : 0.f));
        if (bi < 0 || gs > best) {
          best = gs;
          bi = g;
        }
      }
      gsel[kk] = bi;
    }
  }
  int esel[MAXPICK];
  float sum = 0.f;
  for (int kk = 0; kk < top; ++kk) {
    float best = -INFINITY, bs = 0.f;
    int bi = -1;
    for (int e = 0; e < E; ++e) {
      bool used = false;
      for (int w = 0; w < kk; ++w) used |= esel[w] == e;
      if (G > 1) {
        bool in = false;
        for (int u = 0; u < keep; ++u) in |= gsel[u] == e / per;
        used |= !in;
      }
      if (used) continue;
      const float s = expf(z[e] - mx) * inv;
      const float c = s + (bias != nullptr ? bias[e] : 0.f);
      if (bi < 0 || c > best) {
        best = c;
        bs = s;
        bi = e;
      }
    }
    esel[kk] = bi;
    idx[t * top + kk] = bi;
    wgt[t * top + kk] = bs;
    sum += bs;
  }
  if (renorm) {
    const float norm = 1.0f / (sum + 1e-20f);
    for (int kk = 0; kk < top; ++kk) wgt[t * top + kk] *= norm;
  }
}

std::tuple<at::Tensor, at::Tensor> bias_topk_router(const at::Tensor& logits, const c10::optional<at::Tensor>& bias, int64_t top, int64_t groups,
                                                    int64_t keep, bool renorm) {
  HYB_CHECK(logits.is_cuda() && logits.is_contiguous() && logits.dim() == 2 && logits.scalar_type() == at::kFloat, "logits: contiguous fp32 [T, E]");
  const int64_t T = logits.size(0), E = logits.size(1);
  if (bias.has_value()) HYB_CHECK(bias->is_cuda() && bias->is_contiguous() && bias->scalar_type() == at::kFloat && bias->numel() == E, "bias: fp32 [E]");
  HYB_CHECK(top >= 1 && top <= E && top <= MAXPICK, "top in 1 .. min(E, 64)");
  HYB_CHECK(groups >= 1 && E % groups == 0 && keep >= 1 && keep <= groups && keep <= MAXPICK && (groups == 1 || top <= keep * (E / groups)),
            "experts split into equal groups; top fits the kept groups; keep <= 64");
  c10::DeviceGuard guard(logits.device());
  at::Tensor idx = at::empty({T, top}, logits.options().dtype(at::kLong));
  at::Tensor wgt = at::empty({T, top}, logits.options());
  if (T == 0) return {idx, wgt};
  bias_topk_router_kernel<<<dim3((unsigned)((T + 127) / 128)), 128, 0, cur_stream()>>>(logits.data_ptr<float>(),
                                                                                      bias.has_value() ? bias->data_ptr<float>() : nullptr,
                                                                                      idx.data_ptr<int64_t>(), wgt.data_ptr<float>(), T, (int)E, (int)top,
                                                                                      (int)groups, (int)keep, renorm ? 1 : 0);
  return {idx, wgt};
}

}  // namespace llmctl_hybrid
