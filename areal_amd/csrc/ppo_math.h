// Per-token arithmetic of the clipped PPO surrogate and of its derivative,
// shared by the fused logits kernel and the stand-alone loss kernel.
//
// Follows areal/utils/functional/functional.py:516-539.  The derivative is the
// one PyTorch autograd produces for that sequence of ops: torch.max/torch.min
// of two tensors send half of the gradient to each operand where they are
// equal, and torch.clamp passes gradient on the closed interval [lo, hi].
#pragma once
#include "device_utils.h"

namespace aa {

struct Surrogate {
  float loss;      // pg_loss after the optional dual clip and behave weight
  float dloss_dr;  // d(loss) / d(ratio)
  bool clip;       // pg_loss1 < pg_loss2
  bool dual;       // pg_loss3 < max(pg_loss1, pg_loss2)
};

// max/min that return NaN if either side is NaN (torch.max / torch.min do)
__device__ __forceinline__ float nan_max(float a, float b) { return (a != a || b != b) ? (a + b) : fmaxf(a, b); }
__device__ __forceinline__ float nan_min(float a, float b) { return (a != a || b != b) ? (a + b) : fminf(a, b); }

// Proximal log-prob approximated from the behaviour and the current log-prob of a token sampled by policy version
// `ver` (negative for prompt tokens), areal/trainer/ppo/actor.py:604-684: alpha = (v_prox - v_behave) /
// (v_theta - v_behave) clamped to [0, 1], 0 for prompt tokens; method 0 interpolates the log-probs, 1 the
// probabilities, 2 returns the behaviour log-prob.
__device__ __forceinline__ float prox_approx_value(float lo, float ln, int ver, int current_version, int method) {
  const float v_theta = (float)current_version, v_prox = (float)(current_version - 1);
  const float vb = (float)ver;
  const float diff = v_theta - vb, gap = v_prox - vb;
  float alpha = (diff > 0.f && ver >= 0) ? gap / diff : 0.f;
  alpha = fminf(fmaxf(alpha, 0.f), 1.f);
  if (method == 0) return lo + alpha * (ln - lo);
  if (method == 1) return logf((1.f - alpha) * expf(lo) + alpha * expf(ln) + 1e-10f);
  return lo;
}

__device__ __forceinline__ Surrogate surrogate(float r, float adv, float behave_w, const aa_ppo_params& P) {
  // torch.clamp(r, lo, hi) = min(max(r, lo), hi), NaN stays NaN
  float rc = nan_min(nan_max(r, P.clip_lo), P.clip_hi);
  const bool in_range = (r >= P.clip_lo) && (r <= P.clip_hi);
  const float na = -adv;
  const float l1 = na * r;
  const float l2 = na * rc;
  Surrogate o;
  o.clip = l1 < l2;
  float l = nan_max(l1, l2);
  // share of d(max)/d(l1); the rest goes to l2
  const float w1 = (l1 == l2) ? 0.5f : ((l1 < l2) ? 0.f : 1.f);
  const float w2 = (l1 == l2) ? 0.5f : ((l1 > l2) ? 0.f : 1.f);
  float d = na * w1 + (in_range ? na * w2 : 0.f);
  o.dual = false;
  if (P.has_c_clip) {
    const float sg = (adv > 0.f) ? 1.f : ((adv < 0.f) ? -1.f : adv);  // torch.sign, sign(0)=0, sign(NaN)=NaN
    const float l3 = (sg * P.c_clip) * adv;
    o.dual = l3 < l;
    const float wl = (l == l3) ? 0.5f : ((l > l3) ? 0.f : 1.f);  // share of d(min)/d(l)
    l = nan_min(l, l3);
    d *= wl;
  }
  if (P.has_behave_weight) {
    l *= behave_w;
    d *= behave_w;
  }
  o.loss = l;
  o.dloss_dr = d;
  return o;
}

// SAPO (areal/utils/functional/functional.py:607-620): the clip is replaced by a sigmoid gate of the ratio, scaled by
// 4 / tau so that its slope at r = 1 is 1; tau depends on the sign of the advantage (adv > 0, as torch.where(adv > 0)
// selects: NaN and 0 take the negative branch).  d/dr [4 / tau * sigmoid(tau (r - 1))] = 4 s (1 - s).
__device__ __forceinline__ Surrogate sapo_surrogate(float r, float adv, const aa_ppo_params& P) {
  const float tau = adv > 0.f ? P.sapo_tau_pos : P.sapo_tau_neg;
  const float sg = 1.f / (1.f + expf(-tau * (r - 1.f)));
  Surrogate o;
  o.loss = -(sg * (4.f / tau)) * adv;
  o.dloss_dr = -4.f * sg * (1.f - sg) * adv;
  o.clip = false;
  o.dual = false;
  return o;
}

}  // namespace aa
