// Per-token arithmetic of the stage-2/3 operators, shared by the token-parallel kernels (loss.hip)
// and the kernels in which a workgroup owns whole sequences (owned.hip): both evaluate exactly the
// same expressions, so their outputs agree bit for bit wherever the per-row inputs do.
#pragma once
#include "common.h"

namespace axon {

// max/min with PyTorch's gradient convention: ties split the gradient evenly.
struct ValGrad { float v, g; };
__device__ __forceinline__ ValGrad vg_max(ValGrad a, ValGrad b) {
  // selects, not branches: the four outcomes cost a handful of instructions each, a divergent
  // branch per token costs more than all of them
  const bool gt = a.v > b.v, lt = a.v < b.v, eq = a.v == b.v;
  const float v_tie = eq ? a.v : a.v + b.v;          // NaN operand: propagate
  const float g_tie = eq ? 0.5f * (a.g + b.g) : 0.f;
  return ValGrad{gt ? a.v : (lt ? b.v : v_tie), gt ? a.g : (lt ? b.g : g_tie)};
}

// One token of a policy loss.  vw / gw: loss term and its derivative w.r.t. log_prob, already times
// the importance weight where the loss uses one; c1 / c3: indicator metrics (0 or 1); k2: the value
// whose masked sum is the third metric.  The caller multiplies by mask and aggregation scale.
struct TokenTerm { float vw, gw, c1, k2, c3; };

// The ratio of a clipped surrogate loss and what depends on it alone: the exponent clamped to +-20
// (the clamp passes the gradient inclusively), the ratio, the ratio clipped to [lo, hi] and whether it
// lies inside.
struct Ratio { float xc, r, rc; bool pass, rin; };
__device__ __forceinline__ Ratio ratio_of(float x, float lo, float hi) {
  Ratio q;
  q.pass = (x >= -kSafetyBound && x <= kSafetyBound);
  q.xc = clampf(x, -kSafetyBound, kSafetyBound);
  q.r = exp_bounded(q.xc);
  q.rc = clampf(q.r, lo, hi);
  q.rin = (q.r >= lo && q.r <= hi);
  return q;
}

// PPO (0), GSPO (1) and Clip-Cov (6) from the ratio on: max(-A r, -A clip(r)), the dual clip of PPO,
// the metrics.  d = log_prob - old.
template <int KIND>
__device__ __forceinline__ TokenTerm clipped_token(const Ratio& q, float d, float A, float w, float clip_c,
                                                   bool hit) {
  TokenTerm t{0.f, 0.f, 0.f, 0.f, 0.f};
  const ValGrad p1{-A * q.r, -A * q.r};
  const ValGrad p2{-A * q.rc, q.rin ? -A * q.r : 0.f};
  ValGrad c = vg_max(p1, p2);
  if (KIND == 6) {  // Clip-Cov (loss.py:198-280): the selected tokens drop out of the loss
    if (hit) c = ValGrad{c.v * 0.f, 0.f};
    t.c1 = hit ? 1.f : 0.f;
  } else {
    t.c1 = (p2.v > p1.v) ? 1.f : 0.f;
  }
  t.k2 = (KIND == 1) ? -d : -q.xc;  // ppo_kl: raw for GSPO (loss.py:173), clamped otherwise (loss.py:77-79)
  if (KIND == 0) {
    const float pg3 = -A * clip_c;
    t.c3 = (c.v > pg3 && A < 0.f) ? 1.f : 0.f;
    {  // A < 0: torch.min(pg3, c1), pg3 carries no gradient (selects: see vg_max)
      const bool neg = A < 0.f, lt = pg3 < c.v, eq = pg3 == c.v, gt = pg3 > c.v;
      const float v_min = lt ? pg3 : (eq ? c.v : (gt ? c.v : pg3 + c.v));
      const float g_min = lt ? 0.f : (eq ? 0.5f * c.g : (gt ? c.g : 0.f));
      c = ValGrad{neg ? v_min : c.v, neg ? g_min : c.g};
    }
  }
  t.vw = c.v * w;
  t.gw = (q.pass ? c.g : 0.f) * w;
  return t;
}

// KIND 0 PPO, 1 GSPO (sbar = the sequence's mean log-ratio), 2 REINFORCE / GPG, 3 CISPO, 4 clipped
// value loss, 5 KL-Cov, 6 Clip-Cov (hit: the token is among the selected ones).
template <int KIND>
__device__ __forceinline__ TokenTerm policy_token(float lp, float old, float A, float w, float sbar,
                                                  float lo, float hi, float clip_c, bool hit) {
  const float d = lp - old;
  TokenTerm t{0.f, 0.f, 0.f, 0.f, 0.f};
  if (KIND == 2) {  // REINFORCE / GPG (loss.py:471-512): -A * log_prob * w
    t.k2 = -d;
    t.vw = -A * lp * w;
    t.gw = -A * w;
    return t;
  }
  if (KIND == 3) {  // CISPO (loss.py:411-468): -sg(clip(r)) * A * log_prob, IS weights not used
    const float xc = clampf(d, -kSafetyBound, kSafetyBound);
    const float r_ = exp_bounded(xc);
    const float rc = clampf(r_, lo, hi);
    float tm = 1.f;  // optional token-level mask of the unified formulation (clip_c != 0)
    if (clip_c != 0.f && ((A > 0.f && r_ > hi) || (A < 0.f && r_ < lo))) tm = 0.f;
    t.c1 = (r_ > hi || r_ < lo) ? 1.f : 0.f;
    t.k2 = -xc;
    t.vw = -rc * A * lp * tm;
    t.gw = -rc * A * tm;
    return t;
  }
  if (KIND == 4) {  // clipped value loss (loss.py:547-591): lp = vpreds, old = values, A = returns,
                    // lo = cliprange_value; the caller applies the factor 0.5
    const float vp = lp, up = old + lo, dn = old - lo;
    // clip_by_value = maximum(minimum(vp, up), dn) with tensor bounds (loss/utils.py:94-101)
    const float g_min = (vp < up) ? 1.f : ((vp == up) ? 0.5f : 0.f);
    const float y = fminf(vp, up);
    const float g_clip = (y > dn) ? g_min : ((y == dn) ? 0.5f * g_min : 0.f);
    const float vc = fmaxf(y, dn);
    const float e1 = vp - A, e2 = vc - A;
    const ValGrad c = vg_max(ValGrad{e1 * e1, 2.f * e1}, ValGrad{e2 * e2, 2.f * e2 * g_clip});
    t.c1 = (e2 * e2 > e1 * e1) ? 1.f : 0.f;
    t.k2 = vp;
    t.vw = c.v;
    t.gw = c.g;
    return t;
  }
  if (KIND == 5) {  // KL-Cov (loss.py:283-352): -A*ratio, plus clip_c * |log ratio| on the selected tokens
    const bool pass = (d >= -kSafetyBound && d <= kSafetyBound);
    const float xc = clampf(d, -kSafetyBound, kSafetyBound);
    const float r_ = exp_bounded(xc);
    float v = -A * r_, g = -A * r_;
    if (hit) {
      v += clip_c * fabsf(xc);
      g += clip_c * ((xc > 0.f) ? 1.f : ((xc < 0.f) ? -1.f : 0.f));
      t.c1 = 1.f;
    }
    t.k2 = fabsf(xc);
    t.vw = v * w;
    t.gw = (pass ? g : 0.f) * w;
    return t;
  }
  float x;  // exponent before the +-20 clamp
  if (KIND == 0 || KIND == 6) x = d;
  else x = (lp - lp) + sbar;  // log_prob - sg(log_prob) + sg(seq mean)
  return clipped_token<KIND>(ratio_of(x, lo, hi), d, A, w, clip_c, hit);
}

// GSPO where the sequence's ratio is at hand (ratio_of((0 + sbar), lo, hi), once per sequence): the
// same token as policy_token<1>, bit for bit.  log_prob - sg(log_prob) is zero for a finite log_prob and
// NaN otherwise; added to the ratio and its clipped value it leaves them as they are or makes them
// NaN, which is what the exponential of a NaN exponent gives.
__device__ __forceinline__ TokenTerm gspo_token(const Ratio& seq, float lp, float old, float A, float w,
                                                float clip_c) {
  const float z = lp - lp;
  const bool fin = (z == 0.f);
  return clipped_token<1>(Ratio{seq.xc + z, seq.r + z, seq.rc + z, seq.pass && fin, seq.rin && fin}, lp - old, A, w,
                          clip_c, false);
}

// Adds one token to the running sums a[0..4] (loss, three metrics, mask) and returns its gradient.
__device__ __forceinline__ float accumulate_token(const TokenTerm& t, float m, float scale, float (&a)[6]) {
  a[4] += m;
  a[1] += (t.c1 != 0.f) ? m : 0.f;
  a[2] += t.k2 * m;
  a[3] += (t.c3 != 0.f) ? m : 0.f;
  a[0] += t.vw * m * scale;
  return t.gw * m * scale;
}

// ---- sampler / trainer correction (axon/utils/rl/sampler.py:35-103, 181-256, 413-428) ------------
struct CorrCfg {
  int is_mode;   // 0 off, 1 token, 2 sequence
  float is_thr;
  int rs_mode;   // 0 off, 1 token, 2 sequence, 3 geometric
  float rs_lo, rs_hi;
  int has_veto;
  float log_veto;
};

// What a token inherits from its row: the sequence-level weight, keep decision and veto.
struct CorrRow { float w, keep, veto_keep; };

__device__ __forceinline__ CorrRow corr_row(const CorrCfg& c, float rsum, float rcnt, bool vetoed) {
  CorrRow r{0.f, 1.f, 1.f};
  if (c.is_mode == 2) r.w = expf(clampf(rsum, -kSafetyBound, kSafetyBound));
  if (c.rs_mode == 2) r.keep = (rsum >= c.rs_lo && rsum <= c.rs_hi) ? 1.f : 0.f;
  if (c.rs_mode == 3) {
    const float g = rsum / (rcnt + 1e-8f);
    r.keep = (g >= c.rs_lo && g <= c.rs_hi) ? 1.f : 0.f;
  }
  r.veto_keep = (c.has_veto && vetoed) ? 0.f : 1.f;
  return r;
}

// One token: importance weight `w` and new mask `nm`; a[0] sum mask, a[1] sum of unclamped weights,
// a[2] rejected, a[3] tokens under the veto threshold, a[5] sum of clamped weights.
__device__ __forceinline__ void corr_token(const CorrCfg& c, const CorrRow& row, float oldv, float sampv,
                                           float m, float& w_out, float& nm_out, float (&a)[6]) {
  const float lr = oldv - sampv;
  const bool on = (m != 0.f);
  float w = 0.f;
  if (c.is_mode == 1) w = exp_bounded(clampf(lr, -kSafetyBound, kSafetyBound)) * m;
  if (c.is_mode == 2) w = row.w * m;
  a[1] += on ? w * m : 0.f;
  w = (w != w) ? w : fminf(w, c.is_thr);  // clamp(max=thr), NaN propagates
  w_out = w;
  a[5] += on ? w * m : 0.f;
  float keep = 1.f;
  if (c.rs_mode == 1) keep = (lr >= c.rs_lo && lr <= c.rs_hi) ? 1.f : 0.f;
  if (c.rs_mode >= 2) keep = row.keep;
  a[2] += on ? (1.f - keep) * m : 0.f;
  const bool cat = c.has_veto && on && (lr < c.log_veto);
  a[3] += cat ? m : 0.f;
  a[0] += m;
  nm_out = m * keep * row.veto_keep;
}

}  // namespace axon
