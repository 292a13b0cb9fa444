// (c) Elementwise stage-2/3 kernels: sampler correction and the clipped policy
// loss with its gradient.  One read of every input, one write of every output;
// scalar sums leave through per-workgroup partials that the last workgroup adds up.
#include <type_traits>

#include "common.h"
#include "token_math.h"
#include <mutex>

namespace axon {

// acc[0..7] from the eight totals.  norm_slots != 0: the slots in that bit mask (plain masked sums)
// become token-means, acc[5] the factor 1/denominator.
__device__ __forceinline__ void write_acc(float (&tot)[kPartialStride], int norm_slots,
                                          const double* valid, float* acc) {
  if (norm_slots) {  // token-mean over a plain sum: the denominator is known only now
    const float den = fmaxf(valid != nullptr ? (float)valid[0] : tot[4], 1.f);
    for (int k = 0; k < kPartialStride; ++k)
      if ((norm_slots >> k) & 1) tot[k] = tot[k] / den;
    tot[5] = 1.f / den;
  }
  for (int k = 0; k < kPartialStride; ++k) acc[k] = tot[k];
}

template <int MK>
__global__ __launch_bounds__(kBlock) void sampler_correction_kernel(
    const float* __restrict__ oldp, const float* __restrict__ samp, const void* __restrict__ mask,
    const int32_t* __restrict__ cu, int64_t n_rows, int64_t n_slots, int64_t uniform_len,
    int is_mode, float is_thr, int rs_mode, float rs_lo, float rs_hi, int has_veto, float log_veto,
    const float* __restrict__ row_cnt, const float* __restrict__ row_sum,
    const int32_t* __restrict__ row_flag, float* __restrict__ isw, float* __restrict__ new_mask,
    float* partials, float* __restrict__ acc) {
  __shared__ int32_t lds_cu[kLdsRows];
  __shared__ float lds_red[kPartialStride * (kBlock / kWave)];
  const bool need_row = (is_mode == 2) || (rs_mode >= 2) || has_veto;
  const CorrCfg cfg{is_mode, is_thr, rs_mode, rs_lo, rs_hi, has_veto, log_veto};
  const int64_t n_chunks = (n_slots + kChunk - 1) / kChunk;
  float a[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
  for (int64_t chunk = blockIdx.x; chunk < n_chunks; chunk += gridDim.x) {
  const int64_t c0 = chunk * kChunk;
  const int64_t c1 = min(c0 + (int64_t)kChunk, n_slots);
  RowFinder rf;
  if (need_row) {
    __syncthreads();  // the previous chunk's row window is no longer read
    rf.init(cu, n_rows, uniform_len, c0, c1, lds_cu);
  }
#pragma unroll 1
  for (int it = 0; it < kIter; ++it) {
    const int64_t i = c0 + ((int64_t)it * kBlock + threadIdx.x) * kVec;
    if (i >= c1) continue;
    float ov[4], sv[4], mv[4], wv[4], nm[4];
    const bool full = (i + kVec <= n_slots);
    if (full) {
      load4(oldp, i, ov);
      load4(samp, i, sv);
      load_mask4<MK>(mask, i, mv);
    } else {
      for (int j = 0; j < 4; ++j) {
        const bool ok = i + j < n_slots;
        ov[j] = ok ? oldp[i + j] : 0.f;
        sv[j] = ok ? samp[i + j] : 0.f;
        mv[j] = ok ? load_mask1<MK>(mask, i + j) : 0.f;
      }
    }
    int64_t rend = -1;
    CorrRow row{0.f, 1.f, 1.f};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t p = i + j;
      if (p >= n_slots) { wv[j] = 0.f; nm[j] = 0.f; continue; }
      if (need_row && p >= rend) {
        const int r = rf.row(p);
        rend = rf.row_end(r);
        row = corr_row(cfg, row_sum ? row_sum[r] : 0.f, row_cnt ? row_cnt[r] : 0.f,
                       has_veto && row_flag[r] != 0);
      }
      corr_token(cfg, row, ov[j], sv[j], mv[j], wv[j], nm[j], a);
    }
    if (full) {
      if (isw) store4(isw, i, wv);
      store4(new_mask, i, nm);
    } else {
      for (int j = 0; j < 4 && i + j < n_slots; ++j) {
        if (isw) isw[i + j] = wv[j];
        new_mask[i + j] = nm[j];
      }
    }
  }
  }  // chunk
  if (blockIdx.x == 0 && has_veto) {
    for (int64_t r = threadIdx.x; r < n_rows; r += blockDim.x) a[4] += row_flag[r] ? 1.f : 0.f;
  }
  grid_finish<6>(a, lds_red, partials,
                 [&](float (&tot)[kPartialStride]) { write_acc(tot, 0, nullptr, acc); });
}

// Adds the per-workgroup partial sums in a fixed order and writes acc[0..7] (write_acc).
__global__ __launch_bounds__(1024) void reduce_partials_kernel(
    const float* __restrict__ partials, int n_blocks, int norm_slots,
    const double* __restrict__ valid, float* __restrict__ acc) {
  __shared__ float red[16][kPartialStride];
  float t[kPartialStride];
#pragma unroll
  for (int k = 0; k < kPartialStride; ++k) t[k] = 0.f;
  // four blocks per trip: eight independent 16-byte loads in flight per thread; the order in which a
  // thread adds its blocks stays fixed, so the result is reproducible
  for (int b0 = threadIdx.x; b0 < n_blocks; b0 += 4 * blockDim.x) {
    float4 lo4[4], hi4[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int b = b0 + u * (int)blockDim.x;
      const int bc = b < n_blocks ? b : b0;  // a valid block; its values are dropped below
      lo4[u] = *reinterpret_cast<const float4*>(partials + (size_t)bc * kPartialStride);
      hi4[u] = *reinterpret_cast<const float4*>(partials + (size_t)bc * kPartialStride + 4);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (b0 + u * (int)blockDim.x >= n_blocks) continue;
      t[0] += lo4[u].x; t[1] += lo4[u].y; t[2] += lo4[u].z; t[3] += lo4[u].w;
      t[4] += hi4[u].x; t[5] += hi4[u].y; t[6] += hi4[u].z; t[7] += hi4[u].w;
    }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int k = 0; k < kPartialStride; ++k) {
    t[k] = wave_sum(t[k]);
    if (lane == 0) red[wave][k] = t[k];
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float tot[kPartialStride];
    for (int k = 0; k < kPartialStride; ++k) {
      float s = 0.f;
      for (int w = 0; w < (int)(blockDim.x >> 6); ++w) s += red[w][k];
      tot[k] = s;
    }
    write_acc(tot, norm_slots, valid, acc);
  }
}

__global__ __launch_bounds__(1024) void loss_row_scale_kernel(
    const float* __restrict__ row_cnt, const float* __restrict__ row_sum, int64_t n_rows,
    int64_t row_len, int token_reduce, int batch_reduce, const double* __restrict__ prtc,
    const double* __restrict__ npt, const double* __restrict__ nps,
    const double* __restrict__ valid, float* __restrict__ row_scale,
    float* __restrict__ row_mean) {
  __shared__ float red[2 * 16];
  __shared__ float tot[2];
  float t[2] = {0.f, 0.f};
#pragma unroll 8
  for (int64_t r = threadIdx.x; r < n_rows; r += blockDim.x) {
    const float c = row_cnt[r];
    t[0] += c;
    t[1] += (c > 0.f) ? 1.f : 0.f;
  }
  t[0] = wave_sum(t[0]);
  t[1] = wave_sum(t[1]);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) { red[wave * 2] = t[0]; red[wave * 2 + 1] = t[1]; }
  __syncthreads();
  if (threadIdx.x == 0) {
    float s0 = 0.f, s1 = 0.f;
    for (int w = 0; w < (int)(blockDim.x >> 6); ++w) { s0 += red[w * 2]; s1 += red[w * 2 + 1]; }
    tot[0] = s0; tot[1] = s1;
  }
  __syncthreads();
  float bden;
  if (valid != nullptr) bden = fmaxf((float)valid[0], 1.f);
  else if (batch_reduce == 0) bden = fmaxf(tot[0], 1.f);
  else bden = fmaxf(tot[1], 1.f);
  // every workgroup has formed the same totals in the same order; each writes its own slice of the rows
  const int64_t per = (n_rows + gridDim.x - 1) / gridDim.x;
  const int64_t r_begin = (int64_t)blockIdx.x * per, r_end = min(r_begin + per, n_rows);
#pragma unroll 8
  for (int64_t r = r_begin + threadIdx.x; r < r_end; r += blockDim.x) {
    const float c = row_cnt[r];
    float td = 1.f;
    if (token_reduce == 1) td = fmaxf(prtc ? (float)prtc[r] : c, 1.f);
    if (token_reduce == 2) td = (float)row_len;
    if (token_reduce == 3) td = fmaxf((float)npt[r], 1.f);
    if (batch_reduce == 2) td *= fmaxf((float)nps[r], 1.f);
    row_scale[r] = 1.f / (td * bden);
    if (row_mean) row_mean[r] = (row_sum ? row_sum[r] : 0.f) / fmaxf(c, 1.f);
  }
}

template <int MK, int KIND>
__global__ __launch_bounds__(kBlock) void policy_loss_kernel(
    const float* __restrict__ logp, const float* __restrict__ oldp, const float* __restrict__ adv,
    const void* __restrict__ mask, const float* __restrict__ isw, const int32_t* __restrict__ cu,
    int64_t n_rows, int64_t n_slots, int64_t uniform_len, const float* __restrict__ row_scale,
    const float* __restrict__ row_mean, float uniform_scale, float lo, float hi, float clip_c,
    const uint32_t* __restrict__ sel_keys, const SelectState* __restrict__ sel_state,
    float* __restrict__ grad, float* partials, int norm_slots, const double* __restrict__ valid,
    float* __restrict__ acc) {
  __shared__ int32_t lds_cu[kLdsRows];
  __shared__ float lds_red[kPartialStride * (kBlock / kWave)];
  const bool need_row = (row_scale != nullptr) || (KIND == 1);
  SelectState sel{};
  if (KIND >= 5) sel = *sel_state;
  const int64_t n_chunks = (n_slots + kChunk - 1) / kChunk;
  float a[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
  for (int64_t chunk = blockIdx.x; chunk < n_chunks; chunk += gridDim.x) {
  const int64_t c0 = chunk * kChunk;
  const int64_t c1 = min(c0 + (int64_t)kChunk, n_slots);
  RowFinder rf;
  // the row search of a chunk is a chain of dependent loads: where a whole chunk is streamed it runs
  // after the chunk's first loads have been issued, under their latency
  auto find_rows = [&]() {
    if (need_row) {
      __syncthreads();  // the previous chunk's row window is no longer read
      rf.init(cu, n_rows, uniform_len, c0, c1, lds_cu);
    }
  };
  // the per-token arithmetic on one vector of four slots
  // (full_c: a compile-time true where every slot of the vector exists, so that the common path carries
  // no test per token)
  auto process = [&](int64_t i, auto full_c, const float (&lv)[4], const float (&ov)[4], const float (&av)[4],
                     const float (&mv)[4], const float (&wv)[4]) {
    constexpr bool full = decltype(full_c)::value;
    float gv[4];
    int64_t rend = -1;
    float scale = uniform_scale, sbar = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t p = i + j;
      if (!full && p >= n_slots) { gv[j] = 0.f; continue; }
      if (need_row && p >= rend) {
        const int r = rf.row(p);
        rend = rf.row_end(r);
        if (row_scale) scale = row_scale[r];
        if (KIND == 1) sbar = row_mean[r];
      }
      const float m = mv[j];
      const bool hit = (KIND >= 5) ? select_hit(sel, sel_keys[p], p) : false;
      const TokenTerm t = policy_token<KIND>(lv[j], ov[j], av[j], wv[j], sbar, lo, hi, clip_c, hit);
      gv[j] = accumulate_token(t, m, scale, a);
    }
    if (full) store4(grad, i, gv);
    else
      for (int j = 0; j < 4 && i + j < n_slots; ++j) grad[i + j] = gv[j];
  };
  if (c1 - c0 == kChunk) {
    // whole chunk: the loads of kB steps are issued before the first use, so that each thread has
    // kB x (4 or 5) 16-byte requests in flight (+3 % over one step at a time at 2^26 tokens)
    // (the sequence-level kernel keeps more state per token: two steps at a time there)
    constexpr int kB = (KIND == 1) ? 2 : kIter;
#pragma unroll
    for (int b0 = 0; b0 < kIter; b0 += kB) {
      float lv[kB][4], ov[kB][4], av[kB][4], mv[kB][4], wv[kB][4];
#pragma unroll
      for (int it = 0; it < kB; ++it) {
        const int64_t i = c0 + ((int64_t)(b0 + it) * kBlock + threadIdx.x) * kVec;
        load4(logp, i, lv[it]);
        load4(oldp, i, ov[it]);
        load4(adv, i, av[it]);
        load_mask4<MK>(mask, i, mv[it]);
        if (isw) load4(isw, i, wv[it]);
        else wv[it][0] = wv[it][1] = wv[it][2] = wv[it][3] = 1.f;
      }
      if (b0 == 0) find_rows();
#pragma unroll
      for (int it = 0; it < kB; ++it)
        process(c0 + ((int64_t)(b0 + it) * kBlock + threadIdx.x) * kVec, std::true_type{}, lv[it], ov[it], av[it],
                mv[it], wv[it]);
    }
  } else {
    find_rows();
#pragma unroll 1
    for (int it = 0; it < kIter; ++it) {
      const int64_t i = c0 + ((int64_t)it * kBlock + threadIdx.x) * kVec;
      if (i >= c1) continue;
      float lv[4], ov[4], av[4], mv[4], wv[4] = {1.f, 1.f, 1.f, 1.f};
      const bool full = (i + kVec <= n_slots);
      if (full) {
        load4(logp, i, lv);
        load4(oldp, i, ov);
        load4(adv, i, av);
        load_mask4<MK>(mask, i, mv);
        if (isw) load4(isw, i, wv);
      } else {
        for (int j = 0; j < 4; ++j) {
          const bool ok = i + j < n_slots;
          lv[j] = ok ? logp[i + j] : 0.f;
          ov[j] = ok ? oldp[i + j] : 0.f;
          av[j] = ok ? adv[i + j] : 0.f;
          mv[j] = ok ? load_mask1<MK>(mask, i + j) : 0.f;
          wv[j] = (ok && isw) ? isw[i + j] : 1.f;
        }
      }
      process(i, std::false_type{}, lv, ov, av, mv, wv);
    }
  }
  }  // chunk
  if (blockIdx.x == 0 && threadIdx.x == 0) a[5] = 1.f;  // gradient factor unless post-normalised
  grid_finish<6>(a, lds_red, partials,
                 [&](float (&tot)[kPartialStride]) { write_acc(tot, norm_slots, valid, acc); });
}

// KL penalty estimators of axon/utils/rl/kl.py:154-245 with PyTorch's gradient conventions.
//   type 1: k1 = lp - ref   2: abs   3: k2 = 0.5 (lp - ref)^2   4: k3 = low-variance (clamped)
//   plus != 0 ("k1+", "k3+"): forward value of the type, gradient of k2 (straight-through, :184-190)
__device__ __forceinline__ ValGrad kl_term(float lp, float ref, int type, int plus) {
  const float d = lp - ref;
  ValGrad r{0.f, 0.f};
  if (type == 1) {
    r = ValGrad{d, 1.f};
  } else if (type == 2) {
    r = ValGrad{fabsf(d), (d > 0.f) ? 1.f : ((d < 0.f) ? -1.f : 0.f)};
  } else if (type == 3) {
    r = ValGrad{0.5f * d * d, d};
  } else if (type == 4) {
    const float k = ref - lp;
    const bool in1 = (k >= -kSafetyBound && k <= kSafetyBound);
    const float kc = clampf(k, -kSafetyBound, kSafetyBound);
    const float ratio = expf(kc);
    const float v = ratio - kc - 1.f;
    const bool in2 = (v >= -10.f && v <= 10.f);
    r = ValGrad{clampf(v, -10.f, 10.f), (in1 && in2) ? (1.f - ratio) : 0.f};
  }
  if (plus && type != 3) r.g = d;
  return r;
}

__global__ __launch_bounds__(kBlock) void kl_penalty_kernel(const float* __restrict__ lp,
                                                            const float* __restrict__ ref, int64_t n,
                                                            int type, int plus, float* __restrict__ out,
                                                            float* __restrict__ grad) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const ValGrad r = kl_term(lp[i], ref[i], type, plus);
    out[i] = r.v;
    grad[i] = r.g;
  }
}

// Side terms of the actor loss, aggregated exactly like the policy-gradient term
// (axon/models/fsdp_models.py:247-273): entropy bonus and KL penalty against a reference
// policy.  partial slots: [0] sum entropy*w  [1] sum kld*w  [2] sum entropy*mask  [4] sum mask,
// w = mask * scale.  Outputs agg_w[t] = w (the gradient of slot 0 w.r.t. entropy) and
// grad_kl[t] = w * d kld / d log_prob.
// KL penalty inside the reward (axon/utils/rl/kl.py:276-322): kld = kl_penalty(old, ref) * mask,
// rewards = scores - beta * kld, and per row sum mask -> row_vals[0][r], sum kld -> row_vals[1][r].
template <int MK>
__global__ __launch_bounds__(kBlock) void kl_reward_kernel(
    const float* __restrict__ scores, const float* __restrict__ oldp, const float* __restrict__ refp,
    const void* __restrict__ mask, const int32_t* __restrict__ cu, int64_t n_rows, int64_t n_slots,
    int64_t uniform_len, int kl_type, float beta, float* __restrict__ rewards, float* row_vals) {
  __shared__ int32_t lds_cu[kLdsRows];
  const int64_t n_chunks = (n_slots + kChunk - 1) / kChunk;
#pragma unroll 1
  for (int64_t chunk = blockIdx.x; chunk < n_chunks; chunk += gridDim.x) {
    const int64_t c0 = chunk * kChunk;
    const int64_t c1 = min(c0 + (int64_t)kChunk, n_slots);
    __syncthreads();
    RowFinder rf;
    rf.init(cu, n_rows, uniform_len, c0, c1, lds_cu);
#pragma unroll 1
    for (int it = 0; it < kIter; ++it) {
      const int64_t i = c0 + ((int64_t)it * kBlock + threadIdx.x) * kVec;
      RowSeg<2> s;
      s.row = -1;
      s.v[0] = s.v[1] = 0.f;
      if (i < c1) {
        float sv[4], ov[4], rv[4], mv[4], out[4];
        const bool full = (i + kVec <= n_slots);
        if (full) {
          load4(scores, i, sv);
          load4(oldp, i, ov);
          load4(refp, i, rv);
          load_mask4<MK>(mask, i, mv);
        } else {
          for (int j = 0; j < 4; ++j) {
            const bool ok = i + j < n_slots;
            sv[j] = ok ? scores[i + j] : 0.f;
            ov[j] = ok ? oldp[i + j] : 0.f;
            rv[j] = ok ? refp[i + j] : 0.f;
            mv[j] = ok ? load_mask1<MK>(mask, i + j) : 0.f;
          }
        }
        int r = rf.row(i);
        int64_t rend = rf.row_end(r);
        s.row = r;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int64_t p = i + j;
          if (p >= n_slots) { out[j] = 0.f; continue; }
          if (p >= rend) {
            row_seg_flush(s, row_vals, n_rows);
            r = rf.row(p);
            rend = rf.row_end(r);
            s.row = r;
            s.v[0] = s.v[1] = 0.f;
          }
          const float kld = kl_term(ov[j], rv[j], kl_type, 0).v * mv[j];
          out[j] = sv[j] - beta * kld;
          s.v[0] += mv[j];
          s.v[1] += kld;
        }
        if (full) store4(rewards, i, out);
        else
          for (int j = 0; j < 4 && i + j < n_slots; ++j) rewards[i + j] = out[j];
      }
      row_seg_wave_reduce_flush(s, row_vals, n_rows);
    }
  }
}

template <int MK>
__global__ __launch_bounds__(kBlock) void side_terms_kernel(
    const float* __restrict__ entropy, const float* __restrict__ logp, const float* __restrict__ ref,
    const void* __restrict__ mask, const int32_t* __restrict__ cu, int64_t n_rows, int64_t n_slots,
    int64_t uniform_len, const float* __restrict__ row_scale, float uniform_scale, int kl_type,
    int kl_plus, float* __restrict__ agg_w, float* __restrict__ grad_kl, float* partials,
    int norm_slots, const double* __restrict__ valid, float* __restrict__ acc) {
  __shared__ int32_t lds_cu[kLdsRows];
  __shared__ float lds_red[kPartialStride * (kBlock / kWave)];
  const bool need_row = (row_scale != nullptr);
  const int64_t n_chunks = (n_slots + kChunk - 1) / kChunk;
  float a[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll 1
  for (int64_t chunk = blockIdx.x; chunk < n_chunks; chunk += gridDim.x) {
    const int64_t c0 = chunk * kChunk;
    const int64_t c1 = min(c0 + (int64_t)kChunk, n_slots);
    RowFinder rf;
    if (need_row) {
      __syncthreads();
      rf.init(cu, n_rows, uniform_len, c0, c1, lds_cu);
    }
#pragma unroll 1
    for (int it = 0; it < kIter; ++it) {
      const int64_t i = c0 + ((int64_t)it * kBlock + threadIdx.x) * kVec;
      if (i >= c1) continue;
      float ev[4] = {0.f, 0.f, 0.f, 0.f}, lv[4] = {0.f, 0.f, 0.f, 0.f}, rv[4] = {0.f, 0.f, 0.f, 0.f};
      float mv[4], wv[4], gv[4];
      const bool full = (i + kVec <= n_slots);
      if (full) {
        if (entropy) load4(entropy, i, ev);
        if (kl_type) { load4(logp, i, lv); load4(ref, i, rv); }
        load_mask4<MK>(mask, i, mv);
      } else {
        for (int j = 0; j < 4; ++j) {
          const bool ok = i + j < n_slots;
          ev[j] = (ok && entropy) ? entropy[i + j] : 0.f;
          lv[j] = (ok && kl_type) ? logp[i + j] : 0.f;
          rv[j] = (ok && kl_type) ? ref[i + j] : 0.f;
          mv[j] = ok ? load_mask1<MK>(mask, i + j) : 0.f;
        }
      }
      int64_t rend = -1;
      float scale = uniform_scale;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int64_t p = i + j;
        if (p >= n_slots) { wv[j] = 0.f; gv[j] = 0.f; continue; }
        if (need_row && p >= rend) {
          const int r = rf.row(p);
          rend = rf.row_end(r);
          scale = row_scale[r];
        }
        const float m = mv[j];
        const float w = m * scale;
        wv[j] = w;
        a[4] += m;
        if (entropy) {
          a[0] += ev[j] * w;
          a[2] += ev[j] * m;
        }
        float g = 0.f;
        if (kl_type) {
          const ValGrad k = kl_term(lv[j], rv[j], kl_type, kl_plus);
          a[1] += k.v * w;
          g = k.g * w;
        }
        gv[j] = g;
      }
      if (full) {
        if (agg_w) store4(agg_w, i, wv);
        if (grad_kl) store4(grad_kl, i, gv);
      } else {
        for (int j = 0; j < 4 && i + j < n_slots; ++j) {
          if (agg_w) agg_w[i + j] = wv[j];
          if (grad_kl) grad_kl[i + j] = gv[j];
        }
      }
    }
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) a[5] = 1.f;
  grid_finish<6>(a, lds_red, partials,
                 [&](float (&tot)[kPartialStride]) { write_acc(tot, norm_slots, valid, acc); });
}

// ---- GMPO (geo_mean_loss_fn, axon/trainer/algos/loss/loss.py:355-408) ------------------------------
// Per token: nak_min = sgn(A) * min(sgn(A) * nak, sgn(A) * clamp(nak, -lo, hi)), nak = logp - old.
// Per row: ratio = exp(sum(nak_min * m) / (cnt + 1e-8)), adv = sum(A * m) / (cnt + 1e-8),
// w = exp(sum(log(is_w + 1e-10) * m) / (cnt + 1e-8)); loss = mean over rows with tokens of -adv*ratio*w.
__device__ __forceinline__ ValGrad gmpo_term(float nak, float A, float lo, float hi) {
  const float sg = (A > 0.f) ? 1.f : ((A < 0.f) ? -1.f : 0.f);
  const float c = clampf(nak, -lo, hi);
  const float dclamp = (nak >= -lo && nak <= hi) ? 1.f : 0.f;
  const float a1 = sg * nak, a2 = sg * c;
  float v, g;
  if (a1 < a2) { v = a1; g = sg; }
  else if (a1 > a2) { v = a2; g = sg * dclamp; }
  else { v = a1; g = 0.5f * (sg + sg * dclamp); }  // torch.min splits the gradient on ties
  return ValGrad{sg * v, sg * g};
}

constexpr int kGmpoRowVals = 4;  // cnt, sum nak_min*m, sum A*m, sum log(is_w + 1e-10)*m

// PASS 0: row sums and metric partials.  PASS 1: gradient from the per-row coefficients.
template <int MK, int PASS>
__global__ __launch_bounds__(kBlock) void gmpo_kernel(
    const float* __restrict__ logp, const float* __restrict__ oldp, const float* __restrict__ adv,
    const void* __restrict__ mask, const float* __restrict__ isw, const int32_t* __restrict__ cu,
    int64_t n_rows, int64_t n_slots, int64_t uniform_len, float lo, float hi, float* row_vals,
    const float* __restrict__ row_coef, float* __restrict__ grad, float* partials) {
  __shared__ int32_t lds_cu[kLdsRows];
  __shared__ float lds_red[5 * (kBlock / kWave)];
  float a[5] = {0.f, 0.f, 0.f, 0.f, 0.f};
  const int64_t n_chunks = (n_slots + kChunk - 1) / kChunk;
#pragma unroll 1
  for (int64_t chunk = blockIdx.x; chunk < n_chunks; chunk += gridDim.x) {
    const int64_t c0 = chunk * kChunk;
    const int64_t c1 = min(c0 + (int64_t)kChunk, n_slots);
    __syncthreads();
    RowFinder rf;
    rf.init(cu, n_rows, uniform_len, c0, c1, lds_cu);
#pragma unroll 1
    for (int it = 0; it < kIter; ++it) {
      const int64_t i = c0 + ((int64_t)it * kBlock + threadIdx.x) * kVec;
      RowSeg<kGmpoRowVals> s;
      s.row = -1;
#pragma unroll
      for (int k = 0; k < kGmpoRowVals; ++k) s.v[k] = 0.f;
      if (i < c1) {
        float lv[4], ov[4], av[4], mv[4], wv[4] = {1.f, 1.f, 1.f, 1.f}, gv[4];
        const bool full = (i + kVec <= n_slots);
        if (full) {
          load4(logp, i, lv);
          load4(oldp, i, ov);
          load4(adv, i, av);
          load_mask4<MK>(mask, i, mv);
          if (PASS == 0 && isw) load4(isw, i, wv);
        } else {
          for (int j = 0; j < 4; ++j) {
            const bool ok = i + j < n_slots;
            lv[j] = ok ? logp[i + j] : 0.f;
            ov[j] = ok ? oldp[i + j] : 0.f;
            av[j] = ok ? adv[i + j] : 0.f;
            mv[j] = ok ? load_mask1<MK>(mask, i + j) : 0.f;
            wv[j] = (ok && PASS == 0 && isw) ? isw[i + j] : 1.f;
          }
        }
        int r = rf.row(i);
        int64_t rend = rf.row_end(r);
        s.row = r;
        float coef = (PASS == 1) ? row_coef[r] : 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int64_t p = i + j;
          if (p >= n_slots) { gv[j] = 0.f; continue; }
          if (p >= rend) {
            if (PASS == 0) row_seg_flush(s, row_vals, n_rows);
            r = rf.row(p);
            rend = rf.row_end(r);
            s.row = r;
#pragma unroll
            for (int k = 0; k < kGmpoRowVals; ++k) s.v[k] = 0.f;
            if (PASS == 1) coef = row_coef[r];
          }
          const float m = mv[j], A = av[j];
          const float nak = lv[j] - ov[j];
          const ValGrad t = gmpo_term(nak, A, lo, hi);
          if (PASS == 0) {
            const bool clipped = (nak != clampf(nak, -lo, hi));
            a[1] += (clipped && A > 0.f) ? m : 0.f;
            a[2] += -nak * m;
            a[3] += (clipped && A < 0.f) ? m : 0.f;
            a[4] += m;
            s.v[0] += m;
            s.v[1] += t.v * m;
            s.v[2] += A * m;
            if (isw) s.v[3] += logf(wv[j] + 1e-10f) * m;
          } else {
            gv[j] = coef * m * t.g;
          }
        }
        if (PASS == 1) {
          if (full) store4(grad, i, gv);
          else
            for (int j = 0; j < 4 && i + j < n_slots; ++j) grad[i + j] = gv[j];
        }
      }
      if (PASS == 0) row_seg_wave_reduce_flush(s, row_vals, n_rows);
    }
  }
  if (PASS == 0) store_block_partials<5>(a, lds_red, partials);
}

// One workgroup: per-row loss terms -> acc[0] (mean over rows with tokens; over all rows when no row
// has any) and row_coef[r] = d loss / d (sum nak_min*m)_r.
__global__ __launch_bounds__(1024) void gmpo_rows_kernel(const float* __restrict__ row_vals, int64_t n_rows,
                                                         int has_isw, float* __restrict__ row_coef,
                                                         float* __restrict__ acc) {
  __shared__ double red[16][3];
  __shared__ double tot[3];
  const float* cnt_a = row_vals;
  const float* s1_a = row_vals + n_rows;
  const float* s2_a = row_vals + 2 * n_rows;
  const float* s3_a = row_vals + 3 * n_rows;
  double t[3] = {0.0, 0.0, 0.0};  // valid rows, sum of valid rows' losses, sum of all rows' losses
  for (int64_t r = threadIdx.x; r < n_rows; r += blockDim.x) {
    const float cnt = cnt_a[r], den = cnt + 1e-8f;
    const float ratio = expf(s1_a[r] / den);
    const float w = has_isw ? expf(s3_a[r] / den) : 1.f;
    const float l = -(s2_a[r] / den) * ratio * w;
    if (cnt > 0.f) { t[0] += 1.0; t[1] += (double)l; }
    t[2] += (double)l;
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int k = 0; k < 3; ++k) {
    double v = t[k];
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, kWave);
    if (lane == 0) red[wave][k] = v;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int k = 0; k < 3; ++k) {
      double v = 0.0;
      for (int w = 0; w < (int)(blockDim.x >> 6); ++w) v += red[w][k];
      tot[k] = v;
    }
    acc[0] = (float)(tot[0] > 0.0 ? tot[1] / tot[0] : tot[2] / (double)n_rows);
  }
  __syncthreads();
  const bool any_valid = tot[0] > 0.0;
  const float inv_n = (float)(1.0 / (any_valid ? tot[0] : (double)n_rows));
  for (int64_t r = threadIdx.x; r < n_rows; r += blockDim.x) {
    const float cnt = cnt_a[r], den = cnt + 1e-8f;
    const float ratio = expf(s1_a[r] / den);
    const float w = has_isw ? expf(s3_a[r] / den) : 1.f;
    const float l = -(s2_a[r] / den) * ratio * w;
    row_coef[r] = (any_valid && !(cnt > 0.f)) ? 0.f : l * inv_n / den;
  }
}

}  // namespace axon

using namespace axon;

extern "C" int64_t axon_reduce_partials_bytes(int64_t n_slots) {
  if (n_slots < 0) return AXON_ERR_ARG;
  return kPartialsBytes;  // rows for the largest grid plus the ticket counter
}

static int check_rows2(const int32_t* cu, int64_t n_rows, int64_t n_slots, int64_t uniform_len,
                       bool need_row) {
  if (n_rows < 0 || n_slots < 0 || uniform_len < 0) return AXON_ERR_ARG;
  if (n_rows >= (int64_t)INT32_MAX || n_slots >= (int64_t)INT32_MAX) return AXON_ERR_SHAPE;
  if (need_row && uniform_len == 0 && cu == nullptr && n_slots > 0) return AXON_ERR_ARG;
  if (uniform_len > 0 && n_rows * uniform_len != n_slots) return AXON_ERR_SHAPE;
  // tokens that belong to no row: the row lookup would read in front of cu_seqlens
  if (need_row && uniform_len == 0 && n_rows == 0 && n_slots > 0) return AXON_ERR_SHAPE;
  return AXON_OK;
}

extern "C" int axon_sampler_correction(
    const float* oldp, const float* samp, const void* mask, int mask_kind, const int32_t* cu,
    int64_t n_rows, int64_t n_slots, int64_t uniform_len, int is_mode, float is_thr, int rs_mode,
    float rs_lo, float rs_hi, int has_veto, float log_veto, const float* row_cnt,
    const float* row_sum, const int32_t* row_flag, float* isw, float* new_mask, float* acc,
    float* partials, void* stream) {
  const bool need_row = (is_mode == 2) || (rs_mode >= 2) || has_veto;
  int rc = check_rows2(cu, n_rows, n_slots, uniform_len, need_row);
  if (rc != AXON_OK) return rc;
  if (n_slots == 0) return AXON_OK;
  if (!oldp || !samp || !mask || !new_mask || !acc || !partials) return AXON_ERR_ARG;
  if (is_mode < 0 || is_mode > 2 || rs_mode < 0 || rs_mode > 3) return AXON_ERR_ARG;
  if (is_mode != 0 && isw == nullptr) return AXON_ERR_ARG;
  if ((is_mode == 2 || rs_mode >= 2) && (!row_sum || !row_cnt)) return AXON_ERR_ARG;
  if (has_veto && !row_flag) return AXON_ERR_ARG;
  if (mask_kind != AXON_MASK_F32 && mask_kind != AXON_MASK_I64) return AXON_ERR_ARG;
  const dim3 g(stream_grid(n_slots)), blk(kBlock);
  if (mask_kind == AXON_MASK_F32)
    hipLaunchKernelGGL(sampler_correction_kernel<AXON_MASK_F32>, g, blk, 0, (hipStream_t)stream,
                       oldp, samp, mask, cu, n_rows, n_slots, uniform_len, is_mode, is_thr, rs_mode,
                       rs_lo, rs_hi, has_veto, log_veto, row_cnt, row_sum, row_flag, isw, new_mask,
                       partials, acc);
  else
    hipLaunchKernelGGL(sampler_correction_kernel<AXON_MASK_I64>, g, blk, 0, (hipStream_t)stream,
                       oldp, samp, mask, cu, n_rows, n_slots, uniform_len, is_mode, is_thr, rs_mode,
                       rs_lo, rs_hi, has_veto, log_veto, row_cnt, row_sum, row_flag, isw, new_mask,
                       partials, acc);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

extern "C" int axon_loss_row_scale(const float* row_cnt, const float* row_sum, int64_t n_rows,
                                   int64_t row_len, int token_reduce, int batch_reduce,
                                   const double* prtc, const double* npt, const double* nps,
                                   const double* valid, float* row_scale, float* row_mean,
                                   void* stream) {
  if (n_rows < 0) return AXON_ERR_ARG;
  if (n_rows == 0) return AXON_OK;
  if (!row_cnt || !row_scale) return AXON_ERR_ARG;
  if (token_reduce < 0 || token_reduce > 3 || batch_reduce < 0 || batch_reduce > 2)
    return AXON_ERR_ARG;
  if (token_reduce == 3 && !npt) return AXON_ERR_ARG;
  if (token_reduce == 2 && row_len <= 0) return AXON_ERR_ARG;
  if (batch_reduce == 2 && (!nps || !valid)) return AXON_ERR_ARG;
  // the pass over the counts is repeated by every workgroup (cheap: 4 bytes per row from L2); the per-row
  // pass is shared out
  const unsigned blocks = (unsigned)((n_rows + 2047) / 2048 < 64 ? (n_rows + 2047) / 2048 : 64);
  hipLaunchKernelGGL(loss_row_scale_kernel, dim3(blocks), dim3(1024), 0, (hipStream_t)stream, row_cnt,
                     row_sum, n_rows, row_len, token_reduce, batch_reduce, prtc, npt, nps, valid,
                     row_scale, row_mean);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

static int policy_loss_impl(int kind, const float* logp, const float* oldp, const float* adv,
                            const void* mask, int mask_kind, const float* isw, const int32_t* cu,
                            int64_t n_rows, int64_t n_slots, int64_t uniform_len,
                            const float* row_scale, const float* row_mean, float uniform_scale,
                            int post_normalize, const double* valid, float ratio_lo,
                            float ratio_hi, float clip_c, float* grad, float* acc, float* partials,
                            void* stream) {
  const bool need_row = (row_scale != nullptr) || (kind == 1);
  int rc = check_rows2(cu, n_rows, n_slots, uniform_len, need_row);
  if (rc != AXON_OK) return rc;
  if (n_slots == 0) return AXON_OK;
  if (kind < 0 || kind > 4) return AXON_ERR_ARG;
  if (!logp || !oldp || !adv || !mask || !grad || !acc || !partials) return AXON_ERR_ARG;
  if (post_normalize && (row_scale != nullptr || kind == 1)) return AXON_ERR_ARG;
  if (kind == 1 && !row_mean) return AXON_ERR_ARG;
  if (mask_kind != AXON_MASK_F32 && mask_kind != AXON_MASK_I64) return AXON_ERR_ARG;
  const dim3 g(stream_grid(n_slots)), blk(kBlock);
  const hipStream_t st = (hipStream_t)stream;
#define AXON_LAUNCH_PL(MK, KD)                                                                   \
  hipLaunchKernelGGL((policy_loss_kernel<MK, KD>), g, blk, 0, st, logp, oldp, adv, mask, isw, cu, \
                     n_rows, n_slots, uniform_len, row_scale, row_mean, uniform_scale, ratio_lo, \
                     ratio_hi, clip_c, (const uint32_t*)nullptr, (const SelectState*)nullptr, grad,  \
                     partials, post_normalize ? 1 : 0, valid, acc)
  if (mask_kind == AXON_MASK_F32) {
    if (kind == 0) AXON_LAUNCH_PL(AXON_MASK_F32, 0);
    else if (kind == 1) AXON_LAUNCH_PL(AXON_MASK_F32, 1);
    else if (kind == 2) AXON_LAUNCH_PL(AXON_MASK_F32, 2);
    else if (kind == 3) AXON_LAUNCH_PL(AXON_MASK_F32, 3);
    else AXON_LAUNCH_PL(AXON_MASK_F32, 4);
  } else {
    if (kind == 0) AXON_LAUNCH_PL(AXON_MASK_I64, 0);
    else if (kind == 1) AXON_LAUNCH_PL(AXON_MASK_I64, 1);
    else if (kind == 2) AXON_LAUNCH_PL(AXON_MASK_I64, 2);
    else if (kind == 3) AXON_LAUNCH_PL(AXON_MASK_I64, 3);
    else AXON_LAUNCH_PL(AXON_MASK_I64, 4);
  }
#undef AXON_LAUNCH_PL
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

extern "C" int axon_policy_loss(int kind, const float* logp, const float* oldp, const float* adv,
                                const void* mask, int mask_kind, const float* isw,
                                const int32_t* cu, int64_t n_rows, int64_t n_slots,
                                int64_t uniform_len, const float* row_scale, const float* row_mean,
                                float uniform_scale, int post_normalize, const double* valid,
                                float ratio_lo, float ratio_hi, float clip_c, float* grad,
                                float* acc, float* partials, void* stream) {
  return policy_loss_impl(kind, logp, oldp, adv, mask, mask_kind, isw, cu, n_rows, n_slots,
                          uniform_len, row_scale, row_mean, uniform_scale, post_normalize, valid,
                          ratio_lo, ratio_hi, clip_c, grad, acc, partials, stream);
}

// ---- the entry point that allocates nothing ---------------------------------------------------
// Same kernels as axon_policy_loss; the per-workgroup partial sums and the ticket counter live in a
// fixed array in device memory instead of a caller-provided workspace (522 KB; every
// GPU the library runs on holds its own copy until the process ends).  In host code the array's
// name is only a handle: its device address is looked up once per device (with that device
// current) and kept, and only that address is handed to kernels.
namespace {
constexpr int64_t kNoAllocMaxSlots = (int64_t)1 << 24;  // the stated capacity of the entry point
constexpr int kNoAllocMaxDevices = 64;
}  // namespace
static __device__ __align__(256) float scratch[kPartialsBytes / 4];
static float* g_scratch_addr[kNoAllocMaxDevices];  // per device; null until the first call there
static std::mutex g_scratch_mutex;

static int scratch_of_current_device(float** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess) return AXON_ERR_LAUNCH;
  if (dev < 0 || dev >= kNoAllocMaxDevices) return AXON_ERR_DEVICE;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_addr[dev] == nullptr) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr)
      return AXON_ERR_LAUNCH;
    g_scratch_addr[dev] = static_cast<float*>(p);
  }
  *out = g_scratch_addr[dev];
  return AXON_OK;
}

extern "C" int axon_policy_loss_noalloc(int kind, const float* logp, const float* oldp,
                                        const float* adv, const void* mask, int mask_kind,
                                        const float* isw, const int32_t* cu, int64_t n_rows,
                                        int64_t n_slots, int64_t uniform_len,
                                        const float* row_scale, const float* row_mean,
                                        float uniform_scale, int post_normalize,
                                        const double* valid, float ratio_lo, float ratio_hi,
                                        float clip_c, float* grad, float* acc, void* stream) {
  if (n_slots > kNoAllocMaxSlots) return AXON_ERR_TOO_LARGE;
  float* partials = nullptr;
  const int rc = scratch_of_current_device(&partials);
  if (rc != AXON_OK) return rc;
  // every workgroup overwrites its whole row of the array and the reduction reads only the rows of
  // this launch; the ticket counter starts at zero (static storage) and the kernel's last workgroup
  // puts it back to zero, so nothing left by an earlier call is read and nothing is cleared here
  return policy_loss_impl(kind, logp, oldp, adv, mask, mask_kind, isw, cu, n_rows, n_slots,
                          uniform_len, row_scale, row_mean, uniform_scale, post_normalize, valid,
                          ratio_lo, ratio_hi, clip_c, grad, acc, partials, stream);
}

extern "C" int axon_cov_policy_loss(int kind, const float* logp, const float* oldp, const float* adv,
                                    const void* mask, int mask_kind, const float* isw,
                                    const int32_t* cu, int64_t n_rows, int64_t n_slots,
                                    int64_t uniform_len, const float* row_scale, float uniform_scale,
                                    int post_normalize, const double* valid, float ratio_lo,
                                    float ratio_hi, float kl_coef, const uint32_t* keys,
                                    const void* state, float* grad, float* acc, float* partials,
                                    void* stream) {
  const bool need_row = (row_scale != nullptr);
  int rc = check_rows2(cu, n_rows, n_slots, uniform_len, need_row);
  if (rc != AXON_OK) return rc;
  if (n_slots == 0) return AXON_OK;
  if (kind < 0 || kind > 1) return AXON_ERR_ARG;
  if (!logp || !oldp || !adv || !mask || !grad || !acc || !partials || !keys || !state)
    return AXON_ERR_ARG;
  if (post_normalize && row_scale != nullptr) return AXON_ERR_ARG;
  if (mask_kind != AXON_MASK_F32 && mask_kind != AXON_MASK_I64) return AXON_ERR_ARG;
  const dim3 g(stream_grid(n_slots)), blk(kBlock);
  const hipStream_t st = (hipStream_t)stream;
  const SelectState* sel = static_cast<const SelectState*>(state);
#define AXON_LAUNCH_CV(MK, KD)                                                                    \
  hipLaunchKernelGGL((policy_loss_kernel<MK, KD>), g, blk, 0, st, logp, oldp, adv, mask, isw, cu, \
                     n_rows, n_slots, uniform_len, row_scale, (const float*)nullptr,              \
                     uniform_scale, ratio_lo, ratio_hi, kl_coef, keys, sel, grad, partials,           \
                     post_normalize ? 1 : 0, valid, acc)
  if (mask_kind == AXON_MASK_F32) {
    if (kind == 0) AXON_LAUNCH_CV(AXON_MASK_F32, 5);
    else AXON_LAUNCH_CV(AXON_MASK_F32, 6);
  } else {
    if (kind == 0) AXON_LAUNCH_CV(AXON_MASK_I64, 5);
    else AXON_LAUNCH_CV(AXON_MASK_I64, 6);
  }
#undef AXON_LAUNCH_CV
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

extern "C" int axon_kl_penalty(const float* logp, const float* ref_logp, int64_t n, int kl_type,
                               int kl_plus, float* out, float* grad, void* stream) {
  if (n < 0) return AXON_ERR_ARG;
  if (n == 0) return AXON_OK;
  if (!logp || !ref_logp || !out || !grad) return AXON_ERR_ARG;
  if (kl_type < 1 || kl_type > 4) return AXON_ERR_ARG;
  int64_t nb = (n + kBlock - 1) / kBlock;
  const int grid = (int)(nb < 8192 ? nb : 8192);
  hipLaunchKernelGGL(kl_penalty_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, logp,
                     ref_logp, n, kl_type, kl_plus, out, grad);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

extern "C" int axon_kl_reward(const float* scores, const float* old_logp, const float* ref_logp,
                              const void* mask, int mask_kind, const int32_t* cu, int64_t n_rows,
                              int64_t n_slots, int64_t uniform_len, int kl_type, float beta,
                              float* rewards, float* row_vals, void* stream) {
  int rc = check_rows2(cu, n_rows, n_slots, uniform_len, true);
  if (rc != AXON_OK) return rc;
  if (n_slots == 0) return AXON_OK;
  if (!scores || !old_logp || !ref_logp || !mask || !rewards || !row_vals) return AXON_ERR_ARG;
  if (kl_type < 1 || kl_type > 4) return AXON_ERR_ARG;
  if (mask_kind != AXON_MASK_F32 && mask_kind != AXON_MASK_I64) return AXON_ERR_ARG;
  const dim3 g(stream_grid(n_slots)), blk(kBlock);
  if (mask_kind == AXON_MASK_F32)
    hipLaunchKernelGGL(kl_reward_kernel<AXON_MASK_F32>, g, blk, 0, (hipStream_t)stream, scores, old_logp,
                       ref_logp, mask, cu, n_rows, n_slots, uniform_len, kl_type, beta, rewards, row_vals);
  else
    hipLaunchKernelGGL(kl_reward_kernel<AXON_MASK_I64>, g, blk, 0, (hipStream_t)stream, scores, old_logp,
                       ref_logp, mask, cu, n_rows, n_slots, uniform_len, kl_type, beta, rewards, row_vals);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

extern "C" int axon_side_terms(const float* entropy, const float* logp, const float* ref_logp,
                               const void* mask, int mask_kind, const int32_t* cu, int64_t n_rows,
                               int64_t n_slots, int64_t uniform_len, const float* row_scale,
                               float uniform_scale, int post_normalize, const double* valid,
                               int kl_type, int kl_plus, float* agg_w, float* grad_kl, float* acc,
                               float* partials, void* stream) {
  const bool need_row = (row_scale != nullptr);
  int rc = check_rows2(cu, n_rows, n_slots, uniform_len, need_row);
  if (rc != AXON_OK) return rc;
  if (n_slots == 0) return AXON_OK;
  if (!mask || !acc || !partials) return AXON_ERR_ARG;
  if (kl_type < 0 || kl_type > 4) return AXON_ERR_ARG;
  if (kl_type != 0 && (!logp || !ref_logp || !grad_kl)) return AXON_ERR_ARG;
  if (entropy == nullptr && kl_type == 0) return AXON_ERR_ARG;
  if (post_normalize && row_scale != nullptr) return AXON_ERR_ARG;
  if (mask_kind != AXON_MASK_F32 && mask_kind != AXON_MASK_I64) return AXON_ERR_ARG;
  const dim3 g(stream_grid(n_slots)), blk(kBlock);
  const hipStream_t st = (hipStream_t)stream;
  if (mask_kind == AXON_MASK_F32)
    hipLaunchKernelGGL(side_terms_kernel<AXON_MASK_F32>, g, blk, 0, st, entropy, logp, ref_logp, mask,
                       cu, n_rows, n_slots, uniform_len, row_scale, uniform_scale, kl_type, kl_plus,
                       agg_w, grad_kl, partials, post_normalize ? 3 : 0, valid, acc);
  else
    hipLaunchKernelGGL(side_terms_kernel<AXON_MASK_I64>, g, blk, 0, st, entropy, logp, ref_logp, mask,
                       cu, n_rows, n_slots, uniform_len, row_scale, uniform_scale, kl_type, kl_plus,
                       agg_w, grad_kl, partials, post_normalize ? 3 : 0, valid, acc);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

extern "C" int axon_gmpo_loss(const float* logp, const float* oldp, const float* adv, const void* mask,
                              int mask_kind, const float* isw, const int32_t* cu, int64_t n_rows,
                              int64_t n_slots, int64_t uniform_len, float clip_low, float clip_high,
                              float* row_ws, float* grad, float* acc, float* partials, void* stream) {
  int rc = check_rows2(cu, n_rows, n_slots, uniform_len, true);
  if (rc != AXON_OK) return rc;
  if (n_slots == 0 || n_rows == 0) return AXON_OK;
  if (!logp || !oldp || !adv || !mask || !row_ws || !grad || !acc || !partials) return AXON_ERR_ARG;
  if (mask_kind != AXON_MASK_F32 && mask_kind != AXON_MASK_I64) return AXON_ERR_ARG;
  float* row_vals = row_ws;                          // [4][n_rows], zero-filled by the caller
  float* row_coef = row_ws + kGmpoRowVals * n_rows;  // [n_rows]
  const dim3 g(stream_grid(n_slots)), blk(kBlock);
  const hipStream_t st = (hipStream_t)stream;
#define AXON_LAUNCH_GMPO(MK, PASS)                                                                  \
  hipLaunchKernelGGL((gmpo_kernel<MK, PASS>), g, blk, 0, st, logp, oldp, adv, mask, isw, cu, n_rows, \
                     n_slots, uniform_len, clip_low, clip_high, row_vals, row_coef, grad, partials)
  if (mask_kind == AXON_MASK_F32) AXON_LAUNCH_GMPO(AXON_MASK_F32, 0); else AXON_LAUNCH_GMPO(AXON_MASK_I64, 0);
  AXON_CHECK_LAUNCH();
  hipLaunchKernelGGL(reduce_partials_kernel, dim3(1), dim3(1024), 0, st, partials, (int)g.x, 0,
                     (const double*)nullptr, acc);
  AXON_CHECK_LAUNCH();
  hipLaunchKernelGGL(gmpo_rows_kernel, dim3(1), dim3(1024), 0, st, row_vals, n_rows, isw != nullptr,
                     row_coef, acc);
  AXON_CHECK_LAUNCH();
  if (mask_kind == AXON_MASK_F32) AXON_LAUNCH_GMPO(AXON_MASK_F32, 1); else AXON_LAUNCH_GMPO(AXON_MASK_I64, 1);
#undef AXON_LAUNCH_GMPO
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}
