// Return-based advantage estimators: time recurrences that run from a row's last token to its first,
// global masked whitening, and the per-group scalars of the estimators that need more than mean/std.
//
// A recurrence y[t] = b[t] + a[t] * y[t+1] is a scan over pairs (a, b) under the composition
// (a2, b2) o (a1, b1) = (a2*a1, b2 + a2*b1).  One wavefront owns one row and walks it from the end in
// windows of 256 tokens that are 4-aligned in the token array: a lane holds four consecutive tokens (one
// 16-byte access where the vector lies inside the row, guarded scalar accesses at the row's edges), lane 0
// the last ones.  A lane composes its four elements, the wavefront scans the 64 composites with DPP row shifts and broadcasts,
// and each lane then replays its four tokens from the value that enters it.  The loads of the next window
// are issued before the current one is scanned.
#include "common.h"

namespace axon {

constexpr int kScanVec = 4;                      // tokens per lane
constexpr int kScanStep = kScanVec * kWave;      // tokens per window

struct Pair { float a, b; };

// p after q: y -> p.b + p.a * (q.b + q.a * y)
__device__ __forceinline__ Pair after(Pair p, Pair q) { return Pair{p.a * q.a, p.b + p.a * q.b}; }

// Data-parallel-primitive moves (GFX9 DPP): `row_shr:n` hands lane i the value of lane i-n inside its row
// of 16 lanes, `row_bcast:15` / `row_bcast:31` hand the last lane of a row / of the lower half to the rows
// selected by ROW_MASK, `wave_shr:1` shifts across the whole wavefront.  A lane without a source keeps `old`.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float old, float src) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old),
                                                               __builtin_bit_cast(int, src), CTRL,
                                                               ROW_MASK, 0xf, false));
}

// inclusive scan over lanes 0..63: lane l ends with the composition of the elements of lanes 0..l.
// Lanes without a partner compose with the identity (1, 0).
__device__ __forceinline__ Pair wave_scan(Pair p) {
#define AXON_SCAN_STEP(CTRL, ROW_MASK)                                  \
  {                                                                     \
    const float ap = dpp_move<CTRL, ROW_MASK>(1.f, p.a);                \
    const float bp = dpp_move<CTRL, ROW_MASK>(0.f, p.b);                \
    p = after(p, Pair{ap, bp});                                         \
  }
  AXON_SCAN_STEP(0x111, 0xf)  // row_shr:1
  AXON_SCAN_STEP(0x112, 0xf)  // row_shr:2
  AXON_SCAN_STEP(0x114, 0xf)  // row_shr:4
  AXON_SCAN_STEP(0x118, 0xf)  // row_shr:8
  AXON_SCAN_STEP(0x142, 0xa)  // row_bcast:15 into rows 1 and 3
  AXON_SCAN_STEP(0x143, 0xc)  // row_bcast:31 into rows 2 and 3
#undef AXON_SCAN_STEP
  return p;
}

// Scans the lanes' composites; returns the value that enters this lane (the recurrence at the token after the
// lane's last one) and moves `carry` to the value that leaves lane 63.
__device__ __forceinline__ float scan_enter(Pair lane_total, float& carry) {
  const Pair s = wave_scan(lane_total);
  const float leaves = s.b + s.a * carry;
  const float enters = dpp_move<0x138, 0xf>(carry, leaves);  // wave_shr:1; lane 0 keeps the carry
  carry = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, leaves), kWave - 1));
  return enters;
}

enum { kScanGae = 0, kScanGaeResponseOnly = 1, kScanDiscounted = 2, kScanSuffixSum = 3 };

struct ScanBlock {
  float r[kScanVec], v[kScanVec], m[kScanVec];
  int ok;  // bit j: token p0 + j lies inside the row
};

// window [end - 256, end), end a multiple of 4; this lane's tokens are p0 .. p0 + 3
template <int MK, int MODE>
__device__ __forceinline__ void scan_load(ScanBlock& x, const float* __restrict__ rewards,
                                          const float* __restrict__ values,
                                          const void* __restrict__ mask, int64_t begin, int64_t stop,
                                          int64_t end, bool vec_ok) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t p0 = end - kScanVec * (lane + 1);
  constexpr bool kValues = MODE <= kScanGaeResponseOnly;
  if (vec_ok && p0 >= begin && p0 + kScanVec <= stop) {
    load4(rewards, p0, x.r);
    if (kValues) load4(values, p0, x.v);
    load_mask4<MK>(mask, p0, x.m);
    x.ok = 15;
  } else {
    x.ok = 0;
#pragma unroll
    for (int j = 0; j < kScanVec; ++j) {
      const int64_t p = p0 + j;
      const bool ok = p >= begin && p < stop;
      x.r[j] = ok ? rewards[p] : 0.f;
      x.v[j] = (ok && kValues) ? values[p] : 0.f;
      x.m[j] = ok ? load_mask1<MK>(mask, p) : 0.f;
      x.ok |= ok ? (1 << j) : 0;
    }
  }
  if (!kValues) x.v[0] = x.v[1] = x.v[2] = x.v[3] = 0.f;
  if (MODE == kScanGaeResponseOnly) {
#pragma unroll
    for (int j = 0; j < kScanVec; ++j) x.m[j] = x.m[j] > 0.f ? 1.f : 0.f;
  }
}

// MODE kScanGae:  nv[t] = m v + (1-m) nv[t+1];  delta = r + gamma nv[t+1] - v;
//                 L[t] = m (delta + gamma*lam L[t+1]) + (1-m) L[t+1];  adv = L, ret = L + v.
// MODE kScanGaeResponseOnly: the same over the tokens with mask > 0, 0 elsewhere.
// MODE kScanDiscounted: Q[t] = m (r + gamma Q[t+1]);  ret = r + gamma Q[t+1].
// MODE kScanSuffixSum:  ret[t] = sum_{s >= t} r m;  adv = ret - row_baseline * m.
template <int MK, int MODE>
__global__ __launch_bounds__(kBlock) void reverse_scan_kernel(
    const float* __restrict__ rewards, const float* __restrict__ values,
    const void* __restrict__ mask, const int32_t* __restrict__ cu, int64_t n_rows, int64_t n_slots,
    int64_t uniform_len, float gamma, float gamma_lam, const float* __restrict__ row_baseline,
    float* __restrict__ adv, float* __restrict__ ret, int vec_ok) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row = (int64_t)blockIdx.x * (kBlock / kWave) + (threadIdx.x / kWave);
  if (row >= n_rows) return;  // whole wavefronts leave together; no workgroup barrier below
  int64_t begin = uniform_len > 0 ? row * uniform_len : (int64_t)cu[row];
  int64_t stop = uniform_len > 0 ? begin + uniform_len : (int64_t)cu[row + 1];
  begin = begin < 0 ? 0 : begin;              // offsets outside the arrays (caller error) touch nothing
  stop = stop > n_slots ? n_slots : stop;
  if (stop <= begin) return;
  const float base = (MODE == kScanSuffixSum && row_baseline) ? row_baseline[row] : 0.f;
  float carry0 = 0.f, carry1 = 0.f;  // the recurrences' values at the token after the current window
  const int64_t last = (stop + kScanVec - 1) & ~(int64_t)(kScanVec - 1);
  ScanBlock cur, nxt;
  scan_load<MK, MODE>(cur, rewards, values, mask, begin, stop, last, vec_ok);
  for (int64_t end = last; end > begin; end -= kScanStep) {
    const bool more = end - kScanStep > begin;
    if (more) scan_load<MK, MODE>(nxt, rewards, values, mask, begin, stop, end - kScanStep, vec_ok);
    float out_adv[kScanVec], out_ret[kScanVec];
    if (MODE <= kScanGaeResponseOnly) {
      Pair e[kScanVec];
#pragma unroll
      for (int j = 0; j < kScanVec; ++j) e[j] = Pair{1.f - cur.m[j], cur.m[j] * cur.v[j]};
      float nv = scan_enter(after(e[0], after(e[1], after(e[2], e[3]))), carry0);
#pragma unroll
      for (int j = kScanVec - 1; j >= 0; --j) {
        const float delta = cur.r[j] + gamma * nv - cur.v[j];
        nv = e[j].b + e[j].a * nv;
        e[j] = Pair{cur.m[j] * gamma_lam + (1.f - cur.m[j]), cur.m[j] * delta};
      }
      float l = scan_enter(after(e[0], after(e[1], after(e[2], e[3]))), carry1);
#pragma unroll
      for (int j = kScanVec - 1; j >= 0; --j) {
        l = e[j].b + e[j].a * l;
        const bool keep = (MODE == kScanGae) || cur.m[j] > 0.f;
        out_adv[j] = keep ? l : 0.f;
        out_ret[j] = keep ? l + cur.v[j] : 0.f;
      }
    } else {
      Pair e[kScanVec];
#pragma unroll
      for (int j = 0; j < kScanVec; ++j) {
        const bool ok = (cur.ok >> j) & 1;
        if (MODE == kScanDiscounted) e[j] = Pair{ok ? gamma * cur.m[j] : 1.f, cur.m[j] * cur.r[j]};
        else e[j] = Pair{1.f, cur.r[j] * cur.m[j]};
      }
      float q = scan_enter(after(e[0], after(e[1], after(e[2], e[3]))), carry0);
#pragma unroll
      for (int j = kScanVec - 1; j >= 0; --j) {
        if (MODE == kScanDiscounted) {
          out_ret[j] = cur.r[j] + gamma * q;
          out_adv[j] = 0.f;
          q = e[j].b + e[j].a * q;
        } else {
          q = e[j].b + q;
          out_ret[j] = q;
          out_adv[j] = q - base * cur.m[j];
        }
      }
    }
    const int64_t p0 = end - kScanVec * (lane + 1);
    if (cur.ok == 15 && vec_ok) {
      if (adv != nullptr) store4(adv, p0, out_adv);
      store4(ret, p0, out_ret);
    } else {
#pragma unroll
      for (int j = 0; j < kScanVec; ++j) {
        if ((cur.ok >> j) & 1) {
          if (adv != nullptr) adv[p0 + j] = out_adv[j];
          ret[p0 + j] = out_ret[j];
        }
      }
    }
    if (more) cur = nxt;
  }
}

// ---- masked whitening -------------------------------------------------------------------------
// stats[0] mean, [1] n, [2] variance (times n/(n-1) when n > 1), [3] rsqrt(variance + 1e-8)

// PASS 0: sum m x, sum m.   PASS 1: sum m (x - mean)^2.
template <int MK, int PASS>
__global__ __launch_bounds__(kBlock) void masked_moments_kernel(const float* __restrict__ x,
                                                                const void* __restrict__ mask,
                                                                int64_t n_slots,
                                                                const float* __restrict__ stats,
                                                                float* partials) {
  __shared__ float lds_red[2 * (kBlock / kWave)];
  const float mean = PASS == 1 ? stats[0] : 0.f;
  float a[2] = {0.f, 0.f};
  const int64_t n_vec = n_slots / kVec;
  for (int64_t q = (int64_t)blockIdx.x * kBlock + threadIdx.x; q < n_vec;
       q += (int64_t)gridDim.x * kBlock) {
    float xv[4], mv[4];
    load4(x, q * kVec, xv);
    load_mask4<MK>(mask, q * kVec, mv);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (PASS == 0) {
        a[0] += (mv[j] != 0.f) ? xv[j] * mv[j] : 0.f;
        a[1] += mv[j];
      } else {
        const float d = xv[j] - mean;
        a[0] += (mv[j] != 0.f) ? d * d * mv[j] : 0.f;
      }
    }
  }
  if (blockIdx.x == 0 && threadIdx.x < (int)(n_slots - n_vec * kVec)) {  // the ragged tail
    const int64_t p = n_vec * kVec + threadIdx.x;
    const float xv = x[p], m = load_mask1<MK>(mask, p);
    if (PASS == 0) {
      a[0] += (m != 0.f) ? xv * m : 0.f;
      a[1] += m;
    } else {
      const float d = xv - mean;
      a[0] += (m != 0.f) ? d * d * m : 0.f;
    }
  }
  store_block_partials<2>(a, lds_red, partials);
}

// one workgroup adds the partials in a fixed order and finishes the statistics
__global__ __launch_bounds__(kBlock) void masked_moments_finish_kernel(const float* __restrict__ partials,
                                                                       int n_blocks, int pass,
                                                                       float* __restrict__ stats) {
  __shared__ float lds_red[2 * (kBlock / kWave)];
  float a[2] = {0.f, 0.f};
  for (int b = threadIdx.x; b < n_blocks; b += kBlock) {
    a[0] += partials[(size_t)b * kPartialStride];
    a[1] += partials[(size_t)b * kPartialStride + 1];
  }
  block_sum<2>(a, lds_red);
  if (threadIdx.x == 0) {
    if (pass == 0) {
      stats[0] = a[0] / fmaxf(a[1], 1.f);
      stats[1] = a[1];
    } else {
      const float n = stats[1];
      float var = a[0] / fmaxf(n, 1.f);
      if (n > 1.f) var = var * n / (n - 1.f);
      stats[2] = var;
      stats[3] = rsqrtf(var + 1e-8f);
    }
  }
}

template <int MK>
__global__ __launch_bounds__(kBlock) void whiten_kernel(const float* __restrict__ x,
                                                        const void* __restrict__ mask,
                                                        int64_t n_slots,
                                                        const float* __restrict__ stats, int remask,
                                                        float* __restrict__ out) {
  const float mean = stats[0], rstd = stats[3];
  const int64_t n_vec = n_slots / kVec;
  for (int64_t q = (int64_t)blockIdx.x * kBlock + threadIdx.x; q < n_vec;
       q += (int64_t)gridDim.x * kBlock) {
    float xv[4], mv[4] = {1.f, 1.f, 1.f, 1.f}, o[4];
    load4(x, q * kVec, xv);
    if (remask) load_mask4<MK>(mask, q * kVec, mv);
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = (xv[j] - mean) * rstd * mv[j];
    store4(out, q * kVec, o);
  }
  if (blockIdx.x == 0 && threadIdx.x < (int)(n_slots - n_vec * kVec)) {
    const int64_t p = n_vec * kVec + threadIdx.x;
    const float m = remask ? load_mask1<MK>(mask, p) : 1.f;
    out[p] = (x[p] - mean) * rstd * m;
  }
}

// ---- per-group scalars --------------------------------------------------------------------------
// One thread per group walks the group's rows in row order (members[offsets[g] .. offsets[g+1])), so sums
// are formed in a fixed order without atomics.
//   mode 0 (OPO): s - (n > 1 ? sum(len s) / max(sum len, 1) : 0)
//   mode 1 (REINFORCE++ baseline): s - (n > 1 ? sum s / n : 0)
//   mode 2 (pass@k): best row gets max - second max, divided by (unbiased std + eps) when p_norm; others 0
//   mode 3 (Kimi k1.5): s' = s + coef-scaled length term, then the group-normalised scalar of s'
__global__ __launch_bounds__(kBlock) void group_scalar_kernel(
    int mode, const float* __restrict__ scores, const float* __restrict__ lens,
    const int32_t* __restrict__ members, const int32_t* __restrict__ offsets, int64_t n_groups,
    float eps, int p_norm, float coef, float threshold, float* __restrict__ out) {
  const int64_t g = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (g >= n_groups) return;
  const int lo = offsets[g], hi = offsets[g + 1];
  const float n = (float)(hi - lo);
  if (mode == 0 || mode == 1) {
    float s1 = 0.f, w1 = 0.f, l1 = 0.f;
    for (int k = lo; k < hi; ++k) {
      const int i = members[k];
      const float s = scores[i];
      s1 += s;
      if (mode == 0) { w1 += lens[i] * s; l1 += lens[i]; }
    }
    float base = 0.f;
    if (n > 1.f) base = (mode == 0) ? w1 / fmaxf(l1, 1.f) : s1 / fmaxf(n, 1.f);
    for (int k = lo; k < hi; ++k) out[members[k]] = scores[members[k]] - base;
    return;
  }
  if (mode == 2) {
    float best = -INFINITY, second = -INFINITY, s1 = 0.f;
    int arg = -1;
    for (int k = lo; k < hi; ++k) {
      const int i = members[k];
      const float s = scores[i];
      s1 += s;
      if (arg < 0 || s > best) { second = best; best = s; arg = i; }
      else if (s > second) second = s;
      out[i] = 0.f;
    }
    if (hi - lo < 2) return;  // the caller rejects such groups before the launch
    float a = best - second;
    if (p_norm) {
      const float mean = s1 / n;
      float ss = 0.f;
      for (int k = lo; k < hi; ++k) { const float d = scores[members[k]] - mean; ss += d * d; }
      a = a / (sqrtf(ss / (n - 1.f)) + eps);
    }
    out[arg] = a;
    return;
  }
  // mode 3
  float len_lo = INFINITY, len_hi = -INFINITY;
  for (int k = lo; k < hi; ++k) {
    const float l = lens[members[k]];
    len_lo = fminf(len_lo, l);
    len_hi = fmaxf(len_hi, l);
  }
  const float spread = len_hi - len_lo;
  auto shaped = [&](int i) {
    const float s = scores[i];
    if (!(coef > 0.f)) return s;
    const float lam = coef * (0.5f - (lens[i] - len_lo) / fmaxf(spread, 1.f));
    const float bonus = (s >= threshold) ? lam : fminf(lam, 0.f);
    return s + bonus * (spread > 0.f ? 1.f : 0.f);
  };
  float s1 = 0.f, s2 = 0.f;
  for (int k = lo; k < hi; ++k) { const float s = shaped(members[k]); s1 += s; s2 += s * s; }
  const float nn = fmaxf(n, 1.f);
  float mean = s1 / nn;
  float sd = sqrtf(fmaxf((s2 - s1 * s1 / nn) / fmaxf(n - 1.f, 1.f), eps));
  if (n <= 1.f) { mean = 0.f; sd = 1.f; }
  for (int k = lo; k < hi; ++k) {
    const int i = members[k];
    float a = shaped(i) - mean;
    if (p_norm) a = a / (sd + eps);
    out[i] = (n > 1.f) ? a : 0.f;
  }
}

}  // namespace axon

using namespace axon;

namespace {

template <int MK>
int launch_scan(int mode, const float* rewards, const float* values, const void* mask,
                const int32_t* cu, int64_t n_rows, int64_t n_slots, int64_t uniform_len, float gamma,
                float gamma_lam, const float* row_baseline, float* adv, float* ret, hipStream_t st) {
  // 16-byte accesses need every array on a 16-byte boundary (an int64 mask then is on 32)
  const int vec_ok = ((reinterpret_cast<uintptr_t>(rewards) | reinterpret_cast<uintptr_t>(values) |
                       reinterpret_cast<uintptr_t>(mask) | reinterpret_cast<uintptr_t>(adv) |
                       reinterpret_cast<uintptr_t>(ret)) & 15) == 0;
  const dim3 grid((unsigned)((n_rows + (kBlock / kWave) - 1) / (kBlock / kWave))), blk(kBlock);
#define AXON_SCAN(M)                                                                              \
  hipLaunchKernelGGL((reverse_scan_kernel<MK, M>), grid, blk, 0, st, rewards, values, mask, cu,   \
                     n_rows, n_slots, uniform_len, gamma, gamma_lam, row_baseline, adv, ret, vec_ok)
  switch (mode) {
    case kScanGae: AXON_SCAN(kScanGae); break;
    case kScanGaeResponseOnly: AXON_SCAN(kScanGaeResponseOnly); break;
    case kScanDiscounted: AXON_SCAN(kScanDiscounted); break;
    default: AXON_SCAN(kScanSuffixSum); break;
  }
#undef AXON_SCAN
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

unsigned moments_grid(int64_t n_slots) {
  const int64_t blocks = (n_slots / kVec + kBlock - 1) / kBlock;
  const int64_t cap = 2048;  // eight workgroups per compute unit walk the tokens
  return (unsigned)(blocks < 1 ? 1 : (blocks < cap ? blocks : cap));
}

template <int MK>
int launch_whiten(const float* x, const void* mask, int64_t n_slots, int remask, float* out,
                  float* stats, float* partials, hipStream_t st) {
  const dim3 grid(moments_grid(n_slots)), blk(kBlock);
  hipLaunchKernelGGL((masked_moments_kernel<MK, 0>), grid, blk, 0, st, x, mask, n_slots, stats, partials);
  hipLaunchKernelGGL(masked_moments_finish_kernel, dim3(1), blk, 0, st, partials, (int)grid.x, 0, stats);
  hipLaunchKernelGGL((masked_moments_kernel<MK, 1>), grid, blk, 0, st, x, mask, n_slots, stats, partials);
  hipLaunchKernelGGL(masked_moments_finish_kernel, dim3(1), blk, 0, st, partials, (int)grid.x, 1, stats);
  AXON_CHECK_LAUNCH();
  if (out != nullptr) {
    hipLaunchKernelGGL((whiten_kernel<MK>), grid, blk, 0, st, x, mask, n_slots, stats, remask, out);
    AXON_CHECK_LAUNCH();
  }
  return AXON_OK;
}

}  // namespace

extern "C" int axon_reverse_scan(int mode, const float* rewards, const float* values,
                                 const void* mask, int mask_kind, const int32_t* cu_seqlens,
                                 int64_t n_rows, int64_t n_slots, int64_t uniform_len, float gamma,
                                 float lam, const float* row_baseline, float* adv, float* ret,
                                 void* stream) {
  if (n_rows < 0 || n_slots < 0 || uniform_len < 0) return AXON_ERR_ARG;
  if (n_rows >= (int64_t)INT32_MAX || n_slots >= (int64_t)INT32_MAX) return AXON_ERR_SHAPE;
  if (uniform_len > 0 && n_rows * uniform_len != n_slots) return AXON_ERR_SHAPE;
  if (mode < kScanGae || mode > kScanSuffixSum) return AXON_ERR_ARG;
  if (uniform_len == 0 && n_rows == 0 && n_slots > 0) return AXON_ERR_SHAPE;  // tokens that belong to no row
  if (n_slots == 0 || n_rows == 0) return AXON_OK;
  if (uniform_len == 0 && !cu_seqlens) return AXON_ERR_ARG;
  if (!rewards || !ret) return AXON_ERR_ARG;
  if (mode <= kScanGaeResponseOnly && (!values || !adv)) return AXON_ERR_ARG;
  if (mode == kScanSuffixSum && !adv) return AXON_ERR_ARG;
  if (mask_kind != AXON_MASK_F32 && mask_kind != AXON_MASK_I64) return AXON_ERR_ARG;
  // gamma * lam in double, rounded once: what `gamma * lam * tensor` does with Python scalars
  const float gamma_lam = (float)((double)gamma * (double)lam);
  float* adv_out = (mode == kScanDiscounted) ? nullptr : adv;
  const hipStream_t st = (hipStream_t)stream;
  if (mask_kind == AXON_MASK_F32)
    return launch_scan<AXON_MASK_F32>(mode, rewards, values, mask, cu_seqlens, n_rows, n_slots, uniform_len,
                                      gamma, gamma_lam, row_baseline, adv_out, ret, st);
  return launch_scan<AXON_MASK_I64>(mode, rewards, values, mask, cu_seqlens, n_rows, n_slots, uniform_len,
                                    gamma, gamma_lam, row_baseline, adv_out, ret, st);
}

extern "C" int64_t axon_masked_whiten_workspace_bytes(int64_t n_slots) {
  if (n_slots < 0) return AXON_ERR_ARG;
  return (int64_t)moments_grid(n_slots) * kPartialStride * (int64_t)sizeof(float);
}

extern "C" int axon_masked_whiten(const float* x, const void* mask, int mask_kind, int64_t n_slots,
                                  int remask, float* out, float* stats, float* partials,
                                  void* stream) {
  if (n_slots < 0) return AXON_ERR_ARG;
  if (n_slots >= (int64_t)INT32_MAX * 4) return AXON_ERR_SHAPE;
  if (!stats || !partials) return AXON_ERR_ARG;
  if (n_slots > 0 && (!x || !mask)) return AXON_ERR_ARG;
  if (mask_kind != AXON_MASK_F32 && mask_kind != AXON_MASK_I64) return AXON_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(mask) |
       reinterpret_cast<uintptr_t>(out)) & 15)
    return AXON_ERR_ARG;
  const hipStream_t st = (hipStream_t)stream;
  if (mask_kind == AXON_MASK_F32)
    return launch_whiten<AXON_MASK_F32>(x, mask, n_slots, remask, out, stats, partials, st);
  return launch_whiten<AXON_MASK_I64>(x, mask, n_slots, remask, out, stats, partials, st);
}

extern "C" int axon_group_scalar(int mode, const float* scores, const float* lens,
                                 const int32_t* members, const int32_t* offsets, int64_t n_rows,
                                 int64_t n_groups, float eps, int normalize, float coef,
                                 float threshold, float* scalar, void* stream) {
  if (n_rows < 0 || n_groups < 0 || mode < 0 || mode > 3) return AXON_ERR_ARG;
  if (n_rows >= (int64_t)INT32_MAX || n_groups >= (int64_t)INT32_MAX) return AXON_ERR_SHAPE;
  if (n_rows == 0 || n_groups == 0) return AXON_OK;
  if (!scores || !members || !offsets || !scalar) return AXON_ERR_ARG;
  if ((mode == 0 || mode == 3) && !lens) return AXON_ERR_ARG;
  hipLaunchKernelGGL(group_scalar_kernel, dim3((unsigned)((n_groups + kBlock - 1) / kBlock)),
                     dim3(kBlock), 0, (hipStream_t)stream, mode, scores, lens, members, offsets,
                     n_groups, eps, normalize, coef, threshold, scalar);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}
