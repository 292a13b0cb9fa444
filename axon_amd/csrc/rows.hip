// (b) Ragged segmented reductions over cu_seqlens, token-parallel.
//
// Every workgroup streams a contiguous chunk of slots with 16-byte loads.  A
// thread folds its four slots, then the wave runs a segmented shuffle reduction
// keyed by row id (row ids are non-decreasing across lanes), and the first lane
// of each run adds the run total to the per-row output with one atomic.  A row
// that spans several waves costs one atomic per wave, so load balance does not
// depend on the row-length distribution.
//
// The partial sums of a long row arrive in whatever order its wavefronts finish, and float addition
// is not associative.  The counts are sums of small integers (exact in any order) and the flags are
// ORs; the sums are added as 64-bit fixed-point integers in units of 2^-32, whose addition is
// associative, so a row's sum comes out the same bits on every run however many wavefronts it
// spans.  A partial of 2^20 or more in magnitude, an infinity or a NaN goes to a float slot beside
// it (whether that slot ends up finite, infinite or NaN does not depend on the order either).  A
// finishing pass turns the two into the fp32 sum.  Rounding a partial to 2^-32 is finer than the
// fp32 rounding of any row sum of 2^-8 or more in magnitude.
#include "common.h"

namespace axon {

struct Seg {
  int row;
  float cnt, sum;
  int flag;
};

struct RowSumAcc {
  unsigned long long* fixed;  // [n_rows] two's-complement sums in units of 2^-32
  float* big;                 // [n_rows] what does not fit the fixed-point range
};
constexpr float kRowSumUnit = 4294967296.f;  // 2^32
constexpr float kRowSumLimit = 1048576.f;    // 2^20 per partial: 2^52 units, 2^11 such partials fit 63 bits

__device__ __forceinline__ void row_sum_add(const RowSumAcc& acc, int row, float v) {
  if (fabsf(v) < kRowSumLimit)
    atomicAdd(acc.fixed + row, (unsigned long long)__float2ll_rn(v * kRowSumUnit));
  else
    atomicAdd(acc.big + row, v);
}

__global__ __launch_bounds__(256) void row_sum_finish_kernel(RowSumAcc acc, int64_t n_rows,
                                                             float* __restrict__ sum) {
  const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= n_rows) return;
  const double fixed = (double)(long long)acc.fixed[r] * (1.0 / 4294967296.0);
  sum[r] = (float)((double)acc.big[r] + fixed);
}

__device__ __forceinline__ void seg_flush(const Seg& s, float* cnt, const RowSumAcc& sum, int32_t* flag) {
  if (s.row < 0) return;
  if (cnt != nullptr && s.cnt != 0.f) atomicAdd(cnt + s.row, s.cnt);
  if (sum.fixed != nullptr && s.sum != 0.f) row_sum_add(sum, s.row, s.sum);
  if (flag != nullptr && s.flag) atomicOr(flag + s.row, 1);
}

// Segmented reduction across the wave; lanes hold (row, values) with rows sorted.
__device__ __forceinline__ void seg_wave_reduce_flush(Seg s, float* cnt, const RowSumAcc& sum,
                                                      int32_t* flag) {
  const int lane = threadIdx.x & (kWave - 1);
  // the common case: the whole wavefront sits in one row (rows are mostly longer than 256 slots)
  const int first = __builtin_amdgcn_readfirstlane(s.row);
  if (first >= 0 && __builtin_amdgcn_readlane(s.row, kWave - 1) == first) {  // rows are sorted across lanes
    Seg t;
    t.row = first;
    t.cnt = wave_sum_to_last(s.cnt);
    t.sum = wave_sum_to_last(s.sum);
    t.flag = (flag != nullptr) ? (__ballot(s.flag != 0) != 0) : 0;
    if (lane == kWave - 1) seg_flush(t, cnt, sum, flag);
    return;
  }
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const int r2 = __shfl_down(s.row, off, kWave);
    const float c2 = __shfl_down(s.cnt, off, kWave);
    const float s2 = __shfl_down(s.sum, off, kWave);
    const int f2 = __shfl_down(s.flag, off, kWave);
    if (lane + off < kWave && r2 == s.row) {
      s.cnt += c2;
      s.sum += s2;
      s.flag |= f2;
    }
  }
  const int prev = __shfl_up(s.row, 1, kWave);
  if (lane == 0 || prev != s.row) seg_flush(s, cnt, sum, flag);
}

template <int MK>
__global__ __launch_bounds__(kBlock) void row_stats_kernel(
    const float* __restrict__ a, const float* __restrict__ b, const void* __restrict__ mask,
    const int32_t* __restrict__ cu, int64_t n_rows, int64_t n_slots, int64_t uniform_len,
    int flag_mode, float thr, float* cnt, RowSumAcc sum, int32_t* flag) {
  __shared__ int32_t lds_cu[kLdsRows];
  const int64_t c0 = (int64_t)blockIdx.x * kChunk;
  const int64_t c1 = min(c0 + (int64_t)kChunk, n_slots);
  RowFinder rf;
  const bool whole = (c1 - c0 == kChunk);
  // whole chunk: every load is issued before the first use (twelve 16-byte requests in flight per
  // thread), and before the row search, whose chain of dependent loads then runs under them
  float av_[kIter][4], bv_[kIter][4], mv_[kIter][4];
  if (whole) {
#pragma unroll
    for (int it = 0; it < kIter; ++it) {
      const int64_t i = c0 + ((int64_t)it * kBlock + threadIdx.x) * kVec;
      load4(a, i, av_[it]);
      if (b != nullptr) load4(b, i, bv_[it]);
      else bv_[it][0] = bv_[it][1] = bv_[it][2] = bv_[it][3] = 0.f;
      load_mask4<MK>(mask, i, mv_[it]);
    }
  }
  rf.init(cu, n_rows, uniform_len, c0, c1, lds_cu);

  // the slots of one vector of four -> the wavefront's segmented sums
  auto fold = [&](int64_t i, const float (&av)[4], const float (&bv)[4], const float (&mv)[4]) {
    Seg s{-1, 0.f, 0.f, 0};
    if (i < c1) {
      int r = rf.row(i);
      int64_t rend = rf.row_end(r);
      s.row = r;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int64_t p = i + j;
        if (p >= n_slots) break;
        if (p >= rend) {  // slot belongs to a later row: flush and restart
          seg_flush(s, cnt, sum, flag);
          r = rf.row(p);
          rend = rf.row_end(r);
          s = Seg{r, 0.f, 0.f, 0};
        }
        const float d = av[j] - bv[j];
        const float m = mv[j];
        s.cnt += m;
        // masked_sum in the reference zeroes values outside the mask before the
        // multiply, so NaN/Inf in padding never reaches the sum.
        s.sum += (m != 0.f) ? d * m : 0.f;
        if (flag_mode == 1) s.flag |= (m != 0.f && d < thr);
        if (flag_mode == 2) s.flag |= (m != 0.f && fabsf(d) > thr);
      }
    }
    seg_wave_reduce_flush(s, cnt, sum, flag);
  };
  if (whole) {
#pragma unroll
    for (int it = 0; it < kIter; ++it)
      fold(c0 + ((int64_t)it * kBlock + threadIdx.x) * kVec, av_[it], bv_[it], mv_[it]);
    return;
  }
#pragma unroll 1
  for (int it = 0; it < kIter; ++it) {
    const int64_t i = c0 + ((int64_t)it * kBlock + threadIdx.x) * kVec;
    float av[4] = {0.f, 0.f, 0.f, 0.f}, bv[4] = {0.f, 0.f, 0.f, 0.f}, mv[4] = {0.f, 0.f, 0.f, 0.f};
    if (i < c1) {
      const bool full = (i + kVec <= n_slots);
      if (full) {
        load4(a, i, av);
        if (b != nullptr) load4(b, i, bv);
        load_mask4<MK>(mask, i, mv);
      } else {
        for (int j = 0; j < 4; ++j) {
          const bool ok = i + j < n_slots;
          av[j] = ok ? a[i + j] : 0.f;
          bv[j] = (ok && b != nullptr) ? b[i + j] : 0.f;
          mv[j] = ok ? load_mask1<MK>(mask, i + j) : 0.f;
        }
      }
    }
    fold(i, av, bv, mv);
  }
}

// group_mean_std + GRPO scalar, one workgroup.
__global__ __launch_bounds__(1024) void group_stats_kernel(
    const float* __restrict__ scores, const int64_t* __restrict__ gidx, int64_t n_rows,
    int64_t n_groups, float eps, int norm_by_std, float* mean, float* stdv, float* count,
    float* scalar) {
  __shared__ int nonzero;  // rows with a non-zero score (GPG's alpha)
  if (threadIdx.x == 0) nonzero = 0;
  __syncthreads();
  // phase 1: count -> count[], s1 -> mean[], s2 -> stdv[] (zero-filled by caller)
  for (int64_t i = threadIdx.x; i < n_rows; i += blockDim.x) {
    const int64_t g = gidx[i];
    const float x = scores[i];
    if (norm_by_std == 3 && x != 0.f) atomicAdd(&nonzero, 1);
    if (g < 0 || g >= n_groups) continue;
    atomicAdd(count + g, 1.f);
    atomicAdd(mean + g, x);
    atomicAdd(stdv + g, x * x);
  }
  __threadfence();
  __syncthreads();
  // phase 2: finalise per group
  for (int64_t g = threadIdx.x; g < n_groups; g += blockDim.x) {
    const float c = count[g], s1 = mean[g], s2 = stdv[g];
    const float cc = fmaxf(c, 1.f);
    float mu = s1 / cc;
    const float var = (s2 - (s1 * s1) / cc) / fmaxf(c - 1.f, 1.f);
    float sd = sqrtf(fmaxf(var, eps));
    if (c <= 1.f) { mu = 0.f; sd = 1.f; }
    mean[g] = mu;
    stdv[g] = sd;
  }
  __threadfence();
  __syncthreads();
  if (scalar == nullptr) return;
  for (int64_t i = threadIdx.x; i < n_rows; i += blockDim.x) {
    const int64_t g = gidx[i];
    if (g < 0 || g >= n_groups) { scalar[i] = 0.f; continue; }
    const float x = scores[i];
    const float c = count[g];
    float v;
    if (norm_by_std == 2) {  // RLOO / LOOP: (n*s - S) / (n - 1), S = n * mean (advantage.py:112-146)
      v = (c * x - c * mean[g]) / fmaxf(c - 1.f, 1.f);
    } else if (norm_by_std == 3) {  // GPG: alpha * (s - mean) / f_norm, eps carries f_norm (:336-371)
      const float alpha = (float)n_rows / (float)max(nonzero, 1);
      scalar[i] = alpha * (x - mean[g]) / eps;  // singleton groups have mean 0 and keep their score
      continue;
    } else {
      v = norm_by_std ? (x - mean[g]) / (stdv[g] + eps) : (x - mean[g]);
    }
    v = v * ((c > 1.f) ? 1.f : 0.f);
    scalar[i] = v;
  }
}

template <int MK>
__global__ __launch_bounds__(kBlock) void row_broadcast_kernel(
    const float* __restrict__ row_scalar, const void* __restrict__ mask,
    const int32_t* __restrict__ cu, int64_t n_rows, int64_t n_slots, int64_t uniform_len,
    float clamp_abs, float* __restrict__ out) {
  __shared__ int32_t lds_cu[kLdsRows];
  const int64_t c0 = (int64_t)blockIdx.x * kChunk;
  const int64_t c1 = min(c0 + (int64_t)kChunk, n_slots);
  RowFinder rf;
  if (c1 - c0 == kChunk) {
    // whole chunk: the mask loads of all four steps are in flight before the row search
    float mv[kIter][4];
#pragma unroll
    for (int it = 0; it < kIter; ++it)
      load_mask4<MK>(mask, c0 + ((int64_t)it * kBlock + threadIdx.x) * kVec, mv[it]);
    rf.init(cu, n_rows, uniform_len, c0, c1, lds_cu);
#pragma unroll
    for (int it = 0; it < kIter; ++it) {
      const int64_t i = c0 + ((int64_t)it * kBlock + threadIdx.x) * kVec;
      int r = rf.row(i);
      int64_t rend = rf.row_end(r);
      float sc = row_scalar[r];
      float o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (i + j >= rend) {
          r = rf.row(i + j);
          rend = rf.row_end(r);
          sc = row_scalar[r];
        }
        float v = sc * mv[it][j];
        if (clamp_abs > 0.f) v = fminf(fmaxf(v, -clamp_abs), clamp_abs);
        o[j] = v;
      }
      store4(out, i, o);
    }
    return;
  }
  rf.init(cu, n_rows, uniform_len, c0, c1, lds_cu);
#pragma unroll 1
  for (int it = 0; it < kIter; ++it) {
    const int64_t i = c0 + ((int64_t)it * kBlock + threadIdx.x) * kVec;
    if (i >= c1) continue;
    int r = rf.row(i);
    int64_t rend = rf.row_end(r);
    float sc = row_scalar[r];
    float mv[4], o[4];
    const bool full = (i + kVec <= n_slots);
    if (full) load_mask4<MK>(mask, i, mv);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t p = i + j;
      if (p >= n_slots) break;
      if (p >= rend) {
        r = rf.row(p);
        rend = rf.row_end(r);
        sc = row_scalar[r];
      }
      const float m = full ? mv[j] : load_mask1<MK>(mask, p);
      float v = sc * m;
      if (clamp_abs > 0.f) v = fminf(fmaxf(v, -clamp_abs), clamp_abs);
      o[j] = v;
    }
    if (full) store4(out, i, o);
    else
      for (int j = 0; j < 4 && i + j < n_slots; ++j) out[i + j] = o[j];
  }
}

__global__ __launch_bounds__(kBlock) void fill_zero_kernel(uint32_t* p, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x)
    p[i] = 0u;
}

}  // namespace axon

using namespace axon;

static inline int grid_for(int64_t n_slots) { return (int)((n_slots + kChunk - 1) / kChunk); }

// out[i] = x[i] * s1[0] * (s2 ? s2[0] : 1): the chain rule of a scalar loss whose per-token gradient the
// forward left unscaled (the factors live on the device).
__global__ __launch_bounds__(kBlock) void scale_by_scalars_kernel(const float* __restrict__ x,
                                                                  const float* __restrict__ s1,
                                                                  const float* __restrict__ s2,
                                                                  float* __restrict__ out, int64_t n) {
  const float f = s1[0] * (s2 != nullptr ? s2[0] : 1.f);
  const int64_t n4 = n / 4;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
    const float4 v = reinterpret_cast<const float4*>(x)[i];
    reinterpret_cast<float4*>(out)[i] = make_float4(v.x * f, v.y * f, v.z * f, v.w * f);
  }
  const int64_t t = n4 * 4 + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t < n) out[t] = x[t] * f;
}

extern "C" int axon_scale_f32(const float* x, const float* s1, const float* s2, float* out, int64_t n,
                              void* stream) {
  if (n < 0) return AXON_ERR_SHAPE;
  if (n == 0) return AXON_OK;
  if (!x || !s1 || !out) return AXON_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) & 15) return AXON_ERR_ARG;
  const int64_t blocks = (n / 4 + kBlock - 1) / kBlock;
  const unsigned grid = (unsigned)(blocks < 1 ? 1 : blocks < 4096 ? blocks : 4096);
  hipLaunchKernelGGL(scale_by_scalars_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, x, s1, s2,
                     out, n);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

extern "C" int axon_fill_zero(void* ptr, int64_t n_bytes, void* stream) {
  if (n_bytes < 0 || (n_bytes & 3) != 0) return AXON_ERR_ARG;
  if (n_bytes == 0) return AXON_OK;
  if (ptr == nullptr) return AXON_ERR_ARG;
  const int64_t n = n_bytes / 4;
  int64_t nb = (n + kBlock - 1) / kBlock;
  const int grid = (int)(nb < 4096 ? nb : 4096);
  hipLaunchKernelGGL(fill_zero_kernel, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream,
                     (uint32_t*)ptr, n);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

static int check_rows(const int32_t* cu, int64_t n_rows, int64_t n_slots, int64_t uniform_len) {
  if (n_rows < 0 || n_slots < 0 || uniform_len < 0) return AXON_ERR_ARG;
  if (n_rows >= (int64_t)INT32_MAX || n_slots >= (int64_t)INT32_MAX) return AXON_ERR_SHAPE;
  if (uniform_len == 0 && cu == nullptr && n_slots > 0) return AXON_ERR_ARG;
  if (uniform_len > 0 && n_rows * uniform_len != n_slots) return AXON_ERR_SHAPE;
  if (uniform_len == 0 && n_rows == 0 && n_slots > 0) return AXON_ERR_SHAPE;  // tokens that belong to no row
  return AXON_OK;
}

extern "C" int64_t axon_row_stats_workspace_bytes(int64_t n_rows) {
  return n_rows < 0 ? -1 : n_rows * 12;
}

extern "C" int axon_row_stats(const float* a, const float* b, const void* mask, int mask_kind,
                              const int32_t* cu, int64_t n_rows, int64_t n_slots,
                              int64_t uniform_len, int flag_mode, float thr, float* cnt,
                              float* sum, int32_t* flag, void* sum_workspace, void* stream) {
  int rc = check_rows(cu, n_rows, n_slots, uniform_len);
  if (rc != AXON_OK) return rc;
  if (n_slots == 0 || n_rows == 0) return AXON_OK;
  if (a == nullptr) return AXON_ERR_ARG;
  if (flag_mode < 0 || flag_mode > 2) return AXON_ERR_ARG;
  if (flag_mode != 0 && flag == nullptr) return AXON_ERR_ARG;
  if (mask_kind != AXON_MASK_F32 && mask_kind != AXON_MASK_I64) return AXON_ERR_ARG;
  if (sum != nullptr && (sum_workspace == nullptr || (reinterpret_cast<uintptr_t>(sum_workspace) & 7)))
    return AXON_ERR_WORKSPACE;
  RowSumAcc acc{nullptr, nullptr};
  if (sum != nullptr) {
    acc.fixed = static_cast<unsigned long long*>(sum_workspace);
    acc.big = reinterpret_cast<float*>(acc.fixed + n_rows);
  }
  const dim3 g(grid_for(n_slots)), blk(kBlock);
  if (mask_kind == AXON_MASK_F32)
    hipLaunchKernelGGL(row_stats_kernel<AXON_MASK_F32>, g, blk, 0, (hipStream_t)stream, a, b, mask,
                       cu, n_rows, n_slots, uniform_len, flag_mode, thr, cnt, acc, flag);
  else
    hipLaunchKernelGGL(row_stats_kernel<AXON_MASK_I64>, g, blk, 0, (hipStream_t)stream, a, b, mask,
                       cu, n_rows, n_slots, uniform_len, flag_mode, thr, cnt, acc, flag);
  AXON_CHECK_LAUNCH();
  if (sum != nullptr) {
    hipLaunchKernelGGL(row_sum_finish_kernel, dim3((unsigned)((n_rows + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, acc, n_rows, sum);
    AXON_CHECK_LAUNCH();
  }
  return AXON_OK;
}

extern "C" int axon_group_stats(const float* scores, const int64_t* gidx, int64_t n_rows,
                                int64_t n_groups, float eps, int norm_by_std, float* mean,
                                float* stdv, float* count, float* scalar, void* stream) {
  if (n_rows < 0 || n_groups < 0) return AXON_ERR_ARG;
  if (n_rows >= (int64_t)INT32_MAX) return AXON_ERR_SHAPE;
  if (n_rows == 0 || n_groups == 0) return AXON_OK;
  if (!scores || !gidx || !mean || !stdv || !count) return AXON_ERR_ARG;
  hipLaunchKernelGGL(group_stats_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, scores, gidx,
                     n_rows, n_groups, eps, norm_by_std, mean, stdv, count, scalar);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

extern "C" int axon_row_broadcast_mask(const float* row_scalar, const void* mask, int mask_kind,
                                       const int32_t* cu, int64_t n_rows, int64_t n_slots,
                                       int64_t uniform_len, float clamp_abs, float* out,
                                       void* stream) {
  int rc = check_rows(cu, n_rows, n_slots, uniform_len);
  if (rc != AXON_OK) return rc;
  if (n_slots == 0 || n_rows == 0) return AXON_OK;
  if (!row_scalar || !out) return AXON_ERR_ARG;
  if (mask_kind != AXON_MASK_F32 && mask_kind != AXON_MASK_I64) return AXON_ERR_ARG;
  const dim3 g(grid_for(n_slots)), blk(kBlock);
  if (mask_kind == AXON_MASK_F32)
    hipLaunchKernelGGL(row_broadcast_kernel<AXON_MASK_F32>, g, blk, 0, (hipStream_t)stream,
                       row_scalar, mask, cu, n_rows, n_slots, uniform_len, clamp_abs, out);
  else
    hipLaunchKernelGGL(row_broadcast_kernel<AXON_MASK_I64>, g, blk, 0, (hipStream_t)stream,
                       row_scalar, mask, cu, n_rows, n_slots, uniform_len, clamp_abs, out);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}
