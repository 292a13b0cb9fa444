// Diagnostics of the sampler / trainer mismatch: every scalar the reference reports for the
// importance weights, the rejection mask, the off-policy divergences and the log-prob mismatch,
// from ONE pass over the tokens plus ONE pass over the rows, read back by the host in one copy.
//
// Pass 1 (token-parallel, same streaming skeleton as the loss kernels): per-token quantities are
// folded into per-workgroup partial sums / minima / maxima, per-row sums go through a segmented
// wave reduction and one atomic per (wave, row).
// Pass 2 (one workgroup): adds the partials in a fixed order in double precision and walks the
// rows for the sequence-level statistics.
#include "common.h"

namespace axon {

constexpr int kDiagSums = 23;    // token-level sums, see axon_amd.h
constexpr int kDiagMinMax = 6;   // max e, min e, max |pa-ps|, min |pa-ps|, max |lr|, min |lr|
constexpr int kDiagStride = 32;  // floats per workgroup in `partials`
constexpr int kDiagRowVals = 6;  // cnt, sum old, sum sampler, sum lr, sum e, sum token-rejected
constexpr float kBound = 20.0f;  // axon/utils/rl/sampler.py:27

__device__ __forceinline__ float clampf3(float x, float lo, float hi) {
  return (x != x) ? x : fminf(fmaxf(x, lo), hi);
}

using DiagSeg = RowSeg<kDiagRowVals>;

__device__ __forceinline__ void diag_flush(const DiagSeg& s, float* row_vals, int64_t n_rows) {
  row_seg_flush(s, row_vals, n_rows);
}
__device__ __forceinline__ void diag_wave_reduce_flush(DiagSeg s, float* row_vals, int64_t n_rows) {
  row_seg_wave_reduce_flush(s, row_vals, n_rows);
}

template <int MK>
__global__ __launch_bounds__(kBlock) void sampler_diag_tokens_kernel(
    const float* __restrict__ oldp, const float* __restrict__ samp, const void* __restrict__ mask,
    const int32_t* __restrict__ cu, int64_t n_rows, int64_t n_slots, int64_t uniform_len,
    float is_lo, float is_hi, float rs_lo, float rs_hi, float rs_lr_lo, float rs_lr_hi,
    float* row_vals, float* __restrict__ partials) {
  __shared__ int32_t lds_cu[kLdsRows];
  __shared__ float lds_red[kDiagSums * (kBlock / kWave)];
  __shared__ float lds_mm[kDiagMinMax * (kBlock / kWave)];
  const float kInf = __builtin_huge_valf();
  float a[kDiagSums];
#pragma unroll
  for (int k = 0; k < kDiagSums; ++k) a[k] = 0.f;
  float mx[3] = {-kInf, -kInf, -kInf}, mn[3] = {kInf, kInf, kInf};

  const int64_t n_chunks = (n_slots + kChunk - 1) / kChunk;
#pragma unroll 1
  for (int64_t chunk = blockIdx.x; chunk < n_chunks; chunk += gridDim.x) {
    const int64_t c0 = chunk * kChunk;
    const int64_t c1 = min(c0 + (int64_t)kChunk, n_slots);
    __syncthreads();  // the previous chunk's row window is no longer read
    RowFinder rf;
    rf.init(cu, n_rows, uniform_len, c0, c1, lds_cu);
#pragma unroll 1
    for (int it = 0; it < kIter; ++it) {
      const int64_t i = c0 + ((int64_t)it * kBlock + threadIdx.x) * kVec;
      DiagSeg s;
      s.row = -1;
#pragma unroll
      for (int k = 0; k < kDiagRowVals; ++k) s.v[k] = 0.f;
      if (i < c1) {
        float ov[4], sv[4], mv[4];
        if (i + kVec <= n_slots) {
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
        int r = rf.row(i);
        int64_t rend = rf.row_end(r);
        s.row = r;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int64_t p = i + j;
          if (p >= n_slots) break;
          if (p >= rend) {
            diag_flush(s, row_vals, n_rows);
            r = rf.row(p);
            rend = rf.row_end(r);
            s.row = r;
#pragma unroll
            for (int k = 0; k < kDiagRowVals; ++k) s.v[k] = 0.f;
          }
          const float m = mv[j];
          if (m == 0.f) continue;  // every quantity below is masked
          const float o = ov[j], sp = sv[j];
          const float lr = o - sp;
          // diagnostics tolerate the ~1e-6 relative error of the hardware exp2 path
          const float e = __expf(clampf3(lr, -kBound, kBound));
          const float eu = (lr >= -kBound && lr <= kBound) ? e : __expf(lr);
          const float pa = __expf(o), ps = __expf(sp);
          const float dp = fabsf(pa - ps), dl = fabsf(lr);
          const float rej = (lr >= rs_lr_lo && lr <= rs_lr_hi) ? 0.f : 1.f;
          const float ci = clampf3(e, is_lo, is_hi), cr = clampf3(e, rs_lo, rs_hi);
          a[0] += m;
          a[1] += e * m;
          a[2] += e * e * m;
          a[3] += lr * m;
          a[4] += (eu - lr - 1.f) * m;
          a[5] += (e > is_hi) ? m : 0.f;
          a[6] += (e < is_lo) ? m : 0.f;
          a[7] += ci * m;
          a[8] += ci * ci * m;
          a[9] += (e > rs_hi) ? m : 0.f;
          a[10] += (e < rs_lo) ? m : 0.f;
          a[11] += cr * m;
          a[12] += cr * cr * m;
          a[13] += dp;
          a[14] += dp * dp;
          a[15] += dl;
          a[16] += dl * dl;
          a[17] += pa;
          a[18] += ps;
          a[19] += pa * pa;
          a[20] += ps * ps;
          a[21] += pa * ps;
          a[22] += rej * m;
          mx[0] = fmaxf(mx[0], e);  mn[0] = fminf(mn[0], e);
          mx[1] = fmaxf(mx[1], dp); mn[1] = fminf(mn[1], dp);
          mx[2] = fmaxf(mx[2], dl); mn[2] = fminf(mn[2], dl);
          s.v[0] += m;
          s.v[1] += o * m;
          s.v[2] += sp * m;
          s.v[3] += lr * m;
          s.v[4] += e * m;
          s.v[5] += rej * m;
        }
      }
      diag_wave_reduce_flush(s, row_vals, n_rows);
    }
  }
  // workgroup partials: sums, then max/min pairs
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
#pragma unroll
  for (int k = 0; k < 3; ++k) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      mx[k] = fmaxf(mx[k], __shfl_down(mx[k], off, kWave));
      mn[k] = fminf(mn[k], __shfl_down(mn[k], off, kWave));
    }
    if (lane == 0) {
      lds_mm[wave * kDiagMinMax + 2 * k] = mx[k];
      lds_mm[wave * kDiagMinMax + 2 * k + 1] = mn[k];
    }
  }
  block_sum<kDiagSums>(a, lds_red);  // contains the barrier that also publishes lds_mm
  if (threadIdx.x == 0) {
    float* row = partials + (size_t)blockIdx.x * kDiagStride;
#pragma unroll
    for (int k = 0; k < kDiagSums; ++k) row[k] = a[k];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      float hi = -kInf, lo = kInf;
      for (int w = 0; w < kBlock / kWave; ++w) {
        hi = fmaxf(hi, lds_mm[w * kDiagMinMax + 2 * k]);
        lo = fminf(lo, lds_mm[w * kDiagMinMax + 2 * k + 1]);
      }
      row[kDiagSums + 2 * k] = hi;
      row[kDiagSums + 2 * k + 1] = lo;
    }
  }
}

// ---- pass 2 -------------------------------------------------------------------------------------
constexpr int kOutSums = 50;  // out[0..49]: sums (0..22 token-level, 23..49 row-level)
constexpr int kOutMM = 10;    // out[50..59]: maxima, out[60..69]: minima
constexpr int kDiagOut = 72;

struct DiagCfg {
  int is_mode, rs_mode;  // 0 off, 1 token, 2 sequence, 3 geometric (rs only)
  float is_lo, is_hi, rs_lo, rs_hi;                  // ratio thresholds
  float log_is_lo, log_is_hi, log_rs_lo, log_rs_hi;  // fp32 log of the same
};

__device__ __forceinline__ double wave_sum_d(double v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, kWave);
  return v;
}

// Four wavefronts per workgroup: what a wavefront spends here is mostly the 50 + 20 reductions at the end,
// which cost the same for one row per lane as for four, and sixteen wavefronts would queue four deep on a SIMD.
constexpr int kDiagRowThreads = 256;
// Workgroup b of the grid takes token partials b, b + gridDim.x, ... and rows likewise, and leaves its
// 70 sums / maxima / minima in out[b][kDiagOut]; sampler_diag_final_kernel folds the workgroups.
__global__ __launch_bounds__(kDiagRowThreads) void sampler_diag_rows_kernel(
    const float* __restrict__ partials, int n_blocks, const float* __restrict__ row_vals,
    int64_t n_rows, DiagCfg cfg, double* __restrict__ out_all) {
  double* out = out_all + (size_t)blockIdx.x * kDiagOut;
  __shared__ double red[kDiagRowThreads / kWave][kOutSums];
  __shared__ float red_mx[kDiagRowThreads / kWave][kOutMM], red_mn[kDiagRowThreads / kWave][kOutMM];
  const float kInf = __builtin_huge_valf();
  double acc[kOutSums];
#pragma unroll
  for (int k = 0; k < kOutSums; ++k) acc[k] = 0.0;
  float mx[kOutMM], mn[kOutMM];
#pragma unroll
  for (int k = 0; k < kOutMM; ++k) { mx[k] = -kInf; mn[k] = kInf; }

  // (a) token partials: sums -> acc[0..22]; (max, min) pairs -> slots 0..2
  for (int b = blockIdx.x * blockDim.x + threadIdx.x; b < n_blocks; b += gridDim.x * blockDim.x) {
    const float* row = partials + (size_t)b * kDiagStride;
#pragma unroll
    for (int k = 0; k < kDiagSums; ++k) acc[k] += (double)row[k];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
      mx[k] = fmaxf(mx[k], row[kDiagSums + 2 * k]);
      mn[k] = fminf(mn[k], row[kDiagSums + 2 * k + 1]);
    }
  }
  // (b) rows
  const float* cnt_a = row_vals;
  const float* so_a = row_vals + n_rows;
  const float* ss_a = row_vals + 2 * n_rows;
  const float* sl_a = row_vals + 3 * n_rows;
  const float* se_a = row_vals + 4 * n_rows;
  const float* sr_a = row_vals + 5 * n_rows;
  for (int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; r < n_rows;
       r += (int64_t)gridDim.x * blockDim.x) {
    const float cnt = cnt_a[r], s_lr = sl_a[r];
    const float den = cnt + 1e-8f;  // masked_mean over a row, axon/utils/torch/ops.py:131-145
    if (cfg.is_mode != 0) {
      float x;  // masked row mean of the untruncated weights (sampler.py:306-315)
      if (cfg.is_mode == 1) {
        x = se_a[r] / den;
      } else {  // sequence: one weight per row, exp(clamp(sum lr)) (sampler.py:213-217)
        const float w = expf(clampf3(s_lr, -kBound, kBound));
        const float ws = clampf3(w, cfg.is_lo, cfg.is_hi);
        x = w * cnt / den;
        mx[7] = fmaxf(mx[7], s_lr); mn[7] = fminf(mn[7], s_lr);
        acc[31] += (s_lr > cfg.log_is_hi) ? 1.0 : 0.0;
        acc[32] += (s_lr < cfg.log_is_lo) ? 1.0 : 0.0;
        acc[33] += (double)w * cnt;
        acc[34] += (double)ws * cnt;
        acc[35] += (double)ws * ws * cnt;
      }
      acc[23] += x;
      acc[24] += (double)x * x;
      acc[25] += (x > cfg.is_hi) ? 1.0 : 0.0;
      acc[26] += (x < cfg.is_lo) ? 1.0 : 0.0;
      mx[3] = fmaxf(mx[3], x); mn[3] = fminf(mn[3], x);
      mx[4] = fmaxf(mx[4], fabsf(x - 1.f));
    }
    if (cfg.rs_mode != 0) {
      float x;
      if (cfg.rs_mode == 1) {
        x = se_a[r] / den;
        acc[41] += (sr_a[r] > 0.f) ? 1.0 : 0.0;  // rows with a rejected valid token (sampler.py:96-97)
      } else {  // sequence: sum of lr; geometric: masked mean of lr (sampler.py:70-79)
        const float L = (cfg.rs_mode == 2) ? s_lr : s_lr / den;
        const float w = expf(clampf3(L, -kBound, kBound));
        const float ws = clampf3(w, cfg.rs_lo, cfg.rs_hi);
        x = w * cnt / den;
        mx[8] = fmaxf(mx[8], L); mn[8] = fminf(mn[8], L);
        acc[36] += (L > cfg.log_rs_hi) ? 1.0 : 0.0;
        acc[37] += (L < cfg.log_rs_lo) ? 1.0 : 0.0;
        acc[38] += (double)w * cnt;
        acc[39] += (double)ws * cnt;
        acc[40] += (double)ws * ws * cnt;
        acc[41] += (w >= cfg.rs_lo && w <= cfg.rs_hi) ? 0.0 : 1.0;  // rows rejected (sampler.py:99)
      }
      acc[27] += x;
      acc[28] += (double)x * x;
      acc[29] += (x > cfg.rs_hi) ? 1.0 : 0.0;
      acc[30] += (x < cfg.rs_lo) ? 1.0 : 0.0;
      mx[5] = fmaxf(mx[5], x); mn[5] = fminf(mn[5], x);
      mx[6] = fmaxf(mx[6], fabsf(x - 1.f));
    }
    // off-policy diagnostics (sampler.py:476-517)
    const float a = so_a[r] / den, b = ss_a[r] / den;  // masked row means of old / sampler log-probs
    const float d = b - a;
    acc[42] += (double)expf(-a);
    acc[43] += (double)(-a);
    acc[44] += (double)expf(-b);
    acc[45] += (double)(-b);
    acc[46] += (double)d;
    acc[47] += (double)fabsf(d);
    acc[48] += (double)expf(d);
    acc[49] += (double)expf(2.f * clampf3(s_lr, -kBound, kBound));
    mx[9] = fmaxf(mx[9], d); mn[9] = fminf(mn[9], d);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int k = 0; k < kOutSums; ++k) {
    const double v = wave_sum_d(acc[k]);
    if (lane == 0) red[wave][k] = v;
  }
#pragma unroll
  for (int k = 0; k < kOutMM; ++k) {
    float hi = mx[k], lo = mn[k];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      hi = fmaxf(hi, __shfl_down(hi, off, kWave));
      lo = fminf(lo, __shfl_down(lo, off, kWave));
    }
    if (lane == 0) { red_mx[wave][k] = hi; red_mn[wave][k] = lo; }
  }
  __syncthreads();
  const int n_waves = (int)(blockDim.x >> 6);
  for (int k = threadIdx.x; k < kOutSums; k += blockDim.x) {
    double v = 0.0;
    for (int w = 0; w < n_waves; ++w) v += red[w][k];
    out[k] = v;
  }
  for (int k = threadIdx.x; k < kOutMM; k += blockDim.x) {
    float hi = -kInf, lo = kInf;
    for (int w = 0; w < n_waves; ++w) { hi = fmaxf(hi, red_mx[w][k]); lo = fminf(lo, red_mn[w][k]); }
    out[kOutSums + k] = (double)hi;
    out[kOutSums + kOutMM + k] = (double)lo;
  }
}

// One workgroup folds the row pass's per-workgroup results: wavefront w takes outputs w, w + 16, ...,
// its lanes read the parts side by side (a serial walk over 128 parts would be 128 dependent loads).
// Fixed order: lane l adds parts l, l + 64, ..., then the wavefront's fixed tree.
__global__ __launch_bounds__(1024) void sampler_diag_final_kernel(const double* __restrict__ parts, int n_parts,
                                                                  double* __restrict__ out) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, n_waves = (int)(blockDim.x >> 6);
  const double kInf = (double)__builtin_huge_valf();
  for (int k = wave; k < kOutSums + 2 * kOutMM; k += n_waves) {
    const bool is_sum = k < kOutSums, is_max = !is_sum && k < kOutSums + kOutMM;
    double v = is_sum ? 0.0 : (is_max ? -kInf : kInf);
    for (int b = lane; b < n_parts; b += kWave) {
      const double x = parts[(size_t)b * kDiagOut + k];
      v = is_sum ? v + x : (is_max ? fmax(v, x) : fmin(v, x));
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const double x = __shfl_down(v, off, kWave);
      v = is_sum ? v + x : (is_max ? fmax(v, x) : fmin(v, x));
    }
    if (lane == 0) out[k] = v;
  }
}

}  // namespace axon

using namespace axon;

static inline int diag_row_blocks(int64_t n_rows, int64_t token_blocks) {
  const int64_t work = n_rows > token_blocks ? n_rows : token_blocks;
  const int64_t b = (work + 1023) / 1024;
  return (int)(b < 1 ? 1 : (b > 128 ? 128 : b));
}

extern "C" int64_t axon_sampler_diag_workspace_bytes(int64_t n_rows, int64_t n_slots) {
  if (n_rows < 0 || n_slots < 0) return AXON_ERR_ARG;
  const int64_t blocks = n_slots > 0 ? (int64_t)stream_grid(n_slots) : 1;
  // [6][n_rows] row sums (zero-filled by the caller), the per-workgroup token partials, then the
  // row pass's per-workgroup results (doubles, 8-byte aligned)
  const int64_t floats = kDiagRowVals * n_rows + blocks * kDiagStride;
  return ((floats + 1) / 2 * 2) * (int64_t)sizeof(float) +
         (int64_t)diag_row_blocks(n_rows, blocks) * kDiagOut * (int64_t)sizeof(double);
}

extern "C" int axon_sampler_diag(const float* oldp, const float* samp, const void* mask, int mask_kind,
                                 const int32_t* cu, int64_t n_rows, int64_t n_slots,
                                 int64_t uniform_len, int is_mode, float is_lo, float is_hi,
                                 int rs_mode, float rs_lo, float rs_hi, float rs_lr_lo,
                                 float rs_lr_hi, float log_is_lo, float log_is_hi, float log_rs_lo,
                                 float log_rs_hi, float* workspace, double* out, void* stream) {
  if (n_rows <= 0 || n_slots <= 0 || uniform_len < 0) return AXON_ERR_ARG;
  if (n_rows >= (int64_t)INT32_MAX || n_slots >= (int64_t)INT32_MAX) return AXON_ERR_SHAPE;
  if (uniform_len == 0 && cu == nullptr) return AXON_ERR_ARG;
  if (uniform_len > 0 && n_rows * uniform_len != n_slots) return AXON_ERR_SHAPE;
  if (!oldp || !samp || !mask || !workspace || !out) return AXON_ERR_ARG;
  if (reinterpret_cast<uintptr_t>(workspace) & 7) return AXON_ERR_WORKSPACE;
  if (is_mode < 0 || is_mode > 2 || rs_mode < 0 || rs_mode > 3) return AXON_ERR_ARG;
  if (mask_kind != AXON_MASK_F32 && mask_kind != AXON_MASK_I64) return AXON_ERR_ARG;
  float* row_vals = workspace;
  float* partials = workspace + kDiagRowVals * n_rows;
  const dim3 g(stream_grid(n_slots)), blk(kBlock);
  const hipStream_t st = (hipStream_t)stream;
  if (mask_kind == AXON_MASK_F32)
    hipLaunchKernelGGL(sampler_diag_tokens_kernel<AXON_MASK_F32>, g, blk, 0, st, oldp, samp, mask, cu,
                       n_rows, n_slots, uniform_len, is_lo, is_hi, rs_lo, rs_hi, rs_lr_lo, rs_lr_hi,
                       row_vals, partials);
  else
    hipLaunchKernelGGL(sampler_diag_tokens_kernel<AXON_MASK_I64>, g, blk, 0, st, oldp, samp, mask, cu,
                       n_rows, n_slots, uniform_len, is_lo, is_hi, rs_lo, rs_hi, rs_lr_lo, rs_lr_hi,
                       row_vals, partials);
  AXON_CHECK_LAUNCH();
  DiagCfg cfg;
  cfg.is_mode = is_mode; cfg.rs_mode = rs_mode;
  cfg.is_lo = is_lo; cfg.is_hi = is_hi; cfg.rs_lo = rs_lo; cfg.rs_hi = rs_hi;
  cfg.log_is_lo = log_is_lo; cfg.log_is_hi = log_is_hi;
  cfg.log_rs_lo = log_rs_lo; cfg.log_rs_hi = log_rs_hi;
  const int64_t floats = kDiagRowVals * n_rows + (int64_t)g.x * kDiagStride;
  double* parts = reinterpret_cast<double*>(workspace + (floats + 1) / 2 * 2);
  const int rb = diag_row_blocks(n_rows, g.x);
  hipLaunchKernelGGL(sampler_diag_rows_kernel, dim3(rb), dim3(kDiagRowThreads), 0, st, partials, (int)g.x, row_vals,
                     n_rows, cfg, parts);
  AXON_CHECK_LAUNCH();
  hipLaunchKernelGGL(sampler_diag_final_kernel, dim3(1), dim3(1024), 0, st, parts, rb, out);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}
