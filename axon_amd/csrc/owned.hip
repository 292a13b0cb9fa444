// Operators that need a per-sequence quantity before they can write a token, in ONE pass over HBM:
// GSPO's sequence ratio, the losses aggregated per row (token_reduce mean / mean-norm / mean-program,
// batch_reduce step-mean / program-mean), the per-sequence veto, and sequence-level / geometric
// importance weights and rejection.
//
// A workgroup owns WHOLE rows: range b covers the rows that begin in [b * kOwnStride,
// (b + 1) * kOwnStride), whatever their length.  It loads the tokens of its rows once (16 per thread,
// kept in registers), forms the per-row sums in LDS, and then writes the per-token outputs from the
// registers.  A range longer than the registers hold (a row of more than 2048 tokens in it) is
// walked in blocks of kOwnTokens and read a second time for the output pass (the re-read follows
// the first read within microseconds and is mostly served by the L2); the common case reads every
// input exactly once: 20 bytes per token for GSPO or the veto against 32 for a row pass followed by
// a token pass.
//
// The per-row sums are formed without atomics and in a fixed order: every wavefront adds the tokens
// it sees into its own slots in LDS (in program order), and the four wavefronts' slots are added
// 0 + 1 + 2 + 3.  The sequence ratio, the sequence-level masks and weights are therefore the same
// on every run.
#include "common.h"
#include "token_math.h"

namespace axon {

constexpr int kOwnStride = 2048;                      // tokens between the starts of two ranges
constexpr int kOwnIter = 4;                           // 16-byte vectors per thread per block
constexpr int kOwnTokens = kBlock * kVec * kOwnIter;  // tokens a workgroup holds in registers: 4096
constexpr int kOwnRows = 128;                         // rows whose sums fit the LDS tables at a time
constexpr int kOwnWaves = kBlock / kWave;
constexpr int kOwnBatch = 64;                         // ranges whose row boundaries are looked up together

struct RowStarts {
  const int32_t* cu;
  int64_t uniform, n_rows, n_slots;
  // first slot of row r (r in [0, n_rows]), clamped into [0, n_slots]
  __device__ __forceinline__ int64_t at(int64_t r) const {
    const int64_t v = uniform > 0 ? r * uniform : (int64_t)cu[r];
    return min(max(v, (int64_t)0), n_slots);
  }
  // smallest r in [0, n_rows) whose first slot is >= pos; n_rows when there is none
  __device__ int64_t first_row_from(int64_t pos) const {
    if (uniform > 0) return min((pos + uniform - 1) / uniform, n_rows);
    int64_t lo = 0, hi = n_rows;
    while (lo < hi) {
      const int64_t mid = (lo + hi) >> 1;
      if ((int64_t)cu[mid] >= pos) hi = mid; else lo = mid + 1;
    }
    return lo;
  }
};

// The rows [rs, re) of one segment: their starts in LDS, and the row of a slot by bisection.
struct Segment {
  const int32_t* win;  // LDS: win[i] = first slot of row rs + i, i in [0, n]
  int n;
  __device__ __forceinline__ int row_of(int p) const {  // largest i < n with win[i] <= p
    int a = 0, b = n - 1;
    while (a < b) {
      const int mid = (a + b + 1) >> 1;
      if (win[mid] <= p) a = mid; else b = mid - 1;
    }
    return a;
  }
  __device__ __forceinline__ int end_of(int i) const { return win[i + 1]; }
};

// Segmented sum across the wavefront (rows sorted across lanes, -1 = no token); `flush(seg)` is
// called once per run by its first lane.
template <int NV, class Flush>
__device__ __forceinline__ void row_seg_wave_reduce(RowSeg<NV> s, Flush&& flush) {
  const int lane = threadIdx.x & (kWave - 1);
  const int first = __builtin_amdgcn_readfirstlane(s.row);
  if (first >= 0 && __builtin_amdgcn_readlane(s.row, kWave - 1) == first) {
#pragma unroll
    for (int k = 0; k < NV; ++k) s.v[k] = wave_sum_to_last(s.v[k]);
    if (lane == kWave - 1) flush(s);
    return;
  }
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const int r2 = __shfl_down(s.row, off, kWave);
    float t[NV];
#pragma unroll
    for (int k = 0; k < NV; ++k) t[k] = __shfl_down(s.v[k], off, kWave);
    if (lane + off < kWave && r2 == s.row) {
#pragma unroll
      for (int k = 0; k < NV; ++k) s.v[k] += t[k];
    }
  }
  const int prev = __shfl_up(s.row, 1, kWave);
  if ((lane == 0 || prev != s.row) && s.row >= 0) flush(s);
}

// What the two kernels share: the walk over ranges, segments and blocks.  `Op` provides
//   load(p0, it)                   one vector of four slots starting at p0 into register set `it`
//   stat(it, j, RowSeg&)           add slot j of register set `it` to the row sums
//   rows(seg_first_row, i, tot[])  derive the per-row values of local row i from its sums (one thread)
//   emit(p0, it, ...)              write the outputs of one vector
// and kNV row sums.  Written as a macro-free template: the kernels below instantiate it.
template <class Op>
__device__ __forceinline__ void walk_owned_rows(const RowStarts& rs_, Op& op) {
  constexpr int NV = Op::kNV;
  __shared__ int32_t win[kOwnRows + 1];
  __shared__ float part[kOwnWaves][kOwnRows][NV];
  __shared__ int32_t bnd[kOwnBatch][2];
  const int wave = threadIdx.x / kWave;
  const int64_t n_ranges = (rs_.n_slots + kOwnStride - 1) / kOwnStride;
  // this workgroup's ranges: blockIdx.x, blockIdx.x + gridDim.x, ...
  const int64_t n_mine = (int64_t)blockIdx.x < n_ranges ? (n_ranges - blockIdx.x + gridDim.x - 1) / gridDim.x : 0;
#pragma unroll 1
  for (int64_t k0 = 0; k0 < n_mine; k0 += kOwnBatch) {
  // The first and last row of up to kOwnBatch ranges, found by as many threads at once: a bisection
  // over cu_seqlens is a chain of dependent loads, far too long to sit in front of every range.
  const int n_batch = (int)min((int64_t)kOwnBatch, n_mine - k0);
  __syncthreads();
  if ((int)threadIdx.x < 2 * n_batch) {
    const int64_t b = blockIdx.x + (k0 + (threadIdx.x >> 1)) * gridDim.x;
    int64_t r;
    if ((threadIdx.x & 1) == 0) r = (b == 0) ? 0 : rs_.first_row_from(b * kOwnStride);
    else r = (b == n_ranges - 1) ? rs_.n_rows : rs_.first_row_from((b + 1) * kOwnStride);
    bnd[threadIdx.x >> 1][threadIdx.x & 1] = (int32_t)r;
  }
  __syncthreads();
#pragma unroll 1
  for (int kb = 0; kb < n_batch; ++kb) {
    const int64_t b = blockIdx.x + (k0 + kb) * gridDim.x;
    const int64_t r0 = bnd[kb][0], r1 = bnd[kb][1];
#pragma unroll 1
    for (int64_t rs = r0; rs < r1; rs += kOwnRows) {
      const int n = (int)min((int64_t)kOwnRows, r1 - rs);
      __syncthreads();  // the tables of the previous segment are no longer read
      for (int i = threadIdx.x; i <= n; i += kBlock) win[i] = (int32_t)rs_.at(rs + i);
      for (int i = threadIdx.x; i < kOwnWaves * kOwnRows * NV; i += kBlock) (&part[0][0][0])[i] = 0.f;
      __syncthreads();
      const Segment seg{win, n};
      const int t0 = win[0], t1 = win[n];
      const int base = t0 & ~3;  // vectors stay 16-byte aligned; slots before t0 are not ours
      const int n_blocks = (t1 - base + kOwnTokens - 1) / kOwnTokens;
      // ---- pass 1: row sums.  The registers keep the last block that was loaded.
#pragma unroll 1
      for (int blk = 0; blk < n_blocks; ++blk) {
        const int b0 = base + blk * kOwnTokens;
#pragma unroll
        for (int it = 0; it < kOwnIter; ++it) {
          const int p0 = b0 + (it * kBlock + (int)threadIdx.x) * kVec;
          if (p0 < t1 && p0 + kVec > t0) op.load(p0, it);
        }
#pragma unroll
        for (int it = 0; it < kOwnIter; ++it) {
          const int p0 = b0 + (it * kBlock + (int)threadIdx.x) * kVec;
          RowSeg<NV> s;
          s.row = -1;
#pragma unroll
          for (int k = 0; k < NV; ++k) s.v[k] = 0.f;
          auto flush = [&](const RowSeg<NV>& f) {
#pragma unroll
            for (int k = 0; k < NV; ++k) part[wave][f.row][k] += f.v[k];
          };
          if (p0 < t1 && p0 + kVec > t0) {
            int rend = -1;
#pragma unroll
            for (int j = 0; j < kVec; ++j) {
              const int p = p0 + j;
              if (p < t0 || p >= t1) continue;
              if (p >= rend) {
                if (s.row >= 0) flush(s);
                s.row = seg.row_of(p);
                rend = seg.end_of(s.row);
#pragma unroll
                for (int k = 0; k < NV; ++k) s.v[k] = 0.f;
              }
              op.stat(it, j, s);
            }
          }
          row_seg_wave_reduce<NV>(s, flush);
        }
      }
      __syncthreads();
      // ---- the rows of the segment: sums of the four wavefronts in a fixed order -> derived values
      for (int i = threadIdx.x; i < n; i += kBlock) {
        float tot[NV];
#pragma unroll
        for (int k = 0; k < NV; ++k) tot[k] = ((part[0][i][k] + part[1][i][k]) + part[2][i][k]) + part[3][i][k];
        op.rows(rs + i, i, tot);
      }
      __syncthreads();
      // ---- pass 2: outputs, last block first (its inputs are still in the registers)
#pragma unroll 1
      for (int blk = n_blocks - 1; blk >= 0; --blk) {
        const int b0 = base + blk * kOwnTokens;
        if (blk != n_blocks - 1) {
#pragma unroll
          for (int it = 0; it < kOwnIter; ++it) {
            const int p0 = b0 + (it * kBlock + (int)threadIdx.x) * kVec;
            if (p0 < t1 && p0 + kVec > t0) op.load(p0, it);
          }
        }
#ifdef AXON_EXP_LATE
#pragma unroll
        for (int it = 0; it < kOwnIter; ++it) {
          const int p0 = b0 + (it * kBlock + (int)threadIdx.x) * kVec;
          if (p0 < t1 && p0 + kVec > t0) op.load_late(p0, it);
        }
#endif
#pragma unroll
        for (int it = 0; it < kOwnIter; ++it) {
          const int p0 = b0 + (it * kBlock + (int)threadIdx.x) * kVec;
          if (p0 < t1 && p0 + kVec > t0) op.emit(p0, it, seg, t0, t1);
        }
      }
    }
    // slots outside every row (before the first row's start, after the last row's end) belong to no
    // sequence: the first and the last range write zeros there
    if (b == 0) op.fill_gap(0, rs_.at(0));
    if (b == n_ranges - 1) op.fill_gap(rs_.at(rs_.n_rows), rs_.n_slots);
  }
  }
}

// four slots starting at p0 (p0 % 4 == 0): one 16-byte load when all four exist
__device__ __forceinline__ void load4_guard(const float* p, int64_t p0, int64_t n_slots, float (&v)[4]) {
  if (p0 + kVec <= n_slots) { load4(p, p0, v); return; }
#pragma unroll
  for (int j = 0; j < kVec; ++j) v[j] = (p0 + j < n_slots) ? p[p0 + j] : 0.f;
}
template <int MK>
__device__ __forceinline__ void load_mask4_guard(const void* mask, int64_t p0, int64_t n_slots, float (&m)[4]) {
  if (p0 + kVec <= n_slots) { load_mask4<MK>(mask, p0, m); return; }
#pragma unroll
  for (int j = 0; j < kVec; ++j) m[j] = (p0 + j < n_slots) ? load_mask1<MK>(mask, p0 + j) : 0.f;
}
// write the slots of the vector that belong to [t0, t1): one 16-byte store when all four do
__device__ __forceinline__ void store4_range(float* out, int64_t p0, int64_t t0, int64_t t1, const float (&v)[4]) {
  if (p0 >= t0 && p0 + kVec <= t1) { store4(out, p0, v); return; }
#pragma unroll
  for (int j = 0; j < kVec; ++j)
    if (p0 + j >= t0 && p0 + j < t1) out[p0 + j] = v[j];
}
__device__ __forceinline__ void zero_range(float* out, int64_t a, int64_t b) {
  for (int64_t p = a + threadIdx.x; p < b; p += kBlock) out[p] = 0.f;
}

// ---------------------------------------------------------------------------------------------
// policy losses with a per-row quantity
// ---------------------------------------------------------------------------------------------
struct OwnedLossArgs {
  const float *logp, *oldp, *adv, *isw;
  const void* mask;
  int token_reduce, batch_reduce;  // as in axon_loss_row_scale
  const double *prtc, *npt, *nps, *valid;
  float lo, hi, clip_c;
  float* grad;
};

template <int MK, int KIND>
struct OwnedLossOp {
  static constexpr int kNV = 2;  // sum mask, sum (logp - old) * mask
  const OwnedLossArgs& g;
  const RowStarts& rs;
  float (*rowv)[2];  // LDS [kOwnRows]: scale, mean log-ratio
  float bden;        // the batch denominator when the caller supplied it
  float lv[kOwnIter][4], ov[kOwnIter][4], mv[kOwnIter][4], av[kOwnIter][4], wv[kOwnIter][4];
  float a[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float rows_with_tokens = 0.f;

  __device__ __forceinline__ OwnedLossOp(const OwnedLossArgs& g_, const RowStarts& rs_, float (*rowv_)[2], float bd)
      : g(g_), rs(rs_), rowv(rowv_), bden(bd) {}

  __device__ __forceinline__ void load(int p0, int it) {
    load4_guard(g.logp, p0, rs.n_slots, lv[it]);
    load4_guard(g.oldp, p0, rs.n_slots, ov[it]);
    load_mask4_guard<MK>(g.mask, p0, rs.n_slots, mv[it]);
#ifndef AXON_EXP_LATE
    load_late(p0, it);
#endif
  }
  // read by the output pass only
  __device__ __forceinline__ void load_late(int p0, int it) {
    load4_guard(g.adv, p0, rs.n_slots, av[it]);
    if (g.isw) load4_guard(g.isw, p0, rs.n_slots, wv[it]);
    else wv[it][0] = wv[it][1] = wv[it][2] = wv[it][3] = 1.f;
  }
  __device__ __forceinline__ void stat(int it, int j, RowSeg<2>& s) const {
    const float m = mv[it][j];
    s.v[0] += m;
    // masked sum: values outside the mask never reach it (NaN / Inf in padding)
    s.v[1] += (m != 0.f) ? (lv[it][j] - ov[it][j]) * m : 0.f;
  }
  __device__ __forceinline__ void rows(int64_t r, int i, const float (&tot)[2]) {
    const float c = tot[0];
    float td = 1.f;
    if (g.token_reduce == 1) td = fmaxf(g.prtc ? (float)g.prtc[r] : c, 1.f);
    if (g.token_reduce == 2) td = (float)rs.uniform;
    if (g.token_reduce == 3) td = fmaxf((float)g.npt[r], 1.f);
    if (g.batch_reduce == 2) td *= fmaxf((float)g.nps[r], 1.f);
    // with the batch denominator known this is the scale of the two-pass path, 1 / (td * bden)
    rowv[i][0] = (g.valid != nullptr) ? 1.f / (td * bden) : 1.f / td;
    rowv[i][1] = tot[1] / fmaxf(c, 1.f);
    rows_with_tokens += (c > 0.f) ? 1.f : 0.f;
  }
  __device__ __forceinline__ void emit(int p0, int it, const Segment& seg, int t0, int t1) {
    float gv[4];
    int rend = -1;
    float scale = 0.f, sbar = 0.f;
#pragma unroll
    for (int j = 0; j < kVec; ++j) {
      const int p = p0 + j;
      gv[j] = 0.f;
      if (p < t0 || p >= t1) continue;
      if (p >= rend) {
        const int i = seg.row_of(p);
        rend = seg.end_of(i);
        scale = rowv[i][0];
        sbar = rowv[i][1];
      }
      const TokenTerm t =
          policy_token<KIND>(lv[it][j], ov[it][j], av[it][j], wv[it][j], sbar, g.lo, g.hi, g.clip_c, false);
      gv[j] = accumulate_token(t, mv[it][j], scale, a);
    }
    store4_range(g.grad, p0, t0, t1, gv);
  }
  __device__ __forceinline__ void fill_gap(int64_t a0, int64_t b0) { zero_range(g.grad, a0, b0); }
};

template <int MK, int KIND>
__global__ __launch_bounds__(kBlock) void owned_policy_loss_kernel(OwnedLossArgs g, RowStarts rs, float* ws,
                                                                   float* __restrict__ acc) {
  __shared__ float rowv[kOwnRows][2];
  __shared__ float lds_red[kPartialStride * (kBlock / kWave)];
  // a caller-supplied batch denominator (utils.py:224-229) is known before the first token
  const float bden = (g.valid != nullptr) ? fmaxf((float)g.valid[0], 1.f) : 1.f;
  OwnedLossOp<MK, KIND> op(g, rs, rowv, bden);
  walk_owned_rows(rs, op);
  float part[7] = {op.a[0], op.a[1], op.a[2], op.a[3], op.a[4], 0.f, op.rows_with_tokens};
  const int batch_reduce = g.batch_reduce;
  const bool known = (g.valid != nullptr);
  grid_finish<7>(part, lds_red, ws, [&](float (&tot)[kPartialStride]) {
    // without a supplied denominator the sums were formed without it: token-mean divides by the
    // number of mask tokens, step-mean by the number of rows that have one (utils.py:236-251); the
    // gradient array is left without that division and acc[5] carries the factor
    float factor = 1.f;
    if (!known) {
      const float den = fmaxf(batch_reduce == 0 ? tot[4] : tot[6], 1.f);
      factor = 1.f / den;
      tot[0] = tot[0] / den;
    }
    tot[5] = factor;
    for (int k = 0; k < kPartialStride; ++k) acc[k] = tot[k];
  });
}

// ---------------------------------------------------------------------------------------------
// sampler / trainer correction with a per-row quantity (veto, sequence or geometric level)
// ---------------------------------------------------------------------------------------------
struct OwnedCorrArgs {
  const float *oldp, *samp;
  const void* mask;
  CorrCfg cfg;
  float *isw, *new_mask;
  float *row_cnt, *row_sum;  // optional per-row outputs (the sums the decisions were taken from)
  int32_t* row_flag;         // optional: 1 where the row was vetoed
};

template <int MK>
struct OwnedCorrOp {
  static constexpr int kNV = 3;  // sum mask, sum (old - sampler) * mask, tokens under the veto threshold
  const OwnedCorrArgs& g;
  const RowStarts& rs;
  CorrRow* rowv;  // LDS [kOwnRows]
  float ov[kOwnIter][4], sv[kOwnIter][4], mv[kOwnIter][4];
  float a[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float vetoed_rows = 0.f;

  __device__ __forceinline__ OwnedCorrOp(const OwnedCorrArgs& g_, const RowStarts& rs_, CorrRow* rowv_)
      : g(g_), rs(rs_), rowv(rowv_) {}

  __device__ __forceinline__ void load(int p0, int it) {
    load4_guard(g.oldp, p0, rs.n_slots, ov[it]);
    load4_guard(g.samp, p0, rs.n_slots, sv[it]);
    load_mask4_guard<MK>(g.mask, p0, rs.n_slots, mv[it]);
  }
  __device__ __forceinline__ void load_late(int, int) {}
  __device__ __forceinline__ void stat(int it, int j, RowSeg<3>& s) const {
    const float m = mv[it][j];
    const float d = ov[it][j] - sv[it][j];
    s.v[0] += m;
    s.v[1] += (m != 0.f) ? d * m : 0.f;
    s.v[2] += (g.cfg.has_veto && m != 0.f && d < g.cfg.log_veto) ? 1.f : 0.f;
  }
  __device__ __forceinline__ void rows(int64_t r, int i, const float (&tot)[3]) {
    const bool vetoed = tot[2] > 0.f;
    rowv[i] = corr_row(g.cfg, tot[1], tot[0], vetoed);
    vetoed_rows += (g.cfg.has_veto && vetoed) ? 1.f : 0.f;
    if (g.row_cnt) g.row_cnt[r] = tot[0];
    if (g.row_sum) g.row_sum[r] = tot[1];
    if (g.row_flag) g.row_flag[r] = vetoed ? 1 : 0;
  }
  __device__ __forceinline__ void emit(int p0, int it, const Segment& seg, int t0, int t1) {
    float wv[4], nm[4];
    int rend = -1;
    CorrRow row{0.f, 1.f, 1.f};
#pragma unroll
    for (int j = 0; j < kVec; ++j) {
      const int p = p0 + j;
      wv[j] = 0.f;
      nm[j] = 0.f;
      if (p < t0 || p >= t1) continue;
      if (p >= rend) {
        const int i = seg.row_of(p);
        rend = seg.end_of(i);
        row = rowv[i];
      }
      corr_token(g.cfg, row, ov[it][j], sv[it][j], mv[it][j], wv[j], nm[j], a);
    }
    if (g.isw) store4_range(g.isw, p0, t0, t1, wv);
    store4_range(g.new_mask, p0, t0, t1, nm);
  }
  __device__ __forceinline__ void fill_gap(int64_t a0, int64_t b0) {
    if (g.isw) zero_range(g.isw, a0, b0);
    zero_range(g.new_mask, a0, b0);
  }
};

template <int MK>
__global__ __launch_bounds__(kBlock) void owned_correction_kernel(OwnedCorrArgs g, RowStarts rs, float* ws,
                                                                  float* __restrict__ acc) {
  __shared__ CorrRow rowv[kOwnRows];
  __shared__ float lds_red[kPartialStride * (kBlock / kWave)];
  OwnedCorrOp<MK> op(g, rs, rowv);
  walk_owned_rows(rs, op);
  float part[6] = {op.a[0], op.a[1], op.a[2], op.a[3], op.vetoed_rows, op.a[5]};
  grid_finish<6>(part, lds_red, ws, [&](float (&tot)[kPartialStride]) {
    for (int k = 0; k < kPartialStride; ++k) acc[k] = tot[k];
  });
}

}  // namespace axon

using namespace axon;

namespace {

// one resident wave of workgroups per launch keeps the number of partial rows small; the ranges are
// short (2048 tokens), so the walk balances itself
unsigned owned_grid(int64_t n_slots) {
  const int64_t ranges = (n_slots + kOwnStride - 1) / kOwnStride;
  return (unsigned)(ranges < kStreamGridCap ? ranges : kStreamGridCap);
}

int check_owned_rows(const int32_t* cu, int64_t n_rows, int64_t n_slots, int64_t uniform_len) {
  if (n_rows < 0 || n_slots < 0 || uniform_len < 0) return AXON_ERR_ARG;
  if (n_rows >= (int64_t)INT32_MAX || n_slots >= (int64_t)INT32_MAX - kOwnTokens) return AXON_ERR_SHAPE;
  if (uniform_len == 0 && cu == nullptr && n_slots > 0) return AXON_ERR_ARG;
  if (uniform_len > 0 && n_rows * uniform_len != n_slots) return AXON_ERR_SHAPE;
  if (uniform_len == 0 && n_rows == 0 && n_slots > 0) return AXON_ERR_SHAPE;  // slots without rows
  return AXON_OK;
}

}  // namespace

extern "C" int axon_policy_loss_rows(int kind, const float* logp, const float* oldp, const float* adv,
                                     const void* mask, int mask_kind, const float* isw, const int32_t* cu,
                                     int64_t n_rows, int64_t n_slots, int64_t uniform_len, int token_reduce,
                                     int batch_reduce, const double* prtc, const double* npt, const double* nps,
                                     const double* valid, float ratio_lo, float ratio_hi, float clip_c,
                                     float* grad, float* acc, float* partials, void* stream) {
  int rc = check_owned_rows(cu, n_rows, n_slots, uniform_len);
  if (rc != AXON_OK) return rc;
  if (n_slots == 0) return AXON_OK;
  if (kind < 0 || kind > 4) return AXON_ERR_ARG;
  if (!logp || !oldp || !adv || !mask || !grad || !acc || !partials) return AXON_ERR_ARG;
  if (token_reduce < 0 || token_reduce > 3 || batch_reduce < 0 || batch_reduce > 2) return AXON_ERR_ARG;
  if (token_reduce == 3 && !npt) return AXON_ERR_ARG;
  if (token_reduce == 2 && uniform_len <= 0) return AXON_ERR_ARG;
  if (batch_reduce == 2 && (!nps || !valid)) return AXON_ERR_ARG;
  if (mask_kind != AXON_MASK_F32 && mask_kind != AXON_MASK_I64) return AXON_ERR_ARG;
  const OwnedLossArgs g{logp, oldp, adv, isw, mask, token_reduce, batch_reduce, prtc, npt, nps, valid,
                        ratio_lo, ratio_hi, clip_c, grad};
  const RowStarts rs{cu, uniform_len, n_rows, n_slots};
  const dim3 grid(owned_grid(n_slots)), blk(kBlock);
  const hipStream_t st = (hipStream_t)stream;
#define AXON_LAUNCH_OWNED(MK, KD) \
  hipLaunchKernelGGL((owned_policy_loss_kernel<MK, KD>), grid, blk, 0, st, g, rs, partials, acc)
  if (mask_kind == AXON_MASK_F32) {
    if (kind == 0) AXON_LAUNCH_OWNED(AXON_MASK_F32, 0);
    else if (kind == 1) AXON_LAUNCH_OWNED(AXON_MASK_F32, 1);
    else if (kind == 2) AXON_LAUNCH_OWNED(AXON_MASK_F32, 2);
    else if (kind == 3) AXON_LAUNCH_OWNED(AXON_MASK_F32, 3);
    else AXON_LAUNCH_OWNED(AXON_MASK_F32, 4);
  } else {
    if (kind == 0) AXON_LAUNCH_OWNED(AXON_MASK_I64, 0);
    else if (kind == 1) AXON_LAUNCH_OWNED(AXON_MASK_I64, 1);
    else if (kind == 2) AXON_LAUNCH_OWNED(AXON_MASK_I64, 2);
    else if (kind == 3) AXON_LAUNCH_OWNED(AXON_MASK_I64, 3);
    else AXON_LAUNCH_OWNED(AXON_MASK_I64, 4);
  }
#undef AXON_LAUNCH_OWNED
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

extern "C" int axon_sampler_correction_rows(const float* oldp, const float* samp, const void* mask, int mask_kind,
                                            const int32_t* cu, int64_t n_rows, int64_t n_slots,
                                            int64_t uniform_len, int is_mode, float is_thr, int rs_mode,
                                            float rs_lo, float rs_hi, int has_veto, float log_veto, float* isw,
                                            float* new_mask, float* row_cnt, float* row_sum, int32_t* row_flag,
                                            float* acc, float* partials, void* stream) {
  int rc = check_owned_rows(cu, n_rows, n_slots, uniform_len);
  if (rc != AXON_OK) return rc;
  if (n_slots == 0) return AXON_OK;
  if (!oldp || !samp || !mask || !new_mask || !acc || !partials) return AXON_ERR_ARG;
  if (is_mode < 0 || is_mode > 2 || rs_mode < 0 || rs_mode > 3) return AXON_ERR_ARG;
  if (is_mode != 0 && isw == nullptr) return AXON_ERR_ARG;
  if (mask_kind != AXON_MASK_F32 && mask_kind != AXON_MASK_I64) return AXON_ERR_ARG;
  const OwnedCorrArgs g{oldp, samp, mask, CorrCfg{is_mode, is_thr, rs_mode, rs_lo, rs_hi, has_veto, log_veto},
                        isw, new_mask, row_cnt, row_sum, row_flag};
  const RowStarts rs{cu, uniform_len, n_rows, n_slots};
  const dim3 grid(owned_grid(n_slots)), blk(kBlock);
  if (mask_kind == AXON_MASK_F32)
    hipLaunchKernelGGL(owned_correction_kernel<AXON_MASK_F32>, grid, blk, 0, (hipStream_t)stream, g, rs,
                       partials, acc);
  else
    hipLaunchKernelGGL(owned_correction_kernel<AXON_MASK_I64>, grid, blk, 0, (hipStream_t)stream, g, rs,
                       partials, acc);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}
