// Shared device helpers for the stage-2/3 kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/axon_amd.h"

namespace axon {

constexpr int kWave = 64;
constexpr int kBlock = 256;           // threads per workgroup for streaming kernels
constexpr int kVec = 4;               // tokens per thread per step (one 16-byte load)
constexpr int kIter = 4;              // steps per thread
constexpr int kChunk = kBlock * kVec * kIter;  // tokens per workgroup
constexpr int kLdsRows = 2048;        // cu_seqlens window cached in LDS per workgroup

#define AXON_CHECK_LAUNCH()                                   \
  do {                                                        \
    if (hipGetLastError() != hipSuccess) return AXON_ERR_LAUNCH; \
  } while (0)

constexpr float kSafetyBound = 20.0f;  // axon/utils/rl/sampler.py:27, loss.py:77

__device__ __forceinline__ float clampf(float x, float lo, float hi) {
  // torch.clamp semantics: NaN propagates
  return (x != x) ? x : fminf(fmaxf(x, lo), hi);
}

// expf for an argument already clamped into [-20, 20] (or NaN, which propagates): the same steps and
// the same bits as expf's (product with log2 e in two parts, round to nearest integer, 2^fraction,
// scale by 2^integer) without its tests for overflow and underflow, five instructions fewer per token.
__device__ __forceinline__ float exp_bounded(float x) {
  constexpr float kLog2eHi = 0x1.715476p+0f, kLog2eLo = 0x1.4ae0bep-26f;
  const float t = x * kLog2eHi;
  float e = fmaf(x, kLog2eHi, -t);
  const float n = rintf(t);
  e = fmaf(x, kLog2eLo, e);
  return ldexpf(__builtin_amdgcn_exp2f((t - n) + e), (int)n);
}

// State of a top-k selection over 32-bit keys (largest keys win; key 0 never wins).  A token i is
// selected when key > threshold, or key == threshold and i < index_limit (ties go to the lowest indices).
struct SelectState {
  uint32_t threshold;    // key of the k-th largest element, built 11 + 11 + 10 bits at a time
  uint32_t remaining;    // how many elements with the current prefix are still to be taken
  uint32_t candidates;   // non-zero keys
  uint32_t ties;         // elements equal to the threshold
  int64_t index_limit;   // -1 while a tie pass still has to find it
  float mean_a, mean_b;  // the centring constants of the covariance
  float count;           // sum of the mask (weighted) or number of tokens with mask > 0
  uint32_t k;            // elements to select
};

__device__ __forceinline__ bool select_hit(const SelectState& s, uint32_t key, int64_t i) {
  if (s.k == 0 || key == 0) return false;
  return key > s.threshold || (key == s.threshold && i < s.index_limit);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, kWave);
  return v;
}

// Sum over the wavefront by DPP row shifts and broadcasts (no LDS traffic); the total lands in lane 63.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float v) {
  const float moved = __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, false));
  return v + moved;
}
__device__ __forceinline__ float wave_sum_to_last(float v) {
  v = dpp_add<0x111, 0xf>(v);  // row_shr:1
  v = dpp_add<0x112, 0xf>(v);  // row_shr:2
  v = dpp_add<0x114, 0xf>(v);  // row_shr:4
  v = dpp_add<0x118, 0xf>(v);  // row_shr:8
  v = dpp_add<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
  v = dpp_add<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
  return v;
}

// Sum NV values over the workgroup; the total lands in thread 0.
template <int NV>
__device__ __forceinline__ void block_sum(float (&v)[NV], float* lds /* [NV * 4] */) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
#pragma unroll
  for (int i = 0; i < NV; ++i) v[i] = wave_sum(v[i]);
  if (lane == 0) {
#pragma unroll
    for (int i = 0; i < NV; ++i) lds[wave * NV + i] = v[i];
  }
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      float s = 0.f;
      for (int w = 0; w < kBlock / kWave; ++w) s += lds[w * NV + i];
      v[i] = s;
    }
  }
}

// Grid-wide sums without same-address atomics: a streaming kernel runs at most kMaxStreamBlocks
// workgroups, each walking chunks blockIdx.x, blockIdx.x + gridDim.x, ... and leaving its NV
// partial sums in partials[blockIdx.x][8].  They are added in a fixed order, so results are
// reproducible: either inside the launch (grid_finish below) or by a small kernel launched next on
// the same stream (store_block_partials + a finishing kernel).
constexpr int kMaxStreamBlocks = 16384;  // one chunk per workgroup up to 2^26 tokens
constexpr int kPartialStride = 8;
constexpr int kFinishGroup = 64;         // workgroups whose rows one wavefront adds
constexpr int kMaxFinishGroups = kMaxStreamBlocks / kFinishGroup;  // 256: one workgroup adds the group rows
// workspace of grid_finish: rows, group rows, then the ticket counters (one per group, one for the grid)
constexpr int64_t kGroupRowsOffset = (int64_t)kMaxStreamBlocks * kPartialStride;                    // in floats
constexpr int64_t kTicketsOffset = kGroupRowsOffset + (int64_t)kMaxFinishGroups * kPartialStride;  // in floats
constexpr int64_t kTicketBytes = 2048;  // 257 counters
constexpr int64_t kPartialsBytes = kTicketsOffset * 4 + kTicketBytes;

template <int NV>
__device__ __forceinline__ void store_block_partials(float (&v)[NV], float* lds /* [NV * 4] */,
                                                     float* partials) {
  static_assert(NV <= kPartialStride, "partials row too small");
  block_sum<NV>(v, lds);
  if (threadIdx.x == 0) {
    float* row = partials + (size_t)blockIdx.x * kPartialStride;
#pragma unroll
    for (int k = 0; k < kPartialStride; ++k) row[k] = (k < NV) ? v[k < NV ? k : 0] : 0.f;
  }
}

// One row of eight floats to the level all XCDs share, then a ticket: true for the caller that draws
// the last of `n` tickets.  The row goes out with agent-scope stores, which write through; waiting
// for their acknowledgement orders them before the ticket.  (A release fence would also write back
// every dirty line of this XCD's L2, the kernel's own output stream included, once per workgroup:
// +35 % kernel time at 2^26 tokens.)  What this relies on in the hardware: a store at agent scope is
// acknowledged (vmcnt) only once it has reached the memory level that all XCDs of the device share, so a
// reader on another XCD that sees the ticket afterwards and drops its own cached copies (the acquire fence
// in grid_finish) reads the new values.  For the compiler the relaxed atomics carry no order of their own:
// the two signal fences pin the row's stores before the wait and the ticket after it.
__device__ __forceinline__ bool publish_row_take_ticket(float* row, const float (&v)[kPartialStride],
                                                        unsigned* ticket, unsigned n) {
#pragma unroll
  for (int k = 0; k < kPartialStride; ++k)
    __hip_atomic_store(row + k, v[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0)
  __atomic_signal_fence(__ATOMIC_SEQ_CST);
  const unsigned t = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (t != n - 1) return false;
  __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // ready for the next launch
  return true;
}

// The sums finished inside the launch, in two levels.  Every workgroup publishes its row and takes a
// ticket of its group of kFinishGroup workgroups; the workgroup that draws a group's last ticket adds
// the group's rows (one wavefront: lane l takes row l, then the fixed tree of wave_sum), publishes
// the group row and takes a ticket of the grid; the workgroup that draws the last of those adds the
// group rows (thread t takes group t, then the fixed tree of block_sum) and hands the eight totals
// to `fin` in its thread 0.  The order of every addition is fixed by the grid size alone.  The
// counters must be zero when the kernel starts and are zero again when it ends.
template <int NV, class Fin>
__device__ __forceinline__ void grid_finish(float (&v)[NV], float* lds /* [8 * 4] */, float* ws,
                                            Fin&& fin) {
  static_assert(NV <= kPartialStride, "partials row too small");
  __shared__ int s_stage;
  unsigned* tickets = reinterpret_cast<unsigned*>(ws + kTicketsOffset);
  const unsigned group = blockIdx.x / kFinishGroup;
  const unsigned n_groups = (gridDim.x + kFinishGroup - 1) / kFinishGroup;
  const unsigned first = group * kFinishGroup;
  const unsigned in_group = min((unsigned)kFinishGroup, gridDim.x - first);
  block_sum<NV>(v, lds);
  if (threadIdx.x == 0) {
    float row[kPartialStride];
#pragma unroll
    for (int k = 0; k < kPartialStride; ++k) row[k] = (k < NV) ? v[k < NV ? k : 0] : 0.f;
    s_stage = publish_row_take_ticket(ws + (size_t)blockIdx.x * kPartialStride, row, tickets + 1 + group,
                                      in_group) ? 1 : 0;
  }
  __syncthreads();
  if (s_stage == 0) return;
  // every row of the group was acknowledged at the shared level before its ticket was drawn; drop
  // what this XCD's caches may still hold of those addresses (an earlier launch), then read them
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  if (threadIdx.x < kWave) {
    float t[kPartialStride];
    const bool ok = threadIdx.x < in_group;
    const float* row = ws + (size_t)(first + (ok ? threadIdx.x : 0)) * kPartialStride;
    const float4 lo4 = *reinterpret_cast<const float4*>(row), hi4 = *reinterpret_cast<const float4*>(row + 4);
    t[0] = ok ? lo4.x : 0.f; t[1] = ok ? lo4.y : 0.f; t[2] = ok ? lo4.z : 0.f; t[3] = ok ? lo4.w : 0.f;
    t[4] = ok ? hi4.x : 0.f; t[5] = ok ? hi4.y : 0.f; t[6] = ok ? hi4.z : 0.f; t[7] = ok ? hi4.w : 0.f;
#pragma unroll
    for (int k = 0; k < kPartialStride; ++k) t[k] = wave_sum(t[k]);
    if (threadIdx.x == 0)
      s_stage = publish_row_take_ticket(ws + kGroupRowsOffset + (size_t)group * kPartialStride, t, tickets,
                                        n_groups) ? 2 : 1;
  }
  __syncthreads();
  if (s_stage != 2) return;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  float t[kPartialStride];
  {
    const bool ok = threadIdx.x < n_groups;  // n_groups <= kBlock
    const float* row = ws + kGroupRowsOffset + (size_t)(ok ? threadIdx.x : 0) * kPartialStride;
    const float4 lo4 = *reinterpret_cast<const float4*>(row), hi4 = *reinterpret_cast<const float4*>(row + 4);
    t[0] = ok ? lo4.x : 0.f; t[1] = ok ? lo4.y : 0.f; t[2] = ok ? lo4.z : 0.f; t[3] = ok ? lo4.w : 0.f;
    t[4] = ok ? hi4.x : 0.f; t[5] = ok ? hi4.y : 0.f; t[6] = ok ? hi4.z : 0.f; t[7] = ok ? hi4.w : 0.f;
  }
  block_sum<kPartialStride>(t, lds);  // the barriers above separate this use of `lds` from the first
  if (threadIdx.x == 0) fin(t);
}

// Workgroups of a streaming launch: beyond this many chunks a workgroup walks several (every
// workgroup publishes a row of partial sums and takes a ticket when it ends, which costs more than
// the walk; 6144 measured best between 1024 and 16384 at 2^26 tokens).
constexpr int kStreamGridCap = 6144;
inline unsigned stream_grid(int64_t n_slots) {
  const int64_t chunks = (n_slots + kChunk - 1) / kChunk;
  return (unsigned)(chunks < kStreamGridCap ? chunks : kStreamGridCap);
}

// 16-byte streaming accesses.  Every input of these kernels is read once and every output
// written once, so loads and stores carry the non-temporal hint (measured +12 % on a
// 4-read / 1-write stream of 2^26 tokens).
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef long long i64x2 __attribute__((ext_vector_type(2)));

// Mask loads: four consecutive slots as floats.
template <int KIND>
__device__ __forceinline__ void load_mask4(const void* mask, int64_t i, float (&m)[4]) {
  if (mask == nullptr) {
    m[0] = m[1] = m[2] = m[3] = 1.f;
  } else if (KIND == AXON_MASK_F32) {
    const f32x4 v = __builtin_nontemporal_load(
        reinterpret_cast<const f32x4*>(static_cast<const float*>(mask) + i));
    m[0] = v.x; m[1] = v.y; m[2] = v.z; m[3] = v.w;
  } else {
    const i64x2* p = reinterpret_cast<const i64x2*>(static_cast<const int64_t*>(mask) + i);
    const i64x2 a = __builtin_nontemporal_load(p), b = __builtin_nontemporal_load(p + 1);
    m[0] = (float)a.x; m[1] = (float)a.y; m[2] = (float)b.x; m[3] = (float)b.y;
  }
}
template <int KIND>
__device__ __forceinline__ float load_mask1(const void* mask, int64_t i) {
  if (mask == nullptr) return 1.f;
  if (KIND == AXON_MASK_F32) return static_cast<const float*>(mask)[i];
  return (float)static_cast<const int64_t*>(mask)[i];
}

__device__ __forceinline__ void load4(const float* p, int64_t i, float (&v)[4]) {
  const f32x4 x = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p + i));
  v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
}
__device__ __forceinline__ void store4(float* p, int64_t i, const float (&v)[4]) {
  const f32x4 x = {v[0], v[1], v[2], v[3]};
  __builtin_nontemporal_store(x, reinterpret_cast<f32x4*>(p + i));
}

// Per-row sums of NV values from a token-parallel kernel: a lane folds its slots into a RowSeg,
// the wave runs a segmented shuffle reduction keyed by row id (row ids are non-decreasing across
// lanes) and the first lane of each run adds the run total to row_vals[k][row] with one atomic.
template <int NV>
struct RowSeg {
  int row;
  float v[NV];
};

template <int NV>
__device__ __forceinline__ void row_seg_flush(const RowSeg<NV>& s, float* row_vals, int64_t n_rows) {
  if (s.row < 0) return;
#pragma unroll
  for (int k = 0; k < NV; ++k)
    if (s.v[k] != 0.f) atomicAdd(row_vals + (int64_t)k * n_rows + s.row, s.v[k]);
}

template <int NV>
__device__ __forceinline__ void row_seg_wave_reduce_flush(RowSeg<NV> s, float* row_vals, int64_t n_rows) {
  const int lane = threadIdx.x & (kWave - 1);
  // the common case: the whole wavefront sits in one row (rows are sorted across lanes)
  const int first = __builtin_amdgcn_readfirstlane(s.row);
  if (first >= 0 && __builtin_amdgcn_readlane(s.row, kWave - 1) == first) {
#pragma unroll
    for (int k = 0; k < NV; ++k) s.v[k] = wave_sum_to_last(s.v[k]);
    if (lane == kWave - 1) row_seg_flush(s, row_vals, n_rows);
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
  if (lane == 0 || prev != s.row) row_seg_flush(s, row_vals, n_rows);
}

// Row lookup.  row(pos) = number of s in [1, n_rows] with cu[s] <= pos, i.e. the
// row whose half-open range contains pos; empty rows are skipped.  A workgroup
// owns the contiguous slots [c0, c1); it caches the cu_seqlens entries covering
// that range in LDS when they fit.
struct RowFinder {
  const int32_t* cu;   // global
  const int32_t* win;  // LDS window or nullptr
  int lo;              // first row overlapping the chunk
  int hi;              // last row overlapping the chunk
  int64_t uniform;

  // count of s in (lo_excl, hi_incl] with p[s] <= pos, searching global memory
  __device__ static int upper(const int32_t* cu, int lo, int hi, int64_t pos) {
    // invariant: cu[lo] <= pos (or lo == 0), answer in [lo, hi]
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if ((int64_t)cu[mid] <= pos) lo = mid; else hi = mid - 1;
    }
    return lo;
  }

  // the same count with three probes per step (their loads are independent): half as many dependent loads
  __device__ static int upper4(const int32_t* cu, int lo, int hi, int64_t pos) {
    while (hi - lo >= 4) {
      const int q = (hi - lo) >> 2;
      const int m1 = lo + q, m2 = lo + 2 * q, m3 = lo + 3 * q;
      const bool b1 = (int64_t)cu[m1] <= pos, b2 = (int64_t)cu[m2] <= pos, b3 = (int64_t)cu[m3] <= pos;
      if (b3) lo = m3;
      else if (b2) { lo = m2; hi = m3 - 1; }
      else if (b1) { lo = m1; hi = m2 - 1; }
      else hi = m1 - 1;
    }
    return upper(cu, lo, hi, pos);
  }

  __device__ void init(const int32_t* cu_, int64_t n_rows, int64_t uniform_len, int64_t c0,
                       int64_t c1, int32_t* lds) {
    cu = cu_;
    uniform = uniform_len;
    win = nullptr;
    if (uniform_len > 0) return;
    lo = upper4(cu, 0, (int)n_rows, c0);
    // the chunk's last row is a few rows on: gallop from lo, then search the bracket
    int step = 1, top = lo;
    while (top < (int)n_rows) {
      const int probe = min(top + step, (int)n_rows);
      if ((int64_t)cu[probe] > c1 - 1) { hi = upper(cu, top, probe - 1, c1 - 1); break; }
      top = probe;
      step *= 2;
    }
    if (top >= (int)n_rows) hi = (int)n_rows;
    if (lo >= n_rows) lo = (int)n_rows - 1;  // slots past cu[n_rows] (caller error) stay in range
    if (hi >= n_rows) hi = (int)n_rows - 1;
    const int n = hi - lo + 2;
    if (n <= kLdsRows) {
      for (int i = threadIdx.x; i < n; i += blockDim.x) lds[i] = cu[lo + i];
      win = lds;
    }
    __syncthreads();
  }

  __device__ __forceinline__ int row(int64_t pos) const {
    if (uniform > 0) return (int)(pos / uniform);
    if (win != nullptr) {
      int a = 0, b = hi - lo;
      while (a < b) {
        const int mid = (a + b + 1) >> 1;
        if ((int64_t)win[mid] <= pos) a = mid; else b = mid - 1;
      }
      return lo + a;
    }
    return upper(cu, lo, hi, pos);
  }
  // first slot of the row after `r` (to test whether a 4-vector stays in one row)
  __device__ __forceinline__ int64_t row_end(int r) const {
    if (uniform > 0) return (int64_t)(r + 1) * uniform;
    if (win != nullptr) return win[r - lo + 1];
    return cu[r + 1];
  }
};

}  // namespace axon
