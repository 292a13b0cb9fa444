// Operators that need a per-sequence quantity before they can write a token, in ONE pass over HBM:
// GSPO's sequence ratio, the losses aggregated per row (token_reduce mean / mean-norm / mean-program,
// batch_reduce step-mean / program-mean), the per-sequence veto, and sequence-level / geometric
// importance weights and rejection.
//
// A WORKGROUP owns whole rows.  The slots are cut into as many ranges of `stride` tokens as the
// launch has workgroups (all resident at once); workgroup b takes the rows that BEGIN in range b,
// whatever their length, so every workgroup has the same number of tokens up to one row.  A row is
// walked in chunks of 1024 slots (16 bytes per thread), kRowHold chunks (2048 slots) per wait: the
// row sums are formed across the workgroup, the per-row values derived from them, and the
// per-token outputs written from the registers.  A row of more than 2048 slots is read a second
// time for the output pass, all but its last group: its first read goes without the streaming hint,
// so that the second finds the lines in the L2.  The common case reads every input exactly once:
// 20 bytes per token for GSPO or the veto against 32 for a row pass followed by a token pass.  The
// first group of the next row is requested before the current row is worked on (two banks of two
// chunks in registers), as a fixed number of loads in straight-line code: the compiler then waits
// for the current row's loads by count and leaves the next row's in flight.
//
// The per-row sums are formed without atomics and in a fixed order (a thread adds its slots chunk
// by chunk, then the fixed tree of the wavefront sum, then the four wavefronts 0 + 1 + 2 + 3), so
// the sequence ratio, the sequence-level masks and weights are the same on every run.
#include <type_traits>

#include "common.h"
#include "token_math.h"

namespace axon {

constexpr int kRowChunk = kBlock * kVec;  // slots one workgroup instruction covers: 1024
constexpr int kRowHold = 2;               // chunks of a row kept in registers
constexpr int kOwnWaves = kBlock / kWave;

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

// first_row_from by the whole wavefront: every step probes 64 evenly spaced rows (three dependent loads
// for 10^5 rows instead of seventeen).  The same value in every lane.
__device__ __forceinline__ int first_row_from_wave(const RowStarts& rs, int64_t pos, int lane) {
  if (rs.uniform > 0) return (int)rs.first_row_from(pos);
  int lo = 0, hi = (int)rs.n_rows;  // the answer lies in [lo, hi]
  while (hi > lo) {
    const int step = (hi - lo + kWave - 1) / kWave;
    const int idx = lo + lane * step;
    const bool ge = idx >= hi || (int64_t)rs.cu[idx] >= pos;
    const unsigned long long m = __ballot(ge);
    if (m == 0ull) {  // every probed row begins before pos
      lo = lo + (kWave - 1) * step + 1;
    } else {
      const int f = __builtin_ctzll(m);
      hi = min(hi, lo + f * step);
      if (f > 0) lo = lo + (f - 1) * step + 1;
    }
  }
  return lo;
}

__device__ __forceinline__ float wave_total(float v) {  // the same value in every lane
  v = wave_sum_to_last(v);
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), kWave - 1));
}

// What the two kernels share: the walk over ranges, rows and chunks.  `Op` provides
//   kNV                               number of row sums
//   load(p0, b, c)                    the vector of four slots starting at p0 into register set (b, c) (every input):
//                                     a fixed number of 16-byte loads, p0 + 4 <= n_slots
//   load_edge(p0, b, c)               the same for a vector that may reach beyond the last slot
//   stat(b, c, j, s[])                add slot j of register set (b, c) to the thread's row sums
//   rows(r, tot[], first) -> RowVals  the per-row values from the row's sums (every thread the same)
//   emit(p0, b, c, rv, t0, t1)        write the outputs of the vector in register set (b, c)
//   fill_gap(a, b)                    zeros for slots that belong to no row
// Two banks of register sets: while a step (a row, or two short ones) is worked on in one bank, the
// first group of the next step is already on its way into the other, so its loads have a whole
// step's time to arrive.  Every thread of the workgroup walks the same rows (the loop bounds are
// uniform), so the barrier inside the loop is reached by all; it waits for LDS only, not for the
// loads in flight.
template <class Op>
__device__ __forceinline__ void walk_owned_rows(const RowStarts& rs, int stride, Op& op) {
  constexpr int NV = Op::kNV;
  __shared__ float red[2][kOwnWaves][kRowHold * NV];
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int n_rows = (int)rs.n_rows;
  const int64_t n_ranges = (rs.n_slots + stride - 1) / stride;  // <= workgroups of the launch
  // this workgroup's rows: those that begin in [blockIdx.x * stride, range_end).  Only the first is
  // looked up (by every wavefront, to the same result); the walk ends at the first row that begins
  // beyond the range.
  const int64_t range_end = ((int64_t)blockIdx.x >= n_ranges - 1) ? INT64_MAX : ((int64_t)blockIdx.x + 1) * stride;
  int r = n_rows;
  if ((int64_t)blockIdx.x < n_ranges)
    r = (blockIdx.x == 0) ? 0 : first_row_from_wave(rs, (int64_t)blockIdx.x * stride, lane);
  // row starts, 64 at a time: lane l holds the start of row win0 + l (of row n_rows: the end of the last)
  int win0 = r;
  int win = (int)rs.at(min((int64_t)win0 + lane, rs.n_rows));
  // [t0, t1) of row rr; false when the walk ends before it
  auto fetch = [&](int rr, int& t0, int& t1) -> bool {
    if (rr >= n_rows) return false;
    if (rr - win0 >= kWave - 1) {
      win0 = rr;
      win = (int)rs.at(min((int64_t)win0 + lane, rs.n_rows));
    }
    const int k = __builtin_amdgcn_readfirstlane(rr - win0);
    t0 = __builtin_amdgcn_readlane(win, k);
    t1 = __builtin_amdgcn_readlane(win, k + 1);
    return (int64_t)t0 < range_end;
  };
  // With a slot count that is no multiple of four the last vector is incomplete: `tail_p0` is its
  // first slot (none: -1) and `last_full` the last vector that can be read with one 16-byte load.
  const int n4 = (int)(rs.n_slots & ~(int64_t)3);
  const int tail_p0 = (n4 < rs.n_slots) ? n4 : -1;
  const int last_full = max(n4 - kVec, 0);  // n_slots >= 4 (the host's check)
  // What one step of the walk works on: row r = [a0, a1) and, when that row and the next one fit a
  // chunk each, the next row [b0, b1) beside it (`pair`): the second chunk of the registers would
  // otherwise idle through every short row.  Uniform across the workgroup.
  static_assert(kRowHold == 2, "a step pairs two one-chunk rows in the two chunks of a bank");
  struct Span { int r, a0, a1, b0, b1; bool valid, pair; };
  auto chunks_of = [](int t0, int t1) { return (t1 > t0) ? (t1 - (t0 & ~3) + kRowChunk - 1) / kRowChunk : 0; };
  auto span_at = [&](int rr) -> Span {
    Span sp{rr, 0, 0, 0, 0, false, false};
    int t0 = 0, t1 = 0;
    sp.valid = fetch(rr, t0, t1);
    if (!sp.valid) return sp;
    sp.a0 = t0;
    sp.a1 = t1;
    if (chunks_of(t0, t1) <= 1 && fetch(rr + 1, t0, t1) && chunks_of(t0, t1) <= 1) {
      sp.pair = true;
      sp.b0 = t0;
      sp.b1 = t1;
    }
    return sp;
  };
  // Chunk c of group grp of a span: this thread's vector p0 and the row [t0, t1) it is part of.
  auto unit = [&](const Span& sp, int c, int grp, int& p0, int& t0, int& t1) {
    const bool other = (c == 1) && sp.pair;
    t0 = other ? sp.b0 : sp.a0;
    t1 = other ? sp.b1 : sp.a1;
    p0 = (t0 & ~3) + (int)threadIdx.x * kVec + (other ? 0 : (grp * kRowHold + c) * kRowChunk);  // 16-byte aligned
  };
  // The first group of a span into bank B, as a FIXED number of loads in straight-line code: a vector
  // beyond the row's end is requested at the row's last vector instead (one cache line for the whole
  // wavefront, never used).  A load under a condition would leave the compiler unable to count the
  // loads in flight behind the ones it waits for, and every wait would drain the prefetch as well.
  auto prefetch = [&](auto bank, const Span& sp) {
    constexpr int B = decltype(bank)::value;
    int p0[kRowHold];
#pragma unroll
    for (int c = 0; c < kRowHold; ++c) {
      int t0, t1;
      unit(sp, c, 0, p0[c], t0, t1);
      p0[c] = min(p0[c], min(max(t1 - 1, t0) & ~3, last_full));
    }
    // a row of several groups comes back to this one for its outputs: both arms issue the same loads
    if (sp.a1 - (sp.a0 & ~3) > kRowHold * kRowChunk) {
#pragma unroll
      for (int c = 0; c < kRowHold; ++c) op.template load<true>(p0[c], B, c);
    } else {
#pragma unroll
      for (int c = 0; c < kRowHold; ++c) op.template load<false>(p0[c], B, c);
    }
  };
  // The incomplete last vector of the arrays, when the first group of the span holds it: one thread of
  // the launch reads it slot by slot, and waits at once so that the compiler's count of the loads in
  // flight stays what it is on the path without this block.
  auto fetch_tail = [&](auto bank, const Span& sp) {
    constexpr int B = decltype(bank)::value;
    if (tail_p0 < 0) return;
#pragma unroll
    for (int c = 0; c < kRowHold; ++c) {
      int p0, t0, t1;
      unit(sp, c, 0, p0, t0, t1);
      if (p0 == tail_p0 && tail_p0 < t1) {
        op.template load_edge<false>(tail_p0, B, c);
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
      }
    }
  };
  // a later group of a long row (or an earlier one again, for the output pass)
  auto load_group = [&](auto bank, const Span& sp, int grp, bool keep) {
    constexpr int B = decltype(bank)::value;
#pragma unroll
    for (int c = 0; c < kRowHold; ++c) {
      int p0, t0, t1;
      unit(sp, c, grp, p0, t0, t1);
      if (p0 < t1 && p0 + kVec > t0) {
        if (keep) op.template load_edge<true>(p0, B, c);
        else op.template load_edge<false>(p0, B, c);
      }
    }
  };
  int parity = 0;
  // one span in bank B; its first group has been requested; `nxt` is the next span (not valid: none)
  auto step = [&](auto bank, const Span& sp, const Span& nxt) {
    constexpr int B = decltype(bank)::value;
    prefetch(std::integral_constant<int, B ^ 1>{}, nxt);
    const int n_groups = max((chunks_of(sp.a0, sp.a1) + kRowHold - 1) / kRowHold, 1);
    float s[kRowHold][NV];  // the sums of the chunks apart: two rows, or the two halves of one
#pragma unroll
    for (int c = 0; c < kRowHold; ++c)
#pragma unroll
      for (int i = 0; i < NV; ++i) s[c][i] = 0.f;
    auto stat_group = [&](int grp) {
#pragma unroll
      for (int c = 0; c < kRowHold; ++c) {
        int p0, t0, t1;
        unit(sp, c, grp, p0, t0, t1);
        if (p0 >= t0 && p0 + kVec <= t1) {  // the whole vector belongs to the row
#pragma unroll
          for (int j = 0; j < kVec; ++j) op.stat(B, c, j, s[c]);
        } else if (p0 < t1 && p0 + kVec > t0) {
#pragma unroll
          for (int j = 0; j < kVec; ++j)
            if (p0 + j >= t0 && p0 + j < t1) op.stat(B, c, j, s[c]);
        }
      }
    };
    auto emit_unit = [&](int c, int grp, const typename Op::RowVals& rv) {
      int p0, t0, t1;
      unit(sp, c, grp, p0, t0, t1);
      if (p0 < t1 && p0 + kVec > t0) op.emit(p0, B, c, rv, t0, t1);
    };
    // ---- pass 1: the rows' sums.  The first group is in flight since the previous step (straight-line
    // code up to its first use, so the wait leaves the prefetch alone); a long row fetches the others
    // one wait at a time and the registers keep the last.
    fetch_tail(bank, sp);
    stat_group(0);
#pragma unroll 1
    for (int grp = 1; grp < n_groups; ++grp) {
      load_group(bank, sp, grp, grp < n_groups - 1);
      stat_group(grp);
    }
#pragma unroll
    for (int c = 0; c < kRowHold; ++c)
#pragma unroll
      for (int i = 0; i < NV; ++i) s[c][i] = wave_total(s[c][i]);
    if (lane == 0) {
#pragma unroll
      for (int c = 0; c < kRowHold; ++c)
#pragma unroll
        for (int i = 0; i < NV; ++i) red[parity][wave][c * NV + i] = s[c][i];
    }
    __syncthreads();  // one barrier per step: the next step writes the other half of `red`
    float tot[kRowHold][NV];
#pragma unroll
    for (int c = 0; c < kRowHold; ++c)
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int k = c * NV + i;
        tot[c][i] = ((red[parity][0][k] + red[parity][1][k]) + red[parity][2][k]) + red[parity][3][k];
      }
    parity ^= 1;
    if (!sp.pair) {
#pragma unroll
      for (int i = 0; i < NV; ++i) tot[0][i] += tot[1][i];
    }
    auto rv = op.rows(sp.r, tot[0], threadIdx.x == 0);
    // ---- pass 2: outputs, last group first (its inputs are still in the registers)
    emit_unit(0, n_groups - 1, rv);
    if (sp.pair) rv = op.rows(sp.r + 1, tot[1], threadIdx.x == 0);
    emit_unit(1, n_groups - 1, rv);
#pragma unroll 1
    for (int grp = n_groups - 2; grp >= 0; --grp) {
      load_group(bank, sp, grp, false);
      emit_unit(0, grp, rv);
      emit_unit(1, grp, rv);
    }
  };
  using Bank0 = std::integral_constant<int, 0>;
  using Bank1 = std::integral_constant<int, 1>;
  Span cur = span_at(r);
  if (cur.valid) prefetch(Bank0{}, cur);
#pragma unroll 1
  while (cur.valid) {
    const Span nxt = span_at(cur.r + (cur.pair ? 2 : 1));
    step(Bank0{}, cur, nxt);
    if (!nxt.valid) break;
    cur = span_at(nxt.r + (nxt.pair ? 2 : 1));
    step(Bank1{}, nxt, cur);
  }
  // slots outside every row (before the first row's start, after the last row's end) belong to no
  // sequence: one workgroup writes zeros there
  if (blockIdx.x == 0) {
    op.fill_gap(0, rs.at(0));
    op.fill_gap(rs.at(rs.n_rows), rs.n_slots);
  }
}

// Loads of the row walk.  KEEP: the vector will be read a second time soon (a group of a long row that
// the output pass comes back to), so it is requested without the streaming hint and stays in the L2.
template <bool KEEP>
__device__ __forceinline__ void row_load4(const float* p, int64_t i, float (&v)[4]) {
  const f32x4* q = reinterpret_cast<const f32x4*>(p + i);
  const f32x4 x = KEEP ? *q : __builtin_nontemporal_load(q);
  v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
}
// the mask is known to be there: no branch around the loads
template <int MK, bool KEEP>
__device__ __forceinline__ void row_load_mask4(const void* mask, int64_t i, float (&m)[4]) {
  if (MK == AXON_MASK_F32) {
    row_load4<KEEP>(static_cast<const float*>(mask), i, m);
  } else {
    const i64x2* p = reinterpret_cast<const i64x2*>(static_cast<const int64_t*>(mask) + i);
    const i64x2 a = KEEP ? p[0] : __builtin_nontemporal_load(p), b = KEEP ? p[1] : __builtin_nontemporal_load(p + 1);
    m[0] = (float)a.x; m[1] = (float)a.y; m[2] = (float)b.x; m[3] = (float)b.y;
  }
}
// four slots starting at p0 (p0 % 4 == 0): one 16-byte load when all four exist
template <bool KEEP>
__device__ __forceinline__ void row_load4_guard(const float* p, int64_t p0, int64_t n_slots, float (&v)[4]) {
  if (p0 + kVec <= n_slots) { row_load4<KEEP>(p, p0, v); return; }
#pragma unroll
  for (int j = 0; j < kVec; ++j) v[j] = (p0 + j < n_slots) ? p[p0 + j] : 0.f;
}
template <int MK, bool KEEP>
__device__ __forceinline__ void row_load_mask4_guard(const void* mask, int64_t p0, int64_t n_slots, float (&m)[4]) {
  if (p0 + kVec <= n_slots) { row_load_mask4<MK, KEEP>(mask, p0, m); return; }
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

// HAS_W: importance weights are given (their loads are part of the fixed count of a step's loads, so the
// two cases are two kernels and not a branch)
template <int MK, int KIND, bool HAS_W>
struct OwnedLossOp {
  static constexpr int kNV = 2;  // sum mask, sum (logp - old) * mask
  struct RowVals { float scale, sbar; Ratio seq; };  // seq: GSPO's ratio of the sequence (KIND 1)
  const OwnedLossArgs& g;
  const RowStarts& rs;
  float bden;  // the batch denominator when the caller supplied it
  float lv[2][kRowHold][4], ov[2][kRowHold][4], mv[2][kRowHold][4], av[2][kRowHold][4], wv[2][kRowHold][4];
  float a[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float rows_with_tokens = 0.f;

  __device__ __forceinline__ OwnedLossOp(const OwnedLossArgs& g_, const RowStarts& rs_, float bd)
      : g(g_), rs(rs_), bden(bd) {}

  template <bool KEEP>
  __device__ __forceinline__ void load(int p0, int b, int c) {
    row_load4<KEEP>(g.logp, p0, lv[b][c]);
    row_load4<KEEP>(g.oldp, p0, ov[b][c]);
    row_load_mask4<MK, KEEP>(g.mask, p0, mv[b][c]);
    // read by the output pass only, requested with the rest so that one wait covers all
    row_load4<KEEP>(g.adv, p0, av[b][c]);
    if (HAS_W) row_load4<KEEP>(g.isw, p0, wv[b][c]);
  }
  template <bool KEEP>
  __device__ __forceinline__ void load_edge(int p0, int b, int c) {
    row_load4_guard<KEEP>(g.logp, p0, rs.n_slots, lv[b][c]);
    row_load4_guard<KEEP>(g.oldp, p0, rs.n_slots, ov[b][c]);
    row_load_mask4_guard<MK, KEEP>(g.mask, p0, rs.n_slots, mv[b][c]);
    row_load4_guard<KEEP>(g.adv, p0, rs.n_slots, av[b][c]);
    if (HAS_W) row_load4_guard<KEEP>(g.isw, p0, rs.n_slots, wv[b][c]);
  }
  __device__ __forceinline__ void stat(int b, int c, int j, float (&s)[2]) const {
    const float m = mv[b][c][j];
    s[0] += m;
    // masked sum: values outside the mask never reach it (NaN / Inf in padding)
    s[1] += (m != 0.f) ? (lv[b][c][j] - ov[b][c][j]) * m : 0.f;
  }
  __device__ __forceinline__ RowVals rows(int64_t r, const float (&tot)[2], bool first) {
    const float c = tot[0];
    float td = 1.f;
    if (g.token_reduce == 1) td = fmaxf(g.prtc ? (float)g.prtc[r] : c, 1.f);
    if (g.token_reduce == 2) td = (float)rs.uniform;
    if (g.token_reduce == 3) td = fmaxf((float)g.npt[r], 1.f);
    if (g.batch_reduce == 2) td *= fmaxf((float)g.nps[r], 1.f);
    rows_with_tokens += (first && c > 0.f) ? 1.f : 0.f;
    // with the batch denominator known this is the scale of the two-pass path, 1 / (td * bden)
    RowVals rv{(g.valid != nullptr) ? 1.f / (td * bden) : 1.f / td, tot[1] / fmaxf(c, 1.f), Ratio{}};
    // GSPO's ratio is the same for every token of the sequence: the exponential once per row
    if (KIND == 1) rv.seq = ratio_of(0.f + rv.sbar, g.lo, g.hi);
    return rv;
  }
  __device__ __forceinline__ void emit(int p0, int b, int c, const RowVals& rv, int t0, int t1) {
    const bool whole = p0 >= t0 && p0 + kVec <= t1;
    float gv[4];
#pragma unroll
    for (int j = 0; j < kVec; ++j) {
      const int p = p0 + j;
      gv[j] = 0.f;
      if (!whole && (p < t0 || p >= t1)) continue;
      const float w = HAS_W ? wv[b][c][j] : 1.f;
      const TokenTerm t = (KIND == 1) ? gspo_token(rv.seq, lv[b][c][j], ov[b][c][j], av[b][c][j], w, g.clip_c)
                                      : policy_token<KIND>(lv[b][c][j], ov[b][c][j], av[b][c][j], w, rv.sbar, g.lo,
                                                           g.hi, g.clip_c, false);
      gv[j] = accumulate_token(t, mv[b][c][j], rv.scale, a);
    }
    store4_range(g.grad, p0, t0, t1, gv);
  }
  __device__ __forceinline__ void fill_gap(int64_t a0, int64_t b0) { zero_range(g.grad, a0, b0); }
};

template <int MK, int KIND, bool HAS_W>
// four workgroups per CU: the kernel is bound by the latencies of a step, which only other steps hide
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(4))) void owned_policy_loss_kernel(OwnedLossArgs g, RowStarts rs, int stride,
                                                                   float* ws, float* __restrict__ acc) {
  __shared__ float lds_red[kPartialStride * (kBlock / kWave)];
  // a caller-supplied batch denominator (utils.py:224-229) is known before the first token
  const float bden = (g.valid != nullptr) ? fmaxf((float)g.valid[0], 1.f) : 1.f;
  OwnedLossOp<MK, KIND, HAS_W> op(g, rs, bden);
  walk_owned_rows(rs, stride, op);
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
  typedef CorrRow RowVals;
  const OwnedCorrArgs& g;
  const RowStarts& rs;
  float ov[2][kRowHold][4], sv[2][kRowHold][4], mv[2][kRowHold][4];
  float a[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float vetoed_rows = 0.f;

  __device__ __forceinline__ OwnedCorrOp(const OwnedCorrArgs& g_, const RowStarts& rs_) : g(g_), rs(rs_) {}

  template <bool KEEP>
  __device__ __forceinline__ void load(int p0, int b, int c) {
    row_load4<KEEP>(g.oldp, p0, ov[b][c]);
    row_load4<KEEP>(g.samp, p0, sv[b][c]);
    row_load_mask4<MK, KEEP>(g.mask, p0, mv[b][c]);
  }
  template <bool KEEP>
  __device__ __forceinline__ void load_edge(int p0, int b, int c) {
    row_load4_guard<KEEP>(g.oldp, p0, rs.n_slots, ov[b][c]);
    row_load4_guard<KEEP>(g.samp, p0, rs.n_slots, sv[b][c]);
    row_load_mask4_guard<MK, KEEP>(g.mask, p0, rs.n_slots, mv[b][c]);
  }
  __device__ __forceinline__ void stat(int b, int c, int j, float (&s)[3]) const {
    const float m = mv[b][c][j];
    const float d = ov[b][c][j] - sv[b][c][j];
    s[0] += m;
    s[1] += (m != 0.f) ? d * m : 0.f;
    s[2] += (g.cfg.has_veto && m != 0.f && d < g.cfg.log_veto) ? 1.f : 0.f;
  }
  __device__ __forceinline__ RowVals rows(int64_t r, const float (&tot)[3], bool first) {
    const bool vetoed = tot[2] > 0.f;
    vetoed_rows += (first && g.cfg.has_veto && vetoed) ? 1.f : 0.f;
    if (first) {
      if (g.row_cnt) g.row_cnt[r] = tot[0];
      if (g.row_sum) g.row_sum[r] = tot[1];
      if (g.row_flag) g.row_flag[r] = vetoed ? 1 : 0;
    }
    return corr_row(g.cfg, tot[1], tot[0], vetoed);
  }
  __device__ __forceinline__ void emit(int p0, int b, int c, const RowVals& row, int t0, int t1) {
    const bool whole = p0 >= t0 && p0 + kVec <= t1;
    float wv[4], nm[4];
#pragma unroll
    for (int j = 0; j < kVec; ++j) {
      const int p = p0 + j;
      wv[j] = 0.f;
      nm[j] = 0.f;
      if (!whole && (p < t0 || p >= t1)) continue;
      corr_token(g.cfg, row, ov[b][c][j], sv[b][c][j], mv[b][c][j], wv[j], nm[j], a);
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
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(4))) void owned_correction_kernel(OwnedCorrArgs g, RowStarts rs, int stride,
                                                                  float* ws, float* __restrict__ acc) {
  __shared__ float lds_red[kPartialStride * (kBlock / kWave)];
  OwnedCorrOp<MK> op(g, rs);
  walk_owned_rows(rs, stride, op);
  float part[6] = {op.a[0], op.a[1], op.a[2], op.a[3], op.vetoed_rows, op.a[5]};
  grid_finish<6>(part, lds_red, ws, [&](float (&tot)[kPartialStride]) {
    for (int k = 0; k < kPartialStride; ++k) acc[k] = tot[k];
  });
}

}  // namespace axon

using namespace axon;

namespace {

// Ranges and workgroups of a launch: one range per workgroup, as many workgroups as are resident at
// once (a workgroup that had to wait for a free slot would start its range late), ranges of at
// least one chunk.
struct OwnedLaunch {
  int stride;
  unsigned grid;
};
template <typename K>
int resident_blocks(K kernel) {  // 0 when the runtime cannot say
  int dev = 0, cus = 0, per_cu = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(kernel), kBlock, 0) !=
      hipSuccess)
    return 0;
  return cus * per_cu;
}
OwnedLaunch owned_launch(int64_t n_slots, int resident) {
  const int64_t max_blocks = resident > 0 ? resident : 1024;
  int64_t stride = (n_slots + max_blocks - 1) / max_blocks;
  stride = (stride + kVec - 1) / kVec * kVec;
  if (stride < kRowChunk) stride = kRowChunk;
  return OwnedLaunch{(int)stride, (unsigned)((n_slots + stride - 1) / stride)};
}

int check_owned_rows(const int32_t* cu, int64_t n_rows, int64_t n_slots, int64_t uniform_len) {
  if (n_rows < 0 || n_slots < 0 || uniform_len < 0) return AXON_ERR_ARG;
  // 32-bit positions: a chunk past the last slot and a search step past the last row must still fit
  if (n_rows >= (int64_t)INT32_MAX - kWave || n_slots >= (int64_t)INT32_MAX - 4 * kRowChunk) return AXON_ERR_SHAPE;
  // the kernels read whole 16-byte vectors wherever one fits: fewer than four slots is the other path's case
  if (n_slots > 0 && n_slots < kVec) return AXON_ERR_SHAPE;
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
  // 16-byte vector accesses at every multiple of four slots: the token arrays must start on 16-byte boundaries
  if ((reinterpret_cast<uintptr_t>(logp) | reinterpret_cast<uintptr_t>(oldp) | reinterpret_cast<uintptr_t>(adv) |
       reinterpret_cast<uintptr_t>(mask) | reinterpret_cast<uintptr_t>(isw) | reinterpret_cast<uintptr_t>(grad)) & 15)
    return AXON_ERR_ARG;
  if (token_reduce < 0 || token_reduce > 3 || batch_reduce < 0 || batch_reduce > 2) return AXON_ERR_ARG;
  if (token_reduce == 3 && !npt) return AXON_ERR_ARG;
  if (token_reduce == 2 && uniform_len <= 0) return AXON_ERR_ARG;
  if (batch_reduce == 2 && (!nps || !valid)) return AXON_ERR_ARG;
  if (mask_kind != AXON_MASK_F32 && mask_kind != AXON_MASK_I64) return AXON_ERR_ARG;
  const OwnedLossArgs g{logp, oldp, adv, isw, mask, token_reduce, batch_reduce, prtc, npt, nps, valid,
                        ratio_lo, ratio_hi, clip_c, grad};
  const RowStarts rs{cu, uniform_len, n_rows, n_slots};
  const hipStream_t st = (hipStream_t)stream;
#define AXON_LAUNCH_OWNED_W(MK, KD, HW)                                                                   \
  do {                                                                                                  \
    static const int resident = resident_blocks(owned_policy_loss_kernel<MK, KD, HW>);                  \
    const OwnedLaunch ol = owned_launch(n_slots, resident);                                             \
    hipLaunchKernelGGL((owned_policy_loss_kernel<MK, KD, HW>), dim3(ol.grid), dim3(kBlock), 0, st, g,   \
                       rs, ol.stride, partials, acc);                                                   \
  } while (0)
#define AXON_LAUNCH_OWNED(MK, KD)                 \
  do {                                            \
    if (isw) AXON_LAUNCH_OWNED_W(MK, KD, true);   \
    else AXON_LAUNCH_OWNED_W(MK, KD, false);      \
  } while (0)
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
#undef AXON_LAUNCH_OWNED_W
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
  if ((reinterpret_cast<uintptr_t>(oldp) | reinterpret_cast<uintptr_t>(samp) | reinterpret_cast<uintptr_t>(mask) |
       reinterpret_cast<uintptr_t>(isw) | reinterpret_cast<uintptr_t>(new_mask)) & 15)
    return AXON_ERR_ARG;
  if (is_mode < 0 || is_mode > 2 || rs_mode < 0 || rs_mode > 3) return AXON_ERR_ARG;
  if (is_mode != 0 && isw == nullptr) return AXON_ERR_ARG;
  if (mask_kind != AXON_MASK_F32 && mask_kind != AXON_MASK_I64) return AXON_ERR_ARG;
  const OwnedCorrArgs g{oldp, samp, mask, CorrCfg{is_mode, is_thr, rs_mode, rs_lo, rs_hi, has_veto, log_veto},
                        isw, new_mask, row_cnt, row_sum, row_flag};
  const RowStarts rs{cu, uniform_len, n_rows, n_slots};
  if (mask_kind == AXON_MASK_F32) {
    static const int resident = resident_blocks(owned_correction_kernel<AXON_MASK_F32>);
    const OwnedLaunch ol = owned_launch(n_slots, resident);
    hipLaunchKernelGGL(owned_correction_kernel<AXON_MASK_F32>, dim3(ol.grid), dim3(kBlock), 0,
                       (hipStream_t)stream, g, rs, ol.stride, partials, acc);
  } else {
    static const int resident = resident_blocks(owned_correction_kernel<AXON_MASK_I64>);
    const OwnedLaunch ol = owned_launch(n_slots, resident);
    hipLaunchKernelGGL(owned_correction_kernel<AXON_MASK_I64>, dim3(ol.grid), dim3(kBlock), 0,
                       (hipStream_t)stream, g, rs, ol.stride, partials, acc);
  }
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}
