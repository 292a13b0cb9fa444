// (a) Fused LM head: per-token log-prob and entropy, and its backward, without
// materialising the [tokens x vocab] logits.
//
// Forward    logits^T tile = W[vocab tile] . hidden[token tile]^T on MFMA; the
//            epilogue folds each tile into per-token (max, sum exp, sum logit*exp)
//            partials; a small kernel merges partials and adds the label logit.
// Backward   per vocab chunk:
//   B1  recompute the logits tile (or decode the forward's stash), form dlogit in
//       registers, write it as bf16 dl[token][vocab];
//   B2  dHidden[token][h] (+)= sum_v dl[token][v]  * WT[h][v]
//   B3  dWeight[v][h]      =  sum_t dl[t][v]       * hiddenT[h][t]
// WT and hiddenT are bf16 transposes made once per call: B2 runs on the
// K-contiguous main loop of gemm_nt.h, B3 on its variant that reads dl, K-major
// for this product, as it lies.  Shapes that variant does not take (hidden < 256,
// a vocabulary that is no multiple of 8) get a second, vocab-major copy
// dlT[vocab][token] from B1 and the K-contiguous loop.
#include "common.h"
#include "gemm_nt.h"
#include <vector>

namespace axon {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  // round-to-nearest-even in one instruction (v_cvt_pk_bf16_f32)
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  const f32x2 v = {lo, hi};
  const bf16x2 r = __builtin_convertvector(v, bf16x2);
  return *reinterpret_cast<const uint32_t*>(&r);
}

// ----------------------------------------------------------------------------
// Forward: tile epilogue -> partial statistics
// ----------------------------------------------------------------------------
struct FwdParams {
  float* pm;   // [parts][n_tokens] running max, in log2 units of the scaled logit
  float* ps;   // sum 2^(x*c - max)
  float* pe;   // sum (x*c - max) * 2^(x*c - max)
  int n_tokens, vocab;
  float c;     // inv_temperature * log2(e)
  float cap, inv_cap;  // logit soft-capping cap * tanh(logit / cap) (SOFTCAP kernels only)
  uint4* stash;        // STASH kernels only: 128 KB per tile, see StashLayout
};

// What a stashing forward leaves for the backward: for every logit, w = 2^(y - M) as fp16, where
// y is the scaled logit in log2 units and M the maximum of y over the 128 vocabulary rows of the
// same token that one wavefront holds (the `pm` partial of that (token, 128-row part)), so that
// 0 <= w <= 1 and softmax = w * 2^(M - logsumexp).  fp16 keeps eleven bits of w whatever the size
// of the logit; entries below 2^-24 of their part's maximum read back as 0 and contribute no
// gradient.  Each wavefront's 128 x 128 sub-tile is stored in accumulator order, 16 bytes per lane
// and store (two 16-row blocks), every store one contiguous kilobyte:
//   uint4 index = ((tile * 4 + wave) * 32 + j * 4 + i / 2) * 64 + lane,   tile = tm * tiles_n + tn.
// Elements that do not count in their tile (duplicates of the neighbouring tile, rows beyond the
// matrix) are stored as 0 and never read.
constexpr int64_t kStashTileBytes = 131072;
constexpr int kStashWaveVecs = 2048;  // uint4 per wavefront sub-tile

__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  const f32x2 v = {lo, hi};
  const f16x2 r = __builtin_convertvector(v, f16x2);  // round to nearest even
  return *reinterpret_cast<const uint32_t*>(&r);
}
__device__ __forceinline__ void unpack_f16(uint32_t w, float& lo, float& hi) {
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  const f16x2 r = *reinterpret_cast<const f16x2*>(&w);
  lo = (float)r[0];
  hi = (float)r[1];
}

// tanh(u) = 1 - 2 / (e^(2u) + 1): saturates cleanly at +-1 (2^x -> inf gives rcp 0, 2^x -> 0 gives -1)
__device__ __forceinline__ float fast_tanh(float u) {
  return 1.f - 2.f * __builtin_amdgcn_rcpf(fast_exp2(u * (2.f * kLog2e)) + 1.f);
}

constexpr float kEmptyMax = -3.0e38f;  // running max of a partial that saw no vocabulary row

// Partial statistics of a set of scaled logits y = logit * c (log2 units):
//   M = reference (the set's max), s = sum 2^(y-M), e = sum 2^(y-M) * (y-M).
// Merge (M2,s2,e2) into (M,s,e) under the common reference Mn >= M, M2.
__device__ __forceinline__ void merge_stats(float M, float& s, float& e, float M2, float s2,
                                            float e2, float Mn) {
  const float d1 = M - Mn, d2 = M2 - Mn;
  const float f1 = fast_exp2(d1), f2 = fast_exp2(d2);
  e = f1 * fmaf(s, d1, e) + f2 * fmaf(s2, d2, e2);
  s = s * f1 + s2 * f2;
}

// All-reduce over the four 16-lane rows of the wavefront (lanes l, l^16, l^32, l^48: the four lanes that hold
// the same token), the result in every lane: v_permlane16_swap / v_permlane32_swap hand a lane its
// neighbour row's value and its own in one vector instruction each, where a shuffle would take two trips
// through the LDS crossbar with a wait behind each.  The same pairs in the same order as the xor-16, xor-32
// butterfly, so sums come out bit for bit the same.
// Written as instructions: through the builtins the compiler takes the two results of a swap for one
// value and folds op(a, b) to op(a, a).  The s_nop covers the wait states the swaps need after a
// vector instruction has written their operands.
template <class Op>
__device__ __forceinline__ float rows_all_reduce(float v, Op op) {
  float a = v, b = v;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));  // a: rows 0 0 2 2, b: rows 1 1 3 3
  float c = op(a, b), d = c;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(c), "+v"(d));  // c: rows 01 01 01 01, d: 23 23 23 23
  return op(c, d);
}

// Fold one 256x256 logits tile into per-token partials.  MASKED: some rows of the tile
// do not count (beyond the vocabulary, or duplicates of the neighbouring tile); they are
// excluded by predicate — their accumulators hold finite values.  STASH: also store every
// 2^(y - M) for the backward (`stash_wave`: this wavefront's 32 KB, already offset by the lane).
template <bool MASKED, bool STASH>
__device__ __forceinline__ void fwd_epilogue(AccTile& acc, const FwdParams& p, const LanePos& lp,
                                             const TilePos& t, int tm, uint4* stash_wave) {
  const int part = tm * 2 + lp.wm;
#pragma unroll
  for (int j = 0; j < kBlocks; ++j) {
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < kBlocks; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int mr = lp.m(i, r);
        const bool ok = !MASKED || (mr >= t.m_lo && t.m0 + mr < p.vocab);
        mx = ok ? fmaxf(mx, acc[i][j][r]) : mx;
      }
    // the four lanes that hold the same token (lane ^ 16, lane ^ 32) share one reference
    mx = rows_all_reduce(mx, [](float a, float b) { return fmaxf(a, b); });
    const float M = (MASKED && mx == -INFINITY) ? kEmptyMax : mx * p.c;
    float s = 0.f, e = 0.f;
    uint32_t hw[kBlocks][2];
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) {
      float w[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int mr = lp.m(i, r);
        const bool ok = !MASKED || (mr >= t.m_lo && t.m0 + mr < p.vocab);
        const float y = fmaf(acc[i][j][r], p.c, -M);  // scaled logit relative to the max, <= 0
        w[r] = ok ? fast_exp2(y) : 0.f;
        s += w[r];
        e = fmaf(w[r], y, e);
      }
      if (STASH) {
        hw[i][0] = pack_f16(w[0], w[1]);
        hw[i][1] = pack_f16(w[2], w[3]);
      }
    }
    if (STASH) {
#pragma unroll
      for (int ip = 0; ip < kBlocks / 2; ++ip)
      {  // written once, read once by the backward: kept out of the way of the operand slices in L2
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        const u32x4 x = {hw[2 * ip][0], hw[2 * ip][1], hw[2 * ip + 1][0], hw[2 * ip + 1][1]};
        __builtin_nontemporal_store(x, reinterpret_cast<u32x4*>(stash_wave + (j * 4 + ip) * 64));
      }
    }
    s = rows_all_reduce(s, [](float a, float b) { return a + b; });
    e = rows_all_reduce(e, [](float a, float b) { return a + b; });
    const int nr = lp.n(j);
    const int n = t.n0 + nr;
    if (lp.lq == 0 && nr >= t.n_lo && n < p.n_tokens) {
      const int64_t o = (int64_t)part * p.n_tokens + n;
      p.pm[o] = M;
      p.ps[o] = s;
      p.pe[o] = e;
    }
  }
}

// SOFTCAP: the logits go through cap * tanh(. / cap) before the statistics (fused_linear.py:19-23).
template <class Loop, bool SOFTCAP, bool STASH>
__device__ __forceinline__ void fwd_body(const GemmOperands& g, const FwdParams& p, int tiles_m,
                                         int tiles_n) {
  extern __shared__ __align__(16) char smem[];
  int tm, tn;
  tile_coords<8>(tiles_m, tiles_n, tm, tn);
  const TilePos t = Loop::place(g, tm, tn);
  AccTile acc;
  Loop::run(g, t, acc, smem);
  if (SOFTCAP) {
#pragma unroll
    for (int i = 0; i < kBlocks; ++i)
#pragma unroll
      for (int j = 0; j < kBlocks; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][j][r] = p.cap * fast_tanh(acc[i][j][r] * p.inv_cap);
  }
  const LanePos lp;
  uint4* const stash_wave =
      STASH ? p.stash + ((int64_t)(tm * tiles_n + tn) * 4 + lp.wave) * kStashWaveVecs + lp.lane : nullptr;
  if (t.m_lo > 0 || t.m0 + kTile > p.vocab)
    fwd_epilogue<true, STASH>(acc, p, lp, t, tm, stash_wave);
  else
    fwd_epilogue<false, STASH>(acc, p, lp, t, tm, stash_wave);
}

template <class Loop>
__global__ __launch_bounds__(kGemmThreads) void lmhead_fwd_kernel(GemmOperands g, FwdParams p,
                                                                  int tiles_m, int tiles_n) {
  fwd_body<Loop, false, false>(g, p, tiles_m, tiles_n);
}

template <class Loop>
__global__ __launch_bounds__(kGemmThreads) void lmhead_fwd_softcap_kernel(GemmOperands g,
                                                                          FwdParams p, int tiles_m,
                                                                          int tiles_n) {
  fwd_body<Loop, true, false>(g, p, tiles_m, tiles_n);
}

template <class Loop>
__global__ __launch_bounds__(kGemmThreads) void lmhead_fwd_stash_kernel(GemmOperands g, FwdParams p,
                                                                        int tiles_m, int tiles_n) {
  fwd_body<Loop, false, true>(g, p, tiles_m, tiles_n);
}

template <class Loop>
__global__ __launch_bounds__(kGemmThreads) void lmhead_fwd_softcap_stash_kernel(GemmOperands g,
                                                                                FwdParams p,
                                                                                int tiles_m,
                                                                                int tiles_n) {
  fwd_body<Loop, true, true>(g, p, tiles_m, tiles_n);
}

// Token-aligned packed layout.  With `is_start` (one byte per packed position, 1 where a sequence
// begins) the head works on a packed stream of token ids directly: hidden position n predicts the
// token at position n + 1, so its label is ids[n + 1] and its outputs land at position n + 1; a
// sequence's first position receives 0 (there is no prediction for it) and its upstream gradient
// is ignored.  This is roll(ids, -1) before and the shift-right after the head
// (axon/utils/fsdp/forward_utils.py:131,180-182) without the extra passes.  The position after the
// last one is `last_dst`: 0 for a whole packed stream (it wraps to the first position, which is always
// a sequence start).  A call that covers a block of consecutive positions of a longer stream hands
// over its arrays offset to the block's first position and names where its last row's output goes:
// n_tokens (the stream goes on: the first position of the next block) or minus the block's first
// position (the block ends the stream: position 0 of the stream).
__device__ __forceinline__ int aligned_pos(int n, int n_tokens, const uint8_t* is_start, int last_dst) {
  if (is_start == nullptr) return n;
  return (n + 1 == n_tokens) ? last_dst : n + 1;
}

__global__ __launch_bounds__(256) void seq_start_kernel(const int32_t* __restrict__ cu, int n_seqs,
                                                        int n_tokens, uint8_t* __restrict__ is_start) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n_seqs) return;
  const int s0 = cu[i];
  if (s0 >= 0 && s0 < n_tokens && cu[i + 1] > s0) is_start[s0] = 1;  // empty sequences own no position
}

// Merge partials: lse, entropy_b, entropy.  A workgroup owns kMergeTokens consecutive tokens; its
// kMergeGroups thread groups each fold every kMergeGroups-th partial of a token (four loads ahead of the
// fold), then the first group folds the groups' results in group order.
constexpr int kMergeTokens = 32;
constexpr int kMergeGroups = 8;

__global__ __launch_bounds__(kMergeTokens * kMergeGroups) void lmhead_merge_kernel(
    const float* __restrict__ pm, const float* __restrict__ ps, const float* __restrict__ pe,
    int parts, int n_tokens, float* __restrict__ lse, float* __restrict__ entropy_b,
    float* __restrict__ entropy, float* __restrict__ fin_max, float* __restrict__ fin_log2s,
    const uint8_t* __restrict__ is_start, int last_dst) {
  __shared__ float red[3][kMergeGroups][kMergeTokens];
  const int tok = threadIdx.x % kMergeTokens, grp = threadIdx.x / kMergeTokens;
  const int n = blockIdx.x * kMergeTokens + tok;
  const int nc = n < n_tokens ? n : n_tokens - 1;  // a valid token; its result is dropped below
  float M = 0.f, s = 0.f, e = 0.f;
  bool any = false;  // a group beyond the number of partials folds nothing
  auto fold = [&](float M2, float s2, float e2) {
    if (!any) { M = M2; s = s2; e = e2; any = true; return; }
    const float Mn = fmaxf(M, M2);
    merge_stats(M, s, e, M2, s2, e2, Mn);
    M = Mn;
  };
  int q = grp;
  for (; q + 3 * kMergeGroups < parts; q += 4 * kMergeGroups) {
    float M2[4], s2[4], e2[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t o = (int64_t)(q + u * kMergeGroups) * n_tokens + nc;
      M2[u] = pm[o]; s2[u] = ps[o]; e2[u] = pe[o];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) fold(M2[u], s2[u], e2[u]);
  }
  for (; q < parts; q += kMergeGroups) {
    const int64_t o = (int64_t)q * n_tokens + nc;
    fold(pm[o], ps[o], pe[o]);
  }
  red[0][grp][tok] = M; red[1][grp][tok] = s; red[2][grp][tok] = e;
  __syncthreads();
  if (grp != 0 || n >= n_tokens) return;
  for (int g2 = 1; g2 < kMergeGroups && g2 < parts; ++g2)
    fold(red[0][g2][tok], red[1][g2][tok], red[2][g2][tok]);
  // log2 units: logsumexp = M + L, sum softmax*logit = M + e/s; differences are taken
  // before adding M so that large logits do not cancel
  const float L = __log2f(s);
  const float d = e / s;
  lse[n] = (M + L) * kLn2;
  entropy_b[n] = (M + d) * kLn2;
  const int dst = aligned_pos(n, n_tokens, is_start, last_dst);
  entropy[dst] = (is_start && is_start[dst]) ? 0.f : (L - d) * kLn2;
  fin_max[n] = M;
  fin_log2s[n] = L;
}

// logprob[n] = softcap(hidden[n] . W[label[n]]) / T - lse[n].  One wave per token.
template <typename LabelT>
__global__ __launch_bounds__(256) void lmhead_label_kernel(
    const __bf16* __restrict__ hidden, const __bf16* __restrict__ weight,
    const LabelT* __restrict__ labels, int n_tokens, int hidden_sz, int vocab, float inv_temp,
    float cap, const float* __restrict__ fin_max, const float* __restrict__ fin_log2s,
    float* __restrict__ logprobs, const uint8_t* __restrict__ is_start, int last_dst) {
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (n >= n_tokens) return;
  const int lane = threadIdx.x & 63;
  const int dst = aligned_pos(n, n_tokens, is_start, last_dst);
  const int64_t lab = (int64_t)labels[dst];
  float dot = 0.f;
  if (lab >= 0 && lab < vocab) {
    const uint4* h = reinterpret_cast<const uint4*>(hidden + (int64_t)n * hidden_sz);
    const uint4* w = reinterpret_cast<const uint4*>(weight + lab * hidden_sz);
    for (int c = lane; c < hidden_sz / 8; c += 64) {
      const uint4 hv = h[c], wv = w[c];
      const uint32_t hs[4] = {hv.x, hv.y, hv.z, hv.w}, ws[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        dot = fmaf(__uint_as_float(hs[k] << 16), __uint_as_float(ws[k] << 16), dot);
        dot = fmaf(__uint_as_float(hs[k] & 0xffff0000u), __uint_as_float(ws[k] & 0xffff0000u), dot);
      }
    }
  }
  dot = wave_sum(dot);
  if (cap != 0.f) dot = cap * fast_tanh(dot / cap);
  // (logit*c - M) is formed in one rounding, then log2(sum) is subtracted: no cancellation
  if (lane == 0) {
    const float lpv = (fmaf(dot, inv_temp * kLog2e, -fin_max[n]) - fin_log2s[n]) * kLn2;
    logprobs[dst] = (is_start && is_start[dst]) ? 0.f : lpv;
  }
}

// ----------------------------------------------------------------------------
// Backward B1: recompute logits, write dlogit (bf16) in both orientations
// ----------------------------------------------------------------------------
struct DlogitParams {
  const float* lse;
  const float* entropy_b;
  const float* dlogprobs;
  const float* dentropy;  // may be null
  const void* labels;
  int labels_i64;
  __bf16* dl;    // [n_pad][chunk_cols]   token-major
  __bf16* dlT;   // [chunk_cols][n_pad]   vocab-major; null: not wanted (the dWeight GEMM reads dl as a K-major operand)
  int64_t ld_dl, ld_dlT;
  int n_tokens, vocab, v_begin;  // v_begin: first vocab row of this chunk
  float inv_temp;
  float cap, inv_cap;  // soft-capping (SOFTCAP kernels only)
  const uint8_t* is_start;  // token-aligned packed layout (see aligned_pos), or null
  int last_dst;             // where the last row's label and gradients live (see aligned_pos)
};

// Four rows of four bf16 (rws[f] = row f) -> their transpose (o[e] = column e).
__device__ __forceinline__ void transpose_4x4_bf16(const uint2 (&rws)[4], uint2 (&o)[4]) {
  o[0].x = (rws[0].x & 0xffffu) | (rws[1].x << 16);
  o[0].y = (rws[2].x & 0xffffu) | (rws[3].x << 16);
  o[1].x = (rws[0].x >> 16) | (rws[1].x & 0xffff0000u);
  o[1].y = (rws[2].x >> 16) | (rws[3].x & 0xffff0000u);
  o[2].x = (rws[0].y & 0xffffu) | (rws[1].y << 16);
  o[2].y = (rws[2].y & 0xffffu) | (rws[3].y << 16);
  o[3].x = (rws[0].y >> 16) | (rws[1].y & 0xffff0000u);
  o[3].y = (rws[2].y >> 16) | (rws[3].y & 0xffff0000u);
}

// Per-wave staging of the wave's 128(n) x 128(m) bf16 sub-tile in its own 32 KB of LDS:
// row nw (256 bytes = 32 units of 4 bf16), unit u stored at slot perm(u) ^ swz(nw),
// swz(nw) = (nw & 31) ^ (nw >> 5), perm(u) = u rotated right by two bits (unit = 4 * block + lane
// quarter: the quarter's low bit becomes the slot's high bit).  The three access patterns
// (accumulator write: sixteen rows x two quarters per 32 lanes; row read; 4x4-block read) then each
// touch 32 distinct slots per 32 lanes.
__device__ __forceinline__ int stage_off(int nw, int unit) {
  const int pu = ((unit & 1) << 4) | ((unit & 2) << 2) | (unit >> 2);
  return nw * 256 + ((pu ^ ((nw & 31) ^ (nw >> 5))) << 3);
}

// SOFTCAP: the recomputed logit goes through cap * tanh(. / cap) and the gradient is multiplied by
// the derivative 1 - tanh^2 (fused_linear.py:80-83).
// Accumulators -> bf16 dlogits in the wave's staging area.  MASKED: the tile reaches past the last
// token or the last vocabulary row; those entries are written as zeros.
// Per-token factors of dlogit = softmax * (ca + cb * logit) + onehot * gl for tile-relative token
// row nr; lab_rel is the label's row inside the tile whose first vocabulary row is m0_abs (-1: not
// in this tile).
struct TokenCoef {
  float ca, cb, gl, lse2;
  int lab_rel, nn;
  bool n_ok;
  __device__ __forceinline__ TokenCoef(const DlogitParams& p, int n, int64_t m0_abs) {
    n_ok = n < p.n_tokens;
    nn = n_ok ? n : 0;
    const int src = aligned_pos(nn, p.n_tokens, p.is_start, p.last_dst);  // where the label and the gradients live
    const bool g_ok = n_ok && !(p.is_start && p.is_start[src]);
    const float g_lp = g_ok ? p.dlogprobs[src] : 0.f;
    const float g_en = (g_ok && p.dentropy) ? p.dentropy[src] : 0.f;
    lse2 = p.lse[nn] * kLog2e;
    const float eb = p.entropy_b[nn];
    ca = (-g_lp + g_en * eb) * p.inv_temp;
    cb = -g_en * p.inv_temp * p.inv_temp;
    gl = g_lp * p.inv_temp;
    const int64_t lab = p.labels_i64 ? static_cast<const int64_t*>(p.labels)[src]
                                     : (int64_t) static_cast<const int32_t*>(p.labels)[src];
    const int64_t lab_rel64 = lab - m0_abs;
    lab_rel = (lab_rel64 >= 0 && lab_rel64 < kTile) ? (int)lab_rel64 : -1;
  }
};

template <bool SOFTCAP, bool MASKED>
__device__ __forceinline__ void dlogit_stage(AccTile& acc, const DlogitParams& p, const LanePos& lp,
                                             const TilePos& t, char* stage) {
  const float c = p.inv_temp * kLog2e;
#pragma unroll
  for (int j = 0; j < kBlocks; ++j) {
    const int nw = j * kBlk + lp.l16;  // token row inside the wave's sub-tile
    const TokenCoef k(p, t.n0 + lp.wn * kWaveTile + nw, (int64_t)p.v_begin + t.m0);
    const int m_end = MASKED ? (k.n_ok ? p.vocab - p.v_begin - t.m0 : 0) : kTile;  // rows that count
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) {
      float d[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int mrel = lp.m(i, r);
        float raw = acc[i][j][r];
        float dcap = 1.f;
        if (SOFTCAP) {
          const float th = fast_tanh(raw * p.inv_cap);
          raw = p.cap * th;
          dcap = fmaf(-th, th, 1.f);
        }
        const float pr = fast_exp2(fmaf(raw, c, -k.lse2));
        float v = pr * fmaf(k.cb, raw, k.ca);
        if (mrel == k.lab_rel) v += k.gl;
        if (SOFTCAP) v *= dcap;
        // rows shared with the neighbouring tile keep their (identical) values
        d[r] = (!MASKED || mrel < m_end) ? v : 0.f;
      }
      uint2 w;
      w.x = pack_bf16(d[0], d[1]);
      w.y = pack_bf16(d[2], d[3]);
      *reinterpret_cast<uint2*>(stage + stage_off(nw, i * 4 + lp.lq)) = w;
    }
  }
}

// The same from a forward's stash (see StashLayout above FwdParams): softmax = w * 2^(M - lse), scaled
// logit = log2(w) + M.  One call covers 64 tokens (four 16-token blocks, j0 .. j0 + 3) x 128 vocabulary
// rows of a wavefront's sub-tile; staged row = token - 16 * j0.  SOFTCAP: the stash describes the capped
// logit, whose derivative factor is 1 - (capped / cap)^2.  EDGE: entries that do not count in this tile
// are staged as zeros.
constexpr int kStashHalfBlocks = kBlocks / 2;
template <bool SOFTCAP, bool EDGE>
__device__ __forceinline__ void dlogit_stage_stash(const uint4 (&st)[4 * kStashHalfBlocks], int j0,
                                                   const float* __restrict__ pm, int part,
                                                   const DlogitParams& p, const LanePos& lp,
                                                   const TilePos& t, char* stage) {
  const float inv_c = 1.f / (p.inv_temp * kLog2e);
#pragma unroll
  for (int jl = 0; jl < kStashHalfBlocks; ++jl) {
    const int nw = jl * kBlk + lp.l16;
    const int nr = lp.wn * kWaveTile + j0 * kBlk + nw;
    const TokenCoef k(p, t.n0 + nr, (int64_t)p.v_begin + t.m0);
    const float Mp = pm[(int64_t)part * p.n_tokens + k.nn];
    const float scale = fast_exp2(Mp - k.lse2);
    const bool n_counts = !EDGE || (k.n_ok && nr >= t.n_lo);
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) {
      const uint4 q = st[jl * 4 + (i >> 1)];
      float wv[4];
      unpack_f16((i & 1) ? q.z : q.x, wv[0], wv[1]);
      unpack_f16((i & 1) ? q.w : q.y, wv[2], wv[3]);
      float d[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int mrel = lp.m(i, r);
        const float pr = wv[r] * scale;
        const float raw = (__builtin_amdgcn_logf(fmaxf(wv[r], 1e-30f)) + Mp) * inv_c;
        float v = pr * fmaf(k.cb, raw, k.ca);
        if (mrel == k.lab_rel) v += k.gl;
        if (SOFTCAP) {
          const float th = raw * p.inv_cap;
          v *= fmaf(-th, th, 1.f);
        }
        const bool ok = !EDGE || (n_counts && mrel >= t.m_lo && p.v_begin + t.m0 + mrel < p.vocab);
        d[r] = ok ? v : 0.f;
      }
      uint2 w;
      w.x = pack_bf16(d[0], d[1]);
      w.y = pack_bf16(d[2], d[3]);
      *reinterpret_cast<uint2*>(stage + stage_off(nw, i * 4 + lp.lq)) = w;
    }
  }
}

// A staged 64 x 128 half sub-tile (tokens 16 * j0 .. of the wavefront's sub-tile) -> dl and dlT.  Token-major
// as in dlogit_copy_out (below); vocab-major: sixteen lanes cover the 64 tokens of one vocabulary row (one
// 128-byte line), the four lane groups take units u, u + 8, u + 16, u + 24, whose permuted slots differ in
// a bit that the rows' swizzles (a set with that bit fixed) cannot cancel.  EDGE: entries that duplicate the
// neighbouring tile (tile-relative token < n_lo, vocabulary row < m_lo; both multiples of 4) are left to it.
template <bool EDGE>
__device__ __forceinline__ void dlogit_copy_out_half(const char* stage, int j0, const DlogitParams& p,
                                                     const LanePos& lp, const TilePos& t) {
  const int l32 = lp.lane & 31, lhi = lp.lane >> 5;
  const int m_base = t.m0 + lp.wm * kWaveTile;
  const int n_base = t.n0 + lp.wn * kWaveTile + j0 * kBlk;
  const int m_skip = t.m_lo - lp.wm * kWaveTile, n_skip = t.n_lo - lp.wn * kWaveTile - j0 * kBlk;
  {
    const int unit = l32;
    char* d = reinterpret_cast<char*>(p.dl + (int64_t)(n_base + lhi) * p.ld_dl + m_base + unit * 4);
    const int64_t dstep = p.ld_dl * 4;  // two rows of bf16
    const bool col_ok = !EDGE || unit * 4 >= m_skip;
#pragma unroll 1
    for (int nw0 = lhi; nw0 < kStashHalfBlocks * kBlk; nw0 += 16) {
      uint2 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const uint2*>(stage + stage_off(nw0 + 2 * u, unit));
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (col_ok && (!EDGE || nw0 + 2 * u >= n_skip)) *reinterpret_cast<uint2*>(d) = v[u];
        d += dstep;
      }
    }
  }
  if (p.dlT) {
    const int nq = lp.lane & 15, grp = lp.lane >> 4;
    const int64_t rstep = p.ld_dlT * 2;  // one row of bf16
    char* d = reinterpret_cast<char*>(p.dlT + (int64_t)(m_base + grp * 32) * p.ld_dlT + n_base + nq * 4);
    const bool tok_ok = !EDGE || nq * 4 >= n_skip;
#pragma unroll 2
    for (int u8 = 0; u8 < 8; ++u8) {
      const int unit = grp * 8 + u8;
      uint2 rws[4];
#pragma unroll
      for (int f = 0; f < 4; ++f)
        rws[f] = *reinterpret_cast<const uint2*>(stage + stage_off(nq * 4 + f, unit));
      uint2 o[4];
      transpose_4x4_bf16(rws, o);
      if (tok_ok && (!EDGE || unit * 4 >= m_skip)) {
#pragma unroll
        for (int e = 0; e < 4; ++e) *reinterpret_cast<uint2*>(d + e * rstep) = o[e];
      }
      d += 4 * rstep;
    }
  }
}

// The wave's staged 128 x 128 bf16 sub-tile -> dl (token-major) and dlT (vocab-major).  The wave
// reads back only what it wrote itself; LDS operations of one wave complete in order.
__device__ __forceinline__ void dlogit_copy_out(const char* stage, const DlogitParams& p,
                                                const LanePos& lp, const TilePos& t) {
  const int l32 = lp.lane & 31, lhi = lp.lane >> 5;
  const int m_base = t.m0 + lp.wm * kWaveTile;  // chunk-relative column of the sub-tile
  const int n_base = t.n0 + lp.wn * kWaveTile;
  // token-major copy: 32 lanes cover one 256-byte row.  Eight rows per trip, reads before writes;
  // destinations by running pointers (no 64-bit multiplies in the loop).
  {
    const int unit = l32;
    char* d = reinterpret_cast<char*>(p.dl + (int64_t)(n_base + lhi) * p.ld_dl + m_base + unit * 4);
    const int64_t dstep = p.ld_dl * 4;  // two rows of bf16
#pragma unroll 1
    for (int nw0 = lhi; nw0 < kWaveTile; nw0 += 16) {
      uint2 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = *reinterpret_cast<const uint2*>(stage + stage_off(nw0 + 2 * u, unit));
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        *reinterpret_cast<uint2*>(d) = v[u];
        d += dstep;
      }
    }
  }
  // vocab-major copy: 4x4 blocks transposed in registers; 32 lanes cover 128 tokens of one vocab row
  if (p.dlT) {
    const int nq = l32;  // token quad
    const int64_t rstep = p.ld_dlT * 2;  // one row of bf16
    char* d = reinterpret_cast<char*>(p.dlT + (int64_t)(m_base + lhi * 4) * p.ld_dlT + n_base + nq * 4);
#pragma unroll 2
    for (int unit = lhi; unit < 32; unit += 2) {
      uint2 rws[4];
#pragma unroll
      for (int f = 0; f < 4; ++f)
        rws[f] = *reinterpret_cast<const uint2*>(stage + stage_off(nq * 4 + f, unit));
      uint2 o[4];
      transpose_4x4_bf16(rws, o);
#pragma unroll
      for (int e = 0; e < 4; ++e) *reinterpret_cast<uint2*>(d + e * rstep) = o[e];
      d += 8 * rstep;
    }
  }
}

template <class Loop, bool SOFTCAP>
__device__ __forceinline__ void dlogit_body(const GemmOperands& g, const DlogitParams& p,
                                            int tiles_m, int tiles_n) {
  extern __shared__ __align__(16) char smem[];
  int tm, tn;
  tile_coords(tiles_m, tiles_n, tm, tn);
  const TilePos t = Loop::place(g, tm, tn);  // t.m0 is relative to the chunk
  AccTile acc;
  Loop::run(g, t, acc, smem);
  __syncthreads();  // every wave is past its last main-loop LDS access

  const LanePos lp;
  char* const stage = smem + lp.wave * 32768;
  if (t.n0 + kTile > p.n_tokens || p.v_begin + t.m0 + kTile > p.vocab)
    dlogit_stage<SOFTCAP, true>(acc, p, lp, t, stage);
  else
    dlogit_stage<SOFTCAP, false>(acc, p, lp, t, stage);
  dlogit_copy_out(stage, p, lp, t);
}

template <class Loop>
__global__ __launch_bounds__(kGemmThreads) void lmhead_dlogit_kernel(GemmOperands g, DlogitParams p,
                                                                     int tiles_m, int tiles_n) {
  dlogit_body<Loop, false>(g, p, tiles_m, tiles_n);
}

template <class Loop>
__global__ __launch_bounds__(kGemmThreads) void lmhead_dlogit_softcap_kernel(GemmOperands g,
                                                                             DlogitParams p,
                                                                             int tiles_m,
                                                                             int tiles_n) {
  dlogit_body<Loop, true>(g, p, tiles_m, tiles_n);
}

// Backward B1 without the recompute: one wavefront per workgroup turns half (64 tokens x 128 rows) of a
// sub-tile that a stashing forward stored into bf16 dlogits in both orientations (16 KB of LDS and few
// registers: ten wavefronts per CU hide the latency of the loads and of the per-token operands).  A streaming kernel: 2 bytes
// read and 4 written per logit.  Tiles are the forward's (same shifted or clamped placement), so
// `tm0` is the forward tile row of the chunk's first vocabulary row and t.m0 is made chunk-relative
// only after the edge tests; it is negative only for rows that the tile does not own.
struct StashSource {
  const uint4* stash;
  const float* pm;
  int tiles_n, tm0, shifted;
};

template <bool SOFTCAP>
__global__ __launch_bounds__(64) void lmhead_dlogit_stash_kernel(DlogitParams p, StashSource src) {
  __shared__ __align__(16) char stage[kStashHalfBlocks * kBlk * 256];  // 64 tokens x 128 bf16
  const int half = blockIdx.x & 1, wave = (blockIdx.x >> 1) & 3, tile = blockIdx.x >> 3;
  const int tm = src.tm0 + tile / src.tiles_n, tn = tile % src.tiles_n;
  TilePos t{tm * kTile, tn * kTile, 0, 0};
  if (src.shifted) {
    t.m0 = min(t.m0, p.vocab - kTile);
    t.n0 = min(t.n0, p.n_tokens - kTile);
    t.m_lo = tm * kTile - t.m0;
    t.n_lo = tn * kTile - t.n0;
  }
  LanePos lp;
  lp.wave = wave;
  lp.wm = wave >> 1;
  lp.wn = wave & 1;
  const int j0 = half * kStashHalfBlocks;
  const uint4* sv = src.stash + ((int64_t)(tm * src.tiles_n + tn) * 4 + wave) * kStashWaveVecs +
                    j0 * 4 * 64 + lp.lane;
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  uint4 st[4 * kStashHalfBlocks];
#pragma unroll
  for (int q = 0; q < 4 * kStashHalfBlocks; ++q) {  // read once: keep it out of the way of the GEMMs' operands in L2
    const u32x4 x = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(sv + q * 64));
    st[q] = make_uint4(x[0], x[1], x[2], x[3]);
  }
  const bool edge = t.m_lo > 0 || t.n_lo > 0 || t.m0 + kTile > p.vocab || t.n0 + kTile > p.n_tokens;
  t.m0 -= p.v_begin;
  const int part = tm * 2 + lp.wm;
  if (edge) {
    dlogit_stage_stash<SOFTCAP, true>(st, j0, src.pm, part, p, lp, t, stage);
    dlogit_copy_out_half<true>(stage, j0, p, lp, t);
  } else {
    dlogit_stage_stash<SOFTCAP, false>(st, j0, src.pm, part, p, lp, t, stage);
    dlogit_copy_out_half<false>(stage, j0, p, lp, t);
  }
}

// ----------------------------------------------------------------------------
// Backward B2/B3 and the plain GEMM: store the tile as out[n][m]
// ----------------------------------------------------------------------------
struct StoreParams {
  float* out_f32;     // [n][ld_f32] fp32 accumulator / output (may be null)
  __bf16* out_bf16;   // [n][ld_bf16] (may be null)
  int64_t ld_f32, ld_bf16;
  int m_valid, n_valid;
  int accumulate;     // add the previous contents of out_f32 (or tile_acc) first
  int keep_f32;       // write the sum back to out_f32 / tile_acc (0: it is only read, the sum leaves as bf16)
  // fp32 partial sums that only this kernel ever reads back (the weight gradient carried from one token
  // block to the next): kept per tile in the order the accumulators lie in the registers, so that every
  // wavefront load and store is one contiguous kilobyte.  float4 index =
  // ((tile * 4 + wave) * 64 + i * 8 + j) * 64 + lane, tile = tm * tiles_n + tn.  Null: not used.
  float4* tile_acc;
};
constexpr int64_t kTileAccVecs = 4 * kBlocks * kBlocks * 64;  // float4 per tile (256 KB)

template <class Loop>
__global__ __launch_bounds__(kGemmThreads) void gemm_store_kernel(GemmOperands g, StoreParams p,
                                                                  int tiles_m, int tiles_n) {
  extern __shared__ __align__(16) char smem[];
  int tm, tn;
  tile_coords(tiles_m, tiles_n, tm, tn);
  const TilePos t = Loop::place(g, tm, tn);
  AccTile acc;
  Loop::run(g, t, acc, smem);
  const LanePos lp;
  if (p.tile_acc) {
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    f32x4* ta = reinterpret_cast<f32x4*>(p.tile_acc) +
                ((int64_t)(tm * tiles_n + tn) * 4 + lp.wave) * (kBlocks * kBlocks * 64) + lp.lane;
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) {
      f32x4 old[kBlocks];
      if (p.accumulate) {
#pragma unroll
        for (int j = 0; j < kBlocks; ++j) old[j] = __builtin_nontemporal_load(ta + (i * kBlocks + j) * 64);
      }
#pragma unroll
      for (int j = 0; j < kBlocks; ++j) {
        if (p.accumulate) {
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[i][j][r] += old[j][r];
        }
        if (p.keep_f32) {
          const f32x4 v = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
          __builtin_nontemporal_store(v, ta + (i * kBlocks + j) * 64);
        }
      }
    }
    if (!p.out_bf16) return;
  }
#pragma unroll
  for (int j = 0; j < kBlocks; ++j) {
    const int nr = lp.n(j);
    const int n = t.n0 + nr;
    if (nr < t.n_lo || n >= p.n_valid) continue;
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) {
      const int mr = lp.m(i, 0);
      const int m = t.m0 + mr;
      // m_valid % 4 == 0 and tile shifts are multiples of 4: a quad is all in or all out
      if (mr < t.m_lo || m >= p.m_valid) continue;
      float4 v = make_float4(acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]);
      if (p.out_f32) {
        float4* dst = reinterpret_cast<float4*>(p.out_f32 + (int64_t)n * p.ld_f32 + m);
        if (p.accumulate) {
          const float4 old = *dst;
          v.x += old.x; v.y += old.y; v.z += old.z; v.w += old.w;
        }
        if (p.keep_f32) *dst = v;
      }
      if (p.out_bf16) {
        uint2 w;
        w.x = pack_bf16(v.x, v.y);
        w.y = pack_bf16(v.z, v.w);
        *reinterpret_cast<uint2*>(p.out_bf16 + (int64_t)n * p.ld_bf16 + m) = w;
      }
    }
  }
}

// out[c][r] = in[r][c] for r < rows, c < cols; zero for r in [rows, rows_pad).
// 64x64 tiles through LDS; both sides move 16 bytes per thread and access (two per thread each
// way) where the tile is whole, element by element at the ragged edges.  ld_in and ld_out are
// multiples of 8 elements and both bases 16-byte aligned (checked by the launcher).
__global__ __launch_bounds__(256) void transpose_bf16_kernel(const uint16_t* __restrict__ in,
                                                             int64_t ld_in, int rows, int cols,
                                                             uint16_t* __restrict__ out,
                                                             int64_t ld_out, int rows_pad) {
  __shared__ uint16_t t[64][66 + 6];  // 144-byte rows: 16-byte row writes stay aligned
  const int r0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
#pragma unroll
  for (int q = threadIdx.x; q < 512; q += 256) {
    const int r = q >> 3, c = (q & 7) * 8;
    union { uint4 v; uint16_t h[8]; } u;
    u.v = make_uint4(0, 0, 0, 0);
    if (r0 + r < rows) {
      const uint16_t* src = in + (int64_t)(r0 + r) * ld_in + c0 + c;
      if (c0 + c + 8 <= cols) {
        u.v = *reinterpret_cast<const uint4*>(src);
      } else {
        for (int e = 0; e < 8; ++e)
          if (c0 + c + e < cols) u.h[e] = src[e];
      }
    }
    *reinterpret_cast<uint4*>(&t[r][c]) = u.v;
  }
  __syncthreads();
#pragma unroll
  for (int q = threadIdx.x; q < 512; q += 256) {
    const int c = q >> 3, r = (q & 7) * 8;
    if (c0 + c >= cols || r0 + r >= rows_pad) continue;
    union { uint4 v; uint16_t h[8]; } u;
#pragma unroll
    for (int e = 0; e < 8; ++e) u.h[e] = t[r + e][c];
    uint16_t* dst = out + (int64_t)(c0 + c) * ld_out + r0 + r;
    if (r0 + r + 8 <= rows_pad) {
      *reinterpret_cast<uint4*>(dst) = u.v;
    } else {
      for (int e = 0; e < 8; ++e)
        if (r0 + r + e < rows_pad) dst[e] = u.h[e];
    }
  }
}

// zero the bf16 columns [col0, col0 + ncols) of `rows` rows (reduction padding of dl / dlT)
__global__ __launch_bounds__(256) void zero_cols_bf16_kernel(uint16_t* p, int64_t ld, int rows,
                                                             int col0, int ncols) {
  const int64_t total = (int64_t)rows * ncols;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x)
    p[(i / ncols) * ld + col0 + (i % ncols)] = 0;
}


// ----------------------------------------------------------------------------
// Rows without an upstream gradient (prompt positions, masked or clipped tokens)
// ----------------------------------------------------------------------------
// One workgroup walks the rows in blocks of 4096 (four consecutive rows per thread) and numbers the
// active ones in ascending order (ballots + popcounts inside a wave, wave totals through LDS): the
// list is the same on every run.
__global__ __launch_bounds__(1024) void active_rows_kernel(
    const float* __restrict__ dlogprobs, const float* __restrict__ dentropy,
    const uint8_t* __restrict__ is_start, int n_tokens, int32_t* __restrict__ row_index,
    int32_t* __restrict__ row_rank, int32_t* __restrict__ count) {
  __shared__ int wave_total[16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const unsigned long long below = (1ull << lane) - 1ull;
  int base = 0;
  for (int n0 = 0; n0 < n_tokens; n0 += 4096) {
    const int first = n0 + (int)threadIdx.x * 4;
    bool act[4];
    int before = 0, mine = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = first + j;
      act[j] = false;
      if (n < n_tokens) {
        const int src = aligned_pos(n, n_tokens, is_start, 0);
        if (!(is_start && is_start[src]))
          act[j] = dlogprobs[src] != 0.f || (dentropy && dentropy[src] != 0.f);  // NaN counts as active
      }
      const unsigned long long b = __ballot(act[j]);
      before += __popcll(b & below);  // active rows of the lanes below, this j
      mine += __popcll(b);
    }
    if (lane == 0) wave_total[wave] = mine;
    __syncthreads();
    int total = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      if (w < wave) before += wave_total[w];
      total += wave_total[w];
    }
    int r = base + before;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = first + j;
      if (n < n_tokens) {
        if (act[j]) row_index[r] = n;
        row_rank[n] = act[j] ? r : -1;
        r += act[j] ? 1 : 0;
      }
    }
    base += total;
    __syncthreads();
  }
  if (threadIdx.x == 0) count[0] = base;
}

// One workgroup per active row: its hidden vector (16-byte accesses) and its scalars, the label and the
// gradients taken from the aligned position.
template <typename LabelT>
__global__ __launch_bounds__(256) void gather_rows_kernel(
    const uint4* __restrict__ hidden, int row_vec, const LabelT* __restrict__ labels,
    const float* __restrict__ lse, const float* __restrict__ entropy_b,
    const float* __restrict__ dlogprobs, const float* __restrict__ dentropy,
    const uint8_t* __restrict__ is_start, int n_tokens, const int32_t* __restrict__ row_index,
    uint4* __restrict__ hidden_c, LabelT* __restrict__ labels_c, float* __restrict__ lse_c,
    float* __restrict__ entropy_b_c, float* __restrict__ dlogprobs_c, float* __restrict__ dentropy_c) {
  const int r = blockIdx.x;
  const int n = row_index[r];
  const uint4* src_row = hidden + (int64_t)n * row_vec;
  uint4* dst_row = hidden_c + (int64_t)r * row_vec;
  for (int c = threadIdx.x; c < row_vec; c += 256) dst_row[c] = src_row[c];
  if (threadIdx.x == 0) {
    const int src = aligned_pos(n, n_tokens, is_start, 0);
    labels_c[r] = labels[src];
    lse_c[r] = lse[n];
    entropy_b_c[r] = entropy_b[n];
    dlogprobs_c[r] = dlogprobs[src];
    if (dentropy_c) dentropy_c[r] = dentropy ? dentropy[src] : 0.f;
  }
}

// One workgroup per row of d_hidden: the compact row, or zeros.
__global__ __launch_bounds__(256) void scatter_rows_kernel(const uint4* __restrict__ d_hidden_c,
                                                           const int32_t* __restrict__ row_rank,
                                                           int row_vec, uint4* __restrict__ d_hidden) {
  const int n = blockIdx.x;
  const int r = row_rank[n];
  uint4* dst_row = d_hidden + (int64_t)n * row_vec;
  if (r < 0) {
    for (int c = threadIdx.x; c < row_vec; c += 256) dst_row[c] = make_uint4(0, 0, 0, 0);
    return;
  }
  const uint4* src_row = d_hidden_c + (int64_t)r * row_vec;
  for (int c = threadIdx.x; c < row_vec; c += 256) dst_row[c] = src_row[c];
}

// x *= scale[0] in place on bf16 values, eight per thread and access; nothing is read or written when the
// factor is exactly one (the factor lives on the device: the host does not know it without waiting).
__global__ __launch_bounds__(256) void scale_bf16_kernel(uint4* __restrict__ x, int64_t n_vec,
                                                         const float* __restrict__ scale) {
  const float s = scale[0];
  if (s == 1.f) return;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n_vec; i += (int64_t)gridDim.x * 256) {
    uint4 v = x[i];
    uint32_t* w = reinterpret_cast<uint32_t*>(&v);
#pragma unroll
    for (int k = 0; k < 4; ++k)
      w[k] = pack_bf16(__uint_as_float(w[k] << 16) * s, __uint_as_float(w[k] & 0xffff0000u) * s);
    x[i] = v;
  }
}

}  // namespace axon

using namespace axon;

namespace {

inline int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }
// bf16 dlogits of one chunk exist in both orientations (2 x 2.1 GB at 32768 tokens); every chunk costs one
// read-modify-write pass over the fp32 dHidden accumulator, so fewer, larger chunks are cheaper
constexpr int64_t kDefaultVocabChunk = 32768;
constexpr int64_t kAlign = 256;
using SlowLoop = RegLoop<32>;

inline bool dma_ok(const GemmOperands& g) {
  return g.m_rows >= kTile && g.n_rows >= kTile && (g.k % DmaLoop::kBK) == 0 &&
         g.lda < (1 << 21) && g.ldb < (1 << 21);  // byte offsets inside a tile stay below 2^31
}

template <typename K>
int set_lds(K kernel) {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                             hipFuncAttributeMaxDynamicSharedMemorySize,
                             kGemmLdsBytes) == hipSuccess
             ? AXON_OK
             : AXON_ERR_LAUNCH;
}

// Launch kernel<DmaLoop> or kernel<SlowLoop> over all tiles of the problem.
#define AXON_LAUNCH_GEMM(KERNEL, G, P, ST)                                                        \
  do {                                                                                            \
    const int tiles_m_ = ((G).m_rows + kTile - 1) / kTile, tiles_n_ = ((G).n_rows + kTile - 1) / kTile; \
    if (dma_ok(G)) {                                                                              \
      if (set_lds(KERNEL<DmaLoop>) != AXON_OK) return AXON_ERR_LAUNCH;                            \
      hipLaunchKernelGGL(KERNEL<DmaLoop>, dim3(tiles_m_ * tiles_n_), dim3(kGemmThreads),          \
                         kGemmLdsBytes, ST, G, P, tiles_m_, tiles_n_);                            \
    } else {                                                                                      \
      if (set_lds(KERNEL<SlowLoop>) != AXON_OK) return AXON_ERR_LAUNCH;                           \
      hipLaunchKernelGGL(KERNEL<SlowLoop>, dim3(tiles_m_ * tiles_n_), dim3(kGemmThreads),         \
                         kGemmLdsBytes, ST, G, P, tiles_m_, tiles_n_);                            \
    }                                                                                             \
    AXON_CHECK_LAUNCH();                                                                          \
  } while (0)

struct FwdWs {
  float *pm, *ps, *pe;
  float *fin_max, *fin_log2s;  // [n] merged max and log2(sum), for the label kernel
  int parts;
  int64_t bytes;
};
FwdWs fwd_ws(int64_t n, int64_t vocab, void* base) {
  FwdWs w;
  w.parts = (int)(round_up(vocab, kTile) / kTile) * 2;
  const int64_t one = round_up((int64_t)w.parts * n * 4, kAlign);
  char* p = static_cast<char*>(base);
  w.pm = reinterpret_cast<float*>(p);
  w.ps = reinterpret_cast<float*>(p + one);
  w.pe = reinterpret_cast<float*>(p + 2 * one);
  const int64_t fin = round_up(n * 4, kAlign);
  w.fin_max = reinterpret_cast<float*>(p + 3 * one);
  w.fin_log2s = reinterpret_cast<float*>(p + 3 * one + fin);
  w.bytes = 3 * one + 2 * fin;
  return w;
}

// The stash of a forward for its backward: the tiles' fp16 sub-tiles, then the per-part maxima
// (which the forward then writes there instead of into its workspace).
struct StashWs {
  uint4* tiles;
  float* pm;
  int tiles_m, tiles_n, shifted;
  int64_t bytes;  // 0: this shape cannot be stashed
};
StashWs stash_ws(int64_t n, int64_t h, int64_t v, void* base) {
  StashWs w{};
  if (n <= 0) return w;
  GemmOperands g{};
  g.lda = g.ldb = h;  g.m_rows = (int)v;  g.n_rows = (int)n;  g.k = (int)h;
  w.shifted = dma_ok(g);
  // shifted edge tiles hand their duplicated rows to the neighbouring tile in groups of four
  if (w.shifted && ((v % 4) != 0 || (n % 4) != 0)) return w;
  w.tiles_m = (int)(round_up(v, kTile) / kTile);
  w.tiles_n = (int)(round_up(n, kTile) / kTile);
  const int64_t tile_bytes = (int64_t)w.tiles_m * w.tiles_n * kStashTileBytes;
  w.tiles = static_cast<uint4*>(base);
  w.pm = reinterpret_cast<float*>(static_cast<char*>(base) + tile_bytes);
  w.bytes = tile_bytes + round_up((int64_t)w.tiles_m * 2 * n * 4, kAlign);
  return w;
}

struct BwdWs {
  __bf16 *wT, *hT, *dl, *dlT;
  float* dh_acc;
  int64_t v_pad, n_pad, chunk, bytes;
  int64_t ld_v, ld_n, ld_c;  // leading dimensions of wT, hT/dlT, dl: padded by kLdPad elements
  int chunks;
  // The dWeight GEMM reads dl [token][vocab] as it lies, as its K-major operand: no vocab-major copy
  // (dlT is null).  Needs the DMA loop for every chunk's GEMM and 16-byte vectors along the vocabulary.
  bool dl_kmajor;
  // The dHidden GEMM reads the weight [vocab][hidden] as it lies, as its K-major operand: no transposed
  // copy (wT is null).  Needs the DMA loop (fewer than 256 tokens are padded to 256 with zero dlogit rows)
  // and a reduction that ends with the weight's last row (vocab % 64 == 0).
  bool w_kmajor;
};
// Rows a power of two apart land on the same L2 sets and memory channels; 128 bytes of padding
// per row moves consecutive rows to consecutive cache lines (+5..13 % on a stand-alone GEMM with
// power-of-two leading dimensions, within noise on the whole backward).
constexpr int64_t kLdPad = 64;
// `n`: the tokens the workspace holds (one call's, or the span of a group of blocks whose weight
// gradient is formed by one GEMM)
BwdWs bwd_ws(int64_t n, int64_t h, int64_t vocab, int64_t chunk, void* base) {
  BwdWs w;
  w.v_pad = round_up(vocab, kTile);
  w.n_pad = round_up(n, kTile);
  w.chunk = (chunk <= 0) ? kDefaultVocabChunk : chunk;
  if (w.chunk > w.v_pad) w.chunk = w.v_pad;
  w.chunks = (int)((vocab + w.chunk - 1) / w.chunk);
  w.ld_v = w.v_pad + kLdPad;
  w.ld_n = w.n_pad + kLdPad;
  w.ld_c = w.chunk + kLdPad;
  const int64_t last_rows = vocab - (int64_t)(w.chunks - 1) * w.chunk;
  w.dl_kmajor = h >= kTile && last_rows >= kTile && vocab % 8 == 0 && w.ld_n < (1 << 21) && w.ld_c < (1 << 21);
  w.w_kmajor = h >= kTile && vocab % 64 == 0 && h < (1 << 21) && w.ld_c < (1 << 21);
  char* p = static_cast<char*>(base);
  int64_t off = 0;
  w.wT = nullptr;
  if (!w.w_kmajor) {
    w.wT = reinterpret_cast<__bf16*>(p + off);
    off += round_up(h * w.ld_v * 2, kAlign);
  }
  w.hT = reinterpret_cast<__bf16*>(p + off);  off += round_up(h * w.ld_n * 2, kAlign);
  w.dl = reinterpret_cast<__bf16*>(p + off);  off += round_up(w.n_pad * w.ld_c * 2, kAlign);
  w.dlT = nullptr;
  if (!w.dl_kmajor) {
    w.dlT = reinterpret_cast<__bf16*>(p + off);
    off += round_up(w.chunk * w.ld_n * 2, kAlign);
  }
  w.dh_acc = reinterpret_cast<float*>(p + off);
  if (w.chunks > 1) off += round_up(n * h * 4, kAlign);
  w.bytes = off;
  return w;
}

// Optional per-phase timing with HIP events on the launch stream (used by the *_timed entry points
// only).  Recording does not synchronise: the events are read when the caller collects them.  A
// null timer costs nothing.
struct PhaseTimer {
  struct Rec { hipEvent_t a, b; int phase; };
  hipStream_t st;
  std::vector<Rec> recs;
  Rec cur{};
  bool open = false;
  int base = 0;  // added to the phase ids of the spans being recorded (0 forward, 4 backward)
  explicit PhaseTimer(hipStream_t s) : st(s) {}
  void begin(int ph) {
    if (hipEventCreate(&cur.a) != hipSuccess) return;
    if (hipEventCreate(&cur.b) != hipSuccess) { (void)hipEventDestroy(cur.a); return; }
    cur.phase = base + ph;
    (void)hipEventRecord(cur.a, st);
    open = true;
  }
  void end() {
    if (!open) return;
    (void)hipEventRecord(cur.b, st);
    recs.push_back(cur);
    open = false;
  }
  // synchronises the stream; adds elapsed ms and launch counts per phase, forgets the spans
  void collect(float* ms, int32_t* launches, int n_phases) {
    (void)hipStreamSynchronize(st);
    for (const Rec& r : recs) {
      float t = 0.f;
      (void)hipEventElapsedTime(&t, r.a, r.b);
      if (r.phase < n_phases) {
        ms[r.phase] += t;
        launches[r.phase] += 1;
      }
      (void)hipEventDestroy(r.a);
      (void)hipEventDestroy(r.b);
    }
    recs.clear();
  }
};
struct Span {  // RAII: one timed span around the launches in scope
  PhaseTimer* t;
  Span(PhaseTimer* timer, int ph) : t(timer) { if (t) t->begin(ph); }
  ~Span() { if (t) t->end(); }
};

int check_head_shape(int64_t n, int64_t h, int64_t v) {
  if (n < 0 || h <= 0 || v <= 0) return AXON_ERR_ARG;
  if (h % 32 != 0) return AXON_ERR_SHAPE;
  if (n >= (1 << 30) || v >= (1 << 30) || h >= (1 << 24)) return AXON_ERR_SHAPE;
  return AXON_OK;
}

int launch_store(const GemmOperands& g, const StoreParams& sp, hipStream_t st) {
  AXON_LAUNCH_GEMM(gemm_store_kernel, g, sp, st);
  return AXON_OK;
}

// The same with operands that are K-major ([k][rows], see DmaLoopT): the rows are fetched as 16-byte
// vectors, so the row count (edge tiles are shifted back by it), the leading dimension and the base are
// multiples of 8 elements.  The DMA loop only: the caller keeps a K-contiguous copy for other shapes.
inline bool kmajor_ok(const void* p, int64_t ld, int rows) {
  return rows % 8 == 0 && ld % 8 == 0 && (reinterpret_cast<uintptr_t>(p) & 15) == 0;
}
template <class Loop>
int launch_store_loop(const GemmOperands& g, const StoreParams& sp, hipStream_t st) {
  const int tiles_m = (g.m_rows + kTile - 1) / kTile, tiles_n = (g.n_rows + kTile - 1) / kTile;
  if (set_lds(gemm_store_kernel<Loop>) != AXON_OK) return AXON_ERR_LAUNCH;
  hipLaunchKernelGGL(gemm_store_kernel<Loop>, dim3(tiles_m * tiles_n), dim3(kGemmThreads), kGemmLdsBytes, st, g,
                     sp, tiles_m, tiles_n);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}
bool store_kmajor_ok(const GemmOperands& g, bool a_kmajor, bool b_kmajor) {
  return dma_ok(g) && (!a_kmajor || kmajor_ok(g.a, g.lda, g.m_rows)) && (!b_kmajor || kmajor_ok(g.b, g.ldb, g.n_rows));
}
int launch_store_kmajor(const GemmOperands& g, const StoreParams& sp, bool a_kmajor, bool b_kmajor,
                        hipStream_t st) {
  if (!a_kmajor && !b_kmajor) return launch_store(g, sp, st);
  if (!store_kmajor_ok(g, a_kmajor, b_kmajor)) return AXON_ERR_SHAPE;
  if (a_kmajor && b_kmajor) return launch_store_loop<DmaLoopT<true, true>>(g, sp, st);
  if (a_kmajor) return launch_store_loop<DmaLoopT<true, false>>(g, sp, st);
  return launch_store_loop<DmaLoopT<false, true>>(g, sp, st);
}

int launch_transpose(const void* in, int64_t ld_in, int rows, int cols, void* out, int64_t ld_out,
                     int rows_pad, hipStream_t st) {
  if ((ld_in | ld_out) % 8 != 0 ||
      ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15))
    return AXON_ERR_ARG;
  const dim3 grid((rows_pad + 63) / 64, (cols + 63) / 64);
  hipLaunchKernelGGL(transpose_bf16_kernel, grid, dim3(256), 0, st,
                     static_cast<const uint16_t*>(in), ld_in, rows, cols,
                     static_cast<uint16_t*>(out), ld_out, rows_pad);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

int launch_zero_cols(void* p, int64_t ld, int rows, int col0, int ncols, hipStream_t st) {
  if (ncols <= 0 || rows <= 0) return AXON_OK;
  const int64_t total = (int64_t)rows * ncols;
  const int64_t blocks = (total + 255) / 256;
  const int grid = (int)(blocks < 2048 ? blocks : 2048);
  hipLaunchKernelGGL(zero_cols_bf16_kernel, dim3(grid), dim3(256), 0, st, static_cast<uint16_t*>(p),
                     ld, rows, col0, ncols);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

int fwd_impl(const void* hidden, const void* weight, const void* labels, int labels_i64, int64_t n,
             int64_t h, int64_t v, float inv_temp, float softcap, const uint8_t* is_start,
             int64_t last_dst, float* logprobs, float* entropy, float* lse, float* entropy_b,
             void* workspace, int64_t ws_bytes, void* stash, int64_t stash_bytes, void* stream,
             PhaseTimer* timer) {
  int rc = check_head_shape(n, h, v);
  if (rc != AXON_OK) return rc;
  if (n == 0) return AXON_OK;
  if (!hidden || !weight || !labels || !logprobs || !entropy || !lse || !entropy_b || !workspace)
    return AXON_ERR_ARG;
  if (!(inv_temp > 0.f) || !(softcap >= 0.f)) return AXON_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(hidden) | reinterpret_cast<uintptr_t>(weight)) & 15)
    return AXON_ERR_ARG;
  char* base = reinterpret_cast<char*>(round_up(reinterpret_cast<int64_t>(workspace), kAlign));
  FwdWs w = fwd_ws(n, v, base);
  if ((base - static_cast<char*>(workspace)) + w.bytes > ws_bytes) return AXON_ERR_WORKSPACE;
  const hipStream_t st = (hipStream_t)stream;
  StashWs sw{};
  if (stash) {
    if (reinterpret_cast<uintptr_t>(stash) & 15) return AXON_ERR_ARG;
    sw = stash_ws(n, h, v, stash);
    if (sw.bytes == 0) return AXON_ERR_SHAPE;
    if (sw.bytes > stash_bytes) return AXON_ERR_WORKSPACE;
    w.pm = sw.pm;  // the backward needs the per-part maxima: they live in the stash
  }

  GemmOperands g;
  g.a = static_cast<const __bf16*>(weight);  g.lda = h;  g.m_rows = (int)v;
  g.b = static_cast<const __bf16*>(hidden);  g.ldb = h;  g.n_rows = (int)n;
  g.k = (int)h;
  FwdParams p{w.pm, w.ps, w.pe, (int)n, (int)v, inv_temp * kLog2e, softcap,
              softcap > 0.f ? 1.f / softcap : 0.f, sw.tiles};
  {
    Span span(timer, 0);
    if (stash) {
      if (softcap > 0.f)
        AXON_LAUNCH_GEMM(lmhead_fwd_softcap_stash_kernel, g, p, st);
      else
        AXON_LAUNCH_GEMM(lmhead_fwd_stash_kernel, g, p, st);
    } else if (softcap > 0.f) {
      AXON_LAUNCH_GEMM(lmhead_fwd_softcap_kernel, g, p, st);
    } else {
      AXON_LAUNCH_GEMM(lmhead_fwd_kernel, g, p, st);
    }
  }
  {
    Span span(timer, 1);
    hipLaunchKernelGGL(lmhead_merge_kernel, dim3((unsigned)((n + kMergeTokens - 1) / kMergeTokens)),
                       dim3(kMergeTokens * kMergeGroups), 0, st,
                       w.pm, w.ps, w.pe, w.parts, (int)n, lse, entropy_b, entropy, w.fin_max,
                       w.fin_log2s, is_start, (int)last_dst);
  }
  AXON_CHECK_LAUNCH();
  const dim3 lg((unsigned)((n + 3) / 4));
  Span span(timer, 2);
  if (labels_i64)
    hipLaunchKernelGGL(lmhead_label_kernel<int64_t>, lg, dim3(256), 0, st,
                       static_cast<const __bf16*>(hidden), static_cast<const __bf16*>(weight),
                       static_cast<const int64_t*>(labels), (int)n, (int)h, (int)v, inv_temp,
                       softcap, w.fin_max, w.fin_log2s, logprobs, is_start, (int)last_dst);
  else
    hipLaunchKernelGGL(lmhead_label_kernel<int32_t>, lg, dim3(256), 0, st,
                       static_cast<const __bf16*>(hidden), static_cast<const __bf16*>(weight),
                       static_cast<const int32_t*>(labels), (int)n, (int)h, (int)v, inv_temp,
                       softcap, w.fin_max, w.fin_log2s, logprobs, is_start, (int)last_dst);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

// A backward over a block of consecutive tokens of a longer stream (one call per block, one stream):
// where the last row's label and gradients live (aligned_pos), whether the workspace already holds the
// transposed weight (written by the step's first call), and how this block's share of the weight
// gradient leaves: the blocks of a step add up in one fp32 array, the last one rounds the sum to bf16.
enum { kDwStore = 0, kDwFirst = 1, kDwAdd = 2, kDwLast = 3 };
struct BlockArgs {
  int64_t last_dst = 0;
  int wt_ready = 0;
  int dw_mode = kDwStore;
  float* dw_acc = nullptr;  // axon_lmhead_block_dw_acc_bytes of fp32 partial sums, tile order (modes other than kDwStore)
  // Several consecutive blocks may share ONE weight-gradient GEMM (a longer reduction, fewer passes over
  // the fp32 partial sums): each keeps its dlogits and its transposed hidden rows in the workspace, at
  // `group_pos` tokens from the start (a multiple of 256, the blocks before it rounded up to that), and
  // the GEMM runs with the block that says `dw_now` over everything up to its end.  `ws_tokens`: the
  // tokens the workspace was sized for (0: this call's), the same for every call that shares it.
  int64_t group_pos = 0;
  int dw_now = 1;
  int64_t ws_tokens = 0;
};

int bwd_impl(const float* dlogprobs, const float* dentropy, const void* hidden, const void* weight,
             const void* labels, int labels_i64, const float* lse, const float* entropy_b,
             int64_t n, int64_t h, int64_t v, float inv_temp, float softcap,
             const uint8_t* is_start, void* d_hidden, void* d_weight, int64_t chunk, void* workspace,
             int64_t ws_bytes, const void* stash, int64_t stash_bytes, void* stream, PhaseTimer* timer,
             const BlockArgs& blk = BlockArgs()) {
  int rc = check_head_shape(n, h, v);
  if (rc != AXON_OK) return rc;
  if (chunk < 0 || chunk % kTile != 0) return AXON_ERR_ARG;
  if (!weight) return AXON_ERR_ARG;
  if (blk.dw_mode < kDwStore || blk.dw_mode > kDwLast) return AXON_ERR_ARG;
  if (blk.dw_mode != kDwStore && (!blk.dw_acc || (reinterpret_cast<uintptr_t>(blk.dw_acc) & 15) || n == 0))
    return AXON_ERR_ARG;
  const bool dw_bf16 = blk.dw_now && (blk.dw_mode == kDwStore || blk.dw_mode == kDwLast);
  if (dw_bf16 && !d_weight) return AXON_ERR_ARG;
  const hipStream_t st = (hipStream_t)stream;
  if (n == 0) return axon_fill_zero(d_weight, v * h * 2, stream);
  if (!dlogprobs || !hidden || !labels || !lse || !entropy_b || !d_hidden || !workspace)
    return AXON_ERR_ARG;
  if (!(inv_temp > 0.f) || !(softcap >= 0.f)) return AXON_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(hidden) | reinterpret_cast<uintptr_t>(weight) |
       reinterpret_cast<uintptr_t>(d_hidden) | (dw_bf16 ? reinterpret_cast<uintptr_t>(d_weight) : 0)) & 15)
    return AXON_ERR_ARG;
  const int64_t pos = blk.group_pos, n_tile = round_up(n, kTile);
  const int64_t ws_tokens = blk.ws_tokens > 0 ? blk.ws_tokens : n;
  if (pos < 0 || pos % kTile != 0 || pos + n_tile > round_up(ws_tokens, kTile)) return AXON_ERR_ARG;
  char* base = reinterpret_cast<char*>(round_up(reinterpret_cast<int64_t>(workspace), kAlign));
  const BwdWs w = bwd_ws(ws_tokens, h, v, chunk, base);
  if ((base - static_cast<char*>(workspace)) + w.bytes > ws_bytes) return AXON_ERR_WORKSPACE;
  // blocks that share a weight-gradient GEMM keep their dlogits of the whole vocabulary side by side
  if ((pos > 0 || !blk.dw_now) && !(w.dl_kmajor && w.chunks == 1)) return AXON_ERR_ARG;
  StashWs sw{};
  if (stash) {
    if (reinterpret_cast<uintptr_t>(stash) & 15) return AXON_ERR_ARG;
    sw = stash_ws(n, h, v, const_cast<void*>(stash));
    if (sw.bytes == 0) return AXON_ERR_SHAPE;
    if (sw.bytes > stash_bytes) return AXON_ERR_WORKSPACE;
  }

  // K-contiguous copies for the two output GEMMs
  {
    Span span(timer, 0);
    if (!blk.wt_ready && !w.w_kmajor) {
      rc = launch_transpose(weight, h, (int)v, (int)h, w.wT, w.ld_v, (int)w.v_pad, st);
      if (rc != AXON_OK) return rc;
    }
    rc = launch_transpose(hidden, h, (int)n, (int)h, w.hT + pos, w.ld_n, (int)n_tile, st);
    if (rc != AXON_OK) return rc;
  }
  const int64_t n_red = round_up(n, 64);  // reduction length of B3 (from this block's first token)
  const int64_t tiles_h = round_up(h, kTile) / kTile;
  __bf16* const dl = w.dl + pos * w.ld_c;  // this block's rows

  for (int ci = 0; ci < w.chunks; ++ci) {
    const int64_t v0 = (int64_t)ci * w.chunk;
    const int64_t vc = (v - v0 < w.chunk) ? (v - v0) : w.chunk;  // valid vocab rows in this chunk
    const int64_t vc_red = round_up(vc, 64);                      // reduction length of B2
    // B1: dlogit for vocab rows [v0, v0 + vc)
    {
      Span span(timer, 1);
      GemmOperands g;
      g.a = static_cast<const __bf16*>(weight) + v0 * h;  g.lda = h;  g.m_rows = (int)vc;
      g.b = static_cast<const __bf16*>(hidden);            g.ldb = h;  g.n_rows = (int)n;
      g.k = (int)h;
      DlogitParams p;
      p.lse = lse; p.entropy_b = entropy_b; p.dlogprobs = dlogprobs; p.dentropy = dentropy;
      p.labels = labels; p.labels_i64 = labels_i64;
      p.dl = dl; p.dlT = w.dlT; p.ld_dl = w.ld_c; p.ld_dlT = w.ld_n;
      p.n_tokens = (int)n; p.vocab = (int)v; p.v_begin = (int)v0; p.inv_temp = inv_temp;
      p.cap = softcap; p.inv_cap = softcap > 0.f ? 1.f / softcap : 0.f;
      p.is_start = is_start;
      p.last_dst = (int)blk.last_dst;
      if (stash) {
        const StashSource src{sw.tiles, sw.pm, sw.tiles_n, (int)(v0 / kTile), sw.shifted};
        const unsigned blocks = (unsigned)(round_up(vc, kTile) / kTile) * (unsigned)sw.tiles_n * 8u;
        if (softcap > 0.f)
          hipLaunchKernelGGL(lmhead_dlogit_stash_kernel<true>, dim3(blocks), dim3(64), 0, st, p, src);
        else
          hipLaunchKernelGGL(lmhead_dlogit_stash_kernel<false>, dim3(blocks), dim3(64), 0, st, p, src);
        AXON_CHECK_LAUNCH();
      } else if (softcap > 0.f) {
        AXON_LAUNCH_GEMM(lmhead_dlogit_softcap_kernel, g, p, st);
      } else {
        AXON_LAUNCH_GEMM(lmhead_dlogit_kernel, g, p, st);
      }
      // reduction padding the tiles did not cover (the shifted-tile path writes no padding; the
      // clamped path writes zeros there already, the extra fill is then redundant but harmless)
      rc = launch_zero_cols(dl, w.ld_c, (int)n, (int)vc, (int)(vc_red - vc), st);
      if (rc != AXON_OK) return rc;
      // the token rows up to the next tile boundary: reduction padding of B3 when it reads dl K-major, and
      // rows of B2's operand when fewer than 256 tokens run on the DMA loop
      if (w.dl_kmajor || (w.w_kmajor && n < kTile))
        rc = launch_zero_cols(dl + n * w.ld_c, w.ld_c, (int)(n_tile - n), 0, (int)vc_red, st);
      if (rc == AXON_OK && !w.dl_kmajor)
        rc = launch_zero_cols(w.dlT, w.ld_n, (int)vc, (int)n, (int)(n_red - n), st);
      if (rc != AXON_OK) return rc;
    }
    // B2: dHidden[n][h] (+)= sum_v dl[n][v] * W[v0 + v][h]  (the weight read K-major where it lies, or its
    // transposed copy wT[h][v0 + v])
    {
      Span span(timer, 2);
      GemmOperands g;
      if (w.w_kmajor) { g.a = static_cast<const __bf16*>(weight) + v0 * h;  g.lda = h; }
      else            { g.a = w.wT + v0;                                     g.lda = w.ld_v; }
      g.m_rows = (int)h;
      // fewer than 256 tokens: the zero rows up to 256 are part of the operand, the stores stop at n
      g.b = dl;  g.ldb = w.ld_c;  g.n_rows = (int)((w.w_kmajor && n < kTile) ? kTile : n);
      g.k = (int)vc_red;
      StoreParams sp;
      const bool last = (ci == w.chunks - 1);
      sp.out_f32 = (w.chunks > 1) ? w.dh_acc : nullptr;  sp.ld_f32 = h;
      sp.out_bf16 = last ? static_cast<__bf16*>(d_hidden) : nullptr;  sp.ld_bf16 = h;
      sp.m_valid = (int)h; sp.n_valid = (int)n; sp.accumulate = (ci > 0); sp.keep_f32 = 1;
      sp.tile_acc = nullptr;
      rc = launch_store_kmajor(g, sp, w.w_kmajor, false, st);
      if (rc != AXON_OK) return rc;
    }
    // B3: dWeight[v0 + v][h] = sum_t dl[t][v] * hT[h][t] over the tokens the workspace holds up to this
    // block's end (dl read as the K-major operand, or its vocab-major copy dlT[v][t])
    if (blk.dw_now) {
      Span span(timer, 3);
      GemmOperands g;
      g.a = w.hT;  g.lda = w.ld_n;  g.m_rows = (int)h;
      if (w.dl_kmajor) { g.b = w.dl;   g.ldb = w.ld_c; }
      else             { g.b = w.dlT;  g.ldb = w.ld_n; }
      g.n_rows = (int)vc;
      g.k = (int)(pos + n_red);
      StoreParams sp;
      sp.out_f32 = nullptr;  sp.ld_f32 = 0;
      sp.tile_acc = blk.dw_mode == kDwStore
                        ? nullptr
                        : reinterpret_cast<float4*>(blk.dw_acc) + (v0 / kTile) * tiles_h * kTileAccVecs;
      sp.out_bf16 = dw_bf16 ? static_cast<__bf16*>(d_weight) + v0 * h : nullptr;  sp.ld_bf16 = h;
      sp.m_valid = (int)h; sp.n_valid = (int)vc;
      sp.accumulate = blk.dw_mode == kDwAdd || blk.dw_mode == kDwLast;
      sp.keep_f32 = blk.dw_mode != kDwLast;
      rc = launch_store_kmajor(g, sp, false, w.dl_kmajor, st);
      if (rc != AXON_OK) return rc;
    }
  }
  return AXON_OK;
}

}  // namespace


extern "C" int axon_seq_start_flags(const int32_t* cu_seqlens, int64_t n_seqs, int64_t n_tokens,
                                    uint8_t* flags, void* stream) {
  if (n_seqs < 0 || n_tokens < 0 || n_tokens >= (int64_t)INT32_MAX || n_seqs >= (int64_t)INT32_MAX)
    return AXON_ERR_SHAPE;
  if (n_tokens == 0) return AXON_OK;
  if (!flags || (n_seqs > 0 && !cu_seqlens)) return AXON_ERR_ARG;
  int rc = axon_fill_zero(flags, round_up(n_tokens, 4), stream);
  if (rc != AXON_OK) return rc;
  if (n_seqs == 0) return AXON_OK;
  hipLaunchKernelGGL(seq_start_kernel, dim3((unsigned)((n_seqs + 255) / 256)), dim3(256), 0,
                     (hipStream_t)stream, cu_seqlens, (int)n_seqs, (int)n_tokens, flags);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

extern "C" int axon_lmhead_active_rows(const float* dlogprobs, const float* dentropy,
                                       const uint8_t* seq_start, int64_t n, int32_t* row_index,
                                       int32_t* row_rank, int32_t* count, void* stream) {
  if (n < 0 || n >= (int64_t)INT32_MAX - 8192) return AXON_ERR_SHAPE;  // the walk steps by 4096
  if (!count) return AXON_ERR_ARG;
  if (n > 0 && (!dlogprobs || !row_index || !row_rank)) return AXON_ERR_ARG;
  hipLaunchKernelGGL(active_rows_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, dlogprobs,
                     dentropy, seq_start, (int)n, row_index, row_rank, count);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

extern "C" int axon_lmhead_gather_rows(const void* hidden, const void* labels, int labels_i64,
                                       const float* lse, const float* entropy_b,
                                       const float* dlogprobs, const float* dentropy,
                                       const uint8_t* seq_start, int64_t n, int64_t h,
                                       const int32_t* row_index, int64_t n_active, void* hidden_c,
                                       void* labels_c, float* lse_c, float* entropy_b_c,
                                       float* dlogprobs_c, float* dentropy_c, void* stream) {
  if (n < 0 || n >= (int64_t)INT32_MAX || n_active < 0 || n_active > n) return AXON_ERR_SHAPE;
  if (h < 8 || h % 8 != 0 || h / 8 >= (int64_t)INT32_MAX) return AXON_ERR_SHAPE;
  if (n_active == 0) return AXON_OK;
  if (!hidden || !labels || !lse || !entropy_b || !dlogprobs || !row_index || !hidden_c ||
      !labels_c || !lse_c || !entropy_b_c || !dlogprobs_c)
    return AXON_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(hidden) | reinterpret_cast<uintptr_t>(hidden_c)) & 15)
    return AXON_ERR_ARG;
  const dim3 grid((unsigned)n_active), block(256);
  const hipStream_t st = (hipStream_t)stream;
  if (labels_i64)
    hipLaunchKernelGGL(gather_rows_kernel<int64_t>, grid, block, 0, st,
                       static_cast<const uint4*>(hidden), (int)(h / 8),
                       static_cast<const int64_t*>(labels), lse, entropy_b, dlogprobs, dentropy,
                       seq_start, (int)n, row_index, static_cast<uint4*>(hidden_c),
                       static_cast<int64_t*>(labels_c), lse_c, entropy_b_c, dlogprobs_c, dentropy_c);
  else
    hipLaunchKernelGGL(gather_rows_kernel<int32_t>, grid, block, 0, st,
                       static_cast<const uint4*>(hidden), (int)(h / 8),
                       static_cast<const int32_t*>(labels), lse, entropy_b, dlogprobs, dentropy,
                       seq_start, (int)n, row_index, static_cast<uint4*>(hidden_c),
                       static_cast<int32_t*>(labels_c), lse_c, entropy_b_c, dlogprobs_c, dentropy_c);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

extern "C" int axon_lmhead_scatter_rows(const void* d_hidden_c, const int32_t* row_rank, int64_t n,
                                        int64_t h, void* d_hidden, void* stream) {
  if (n < 0 || n >= (int64_t)INT32_MAX) return AXON_ERR_SHAPE;
  if (h < 8 || h % 8 != 0 || h / 8 >= (int64_t)INT32_MAX) return AXON_ERR_SHAPE;
  if (n == 0) return AXON_OK;
  if (!row_rank || !d_hidden) return AXON_ERR_ARG;  // d_hidden_c may be NULL when no row is active
  if ((reinterpret_cast<uintptr_t>(d_hidden_c) | reinterpret_cast<uintptr_t>(d_hidden)) & 15)
    return AXON_ERR_ARG;
  hipLaunchKernelGGL(scatter_rows_kernel, dim3((unsigned)n), dim3(256), 0, (hipStream_t)stream,
                     static_cast<const uint4*>(d_hidden_c), row_rank, (int)(h / 8),
                     static_cast<uint4*>(d_hidden));
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

extern "C" int64_t axon_lmhead_fwd_workspace_bytes(int64_t n, int64_t h, int64_t v) {
  if (check_head_shape(n, h, v) != AXON_OK) return -1;
  return fwd_ws(n, v, nullptr).bytes + kAlign;
}

extern "C" int64_t axon_lmhead_stash_bytes(int64_t n, int64_t h, int64_t v) {
  if (check_head_shape(n, h, v) != AXON_OK) return -1;
  return stash_ws(n, h, v, nullptr).bytes;
}

extern "C" int axon_lmhead_fwd(const void* hidden, const void* weight, const void* labels,
                               int labels_i64, int64_t n, int64_t h, int64_t v, float inv_temp,
                               float softcap, const uint8_t* seq_start, float* logprobs,
                               float* entropy, float* lse, float* entropy_b, void* workspace,
                               int64_t ws_bytes, void* stash, int64_t stash_bytes, void* stream) {
  return fwd_impl(hidden, weight, labels, labels_i64, n, h, v, inv_temp, softcap, seq_start, 0,
                  logprobs, entropy, lse, entropy_b, workspace, ws_bytes, stash, stash_bytes, stream,
                  nullptr);
}

extern "C" void* axon_timer_create(void* stream) { return new (std::nothrow) PhaseTimer((hipStream_t)stream); }

extern "C" int axon_timer_collect(void* timer, float* phase_ms, int32_t* phase_launches) {
  if (!timer || !phase_ms || !phase_launches) return AXON_ERR_ARG;
  static_cast<PhaseTimer*>(timer)->collect(phase_ms, phase_launches, 8);
  return AXON_OK;
}

extern "C" void axon_timer_destroy(void* timer) {
  if (!timer) return;
  float ms[8] = {0};
  int32_t n[8] = {0};
  static_cast<PhaseTimer*>(timer)->collect(ms, n, 8);  // releases the events
  delete static_cast<PhaseTimer*>(timer);
}

extern "C" int axon_lmhead_fwd_timed(const void* hidden, const void* weight, const void* labels,
                                     int labels_i64, int64_t n, int64_t h, int64_t v,
                                     float inv_temp, float softcap, const uint8_t* seq_start,
                                     float* logprobs, float* entropy, float* lse,
                                     float* entropy_b, void* workspace, int64_t ws_bytes,
                                     void* stash, int64_t stash_bytes, void* stream, void* timer) {
  if (!timer) return AXON_ERR_ARG;
  PhaseTimer* t = static_cast<PhaseTimer*>(timer);
  if (t->st != (hipStream_t)stream) return AXON_ERR_ARG;
  t->base = 0;
  return fwd_impl(hidden, weight, labels, labels_i64, n, h, v, inv_temp, softcap, seq_start, 0, logprobs,
                  entropy, lse, entropy_b, workspace, ws_bytes, stash, stash_bytes, stream, t);
}

extern "C" int64_t axon_lmhead_bwd_workspace_bytes(int64_t n, int64_t h, int64_t v,
                                                   int64_t chunk) {
  if (check_head_shape(n, h, v) != AXON_OK) return -1;
  if (chunk < 0 || chunk % kTile != 0) return -1;
  return bwd_ws(n, h, v, chunk, nullptr).bytes + kAlign;
}

extern "C" int axon_lmhead_bwd(const float* dlogprobs, const float* dentropy, const void* hidden,
                               const void* weight, const void* labels, int labels_i64,
                               const float* lse, const float* entropy_b, int64_t n, int64_t h,
                               int64_t v, float inv_temp, float softcap, const uint8_t* seq_start,
                               void* d_hidden, void* d_weight, int64_t chunk, void* workspace,
                               int64_t ws_bytes, const void* stash, int64_t stash_bytes, void* stream) {
  return bwd_impl(dlogprobs, dentropy, hidden, weight, labels, labels_i64, lse, entropy_b, n, h, v,
                  inv_temp, softcap, seq_start, d_hidden, d_weight, chunk, workspace, ws_bytes,
                  stash, stash_bytes, stream, nullptr);
}

extern "C" int axon_lmhead_bwd_timed(const float* dlogprobs, const float* dentropy,
                                     const void* hidden, const void* weight, const void* labels,
                                     int labels_i64, const float* lse, const float* entropy_b,
                                     int64_t n, int64_t h, int64_t v, float inv_temp,
                                     float softcap, const uint8_t* seq_start, void* d_hidden,
                                     void* d_weight, int64_t chunk, void* workspace,
                                     int64_t ws_bytes, const void* stash, int64_t stash_bytes,
                                     void* stream, void* timer) {
  if (!timer) return AXON_ERR_ARG;
  PhaseTimer* t = static_cast<PhaseTimer*>(timer);
  if (t->st != (hipStream_t)stream) return AXON_ERR_ARG;
  t->base = 4;
  return bwd_impl(dlogprobs, dentropy, hidden, weight, labels, labels_i64, lse, entropy_b, n, h, v,
                  inv_temp, softcap, seq_start, d_hidden, d_weight, chunk, workspace, ws_bytes, stash,
                  stash_bytes, stream, t);
}

extern "C" int axon_gemm_nt_bf16(const void* a, int64_t lda, const void* b, int64_t ldb, float* out,
                                 int64_t ldo, int64_t m, int64_t n, int64_t k, void* stream) {
  if (!a || !b || !out) return AXON_ERR_ARG;
  if (m <= 0 || n <= 0 || k <= 0) return AXON_ERR_ARG;
  if (k % 32 != 0 || lda % 8 != 0 || ldb % 8 != 0 || m % 4 != 0 || ldo % 4 != 0)
    return AXON_ERR_SHAPE;
  if (m >= (1 << 30) || n >= (1 << 30)) return AXON_ERR_SHAPE;
  GemmOperands g;
  g.a = static_cast<const __bf16*>(a);  g.lda = lda;  g.m_rows = (int)m;
  g.b = static_cast<const __bf16*>(b);  g.ldb = ldb;  g.n_rows = (int)n;
  g.k = (int)k;
  StoreParams sp;
  sp.out_f32 = out; sp.ld_f32 = ldo; sp.out_bf16 = nullptr; sp.ld_bf16 = 0;
  sp.m_valid = (int)m; sp.n_valid = (int)n; sp.accumulate = 0; sp.keep_f32 = 1; sp.tile_acc = nullptr;
  return launch_store(g, sp, (hipStream_t)stream);
}

extern "C" int axon_gemm_bf16(const void* a, int64_t lda, int a_kmajor, const void* b, int64_t ldb,
                              int b_kmajor, float* out, int64_t ldo, int64_t m, int64_t n, int64_t k,
                              void* stream) {
  if (!a || !b || !out) return AXON_ERR_ARG;
  if (m <= 0 || n <= 0 || k <= 0) return AXON_ERR_ARG;
  if (k % 32 != 0 || lda % 8 != 0 || ldb % 8 != 0 || m % 4 != 0 || ldo % 4 != 0) return AXON_ERR_SHAPE;
  if (m >= (1 << 30) || n >= (1 << 30)) return AXON_ERR_SHAPE;
  GemmOperands g;
  g.a = static_cast<const __bf16*>(a);  g.lda = lda;  g.m_rows = (int)m;
  g.b = static_cast<const __bf16*>(b);  g.ldb = ldb;  g.n_rows = (int)n;
  g.k = (int)k;
  StoreParams sp;
  sp.out_f32 = out; sp.ld_f32 = ldo; sp.out_bf16 = nullptr; sp.ld_bf16 = 0;
  sp.m_valid = (int)m; sp.n_valid = (int)n; sp.accumulate = 0; sp.keep_f32 = 1; sp.tile_acc = nullptr;
  return launch_store_kmajor(g, sp, a_kmajor != 0, b_kmajor != 0, (hipStream_t)stream);
}

// ----------------------------------------------------------------------------
// One step as token blocks: forward (with stash), loss and backward of one block of consecutive
// tokens before the next block's forward, so that what is kept from a forward to its backward is
// one block's stash whatever the number of tokens.  One call per block and phase, all on one stream.
// ----------------------------------------------------------------------------
namespace {
PhaseTimer* block_timer(void* timer, void* stream, int base, int* rc) {
  *rc = AXON_OK;
  if (!timer) return nullptr;
  PhaseTimer* t = static_cast<PhaseTimer*>(timer);
  if (t->st != (hipStream_t)stream) { *rc = AXON_ERR_ARG; return nullptr; }
  t->base = base;
  return t;
}
bool last_dst_ok(int64_t last_dst, int64_t n) { return last_dst <= n && last_dst > -(int64_t(1) << 30); }
}  // namespace

extern "C" int64_t axon_lmhead_block_dw_acc_bytes(int64_t h, int64_t v) {
  if (check_head_shape(0, h, v) != AXON_OK) return -1;
  return (round_up(h, kTile) / kTile) * (round_up(v, kTile) / kTile) * kTileAccVecs * 16;
}

extern "C" int axon_lmhead_bwd_dlogit_copies(int64_t h, int64_t v, int64_t chunk) {
  if (check_head_shape(0, h, v) != AXON_OK || chunk < 0 || chunk % kTile != 0) return -1;
  return bwd_ws(kTile, h, v, chunk, nullptr).dl_kmajor ? 1 : 2;
}

extern "C" int axon_lmhead_block_can_group(int64_t h, int64_t v, int64_t chunk) {
  if (check_head_shape(0, h, v) != AXON_OK || chunk < 0 || chunk % kTile != 0) return 0;
  const BwdWs w = bwd_ws(kTile, h, v, chunk, nullptr);
  return (w.dl_kmajor && w.chunks == 1) ? 1 : 0;
}

extern "C" int axon_lmhead_block_begin(const void* weight, int64_t h, int64_t v, int64_t chunk,
                                       void* workspace, int64_t ws_bytes, void* stream, void* timer) {
  int rc = check_head_shape(0, h, v);
  if (rc != AXON_OK) return rc;
  if (chunk < 0 || chunk % kTile != 0) return AXON_ERR_ARG;
  if (!weight || !workspace || (reinterpret_cast<uintptr_t>(weight) & 15)) return AXON_ERR_ARG;
  PhaseTimer* t = block_timer(timer, stream, 4, &rc);
  if (rc != AXON_OK) return rc;
  char* base = reinterpret_cast<char*>(round_up(reinterpret_cast<int64_t>(workspace), kAlign));
  const BwdWs w = bwd_ws(0, h, v, chunk, base);
  if (w.w_kmajor) return AXON_OK;  // the dHidden GEMM reads the weight where it lies
  if ((base - static_cast<char*>(workspace)) + round_up(h * w.ld_v * 2, kAlign) > ws_bytes)
    return AXON_ERR_WORKSPACE;
  Span span(t, 0);
  return launch_transpose(weight, h, (int)v, (int)h, w.wT, w.ld_v, (int)w.v_pad, (hipStream_t)stream);
}

extern "C" int axon_lmhead_block_fwd(const void* hidden, const void* weight, const void* labels,
                                     int labels_i64, int64_t n, int64_t h, int64_t v, float inv_temp,
                                     float softcap, const uint8_t* seq_start, int64_t last_dst,
                                     float* logprobs, float* entropy, float* lse, float* entropy_b,
                                     void* workspace, int64_t ws_bytes, void* stash,
                                     int64_t stash_bytes, void* stream, void* timer) {
  if (!last_dst_ok(last_dst, n)) return AXON_ERR_ARG;
  int rc;
  PhaseTimer* t = block_timer(timer, stream, 0, &rc);
  if (rc != AXON_OK) return rc;
  return fwd_impl(hidden, weight, labels, labels_i64, n, h, v, inv_temp, softcap, seq_start, last_dst,
                  logprobs, entropy, lse, entropy_b, workspace, ws_bytes, stash, stash_bytes, stream, t);
}

extern "C" int axon_lmhead_block_bwd(const float* dlogprobs, const float* dentropy, const void* hidden,
                                     const void* weight, const void* labels, int labels_i64,
                                     const float* lse, const float* entropy_b, int64_t n, int64_t h,
                                     int64_t v, float inv_temp, float softcap,
                                     const uint8_t* seq_start, int64_t last_dst, void* d_hidden,
                                     void* d_weight, float* dw_acc, int dw_mode, int wt_ready,
                                     int64_t group_pos, int dw_now, int64_t ws_tokens,
                                     int64_t chunk, void* workspace, int64_t ws_bytes,
                                     const void* stash, int64_t stash_bytes, void* stream,
                                     void* timer) {
  if (!last_dst_ok(last_dst, n) || n <= 0) return AXON_ERR_ARG;
  int rc;
  PhaseTimer* t = block_timer(timer, stream, 4, &rc);
  if (rc != AXON_OK) return rc;
  BlockArgs blk;
  blk.last_dst = last_dst;
  blk.wt_ready = wt_ready != 0;
  blk.dw_mode = dw_mode;
  blk.dw_acc = dw_acc;
  blk.group_pos = group_pos;
  blk.dw_now = dw_now != 0;
  blk.ws_tokens = ws_tokens;
  return bwd_impl(dlogprobs, dentropy, hidden, weight, labels, labels_i64, lse, entropy_b, n, h, v,
                  inv_temp, softcap, seq_start, d_hidden, d_weight, chunk, workspace, ws_bytes, stash,
                  stash_bytes, stream, t, blk);
}

extern "C" int axon_scale_bf16_unless_one(void* x, int64_t n, const float* scale, void* stream) {
  if (n < 0 || n % 8 != 0) return AXON_ERR_SHAPE;
  if (n == 0) return AXON_OK;
  if (!x || !scale || (reinterpret_cast<uintptr_t>(x) & 15)) return AXON_ERR_ARG;
  const int64_t n_vec = n / 8, blocks = (n_vec + 255) / 256;
  hipLaunchKernelGGL(scale_bf16_kernel, dim3((unsigned)(blocks < 4096 ? blocks : 4096)), dim3(256), 0,
                     (hipStream_t)stream, static_cast<uint4*>(x), n_vec, scale);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}
