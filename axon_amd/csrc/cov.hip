// Token selection of the covariance-based losses (axon/trainer/algos/loss/loss.py:198-352):
//   KL-Cov   picks the k tokens with the largest (A - mean A)(logp - mean logp) among the tokens with mask > 0;
//   Clip-Cov picks k tokens at random among the unclipped tokens whose covariance lies in a band.
// Both are a top-k over 32-bit keys: the covariance mapped to an order-preserving integer, or a hash of
// (token index, seed) for the random pick.  The k-th largest key is found by a three-round radix select
// (11 + 11 + 10 bits, histograms in LDS merged with integer atomics, so the result is reproducible); ties at
// the threshold go to the lowest token indices.
#include "common.h"

namespace axon {

constexpr int kBins = 2048;

__device__ __forceinline__ uint32_t order_key(float x) {
  const uint32_t b = __float_as_uint(x);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x ^= x >> 16; x *= 0x85ebca6bu; x ^= x >> 13; x *= 0xc2b2ae35u; x ^= x >> 16;
  return x;
}

__device__ __forceinline__ int round_shift(int round) { return round == 0 ? 21 : (round == 1 ? 10 : 0); }
__device__ __forceinline__ int round_bins(int round) { return round == 2 ? 1024 : 2048; }

// sums over the tokens: WEIGHTED: sum A m, sum logp m, sum m (masked_mean, loss/utils.py:88-91);
// otherwise over mask > 0: sum A, sum logp, count (loss.py:311-320)
template <int MK, bool WEIGHTED>
__global__ __launch_bounds__(kBlock) void cov_moments_kernel(const float* __restrict__ adv,
                                                             const float* __restrict__ logp,
                                                             const void* __restrict__ mask,
                                                             int64_t n_slots, float* partials) {
  __shared__ float lds_red[3 * (kBlock / kWave)];
  float a[3] = {0.f, 0.f, 0.f};
  const int64_t n_vec = n_slots / kVec;
  auto add = [&](float A, float l, float m) {
    if (WEIGHTED) { a[0] += A * m; a[1] += l * m; a[2] += m; }
    else if (m > 0.f) { a[0] += A; a[1] += l; a[2] += 1.f; }
  };
  for (int64_t q = (int64_t)blockIdx.x * kBlock + threadIdx.x; q < n_vec;
       q += (int64_t)gridDim.x * kBlock) {
    float av[4], lv[4], mv[4];
    load4(adv, q * kVec, av);
    load4(logp, q * kVec, lv);
    load_mask4<MK>(mask, q * kVec, mv);
#pragma unroll
    for (int j = 0; j < 4; ++j) add(av[j], lv[j], mv[j]);
  }
  if (blockIdx.x == 0 && threadIdx.x < (int)(n_slots - n_vec * kVec)) {
    const int64_t p = n_vec * kVec + threadIdx.x;
    add(adv[p], logp[p], load_mask1<MK>(mask, p));
  }
  store_block_partials<3>(a, lds_red, partials);
}

// kind 0 (KL-Cov): k = max(1, int(count * ratio)), 0 without tokens.  kind 1 (Clip-Cov):
// k = max(int(ratio * sum mask), 1), capped by the number of candidates once that is known.
__global__ __launch_bounds__(kBlock) void cov_moments_finish_kernel(const float* __restrict__ partials,
                                                                    int n_blocks, int kind, double ratio,
                                                                    SelectState* st, uint32_t* hist) {
  __shared__ float lds_red[3 * (kBlock / kWave)];
  __shared__ double lds_cnt[kBlock / kWave];
  float a[3] = {0.f, 0.f, 0.f};
  double cnt = 0.0;  // a workgroup's count is exact in fp32; their total may not be
  for (int b = threadIdx.x; b < n_blocks; b += kBlock) {
    a[0] += partials[(size_t)b * kPartialStride];
    a[1] += partials[(size_t)b * kPartialStride + 1];
    a[2] += partials[(size_t)b * kPartialStride + 2];
    cnt += (double)partials[(size_t)b * kPartialStride + 2];
  }
  for (int off = 32; off > 0; off >>= 1) cnt += __shfl_down(cnt, off, kWave);
  if ((threadIdx.x & (kWave - 1)) == 0) lds_cnt[threadIdx.x / kWave] = cnt;
  block_sum<3>(a, lds_red);  // has a workgroup barrier: lds_cnt is visible after it
  for (int b = threadIdx.x; b < kBins; b += kBlock) hist[b] = 0;
  if (threadIdx.x == 0) {
    double total = 0.0;
    for (int w = 0; w < kBlock / kWave; ++w) total += lds_cnt[w];
    const float den = (kind == 0) ? a[2] : fmaxf(a[2], 1.f);
    st->mean_a = a[2] > 0.f || kind == 1 ? a[0] / den : 0.f;
    st->mean_b = a[2] > 0.f || kind == 1 ? a[1] / den : 0.f;
    st->count = a[2];
    const long long want = (long long)(total * ratio);
    uint32_t k = (uint32_t)(want < 1 ? 1 : (want > 0x7fffffffLL ? 0x7fffffffLL : want));
    if (kind == 0 && !(a[2] > 0.f)) k = 0;
    st->k = k;
    st->threshold = 0;
    st->remaining = k;
    st->candidates = 0;
    st->ties = 0;
    st->index_limit = -1;
  }
}

// keys[i]: kind 0: the covariance in integer order for mask > 0, else 0.
//          kind 1: a non-zero hash of (i, seed) for the unclipped tokens with lb < covariance < ub, else 0.
template <int MK, int KIND>
__global__ __launch_bounds__(kBlock) void cov_key_kernel(
    const float* __restrict__ logp, const float* __restrict__ oldp, const float* __restrict__ adv,
    const void* __restrict__ mask, int64_t n_slots, float lb, float ub, float ratio_lo, float ratio_hi,
    uint32_t seed, SelectState* st, uint32_t* __restrict__ keys) {
  __shared__ float lds_red[kBlock / kWave];
  const float mean_a = st->mean_a, mean_b = st->mean_b;
  float cand[1] = {0.f};
  auto key_of = [&](int64_t i, float A, float l, float o, float m) -> uint32_t {
    if (!(m > 0.f)) return 0u;
    float cov = (A - mean_a) * (l - mean_b);
    if (cov == 0.f) cov = 0.f;  // -0 and +0 compare equal: one key for both
    if (KIND == 0) { cand[0] += 1.f; return order_key(cov); }
    const float r_ = expf(clampf(l - o, -kSafetyBound, kSafetyBound));
    const float p1 = -A * r_, p2 = -A * clampf(r_, ratio_lo, ratio_hi);
    if (p2 > p1 || !(cov < ub && cov > lb)) return 0u;
    cand[0] += 1.f;
    return mix32(mix32((uint32_t)i ^ seed) + (uint32_t)((uint64_t)i >> 32) + 0x9e3779b9u) | 1u;
  };
  const int64_t n_vec = n_slots / kVec;
  for (int64_t q = (int64_t)blockIdx.x * kBlock + threadIdx.x; q < n_vec;
       q += (int64_t)gridDim.x * kBlock) {
    float av[4], lv[4], ov[4] = {0.f, 0.f, 0.f, 0.f}, mv[4];
    load4(adv, q * kVec, av);
    load4(logp, q * kVec, lv);
    if (KIND == 1) load4(oldp, q * kVec, ov);
    load_mask4<MK>(mask, q * kVec, mv);
    uint4 k4;
    k4.x = key_of(q * kVec + 0, av[0], lv[0], ov[0], mv[0]);
    k4.y = key_of(q * kVec + 1, av[1], lv[1], ov[1], mv[1]);
    k4.z = key_of(q * kVec + 2, av[2], lv[2], ov[2], mv[2]);
    k4.w = key_of(q * kVec + 3, av[3], lv[3], ov[3], mv[3]);
    *reinterpret_cast<uint4*>(keys + q * kVec) = k4;
  }
  if (blockIdx.x == 0 && threadIdx.x < (int)(n_slots - n_vec * kVec)) {
    const int64_t p = n_vec * kVec + threadIdx.x;
    keys[p] = key_of(p, adv[p], logp[p], KIND == 1 ? oldp[p] : 0.f, load_mask1<MK>(mask, p));
  }
  block_sum<1>(cand, lds_red);
  if (threadIdx.x == 0 && cand[0] > 0.f) atomicAdd(&st->candidates, (uint32_t)cand[0]);
}

// histogram of this round's digit over the keys that carry the prefix found so far
__global__ __launch_bounds__(kBlock) void radix_hist_kernel(const uint32_t* __restrict__ keys,
                                                            int64_t n_slots, const SelectState* st,
                                                            int round, uint32_t* hist) {
  __shared__ uint32_t lds_hist[kBins];
  if (st->k == 0) return;
  for (int b = threadIdx.x; b < kBins; b += kBlock) lds_hist[b] = 0;
  __syncthreads();
  const int shift = round_shift(round);
  const uint32_t digit_mask = (uint32_t)round_bins(round) - 1u;
  const int above = shift + (round == 2 ? 10 : 11);  // bits above this digit
  const uint32_t prefix = st->threshold;
  auto take = [&](uint32_t key) {
    if (above < 32 && (key >> above) != (prefix >> above)) return;
    atomicAdd(&lds_hist[(key >> shift) & digit_mask], 1u);
  };
  const int64_t n_vec = n_slots / kVec;
  for (int64_t q = (int64_t)blockIdx.x * kBlock + threadIdx.x; q < n_vec;
       q += (int64_t)gridDim.x * kBlock) {
    const uint4 k4 = *reinterpret_cast<const uint4*>(keys + q * kVec);
    take(k4.x); take(k4.y); take(k4.z); take(k4.w);
  }
  if (blockIdx.x == 0 && threadIdx.x < (int)(n_slots - n_vec * kVec)) take(keys[n_vec * kVec + threadIdx.x]);
  __syncthreads();
  for (int b = threadIdx.x; b < kBins; b += kBlock)
    if (lds_hist[b] != 0) atomicAdd(hist + b, lds_hist[b]);
}

// one workgroup: walks the bins from the top until `remaining` elements are covered, extends the threshold by
// that bin's digit, clears the histogram for the next round
__global__ __launch_bounds__(kBlock) void radix_pick_kernel(uint32_t* hist, SelectState* st, int round) {
  __shared__ uint32_t lds_hist[kBins];
  for (int b = threadIdx.x; b < kBins; b += kBlock) {
    lds_hist[b] = hist[b];
    hist[b] = 0;
  }
  __syncthreads();
  if (threadIdx.x != 0 || st->k == 0) return;
  if (round == 0) {  // key 0 never wins: cap k by the number of candidates
    if (st->k > st->candidates) st->k = st->candidates;
    st->remaining = st->k;
    if (st->k == 0) return;
  }
  uint32_t need = st->remaining;
  int bin = round_bins(round) - 1;
  for (; bin > 0; --bin) {
    const uint32_t c = lds_hist[bin];
    if (c >= need) break;
    need -= c;
  }
  st->threshold |= (uint32_t)bin << round_shift(round);
  st->remaining = need;
  if (round == 2) {
    st->ties = lds_hist[bin];
    st->index_limit = (st->ties <= need) ? INT64_MAX : -1;
  }
}

// Only when more elements equal the threshold than are still to be taken: ties per chunk of kChunk tokens ...
__global__ __launch_bounds__(kBlock) void tie_count_kernel(const uint32_t* __restrict__ keys, int64_t n_slots,
                                                           const SelectState* st, uint32_t* chunk_ties) {
  __shared__ float lds_red[kBlock / kWave];
  if (st->k == 0 || st->index_limit != -1) return;
  const uint32_t thr = st->threshold;
  const int64_t c0 = (int64_t)blockIdx.x * kChunk;
  const int64_t c1 = min(c0 + (int64_t)kChunk, n_slots);
  float t[1] = {0.f};
  for (int64_t i = c0 + threadIdx.x; i < c1; i += kBlock) t[0] += keys[i] == thr ? 1.f : 0.f;
  block_sum<1>(t, lds_red);
  if (threadIdx.x == 0) chunk_ties[blockIdx.x] = (uint32_t)t[0];
}

// ... and the index just past the `remaining`-th tie in token order (one thread; ties are rare).
__global__ void tie_limit_kernel(const uint32_t* __restrict__ keys, int64_t n_slots, SelectState* st,
                                 const uint32_t* __restrict__ chunk_ties, int64_t n_chunks) {
  if (st->k == 0 || st->index_limit != -1) return;
  uint32_t need = st->remaining;
  int64_t c = 0;
  for (; c < n_chunks - 1; ++c) {
    if (chunk_ties[c] >= need) break;
    need -= chunk_ties[c];
  }
  const uint32_t thr = st->threshold;
  int64_t i = c * kChunk;
  for (; i < n_slots && need > 0; ++i)
    if (keys[i] == thr) --need;
  st->index_limit = i;
}

}  // namespace axon

using namespace axon;

namespace {

unsigned walk_grid(int64_t n_slots) {
  const int64_t blocks = (n_slots / kVec + kBlock - 1) / kBlock;
  const int64_t cap = 2048;
  return (unsigned)(blocks < 1 ? 1 : (blocks < cap ? blocks : cap));
}

struct CovWs {
  float* partials;
  uint32_t* hist;
  uint32_t* chunk_ties;
  int64_t n_chunks;
  int64_t bytes;
};

CovWs cov_ws(int64_t n_slots, char* base) {
  CovWs w;
  int64_t off = 0;
  w.partials = reinterpret_cast<float*>(base + off);
  off += (int64_t)walk_grid(n_slots) * kPartialStride * 4;
  w.hist = reinterpret_cast<uint32_t*>(base + off);
  off += kBins * 4;
  w.n_chunks = (n_slots + kChunk - 1) / kChunk;
  w.chunk_ties = reinterpret_cast<uint32_t*>(base + off);
  off += (w.n_chunks > 0 ? w.n_chunks : 1) * 4;
  w.bytes = off;
  return w;
}

template <int MK>
int run_select(int kind, const float* logp, const float* oldp, const float* adv, const void* mask,
               int64_t n_slots, double ratio, float lb, float ub, float ratio_lo, float ratio_hi,
               uint32_t seed, uint32_t* keys, SelectState* st, const CovWs& w, hipStream_t s) {
  const dim3 grid(walk_grid(n_slots)), blk(kBlock);
  if (kind == 0)
    hipLaunchKernelGGL((cov_moments_kernel<MK, false>), grid, blk, 0, s, adv, logp, mask, n_slots, w.partials);
  else
    hipLaunchKernelGGL((cov_moments_kernel<MK, true>), grid, blk, 0, s, adv, logp, mask, n_slots, w.partials);
  hipLaunchKernelGGL(cov_moments_finish_kernel, dim3(1), blk, 0, s, w.partials, (int)grid.x, kind, ratio, st,
                     w.hist);
  if (kind == 0)
    hipLaunchKernelGGL((cov_key_kernel<MK, 0>), grid, blk, 0, s, logp, oldp, adv, mask, n_slots, lb, ub,
                       ratio_lo, ratio_hi, seed, st, keys);
  else
    hipLaunchKernelGGL((cov_key_kernel<MK, 1>), grid, blk, 0, s, logp, oldp, adv, mask, n_slots, lb, ub,
                       ratio_lo, ratio_hi, seed, st, keys);
  AXON_CHECK_LAUNCH();
  for (int round = 0; round < 3; ++round) {
    hipLaunchKernelGGL(radix_hist_kernel, grid, blk, 0, s, keys, n_slots, st, round, w.hist);
    hipLaunchKernelGGL(radix_pick_kernel, dim3(1), blk, 0, s, w.hist, st, round);
  }
  AXON_CHECK_LAUNCH();
  hipLaunchKernelGGL(tie_count_kernel, dim3((unsigned)w.n_chunks), blk, 0, s, keys, n_slots, st, w.chunk_ties);
  hipLaunchKernelGGL(tie_limit_kernel, dim3(1), dim3(1), 0, s, keys, n_slots, st, w.chunk_ties, w.n_chunks);
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

}  // namespace

extern "C" int64_t axon_cov_select_state_bytes(void) { return (int64_t)sizeof(SelectState); }

extern "C" int64_t axon_cov_select_workspace_bytes(int64_t n_slots) {
  if (n_slots < 0) return AXON_ERR_ARG;
  return cov_ws(n_slots, nullptr).bytes;
}

extern "C" int axon_cov_select(int kind, const float* logp, const float* old_logp, const float* adv,
                               const void* mask, int mask_kind, int64_t n_slots, double ratio, float cov_lb,
                               float cov_ub, float ratio_lo, float ratio_hi, uint32_t seed, uint32_t* keys,
                               void* state, void* workspace, void* stream) {
  if (n_slots < 0 || kind < 0 || kind > 1 || !(ratio > 0.0)) return AXON_ERR_ARG;
  if (n_slots >= (int64_t)INT32_MAX) return AXON_ERR_SHAPE;
  if (!state || !workspace) return AXON_ERR_ARG;
  if (n_slots == 0) return axon_fill_zero(state, (sizeof(SelectState) + 3) / 4 * 4, stream);
  if (!logp || !adv || !mask || !keys || (kind == 1 && !old_logp)) return AXON_ERR_ARG;
  if (mask_kind != AXON_MASK_F32 && mask_kind != AXON_MASK_I64) return AXON_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(logp) | reinterpret_cast<uintptr_t>(old_logp) |
       reinterpret_cast<uintptr_t>(adv) | reinterpret_cast<uintptr_t>(mask) |
       reinterpret_cast<uintptr_t>(keys) | reinterpret_cast<uintptr_t>(workspace)) & 15)
    return AXON_ERR_ARG;
  const CovWs w = cov_ws(n_slots, static_cast<char*>(workspace));
  SelectState* st = static_cast<SelectState*>(state);
  const hipStream_t s = (hipStream_t)stream;
  if (mask_kind == AXON_MASK_F32)
    return run_select<AXON_MASK_F32>(kind, logp, old_logp, adv, mask, n_slots, ratio, cov_lb, cov_ub,
                                     ratio_lo, ratio_hi, seed, keys, st, w, s);
  return run_select<AXON_MASK_I64>(kind, logp, old_logp, adv, mask, n_slots, ratio, cov_lb, cov_ub,
                                   ratio_lo, ratio_hi, seed, keys, st, w, s);
}
