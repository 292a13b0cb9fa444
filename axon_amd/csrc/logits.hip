// The non-fused branch of the trainer's forward: the model has already written the [tokens, vocab] logits;
// per token, log_softmax(logits)[label] and the entropy come out of ONE read of the row (online max /
// sum / sum-times-logit, as in the fused head), and the backward turns the row into its gradient in one
// more read and one write (in place when asked to).  HBM-bound: 2 or 4 bytes per logit forward, twice that
// plus the write backward.
#include "common.h"

namespace axon {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

typedef unsigned short u16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ float bf16_to_f32(unsigned short h) { return __uint_as_float((uint32_t)h << 16); }
__device__ __forceinline__ unsigned short f32_to_bf16(float f) {  // round to nearest even, NaN kept
  const uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40);
  return (unsigned short)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

template <typename T> struct Row;
template <> struct Row<float> {
  static constexpr int kPer = 4;
  __device__ static void load(const float* p, float (&v)[8]) {
    const f32x4 x = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
  }
  __device__ static float one(const float* p) { return *p; }
  __device__ static void store(float* p, const float (&v)[8]) {
    const f32x4 x = {v[0], v[1], v[2], v[3]};
    __builtin_nontemporal_store(x, reinterpret_cast<f32x4*>(p));
  }
  __device__ static void store_one(float* p, float v) { *p = v; }
};
template <> struct Row<unsigned short> {
  static constexpr int kPer = 8;
  __device__ static void load(const unsigned short* p, float (&v)[8]) {
    const u16x8 x = __builtin_nontemporal_load(reinterpret_cast<const u16x8*>(p));
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = bf16_to_f32(x[j]);
  }
  __device__ static float one(const unsigned short* p) { return bf16_to_f32(*p); }
  __device__ static void store(unsigned short* p, const float (&v)[8]) {
    u16x8 x;
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = f32_to_bf16(v[j]);
    __builtin_nontemporal_store(x, reinterpret_cast<u16x8*>(p));
  }
  __device__ static void store_one(unsigned short* p, float v) { *p = f32_to_bf16(v); }
};

// Running statistics of a set of logits y (log2 units): M >= every y, s = sum 2^(y-M), e = sum 2^(y-M)(y-M).
struct Stats { float M, s, e; };

constexpr float kTiny = -150.f;  // 2^-150 flushes to zero: a logit that far below the maximum (or -inf) adds nothing

// Folds N logits (natural units) at once: one rescale at most, then four arithmetic instructions and one
// exponential per logit.
template <int N>
__device__ __forceinline__ void fold(Stats& a, const float (&z)[8]) {
  float m = z[0];
#pragma unroll
  for (int j = 1; j < N; ++j) m = fmaxf(m, z[j]);
  m *= kLog2e;
  if (m > a.M) {  // rescale what is there to the new reference
    const float d = fmaxf(a.M - m, kTiny), f = __builtin_amdgcn_exp2f(d);
    a.e = f * fmaf(a.s, d, a.e);
    a.s = a.s * f;
    a.M = m;
  }
  // four independent partial sums: the additions of consecutive logits do not wait for one another
  float s4[4] = {a.s, 0.f, 0.f, 0.f}, e4[4] = {a.e, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const float d = fmaxf(fmaf(z[j], kLog2e, -a.M), kTiny), f = __builtin_amdgcn_exp2f(d);
    s4[j & 3] += f;
    e4[j & 3] = fmaf(f, d, e4[j & 3]);
  }
  a.s = (s4[0] + s4[1]) + (s4[2] + s4[3]);
  a.e = (e4[0] + e4[1]) + (e4[2] + e4[3]);
}
__device__ __forceinline__ Stats merge(Stats a, Stats b) {
  const float Mn = fmaxf(a.M, b.M);
  const float d1 = fmaxf(a.M - Mn, kTiny), d2 = fmaxf(b.M - Mn, kTiny);
  const float f1 = __builtin_amdgcn_exp2f(d1), f2 = __builtin_amdgcn_exp2f(d2);
  Stats r;
  r.M = Mn;
  r.e = f1 * fmaf(a.s, d1, a.e) + f2 * fmaf(b.s, d2, b.e);
  r.s = a.s * f1 + b.s * f2;
  return r;
}
constexpr float kFloor = -1e30f;  // below any logit; finite, so that differences stay finite

// One workgroup per token row.  VEC_OK: every row starts on a 16-byte boundary.
template <typename T, typename LabelT>
__global__ __launch_bounds__(kBlock) void logits_stats_kernel(
    const T* __restrict__ logits, int64_t ld, int vocab, const LabelT* __restrict__ labels,
    float* __restrict__ logprob, float* __restrict__ entropy, float* __restrict__ lse, int vec_ok) {
  __shared__ float red[3][kBlock / kWave];
  const T* row = logits + (int64_t)blockIdx.x * ld;
  constexpr int kPer = Row<T>::kPer;
  Stats st{kFloor, 0.f, 0.f};
  const int n_vec = vec_ok ? vocab / kPer : 0;
  int q = threadIdx.x;
  for (; q + kBlock < n_vec; q += 2 * kBlock) {  // two loads in flight per thread
    float v0[8], v1[8];
    Row<T>::load(row + (int64_t)q * kPer, v0);
    Row<T>::load(row + (int64_t)(q + kBlock) * kPer, v1);
    fold<kPer>(st, v0);
    fold<kPer>(st, v1);
  }
  for (; q < n_vec; q += kBlock) {
    float v[8];
    Row<T>::load(row + (int64_t)q * kPer, v);
    fold<kPer>(st, v);
  }
  for (int i = n_vec * kPer + threadIdx.x; i < vocab; i += kBlock) {
    const float v[8] = {Row<T>::one(row + i)};
    fold<1>(st, v);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    Stats o;
    o.M = __shfl_down(st.M, off, kWave);
    o.s = __shfl_down(st.s, off, kWave);
    o.e = __shfl_down(st.e, off, kWave);
    st = merge(st, o);
  }
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  if (lane == 0) { red[0][wave] = st.M; red[1][wave] = st.s; red[2][wave] = st.e; }
  __syncthreads();
  if (threadIdx.x != 0) return;
  for (int w = 1; w < kBlock / kWave; ++w) st = merge(st, Stats{red[0][w], red[1][w], red[2][w]});
  const float L = __log2f(st.s), d = st.e / st.s;
  const float lse_v = (st.M + L) * kLn2;
  lse[blockIdx.x] = lse_v;
  if (entropy != nullptr) entropy[blockIdx.x] = (L - d) * kLn2;  // lse - sum p z, the common max cancelled
  if (logprob != nullptr) {
    const int64_t lab = (int64_t)labels[blockIdx.x];
    logprob[blockIdx.x] = (lab >= 0 && lab < vocab) ? Row<T>::one(row + lab) - lse_v : 0.f;
  }
}

// dlogits[j] = g_lp (onehot_j - p_j) - g_ent p_j (log p_j + H),  p_j = exp(z_j - lse).
// dlogits may be the logits' own storage: every element is read before it is written by the same thread.
template <typename T, typename LabelT>
__global__ __launch_bounds__(kBlock) void logits_grad_kernel(
    const T* logits, int64_t ld, int vocab, const LabelT* __restrict__ labels,
    const float* __restrict__ lse, const float* __restrict__ entropy, const float* __restrict__ g_logprob,
    const float* __restrict__ g_entropy, T* dlogits, int64_t ld_d, int vec_ok) {
  const T* row = logits + (int64_t)blockIdx.x * ld;
  T* out = dlogits + (int64_t)blockIdx.x * ld_d;
  constexpr int kPer = Row<T>::kPer;
  const float lse_v = lse[blockIdx.x];
  const float g_lp = g_logprob ? g_logprob[blockIdx.x] : 0.f;
  const float g_en = g_entropy ? g_entropy[blockIdx.x] : 0.f;
  const float H = g_entropy ? entropy[blockIdx.x] : 0.f;
  const int64_t lab = g_logprob ? (int64_t)labels[blockIdx.x] : -1;
  auto grad = [&](int64_t j, float z) {
    const float lp = z - lse_v;
    const float p = __expf(lp);
    float g = -g_lp * p;
    if (g_en != 0.f) g -= (p > 0.f) ? g_en * p * (lp + H) : 0.f;
    if (j == lab) g += g_lp;
    return g;
  };
  const int n_vec = vec_ok ? vocab / kPer : 0;
  for (int q = threadIdx.x; q < n_vec; q += kBlock) {
    float v[8], o[8];
    Row<T>::load(row + (int64_t)q * kPer, v);
#pragma unroll
    for (int j = 0; j < kPer; ++j) o[j] = grad((int64_t)q * kPer + j, v[j]);
    Row<T>::store(out + (int64_t)q * kPer, o);
  }
  for (int i = n_vec * kPer + threadIdx.x; i < vocab; i += kBlock)
    Row<T>::store_one(out + i, grad(i, Row<T>::one(row + i)));
}

}  // namespace axon

using namespace axon;

namespace {

bool rows_on_16_bytes(const void* p, int64_t ld, int elem_bytes) {
  return (reinterpret_cast<uintptr_t>(p) & 15) == 0 && (ld * elem_bytes) % 16 == 0;
}

int check_logits(const void* logits, int dtype, int64_t ld, int64_t n, int64_t v) {
  if (n < 0 || v <= 0 || ld < v) return AXON_ERR_ARG;
  if (dtype != AXON_LOGITS_F32 && dtype != AXON_LOGITS_BF16) return AXON_ERR_ARG;
  if (n >= (int64_t)INT32_MAX || v >= (int64_t)INT32_MAX) return AXON_ERR_SHAPE;
  if (n > 0 && !logits) return AXON_ERR_ARG;
  return AXON_OK;
}

}  // namespace

extern "C" int axon_logits_fwd(const void* logits, int dtype, int64_t ld, int64_t n, int64_t vocab,
                               const void* labels, int labels_i64, float* logprob, float* entropy,
                               float* lse, void* stream) {
  int rc = check_logits(logits, dtype, ld, n, vocab);
  if (rc != AXON_OK) return rc;
  if (n == 0) return AXON_OK;
  if (!lse || (logprob && !labels)) return AXON_ERR_ARG;
  const hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)n), blk(kBlock);
  const int eb = dtype == AXON_LOGITS_F32 ? 4 : 2;
  const int vec_ok = rows_on_16_bytes(logits, ld, eb);
#define AXON_STATS(T, L)                                                                           \
  hipLaunchKernelGGL((logits_stats_kernel<T, L>), grid, blk, 0, st, static_cast<const T*>(logits), ld, \
                     (int)vocab, static_cast<const L*>(labels), logprob, entropy, lse, vec_ok)
  if (dtype == AXON_LOGITS_F32) {
    if (labels_i64) AXON_STATS(float, int64_t); else AXON_STATS(float, int32_t);
  } else {
    if (labels_i64) AXON_STATS(unsigned short, int64_t); else AXON_STATS(unsigned short, int32_t);
  }
#undef AXON_STATS
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}

extern "C" int axon_logits_bwd(const void* logits, int dtype, int64_t ld, int64_t n, int64_t vocab,
                               const void* labels, int labels_i64, const float* lse,
                               const float* entropy, const float* g_logprob, const float* g_entropy,
                               void* dlogits, int64_t ld_d, void* stream) {
  int rc = check_logits(logits, dtype, ld, n, vocab);
  if (rc != AXON_OK) return rc;
  if (n == 0) return AXON_OK;
  if (!lse || !dlogits || ld_d < vocab) return AXON_ERR_ARG;
  if ((g_logprob && !labels) || (g_entropy && !entropy)) return AXON_ERR_ARG;
  const hipStream_t st = (hipStream_t)stream;
  const dim3 grid((unsigned)n), blk(kBlock);
  const int eb = dtype == AXON_LOGITS_F32 ? 4 : 2;
  const int vec_ok = rows_on_16_bytes(logits, ld, eb) && rows_on_16_bytes(dlogits, ld_d, eb);
#define AXON_GRAD(T, L)                                                                            \
  hipLaunchKernelGGL((logits_grad_kernel<T, L>), grid, blk, 0, st, static_cast<const T*>(logits), ld,  \
                     (int)vocab, static_cast<const L*>(labels), lse, entropy, g_logprob, g_entropy,    \
                     static_cast<T*>(dlogits), ld_d, vec_ok)
  if (dtype == AXON_LOGITS_F32) {
    if (labels_i64) AXON_GRAD(float, int64_t); else AXON_GRAD(float, int32_t);
  } else {
    if (labels_i64) AXON_GRAD(unsigned short, int64_t); else AXON_GRAD(unsigned short, int32_t);
  }
#undef AXON_GRAD
  AXON_CHECK_LAUNCH();
  return AXON_OK;
}
