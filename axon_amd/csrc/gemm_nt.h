// bf16 "NT" GEMM main loop for gfx950:  D[m][n] = sum_k A[m][k] * B[n][k]
//
// Both operands are K-contiguous, which is the layout the 32x32x16 bf16 MFMA
// wants on both sides: every lane feeds eight consecutive k of one row.  The
// LM-head forward, its logit recompute, dHidden and dWeight are all brought to
// this one form (by pre-transposed copies where needed), so one main loop
// serves the whole path; they differ only in the epilogue.
//
// Workgroup: 256 threads = 4 waves in a 2x2 grid, tile 256(m) x 256(n), each
// wave 128 x 128 = 4x4 MFMA blocks of 32x32 (256 fp32 accumulators per lane).
// LDS: two stages of (256 + 256) rows x BK bf16, 16-byte chunks XOR-swizzled by
// row so that the 16-byte fragment reads of 32 consecutive rows spread over all
// banks.
//
// Accumulator layout of one 32x32 block (v16f32, index q = 4*r + e):
//   m = 8*r + 4*(lane/32) + e,   n = lane%32.
// So a lane owns ONE n per block column and four consecutive m per register
// quad: per-n statistics need no cross-lane traffic beyond lane^32, and stores
// to an [n][m] output are 4-element vectors.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace axon {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int kTile = 256;       // tile edge in m and n
constexpr int kWaveTile = 128;   // per-wave edge
constexpr int kGemmThreads = 256;

struct GemmOperands {
  const __bf16* a;  // [m_rows][lda], K-contiguous
  const __bf16* b;  // [n_rows][ldb]
  int64_t lda, ldb;
  int m_rows, n_rows;  // valid rows; tile rows beyond are clamped on load
  int k;               // reduction length, multiple of BK
};

template <int BK>
struct TileLds {
  static constexpr int kChunks = BK / 8;                 // 16-byte chunks per row
  static constexpr int kRowBytes = BK * 2;
  static constexpr int kRowsPerLine = 256 / kRowBytes;   // rows per 256-byte bank line
  static constexpr int kOperandBytes = kTile * kRowBytes;
  static constexpr int kStageBytes = 2 * kOperandBytes;
  static constexpr int kBytes = 2 * kStageBytes;
  __device__ static __forceinline__ int offset(int row, int chunk) {
    const int sw = (row / kRowsPerLine) % kChunks;
    return row * kRowBytes + ((chunk ^ sw) << 4);
  }
};

// Position of this lane inside the workgroup tile.
struct LanePos {
  int lane, l32, lhi, wm, wn;
  __device__ __forceinline__ LanePos() {
    lane = threadIdx.x & 63;
    l32 = lane & 31;
    lhi = lane >> 5;
    const int w = threadIdx.x >> 6;
    wm = w >> 1;
    wn = w & 1;
  }
  // tile-relative coordinates of accumulator (i, j, q)
  __device__ __forceinline__ int m(int i, int q) const {
    return wm * kWaveTile + i * 32 + 8 * (q >> 2) + 4 * lhi + (q & 3);
  }
  __device__ __forceinline__ int n(int j) const { return wn * kWaveTile + j * 32 + l32; }
};

template <int BK>
__device__ __forceinline__ void gemm_mainloop(const GemmOperands& g, int m0, int n0,
                                              f32x16 (&acc)[4][4], char* smem) {
  using L = TileLds<BK>;
  constexpr int kLoads = (kTile * L::kChunks) / kGemmThreads;  // 16-byte loads per operand per thread
  constexpr int kRowStep = kGemmThreads / L::kChunks;
  const LanePos lp;

  const int ld_chunk = threadIdx.x % L::kChunks;
  const int ld_row = threadIdx.x / L::kChunks;
  const uint4* ga[kLoads];
  const uint4* gb[kLoads];
  int lds_off[kLoads];
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    const int row = ld_row + i * kRowStep;
    const int ra = min(m0 + row, g.m_rows - 1);
    const int rb = min(n0 + row, g.n_rows - 1);
    ga[i] = reinterpret_cast<const uint4*>(g.a + (int64_t)ra * g.lda) + ld_chunk;
    gb[i] = reinterpret_cast<const uint4*>(g.b + (int64_t)rb * g.ldb) + ld_chunk;
    lds_off[i] = L::offset(row, ld_chunk);
  }
  int a_off[4], b_off[4];  // fragment row offsets (chunk applied per k-step)
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a_off[i] = lp.wm * kWaveTile + i * 32 + lp.l32;
    b_off[i] = lp.wn * kWaveTile + i * 32 + lp.l32;
  }

#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;

  uint4 ra[kLoads], rb[kLoads];
  const int kt_n = g.k / BK;
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    ra[i] = ga[i][0];
    rb[i] = gb[i][0];
  }
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    *reinterpret_cast<uint4*>(smem + lds_off[i]) = ra[i];
    *reinterpret_cast<uint4*>(smem + L::kOperandBytes + lds_off[i]) = rb[i];
  }
  __syncthreads();

  for (int kt = 0; kt < kt_n; ++kt) {
    const char* cur = smem + (kt & 1) * L::kStageBytes;
    char* nxt = smem + ((kt + 1) & 1) * L::kStageBytes;
    const bool more = (kt + 1 < kt_n);
    if (more) {
      const int ko = (kt + 1) * L::kChunks;
#pragma unroll
      for (int i = 0; i < kLoads; ++i) {
        ra[i] = ga[i][ko];
        rb[i] = gb[i][ko];
      }
    }
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      bf16x8 af[4], bf[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        af[i] = *reinterpret_cast<const bf16x8*>(cur + L::offset(a_off[i], kk * 2 + lp.lhi));
        bf[i] = *reinterpret_cast<const bf16x8*>(cur + L::kOperandBytes +
                                                 L::offset(b_off[i], kk * 2 + lp.lhi));
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
    if (more) {
#pragma unroll
      for (int i = 0; i < kLoads; ++i) {
        *reinterpret_cast<uint4*>(nxt + lds_off[i]) = ra[i];
        *reinterpret_cast<uint4*>(nxt + L::kOperandBytes + lds_off[i]) = rb[i];
      }
    }
    __syncthreads();
  }
}

// Workgroup id -> (tile_m, tile_n).  Consecutive workgroup ids land on
// different XCDs (round-robin over 8), so ids are first regrouped so that each
// XCD walks a contiguous range, and inside that range tiles are visited in
// bands of `kBand` n-tiles so that concurrently resident workgroups of one XCD
// share A and B tiles in its L2.
__device__ __forceinline__ void tile_coords(int tiles_m, int tiles_n, int& tm, int& tn) {
  constexpr int kXcd = 8, kBand = 4;
  const int total = tiles_m * tiles_n;
  int pid = blockIdx.x;
  const int per = total / kXcd;  // ids beyond kXcd*per keep their natural position
  if (pid < per * kXcd) pid = (pid % kXcd) * per + pid / kXcd;
  const int band_sz = kBand * tiles_m;
  const int band = pid / band_sz;
  const int first_n = band * kBand;
  const int width = min(tiles_n - first_n, kBand);
  const int r = pid - band * band_sz;
  tn = first_n + r % width;
  tm = r / width;
}

}  // namespace axon
