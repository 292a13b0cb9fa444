// bf16 "NT" GEMM main loops for gfx950:  D[m][n] = sum_k A[m][k] * B[n][k]
//
// Both operands are K-contiguous, which is the layout the 32x32x16 bf16 MFMA
// wants on both sides: every lane feeds eight consecutive k of one row.  The
// LM-head forward, its logit recompute, dHidden and dWeight are all brought to
// this one form (by pre-transposed copies where needed), so one main loop
// serves the whole path; they differ only in the epilogue.
//
// Workgroup: 256 threads = 4 waves in a 2x2 grid, tile 256(m) x 256(n), each
// wave 128 x 128 = 4x4 MFMA blocks of 32x32 (256 fp32 accumulators per lane,
// one wave per SIMD).
//
// Two main loops:
//  * DmaLoop  (the fast path; needs m_rows >= 256, n_rows >= 256, k % 64 == 0)
//      global -> LDS by `buffer_load_dwordx4 ... lds` (no VGPR staging), 32 KB
//      slots of 256 x 64 bf16 (three for A, two for B), 16-byte chunks
//      XOR-swizzled by row; fragment reads for k-step kk+1 are issued under the
//      MFMAs of k-step kk; A is fetched two k-tiles ahead, B one.  Edge tiles are
//      shifted back inside the matrix (uniform addressing, no per-lane clamps);
//      the rows that then belong to the neighbouring tile are masked by the
//      epilogue through `m_lo` / `n_lo`.
//  * RegLoop<32>  (any shape with k % 32 == 0): loads through registers with
//      per-row clamping.  Used for small or odd shapes.
//
// Accumulator layout of one 32x32 block (v16f32, index q = 4*r + e):
//   m = 8*r + 4*(lane/32) + e,   n = lane%32.
// So a lane owns ONE n per block column and four consecutive m per register
// quad: per-n statistics need no cross-lane traffic beyond lane^32, and stores
// to an [n][m] output are 4-element vectors.
#pragma once
#include <type_traits>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace axon {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int kTile = 256;       // tile edge in m and n
constexpr int kWaveTile = 128;   // per-wave edge
constexpr int kGemmThreads = 256;
constexpr int kGemmLdsBytes = 163840;  // all of a CU's LDS: five 32 KB operand slots; the dlogit epilogue stages in the first 128 KB

struct GemmOperands {
  const __bf16* a;  // [m_rows][lda], K-contiguous
  const __bf16* b;  // [n_rows][ldb]
  int64_t lda, ldb;
  int m_rows, n_rows;  // valid rows
  int k;               // reduction length
};

// Where a workgroup's tile sits.  (m0, n0) is the first row/column actually
// computed; rows with tile-relative index < m_lo (columns < n_lo) duplicate the
// previous tile and must be ignored by the epilogue.
struct TilePos {
  int m0, n0, m_lo, n_lo;
};

// Position of this lane inside the workgroup tile.
struct LanePos {
  int lane, l32, lhi, wave, wm, wn;
  __device__ __forceinline__ LanePos() {
    lane = threadIdx.x & 63;
    l32 = lane & 31;
    lhi = lane >> 5;
    wave = threadIdx.x >> 6;
    wm = wave >> 1;
    wn = wave & 1;
  }
  // tile-relative coordinates of accumulator (i, j, q)
  __device__ __forceinline__ int m(int i, int q) const {
    return wm * kWaveTile + i * 32 + 8 * (q >> 2) + 4 * lhi + (q & 3);
  }
  __device__ __forceinline__ int n(int j) const { return wn * kWaveTile + j * 32 + l32; }
};

__device__ __forceinline__ void zero_acc(f32x16 (&acc)[4][4]) {
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;
}

// ---------------------------------------------------------------------------------------
// DmaLoop: k-tiles of 64 go global -> LDS by buffer_load ... lds (no register staging) into
// XOR-swizzled [row][128 B] slots.  The 160 KB of LDS hold THREE slots for the A operand and
// TWO for B.  B of k-tile t+2 is issued right after the barrier that frees its slot and has one
// k-tile of time to land; A of k-tile t+2 is issued a whole k-tile earlier, spread under the
// MFMAs of k-steps 0..2, into the slot freed one barrier before.  Compared with a symmetric
// double buffer this halves the data that has only one k-tile to arrive, which is what keeps the
// single wave per SIMD from waiting at the barrier (measured: +20 % on long-k GEMMs).
// ---------------------------------------------------------------------------------------
struct DmaLoop {
  static constexpr int kBK = 64;
  static constexpr int kRowBytes = 128;
  static constexpr int kOperandBytes = kTile * kRowBytes;  // 32 KB
  static constexpr int kBBase = 3 * kOperandBytes;         // A slots at 0/32/64 KB, B slots at 96/128 KB
  static constexpr bool kShiftsEdgeTiles = true;

  __device__ static __forceinline__ bool supports(const GemmOperands& g) {
    return g.m_rows >= kTile && g.n_rows >= kTile && (g.k % kBK) == 0;
  }

  // Edge tiles are shifted back inside the matrix; the epilogue skips the duplicated rows.
  __device__ static __forceinline__ TilePos place(const GemmOperands& g, int tm, int tn) {
    TilePos t;
    const int m0 = tm * kTile, n0 = tn * kTile;
    t.m0 = min(m0, g.m_rows - kTile);
    t.n0 = min(n0, g.n_rows - kTile);
    t.m_lo = m0 - t.m0;
    t.n_lo = n0 - t.n0;
    return t;
  }

  __device__ static __forceinline__ void dma16(__amdgpu_buffer_rsrc_t rsrc, int voffset, int soffset,
                                               char* lds) {
    // LDS destination = lds + 16 * lane (wave-contiguous); memory source = base + voffset + soffset
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)lds, 16,
                                             voffset, soffset, 0, 0);
  }

  __device__ static __forceinline__ void run(const GemmOperands& g, const TilePos& t,
                                             f32x16 (&acc)[4][4], char* smem) {
    const LanePos lp;
    // --- DMA addressing.  One wave instruction fills 1 KB of LDS = 8 rows x 128 B; wave w owns
    // rows [64w, 64w+64) of each operand (8 instructions).  Lane i lands on row i/8, chunk slot
    // i%8, and therefore fetches global chunk (i%8) ^ swizzle(row); swizzle(row) = (row/2) % 8.
    const int lrow = lp.lane >> 3;
    const int sw_even = (lp.lane >> 4) & 7;
    const int sw_odd = (4 + (lp.lane >> 4)) & 7;
    const int row_a = (lp.wave * 64 + lrow) * (int)g.lda * 2;
    const int row_b = (lp.wave * 64 + lrow) * (int)g.ldb * 2;
    const int va_e = row_a + (((lp.lane & 7) ^ sw_even) << 4);
    const int va_o = row_a + (((lp.lane & 7) ^ sw_odd) << 4);
    const int vb_e = row_b + (((lp.lane & 7) ^ sw_even) << 4);
    const int vb_o = row_b + (((lp.lane & 7) ^ sw_odd) << 4);
    const int step_a = (int)g.lda * 16, step_b = (int)g.ldb * 16;
    const __bf16* base_a = g.a + (int64_t)t.m0 * g.lda;
    const __bf16* base_b = g.b + (int64_t)t.n0 * g.ldb;
    const __amdgpu_buffer_rsrc_t ra =
        __builtin_amdgcn_make_buffer_rsrc((void*)base_a, 0, 0x7fffffff, 0x00020000);
    const __amdgpu_buffer_rsrc_t rb =
        __builtin_amdgcn_make_buffer_rsrc((void*)base_b, 0, 0x7fffffff, 0x00020000);
    // wave-uniform, so the LDS destination of every DMA instruction is scalar arithmetic into M0
    char* const dst = smem + __builtin_amdgcn_readfirstlane(lp.wave) * 64 * kRowBytes;

    // --- fragment addressing: row = 128*wm + 32*i + l32, chunk = 2*kk + lhi, swizzle = (l32/2)%8
    const int sw = (lp.l32 >> 1) & 7;
    int fa[4], fb[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      fa[kk] = (lp.wm * kWaveTile + lp.l32) * kRowBytes + (((kk * 2 + lp.lhi) ^ sw) << 4);
      fb[kk] = kBBase + (lp.wn * kWaveTile + lp.l32) * kRowBytes + (((kk * 2 + lp.lhi) ^ sw) << 4);
    }

    zero_acc(acc);
    bf16x8 af[2][4], bf[2][4];
    const int kt_n = g.k / kBK;
    // byte offset of k-tile kt inside a row; past the end: refetches the last tile, never consumed
    auto k_byte = [&](int kt) { return min(kt, kt_n - 1) * kRowBytes; };
    auto dma_a = [&](int slot_off, int ko, int j) {
      dma16(ra, (j & 1) ? va_o : va_e, ko + j * step_a, dst + slot_off + j * 8 * kRowBytes);
    };
    auto dma_b = [&](int slot_off, int ko, int j) {
      dma16(rb, (j & 1) ? vb_o : vb_e, ko + j * step_b, dst + kBBase + slot_off + j * 8 * kRowBytes);
    };
    // One k-step: 16 MFMAs on fragment set mm_set; the eight fragments of the next k-step are read
    // one per MFMA; `NA` A instructions [a_first, a_first + NA) and `NB` B instructions [0, NB) are
    // issued in between, in source order (the compiler keeps LDS DMA and LDS reads ordered).
    auto step = [&](int rd_a, int rd_b, int rd_kk, int mm_set, int a_slot, int a_ko, int a_first,
                    auto na_c, int b_slot, int b_ko, auto nb_c) {
      constexpr int NA = decltype(na_c)::value, NB = decltype(nb_c)::value;
      constexpr int vmem = NA + NB;
      const int rd_set = mm_set ^ 1;
#pragma unroll
      for (int m = 0; m < 16; ++m) {
        const int before = (m * vmem) / 16, due = ((m + 1) * vmem) / 16 - before;
#pragma unroll
        for (int d = 0; d < due; ++d) {
          const int idx = before + d;  // B first: it has the shorter time to land
          if (idx < NB) dma_b(b_slot, b_ko, idx);
          else dma_a(a_slot, a_ko, a_first + idx - NB);
        }
        if (m == 0) af[rd_set][0] = *reinterpret_cast<const bf16x8*>(smem + rd_a + fa[rd_kk]);
        if (m >= 1 && m <= 4)
          bf[rd_set][m - 1] =
              *reinterpret_cast<const bf16x8*>(smem + rd_b + fb[rd_kk] + (m - 1) * 32 * kRowBytes);
        if (m >= 5 && m <= 7)
          af[rd_set][m - 4] =
              *reinterpret_cast<const bf16x8*>(smem + rd_a + fa[rd_kk] + (m - 4) * 32 * kRowBytes);
        acc[m >> 2][m & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[mm_set][m >> 2], bf[mm_set][m & 3],
                                                                     acc[m >> 2][m & 3], 0, 0, 0);
        if (due == 1) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        if (due >= 2) __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
        if (m < 8) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    };
    using I0 = std::integral_constant<int, 0>;
    using I8 = std::integral_constant<int, 8>;
    constexpr int kA[3] = {3, 3, 2};  // A instructions under k-steps 0, 1, 2
    static_assert(kA[0] + kA[1] + kA[2] == 8, "eight A instructions per wave and k-tile");
    using A0 = std::integral_constant<int, kA[0]>;
    using A1 = std::integral_constant<int, kA[1]>;
    using A2 = std::integral_constant<int, kA[2]>;

    // prologue: tiles 0 and 1 whole (A slots 0, 1; B slots 0, 1)
#pragma unroll
    for (int j = 0; j < 8; ++j) dma_a(0, k_byte(0), j);
#pragma unroll
    for (int j = 0; j < 8; ++j) dma_b(0, k_byte(0), j);
#pragma unroll
    for (int j = 0; j < 8; ++j) dma_a(kOperandBytes, k_byte(1), j);
#pragma unroll
    for (int j = 0; j < 8; ++j) dma_b(kOperandBytes, k_byte(1), j);
    __builtin_amdgcn_s_waitcnt(0x4F70);  // vmcnt(16): tile 0 has landed
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      af[0][i] = *reinterpret_cast<const bf16x8*>(smem + fa[0] + i * 32 * kRowBytes);
      bf[0][i] = *reinterpret_cast<const bf16x8*>(smem + fb[0] + i * 32 * kRowBytes);
    }
    __builtin_amdgcn_sched_barrier(0);

    int a_cur = 0, b_cur = 0;  // slots of the tile being consumed
    for (int kt = 0; kt < kt_n; ++kt) {
      const int a_nxt = (a_cur == 2 * kOperandBytes) ? 0 : a_cur + kOperandBytes;
      const int a_fill = (a_nxt == 2 * kOperandBytes) ? 0 : a_nxt + kOperandBytes;  // freed one barrier ago
      const int b_nxt = b_cur ^ kOperandBytes;
      const int ko2 = k_byte(kt + 2);
      // k-steps 0..2: A of tile kt+2
      step(a_cur, b_cur, 1, 0, a_fill, ko2, 0, A0{}, 0, 0, I0{});
      step(a_cur, b_cur, 2, 1, a_fill, ko2, kA[0], A1{}, 0, 0, I0{});
      step(a_cur, b_cur, 3, 0, a_fill, ko2, kA[0] + kA[1], A2{}, 0, 0, I0{});
      // last k-step: tile kt+1 must have landed for every wave (the eight younger instructions are
      // A of tile kt+2) and every wave must be done reading this tile's B slot before it is refilled
      __builtin_amdgcn_s_waitcnt(0x0078);  // vmcnt(8) lgkmcnt(0)
      __builtin_amdgcn_s_barrier();
      step(a_nxt, b_nxt, 0, 1, 0, 0, 0, I0{}, b_cur, ko2, I8{});
      a_cur = a_nxt;
      b_cur = b_nxt;
    }
    __builtin_amdgcn_s_waitcnt(0x0070);  // drain the DMA issued for tiles past the end
    __builtin_amdgcn_s_barrier();
  }
};

// ---------------------------------------------------------------------------------------
// RegLoop: loads through registers with per-row clamping; any k % BK == 0
// ---------------------------------------------------------------------------------------
template <int BK>
struct RegLoop {
  static constexpr int kBK = BK;
  static constexpr int kChunks = BK / 8;                 // 16-byte chunks per row
  static constexpr int kRowBytes = BK * 2;
  static constexpr int kRowsPerLine = 256 / kRowBytes;   // rows per 256-byte bank line
  static constexpr int kOperandBytes = kTile * kRowBytes;
  static constexpr int kStageBytes = 2 * kOperandBytes;

  __device__ static __forceinline__ int offset(int row, int chunk) {
    const int sw = (row / kRowsPerLine) % kChunks;
    return row * kRowBytes + ((chunk ^ sw) << 4);
  }

  __device__ static __forceinline__ TilePos place(const GemmOperands&, int tm, int tn) {
    return TilePos{tm * kTile, tn * kTile, 0, 0};
  }

  __device__ static __forceinline__ void run(const GemmOperands& g, const TilePos& t,
                                             f32x16 (&acc)[4][4], char* smem) {
    constexpr int kLoads = (kTile * kChunks) / kGemmThreads;  // 16-byte loads per operand per thread
    constexpr int kRowStep = kGemmThreads / kChunks;
    const LanePos lp;
    const int ld_chunk = threadIdx.x % kChunks;
    const int ld_row = threadIdx.x / kChunks;
    const uint4* ga[kLoads];
    const uint4* gb[kLoads];
    int lds_off[kLoads];
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const int row = ld_row + i * kRowStep;
      const int ra = min(t.m0 + row, g.m_rows - 1);
      const int rb = min(t.n0 + row, g.n_rows - 1);
      ga[i] = reinterpret_cast<const uint4*>(g.a + (int64_t)ra * g.lda) + ld_chunk;
      gb[i] = reinterpret_cast<const uint4*>(g.b + (int64_t)rb * g.ldb) + ld_chunk;
      lds_off[i] = offset(row, ld_chunk);
    }
    int a_off[4], b_off[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a_off[i] = lp.wm * kWaveTile + i * 32 + lp.l32;
      b_off[i] = lp.wn * kWaveTile + i * 32 + lp.l32;
    }
    zero_acc(acc);

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
      *reinterpret_cast<uint4*>(smem + kOperandBytes + lds_off[i]) = rb[i];
    }
    __syncthreads();

    for (int kt = 0; kt < kt_n; ++kt) {
      const char* cur = smem + (kt & 1) * kStageBytes;
      char* nxt = smem + ((kt + 1) & 1) * kStageBytes;
      const bool more = (kt + 1 < kt_n);
      if (more) {
        const int ko = (kt + 1) * kChunks;
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
          af[i] = *reinterpret_cast<const bf16x8*>(cur + offset(a_off[i], kk * 2 + lp.lhi));
          bf[i] = *reinterpret_cast<const bf16x8*>(cur + kOperandBytes + offset(b_off[i], kk * 2 + lp.lhi));
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
          *reinterpret_cast<uint4*>(nxt + kOperandBytes + lds_off[i]) = rb[i];
        }
      }
      __syncthreads();
    }
  }
};

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
