// bf16 "NT" GEMM main loops for gfx950:  D[m][n] = sum_k A[m][k] * B[n][k]
//
// The 16x16x32 bf16 MFMA wants eight consecutive k of one row in every lane on
// both sides.  K-contiguous operands ([row][k]) give that with one 16-byte LDS
// read per fragment; the LM-head forward, its logit recompute and dHidden are
// brought to this form (by pre-transposed copies of the weight and the hidden
// states where needed).  An operand stored the other way round ([k][row],
// "K-major": the dlogits in the dWeight product) is read as it lies with the LDS
// transpose read of gfx950, two 8-byte reads per fragment, at the same speed
// within a per cent.  One main loop serves the whole path; the kernels differ
// only in the epilogue.
//
// Workgroup: 256 threads = 4 waves in a 2x2 grid, tile 256(m) x 256(n), each
// wave 128 x 128 = 8x8 MFMA blocks of 16x16 (256 fp32 accumulators per lane,
// one wave per SIMD).  The 16x16x32 shape reads and writes each accumulator once
// per 32 k (the 32x32x16 shape once per 16 k); under sustained load the part
// holds a higher clock with it (MFMA-only loop on random data: 2047 vs 1795
// TFLOP/s), which is worth more than the larger block's operand reuse.
//
// Two main loops:
//  * DmaLoopT<kAT, kBT>, DmaLoop = DmaLoopT<false, false>  (the fast path; needs
//      m_rows >= 256, n_rows >= 256, k % 64 == 0; kAT / kBT: that side is K-major)
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
// Accumulator layout of one 16x16 block (four floats, index r):
//   m = 4*(lane/16) + r,   n = lane%16.
// So a lane owns ONE n per block column and four consecutive m per block: per-n
// statistics need cross-lane traffic only over lane^16 and lane^32, and stores to
// an [n][m] output are 4-element vectors, 16 consecutive m per four lanes.
#pragma once
#include <type_traits>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace axon {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float acc4;

constexpr int kTile = 256;       // tile edge in m and n
constexpr int kWaveTile = 128;   // per-wave edge
constexpr int kBlk = 16;         // MFMA block edge
constexpr int kBlocks = kWaveTile / kBlk;  // 8 x 8 blocks per wave
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
  int lane, l16, lq, wave, wm, wn;
  __device__ __forceinline__ LanePos() {
    lane = threadIdx.x & 63;
    l16 = lane & 15;
    lq = lane >> 4;
    wave = threadIdx.x >> 6;
    wm = wave >> 1;
    wn = wave & 1;
  }
  // tile-relative coordinates of accumulator (i, j, r)
  __device__ __forceinline__ int m(int i, int r) const { return wm * kWaveTile + i * kBlk + 4 * lq + r; }
  __device__ __forceinline__ int n(int j) const { return wn * kWaveTile + j * kBlk + l16; }
};

typedef acc4 AccTile[kBlocks][kBlocks];

__device__ __forceinline__ void zero_acc(AccTile& acc) {
#pragma unroll
  for (int i = 0; i < kBlocks; ++i)
#pragma unroll
    for (int j = 0; j < kBlocks; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
}

// c += a * b on one 16x16 block, accumulator held in place in the AGPR file.  Written as an
// instruction because the register allocator otherwise rotates the 64 four-register accumulators
// through the VGPR file on every trip of the unrolled loop (hundreds of copies per k-tile).
__device__ __forceinline__ void mfma_16x16x32(acc4& c, const bf16x8& a, const bf16x8& b) {
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

// The compiler does not see the matrix instructions above, so it cannot count the wait states
// between the last of them and the first read of an accumulator: spend them here.
__device__ __forceinline__ void settle_acc() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }

// ---------------------------------------------------------------------------------------
// DmaLoop: k-tiles of 64 go global -> LDS by buffer_load ... lds (no register staging) into
// XOR-swizzled 32 KB slots.  The 160 KB of LDS hold THREE slots for the A operand and
// TWO for B.  A k-tile is two k-steps of 32 (64 MFMAs per wave each).  A of k-tile t+2 is
// issued under the first k-step of tile t into the slot freed one barrier before; the one
// barrier of the tile follows; B of k-tile t+2 is issued under the second k-step into the B slot
// that the barrier has just freed.  Compared with a symmetric double buffer this halves the data
// that has only one k-tile to arrive.
//
// An operand is either K-contiguous (row-major [row][k], the NT form) or K-MAJOR ([k][row], rows
// contiguous: a matrix that would otherwise need a transposed copy).  A K-major operand's slot holds
// the k-tile as 64 k-rows of 512 bytes, and its fragments are read with the LDS transpose read
// (ds_read_b64_tr_b16: the sixteen lanes of a group each name four consecutive 16-bit elements of one
// k-row; lane i of the group receives element i of each of the group's four k-rows), two reads per
// fragment instead of one.  kAT / kBT select the form of each side at compile time.
// ---------------------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(4))) short i16x4;
typedef __attribute__((ext_vector_type(8))) short i16x8;

// What the loop needs to know of one operand side.  T: the operand is K-major.
template <bool T>
struct DmaSide {
  static constexpr int kVariants = T ? 4 : 2;
  static constexpr int kFrag = T ? kBlocks : 2;
  int vo[kVariants];   // per-lane source byte offset of a DMA instruction, by variant(j)
  int step;            // source bytes from DMA instruction j to j + 1
  int64_t kt_bytes;    // source bytes from one k-tile to the next
  const __bf16* base;  // the tile's first element of k-tile 0
  int frag[kFrag];     // per-lane fragment offsets inside a slot: by k-step (row-major) or by block (K-major)

  __device__ static __forceinline__ int variant(int j) { return T ? (j & 1) + 2 * (j >> 2) : (j & 1); }

  // `row0`: first tile row (m0 or n0); `sub`: which half of the tile the wave computes (wm or wn);
  // `lds_base`: where the operand's first slot begins.  It is part of the per-lane fragment offsets so that
  // what is left to add per read (the slot: a scalar; block, k-step, half: constants) fits the 16-bit offset
  // field of the LDS instructions: a constant beyond it costs a vector addition right before the read that
  // needs its result, and every such pair delays the MFMA behind it.
  __device__ __forceinline__ void init(const __bf16* p, int64_t ld, int row0, int sub, const LanePos& lp,
                                       int lds_base) {
    if (!T) {
      // One DMA instruction fills 1 KB of LDS = 8 rows x 128 B; wave w owns rows [64w, 64w+64) of the
      // operand (8 instructions).  Lane i lands on row i/8, chunk slot i%8, and therefore fetches
      // global chunk (i%8) ^ swizzle(row); swizzle(row) = (row/2) % 8.
      const int lrow = lp.lane >> 3;
      const int sw_even = (lp.lane >> 4) & 7;
      const int sw_odd = (4 + (lp.lane >> 4)) & 7;
      const int row = (lp.wave * 64 + lrow) * (int)ld * 2;
      vo[0] = row + (((lp.lane & 7) ^ sw_even) << 4);
      vo[1] = row + (((lp.lane & 7) ^ sw_odd) << 4);
      step = (int)ld * 16;
      kt_bytes = 128;
      base = p + (int64_t)row0 * ld;
      // fragment addressing: row = 128*sub + 16*i + l16, chunk = 4*kk + lq, swizzle = (l16/2)%8.
      // Sixteen lanes (one chunk column of sixteen rows) cover all 64 banks once.
      const int sw = (lp.l16 >> 1) & 7;
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
        frag[kk] = lds_base + (sub * kWaveTile + lp.l16) * 128 + (((kk * 4 + lp.lq) ^ sw) << 4);
    } else {
      // One DMA instruction fills 1 KB of LDS = 2 k-rows x 512 B; wave w owns k-rows [16w, 16w+16) of
      // the k-tile (8 instructions).  Lane i lands on k-row 2j + i/32, 16-byte granule i%32, and fetches
      // global granule (i%32) ^ S(k-row), S(r) = 2 * (r%4 + 4 * ((r/8)%4)): the sixteen k-rows that one
      // transpose read touches (r%4 and (r/8)%4 free) land on sixteen different 32-byte bank groups.
      const int hi = lp.lane >> 5, p32 = lp.lane & 31;
#pragma unroll
      for (int q = 0; q < 4; ++q) {  // q = variant(j) = (j & 1) + 2 * (j >> 2)
        const int s = 4 * (q & 1) + 2 * hi + 8 * ((2 * lp.wave + (q >> 1)) & 3);
        vo[q] = (16 * lp.wave + hi) * (int)ld * 2 + ((p32 ^ s) << 4);
      }
      step = (int)ld * 4;
      kt_bytes = (int64_t)ld * 128;
      base = p + row0;
      // fragment of block i, k-step kk, half h: k-row 32kk + 8lq + 4h + l16/4, elements
      // 128*sub + 16i + 4*(l16%4) ..+3: granule 16*sub + 2i + (l16%4)/2, second half of it for odd l16.
      const int s15 = (2 * (lp.l16 >> 2) + 8 * lp.lq) & 15;
      const int fb = (8 * lp.lq + (lp.l16 >> 2)) * 512 + (((16 * sub) ^ (16 * (lp.lq >> 1))) << 4) +
                     8 * (lp.l16 & 1) + (((lp.l16 & 3) >> 1) << 4);
#pragma unroll
      for (int i = 0; i < kBlocks; ++i) frag[i] = lds_base + fb + ((i << 5) ^ (s15 << 4));
    }
  }
  // source byte offset of k-tile kt; past the end: refetches the last tile, never consumed
  __device__ __forceinline__ int64_t k_off(int kt, int kt_n) const { return (int64_t)min(kt, kt_n - 1) * kt_bytes; }
  __device__ __forceinline__ __amdgpu_buffer_rsrc_t rsrc_at(int64_t ko) const {
    return __builtin_amdgcn_make_buffer_rsrc((void*)(reinterpret_cast<const char*>(base) + ko), 0, 0x7fffffff,
                                             0x00020000);
  }
};

template <bool kAT, bool kBT>
struct DmaLoopT {
  static constexpr int kBK = 64;
  static constexpr int kRowBytes = 128;
  static constexpr int kOperandBytes = kTile * kRowBytes;  // 32 KB
  static constexpr int kBBase = 3 * kOperandBytes;         // A slots at 0/32/64 KB, B slots at 96/128 KB
  static constexpr bool kShiftsEdgeTiles = true;
  static constexpr int kReadsA = kAT ? 2 : 1, kReadsB = kBT ? 2 : 1;  // LDS reads per fragment

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

  // One DMA instruction: 16 bytes per lane, LDS destination = lds + IMM + 16 * lane
  // (wave-contiguous), memory source = base + voffset + soffset + IMM.  The instruction's immediate
  // offset moves both sides, so four consecutive 1 KB destinations share one M0 value.
  template <int IMM>
  __device__ static __forceinline__ void dma16(__amdgpu_buffer_rsrc_t rsrc, int voffset, int soffset,
                                               char* lds) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)lds, 16,
                                             voffset, soffset, IMM, 0);
  }
  // instruction j of an operand tile (the wave's j-th kilobyte of the slot): lds = tile base of the wave
  __device__ static __forceinline__ void dma_kb(__amdgpu_buffer_rsrc_t rsrc, int voffset, int step_bytes,
                                                char* lds, int j) {
    char* const l = lds + (j >> 2) * 4096;
    const int so = j * step_bytes - (j & 3) * 1024;
    switch (j & 3) {
      case 0: dma16<0>(rsrc, voffset, so, l); break;
      case 1: dma16<1024>(rsrc, voffset, so, l); break;
      case 2: dma16<2048>(rsrc, voffset, so, l); break;
      default: dma16<3072>(rsrc, voffset, so, l); break;
    }
  }
  // Written as an instruction: the compiler's builtin for it carries no memory operand, so every such
  // read would be made to wait for ALL DMA in flight (vmcnt(0)), the next tiles' included.  The compiler
  // therefore does not count these reads either: the loop waits for them itself (lgkmcnt(0) before the
  // barrier and before the first MFMA of a k-tile), and the values are used by the MFMAs only.
  // `imm`: a constant once the loops around the call are unrolled (the instruction's offset field)
  // `a`: LDS byte address
  __device__ static __forceinline__ i16x4 read_tr(uint32_t a, int imm) {
    i16x4 v;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(a), "i"(imm));
    return v;
  }
  // lgkmcnt(0) alone (vmcnt and expcnt at their maxima).  For every form of the loop: left to the compiler,
  // the wait for the fragments read under a tile's second k-step comes out BEHIND the next tile's first read
  // and waits for that one as well, a full LDS latency per k-tile.
  __device__ static __forceinline__ void wait_lds_reads() { __builtin_amdgcn_s_waitcnt(0xC07F); }
  __device__ static __forceinline__ bf16x8 join(const i16x4& lo, const i16x4& hi) {
    return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
  }

  __device__ static __forceinline__ void run(const GemmOperands& g, const TilePos& t, AccTile& acc,
                                             char* smem) {
    const LanePos lp;
    DmaSide<kAT> sa;
    DmaSide<kBT> sb;
    sa.init(g.a, g.lda, t.m0, lp.wm, lp, 0);
    sb.init(g.b, g.ldb, t.n0, lp.wn, lp, kBBase);
    // wave-uniform, so the LDS destination of every DMA instruction is scalar arithmetic into M0
    char* const dst = smem + __builtin_amdgcn_readfirstlane(lp.wave) * 8192;

    zero_acc(acc);
    // fragments of two k-steps: whole (one 16-byte read) or as the two halves of a transpose read
    bf16x8 af[2][kBlocks], bf[2][kBlocks];
    i16x4 aft[2][kBlocks][2], bft[2][kBlocks][2];
    const int kt_n = g.k / kBK;
    auto dma_a = [&](int slot_off, const __amdgpu_buffer_rsrc_t& r, int j) {
      dma_kb(r, sa.vo[DmaSide<kAT>::variant(j)], sa.step, dst + slot_off, j);
    };
    auto dma_b = [&](int slot_off, const __amdgpu_buffer_rsrc_t& r, int j) {
      dma_kb(r, sb.vo[DmaSide<kBT>::variant(j)], sb.step, dst + kBBase + slot_off, j);
    };
    // LDS addresses of the fragments in the slots being read: slot + per-lane offset, formed well before the
    // reads that use them (a vector addition right before the read that needs its result delays the MFMA
    // behind the pair; sixteen such pairs per k-tile cost 3-4 % of the loop).  The reads under a tile's second
    // k-step (k-step 0 of the next tile) and under the next tile's first k-step (its k-step 1) go to the same
    // slots, so the addresses change once per k-tile: after the last read of a tile's first k-step.
    constexpr int kAddrA = DmaSide<kAT>::kFrag, kAddrB = DmaSide<kBT>::kFrag;
    // room for the additions behind the reads of a k-step (not with both operands K-major, whose reads fill it:
    // that form, which no kernel of the library uses, forms them in one piece after the barrier)
    constexpr bool kLateAdr = 2 * kBlocks * (kReadsA + kReadsB) + kAddrA + kAddrB <= kBlocks * kBlocks;
    typedef __attribute__((address_space(3))) const char* LdsPtr;
    const uint32_t smem_lds = (uint32_t)(uintptr_t)(LdsPtr)smem;
    uint32_t adr_a[kAddrA], adr_b[kAddrB];
    auto set_adr_a = [&](int q, int slot) { adr_a[q] = smem_lds + slot + sa.frag[q]; };
    auto set_adr_b = [&](int q, int slot) { adr_b[q] = smem_lds + slot + sb.frag[q]; };
    // read `half` of fragment `blk` of k-step kk from the slots the addresses were formed for into set `set`
    auto read_a = [&](int kk, int set, int blk, int half) {
      if (kAT) aft[set][blk][half] = read_tr(adr_a[blk], kk * 16384 + half * 2048);
      else af[set][blk] = *(const __attribute__((address_space(3))) bf16x8*)(LdsPtr)(uintptr_t)(adr_a[kk] + blk * kBlk * kRowBytes);
    };
    auto read_b = [&](int kk, int set, int blk, int half) {
      if (kBT) bft[set][blk][half] = read_tr(adr_b[blk], kk * 16384 + half * 2048);
      else bf[set][blk] = *(const __attribute__((address_space(3))) bf16x8*)(LdsPtr)(uintptr_t)(adr_b[kk] + blk * kBlk * kRowBytes);
    };
    // One k-step of 32: 64 MFMAs on fragment set mm_set.  The sixteen fragments of the next k-step
    // (k-step rd_kk of the slots the addresses stand for) are read under the first part of the step, one read
    // per two MFMAs (A block 0, then the eight B blocks, then A blocks 1..7), into the other set, so that they
    // have landed long before the barrier's wait; NA A-operand or NB B-operand DMA instructions are
    // issued one per eight MFMAs, in slots that carry no fragment read.  With `adr_c` the addresses for the
    // slots nxt_a / nxt_b are formed after the step's last read, one per MFMA.  The scheduling fence after
    // every MFMA keeps the source order: the compiler treats an LDS DMA and an LDS read as aliasing
    // accesses and would otherwise bunch them.
    auto step = [&](int rd_kk, int mm_set, int a_slot, auto na_c, int b_slot, auto nb_c,
                    const __amdgpu_buffer_rsrc_t& rsrc, auto&& mid, auto adr_c, int nxt_a, int nxt_b) {
      constexpr int NA = decltype(na_c)::value, NB = decltype(nb_c)::value;
      constexpr bool kAdr = decltype(adr_c)::value != 0;
      static_assert((NA == 0 || NA == 8) && (NB == 0 || NB == 8) && NA + NB <= 8, "");
      constexpr int RA = kReadsA, RB = kReadsB;
      constexpr int kFirstAdr = 2 * kBlocks * (RA + RB);  // the MFMA after the last read
      static_assert(!kAdr || kLateAdr, "");
      const int rd_set = mm_set ^ 1;
#pragma unroll
      for (int i = 0; i < kBlocks; ++i) {
#pragma unroll
        for (int j = 0; j < kBlocks; ++j) {
          const int m = i * kBlocks + j;
          // scalar bookkeeping for the coming k-tile, in pieces of at most four instructions, in slots without
          // other work (a wavefront issues in order: a dozen scalar instructions in one MFMA gap hold up the
          // MFMA behind them); pieces 3 and 4 come behind the step's last DMA instruction
          if (m == 37) mid(std::integral_constant<int, 0>{});
          if (m == 39) mid(std::integral_constant<int, 1>{});
          if (m == 41) mid(std::integral_constant<int, 2>{});
          if (m == 61) mid(std::integral_constant<int, 3>{});
          if (m == 63) mid(std::integral_constant<int, 4>{});
          if ((m & 7) == 3) {
            if (NB) dma_b(b_slot, rsrc, m >> 3);
            if (NA) dma_a(a_slot, rsrc, m >> 3);
          }
          if ((m & 1) == 0) {
            const int s = m >> 1;
            if (s < RA) read_a(rd_kk, rd_set, 0, s);
            else if (s < RA + kBlocks * RB) read_b(rd_kk, rd_set, (s - RA) / RB, (s - RA) % RB);
            else if (s < kBlocks * (RA + RB))
              read_a(rd_kk, rd_set, 1 + (s - RA - kBlocks * RB) / RA, (s - RA - kBlocks * RB) % RA);
          }
          if (kAdr && m >= kFirstAdr && m < kFirstAdr + kAddrA) set_adr_a(m - kFirstAdr, nxt_a);
          if (kAdr && m >= kFirstAdr + kAddrA && m < kFirstAdr + kAddrA + kAddrB)
            set_adr_b(m - kFirstAdr - kAddrA, nxt_b);
          mfma_16x16x32(acc[i][j], kAT ? join(aft[mm_set][i][0], aft[mm_set][i][1]) : af[mm_set][i],
                        kBT ? join(bft[mm_set][j][0], bft[mm_set][j][1]) : bf[mm_set][j]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    };
    using I0 = std::integral_constant<int, 0>;
    using I8 = std::integral_constant<int, 8>;

    // prologue: tiles 0 and 1 whole (A slots 0, 1; B slots 0, 1)
    {
      const __amdgpu_buffer_rsrc_t ra = sa.rsrc_at(0), rb = sb.rsrc_at(0);
#pragma unroll
      for (int j = 0; j < 8; ++j) dma_a(0, ra, j);
#pragma unroll
      for (int j = 0; j < 8; ++j) dma_b(0, rb, j);
      const __amdgpu_buffer_rsrc_t ra1 = sa.rsrc_at(sa.k_off(1, kt_n)), rb1 = sb.rsrc_at(sb.k_off(1, kt_n));
#pragma unroll
      for (int j = 0; j < 8; ++j) dma_a(kOperandBytes, ra1, j);
#pragma unroll
      for (int j = 0; j < 8; ++j) dma_b(kOperandBytes, rb1, j);
    }
    __builtin_amdgcn_s_waitcnt(0x4F70);  // vmcnt(16): tile 0 has landed
    __builtin_amdgcn_s_barrier();
#pragma unroll
    for (int q = 0; q < kAddrA; ++q) set_adr_a(q, 0);
#pragma unroll
    for (int q = 0; q < kAddrB; ++q) set_adr_b(q, 0);
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) {
#pragma unroll
      for (int h = 0; h < kReadsA; ++h) read_a(0, 0, i, h);
#pragma unroll
      for (int h = 0; h < kReadsB; ++h) read_b(0, 0, i, h);
    }
    __builtin_amdgcn_sched_barrier(0);
    wait_lds_reads();

    // per-tile scalars: the slots of the tile being consumed (cur; the next tile's B slot is the other one),
    // of the next one (nxt), the A slot being filled, and where k-tile kt+2 of either operand begins in
    // memory.  Each is moved on to the next k-tile in place, under the second k-step, as soon as its value for
    // this tile has been used for the last time (`pin` keeps the compiler from gathering the arithmetic at the
    // loop's back edge), so that the back edge carries the counter and the branch only.
    auto next_a_slot = [](int slot) { return (slot == 2 * kOperandBytes) ? 0 : slot + kOperandBytes; };
    auto pin = [](auto& x) { asm volatile("" : "+s"(x)); };
    int a_nxt = kOperandBytes, a_fill = 2 * kOperandBytes, b_cur = 0;
    const char* pa = reinterpret_cast<const char*>(sa.base) + sa.k_off(2, kt_n);
    const char* pb = reinterpret_cast<const char*>(sb.base) + sb.k_off(2, kt_n);
    auto rsrc_of = [](const char* p) {
      return __builtin_amdgcn_make_buffer_rsrc((void*)p, 0, 0x7fffffff, 0x00020000);
    };
    auto k_tile = [&](int kt) {
      // first k-step: A of tile kt+2; the fragments of this tile's second k-step are read (the addresses stand
      // for this tile's slots), then the addresses move on to the next tile's slots
      step(1, 0, a_fill, I8{}, 0, I0{}, rsrc_of(pa), [](auto) {}, std::integral_constant<int, kLateAdr ? 1 : 0>{},
           a_nxt, b_cur ^ kOperandBytes);
      // second k-step: tile kt+1 must have landed for every wave (the eight younger instructions are
      // A of tile kt+2) and every wave must be done reading this tile's B slot before it is refilled
      __builtin_amdgcn_s_waitcnt(0x0078);  // vmcnt(8) lgkmcnt(0)
      __builtin_amdgcn_s_barrier();
      if (!kLateAdr) {
#pragma unroll
        for (int q = 0; q < kAddrA; ++q) set_adr_a(q, a_nxt);
#pragma unroll
        for (int q = 0; q < kAddrB; ++q) set_adr_b(q, b_cur ^ kOperandBytes);
      }
      const bool more = kt + 3 < kt_n;  // else: past the end, the last tile is fetched again and never consumed
      step(0, 1, 0, I0{}, b_cur, I8{}, rsrc_of(pb),
           [&](auto part) {
             constexpr int kPart = decltype(part)::value;
             if (kPart == 0) { a_nxt = next_a_slot(a_nxt); pin(a_nxt); }
             if (kPart == 1) { a_fill = next_a_slot(a_nxt); pin(a_fill); }
             if (kPart == 2) { pa += more ? sa.kt_bytes : 0; pin(pa); }
             if (kPart == 3) { pb += more ? sb.kt_bytes : 0; pin(pb); }
             if (kPart == 4) { b_cur ^= kOperandBytes; pin(b_cur); }
           },
           I0{}, 0, 0);
      wait_lds_reads();  // the next tile's first fragments, read under the second k-step
    };
    // two k-tiles per trip: half as many back edges
    int kt = 0;
    for (; kt + 1 < kt_n; kt += 2) {
      k_tile(kt);
      k_tile(kt + 1);
    }
    if (kt < kt_n) k_tile(kt);
    __builtin_amdgcn_s_waitcnt(0x0070);  // drain the DMA issued for tiles past the end
    __builtin_amdgcn_s_barrier();
    settle_acc();
  }
};
using DmaLoop = DmaLoopT<false, false>;

// ---------------------------------------------------------------------------------------
// RegLoop: loads through registers with per-row clamping; any k % BK == 0
// ---------------------------------------------------------------------------------------
template <int BK>
struct RegLoop {
  static_assert(BK == 32, "one 16x16x32 k-step per staged tile");
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

  __device__ static __forceinline__ void run(const GemmOperands& g, const TilePos& t, AccTile& acc,
                                             char* smem) {
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
    int a_off[kBlocks], b_off[kBlocks];
#pragma unroll
    for (int i = 0; i < kBlocks; ++i) {
      a_off[i] = offset(lp.wm * kWaveTile + i * kBlk + lp.l16, lp.lq);
      b_off[i] = kOperandBytes + offset(lp.wn * kWaveTile + i * kBlk + lp.l16, lp.lq);
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
      bf16x8 af[kBlocks], bf[kBlocks];
#pragma unroll
      for (int i = 0; i < kBlocks; ++i) {
        af[i] = *reinterpret_cast<const bf16x8*>(cur + a_off[i]);
        bf[i] = *reinterpret_cast<const bf16x8*>(cur + b_off[i]);
      }
#pragma unroll
      for (int i = 0; i < kBlocks; ++i)
#pragma unroll
        for (int j = 0; j < kBlocks; ++j) mfma_16x16x32(acc[i][j], af[i], bf[j]);
      if (more) {
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
          *reinterpret_cast<uint4*>(nxt + lds_off[i]) = ra[i];
          *reinterpret_cast<uint4*>(nxt + kOperandBytes + lds_off[i]) = rb[i];
        }
      }
      __syncthreads();
    }
    settle_acc();
  }
};

// Workgroup id -> (tile_m, tile_n).  Consecutive workgroup ids land on
// different XCDs (round-robin over 8), so ids are first regrouped so that each
// XCD walks a contiguous range, and inside that range tiles are visited in
// bands of `kBand` n-tiles so that concurrently resident workgroups of one XCD
// share A and B tiles in its L2 (32 workgroups per XCD: 8 x 4 tiles at kBand = 4, 4 x 8 at kBand = 8; the
// forward, whose A operand is the weight, is 1.7 % faster with 8, the output GEMMs 2.3 % faster with 4).
template <int kBand = 4>
__device__ __forceinline__ void tile_coords(int tiles_m, int tiles_n, int& tm, int& tn) {
  constexpr int kXcd = 8;
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
