// bf16 MFMA GEMM for gfx950 (MI355X), fp32 accumulate.
//
//   C[M,N] = opA(A) * opB(B)      with A given as [M,K] ("row": K contiguous)
//                                 or [K,M] ("col": M contiguous), and B given
//                                 as [N,K] ("row") or [K,N] ("col").
//
// The three products of a linear layer map onto it as
//   forward  Y  = X  W^T : A = X  row, B = W row           (M=tokens, N=out, K=in)
//   dgrad    dX = dY W   : A = dY row, B = W col            (M=tokens, N=in,  K=out)
//   wgrad    dW = dY^T X : A = dY col, B = X col            (M=out,    N=in,  K=tokens)
//
// Structure (one workgroup = 4 or 8 waves = one BMxBN tile, BK = 32):
//   * global -> LDS with buffer_load_dwordx4 ... lds (no VGPR staging; rows and
//     columns past the matrix edge read as zero through the buffer range check),
//     a ring of 4 stages of 32-deep k-tiles: tile kt+3 is requested while tile
//     kt is multiplied, its DMA instructions spread evenly between the MFMAs
//     (a burst of them right after a barrier backs up the address path and
//     stalls MFMA issue), one s_barrier per k-tile;
//   * LDS tiles are XOR-swizzled at 16-byte granularity so both the 1 KiB
//     linear DMA writes and the ds_read_b128 / ds_read_b64_tr_b16 fragment
//     reads are bank-conflict free;
//   * each wave owns a (BM/2)x(BN/2) sub-tile as 32x32 blocks of
//     v_mfma_f32_32x32x16_bf16.  The MFMA is issued with the B fragment as its
//     first operand, so a lane ends up holding 4 consecutive output columns of
//     one row: the epilogue packs them to bf16, stages 32 rows through LDS
//     and writes 16 bytes per lane, 256 contiguous bytes per row;
//   * workgroup ids are remapped so that the 32 CUs of one XCD (which share an
//     L2) walk neighbouring tiles.
#pragma once
#include "mtp_common.h"
#include <stdlib.h>
#include <type_traits>
#include <utility>

namespace {

#ifndef MTP_GEMM_VSTAGE
#define MTP_GEMM_VSTAGE 1
#endif
#ifndef MTP_STAGE_SKEW
#define MTP_STAGE_SKEW 1
#endif
#ifndef MTP_VSTAGE_SPREAD
#define MTP_VSTAGE_SPREAD 1
#endif
constexpr int BK = 32;      // k-tile depth
constexpr int NSTAGE = 4;   // LDS ring: 4 x (16 KiB A + 16 KiB B) at 256x256
constexpr int KSTEPS = BK / 16;  // MFMA k16 steps per k-tile
constexpr int LAY_ROW = 0;  // reduction dimension contiguous
constexpr int LAY_COL = 1;  // M (or N) contiguous

struct GemmArgs {
  const uint16_t* A;
  const uint16_t* B;
  void* C;             // main output (bf16 or fp32), may be null when C2 carries the result
  void* C2;            // activation output (bf16), epilogue dependent
  const uint16_t* bias;
  void* rowsum;        // EPI_ROWSUM: [M] sums of the rows of opA(A) over k (bf16 or fp32 like C; (+)= with accumulate)
  int M, N, K;
  int64_t lda, ldb, ldc, ldc2;
  int accumulate;      // C += result
  int half;            // SwiGLU: number of gate columns (N/2)
  // Stream-K (64-deep loop, 16x16x32, 4 waves only; sk_wgs == 0: every tile is one workgroup).  The tiles at
  // positions [0, sk_full) are one workgroup each; the k-tiles of the others, taken as one sequence tile after
  // tile, are dealt to sk_wgs further workgroups in runs of sk_ipw.  ws: device scratch, see SkLayout.
  int sk_full, sk_wgs, sk_ipw;
  void* ws;
#ifdef MTP_MEASURE
  int debug;           // measurement builds only (MTP_GEMM_DEBUG): 1 = every tile loads tile (0,0), 2 = no epilogue
                       // stores, 4 = every DMA reads out of range (no memory traffic).  Results are wrong with any bit set.
#endif
};
// The measurement switches exist only in builds made with -DMTP_MEASURE; the shipped library has none of them.
#ifdef MTP_MEASURE
#define MTP_DBG(p, bits) (((p).debug & (bits)) != 0)
#else
#define MTP_DBG(p, bits) false
#endif

enum : int { OUT_BF16 = 0, OUT_F32 = 1 };
// Plain product that also sums the rows of its A operand along k: with A = dY^T (the wgrad product) those sums
// are the bias gradient.  Every wave adds up the fragments it feeds to the MFMAs (one v_dot2 per pair of
// elements, in the shadow of the MFMAs); the first column of tiles writes the result.
constexpr int EPI_ROWSUM = 18;

// compile-time loop: f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N-1>{})
template <int... Is, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F&& f) {
  (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}
// one scheduling group of N instructions of the class MASK (N may be 0: nothing emitted)
template <int MASK, int N>
__device__ __forceinline__ void sched_group() {
  if constexpr (N > 0) __builtin_amdgcn_sched_group_barrier(MASK, N, 0);
}
constexpr int SG_MFMA = 0x008, SG_VMEM_RD = 0x020, SG_DS_RD = 0x100;

// LDS hand-over between lanes of one wave: DS operations of a wave complete in order, the fence and
// the scheduling barrier keep the compiler from moving accesses across the hand-over point.
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
  __builtin_amdgcn_wave_barrier();
}

// s_waitcnt immediate that waits for vmcnt <= n only (gfx9 encoding: vmcnt in bits 3:0 and 15:14,
// expcnt 6:4 and lgkmcnt 11:8 left at their maxima)
constexpr int vmcnt_imm(int n) { return (n & 0xf) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

// Raw buffer resource (stride 0): base address, num_records in bytes, gfx9 dword3 for untyped 32-bit data.
typedef __attribute__((ext_vector_type(4))) int rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void* base, int64_t bytes) {
  if (bytes < 0) bytes = 0;
  // offsets are tile relative and below 2^31; 0x80000000 is the "read as zero" marker
  const uint32_t n = bytes > 0x80000000ll ? 0x80000000u : (uint32_t)bytes;
  const uint64_t b = reinterpret_cast<uint64_t>(base);
  return rsrc_t{(int)(uint32_t)b, (int)((b >> 32) & 0xffffu), (int)n, 0x00020000};
}

// One DMA instruction: 64 lanes x 16 bytes from the buffer (VGPR offset voff, range checked; scalar offset
// soff, not checked) to LDS bytes [lds_addr, lds_addr + 1024) in lane order.  Written as inline assembly on
// purpose: the compiler then does not model the LDS write, and so does not put an s_waitcnt vmcnt(0) in
// front of every later ds_read_b64_tr_b16 (which it cannot prove independent of an in-flight DMA).  The
// kernel orders DMA against LDS reads itself: s_waitcnt vmcnt(0) + s_barrier once per k-tile.
__device__ __forceinline__ void dma16(rsrc_t rsrc, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff));
}
// The same with the LDS address given as a scalar base plus a compile-time offset: the many destinations of an
// unrolled loop then cost one live scalar register instead of one each (s_add_u32 leaves its carry in SCC).
// INST_OFF goes into the instruction's offset field, which moves the LDS address and the memory address alike:
// instructions that fill consecutive KiB of LDS can share one setting of M0 when each one's VGPR offset has
// INST_OFF taken off (the range check sees the sum, the true offset).  SET_M0: first instruction of such a run.
// The statements that follow a setting one read M0 without saying so (an inline-assembly statement can name M0
// neither as an input nor as a clobber: it is a reserved register, which the compiler never allocates and writes
// only where it lowers an instruction that needs it).  Between the statements of a run this file therefore puts
// MFMAs, LDS reads and scalar address arithmetic only: no indexed register access, no messages, no LDS-direct
// builtins, nothing that is lowered through M0.
template <bool SET_M0, int LDS_OFF, int INST_OFF>
__device__ __forceinline__ void dma16_at(rsrc_t rsrc, uint32_t lds_base, uint32_t voff, uint32_t soff) {
  static_assert(INST_OFF >= 0 && INST_OFF < 4096, "12-bit instruction offset");
  if constexpr (SET_M0)
    asm volatile("s_add_u32 m0, %0, %4\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen offset:%5 lds"
                 :
                 : "s"(lds_base), "v"(voff), "s"(rsrc), "s"(soff), "n"(LDS_OFF), "n"(INST_OFF)
                 : "scc");
  else
    asm volatile("buffer_load_dwordx4 %0, %1, %2 offen offset:%3 lds" : : "v"(voff), "s"(rsrc), "s"(soff), "n"(INST_OFF));
}
// Register-staged loads, also inline assembly so that their order against the DMA-style waits stays in this
// file's hands: 64 lanes x 16 bytes from the buffer into four VGPRs ...
__device__ __forceinline__ u32x4_t load16_to_vgpr(rsrc_t rsrc, uint32_t voff, uint32_t soff) {
  u32x4_t v;
  asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(v) : "v"(voff), "s"(rsrc), "s"(soff));
  return v;
}
// ... and, once at most PENDING younger loads are outstanding, from there to LDS
template <int PENDING, int OFFSET>
__device__ __forceinline__ void wait_and_write16(uint32_t lds_addr, u32x4_t v) {
  static_assert(OFFSET >= 0 && OFFSET < 65536 && PENDING >= 0 && PENDING < 64, "ds_write offset / vmcnt range");
  asm volatile("s_waitcnt vmcnt(%2)\n\tds_write_b128 %0, %1 offset:%3"
               :
               : "v"(lds_addr), "v"(v), "n"(PENDING), "n"(OFFSET)
               : "memory");
}
__device__ __forceinline__ uint32_t lds_addr_of(const void* p) {
  return (uint32_t)(uintptr_t)(const void __attribute__((address_space(3)))*)p;
}

// XCD-aware, grouped mapping of the linear workgroup id to a tile.
__device__ __forceinline__ void tile_of(int pid, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int total = tiles_m * tiles_n;
  constexpr int XCDS = 8, GROUP = 8;
  int id = pid;
  if (total >= XCDS * 4) {
    const int per = (total + XCDS - 1) / XCDS;
    int tall = total % XCDS;
    if (tall == 0) tall = XCDS;
    const int xcd = pid % XCDS, local = pid / XCDS;
    id = xcd < tall ? xcd * per + local : tall * per + (xcd - tall) * (per - 1) + local;
  }
  const int in_group = GROUP * tiles_n;
  const int gid = id / in_group;
  const int first = gid * GROUP;
  const int gsz = (tiles_m - first) < GROUP ? (tiles_m - first) : GROUP;
  const int r = id - gid * in_group;
  tm = first + r % gsz;
  tn = r / gsz;
}

// t-th block of a TI x TJ grid walked in growing squares: (0,0); (1,0) (1,1) (0,1); (2,0) (2,1) (2,2) (0,2) (1,2); ...
struct BlockIJ {
  int i, j;
};
constexpr BlockIJ shell_pair(int t, int TI, int TJ) {
  int n = 0;
  for (int d = 0; d < (TI > TJ ? TI : TJ); d++) {
    for (int j = 0; j <= d; j++)
      if (d < TI && j < TJ) {
        if (n == t) return BlockIJ{d, j};
        n++;
      }
    for (int i = 0; i < d; i++)
      if (i < TI && d < TJ) {
        if (n == t) return BlockIJ{i, d};
        n++;
      }
  }
  return BlockIJ{0, 0};
}

// ---------------------------------------------------------------------------
// Operands.  Each describes one side of the product for one workgroup: how its
// 32-deep k-tile is fetched into LDS by DMA and how a wave reads its MFMA
// fragments back.  "rows" below are the operand's M (or N) indices.
//
// RowOperand: memory is [rows, K] with K contiguous.  LDS tile = ROWS x 32 bf16,
//   64 bytes per row; the 16-byte chunk c of row r sits at chunk position
//   c ^ ((r >> 2) & 3), which spreads any 16 consecutive rows read at one k over
//   all 64 banks.  One DMA instruction fills 16 rows (lane l -> row l/4,
//   position l%4).  Fragment = one ds_read_b128 (8 consecutive k of one row).
//
// ColOperand: memory is [K, rows] with rows contiguous (a transposed operand).
//   LDS tile = 32 x ROWS bf16 in the same orientation, 2*ROWS bytes per k-row;
//   chunk c of k-row k sits at position c ^ ((k & 3) << 2).  One DMA
//   instruction fills 1 KiB of consecutive k-rows.  Fragment = two
//   ds_read_b64_tr_b16: inside each group of 16 lanes, lane i supplies the address
//   of 4 consecutive rows-elements of k-row (i/4) and receives, transposed, the
//   4 consecutive k of row i — exactly the MFMA operand layout.
// ---------------------------------------------------------------------------
constexpr int LROWS = 256;  // rows of the LDS tile layout; narrower tiles (192, 128) use its first rows

template <int ROWS, int NW>
struct RowOperand {
  static_assert(ROWS <= LROWS && ROWS % 64 == 0, "tile rows: 64, 128, 192 or 256");
  static constexpr int BYTES = LROWS * BK * 2;
  // DMA instructions per wave per k-tile (16 rows each); instructions whose rows all lie past ROWS are skipped
  static constexpr int NINSTR = (ROWS / 16 + NW - 1) / NW;
  static constexpr int NREADS = 1;               // LDS reads per fragment
  // Register-staged path (forward kernels): two k-tiles at a time, so that a load instruction covers whole
  // 128-byte lines: 8 rows x 128 bytes, lane l -> row l/8, 16-byte piece l%8 (pieces 0-3 belong to the even
  // k-tile of the pair, 4-7 to the odd one).  NPAIR such instructions per wave and pair of k-tiles.
  static constexpr int NPAIR = (ROWS / 8 + NW - 1) / NW;
  rsrc_t rsrc;
  uint32_t voff[NINSTR];
  uint32_t pvoff[NPAIR];   // global byte offsets of the paired loads (0x80000000: no such row)
  uint32_t pwoff;          // LDS byte offset (inside the operand's part of the even stage) of paired instruction 0
  uint32_t fo[KSTEPS];
  int chunk, K;

  // rowmap(r): global row (relative to row0) of tile row r, or a negative value for "no such row"
  template <typename RowMap>
  __device__ __forceinline__ void init(const uint16_t* base, int64_t ld, int row0, int nrows, int K_, int lane,
                                       int wave, int wave_row0, RowMap rowmap) {
    K = K_;
    // VGPR offsets are range checked against num_records: rows past the edge read as zero.  The k-tile
    // advance goes into the scalar offset (not checked; the ragged last k-tile is masked by hand).
    rsrc = make_rsrc(base + (int64_t)row0 * ld, (int64_t)(nrows - row0) * ld * 2);
    // lane l of instruction q fills row 16q + l/4, position l%4; (row >> 2) & 3 = (l >> 4) & 3
    chunk = (lane & 3) ^ ((lane >> 4) & 3);
    const int lrow = lane >> 2;
#pragma unroll
    for (int j = 0; j < NINSTR; j++) {
      const int r = (wave + NW * j) * 16 + lrow;
      const int64_t gr = r < ROWS ? rowmap(r) : -1;
      voff[j] = (gr < 0 || gr >= nrows - row0) ? 0x80000000u : (uint32_t)((gr * ld + chunk * 8) * 2);
    }
    const int row = wave_row0 + (lane & 31), h = lane >> 5;
#pragma unroll
    for (int kk = 0; kk < KSTEPS; kk++) fo[kk] = (uint32_t)(row * 64 + ((((2 * kk + h) ^ (row >> 2)) & 3) << 4));
    // paired loads: instruction j of this wave covers tile rows 8 (wave + NW j) .. + 7
    const int prow = lane >> 3, c8 = lane & 7;
#pragma unroll
    for (int j = 0; j < NPAIR; j++) {
      const int r = (wave + NW * j) * 8 + prow;
      const int64_t gr = r < ROWS ? rowmap(r) : -1;
      pvoff[j] = (gr < 0 || gr >= nrows - row0) ? 0x80000000u : (uint32_t)((gr * ld + c8 * 8) * 2);
    }
    // where the lane's 16 bytes go: stage of the even or odd k-tile, row r, piece (c8 & 3) swizzled like the
    // DMA path does; (r >> 2) & 3 = (2 wave + lane / 32) & 3 for every j (8 NW j is a multiple of 4)
    {
      const int r0 = wave * 8 + prow;
      pwoff = (uint32_t)(r0 * 64 + ((((c8 & 3) ^ (r0 >> 2)) & 3) << 4));
    }
  }
  // odd k-tile of the pair: the lane's piece goes one stage further
  __device__ __forceinline__ bool pair_odd(int lane) const { return (lane & 4) != 0; }
  // Per k-tile state of the DMA.  INSIDE: the caller knows the k-tile lies completely below K (no tail
  // masking needed).
  struct Prep {
    uint32_t soff;
    bool dead;
  };
  template <bool INSIDE>
  __device__ __forceinline__ Prep prep(int kt) const {
    return Prep{(uint32_t)(kt * BK * 2), !INSIDE && kt * BK + chunk * 8 >= K};  // ragged last k-tile / past the end
  }
  // j-th DMA instruction of this wave; tile = LDS byte address of the operand's stage
  __device__ __forceinline__ void issue(const Prep& pp, uint32_t tile, int wave, int j) const {
    dma16(rsrc, tile + (wave + NW * j) * 1024, pp.dead ? 0x80000000u : voff[j], pp.soff);
  }
  __device__ __forceinline__ bf16x8_t frag(const char* tile, int kk, int blk) const {
    return *reinterpret_cast<const bf16x8_t*>(tile + fo[kk] + blk * (32 * BK * 2));
  }
};

template <int ROWS, int NW>
struct ColOperand {
  static_assert(ROWS <= LROWS && ROWS % 64 == 0, "tile rows: 64, 128, 192 or 256");
  static constexpr int BYTES = BK * LROWS * 2;
  static constexpr int NINSTR = BYTES / 1024 / NW;
  static constexpr int NREADS = 2;
  static constexpr int NPAIR = 0;   // no register-staged form: a DMA instruction already covers whole lines
  const char* base;    // &mem[0][row0]
  int64_t total;       // bytes from base to the end of the matrix
  int64_t ktile_bytes; // BK * ld * 2
  uint32_t voff[NINSTR];
  uint32_t lane_base;
  uint32_t moff[4];

  __device__ __forceinline__ void init(const uint16_t* mem, int64_t ld, int row0, int K_, int lane, int wave,
                                       int wave_row0) {
    base = reinterpret_cast<const char*>(mem + row0);
    total = ((int64_t)K_ * ld - row0) * 2;
    ktile_bytes = (int64_t)BK * ld * 2;
    // DMA: instruction q = wave + NW*j covers k-rows 2q, 2q+1 (512 bytes each); lane l -> k-row 2q + l/32,
    // LDS position l%32, which holds chunk position ^ ((k & 3) << 2)
    const int ksub = lane >> 5;
    const int c = (lane & 31) ^ (((2 * wave + ksub) & 3) << 2);
#pragma unroll
    for (int j = 0; j < NINSTR; j++) {
      const int krow = 2 * (wave + NW * j) + ksub;
      // chunks past the tile's ROWS are not fetched (narrow tiles)
      voff[j] = c * 8 < ROWS ? (uint32_t)(((int64_t)krow * ld + c * 8) * 2) : 0x80000000u;
    }
    // fragment reads: lane (group G = l/16, i = l%16) addresses k-row 8*(G/2) + i/4 (+16kk, +4 for the
    // second read) and rows 16*(G%2) + 4*(i%4) .. +3 of the block; the chunk swizzle is applied per block
    const int G = lane >> 4, i = lane & 15, kq = i >> 2;
    const int cw = wave_row0 >> 3;  // first chunk of the wave's rows
    lane_base = (uint32_t)((8 * (G >> 1) + kq) * (LROWS * 2) + 8 * (i & 1));
#pragma unroll
    for (int blk = 0; blk < 4; blk++) {
      const int c2 = cw + 4 * blk + 2 * (G & 1) + ((i & 3) >> 1);
      moff[blk] = (uint32_t)((c2 ^ (kq << 2)) * 16);
    }
  }
  struct Prep {
    rsrc_t r;
  };
  template <bool INSIDE>
  __device__ __forceinline__ Prep prep(int kt) const {
    // the whole address, k-tile advance included, goes through the range check: k-rows past K and the
    // tail of the last row read as zero
    return Prep{make_rsrc(base + kt * ktile_bytes, total - kt * ktile_bytes)};
  }
  __device__ __forceinline__ void issue(const Prep& pp, uint32_t tile, int wave, int j) const {
    dma16(pp.r, tile + (wave + NW * j) * 1024, voff[j], 0);
  }
  __device__ __forceinline__ bf16x8_t frag(const char* tile, int kk, int blk) const {
    const char* a = tile + lane_base + moff[blk] + kk * (16 * LROWS * 2);
    const bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
        (bf16x4_t __attribute__((address_space(3)))*)(a));
    const bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
        (bf16x4_t __attribute__((address_space(3)))*)(a + 4 * LROWS * 2));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  }
};

template <int LAY, int ROWS, int NW> struct OperandOf { using type = RowOperand<ROWS, NW>; };
template <int ROWS, int NW> struct OperandOf<LAY_COL, ROWS, NW> { using type = ColOperand<ROWS, NW>; };

// ---------------------------------------------------------------------------
// Epilogue, shared by the two main loops.  acc[i][j] is the 32x32 block (i, j) of the wave's part of the tile;
// which rows and columns of the tile that is depends on the main loop:
//   QMAP = false: the wave owns a contiguous (BM/2) x (BN/WGN) rectangle: block row i starts at tile row
//                 wm*BM/2 + 32 i, block column j at tile column wn*BN/WGN + 32 j;
//   QMAP = true:  the tile's rows (columns) form two halves, and a wave owns HI (HJ) blocks of each half:
//                 block row i starts at tile row (i/HI)*BM/2 + wm*32*HI + 32 (i%HI), columns likewise.
// With SwiGLU both forms put the gate columns into blocks j < TJ/2 and the matching up columns into the others.
// ---------------------------------------------------------------------------
//
// The accumulators come through an accessor, so that both MFMA shapes are served.  Seen from here the wave's part
// is a TI x TJ grid of 32x32 blocks, and of block (i, j) a lane holds four groups g of four consecutive columns:
//   BLK = 32 (v_mfma_f32_32x32x16, B fragment first): group g = row l%32, columns 8 g + 4 (l/32) .. +3;
//   BLK = 16 (v_mfma_f32_16x16x32, B fragment first; the block is 2x2 MFMA blocks): group g = row
//            16 (g/2) + l%16, columns 16 (g%2) + 4 (l/16) .. +3.
// accv(i, j, g, e) is element e of group g; rsum_of(i, g) (EPI_ROWSUM only) the lane's part of the k sum of the
// A row that group g sits in.
// The wave grid is WGM x WGN.  Along a dimension with one wave only (the 64-deep loop's 160- and 192-wide tiles:
// 4 x 1 or 1 x 4 waves) the two units lie side by side and the wave's blocks are simply consecutive.
template <int BM, int BN, int EPI, int OUT, int WGM, int WGN, bool F16, bool QMAP, int LDS_BYTES, int TI, int TJ, int BLK,
          typename AccFn, typename RsumFn>
__device__ __forceinline__ void gemm_epilogue(const GemmArgs& p, AccFn accv, RsumFn rsum_of, char* lds, int m0, int n0,
                                              int tn, int wave, int lane) {
  using X = X16<F16>;
  static_assert(BLK == 32 || BLK == 16, "MFMA block: 32x32 or 16x16");
  constexpr int NW = WGM * WGN;
  constexpr int HI = TI / 2, HJ = TJ / 2;
  constexpr bool QM = QMAP && WGM > 1, QN = QMAP && WGN > 1;    // unit mapping along m / n
  static_assert((!QM || TI % 2 == 0) && (!QN || TJ % 2 == 0), "two units of whole 32-wide blocks per wave");
  const int wm = wave / WGN, wn = wave % WGN;
  // row (inside the 32-row block) and first column (inside the 32-column block) of group g
  auto row_off = [&](int g) -> int { return BLK == 32 ? (lane & 31) : 16 * (g >> 1) + (lane & 15); };
  auto col_off = [&](int g) -> int { return BLK == 32 ? 8 * g + 4 * (lane >> 5) : 16 * (g & 1) + 4 * (lane >> 4); };
  // first tile row of the wave's block row i
  auto blk_row = [&](int i) -> int {
    if (QM) return (i / HI) * (BM / 2) + wm * (32 * HI) + (i % HI) * 32;
    return wm * (BM / WGM) + 32 * i;
  };

  if constexpr (EPI == EPI_ROWSUM) {

    if (tn == 0 && wn == 0) {
#pragma unroll
      for (int i = 0; i < TI; i++)
#pragma unroll
        for (int g = 0; g < (BLK == 32 ? 1 : 4); g += 2) {
          // the lanes that hold the same row at other k add up: 2 halves (32x32x16) or 4 quarters (16x16x32)
          float t = rsum_of(i, g);
          t += __shfl_xor(t, 32, 64);
          if (BLK == 16) t += __shfl_xor(t, 16, 64);
          const int row = m0 + blk_row(i) + row_off(g);
          if (lane < BLK && row < p.M) {
            if (OUT == OUT_F32) {
              float* q = (float*)p.rowsum + row;
              *q = p.accumulate ? *q + t : t;
            } else {
              uint16_t* q = (uint16_t*)p.rowsum + row;
              *q = X::to_bits(p.accumulate ? X::from_bits(*q) + t : t);
            }
          }
        }
    }
  }

  // ---- epilogue ----------------------------------------------------------------
  // group g of block (i, j): row m0 + blk_row(i) + row_off(g), columns col_of_block(j) + col_off(g) .. +3.
  // Stage 32 rows x (BN/2) columns per wave through LDS, then 16-byte row-contiguous stores.
  constexpr int WN = BN / WGN;                     // columns per wave
  constexpr int ESZ = (OUT == OUT_F32) ? 4 : 2;
  constexpr int PITCH = WN * ESZ + 16;             // bytes per staged row (+16: spread rows over banks)
  static_assert(NW * 32 * PITCH <= LDS_BYTES, "epilogue staging exceeds the tile buffers");
  char* stage = lds + wave * (32 * PITCH);

  // global column of the first element of block j for this wave (main output C)
  auto col_of_block = [&](int j) -> int {
    if (EPI == MTP_EPI_SWIGLU) {
      const int hj = TJ / 2;
      return (j < hj ? 0 : p.half) + n0 + wn * (WN / 2) + (j % hj) * 32;
    }
    if (QN) return n0 + (j / HJ) * (BN / 2) + wn * (32 * HJ) + (j % HJ) * 32;
    return n0 + wn * WN + j * 32;
  };
  // first column past the valid range of block j: SwiGLU gate blocks end at `half` (the columns after it
  // are the up matrix, owned by other blocks)
  auto lim_of_block = [&](int j) -> int {
    if (EPI == MTP_EPI_SWIGLU) return j < TJ / 2 ? p.half : p.N;
    return p.N;
  };

  // The whole tile lies inside the matrix: the epilogue needs no bounds checks.
  const bool tile_inside = m0 + BM <= p.M && (EPI == MTP_EPI_SWIGLU ? n0 + BN / 2 <= p.half : n0 + BN <= p.N);

  // Fast path of flush, for the blocks [JB, JB + NB) of the staged row (NB a power of two, at most 4): 16-byte
  // aligned rows of a tile that is completely inside: lane l owns chunk l % CPR of rows l / CPR, l / CPR + 64 / CPR,
  // ...; one address computation, then constant strides.
  // Accumulating into C (C += result): the old values of block row i, one 16-byte vector per store of the fast
  // path (piece JB holds its ITERS vectors from old_c[JB * esz] on).  They are asked for at the top of the block
  // row, before its values are rounded and staged, so that one memory latency stands in front of the stores of a
  // block row instead of one in front of every store (a load may not move up past the store before it).
  constexpr int OLD_N = TJ * ESZ;
  [[maybe_unused]] u32x4_t old_c[OLD_N];
  const bool c_fast = tile_inside && p.C && ((reinterpret_cast<uintptr_t>(p.C) | (uintptr_t)(p.ldc * ESZ)) & 15) == 0;
  const bool preload_c = c_fast && p.accumulate != 0;
  auto piece_addr = [&](int i, void* out, int64_t ld, auto jb_tag, auto nb_tag, auto colfn, auto f32_tag, char*& gp,
                        int64_t& gstride) {
    constexpr int JB = decltype(jb_tag)::value, NB = decltype(nb_tag)::value;
    constexpr int esz_c = decltype(f32_tag)::value ? 4 : 2;
    constexpr int CPR = NB * 32 * esz_c / 16, RPI = 64 / CPR;
    const int r0 = lane / CPR, cc = lane % CPR;
    const int e0 = cc * (16 / esz_c);
    const int col = colfn(JB + (e0 >> 5)) + (e0 & 31);
    gp = (char*)out + ((int64_t)(m0 + blk_row(i) + r0) * ld + col) * esz_c;
    gstride = (int64_t)RPI * ld * esz_c;
  };
  auto preload_piece = [&](int i, auto jb_tag, auto nb_tag, auto colfn) {
    constexpr int JB = decltype(jb_tag)::value, NB = decltype(nb_tag)::value;
    constexpr int CPR = NB * 32 * ESZ / 16, RPI = 64 / CPR, ITERS = 32 / RPI;
    static_assert(JB * ESZ + ITERS <= OLD_N, "old values of a block row");
    char* gp;
    int64_t gstride;
    piece_addr(i, p.C, p.ldc, jb_tag, nb_tag, colfn, std::integral_constant<bool, OUT == OUT_F32>{}, gp, gstride);
#pragma unroll
    for (int it = 0; it < ITERS; it++) old_c[JB * ESZ + it] = *reinterpret_cast<const u32x4_t*>(gp + it * gstride);
  };
  auto flush_piece = [&](int i, void* out, int64_t ld, auto jb_tag, auto nb_tag, auto colfn, auto f32_tag, bool accumulate) {
    constexpr int JB = decltype(jb_tag)::value, NB = decltype(nb_tag)::value;
    constexpr bool f32out = decltype(f32_tag)::value;
    constexpr int esz_c = f32out ? 4 : 2;
    constexpr int CPR = NB * 32 * esz_c / 16;                              // 16-byte chunks per staged row piece
    static_assert(CPR == 4 || CPR == 8 || CPR == 16 || CPR == 32, "a power of two of lanes per row");
    constexpr int RPI = 64 / CPR, ITERS = 32 / RPI;
    const int r0 = lane / CPR, cc = lane % CPR;
    const int e0 = cc * (16 / esz_c);
    const int col = colfn(JB + (e0 >> 5)) + (e0 & 31);
    char* gp = (char*)out + ((int64_t)(m0 + blk_row(i) + r0) * ld + col) * esz_c;
    const char* sp = stage + r0 * PITCH + JB * 32 * esz_c + cc * 16;
    const int64_t gstride = (int64_t)RPI * ld * esz_c;
#pragma unroll
    for (int it = 0; it < ITERS; it++) {
      u32x4_t v = *reinterpret_cast<const u32x4_t*>(sp + it * RPI * PITCH);
      u32x4_t* q = reinterpret_cast<u32x4_t*>(gp + it * gstride);
      if (accumulate) {
        // (accumulation only ever goes into C, whose old values were asked for ahead)
        const u32x4_t o = (esz_c == ESZ && JB * esz_c + it < OLD_N) ? old_c[JB * esz_c + it] : *q;
        if (f32out) {
          v.x = __float_as_uint(__uint_as_float(v.x) + __uint_as_float(o.x));
          v.y = __float_as_uint(__uint_as_float(v.y) + __uint_as_float(o.y));
          v.z = __float_as_uint(__uint_as_float(v.z) + __uint_as_float(o.z));
          v.w = __float_as_uint(__uint_as_float(v.w) + __uint_as_float(o.w));
        } else {
          v.x = X::pack2(X::lo(v.x) + X::lo(o.x), X::hi(v.x) + X::hi(o.x));
          v.y = X::pack2(X::lo(v.y) + X::lo(o.y), X::hi(v.y) + X::hi(o.y));
          v.z = X::pack2(X::lo(v.z) + X::lo(o.z), X::hi(v.z) + X::hi(o.z));
          v.w = X::pack2(X::lo(v.w) + X::lo(o.w), X::hi(v.w) + X::hi(o.w));
        }
      }
      __builtin_nontemporal_store(v, q);  // written once, read by a later kernel: keep it out of the way of A/B in L2
    }
  };
  auto flush = [&](int i, void* out, int64_t ld, auto nblk_tag, auto colfn, auto limfn, auto f32_tag, bool accumulate) {
    constexpr int nblk = decltype(nblk_tag)::value;
    constexpr bool f32out = decltype(f32_tag)::value;
    {
      constexpr int esz_c = f32out ? 4 : 2;
      const bool aligned = ((reinterpret_cast<uintptr_t>(out) | (uintptr_t)(ld * esz_c)) & 15) == 0;
      if (tile_inside && aligned) {
        // the staged row goes out in pieces of 4, 2 and 1 blocks (a 5-block row: 4 + 1), each with a power of two
        // of lanes per row
        constexpr int STEP = 4;
        constexpr int N4 = nblk / STEP, REM = nblk % STEP;
        static_for<N4>([&](auto t) {
          flush_piece(i, out, ld, std::integral_constant<int, decltype(t)::value * STEP>{}, std::integral_constant<int, STEP>{},
                      colfn, f32_tag, accumulate);
        });
        if constexpr (REM >= 2)
          flush_piece(i, out, ld, std::integral_constant<int, N4 * STEP>{}, std::integral_constant<int, 2>{}, colfn, f32_tag,
                      accumulate);
        if constexpr (REM % 2 == 1)
          flush_piece(i, out, ld, std::integral_constant<int, N4 * STEP + (REM >= 2 ? 2 : 0)>{}, std::integral_constant<int, 1>{},
                      colfn, f32_tag, accumulate);
        return;
      }
    }
    // 16-byte chunks of the staged 32 x (nblk*32) block
    const int esz = f32out ? 4 : 2;
    const int chunks_per_row = nblk * 32 * esz / 16;
    const int epc = 16 / esz;  // elements per chunk
    const int total = 32 * chunks_per_row;
    const int mrow0 = m0 + blk_row(i);
    for (int c = lane; c < total; c += 64) {
      const int r = c / chunks_per_row, cc = c - r * chunks_per_row;
      const int e0 = cc * epc;           // element offset inside the staged row
      const int j = e0 >> 5;
      const int col = colfn(j) + (e0 & 31);
      const int col_limit = limfn(j);
      const int row = mrow0 + r;
      if (row < p.M && col < col_limit) {
        u32x4_t v = *reinterpret_cast<const u32x4_t*>(stage + r * PITCH + cc * 16);
        char* gp = (char*)out + ((int64_t)row * ld + col) * esz;
        if (col + epc <= col_limit && ((reinterpret_cast<uintptr_t>(gp) & 15) == 0)) {
          if (accumulate) {
            u32x4_t o = *reinterpret_cast<const u32x4_t*>(gp);
            if (f32out) {
              v.x = __float_as_uint(__uint_as_float(v.x) + __uint_as_float(o.x));
              v.y = __float_as_uint(__uint_as_float(v.y) + __uint_as_float(o.y));
              v.z = __float_as_uint(__uint_as_float(v.z) + __uint_as_float(o.z));
              v.w = __float_as_uint(__uint_as_float(v.w) + __uint_as_float(o.w));
            } else {
              v.x = X::pack2(X::lo(v.x) + X::lo(o.x), X::hi(v.x) + X::hi(o.x));
              v.y = X::pack2(X::lo(v.y) + X::lo(o.y), X::hi(v.y) + X::hi(o.y));
              v.z = X::pack2(X::lo(v.z) + X::lo(o.z), X::hi(v.z) + X::hi(o.z));
              v.w = X::pack2(X::lo(v.w) + X::lo(o.w), X::hi(v.w) + X::hi(o.w));
            }
          }
          *reinterpret_cast<u32x4_t*>(gp) = v;
        } else {
          // ragged right edge or unaligned row: element by element
          const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
          for (int e = 0; e < epc && col + e < col_limit; e++) {
            if (f32out) {
              float* q = reinterpret_cast<float*>(gp) + e;
              const float nv = __uint_as_float(w4[e]);
              *q = accumulate ? *q + nv : nv;
            } else {
              uint16_t* q = reinterpret_cast<uint16_t*>(gp) + e;
              const uint32_t pr = w4[e >> 1];
              const float nv = (e & 1) ? X::hi(pr) : X::lo(pr);
              *q = X::to_bits(accumulate ? X::from_bits(*q) + nv : nv);
            }
          }
        }
      }
    }
  };

  // the pieces of flush's fast path for the TJ blocks of a row of C
  auto preload_row = [&](int i) {
    constexpr int STEP = 4, N4 = TJ / STEP, REM = TJ % STEP;
    static_for<N4>([&](auto t) {
      preload_piece(i, std::integral_constant<int, decltype(t)::value * STEP>{}, std::integral_constant<int, STEP>{}, col_of_block);
    });
    if constexpr (REM >= 2) preload_piece(i, std::integral_constant<int, N4 * STEP>{}, std::integral_constant<int, 2>{}, col_of_block);
    if constexpr (REM % 2 == 1)
      preload_piece(i, std::integral_constant<int, N4 * STEP + (REM >= 2 ? 2 : 0)>{}, std::integral_constant<int, 1>{}, col_of_block);
  };

#pragma unroll
  for (int i = 0; i < TI; i++) {
    if (preload_c) preload_row(i);
    // -- pre-activation (or plain) output: add bias, round, stage
    float pre[TJ][16];
#pragma unroll
    for (int j = 0; j < TJ; j++) {
      const int cb = col_of_block(j);
#pragma unroll
      for (int g = 0; g < 4; g++) {
        float b4[4] = {0.f, 0.f, 0.f, 0.f};
        if (EPI == MTP_EPI_BIAS || EPI == MTP_EPI_BIAS_GELU || (EPI == MTP_EPI_SWIGLU)) {
          if (p.bias) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
              const int col = cb + col_off(g) + e;
              b4[e] = col < lim_of_block(j) ? X::from_bits(p.bias[col]) : 0.f;
            }
          }
        }
        // (without a bias there is nothing to add: x + 0 is not x for the compiler, which would keep 256 additions)
#pragma unroll
        for (int e = 0; e < 4; e++) {
          if constexpr (EPI == MTP_EPI_BIAS || EPI == MTP_EPI_BIAS_GELU || EPI == MTP_EPI_SWIGLU)
            pre[j][4 * g + e] = accv(i, j, g, e) + b4[e];
          else
            pre[j][4 * g + e] = accv(i, j, g, e);
        }
      }
    }
    if (OUT == OUT_F32) {
      if (p.C) {
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
          for (int g = 0; g < 4; g++) {
            f32x4_t v = {pre[j][4 * g], pre[j][4 * g + 1], pre[j][4 * g + 2], pre[j][4 * g + 3]};
            *reinterpret_cast<f32x4_t*>(stage + row_off(g) * PITCH + (32 * j + col_off(g)) * 4) = v;
          }
        wave_lds_sync();
        flush(i, p.C, p.ldc, std::integral_constant<int, TJ>{}, col_of_block, lim_of_block, std::true_type{}, p.accumulate != 0);
        wave_lds_sync();
      }
    } else {
      // round to bf16 once (one v_cvt_pk_bf16_f32 per pair); an activation sees the rounded value, as
      // the unfused layers would
      uint32_t pk[TJ][8];
#pragma unroll
      for (int j = 0; j < TJ; j++)
#pragma unroll
        for (int q = 0; q < 8; q++) pk[j][q] = X::pack2(pre[j][2 * q], pre[j][2 * q + 1]);
      if (p.C) {
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
          for (int g = 0; g < 4; g++) {
            u32x2_t v = {pk[j][2 * g], pk[j][2 * g + 1]};
            *reinterpret_cast<u32x2_t*>(stage + row_off(g) * PITCH + (32 * j + col_off(g)) * 2) = v;
          }
        wave_lds_sync();
        flush(i, p.C, p.ldc, std::integral_constant<int, TJ>{}, col_of_block, lim_of_block, std::false_type{}, p.accumulate != 0);
        wave_lds_sync();
      }
      if (EPI != MTP_EPI_NONE && EPI != MTP_EPI_BIAS && EPI != EPI_ROWSUM) {
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
          for (int q = 0; q < 8; q++) {
            pre[j][2 * q] = X::lo(pk[j][q]);
            pre[j][2 * q + 1] = X::hi(pk[j][q]);
          }
      }
      if constexpr (EPI == MTP_EPI_BIAS_GELU || EPI == MTP_EPI_GELU) {
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
          for (int g = 0; g < 4; g++) {
            u32x2_t v = {X::pack2(gelu_new_f(pre[j][4 * g]), gelu_new_f(pre[j][4 * g + 1])),
                         X::pack2(gelu_new_f(pre[j][4 * g + 2]), gelu_new_f(pre[j][4 * g + 3]))};
            *reinterpret_cast<u32x2_t*>(stage + row_off(g) * PITCH + (32 * j + col_off(g)) * 2) = v;
          }
        wave_lds_sync();
        flush(i, p.C2, p.ldc2, std::integral_constant<int, TJ>{}, col_of_block, lim_of_block, std::false_type{}, false);
        wave_lds_sync();
      }
      if constexpr (EPI == MTP_EPI_SWIGLU) {
        constexpr int HJ = TJ / 2;
#pragma unroll
        for (int j = 0; j < HJ; j++)
#pragma unroll
          for (int g = 0; g < 4; g++) {
            float a4[4];
#pragma unroll
            for (int e = 0; e < 4; e++) a4[e] = silu_f(pre[j][4 * g + e]) * pre[j + HJ][4 * g + e];
            u32x2_t v = {X::pack2(a4[0], a4[1]), X::pack2(a4[2], a4[3])};
            *reinterpret_cast<u32x2_t*>(stage + row_off(g) * PITCH + (32 * j + col_off(g)) * 2) = v;
          }
        wave_lds_sync();
        auto act_col = [&](int j) -> int { return n0 + wn * (WN / 2) + j * 32; };
        auto act_lim = [&](int) -> int { return p.half; };
        flush(i, p.C2, p.ldc2, std::integral_constant<int, HJ>{}, act_col, act_lim, std::false_type{}, false);
        wave_lds_sync();
      }
    }
  }
}

// ---------------------------------------------------------------------------
// The 64-deep main loop ("Q" configurations of the 256x256 tile).
//
// A k-tile is 64 deep, so that the slice of a K-contiguous row is one whole 128-byte line and one DMA
// instruction requests 8 whole lines.  LDS holds two k-tiles (2 x 64 KiB); each operand's tile is split by rows
// into two units of 128 rows (16 KiB), and a wave owns HI (HJ) 32-row blocks of either unit, so its part of the
// tile is four quadrants Q(I,J) = unit I of A x unit J of B.  A wave keeps the fragments of all four units of
// the current k-tile in registers (one register set per unit) and works through the quadrants, 4 k16 steps
// each, in an order in which consecutive quadrants share a unit:
//
//   even tile t:  Q00  Q01 | Q11  Q10        reads meanwhile:  B1[t]  A1[t]   | A0[t+1]  B1[t+1]
//   odd  tile t:  Q01  Q00 | Q10  Q11                          B0[t]  A1[t]   | A0[t+1]  B0[t+1]
//
// (every register set is refilled during the phase after its last use).  A unit of LDS is free as soon as every
// wave has copied it to registers, long before the MFMAs that use the copy are done: one barrier per half
// k-tile (the "|") hands the two units read since the previous barrier to the DMA, which refills them with
// the tile after next while the following half tile is multiplied.  A unit is requested three half tiles
// (about 1.5 k-tiles of 64) before it is read; s_waitcnt vmcnt(n) in front of the barrier asks for exactly
// the two units the next half tile reads.  The requests of tiles past the end of k are still issued, with
// every lane out of range (zero fill, no memory traffic), so that the counting never changes.
// ---------------------------------------------------------------------------
//
// BLK picks the MFMA: 32 = v_mfma_f32_32x32x16 (4 steps of 16 per k-tile), 16 = v_mfma_f32_16x16x32 (2 steps of 32).
// Per flop the 16x16x32 form moves half the accumulator registers and twice the operand registers, 8 against 10
// KiB per 32 Kflop in all, and on operands of random sign and mantissa the matrix cores sustain about 15 % more
// with it at the board's power limit (register-resident loops with 256 accumulator registers per lane: 2120
// against 1850 TFLOP/s).
constexpr int QBK = 64;    // k-tile depth

// K-contiguous operand: LDS unit = 128 rows x 128 bytes; the 16-byte chunk c of row r sits at position
// c ^ ((r >> 1) & 7): 16 consecutive rows read at one k cover all 64 banks.  One DMA instruction fills 8 rows
// (lane l -> row l/8, position l%8, fetching chunk (l%8) ^ swizzle of its row: the 8 lanes of a row still ask
// for one whole line); a wave's NU instructions of a unit fill 8 NU consecutive rows, so that they share one
// setting of M0 (dma16_at).  Fragment = one ds_read_b128.
//
// UR = rows per unit: 128 (256-row tile), or 96 / 80 for the 192- and 160-row tiles, whose units are padded in LDS
// to the rows the waves' DMA instructions cover (8 NU NW); the instructions of the padding rows read out of range.
template <int NW, int WG, int BLK, int UR = 128>
struct RowOperandQ {
  static constexpr int UROWS = UR;                   // rows per unit
  static constexpr int NU = (UROWS / 8 + NW - 1) / NW;   // DMA instructions per wave and unit
  static constexpr int UBYTES = NU * NW * 8 * QBK * 2;   // 16 KiB at 128 rows
  static constexpr int BYTES = 2 * UBYTES;           // per k-tile buffer
  static constexpr int QKS = BLK == 32 ? 4 : 2;      // MFMA steps per k-tile
  static constexpr int H = UROWS / (BLK * WG);       // BLK-row blocks per wave and unit
  static_assert(H >= 1 && NU >= 1 && H * BLK * WG == UROWS && UROWS % 8 == 0, "wave grid does not divide the unit");
  rsrc_t rsrc;
  uint32_t voff[2][NU];
  uint32_t fo[2][QKS];   // [k-tile buffer][step]: the buffer's 64 KiB do not fit the 16-bit offset field of a read

  // rowmap(r): global row (relative to row0) of tile row r (unit r / UROWS), or a negative value for "no such row";
  // wsub: the wave's index along this operand's dimension
  template <typename RowMap>
  __device__ __forceinline__ void init(const uint16_t* base, int64_t ld, int row0, int nrows, int K_, int lane,
                                       int wave, int wsub, RowMap rowmap) {
    (void)K_;   // a multiple of the k-tile depth (the host checks): no k-tile is ragged
    rsrc = make_rsrc(base + (int64_t)row0 * ld, (int64_t)(nrows - row0) * ld * 2);
    // tile row of lane l in instruction j of unit u: 128 u + 8 (NU wave + j) + l/8; its swizzle (row >> 1) & 7
    // = (4 (NU wave + j) + l/16) & 7
#pragma unroll
    for (int u = 0; u < 2; u++)
#pragma unroll
      for (int j = 0; j < NU; j++) {
        const int q = NU * wave + j;
        const int gchunk = (lane & 7) ^ ((4 * q + (lane >> 4)) & 7);
        const int ru = q * 8 + (lane >> 3);                       // row inside the (padded) unit
        const int64_t gr = ru < UROWS ? rowmap(u * UROWS + ru) : -1;
        // a valid row r >= 8 j lies at least 1024 j bytes into the buffer (rows are at least 128 bytes long)
        voff[u][j] = ((gr < 0 || gr >= nrows - row0) ? 0x80000000u : (uint32_t)((gr * ld + gchunk * 8) * 2)) - 1024u * j;
      }
    // fragment of block b at step kk: row BLK (H wsub + b) + l % BLK of the unit, 8 k from 8 (64 / BLK) kk + 8 (l / BLK)
    const int lr = lane & (BLK - 1), h = lane / BLK;
#pragma unroll
    for (int kk = 0; kk < QKS; kk++) {
      fo[0][kk] = (uint32_t)((wsub * BLK * H + lr) * 128 + (((((64 / BLK) * kk + h) ^ (lr >> 1)) & 7) << 4));
      fo[1][kk] = fo[0][kk] + 65536;
    }
  }
  struct Prep {
    rsrc_t r;
    uint32_t soff;
  };
  // kend: first k-tile past the range this workgroup multiplies: requests beyond it go through an empty resource
  // (zero fill, no memory traffic), a scalar choice that costs the lanes nothing
  __device__ __forceinline__ Prep prep(int kt, int kend) const {
    rsrc_t r = rsrc;
    if (kt >= kend) r[2] = 0;
    return Prep{r, (uint32_t)(kt * QBK * 2)};
  }
  // J-th DMA instruction of this wave for unit U, which sits UNIT_OFF bytes into the tile buffers;
  // wave_lds = LDS byte address of the tile buffers + 1024 * NU * wave
  template <int UNIT_OFF, int U, int J>
  __device__ __forceinline__ void issue(const Prep& pp, uint32_t wave_lds) const {
    dma16_at<J == 0, UNIT_OFF, 1024 * J>(pp.r, wave_lds, voff[U][J], pp.soff);
  }
  // unit: address of the unit in k-tile buffer 0
  __device__ __forceinline__ bf16x8_t frag(const char* unit, int buf, int b, int kk) const {
    return *reinterpret_cast<const bf16x8_t*>(unit + b * (BLK * 128) + fo[buf][kk]);
  }
};

// Transposed operand (memory [K, rows], rows contiguous): LDS unit = 64 k-rows x 128 rows, 256 bytes per k-row;
// chunk c of k-row k sits at position c ^ ((k & 3) << 2) ^ ((k >> 3 & 1) << 1): the four k-rows a group of 16
// lanes reads land on four different 64-byte bank groups, and the k-rows 8 apart that the two groups of one
// ds_read_b64_tr_b16 pass read in the 16x16x32 form land 32 bytes apart.  One DMA instruction fills 4 k-rows
// (lane l -> k-row l/16, position l%16).  Fragment = two ds_read_b64_tr_b16: in each group of 16 lanes, lane i
// supplies the address of 4 consecutive rows-elements of one k-row and receives, transposed, 4 consecutive k of
// one row; BLK = 32: group G holds rows 16 (G%2) .. +15 at k 8 (G/2) .. +7, BLK = 16: rows 0 .. 15 at k 8 G .. +7.
//
// UR = rows per unit.  Units of 96 / 80 rows keep the 256-byte k-rows in LDS; the lanes whose chunk lies past the
// unit's rows read out of range (zero fill, no memory traffic).
template <int NW, int WG, int BLK, int UR = 128>
struct ColOperandQ {
  static constexpr int UROWS = UR;
  static constexpr int LROWS_U = 128;                // rows of a k-row in LDS
  static constexpr int UBYTES = QBK * LROWS_U * 2;
  static constexpr int BYTES = 2 * UBYTES;
  static constexpr int QKS = BLK == 32 ? 4 : 2;
  static constexpr int H = UROWS / (BLK * WG);
  static constexpr int NU = QBK / 4 / NW;
  static_assert(H >= 1 && NU >= 1 && H * BLK * WG == UROWS && UROWS % 8 == 0, "wave grid does not divide the unit");
  const char* base;     // &mem[0][row0]
  int64_t total;        // bytes from base to the end of the matrix
  int64_t ktile_bytes;  // QBK * ld * 2
  uint32_t voff[2][NU];
  uint32_t moff[2][H];   // [k-tile buffer][block], the lane's k-row and element included

  __device__ __forceinline__ void init(const uint16_t* mem, int64_t ld, int row0, int K_, int lane, int wave, int wsub) {
    base = reinterpret_cast<const char*>(mem + row0);
    total = ((int64_t)K_ * ld - row0) * 2;
    ktile_bytes = (int64_t)QBK * ld * 2;
    const int ksub = lane >> 4;                        // k-row inside the instruction = k & 3
#pragma unroll
    for (int u = 0; u < 2; u++)
#pragma unroll
      for (int j = 0; j < NU; j++) {
        // a wave's NU instructions of a unit fill 4 NU consecutive k-rows (one setting of M0, see dma16_at)
        const int q = NU * wave + j;
        const int krow = 4 * q + ksub;
        // chunk of the unit's 128 rows this lane fetches; k >> 3 & 1 = q >> 1 & 1
        const int c = (lane & 15) ^ (ksub << 2) ^ (((q >> 1) & 1) << 1);
        // k-row 4 j lies at least 1024 j bytes in: rows are at least 256 bytes long (the host checks)
        voff[u][j] = (c * 8 < UROWS ? (uint32_t)(((int64_t)krow * ld + u * UROWS + c * 8) * 2) : 0x80000000u) - 1024u * j;
      }
    // lane (group G = l/16, i = l%16) addresses k-row kg + i/4 (+ (1024 / BLK) kk, +4 for the second read) and
    // elements eg + 4 (i%4) .. +3 of the block, with (kg, eg) = (8 (G/2), 16 (G%2)) for BLK = 32, (8 G, 0) for 16
    const int G = lane >> 4, i = lane & 15, kq = i >> 2;
    const int kg = BLK == 32 ? 8 * (G >> 1) : 8 * G, eg = BLK == 32 ? 16 * (G & 1) : 0;
    const uint32_t lane_base = (uint32_t)((kg + kq) * (LROWS_U * 2) + 8 * (i & 1));
#pragma unroll
    for (int b = 0; b < H; b++) {
      const int c2 = (wsub * BLK * H + BLK * b + eg) / 8 + ((i & 3) >> 1);
      moff[0][b] = lane_base + (uint32_t)((c2 ^ (kq << 2) ^ (((kg >> 3) & 1) << 1)) * 16);
      moff[1][b] = moff[0][b] + 65536;
    }
  }
  struct Prep {
    rsrc_t r;
  };
  __device__ __forceinline__ Prep prep(int kt, int kend) const {
    // the whole address goes through the range check: k-rows past K read as zero
    return Prep{make_rsrc(base + kt * ktile_bytes, kt >= kend ? 0 : total - kt * ktile_bytes)};
  }
  template <int UNIT_OFF, int U, int J>
  __device__ __forceinline__ void issue(const Prep& pp, uint32_t wave_lds) const {
    dma16_at<J == 0, UNIT_OFF, 1024 * J>(pp.r, wave_lds, voff[U][J], 0);
  }
  __device__ __forceinline__ bf16x8_t frag(const char* unit, int buf, int b, int kk) const {
    const char* a = unit + moff[buf][b] + kk * ((QBK / QKS) * LROWS_U * 2);
    const bf16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
        (bf16x4_t __attribute__((address_space(3)))*)(a));
    const bf16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
        (bf16x4_t __attribute__((address_space(3)))*)(a + 4 * LROWS_U * 2));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  }
};

template <int LAY, int NW, int WG, int BLK, int UR> struct QOperandOf { using type = RowOperandQ<NW, WG, BLK, UR>; };
template <int NW, int WG, int BLK, int UR> struct QOperandOf<LAY_COL, NW, WG, BLK, UR> { using type = ColOperandQ<NW, WG, BLK, UR>; };

// compile-time list of ints, read by index
template <int... V>
struct IntList {
  static constexpr int v[sizeof...(V)] = {V...};
};

// Stream-K scratch: two slots per stream workgroup; a slot holds one workgroup's accumulators of a tile whose k
// range it shares with others: 64 x 16 bytes per lane, lane-interleaved (vector v of thread t at byte
// (v * 256 + t) * 16), + the row sums of EPI_ROWSUM in vectors 64 and 65.  A workgroup's first slot takes the piece
// that begins its run of k-tiles, the second the piece that ends it.  gemm_sk_reduce_kernel adds the pieces of
// every shared tile up, in k order, and writes the tile.
constexpr int SK_MAX_WGS = 256;
constexpr int SK_SLOT_VECS = 66;                              // 16-byte vectors per lane and slot
constexpr int64_t SK_SLOT_BYTES = (int64_t)SK_SLOT_VECS * 256 * 16;
constexpr int64_t SK_WORKSPACE_BYTES = 2 * SK_MAX_WGS * SK_SLOT_BYTES;
static_assert(SK_WORKSPACE_BYTES == 2ll * 256 * 66 * 256 * 16, "linear.hip states the same size");
// slot of the piece of shared tile r (k-tiles [r KT, (r + 1) KT) of the stream) that workgroup w multiplied
__device__ __forceinline__ int64_t sk_slot_of(int w, int r, int KT, int ipw) {
  return (int64_t)(2 * w + (w * ipw < r * KT ? 1 : 0)) * SK_SLOT_BYTES;
}

// bid: this workgroup's index among the workgroups of the product p (blockIdx.x, or less where one launch holds
// two products); lds: the workgroup's Q_LDS_BYTES of LDS, 1 KiB aligned
//
// BM x BN: 256 x 256 (waves 2 x 2, or 2 x 4 with 8 waves), or a tile narrowed along one dimension to 192 or 160 for
// products whose 256 x 256 tiling fills the 256 compute units badly (8192 x 1280 is 160 tiles of 256 x 256 and 256
// of 256 x 160).  A narrow tile's four waves stand in one line along the wide dimension (4 x 1 for 256 x BN, 1 x 4
// for BM x 256): each wave owns 64 rows (columns) of the wide operand, 32 in either unit, and the narrow operand
// whole, whose units of BN / 2 = 80 or 96 rows are 5 or 6 blocks of 16.
constexpr int Q_LDS_BYTES = 2 * 65536;
//
// OFF (measurement builds only, results wrong): bit 0 = the main loop issues no DMA requests, bit 1 = it reads no
// fragments from LDS (the MFMAs keep multiplying the first k-tile's fragments): what the loop costs without either.
template <int ALAY, int BLAY, int EPI, int OUT, int NW, bool F16, int BLK, bool SK, int BM = 256, int BN = 256, int OFF = 0>
__device__ __forceinline__ void gemm_q_body(const GemmArgs& p, const int bid, char* lds) {
  using X = X16<F16>;
  constexpr bool NARROW = BM != 256 || BN != 256;
  static_assert(BM == 256 || BN == 256, "at most one dimension of the tile is narrowed");
  static_assert(!NARROW || (BLK == 16 && NW == 4 && !SK && EPI != MTP_EPI_SWIGLU),
                "narrow tiles: 4 waves, 16x16x32, whole tiles, no SwiGLU interleave");
  static_assert(!SK || (BLK == 16 && NW == 4), "stream-K is built for the 4-wave 16x16x32 form");
  static_assert(EPI != MTP_EPI_SWIGLU || BLAY == LAY_ROW, "the SwiGLU row interleave is a forward (row B) feature");
  static_assert(NW == 4 || NW == 8, "4 waves (2x2) or 8 waves (2x4) per workgroup");
  constexpr int WGM = BN != 256 ? 4 : BM != 256 ? 1 : 2, WGN = NW / WGM;
  constexpr int TI = BM / (BLK * WGM), TJ = BN / (BLK * WGN);   // MFMA blocks per wave in m and n
  using AOp = typename QOperandOf<ALAY, NW, WGM, BLK, BM / 2>::type;
  using BOp = typename QOperandOf<BLAY, NW, WGN, BLK, BN / 2>::type;
  constexpr int HI = AOp::H, HJ = BOp::H, QKS = AOp::QKS;
  static_assert(2 * HI == TI && 2 * HJ == TJ, "two units per operand");
  using AccT = std::conditional_t<BLK == 32, f32x16_t, f32x4_t>;
  constexpr int S = 32 / BLK;           // MFMA blocks per 32 rows (columns)
  constexpr int TI32 = TI / S, TJ32 = TJ / S;
  static_assert(TI32 * S == TI && TJ32 * S == TJ, "whole 32 x 32 blocks per wave");
  constexpr int QBUF = 65536;                     // one k-tile of both operands: at most 64 KiB, buffers 64 KiB apart
  static_assert(AOp::BYTES + BOp::BYTES <= QBUF, "the operands keep per-buffer read offsets 64 KiB apart");
  constexpr int LDS_BYTES = 2 * QBUF;
  static_assert(LDS_BYTES == Q_LDS_BYTES, "the kernels allocate Q_LDS_BYTES");

  const int tid = threadIdx.x;
  int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;

  const int tiles_m = (p.M + BM - 1) / BM;
  const int n_span = (EPI == MTP_EPI_SWIGLU) ? p.half : p.N;  // SwiGLU tiles cover BN/2 gate + BN/2 up columns
  constexpr int BN_SPAN = (EPI == MTP_EPI_SWIGLU) ? BN / 2 : BN;
  const int tiles_n = (n_span + BN_SPAN - 1) / BN_SPAN;
  const int KT = (p.K + QBK - 1) / QBK;
  // This workgroup's run of k-tiles in the sequence "all k-tiles of tile position 0, of position 1, ...": one whole
  // tile, or (stream-K) sk_ipw k-tiles that may end one tile and begin the next.
  int it = bid * KT, it_end = it + KT;
  [[maybe_unused]] int sk_w = -1;
  if constexpr (SK) {
    if (bid >= p.sk_full) {
      sk_w = bid - p.sk_full;
      it = p.sk_full * KT + sk_w * p.sk_ipw;
      const int all = tiles_m * tiles_n * KT;
      it_end = it + p.sk_ipw < all ? it + p.sk_ipw : all;
    }
  }
  // where this wave's DMA instructions of a unit of A (of B) put their first KiB
  const uint32_t lds_base = __builtin_amdgcn_readfirstlane(lds_addr_of(lds));
  const uint32_t lds_wave_a = lds_base + wave * (AOp::NU * 1024);
  const uint32_t lds_wave_b = AOp::NU == BOp::NU ? lds_wave_a : lds_base + wave * (BOp::NU * 1024);
  // byte offsets of the units inside lds
  auto unit_a = [](int buf, int u) constexpr { return buf * QBUF + u * AOp::UBYTES; };
  auto unit_b = [](int buf, int u) constexpr { return buf * QBUF + AOp::BYTES + u * BOp::UBYTES; };

 do {
  // One piece (for all but stream-K workgroups the only one).  Everything a lane derives from its number is
  // derived again per piece: hoisted out of this loop it would stay live through the main loop, where every
  // register is taken, and come back from scratch memory on the critical path of the next piece's first requests.
  if constexpr (SK) asm volatile("" : "+v"(lane));
  const int pos = it / KT;                         // tile position
  const int k0 = it - pos * KT;                    // first k-tile of this piece
  const int k1 = it_end - pos * KT < KT ? it_end - pos * KT : KT;   // one past its last
  it += k1 - k0;
  int tm, tn;
  tile_of(pos, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM;
  const int n0 = tn * BN_SPAN;
  const int lm0 = MTP_DBG(p, 1) ? 0 : MTP_DBG(p, 8) ? (tm & 1) * BM : m0;
  const int ln0 = MTP_DBG(p, 9) ? 0 : n0;

  AOp opA;
  BOp opB;
  if constexpr (ALAY == LAY_ROW)
    opA.init(p.A, p.lda, lm0, p.M, p.K, lane, wave, wm, [](int r) -> int64_t { return r; });
  else
    opA.init(p.A, p.lda, lm0, p.K, lane, wave, wm);
  if constexpr (BLAY == LAY_ROW) {
    // SwiGLU: unit 0 of the B tile holds BN/2 gate rows, unit 1 the matching up rows
    opB.init(p.B, p.ldb, ln0, p.N, p.K, lane, wave, wn, [&](int r) -> int64_t {
      if (EPI == MTP_EPI_SWIGLU) {
        if (r < BN / 2) return ln0 + r >= p.half ? -1 : r;   // gate rows at or past `half` belong to the up matrix
        return (int64_t)p.half + (r - BN / 2);
      }
      return r;
    });
  } else {
    opB.init(p.B, p.ldb, ln0, p.K, lane, wave, wn);
  }
#ifdef MTP_MEASURE
  if (MTP_DBG(p, 4)) {  // measurement: every DMA reads out of range (zero fill, no memory traffic)
#pragma unroll
    for (int u = 0; u < 2; u++) {
#pragma unroll
      for (int j = 0; j < AOp::NU; j++) opA.voff[u][j] = 0x80000000u;
#pragma unroll
      for (int j = 0; j < BOp::NU; j++) opB.voff[u][j] = 0x80000000u;
    }
  }
#endif

  AccT acc[TI][TJ];
#pragma unroll
  for (int i = 0; i < TI; i++)
#pragma unroll
    for (int j = 0; j < TJ; j++)
#pragma unroll
      for (int r = 0; r < (BLK == 32 ? 16 : 4); r++) acc[i][j][r] = 0.f;
  float rsum[TI];
#pragma unroll
  for (int i = 0; i < TI; i++) rsum[i] = 0.f;

  // register sets: fragments of A unit u / B unit u of the current (or next) k-tile
  bf16x8_t ra[2][HI][QKS], rb[2][HJ][QKS];

  constexpr int PH = HI * HJ * QKS;          // MFMAs per phase (one quadrant)
  constexpr int HT = 2 * PH;                 // MFMAs per half tile
  constexpr int NDH = AOp::NU + BOp::NU;     // DMA instructions per wave and half tile (one unit of A, one of B)
  constexpr int BPOST = (BLK == 32 ? 1 : 2) * (HI * HJ >= 4 ? 4 : 2);   // MFMAs of a half tile issued behind its barrier
  constexpr int BARRIER_AT = HT - BPOST;
  // the d-th DMA instruction of a half tile is issued behind MFMA number dma_at(d) of the half tile
  auto dma_at = [](int d) constexpr { return d * HT / NDH + 1; };
  constexpr int NAFTER = [&]() constexpr {   // DMA instructions of a half tile issued behind its barrier
    int n = 0;
    for (int d = 0; d < NDH; d++) n += (d * HT / NDH + 1) >= BARRIER_AT ? 1 : 0;
    return n;
  }();
  // At a barrier the two units the next half tile reads must have landed: they were requested three half tiles
  // ago, and behind them came one whole half tile of requests and this half tile's up to the barrier.
  constexpr int VM_AT_BARRIER = 2 * NDH - NAFTER;
  static_assert(VM_AT_BARRIER < 64, "vmcnt range");

  // m-th MFMA of a phase on the register sets (MA, MB): k16 step m / (HI HJ), blocks walked in a snake
  auto mfma_q = [&](auto ma_tag, auto mb_tag, auto m_tag) {
    constexpr int MA = decltype(ma_tag)::value, MB = decltype(mb_tag)::value, m = decltype(m_tag)::value;
    constexpr int kk = m / (HI * HJ), w = m % (HI * HJ);
    constexpr int i = w / HJ, j = (i & 1) ? HJ - 1 - w % HJ : w % HJ;
    constexpr int bi = MA * HI + i, bj = MB * HJ + j;   // MFMA block of the wave's part
    if constexpr (BLK == 32) {
      acc[bi][bj] = X::mfma32(rb[MB][j][kk], ra[MA][i][kk], acc[bi][bj]);
    } else {
      // Inline assembly with the accumulator tied in place: left to itself the register allocator moves the 64
      // four-register accumulators about (hundreds of v_accvgpr copies per k-tile, and spills).  The statement
      // hides the instruction from the compiler's hazard checks; what they would cover holds by construction:
      // an accumulator is touched again 16 MFMAs later at the earliest, the operand registers are written by LDS
      // reads only (s_waitcnt lgkmcnt, which the compiler does insert for the statement's inputs), and the
      // first read of an accumulator by another instruction sits behind the wait states after the loop.
      if constexpr (F16)
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[bi][bj]) : "v"(rb[MB][j][kk]), "v"(ra[MA][i][kk]));
      else
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[bi][bj]) : "v"(rb[MB][j][kk]), "v"(ra[MA][i][kk]));
    }
    if constexpr (EPI == EPI_ROWSUM && MB == 0 && j == 0) rsum[MA * HI + i] = X::sum8(ra[MA][i][kk], rsum[MA * HI + i]);
  };
  // f-th fragment read of a phase that refills register set U of A (IS_A) or B from buffer BUF; fragments in the
  // order they are used: step 0 of every block, step 1, ...
  auto read_q = [&](auto isa_tag, auto u_tag, auto buf_tag, auto f_tag) {
    constexpr bool IS_A = decltype(isa_tag)::value != 0;
    constexpr int U = decltype(u_tag)::value, BUF = decltype(buf_tag)::value, f = decltype(f_tag)::value;
    if constexpr (IS_A) {
      constexpr int kk = f / HI, b = f % HI;
      ra[U][b][kk] = opA.frag(lds + unit_a(0, U), BUF, b, kk);
    } else {
      constexpr int kk = f / HJ, b = f % HJ;
      rb[U][b][kk] = opB.frag(lds + unit_b(0, U), BUF, b, kk);
    }
  };
  // d-th DMA instruction of the group (A unit UA, B unit UB, buffer BUF): A's, then B's (each run shares M0)
  auto dma_q = [&](const typename AOp::Prep& pa, const typename BOp::Prep& pb, auto ua_tag, auto ub_tag, auto buf_tag,
                   auto d_tag) {
    constexpr int UA = decltype(ua_tag)::value, UB = decltype(ub_tag)::value, BUF = decltype(buf_tag)::value;
    constexpr int d = decltype(d_tag)::value;
    if constexpr (d < AOp::NU)
      opA.template issue<unit_a(BUF, UA), UA, d>(pa, lds_wave_a);
    else
      opB.template issue<unit_b(BUF, UB), UB, d - AOp::NU>(pb, lds_wave_b);
  };
  auto dma_group = [&](int kt, auto ua_tag, auto ub_tag, auto buf_tag) {
    const auto pa = opA.prep(kt, k1);
    const auto pb = opB.prep(kt, k1);
    static_for<NDH>([&](auto d) { dma_q(pa, pb, ua_tag, ub_tag, buf_tag, d); });
  };

  // One half tile.  D = IntList<MA0, MB0, MA1, MB1,  R0A, R0U, R0BUF,  R1A, R1U, R1BUF,  DUA, DUB, DBUF>:
  // phase 0 multiplies register sets (MA0, MB0) while set R0U of A (R0A = 1) or B is refilled from buffer R0BUF,
  // phase 1 likewise; the DMA group (A unit DUA, B unit DUB) of k-tile kt_dma goes to buffer DBUF.
  // The fragment reads of a phase sit behind its first MFMAs, so that every read of the half tile has been
  // issued well before the barrier (which hands the units over) and has about half a phase to land.
  auto half_tile = [&](int kt_dma, auto desc) {
    using D = decltype(desc);
    const auto pa = opA.prep(kt_dma, k1);
    const auto pb = opB.prep(kt_dma, k1);
    __builtin_amdgcn_sched_barrier(0);
    static_for<HT>([&](auto g_tag) {
      constexpr int g = decltype(g_tag)::value;
      constexpr int ph = g / PH, m = g % PH;
      constexpr int MA = D::v[ph ? 2 : 0], MB = D::v[ph ? 3 : 1];
      constexpr int RA = D::v[ph ? 7 : 4], RU = D::v[ph ? 8 : 5], RBUF = D::v[ph ? 9 : 6];
      constexpr int NR = (RA ? HI : HJ) * QKS;     // fragment reads of this phase
      constexpr int RSPAN = PH / 2;                // spread over the first half of the phase
      if constexpr (g == BARRIER_AT) {
        // own reads of this half tile done, own requests for the next half tile's units landed ...
#if defined(MTP_MEASURE) && defined(QX_NOVMWAIT)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // timing only: results are wrong
#else
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(VM_AT_BARRIER) : "memory");
#endif
#if !(defined(MTP_MEASURE) && defined(QX_NOBARRIER))
        __syncthreads();  // ... for every wave
#endif
        __builtin_amdgcn_sched_barrier(0);
      }
      mfma_q(std::integral_constant<int, MA>{}, std::integral_constant<int, MB>{}, std::integral_constant<int, m>{});
      if constexpr (!(OFF & 1))
        static_for<NDH>([&](auto d_tag) {
          constexpr int d = decltype(d_tag)::value;
          if constexpr (d * HT / NDH + 1 == g + 1)
            dma_q(pa, pb, std::integral_constant<int, D::v[10]>{}, std::integral_constant<int, D::v[11]>{},
                  std::integral_constant<int, D::v[12]>{}, d_tag);
        });
      if constexpr (!(OFF & 2) && m < RSPAN) {
        static_for<(m + 1) * NR / RSPAN - m * NR / RSPAN>([&](auto e) {
          read_q(std::integral_constant<int, RA>{}, std::integral_constant<int, RU>{},
                 std::integral_constant<int, RBUF>{}, std::integral_constant<int, m * NR / RSPAN + decltype(e)::value>{});
        });
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  //                       MA0 MB0 MA1 MB1   R0: A  U BUF   R1: A  U BUF   DMA: UA UB BUF
  using EvenH0 = IntList<0, 0, 0, 1, /**/ 0, 1, 0, /**/ 1, 1, 0, /**/ 0, 0, 0>;  // Q00 Q01; reads B1[t] A1[t]
  using EvenH1 = IntList<1, 1, 1, 0, /**/ 1, 0, 1, /**/ 0, 1, 1, /**/ 1, 1, 0>;  // Q11 Q10; reads A0[t+1] B1[t+1]
  using OddH0 = IntList<0, 1, 0, 0, /**/ 0, 0, 1, /**/ 1, 1, 1, /**/ 0, 1, 1>;   // Q01 Q00; reads B0[t] A1[t]
  using OddH1 = IntList<1, 0, 1, 1, /**/ 1, 0, 0, /**/ 0, 0, 0, /**/ 1, 0, 1>;   // Q10 Q11; reads A0[t+1] B0[t+1]

  {
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    // the four request groups in front of the loop, in the order the loop would have issued them
    dma_group(k0, I0{}, I0{}, I0{});       // A0[0] B0[0]
    dma_group(k0, I1{}, I1{}, I0{});       // A1[0] B1[0]
    dma_group(k0 + 1, I0{}, I1{}, I1{});   // A0[1] B1[1]
    dma_group(k0 + 1, I1{}, I0{}, I1{});   // A1[1] B0[1]
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NDH) : "memory");   // all of the first k-tile
    __syncthreads();
    static_for<HI * QKS>([&](auto f) { read_q(I1{}, I0{}, I0{}, f); });
    static_for<HJ * QKS>([&](auto f) { read_q(I0{}, I0{}, I0{}, f); });
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __syncthreads();   // everyone holds A0[0], B0[0]: the loop's first requests may overwrite them
  }
  int kt = k0;
  for (; kt + 1 < k1; kt += 2) {
    half_tile(kt + 2, EvenH0{});
    half_tile(kt + 2, EvenH1{});
    half_tile(kt + 3, OddH0{});
    half_tile(kt + 3, OddH1{});
  }
  if (kt < k1) {
    half_tile(kt + 2, EvenH0{});
    half_tile(kt + 2, EvenH1{});
  }
  __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
  // the last MFMAs' results must have reached the registers before anything else reads them (see mfma_q)
  if constexpr (BLK == 16) asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  __syncthreads();  // the epilogue reuses the tile buffers
  if (MTP_DBG(p, 2)) return;

  auto write_tile = [&]() {
    gemm_epilogue<BM, BN, EPI, OUT, WGM, WGN, F16, true, LDS_BYTES, TI32, TJ32, BLK>(
        p,
        [&](int i, int j, int g, int e) -> float {
          if constexpr (BLK == 32) return acc[i][j][4 * g + e];
          else return acc[2 * i + (g >> 1)][2 * j + (g & 1)][e];
        },
        [&](int i, int g) -> float { return BLK == 32 ? rsum[i] : rsum[2 * i + (g >> 1)]; }, lds, m0, n0, tn, wave, lane);
  };
  if constexpr (!SK) {
    write_tile();
  } else {
    if (k0 == 0 && k1 == KT) {
      write_tile();
    } else {
      // part of a tile whose k range is shared: the accumulators go to this workgroup's slot as they are
      char* q = static_cast<char*>(p.ws) + sk_slot_of(sk_w, pos - p.sk_full, KT, p.sk_ipw) + tid * 16;
      constexpr int NT = NW * 64;
#pragma unroll
      for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < TJ; j++) *reinterpret_cast<f32x4_t*>(q + (i * TJ + j) * (NT * 16)) = acc[i][j];
      if constexpr (EPI == EPI_ROWSUM) {
        *reinterpret_cast<f32x4_t*>(q + 64 * (NT * 16)) = f32x4_t{rsum[0], rsum[1], rsum[2], rsum[3]};
        *reinterpret_cast<f32x4_t*>(q + 65 * (NT * 16)) = f32x4_t{rsum[4], rsum[5], rsum[6], rsum[7]};
      }
    }
  }
  if (SK && it < it_end) __syncthreads();   // the next piece's requests overwrite what the epilogue staged in LDS
 } while (SK && it < it_end);
}

// The body lives in a __device__ function: it uses inline assembly operands that the host pass over a
// __global__ function would trip on.
template <int BM, int BN, int ALAY, int BLAY, int EPI, int OUT, int NW, bool F16>
__device__ __forceinline__ void gemm_bf16_body(const GemmArgs& p) {
  using X = X16<F16>;   // element type of A, B, bias and the 16-bit outputs: bf16 or IEEE half
  static_assert(EPI != MTP_EPI_SWIGLU || BLAY == LAY_ROW, "the SwiGLU row interleave is a forward (row B) feature");
  static_assert(NW == 4 || NW == 8, "4 waves (2x2) or 8 waves (2x4) per workgroup");
  constexpr int WGM = 2, WGN = NW / 2;                         // wave grid over the tile
  constexpr int TI = BM / (32 * WGM), TJ = BN / (32 * WGN);    // 32x32 blocks per wave in m and n
  static_assert(EPI != MTP_EPI_SWIGLU || TJ % 2 == 0, "SwiGLU pairs gate and up blocks inside a wave");
  using AOp = typename OperandOf<ALAY, BM, NW>::type;
  using BOp = typename OperandOf<BLAY, BN, NW>::type;
  constexpr int STAGE_BYTES = AOp::BYTES + BOp::BYTES;
  static_assert(NSTAGE * STAGE_BYTES <= 128 * 1024, "LDS ring too large");
  // Stages sit STAGE_SKEW bytes further apart than their size.  A register-staged write instruction puts the two
  // 64-byte halves of a row into neighbouring stages; with the stages a multiple of 256 bytes apart the two
  // halves fall on the same banks (two-way conflict on every write), 64 bytes of skew puts them side by side.
  constexpr int STAGE_SKEW = (MTP_GEMM_VSTAGE && MTP_STAGE_SKEW && ALAY == LAY_ROW && BLAY == LAY_ROW) ? 64 : 0;
  constexpr int STAGE_STRIDE = STAGE_BYTES + STAGE_SKEW;
  __shared__ __attribute__((aligned(1024))) char lds[NSTAGE * STAGE_STRIDE];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;
  const int lh = lane >> 5, l32 = lane & 31;

  const int tiles_m = (p.M + BM - 1) / BM;
  const int n_span = (EPI == MTP_EPI_SWIGLU) ? p.half : p.N;  // SwiGLU tiles cover BN/2 gate + BN/2 up columns
  constexpr int BN_SPAN = (EPI == MTP_EPI_SWIGLU) ? BN / 2 : BN;
  const int tiles_n = (n_span + BN_SPAN - 1) / BN_SPAN;
  int tm, tn;
  tile_of(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM;
  const int n0 = tn * BN_SPAN;
  // load origins (debug 1: all tiles load tile (0,0); debug 8: two A tiles, one B tile: a cache-resident set)
  const int lm0 = MTP_DBG(p, 1) ? 0 : MTP_DBG(p, 8) ? (tm & 1) * BM : m0;
  const int ln0 = MTP_DBG(p, 9) ? 0 : n0;

  AOp opA;
  BOp opB;
  if constexpr (ALAY == LAY_ROW)
    opA.init(p.A, p.lda, lm0, p.M, p.K, lane, wave, wm * (BM / WGM), [](int r) -> int64_t { return r; });
  else
    opA.init(p.A, p.lda, lm0, p.K, lane, wave, wm * (BM / WGM));
  if constexpr (BLAY == LAY_ROW) {
    // LDS row r of the B tile maps to a global row of [N,K].  Plain: n0 + r.  SwiGLU: the wave-column wn
    // owns LDS rows [wn*BN/WGN, (wn+1)*BN/WGN): first half gate rows, second half the matching up rows.
    opB.init(p.B, p.ldb, ln0, p.N, p.K, lane, wave, wn * (BN / WGN), [&](int r) -> int64_t {
      if (EPI == MTP_EPI_SWIGLU) {
        constexpr int SEG = BN / (2 * WGN);
        const int seg = r / SEG, in = r % SEG;
        const int64_t gr = ((seg & 1) ? p.half : 0) + (seg >> 1) * SEG + in;
        // gate rows at or past `half` belong to the up matrix: no such row
        return (!(seg & 1) && ln0 + gr >= p.half) ? -1 : gr;
      }
      return r;
    });
  } else {
    opB.init(p.B, p.ldb, ln0, p.K, lane, wave, wn * (BN / WGN));
  }
  if (MTP_DBG(p, 4)) {  // measurement: every DMA reads out of range (zero fill, no memory traffic)
#pragma unroll
    for (int j = 0; j < AOp::NINSTR; j++) opA.voff[j] = 0x80000000u;
#pragma unroll
    for (int j = 0; j < BOp::NINSTR; j++) opB.voff[j] = 0x80000000u;
    if constexpr (ALAY == LAY_ROW && BLAY == LAY_ROW) {
#pragma unroll
      for (int j = 0; j < AOp::NPAIR; j++) opA.pvoff[j] = 0x80000000u;
#pragma unroll
      for (int j = 0; j < BOp::NPAIR; j++) opB.pvoff[j] = 0x80000000u;
    }
  }

  constexpr int NDMA = AOp::NINSTR + BOp::NINSTR;  // DMA instructions per wave per k-tile
  const uint32_t lds0 = __builtin_amdgcn_readfirstlane(lds_addr_of(lds));
  // d-th DMA instruction of a k-tile whose per-tile state (pa, pb) has been prepared; A and B alternate
  auto issue_one = [&](const typename AOp::Prep& pa, const typename BOp::Prep& pb, int stage, int d) {
    const uint32_t la = lds0 + stage * STAGE_STRIDE;
    // A and B alternate while both have instructions left
    constexpr int NMIN = AOp::NINSTR < BOp::NINSTR ? AOp::NINSTR : BOp::NINSTR;
    if (d < 2 * NMIN) {
      if ((d & 1) == 0)
        opA.issue(pa, la, wave, d >> 1);
      else
        opB.issue(pb, la + AOp::BYTES, wave, d >> 1);
    } else if (AOp::NINSTR > BOp::NINSTR) {
      opA.issue(pa, la, wave, d - NMIN);
    } else {
      opB.issue(pb, la + AOp::BYTES, wave, d - NMIN);
    }
  };
  auto issue_loads = [&](int kt) {  // all of k-tile kt, tail masking on
    const auto pa = opA.template prep<false>(kt);
    const auto pb = opB.template prep<false>(kt);
#pragma unroll
    for (int d = 0; d < NDMA; d++) issue_one(pa, pb, kt % NSTAGE, d);
  };

  f32x16_t acc[TI][TJ];
#pragma unroll
  for (int i = 0; i < TI; i++)
#pragma unroll
    for (int j = 0; j < TJ; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  // ---- main loop ---------------------------------------------------------------
  const int KT = (p.K + BK - 1) / BK;
  bf16x8_t af[2][TI], bfr[2][TJ];
  // Fragments are read in the order A0 B0 A1 B1 ... and the MFMAs walk the block grid in growing squares
  // ((0,0); (1,0) (1,1) (0,1); ...), so the first MFMAs of a step depend only on the oldest reads.
  constexpr int NFR = TI + TJ;   // fragments per k16 step
  constexpr int NMF = TI * TJ;   // MFMAs per k16 step
  auto read_one = [&](int stage, int kk, int slot, auto u_tag) {  // u-th fragment in A0 B0 A1 B1 ... order
    constexpr int u = decltype(u_tag)::value;
    const char* la = lds + stage * STAGE_STRIDE;
    // with TI == TJ the order alternates; otherwise the longer side's leftovers come last
    constexpr int d = u < 2 * (TI < TJ ? TI : TJ) ? u / 2 : u - (TI < TJ ? TI : TJ);
    constexpr bool is_a = u < 2 * (TI < TJ ? TI : TJ) ? (u % 2 == 0) : (TI > TJ);
    if constexpr (is_a)
      af[slot][d] = opA.frag(la, kk, d);
    else
      bfr[slot][d] = opB.frag(la + AOp::BYTES, kk, d);
  };
  auto read_frags = [&](int stage, int kk, int slot) {
    static_for<NFR>([&](auto u) { read_one(stage, kk, slot, u); });
  };
  float rsum[TI];
#pragma unroll
  for (int i = 0; i < TI; i++) rsum[i] = 0.f;
  auto mfma_one = [&](int slot, auto t_tag) {  // t-th MFMA of a step in shell order
    constexpr int t = decltype(t_tag)::value;
    constexpr int i = shell_pair(t, TI, TJ).i, j = shell_pair(t, TI, TJ).j;
    acc[i][j] = X::mfma32(bfr[slot][j], af[slot][i], acc[i][j]);
    if constexpr (EPI == EPI_ROWSUM && t < TI) {
      // the t-th A fragment of this step: 8 k of one row per lane
      rsum[t] = X::sum8(af[slot][t], rsum[t]);
    }
  };
  auto mfmas = [&](int slot) {
    static_for<NMF>([&](auto t) { mfma_one(slot, t); });
  };

  // One k-tile = KSTEPS k16 steps.  Step s multiplies the fragments in register slot s%2 while the
  // fragments of the following step (the first step of tile kt+1 for the last one) are read into the
  // other slot, and while the DMA instructions of tile kt+NSTAGE-1 — whose stage was released by the
  // barrier that ended tile kt-1 — are issued one every few MFMAs.
  //
  // In the last step the first PRE MFMAs are issued before the barrier: they use the step's oldest
  // fragments and give its youngest LDS reads time to land, so the lgkmcnt(0) the barrier needs is free.
  // The s_waitcnt vmcnt in front of the barrier only asks for tile kt+1; the tiles requested after it
  // may still be in flight.
  //
  // FULL: tiles up to kt+NSTAGE-1 lie completely below K.  The instruction order of the whole tile is
  // pinned with scheduling barriers (the DMA is inline assembly, which sched_group_barrier cannot place).
  constexpr int TILE_MF = KSTEPS * NMF;       // MFMAs per k-tile
  constexpr int PRE = NMF * 3 / 8, REST = NMF - PRE;
  // MFMA index (0 .. TILE_MF-1) after which the d-th DMA instruction is issued
  auto dma_slot = [](int d) constexpr { return d * TILE_MF / NDMA + 1; };
  // VSTAGE (row operands on both sides: the forward product).  A k-tile of a row operand is 64 bytes per row,
  // half a cache line; fetched one k-tile at a time every line is requested twice from the L2.  Here the k-tiles
  // travel in pairs: one load instruction covers 8 rows x 128 bytes (both k-tiles of the pair), lands in
  // registers and is written to the two LDS stages two k-tiles later — the prefetch distance of the DMA ring,
  // with whole lines per request and one barrier per pair of k-tiles.  During the even tile kt of a pair the
  // registers (pair kt+2, kt+3) are written to the stages the barrier behind tile kt-1 released and are
  // refilled with pair kt+4, kt+5, one instruction of each kind every second MFMA.
  constexpr bool VSTAGE = MTP_GEMM_VSTAGE && ALAY == LAY_ROW && BLAY == LAY_ROW && NSTAGE == 4 && KSTEPS == 2;
  constexpr int NPA = VSTAGE ? AOp::NPAIR : 0, NPB = VSTAGE ? BOp::NPAIR : 0, NPL = NPA + NPB;
  u32x4_t st[NPL > 0 ? NPL : 1];
  [[maybe_unused]] uint32_t wlane_a = 0, wlane_b = 0;
  if constexpr (VSTAGE) {
    wlane_a = opA.pwoff + (opA.pair_odd(lane) ? STAGE_STRIDE : 0);
    wlane_b = opB.pwoff + (opB.pair_odd(lane) ? STAGE_STRIDE : 0);
  }
  // q-th paired instruction of a pair: A and B alternate while both have instructions left
  auto pair_sel = [](int q, int na, int nb, bool& is_a, int& jj) constexpr {
    const int nmin = na < nb ? na : nb;
    if (q < 2 * nmin) {
      is_a = (q & 1) == 0;
      jj = q >> 1;
    } else {
      is_a = na > nb;
      jj = q - nmin;
    }
  };
  auto pair_load = [&](int kt_even, auto q_tag) {
    if constexpr (VSTAGE) {
      constexpr int q = decltype(q_tag)::value;
      bool is_a = true;
      int jj = 0;
      pair_sel(q, NPA, NPB, is_a, jj);
      const uint32_t soff = (uint32_t)(kt_even * BK * 2);
      st[q] = is_a ? load16_to_vgpr(opA.rsrc, opA.pvoff[jj], soff) : load16_to_vgpr(opB.rsrc, opB.pvoff[jj], soff);
    }
  };
  auto pair_write = [&](int kt_even, auto q_tag, auto pending_tag) {
    if constexpr (VSTAGE) {
      constexpr int q = decltype(q_tag)::value;
      constexpr int PENDING = decltype(pending_tag)::value;
      constexpr bool is_a = q < 2 * (NPA < NPB ? NPA : NPB) ? (q & 1) == 0 : (NPA > NPB);
      constexpr int jj = q < 2 * (NPA < NPB ? NPA : NPB) ? (q >> 1) : q - (NPA < NPB ? NPA : NPB);
      const uint32_t base = lds0 + (uint32_t)((kt_even % NSTAGE) * STAGE_STRIDE) + (is_a ? 0u : (uint32_t)AOp::BYTES);
      wait_and_write16<PENDING, jj * NW * 8 * 64>(base + (is_a ? wlane_a : wlane_b), st[q]);
    }
  };
  auto ktile_v = [&](int kt, auto odd_tag, auto loads_tag) {
    constexpr bool ODD = decltype(odd_tag)::value, LOADS = decltype(loads_tag)::value;
    const int stage = kt % NSTAGE, nxt = (kt + 1) % NSTAGE;
    __builtin_amdgcn_sched_barrier(0);
    static_for<KSTEPS>([&](auto s_tag) {
      constexpr int s = decltype(s_tag)::value;
      constexpr bool last = s == KSTEPS - 1;
      static_for<NMF>([&](auto t_tag) {
        constexpr int t = decltype(t_tag)::value;
        constexpr int g = s * NMF + t;  // MFMA index inside the tile
        if constexpr (ODD && last && t == PRE) {
          // one barrier per pair: every wave's writes of the pair behind this one are in LDS, and everyone is
          // done reading the two stages the next even tile writes to
          asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
          __syncthreads();
          __builtin_amdgcn_sched_barrier(0);
        }
        mfma_one(s & 1, t_tag);
        {
          // the pair's instructions are spread over the MFMAs of both tiles up to the barrier
          constexpr int SPAN = MTP_VSTAGE_SPREAD ? TILE_MF + (KSTEPS - 1) * NMF + PRE - 2 : TILE_MF;
          constexpr int gp = (ODD ? TILE_MF : 0) + g;   // MFMA index inside the pair
          const int kb = ODD ? kt - 1 : kt;             // the pair's even tile
          static_for<(NPL > 0 ? NPL : 1)>([&](auto q_tag) {
            constexpr int q = decltype(q_tag)::value;
            if constexpr (NPL > 0 && q * SPAN / (NPL > 0 ? NPL : 1) + 1 == gp + 1) {
              pair_write(kb + 2, q_tag, std::integral_constant<int, LOADS ? NPL - 1 : NPL - 1 - q>{});
              if constexpr (LOADS) pair_load(kb + 4, q_tag);
            }
          });
        }
        if constexpr (!last) {
          static_for<(t + 1) * NFR / NMF - t * NFR / NMF>([&](auto e) {
            read_one(stage, s + 1, (s + 1) & 1, std::integral_constant<int, t * NFR / NMF + decltype(e)::value>{});
          });
        } else if constexpr (t >= PRE) {
          constexpr int r = t - PRE;
          static_for<(r + 1) * NFR / REST - r * NFR / REST>([&](auto e) {
            read_one(nxt, 0, (s + 1) & 1, std::integral_constant<int, r * NFR / REST + decltype(e)::value>{});
          });
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };
  constexpr int AHEAD = VSTAGE ? 2 : NSTAGE - 1;   // the DMA tiles (tail, short k) request tile kt + AHEAD
  auto ktile = [&](int kt, auto full_tag) {
    constexpr bool FULL = decltype(full_tag)::value;
    const int stage = kt % NSTAGE, nxt = (kt + 1) % NSTAGE;
    if constexpr (FULL) {
      const auto pa = opA.template prep<true>(kt + NSTAGE - 1);
      const auto pb = opB.template prep<true>(kt + NSTAGE - 1);
      const int dst = (kt + NSTAGE - 1) % NSTAGE;
      constexpr int dma_before_barrier = [&]() constexpr {
        int n = 0;
        for (int d = 0; d < NDMA; d++) n += (d * TILE_MF / NDMA + 1) < (KSTEPS - 1) * NMF + PRE ? 1 : 0;
        return n;
      }();
      __builtin_amdgcn_sched_barrier(0);
      static_for<KSTEPS>([&](auto s_tag) {
        constexpr int s = decltype(s_tag)::value;
        constexpr bool last = s == KSTEPS - 1;
        static_for<NMF>([&](auto t_tag) {
          constexpr int t = decltype(t_tag)::value;
          constexpr int g = s * NMF + t;  // MFMA index inside the tile
          if constexpr (last && t == PRE) {
            // tile kt+1 has landed (later tiles may still be in flight) ...
            __builtin_amdgcn_s_waitcnt(vmcnt_imm((NSTAGE - 3) * NDMA + dma_before_barrier));
            __syncthreads();  // ... for every wave, and everyone is done reading this stage
            __builtin_amdgcn_sched_barrier(0);
          }
          mfma_one(s & 1, t_tag);
          static_for<NDMA>([&](auto d_tag) {
            constexpr int d = decltype(d_tag)::value;
            if constexpr (d * TILE_MF / NDMA + 1 == g + 1) issue_one(pa, pb, dst, d);
          });
          if constexpr (!last) {
            // fragments of step s+1, spread over this step's MFMAs
            static_for<(t + 1) * NFR / NMF - t * NFR / NMF>([&](auto e) {
              read_one(stage, s + 1, (s + 1) & 1, std::integral_constant<int, t * NFR / NMF + decltype(e)::value>{});
            });
          } else if constexpr (t >= PRE) {
            // fragments of the first step of tile kt+1, spread over the MFMAs after the barrier
            constexpr int r = t - PRE;
            static_for<(r + 1) * NFR / REST - r * NFR / REST>([&](auto e) {
              read_one(nxt, 0, (s + 1) & 1, std::integral_constant<int, r * NFR / REST + decltype(e)::value>{});
            });
          }
          __builtin_amdgcn_sched_barrier(0);
        });
      });
    } else {
      if (kt + AHEAD < KT) issue_loads(kt + AHEAD);
      static_for<KSTEPS - 1>([&](auto s_tag) {
        constexpr int s = decltype(s_tag)::value;
        read_frags(stage, s + 1, (s + 1) & 1);
        mfmas(s & 1);
      });
      // wait for everything but (at most) the tile just requested
      if (kt + AHEAD < KT)
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(NSTAGE >= 3 ? NDMA : 0));
      else
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
      __syncthreads();
      if (kt + 1 < KT) read_frags(nxt, 0, KSTEPS & 1);
      mfmas((KSTEPS - 1) & 1);
    }
  };
  static_assert(KSTEPS % 2 == 0, "slot parity assumes an even number of k16 steps per tile");

  int kt = 0;
  const int KT_inside = p.K / BK;  // k-tiles that lie completely below K
  bool staged = false;
  if constexpr (VSTAGE) {
    if (KT_inside >= 6) {
      staged = true;
      // pair (0, 1) through the registers into stages 0 and 1, pair (2, 3) requested
      static_for<NPL>([&](auto q) { pair_load(0, q); });
      static_for<NPL>([&](auto q) { pair_write(0, q, std::integral_constant<int, NPL - 1 - decltype(q)::value>{}); });
      static_for<NPL>([&](auto q) { pair_load(2, q); });
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __syncthreads();
      read_frags(0, 0, 0);
      for (; kt + 5 < KT_inside; kt += 2) {
        ktile_v(kt, std::false_type{}, std::true_type{});
        ktile_v(kt + 1, std::true_type{}, std::true_type{});
      }
      // the pair still in registers goes to LDS, nothing new is requested; the DMA tiles take over behind it
      ktile_v(kt, std::false_type{}, std::false_type{});
      ktile_v(kt + 1, std::true_type{}, std::false_type{});
      kt += 2;
    }
  }
  if (!staged) {
#pragma unroll
    for (int t = 0; t < AHEAD; t++)
      if (t < KT) issue_loads(t);
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();
    read_frags(0, 0, 0);
    if constexpr (!VSTAGE)
      for (; kt + NSTAGE - 1 < KT_inside; kt++) ktile(kt, std::true_type{});
  }
  for (; kt < KT; kt++) ktile(kt, std::false_type{});
  __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
  __syncthreads();  // the epilogue reuses the tile buffers
  if (MTP_DBG(p, 2)) return;

  if constexpr (EPI == EPI_ROWSUM) static_assert(NMF >= TI, "every A fragment of a step must meet an MFMA");
  gemm_epilogue<BM, BN, EPI, OUT, WGM, WGN, F16, false, NSTAGE * STAGE_BYTES, TI, TJ, 32>(
      p, [&](int i, int j, int g, int e) -> float { return acc[i][j][4 * g + e]; },
      [&](int i, int) -> float { return rsum[i]; }, lds, m0, n0, tn, wave, lane);
}

template <int BM, int BN, int ALAY, int BLAY, int EPI, int OUT, int NW, bool F16>
__global__ __launch_bounds__(NW * 64) void gemm_bf16_kernel(const GemmArgs p) {
  gemm_bf16_body<BM, BN, ALAY, BLAY, EPI, OUT, NW, F16>(p);
}

template <int ALAY, int BLAY, int EPI, int OUT, int NW, bool F16, int BLK, bool SK, int BM = 256, int BN = 256, int OFF = 0>
__global__ __launch_bounds__(NW * 64) void gemm_q_kernel(const GemmArgs p) {
  __shared__ __attribute__((aligned(1024))) char lds[Q_LDS_BYTES];
  gemm_q_body<ALAY, BLAY, EPI, OUT, NW, F16, BLK, SK, BM, BN, OFF>(p, (int)blockIdx.x, lds);
}

// Input gradient and weight gradient of one layer in one launch: workgroups [0, n1) are the tiles of p1 (dX = dY W),
// the others the tiles of p2 (dW = dY^T X, with or without the bias gradient).  The tiles of both products fill
// the 256 compute units together: 896 + 896 tiles of Llama-3-8B's down layer are 7 whole rounds instead of twice
// 3.5, 128 + 128 of the Llama-70B shard's o-proj one round instead of two launches cut along k, and the 160 long
// tiles of that shard's QKV weight gradient leave 96 compute units to its input gradient's 1024 short ones.
// The tiles of the product with the longer k come first (n1 > 0: p1's n1 tiles, then p2's; n1 < 0: p2's -n1 tiles,
// then p1's): workgroups are handed out in index order as compute units fall free, so the long tiles start at once
// and the short ones fill in behind them.
template <int EPI2, int OUT2, bool F16>
__global__ __launch_bounds__(256) void gemm_q_bwd_kernel(const GemmArgs p1, const GemmArgs p2, const int n1) {
  __shared__ __attribute__((aligned(1024))) char lds[Q_LDS_BYTES];
  const int bid = (int)blockIdx.x;
  const bool first = n1 > 0 ? bid < n1 : bid >= -n1;      // this workgroup multiplies a tile of p1
  if (first)
    gemm_q_body<LAY_ROW, LAY_COL, MTP_EPI_NONE, OUT_BF16, 4, F16, 16, false>(p1, n1 > 0 ? bid : bid + n1, lds);
  else
    gemm_q_body<LAY_COL, LAY_COL, EPI2, OUT2, 4, F16, 16, false>(p2, n1 > 0 ? bid - n1 : bid, lds);
}

// Second pass of stream-K: one workgroup per (shared tile, row of 16x16 blocks) adds that row's pieces up in k
// order and does what the GEMM's epilogue does for a whole tile, on the 8 vectors (16 rows x 128 columns of the
// wave's part) each of its lanes holds; grid.y == 8 is the bias-gradient row (EPI_ROWSUM).  Thread t here stands
// for thread t of the GEMM workgroup: same wave, same lane, same blocks.
template <int EPI, int OUT, bool F16>
__global__ __launch_bounds__(256) void gemm_sk_reduce_kernel(const GemmArgs p) {
  using X = X16<F16>;
  constexpr int BM = 256, BN = 256, TI = 8, TJ = 8, HI = 4, HJ = 4;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
  const int KT = (p.K + QBK - 1) / QBK;
  const int tiles_m = (p.M + BM - 1) / BM;
  const int n_span = (EPI == MTP_EPI_SWIGLU) ? p.half : p.N;
  constexpr int BN_SPAN = (EPI == MTP_EPI_SWIGLU) ? BN / 2 : BN;
  const int tiles_n = (n_span + BN_SPAN - 1) / BN_SPAN;
  const int r = blockIdx.x;
  int tm, tn;
  tile_of(p.sk_full + r, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN_SPAN;
  const int w_first = r * KT / p.sk_ipw;
  const int pieces = ((r + 1) * KT - 1) / p.sk_ipw - w_first + 1;
  if (pieces == 1) return;   // one workgroup had the whole tile and wrote it
  const char* ws = static_cast<const char*>(p.ws) + tid * 16;
  const int i = blockIdx.y;
  if (i == TI) {
    if constexpr (EPI == EPI_ROWSUM) {
      if (tn != 0 || wn != 0) return;
      f32x4_t a = {0.f, 0.f, 0.f, 0.f}, b = a;
      for (int pc = 0; pc < pieces; pc++) {
        const char* q = ws + sk_slot_of(w_first + pc, r, KT, p.sk_ipw);
        const f32x4_t va = *reinterpret_cast<const f32x4_t*>(q + 64 * 4096), vb = *reinterpret_cast<const f32x4_t*>(q + 65 * 4096);
        a = pc == 0 ? va : a + va;
        b = pc == 0 ? vb : b + vb;
      }
#pragma unroll
      for (int e = 0; e < 8; e++) {
        float t = e < 4 ? a[e & 3] : b[e & 3];   // lanes holding the same row at other k add up
        t += __shfl_xor(t, 32, 64);
        t += __shfl_xor(t, 16, 64);
        const int row = m0 + (e / HI) * (BM / 2) + wm * (16 * HI) + (e % HI) * 16 + (lane & 15);
        if (lane < 16 && row < p.M) {
          if (OUT == OUT_F32) {
            float* q = (float*)p.rowsum + row;
            *q = p.accumulate ? *q + t : t;
          } else {
            uint16_t* q = (uint16_t*)p.rowsum + row;
            *q = X::to_bits(p.accumulate ? X::from_bits(*q) + t : t);
          }
        }
      }
    }
    return;
  }
  f32x4_t v[TJ];
  for (int pc = 0; pc < pieces; pc++) {
    const char* q = ws + sk_slot_of(w_first + pc, r, KT, p.sk_ipw) + (int64_t)i * TJ * 4096;
#pragma unroll
    for (int j = 0; j < TJ; j++) {
      const f32x4_t t = *reinterpret_cast<const f32x4_t*>(q + j * 4096);
      v[j] = pc == 0 ? t : v[j] + t;
    }
  }
  const int row = m0 + (i / HI) * (BM / 2) + wm * (16 * HI) + (i % HI) * 16 + (lane & 15);
  if (row >= p.M) return;
  // first column of block j, and one past the last valid column for it (as in gemm_epilogue)
  auto col_of = [&](int j) -> int {
    if (EPI == MTP_EPI_SWIGLU) return (j < HJ ? 0 : p.half) + n0 + wn * (16 * HJ) + (j % HJ) * 16 + 4 * (lane >> 4);
    return n0 + (j / HJ) * (BN / 2) + wn * (16 * HJ) + (j % HJ) * 16 + 4 * (lane >> 4);
  };
  auto lim_of = [&](int j) -> int { return (EPI == MTP_EPI_SWIGLU && j < HJ) ? p.half : p.N; };
  float pre[TJ][4];
#pragma unroll
  for (int j = 0; j < TJ; j++) {
    const int col = col_of(j), lim = lim_of(j);
#pragma unroll
    for (int e = 0; e < 4; e++) {
      float bv = 0.f;
      if (EPI == MTP_EPI_BIAS || EPI == MTP_EPI_BIAS_GELU || EPI == MTP_EPI_SWIGLU)
        if (p.bias && col + e < lim) bv = X::from_bits(p.bias[col + e]);
      pre[j][e] = v[j][e] + bv;
    }
  }
  if (OUT == OUT_F32) {
    if (p.C) {
#pragma unroll
      for (int j = 0; j < TJ; j++) {
        const int col = col_of(j), lim = lim_of(j);
        float* q = (float*)p.C + (int64_t)row * p.ldc + col;
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (col + e < lim) q[e] = p.accumulate ? q[e] + pre[j][e] : pre[j][e];
      }
    }
    return;
  }
  // 16-bit outputs: round once; an activation sees the rounded value, as the unfused layers would
#pragma unroll
  for (int j = 0; j < TJ; j++)
#pragma unroll
    for (int e = 0; e < 4; e++) pre[j][e] = X::from_bits(X::to_bits(pre[j][e]));
  if (p.C) {
#pragma unroll
    for (int j = 0; j < TJ; j++) {
      const int col = col_of(j), lim = lim_of(j);
      uint16_t* q = (uint16_t*)p.C + (int64_t)row * p.ldc + col;
#pragma unroll
      for (int e = 0; e < 4; e++)
        if (col + e < lim) q[e] = X::to_bits(p.accumulate ? X::from_bits(q[e]) + pre[j][e] : pre[j][e]);
    }
  }
  if constexpr (EPI == MTP_EPI_BIAS_GELU || EPI == MTP_EPI_GELU) {
#pragma unroll
    for (int j = 0; j < TJ; j++) {
      const int col = col_of(j), lim = lim_of(j);
      uint16_t* q = (uint16_t*)p.C2 + (int64_t)row * p.ldc2 + col;
#pragma unroll
      for (int e = 0; e < 4; e++)
        if (col + e < lim) q[e] = X::to_bits(gelu_new_f(pre[j][e]));
    }
  }
  if constexpr (EPI == MTP_EPI_SWIGLU) {
#pragma unroll
    for (int j = 0; j < HJ; j++) {
      const int col = n0 + wn * (16 * HJ) + j * 16 + 4 * (lane >> 4);
      uint16_t* q = (uint16_t*)p.C2 + (int64_t)row * p.ldc2 + col;
#pragma unroll
      for (int e = 0; e < 4; e++)
        if (col + e < p.half) q[e] = X::to_bits(silu_f(pre[j][e]) * pre[j + HJ][e]);
    }
  }
}

// ---------------------------------------------------------------------------
// Tile configurations and their choice.
//
// All 256 CUs work on one tile each, so a launch takes ceil(tiles / 256) rounds of one tile time.  A
// 256x256 tile has the best arithmetic intensity, but problems whose tile count is a little over a
// multiple of 256 (or well below 256) finish sooner with a narrower tile.  pick_config() estimates
// rounds x tile cost for each configuration that the kernel at hand was built with.
// ---------------------------------------------------------------------------
#ifndef MTP_EFF_192
#define MTP_EFF_192 1.05f
#endif
#ifndef MTP_EFF_160
#define MTP_EFF_160 1.05f
#endif
struct TileCfg {
  int bm, bn, nw;
  float eff;  // relative speed of one tile's inner loop per flop (256x256 = 1), from measurement
  int q;      // 0: the 32-deep ring; 32 / 16: the 64-deep main loop (256x256 only) on 32x32x16 / 16x16x32 MFMAs
};
// 256x256 exists as the 32-deep ring (8 waves, or 4 waves with 128x128 per wave) and as the 64-deep loop (4 or 8
// waves, 32x32x16 or 16x16x32 MFMAs).  Measured on the Llama-3-8B shapes (TFLOP/s, forward / dgrad / wgrad of
// 4096x28672x4096): ring 4 waves 1290 / 1334 / 1300; 64-deep 32x32x16 4 waves 1378 / 1393 / 1358; 64-deep
// 16x16x32 4 waves 1490 / 1538 / 1484, 8 waves 1432 / 1502 / 1411.  The narrow tiles (ring only) were measured
// best as listed.
// Configurations 10-13: the 64-deep loop on tiles narrowed to 192 or 160 along n (forward: a layer with few output
// features per rank) or along m (weight gradient of such a layer); each is built for that one product only.
constexpr TileCfg kCfgs[] = {
    {256, 256, 8, 1.00f, 0}, {256, 192, 4, 0.92f, 0}, {192, 256, 4, 0.92f, 0},  {256, 128, 4, 0.85f, 0},
    {128, 256, 8, 0.85f, 0}, {256, 256, 4, 1.02f, 0}, {256, 256, 4, 1.08f, 32}, {256, 256, 8, 1.06f, 32},
    {256, 256, 4, 1.16f, 16}, {256, 256, 8, 1.12f, 16},
    {256, 192, 4, MTP_EFF_192, 16}, {192, 256, 4, MTP_EFF_192, 16}, {256, 160, 4, MTP_EFF_160, 16}, {160, 256, 4, MTP_EFF_160, 16},
};
constexpr int kNumCfgs = sizeof(kCfgs) / sizeof(kCfgs[0]);

// Can configuration c serve the product (A layout, B layout) with epilogue EPI?  (It is instantiated only then.)
template <int EPI, int ALAY = LAY_ROW, int BLAY = LAY_ROW>
constexpr bool cfg_valid(int c) {
  const TileCfg t = kCfgs[c];
  if (t.q != 0 && (t.bm != 256 || t.bn != 256)) {
    if (EPI == MTP_EPI_SWIGLU) return false;
    // narrow along n: the forward product; narrow along m: the weight gradient
    return t.bn != 256 ? (ALAY == LAY_ROW && BLAY == LAY_ROW) : (ALAY == LAY_COL && BLAY == LAY_COL);
  }
  const int wgn = t.nw / 2;
  if (t.bn % (32 * wgn) != 0) return false;
  const int tj = t.bn / (32 * wgn);
  if (EPI == MTP_EPI_SWIGLU && tj % 2 != 0) return false;
  return true;
}

// The 64-deep loop takes whole k-tiles only, and rows of at least 256 bytes (its DMA instructions carry part of
// their address in the offset field, see dma16_at)
inline bool q_loop_ok(const GemmArgs& a) { return a.K % QBK == 0 && a.lda >= 128 && a.ldb >= 128; }

// Mixed tiling for the 64-deep loop.  One and a half rounds of 256x256 tiles take the time of two (QKV of
// Llama-3-8B: 384 tiles).  Where the tiles of the half-empty round form whole tile columns (or rows) of the output,
// the product is launched in two parts instead: the whole round on the 64-deep loop, the remaining columns (rows)
// as twice as many 256x128 (128x256) tiles of the 32-deep ring loop, which fit one round and take 0.72-0.78 of a
// full tile's time.  Measured: QKV forward 4096 x 6144 x 4096 1215 -> 1332 TFLOP/s, its weight gradient 1210 ->
// 1258 (the 256x192 tiling they ran on before: 1150-1165).  Not with the SwiGLU epilogue (its tiles interleave
// two column ranges); the bias gradient (row sums of A) only splits along rows.  MTP_GEMM_MIXED = 0 switches it off.
struct MixedSplit {
  int dim;   // 0: none, 1: columns [at, N) go to the second launch, 2: rows [at, M)
  int at;
};
template <int EPI>
MixedSplit plan_mixed(const GemmArgs& a);

template <int EPI, int ALAY = LAY_ROW, int BLAY = LAY_ROW>
int pick_config(const GemmArgs& a) {
  static MtpTune tune_cfg("MTP_GEMM_CFG"), tune_skip("MTP_GEMM_SKIP");
  if (tune_cfg.is_set()) {
    const int c = tune_cfg.get(0);
    if (c >= 0 && c < kNumCfgs && cfg_valid<EPI, ALAY, BLAY>(c) && !(kCfgs[c].q != 0 && !q_loop_ok(a))) return c;
  }
  const int64_t span = (EPI == MTP_EPI_SWIGLU) ? a.half : a.N;
  const int skip = tune_skip.get(0);  // bit c set = leave configuration c out of the choice
  int best = 0;
  double best_t = 1e300;
  for (int c = 0; c < kNumCfgs; c++) {
    if ((skip >> c) & 1) continue;
    const TileCfg t = kCfgs[c];
    const int bn_span = (EPI == MTP_EPI_SWIGLU) ? t.bn / 2 : t.bn;
    const int64_t tiles = ((a.M + t.bm - 1) / t.bm) * ((span + bn_span - 1) / bn_span);
    const int64_t rounds = (tiles + 255) / 256;
    if (!cfg_valid<EPI, ALAY, BLAY>(c) || (t.q != 0 && !q_loop_ok(a))) continue;
    double cost = (double)rounds * t.bm * t.bn / t.eff;
    if (t.q == 16 && t.nw == 4 && t.bm == 256 && t.bn == 256 && plan_mixed<EPI>(a).dim != 0) cost = ((double)(tiles / 256) + 0.78) * t.bm * t.bn / t.eff;
    if (cost < best_t * 0.999) {
      best_t = cost;
      best = c;
    }
  }
  return best;
}

template <int EPI>
MixedSplit plan_mixed(const GemmArgs& a) {
  static MtpTune tune_mixed("MTP_GEMM_MIXED");
  if (tune_mixed.get(1) == 0 || EPI == MTP_EPI_SWIGLU || !q_loop_ok(a)) return MixedSplit{0, 0};
  const int tiles_m = (a.M + 255) / 256, tiles_n = (a.N + 255) / 256;
  const int64_t tiles = (int64_t)tiles_m * tiles_n;
  const int R = (int)(tiles % 256);
  // only behind a single whole round: behind three, the half-empty round already costs less than a full one
  // (down dgrad 4096 x 14336 x 4096, 3.5 rounds: 339 us in one launch, 346 us in two)
  if (tiles / 256 != 1 || R == 0 || R > 128) return MixedSplit{0, 0};
  if (EPI != EPI_ROWSUM && R % tiles_m == 0 && cfg_valid<EPI>(3)) return MixedSplit{1, (tiles_n - R / tiles_m) * 256};
  if (R % tiles_n == 0 && cfg_valid<EPI>(4)) return MixedSplit{2, (tiles_m - R / tiles_n) * 256};
  return MixedSplit{0, 0};
}

// Stream-K for a 256x256 tiling that leaves most compute units without a tile: the k-tiles of all tiles, taken as
// one sequence, are dealt evenly to (up to) 256 workgroups; tiles that several workgroups share go through the
// scratch and gemm_sk_reduce_kernel.  Measured (Llama-70B tp=8 shard, 8192 tokens): 128 tiles with 128 k-tiles
// each (o-proj dgrad / wgrad) 138 -> 125 us.  It does not pay where at least 160 of the 256 compute units have a
// tile, nor behind full rounds: the chip runs against its power limit, so the compute units that still work in a
// part-empty round run at a higher clock and the round costs much less than its tile count suggests (160 tiles
// with 128 k-tiles: 147 us as they are, 166 us dealt out; 3.5 rounds of 64 k-tiles: 344 against 355 us), while
// the hand-over costs about 40 us per 128 shared tiles.  MTP_GEMM_SK = 0 switches it off, 1 takes it whenever
// the last round is part empty, 2 runs every tile as one workgroup through the stream-K kernel.
inline bool plan_stream_k(GemmArgs& a, int tiles, int KT) {
  static MtpTune tune_sk("MTP_GEMM_SK");
  a.sk_wgs = 0;
  const int force = tune_sk.get(-1);
  if (!a.ws || force == 0) return false;
  if (force == 2) {
    a.sk_full = tiles;
    a.sk_ipw = KT;
    return true;
  }
  const int R = tiles % SK_MAX_WGS;
  if (R == 0 || KT < 2 || (int64_t)tiles * KT >= (1ll << 31)) return false;
  if (force != 1 && !(tiles <= SK_MAX_WGS / 2 && KT >= 32)) return false;
  // at most about five pieces per tile, at least four k-tiles per piece (one where the whole k is shorter)
  int ipw = (R * KT + SK_MAX_WGS - 1) / SK_MAX_WGS;
  if (ipw < KT / 4) ipw = KT / 4;
  if (ipw < 4) ipw = KT < 4 ? KT : 4;
  a.sk_full = tiles - R;
  a.sk_ipw = ipw;
  a.sk_wgs = (R * KT + ipw - 1) / ipw;
  return a.sk_wgs <= SK_MAX_WGS;
}

template <int C, int ALAY, int BLAY, int EPI, int OUT, bool F16>
int launch_cfg(const GemmArgs& a, hipStream_t s) {
  if constexpr (!cfg_valid<EPI, ALAY, BLAY>(C)) {
    mtp_set_error("gemm_bf16: tile configuration %d cannot serve this epilogue", C);
    return MTP_EINVAL;
  } else {
    constexpr int BM = kCfgs[C].bm, BN = kCfgs[C].bn, NW = kCfgs[C].nw;
    const int tiles_m = (a.M + BM - 1) / BM;
    const int span = (EPI == MTP_EPI_SWIGLU) ? a.half : a.N;
    const int bn_span = (EPI == MTP_EPI_SWIGLU) ? BN / 2 : BN;
    const int tiles_n = (span + bn_span - 1) / bn_span;
    if constexpr (kCfgs[C].q == 16 && NW == 4 && BM == 256 && BN == 256) {
      GemmArgs b = a;
      if (plan_stream_k(b, tiles_m * tiles_n, (a.K + QBK - 1) / QBK)) {
        hipLaunchKernelGGL((gemm_q_kernel<ALAY, BLAY, EPI, OUT, NW, F16, 16, true>), dim3((unsigned)(b.sk_full + b.sk_wgs)),
                           dim3(NW * 64), 0, s, b);
        MTP_CHECK_LAUNCH("gemm_bf16");
        if (b.sk_wgs > 0) {
          const int shared = tiles_m * tiles_n - b.sk_full;
          hipLaunchKernelGGL((gemm_sk_reduce_kernel<EPI, OUT, F16>), dim3((unsigned)shared, EPI == EPI_ROWSUM ? 9u : 8u),
                             dim3(256), 0, s, b);
          MTP_CHECK_LAUNCH("gemm_bf16 stream-K reduce");
        }
        return MTP_OK;
      }
    }
#ifdef MTP_MEASURE
    // measurement builds: the forward product's 64-deep loop with its DMA requests (debug bit 16) and / or its
    // fragment reads (bit 32) left out, for the decomposition of the loop's time; results are wrong
    if constexpr (C == 8 && ALAY == LAY_ROW && BLAY == LAY_ROW && !F16 && OUT == OUT_BF16 &&
                  (EPI == MTP_EPI_NONE || EPI == MTP_EPI_SWIGLU)) {
      const int off = (a.debug >> 4) & 3;
      const dim3 grid((unsigned)(tiles_m * tiles_n)), block(NW * 64);
      if (off == 1) hipLaunchKernelGGL((gemm_q_kernel<ALAY, BLAY, EPI, OUT, NW, F16, 16, false, 256, 256, 1>), grid, block, 0, s, a);
      if (off == 2) hipLaunchKernelGGL((gemm_q_kernel<ALAY, BLAY, EPI, OUT, NW, F16, 16, false, 256, 256, 2>), grid, block, 0, s, a);
      if (off == 3) hipLaunchKernelGGL((gemm_q_kernel<ALAY, BLAY, EPI, OUT, NW, F16, 16, false, 256, 256, 3>), grid, block, 0, s, a);
      if (off != 0) {
        MTP_CHECK_LAUNCH("gemm_bf16 (parts of the loop off)");
        return MTP_OK;
      }
    }
#endif
    if constexpr (kCfgs[C].q != 0)
      hipLaunchKernelGGL((gemm_q_kernel<ALAY, BLAY, EPI, OUT, NW, F16, (kCfgs[C].q ? kCfgs[C].q : 32), false, BM, BN>),
                         dim3((unsigned)(tiles_m * tiles_n)), dim3(NW * 64), 0, s, a);
    else
      hipLaunchKernelGGL((gemm_bf16_kernel<BM, BN, ALAY, BLAY, EPI, OUT, NW, F16>), dim3((unsigned)(tiles_m * tiles_n)),
                         dim3(NW * 64), 0, s, a);
    MTP_CHECK_LAUNCH("gemm_bf16");
    return MTP_OK;
  }
}

template <int ALAY, int BLAY, int EPI, int OUT, bool F16>
int launch_typed(GemmArgs a, hipStream_t s) {
#ifdef MTP_MEASURE
  static MtpTune tune_debug("MTP_GEMM_DEBUG");
  a.debug = tune_debug.get(0);
#endif
  int c = pick_config<EPI, ALAY, BLAY>(a);
  if (!cfg_valid<EPI, ALAY, BLAY>(c)) c = 0;
  static MtpTune tune_forced("MTP_GEMM_CFG");
  if (c == 8 && !tune_forced.is_set()) {
    const MixedSplit ms = plan_mixed<EPI>(a);
    constexpr int64_t esz = OUT == OUT_F32 ? 4 : 2;
    if (ms.dim == 1) {
      GemmArgs a1 = a, a2 = a;
      a1.N = ms.at;
      a2.N = a.N - ms.at;
      a2.B = a.B + (BLAY == LAY_ROW ? (int64_t)ms.at * a.ldb : (int64_t)ms.at);
      a2.C = a.C ? (char*)a.C + (int64_t)ms.at * esz : nullptr;
      a2.C2 = a.C2 ? (char*)a.C2 + (int64_t)ms.at * 2 : nullptr;
      a2.bias = a.bias ? a.bias + ms.at : nullptr;
      const int rc = launch_cfg<8, ALAY, BLAY, EPI, OUT, F16>(a1, s);
      return rc ? rc : launch_cfg<3, ALAY, BLAY, EPI, OUT, F16>(a2, s);
    }
    if (ms.dim == 2) {
      GemmArgs a1 = a, a2 = a;
      a1.M = ms.at;
      a2.M = a.M - ms.at;
      a2.A = a.A + (ALAY == LAY_ROW ? (int64_t)ms.at * a.lda : (int64_t)ms.at);
      a2.C = a.C ? (char*)a.C + (int64_t)ms.at * a.ldc * esz : nullptr;
      a2.C2 = a.C2 ? (char*)a.C2 + (int64_t)ms.at * a.ldc2 * 2 : nullptr;
      a2.rowsum = a.rowsum ? (char*)a.rowsum + (int64_t)ms.at * esz : nullptr;
      const int rc = launch_cfg<8, ALAY, BLAY, EPI, OUT, F16>(a1, s);
      return rc ? rc : launch_cfg<4, ALAY, BLAY, EPI, OUT, F16>(a2, s);
    }
  }
  switch (c) {
    case 0: return launch_cfg<0, ALAY, BLAY, EPI, OUT, F16>(a, s);
    case 1: return launch_cfg<1, ALAY, BLAY, EPI, OUT, F16>(a, s);
    case 2: return launch_cfg<2, ALAY, BLAY, EPI, OUT, F16>(a, s);
    case 3: return launch_cfg<3, ALAY, BLAY, EPI, OUT, F16>(a, s);
    case 4: return launch_cfg<4, ALAY, BLAY, EPI, OUT, F16>(a, s);
    case 5: return launch_cfg<5, ALAY, BLAY, EPI, OUT, F16>(a, s);
    case 6: return launch_cfg<6, ALAY, BLAY, EPI, OUT, F16>(a, s);
    case 7: return launch_cfg<7, ALAY, BLAY, EPI, OUT, F16>(a, s);
    case 8: return launch_cfg<8, ALAY, BLAY, EPI, OUT, F16>(a, s);
    case 9: return launch_cfg<9, ALAY, BLAY, EPI, OUT, F16>(a, s);
    case 10: return launch_cfg<10, ALAY, BLAY, EPI, OUT, F16>(a, s);
    case 11: return launch_cfg<11, ALAY, BLAY, EPI, OUT, F16>(a, s);
    case 12: return launch_cfg<12, ALAY, BLAY, EPI, OUT, F16>(a, s);
    case 13: return launch_cfg<13, ALAY, BLAY, EPI, OUT, F16>(a, s);
  }
  return MTP_EINVAL;
}

// f16 != 0: the 16-bit tensors (A, B, bias, and C / C2 / rowsum unless OUT_F32) are IEEE half instead of bf16
template <int ALAY, int BLAY, int EPI, int OUT>
int launch(const GemmArgs& a, hipStream_t s, int f16) {
  return f16 ? launch_typed<ALAY, BLAY, EPI, OUT, true>(a, s) : launch_typed<ALAY, BLAY, EPI, OUT, false>(a, s);
}

}  // namespace
