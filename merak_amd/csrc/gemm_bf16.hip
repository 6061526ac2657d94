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
// Structure (one workgroup = 4 waves = one BMxBN tile, BK = 64):
//   * global -> LDS with buffer_load_dwordx4 ... lds (no VGPR staging; rows and
//     columns past the matrix edge read as zero through the buffer range check),
//     double buffered, one s_barrier per k-tile;
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
#include "mtp_common.h"
#include <type_traits>

namespace {

constexpr int BK = 64;
constexpr int LAY_ROW = 0;  // reduction dimension contiguous
constexpr int LAY_COL = 1;  // M (or N) contiguous

struct GemmArgs {
  const uint16_t* A;
  const uint16_t* B;
  void* C;             // main output (bf16 or fp32), may be null when C2 carries the result
  void* C2;            // activation output (bf16), epilogue dependent
  const uint16_t* bias;
  int M, N, K;
  int64_t lda, ldb, ldc, ldc2;
  int accumulate;      // C += result
  int half;            // SwiGLU: number of gate columns (N/2)
};

enum : int { OUT_BF16 = 0, OUT_F32 = 1 };

// LDS hand-over between lanes of one wave: DS operations of a wave complete in order, the fence and
// the scheduling barrier keep the compiler from moving accesses across the hand-over point.
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
  __builtin_amdgcn_wave_barrier();
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, int64_t bytes) {
  if (bytes < 0) bytes = 0;
  // offsets are tile relative and below 2^31; 0x80000000 is the "read as zero" marker
  const uint32_t n = bytes > 0x80000000ll ? 0x80000000u : (uint32_t)bytes;
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, n, 0x00020000);
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

// ---------------------------------------------------------------------------
// LDS tile of a "row" operand: ROWS x 64 bf16, 128 bytes per row, the 16-byte
// chunk c of row r is stored at chunk position c ^ ((r >> 1) & 7).
// One DMA instruction fills 8 rows (1 KiB, lane l -> row l/8, position l%8).
// ---------------------------------------------------------------------------
template <int ROWS>
struct RowTile {
  static constexpr int BYTES = ROWS * 128;
  static constexpr int INSTR_PER_WAVE = ROWS / 32;  // 4 waves, 8 rows per instruction

  // LDS byte address of fragment rows (row = row0 + lane%32), k16 step kk: 8 elements at k = 16kk + 8(lane/32)
  __device__ static __forceinline__ uint32_t frag_offset(int row, int kk, int h) {
    return (uint32_t)(row * 128 + ((((2 * kk + h) ^ (row >> 1)) & 7) << 4));
  }
};

// The body lives in a __device__ function: it uses device-only types (__amdgpu_buffer_rsrc_t) that the
// host pass over a __global__ function cannot digest.
template <int BM, int BN, int ALAY, int BLAY, int EPI, int OUT>
__device__ __forceinline__ void gemm_bf16_body(const GemmArgs& p) {
  static_assert(ALAY == LAY_ROW && BLAY == LAY_ROW, "layout not built yet");
  constexpr int TI = BM / 64, TJ = BN / 64;  // 32x32 blocks per wave in m and n
  using ATile = RowTile<BM>;
  using BTile = RowTile<BN>;
  constexpr int STAGE_BYTES = ATile::BYTES + BTile::BYTES;
  __shared__ __attribute__((aligned(1024))) char lds[2 * STAGE_BYTES];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int lh = lane >> 5, l32 = lane & 31;

  const int tiles_m = (p.M + BM - 1) / BM;
  const int n_span = (EPI == MTP_EPI_SWIGLU) ? p.half : p.N;  // SwiGLU tiles cover BN/2 gate + BN/2 up columns
  constexpr int BN_SPAN = (EPI == MTP_EPI_SWIGLU) ? BN / 2 : BN;
  const int tiles_n = (n_span + BN_SPAN - 1) / BN_SPAN;
  int tm, tn;
  tile_of(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM;
  const int n0 = tn * BN_SPAN;

  // ---- DMA addressing -------------------------------------------------------
  // Every DMA instruction moves 8 tile rows; instruction q = wave + 4j.  The per-lane byte offset
  // (row * ld + chunk * 8) * 2 goes into the VGPR offset, which the buffer range check covers: rows
  // past the matrix edge land beyond num_records and read as zero.  The k-tile advance goes into the
  // scalar offset (not range checked, always inside the row; the ragged last k-tile is masked by hand).
  // A: rows m0.. of [M,K]
  const __amdgpu_buffer_rsrc_t rsrcA = make_rsrc(p.A + (int64_t)m0 * p.lda, (int64_t)(p.M - m0) * p.lda * 2);
  // B: LDS row r of the tile maps to a global row of [N,K].  Plain: n0 + r.  SwiGLU: the wave-column wn
  // owns LDS rows [wn*BN/2, (wn+1)*BN/2): first half gate rows, second half the matching up rows.
  const __amdgpu_buffer_rsrc_t rsrcB = make_rsrc(p.B + (int64_t)n0 * p.ldb, (int64_t)(p.N - n0) * p.ldb * 2);
  const int chunk = (lane & 7) ^ ((4 * wave + (lane >> 4)) & 7);  // k chunk (8 elements) this lane fetches
  const int lrow = lane >> 3;
  uint32_t voffA[ATile::INSTR_PER_WAVE], voffB[BTile::INSTR_PER_WAVE];
#pragma unroll
  for (int j = 0; j < ATile::INSTR_PER_WAVE; j++) {
    const int r = (wave + 4 * j) * 8 + lrow;
    voffA[j] = (uint32_t)(((int64_t)r * p.lda + chunk * 8) * 2);
  }
#pragma unroll
  for (int j = 0; j < BTile::INSTR_PER_WAVE; j++) {
    const int r = (wave + 4 * j) * 8 + lrow;
    int64_t gr = r;  // relative to n0
    if (EPI == MTP_EPI_SWIGLU) {
      const int seg = r / (BN / 4), in = r % (BN / 4);
      gr = ((seg & 1) ? p.half : 0) + (seg >> 1) * (BN / 4) + in;
      // gate rows at or past `half` belong to the up matrix: treat as out of range
      if (!(seg & 1) && n0 + gr >= p.half) gr = (int64_t)p.N;
    }
    voffB[j] = (uint32_t)((gr * p.ldb + chunk * 8) * 2);
    if (gr >= p.N - n0) voffB[j] = 0x80000000u;
  }

  auto issue_loads = [&](int kt, int buf) {
    char* la = lds + buf * STAGE_BYTES;
    char* lb = la + ATile::BYTES;
    const bool dead = kt * BK + chunk * 8 >= p.K;  // only ever true in a ragged last k-tile
    const uint32_t soff = (uint32_t)(kt * BK * 2);
#pragma unroll
    for (int j = 0; j < ATile::INSTR_PER_WAVE; j++) {
      const int q = wave + 4 * j;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcA, LDS_PTR(la + q * 1024), 16, dead ? 0x80000000u : voffA[j], soff,
                                               0, 0);
    }
#pragma unroll
    for (int j = 0; j < BTile::INSTR_PER_WAVE; j++) {
      const int q = wave + 4 * j;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcB, LDS_PTR(lb + q * 1024), 16, dead ? 0x80000000u : voffB[j], soff,
                                               0, 0);
    }
  };

  // ---- fragment addressing ---------------------------------------------------
  uint32_t fa[4], fb[4];  // per k16 step, block 0; further blocks are +32 rows = +4096 bytes
#pragma unroll
  for (int kk = 0; kk < 4; kk++) {
    fa[kk] = ATile::frag_offset(wm * (BM / 2) + l32, kk, lh);
    fb[kk] = BTile::frag_offset(wn * (BN / 2) + l32, kk, lh);
  }

  f32x16_t acc[TI][TJ];
#pragma unroll
  for (int i = 0; i < TI; i++)
#pragma unroll
    for (int j = 0; j < TJ; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  // ---- main loop ---------------------------------------------------------------
  // Two LDS stages.  Tile kt+1 is requested as soon as the barrier at the end of tile kt-1 has freed its
  // stage, i.e. a full k-tile (64 MFMAs per wave) ahead of its first use.  Fragments are double buffered
  // in registers: the ds_reads of k16-step s+1 are in flight while the MFMAs of step s issue.
  const int KT = (p.K + BK - 1) / BK;
  bf16x8_t af[2][TI], bfr[2][TJ];
  // Reads are issued A0 B0 A1 B1 ... and the MFMAs walk the block grid in growing squares
  // ((0,0); (1,0) (1,1) (0,1); ...), so the first MFMAs of a step depend only on the oldest reads.
  auto read_frags = [&](int buf, int kk, int slot) {
    const char* la = lds + buf * STAGE_BYTES;
    const char* lb = la + ATile::BYTES;
#pragma unroll
    for (int d = 0; d < (TI > TJ ? TI : TJ); d++) {
      if (d < TI) af[slot][d] = *reinterpret_cast<const bf16x8_t*>(la + fa[kk] + d * 4096);
      if (d < TJ) bfr[slot][d] = *reinterpret_cast<const bf16x8_t*>(lb + fb[kk] + d * 4096);
    }
  };
  auto mfmas = [&](int slot) {
#pragma unroll
    for (int d = 0; d < (TI > TJ ? TI : TJ); d++) {
#pragma unroll
      for (int j = 0; j <= d; j++)  // row d of the shell
        if (d < TI && j < TJ)
          acc[d][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[slot][j], af[slot][d], acc[d][j], 0, 0, 0);
#pragma unroll
      for (int i = 0; i < d; i++)  // column d of the shell
        if (i < TI && d < TJ)
          acc[i][d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[slot][d], af[slot][i], acc[i][d], 0, 0, 0);
    }
  };

  // One k-tile.  FULL: tiles kt+1 and kt+2 exist, so the prefetches are unconditional and the body is a
  // single basic block whose instruction mix is pinned by the sched_group_barrier sequence:
  //   steps 0-2 : 8 x (2 MFMA, 1 LDS read)
  //   step 3    : 8 x (1 MFMA, 1 DMA, 1 LDS read, 1 MFMA, 1 DMA)   [16 DMA instructions per wave at 256x256]
  auto ktile = [&](int kt, auto full_tag) {
    constexpr bool FULL = decltype(full_tag)::value;
    const int buf = kt & 1;
    read_frags(buf, 1, 1);
    mfmas(0);
    read_frags(buf, 2, 0);
    mfmas(1);
    read_frags(buf, 3, 1);
    mfmas(0);
    if (FULL) {
#pragma unroll
      for (int t = 0; t < 3 * (TI + TJ); t++) {
        __builtin_amdgcn_sched_group_barrier(0x008, (TI * TJ) / (TI + TJ), 0);  // MFMA
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                      // DS read
      }
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): tile kt+1 has landed in the other stage
    __syncthreads();                     // ... for every wave, and everyone is done reading this stage
    if (FULL || kt + 2 < KT) issue_loads(kt + 2, buf);
    if (FULL || kt + 1 < KT) read_frags(buf ^ 1, 0, 0);
    mfmas(1);
    if (FULL) {
      constexpr int NDMA = ATile::INSTR_PER_WAVE + BTile::INSTR_PER_WAVE;
      constexpr int NMF = TI * TJ, NDS = TI + TJ;
      static_assert(NMF % NDS == 0 && NDMA % NDS == 0, "schedule assumes these ratios");
#pragma unroll
      for (int t = 0; t < NDS; t++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                 // MFMA
        __builtin_amdgcn_sched_group_barrier(0x020, NDMA / NDS, 0);        // VMEM read (DMA)
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                 // DS read
        __builtin_amdgcn_sched_group_barrier(0x008, NMF / NDS - 1, 0);     // MFMA
      }
    }
  };

  issue_loads(0, 0);
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();
  if (KT > 1) issue_loads(1, 1);
  read_frags(0, 0, 0);
  int kt = 0;
  for (; kt + 2 < KT; kt++) ktile(kt, std::true_type{});
  for (; kt < KT; kt++) ktile(kt, std::false_type{});
  __builtin_amdgcn_s_waitcnt(0x0f70);
  __syncthreads();  // the epilogue reuses the tile buffers

  // ---- epilogue ----------------------------------------------------------------
  // acc[i][j][r]: row m = m0 + wm*BM/2 + 32i + l32, column block j, n_local = 8*(r/4) + 4*lh + r%4.
  // Stage 32 rows x (BN/2) columns per wave through LDS, then 16-byte row-contiguous stores.
  constexpr int WN = BN / 2;                       // columns per wave
  constexpr int ESZ = (OUT == OUT_F32) ? 4 : 2;
  constexpr int PITCH = WN * ESZ + 16;             // bytes per staged row (+16: spread rows over banks)
  static_assert(4 * 32 * PITCH <= 2 * STAGE_BYTES, "epilogue staging exceeds the tile buffers");
  char* stage = lds + wave * (32 * PITCH);

  // global column of the first element of block j for this wave (main output C)
  auto col_of_block = [&](int j) -> int {
    if (EPI == MTP_EPI_SWIGLU) {
      const int hj = TJ / 2;
      return (j < hj ? 0 : p.half) + n0 + wn * (BN / 4) + (j % hj) * 32;
    }
    return n0 + wn * WN + j * 32;
  };
  // first column past the valid range of block j: SwiGLU gate blocks end at `half` (the columns after it
  // are the up matrix, owned by other blocks)
  auto lim_of_block = [&](int j) -> int {
    if (EPI == MTP_EPI_SWIGLU) return j < TJ / 2 ? p.half : p.N;
    return p.N;
  };

  auto flush = [&](int i, void* out, int64_t ld, int nblk, auto colfn, auto limfn, bool f32out, bool accumulate) {
    // 16-byte chunks of the staged 32 x (nblk*32) block
    const int esz = f32out ? 4 : 2;
    const int chunks_per_row = nblk * 32 * esz / 16;
    const int epc = 16 / esz;  // elements per chunk
    const int total = 32 * chunks_per_row;
    const int mrow0 = m0 + wm * (BM / 2) + 32 * i;
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
              v.x = pack_bf16x2(bf16_lo(v.x) + bf16_lo(o.x), bf16_hi(v.x) + bf16_hi(o.x));
              v.y = pack_bf16x2(bf16_lo(v.y) + bf16_lo(o.y), bf16_hi(v.y) + bf16_hi(o.y));
              v.z = pack_bf16x2(bf16_lo(v.z) + bf16_lo(o.z), bf16_hi(v.z) + bf16_hi(o.z));
              v.w = pack_bf16x2(bf16_lo(v.w) + bf16_lo(o.w), bf16_hi(v.w) + bf16_hi(o.w));
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
              const float nv = (e & 1) ? bf16_hi(pr) : bf16_lo(pr);
              *q = f32_to_bf16_bits(accumulate ? bf16_bits_to_f32(*q) + nv : nv);
            }
          }
        }
      }
    }
  };

#pragma unroll
  for (int i = 0; i < TI; i++) {
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
              const int col = cb + 8 * g + 4 * lh + e;
              b4[e] = col < lim_of_block(j) ? bf16_bits_to_f32(p.bias[col]) : 0.f;
            }
          }
        }
#pragma unroll
        for (int e = 0; e < 4; e++) pre[j][4 * g + e] = acc[i][j][4 * g + e] + b4[e];
      }
    }
    if (OUT == OUT_F32) {
      if (p.C) {
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
          for (int g = 0; g < 4; g++) {
            f32x4_t v = {pre[j][4 * g], pre[j][4 * g + 1], pre[j][4 * g + 2], pre[j][4 * g + 3]};
            *reinterpret_cast<f32x4_t*>(stage + l32 * PITCH + (32 * j + 8 * g + 4 * lh) * 4) = v;
          }
        wave_lds_sync();
        flush(i, p.C, p.ldc, TJ, col_of_block, lim_of_block, true, p.accumulate != 0);
        wave_lds_sync();
      }
    } else {
      // round to bf16 once; the activation sees the rounded value, as the unfused layers would
#pragma unroll
      for (int j = 0; j < TJ; j++)
#pragma unroll
        for (int r = 0; r < 16; r++) pre[j][r] = bf16_bits_to_f32(f32_to_bf16_bits(pre[j][r]));
      if (p.C) {
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
          for (int g = 0; g < 4; g++) {
            u32x2_t v = {pack_bf16x2(pre[j][4 * g], pre[j][4 * g + 1]), pack_bf16x2(pre[j][4 * g + 2], pre[j][4 * g + 3])};
            *reinterpret_cast<u32x2_t*>(stage + l32 * PITCH + (32 * j + 8 * g + 4 * lh) * 2) = v;
          }
        wave_lds_sync();
        flush(i, p.C, p.ldc, TJ, col_of_block, lim_of_block, false, p.accumulate != 0);
        wave_lds_sync();
      }
      if (EPI == MTP_EPI_BIAS_GELU || EPI == MTP_EPI_GELU) {
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
          for (int g = 0; g < 4; g++) {
            u32x2_t v = {pack_bf16x2(gelu_new_f(pre[j][4 * g]), gelu_new_f(pre[j][4 * g + 1])),
                         pack_bf16x2(gelu_new_f(pre[j][4 * g + 2]), gelu_new_f(pre[j][4 * g + 3]))};
            *reinterpret_cast<u32x2_t*>(stage + l32 * PITCH + (32 * j + 8 * g + 4 * lh) * 2) = v;
          }
        wave_lds_sync();
        flush(i, p.C2, p.ldc2, TJ, col_of_block, lim_of_block, false, false);
        wave_lds_sync();
      }
      if (EPI == MTP_EPI_SWIGLU) {
        constexpr int HJ = TJ / 2;
#pragma unroll
        for (int j = 0; j < HJ; j++)
#pragma unroll
          for (int g = 0; g < 4; g++) {
            float a4[4];
#pragma unroll
            for (int e = 0; e < 4; e++) a4[e] = silu_f(pre[j][4 * g + e]) * pre[j + HJ][4 * g + e];
            u32x2_t v = {pack_bf16x2(a4[0], a4[1]), pack_bf16x2(a4[2], a4[3])};
            *reinterpret_cast<u32x2_t*>(stage + l32 * PITCH + (32 * j + 8 * g + 4 * lh) * 2) = v;
          }
        wave_lds_sync();
        auto act_col = [&](int j) -> int { return n0 + wn * (BN / 4) + j * 32; };
        auto act_lim = [&](int) -> int { return p.half; };
        flush(i, p.C2, p.ldc2, HJ, act_col, act_lim, false, false);
        wave_lds_sync();
      }
    }
  }
}

template <int BM, int BN, int ALAY, int BLAY, int EPI, int OUT>
__global__ __launch_bounds__(256) void gemm_bf16_kernel(const GemmArgs p) {
  gemm_bf16_body<BM, BN, ALAY, BLAY, EPI, OUT>(p);
}

template <int BM, int BN, int ALAY, int BLAY, int EPI, int OUT>
int launch(const GemmArgs& a, hipStream_t s) {
  const int tiles_m = (a.M + BM - 1) / BM;
  const int span = (EPI == MTP_EPI_SWIGLU) ? a.half : a.N;
  const int bn_span = (EPI == MTP_EPI_SWIGLU) ? BN / 2 : BN;
  const int tiles_n = (span + bn_span - 1) / bn_span;
  hipLaunchKernelGGL((gemm_bf16_kernel<BM, BN, ALAY, BLAY, EPI, OUT>), dim3((unsigned)(tiles_m * tiles_n)), dim3(256),
                     0, s, a);
  MTP_CHECK_LAUNCH("gemm_bf16");
  return MTP_OK;
}

}  // namespace

// Entry used by the C API layer (linear.hip).
int mtp_gemm_bf16_nt(const void* A, const void* B, const void* bias, void* C, void* C2, int64_t M, int64_t N,
                     int64_t K, int epilogue, hipStream_t s) {
  GemmArgs a{};
  a.A = (const uint16_t*)A;
  a.B = (const uint16_t*)B;
  a.bias = (const uint16_t*)bias;
  a.C = C;
  a.C2 = C2;
  a.M = (int)M;
  a.N = (int)N;
  a.K = (int)K;
  a.lda = K;
  a.ldb = K;
  a.ldc = N;
  a.accumulate = 0;
  a.half = (int)(N / 2);
  a.ldc2 = (epilogue == MTP_EPI_SWIGLU) ? N / 2 : N;
  switch (epilogue) {
    case MTP_EPI_NONE: return launch<256, 256, LAY_ROW, LAY_ROW, MTP_EPI_NONE, OUT_BF16>(a, s);
    case MTP_EPI_BIAS: return launch<256, 256, LAY_ROW, LAY_ROW, MTP_EPI_BIAS, OUT_BF16>(a, s);
    case MTP_EPI_BIAS_GELU: return launch<256, 256, LAY_ROW, LAY_ROW, MTP_EPI_BIAS_GELU, OUT_BF16>(a, s);
    case MTP_EPI_GELU: return launch<256, 256, LAY_ROW, LAY_ROW, MTP_EPI_GELU, OUT_BF16>(a, s);
    case MTP_EPI_SWIGLU: return launch<256, 256, LAY_ROW, LAY_ROW, MTP_EPI_SWIGLU, OUT_BF16>(a, s);
  }
  mtp_set_error("gemm_bf16: unknown epilogue %d", epilogue);
  return MTP_EINVAL;
}

// dgrad / wgrad on the bf16 MFMA kernel: not built yet, the caller falls back to the general kernel.
int mtp_gemm_bf16_dgrad(const void*, const void*, void*, int64_t, int64_t, int64_t, hipStream_t) {
  return MTP_EUNSUPPORTED;
}
int mtp_gemm_bf16_wgrad(const void*, const void*, void*, void*, int64_t, int64_t, int64_t, int, int, hipStream_t) {
  return MTP_EUNSUPPORTED;
}
