// fp32 MFMA GEMM for gfx950: the linear layers of an fp32 model (the
// GPT-2-small shaped configuration), fp32 in, fp32 accumulate, fp32 out.
//
//   C[M,N] (+)= opA(A) * opB(B) (+ bias[n])
// with A given as [M,K] ("row": K contiguous) or [K,M] ("col"), B as [N,K]
// ("row") or [K,N] ("col"): forward = (row,row), dgrad = (row,col), wgrad =
// (col,col), as in the bf16 kernel.
//
// v_mfma_f32_32x32x2_f32 delivers a sixteenth of the bf16 rate, so the tile
// can be small and several workgroups share a CU: 128x128 tile (128x64, 64x128
// or 64x64 when that is needed to fill the chip), BK = 16, 4 waves (2x2), a
// ring of 3 stages of at most 16 KiB filled by
// buffer_load_dwordx4 ... lds (no VGPR staging; out-of-range rows, columns
// and k read as zero), one barrier per k-tile.
//   "row" tiles: [128 rows][16 floats], 16-byte chunks XOR-swizzled by
//     (row >> 2) & 3; lane (i = l%32, h = l/32) reads chunks 2q+h (q = 0,1)
//     with ds_read_b128: its four floats feed four MFMA steps (which k of
//     the pair a lane supplies is free as long as A and B agree).
//   "col" tiles: [16 k][128 floats]; the two half-waves of a ds_read_b32 read
//     k rows 4 apart (the k the row layout gives them), so k rows with bit 2 set
//     are rotated by 32 floats to land in the other half of the banks.
// The MFMA is issued with the B fragment first, so a lane holds 4 consecutive
// output columns; 32 rows x 64 columns per wave are staged through LDS and
// stored 16 bytes per lane, 256 contiguous bytes per row.
#include "gemm_bf16_kernel.h"

namespace {

constexpr int FBK = 16, FSTAGES = 3;

struct F32Args {
  const float* A;
  const float* B;
  const float* bias;
  float* C;
  float* rowsum;  // optional [M]: rowsum[m] (+)= sum_k opA(A)[m,k] (the bias gradient when A = dY^T)
  int M, N, K;
  int64_t lda, ldb, ldc;
  int accumulate;
  // k slices (gridDim.y > 1): slice y multiplies k in [y * kslice, min(K, (y + 1) * kslice)) and stores its tile, as
  // it is, into part + y * M * N (row length N) and its row sums into part_rowsum + y * M; f32_slices_sum_kernel
  // adds the slices up in slice order
  int kslice;
  float* part;
  float* part_rowsum;
};

// One operand tile of ROWS (rows of A / rows of B; 128 or 64) x 16 k.
template <int LAY, int ROWS>
struct FOperand {
  static constexpr int BYTES = ROWS * FBK * 4;
  static constexpr int F_NI = BYTES / 1024 / 4;  // DMA instructions per wave: 2 or 1
  static constexpr int LPR = ROWS / 4;           // col layout: lanes (16-byte pieces) per k row
  rsrc_t rsrc;
  uint32_t voff[F_NI];   // byte offset of this lane's 16 bytes at k-tile 0 (0x80000000: reads zero)
  uint32_t kstep;        // bytes per k-tile
  int kchunk[F_NI];      // row layout: first k of this lane's chunk inside a k-tile
  // rows_total: rows of the whole matrix; ld in floats
  __device__ __forceinline__ void init(const float* base, int64_t ld, int row0, int rows_total, int K, int lane,
                                       int wave) {
    if (LAY == LAY_ROW) {
      // memory [rows][K]: instruction q = wave + 4 j covers tile rows 16q .. 16q+15, lane l -> row 16q + l/4
      rsrc = make_rsrc(base + (int64_t)row0 * ld, (int64_t)(rows_total - row0) * ld * 4);
      kstep = FBK * 4;
#pragma unroll
      for (int j = 0; j < F_NI; j++) {
        const int r = (wave + 4 * j) * 16 + (lane >> 2);
        const int chunk = (lane & 3) ^ ((lane >> 4) & 3);  // (r >> 2) & 3 == (lane >> 4) & 3
        kchunk[j] = chunk * 4;
        voff[j] = (row0 + r < rows_total) ? (uint32_t)((r * ld + chunk * 4) * 4) : 0x80000000u;
      }
    } else {
      // memory [K][rows]: an instruction covers 64 / LPR k rows; LDS position p (16-byte units) of k row k
      // holds columns 4 * ((p - 8 ((k >> 2) & 1)) mod LPR) ..: the two half-waves of a fragment read are 4 k
      // rows apart (see frags) and must not share banks
      rsrc = make_rsrc(base + row0, ((int64_t)K * ld - row0) * 4);
      kstep = (uint32_t)(FBK * ld * 4);
#pragma unroll
      for (int j = 0; j < F_NI; j++) {
        const int k = (wave + 4 * j) * (64 / LPR) + lane / LPR;
        const int col = 4 * (((lane % LPR) - 8 * ((k >> 2) & 1)) & (LPR - 1));
        kchunk[j] = 0;
        voff[j] = (row0 + col < rows_total) ? (uint32_t)((k * ld + col) * 4) : 0x80000000u;
      }
    }
  }
  // request k-tile kt into the tile at LDS address `tile`
  __device__ __forceinline__ void issue(uint32_t tile, int kt, int K, int wave) const {
#pragma unroll
    for (int j = 0; j < F_NI; j++) {
      uint32_t v = voff[j] + (uint32_t)kt * kstep;
      // row layout: k past the end of the row would read the next row; col layout: k rows past K lie beyond
      // the buffer and read zero by themselves
      if (LAY == LAY_ROW && kt * FBK + kchunk[j] >= K) v = 0x80000000u;
      if (voff[j] == 0x80000000u) v = 0x80000000u;
      dma16(rsrc, tile + (wave + 4 * j) * 1024, v, 0);
    }
  }
  // fragments of the 32-row block starting at tile row r0 for the 8 MFMA steps of a k-tile: f[s], s = 4q + t
  __device__ __forceinline__ void frags(const char* tile, int r0, int lane, float* f) const {
    const int i = lane & 31, h = lane >> 5;
    if (LAY == LAY_ROW) {
      const int row = r0 + i;
#pragma unroll
      for (int q = 0; q < 2; q++) {
        const int pos = (2 * q + h) ^ ((row >> 2) & 3);
        const f32x4_t v = *reinterpret_cast<const f32x4_t*>(tile + row * 64 + pos * 16);
        f[4 * q] = v.x; f[4 * q + 1] = v.y; f[4 * q + 2] = v.z; f[4 * q + 3] = v.w;
      }
    } else {
      // the same k as the row layout hands to step s = 4q + t of lane half h: k = 8q + 4h + t
#pragma unroll
      for (int s = 0; s < 8; s++) {
        const int k = 8 * (s >> 2) + 4 * h + (s & 3);
        f[s] = *reinterpret_cast<const float*>(tile + k * (ROWS * 4) + (((r0 + i) + 32 * ((k >> 2) & 1)) & (ROWS - 1)) * 4);
      }
    }
  }
};

template <int ALAY, int BLAY, int BM, int BN>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const F32Args q) {
  F32Args p = q;
  if (gridDim.y > 1) {
    const int k0 = (int)blockIdx.y * q.kslice;
    p.K = min(q.K - k0, q.kslice);
    p.A = q.A + (ALAY == LAY_ROW ? (int64_t)k0 : (int64_t)k0 * q.lda);
    p.B = q.B + (BLAY == LAY_ROW ? (int64_t)k0 : (int64_t)k0 * q.ldb);
    p.C = q.part + (int64_t)blockIdx.y * q.M * q.N;
    p.ldc = q.N;
    p.bias = nullptr;
    p.accumulate = 0;
    p.rowsum = q.rowsum ? q.part_rowsum + (int64_t)blockIdx.y * q.M : nullptr;
  }
  using AOp = FOperand<ALAY, BM>;
  using BOp = FOperand<BLAY, BN>;
  constexpr int STAGE = AOp::BYTES + BOp::BYTES;
  constexpr int TI = BM / 64, TJ = BN / 64;  // 32x32 blocks per wave
  constexpr int WN = BN / 2;                 // columns per wave
  constexpr int PITCH = WN * 4 + 16;
  static_assert(4 * 32 * PITCH <= FSTAGES * STAGE, "epilogue staging exceeds the ring");
  __shared__ __attribute__((aligned(1024))) char lds[FSTAGES * STAGE];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lh = lane >> 5;
  const int tiles_m = (p.M + BM - 1) / BM, tiles_n = (p.N + BN - 1) / BN;
  int tm, tn;
  tile_of(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;

  AOp opA;
  BOp opB;
  opA.init(p.A, p.lda, m0, p.M, p.K, lane, wave);
  opB.init(p.B, p.ldb, n0, p.N, p.K, lane, wave);
  const uint32_t lds0 = lds_addr_of(lds);

  f32x16_t acc[TI][TJ];
#pragma unroll
  for (int i = 0; i < TI; i++)
#pragma unroll
    for (int j = 0; j < TJ; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  // the first column of tiles also sums the rows of A: each lane adds up the k it feeds to the MFMAs
  const bool do_rowsum = p.rowsum != nullptr && tn == 0 && wn == 0;
  float rsum[TI];
#pragma unroll
  for (int i = 0; i < TI; i++) rsum[i] = 0.f;

  const int KT = (p.K + FBK - 1) / FBK;
  auto issue = [&](int kt) {
    const uint32_t st = lds0 + (uint32_t)(kt % FSTAGES) * STAGE;
    opA.issue(st, kt, p.K, wave);
    opB.issue(st + AOp::BYTES, kt, p.K, wave);
  };
  issue(0);
  if (KT > 1) issue(1);
  for (int kt = 0; kt < KT; kt++) {
    // tile kt has landed (tile kt+1 may still be in flight), for every wave; everyone is also done reading
    // the stage tile kt+2 goes into (it held tile kt-1)
    if (kt + 1 < KT)
      __builtin_amdgcn_s_waitcnt(vmcnt_imm(AOp::F_NI + BOp::F_NI));
    else
      __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
    __syncthreads();
    if (kt + 2 < KT) issue(kt + 2);
    const char* st = lds + (kt % FSTAGES) * STAGE;
    float af[TI][8], bf[TJ][8];
#pragma unroll
    for (int i = 0; i < TI; i++) opA.frags(st, wm * (BM / 2) + 32 * i, lane, af[i]);
#pragma unroll
    for (int j = 0; j < TJ; j++) opB.frags(st + AOp::BYTES, wn * WN + 32 * j, lane, bf[j]);
    if (do_rowsum) {
#pragma unroll
      for (int i = 0; i < TI; i++)
#pragma unroll
        for (int s = 0; s < 8; s++) rsum[i] += af[i][s];
    }
#pragma unroll
    for (int s = 0; s < 8; s++)
#pragma unroll
      for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < TJ; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[j][s], af[i][s], acc[i][j], 0, 0, 0);
  }
  __syncthreads();  // the epilogue reuses the ring

  if (do_rowsum) {
#pragma unroll
    for (int i = 0; i < TI; i++) {
      const float t = rsum[i] + __shfl_xor(rsum[i], 32, 64);  // the two k halves of a row
      const int row = m0 + wm * (BM / 2) + 32 * i + l32;
      if (lh == 0 && row < p.M) p.rowsum[row] = p.accumulate ? p.rowsum[row] + t : t;
    }
  }

  // ---- epilogue: D'[n][m]: lane (m = l32, h), register r -> n = 8 (r / 4) + 4 h + r % 4 -----------------
  char* stage = lds + wave * (32 * PITCH);
  const bool inside = m0 + BM <= p.M && n0 + BN <= p.N;
  const bool aligned = ((reinterpret_cast<uintptr_t>(p.C) | (uintptr_t)(p.ldc * 4)) & 15) == 0 &&
                       (!p.bias || (reinterpret_cast<uintptr_t>(p.bias) & 15) == 0);
  constexpr int CPR = WN / 4, RPI = 64 / CPR, ITERS = 32 / RPI;  // 16-byte chunks per staged row; rows per pass
#pragma unroll
  for (int i = 0; i < TI; i++) {
#pragma unroll
    for (int j = 0; j < TJ; j++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const f32x4_t v = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
        *reinterpret_cast<f32x4_t*>(stage + l32 * PITCH + (32 * j + 8 * g + 4 * lh) * 4) = v;
      }
    wave_lds_sync();
    const int mrow0 = m0 + wm * (BM / 2) + 32 * i, ncol0 = n0 + wn * WN;
    const int cc = lane % CPR, r0 = lane / CPR;
    const int col = ncol0 + cc * 4;
    if (inside && aligned) {
      f32x4_t b4 = {0.f, 0.f, 0.f, 0.f};
      if (p.bias) b4 = *reinterpret_cast<const f32x4_t*>(p.bias + col);
#pragma unroll
      for (int it = 0; it < ITERS; it++) {
        const int r = r0 + RPI * it;
        f32x4_t v = *reinterpret_cast<const f32x4_t*>(stage + r * PITCH + cc * 16);
        f32x4_t* q = reinterpret_cast<f32x4_t*>(p.C + (int64_t)(mrow0 + r) * p.ldc + col);
        v += b4;
        if (p.accumulate) v += *q;
        *q = v;
      }
    } else {
      for (int it = 0; it < ITERS; it++) {
        const int r = r0 + RPI * it, row = mrow0 + r;
        if (row >= p.M) continue;
        const float* sp = reinterpret_cast<const float*>(stage + r * PITCH + cc * 16);
        for (int e = 0; e < 4; e++) {
          if (col + e < p.N) {
            float v = sp[e];
            if (p.bias) v += p.bias[col + e];
            float* q = p.C + (int64_t)row * p.ldc + col + e;
            *q = p.accumulate ? *q + v : v;
          }
        }
      }
    }
    wave_lds_sync();
  }
}

// C[m][n] (+)= sum over the slices, in slice order, (+ bias[n]); rowsum likewise.  Four columns per thread.
__global__ __launch_bounds__(256) void f32_slices_sum_kernel(const F32Args p, int S) {
  const int64_t quads = ((int64_t)p.M * p.N) >> 2;   // N % 4 == 0 on this path
  const int64_t slice = (int64_t)p.M * p.N;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < quads; i += (int64_t)gridDim.x * 256) {
    f32x4_t v = *reinterpret_cast<const f32x4_t*>(p.part + 4 * i);
    for (int sl = 1; sl < S; sl++) v += *reinterpret_cast<const f32x4_t*>(p.part + sl * slice + 4 * i);
    const int64_t m = (4 * i) / p.N, n = (4 * i) - m * p.N;
    if (p.bias) v += f32x4_t{p.bias[n], p.bias[n + 1], p.bias[n + 2], p.bias[n + 3]};
    float* c = p.C + m * p.ldc + n;
    if (p.accumulate) v += f32x4_t{c[0], c[1], c[2], c[3]};
    c[0] = v.x; c[1] = v.y; c[2] = v.z; c[3] = v.w;
  }
  if (p.rowsum) {
    for (int64_t m = (int64_t)blockIdx.x * 256 + threadIdx.x; m < p.M; m += (int64_t)gridDim.x * 256) {
      float t = p.part_rowsum[m];
      for (int sl = 1; sl < S; sl++) t += p.part_rowsum[(int64_t)sl * p.M + m];
      p.rowsum[m] = p.accumulate ? p.rowsum[m] + t : t;
    }
  }
}

template <int ALAY, int BLAY, int BM, int BN>
int launch_f32_tile(const F32Args& a, hipStream_t s, int slices = 1) {
  const int tiles = ((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  hipLaunchKernelGGL((gemm_f32_kernel<ALAY, BLAY, BM, BN>), dim3((unsigned)tiles, (unsigned)slices), dim3(256), 0, s, a);
  MTP_CHECK_LAUNCH("gemm_f32");
  if (slices > 1) {
    const int64_t quads = ((int64_t)a.M * a.N) >> 2;
    const unsigned wgs = (unsigned)((quads + 255) / 256 < 2048 ? (quads + 255) / 256 : 2048);
    hipLaunchKernelGGL(f32_slices_sum_kernel, dim3(wgs ? wgs : 1u), dim3(256), 0, s, a, slices);
    MTP_CHECK_LAUNCH("gemm_f32 slices");
  }
  return MTP_OK;
}

// 128x128 unless that leaves CUs idle: three workgroups fit a CU, so below 512 tiles the tile is halved
// along the longer side, and once more if that is still not enough.
// Fewer 128x128 output tiles than CUs and a long k (the weight gradient of an fp32 layer: 3072 x 768 outputs over
// 8192 tokens): with a workspace the 128x128 tiling is kept and k is cut into up to 8 slices of at least 512, one
// workgroup per (tile, slice), until about a thousand workgroups exist; a second kernel adds the slices in slice
// order (bit-reproducible).  Measured on 3072 x 768 x 8192: 441 us as 576 tiles of 64x64 (which read every operand
// element twice as often per flop), 521 / 390 / 340 us with 2 / 4 / 8 slices.
// MTP_GEMM_F32_SLICES = 1 switches the cut off, 2 / 4 / 8 force it.
template <int ALAY, int BLAY>
int launch_f32(F32Args a, hipStream_t s, void* ws, int64_t ws_bytes) {
  auto tiles = [&](int bm, int bn) { return (int64_t)((a.M + bm - 1) / bm) * ((a.N + bn - 1) / bn); };
  static MtpTune tune_tile("MTP_GEMM_F32_TILE"), tune_slices("MTP_GEMM_F32_SLICES");
  const int force = tune_tile.get(0);  // 1..4 picks a tile
  const int want = tune_slices.get(0);
  if (ws && !force && a.N % 4 == 0 && (want > 1 || tiles(128, 128) < 256)) {
    int S = 1;
    while (S < 8 && (want ? S < want : tiles(128, 128) * S < 1024) && a.K / (2 * S) >= 512) S *= 2;
    const int64_t need = (int64_t)S * ((int64_t)a.M * a.N + a.M) * 4;
    if (S > 1 && need <= ws_bytes && want != 1) {
      a.kslice = (((a.K + S - 1) / S) + FBK - 1) / FBK * FBK;   // whole k-tiles per slice
      a.part = static_cast<float*>(ws);
      a.part_rowsum = a.part + (int64_t)S * a.M * a.N;
      return launch_f32_tile<ALAY, BLAY, 128, 128>(a, s, S);
    }
  }
  if (force == 1 || (!force && tiles(128, 128) >= 512)) return launch_f32_tile<ALAY, BLAY, 128, 128>(a, s);
  const bool tall = a.M >= a.N;
  if (force == 2 || force == 3 || (!force && tiles(tall ? 64 : 128, tall ? 128 : 64) >= 512)) {
    if (force == 2 || (!force && tall)) return launch_f32_tile<ALAY, BLAY, 64, 128>(a, s);
    return launch_f32_tile<ALAY, BLAY, 128, 64>(a, s);
  }
  return launch_f32_tile<ALAY, BLAY, 64, 64>(a, s);
}

}  // namespace

// kind 0: C[M,N] = A[M,K] B[N,K]^T (+bias); 1: C[M,N] = A[M,K] B[K,N]; 2: C[M,N] (+)= A[K,M]^T B[K,N] and,
// if rowsum is given, rowsum[m] (+)= sum_k A[k,m]
int mtp_gemm_f32(int kind, const float* A, int64_t lda, const float* B, int64_t ldb, const float* bias, float* C,
                 float* rowsum, int64_t ldc, int64_t M, int64_t N, int64_t K, int accumulate, void* ws, int64_t ws_bytes,
                 hipStream_t s) {
  F32Args a{};
  a.A = A; a.B = B; a.bias = bias; a.C = C; a.rowsum = rowsum;
  a.M = (int)M; a.N = (int)N; a.K = (int)K;
  a.lda = lda; a.ldb = ldb; a.ldc = ldc;
  a.accumulate = accumulate;
  switch (kind) {
    case 0: return launch_f32<LAY_ROW, LAY_ROW>(a, s, ws, ws_bytes);
    case 1: return launch_f32<LAY_ROW, LAY_COL>(a, s, ws, ws_bytes);
    case 2: return launch_f32<LAY_COL, LAY_COL>(a, s, ws, ws_bytes);
  }
  mtp_set_error("gemm_f32: unknown kind %d", kind);
  return MTP_EINVAL;
}
