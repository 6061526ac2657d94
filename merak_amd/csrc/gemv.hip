// Decode-step GEMV for gfx950: Y[B,N] = X[B,K] W[N,K]^T with B <= 32 rows of
// single-token activations, bf16 in / fp32 accumulate, and a variant that
// reduces the LM-head row straight to (max, argmax) without ever writing the
// logits (Merak/inference/text_generation_inference.py:223,226-227).
//
// The weight matrix is streamed from HBM exactly once.  It feeds the A operand
// of v_mfma_f32_16x16x32_bf16 directly from global memory: lane (i = l%16,
// g = l/16) loads the 16 bytes W[row0+i][k0+8g .. k0+8g+7], so four lanes
// cover 64 contiguous bytes of a weight row and consecutive k-steps walk
// along it.  The B operand is X^T (lane (b = l%16, g) loads X[b][k0+8g..]);
// X is tiny and stays in L2/L1.  The result tile D[i][b] needs no cross-lane
// reduction.
//
// A workgroup of 8 waves owns 16*R weight rows; the 128-byte k-pairs of those
// rows are dealt round-robin to the waves (split-K inside the workgroup), the 8
// partial tiles are summed through LDS in a fixed order, so results are
// bit-reproducible run to run.
#include "mtp_common.h"
#include <stdlib.h>

namespace {

constexpr int GV_WAVES = 8;
constexpr int GV_THREADS = GV_WAVES * MTP_WAVE;

struct ArgPart {
  float v;
  int32_t i;
};

// torch.argmax ordering: NaN beats everything, ties go to the lower index
__device__ __forceinline__ bool arg_better(float va, int64_t ia, float vb, int64_t ib) {
  const bool na = va != va, nb = vb != vb;
  if (na != nb) return na;
  if (na) return ia < ib;
  return va > vb || (va == vb && ia < ib);
}

// `ok` is a compile-time true on the unguarded path, which then has no branches at all
__device__ __forceinline__ bf16x8_t load_frag(const uint16_t* p, bool ok) {
  u32x4_t v = {0u, 0u, 0u, 0u};
  if (ok) v = *reinterpret_cast<const u32x4_t*>(p);
  return __builtin_bit_cast(bf16x8_t, v);
}

// weights are read exactly once: streaming (non-temporal) loads keep them from displacing X in the caches
__device__ __forceinline__ bf16x8_t load_frag_nt(const uint16_t* p, bool ok) {
  u32x4_t v = {0u, 0u, 0u, 0u};
  if (ok) v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
  return __builtin_bit_cast(bf16x8_t, v);
}

// MODE 0: store Y (+bias); MODE 1: SwiGLU store; MODE 2: argmax partials
template <int R, int NB, int MODE, bool GUARD>
__global__ __launch_bounds__(GV_THREADS) void gemv_kernel(const uint16_t* __restrict__ x,
                                                          const uint16_t* __restrict__ w,
                                                          const uint16_t* __restrict__ bias,
                                                          uint16_t* __restrict__ y, ArgPart* __restrict__ part,
                                                          int B, int64_t N, int64_t K) {
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int li = lane & 15;  // weight row inside a 16-row group / batch column
  const int lg = lane >> 4;  // 8-element k group

  // rows of the R groups owned by this workgroup
  const int64_t half = N >> 1;  // SwiGLU: W = [gate rows | up rows]
  int64_t grow[R];
#pragma unroll
  for (int r = 0; r < R; r++) {
    int64_t row;
    if (MODE == 1) {
      const int64_t j0 = (int64_t)blockIdx.x * (8 * R);
      row = (r < R / 2) ? j0 + 16 * r + li : half + j0 + 16 * (r - R / 2) + li;
      const int64_t lim = (r < R / 2) ? half : N;
      if (row >= lim) row = lim - 1;
    } else {
      row = (int64_t)blockIdx.x * (16 * R) + 16 * r + li;
      if (row >= N) row = N - 1;
    }
    grow[r] = row;
  }
  const uint16_t* wp[R];
#pragma unroll
  for (int r = 0; r < R; r++) wp[r] = w + grow[r] * K + 8 * lg;
  const uint16_t* xp[NB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    int b = li + 16 * nb;
    if (b >= B) b = B - 1;
    xp[nb] = x + (int64_t)b * K + 8 * lg;
  }

  // This wave's k range, in pairs of 32-element steps: a pair covers 64 elements = one 128-byte line of
  // every weight row, and the two 64-byte halves of a line are requested by adjacent instructions, so the
  // second request merges with the first one's miss instead of finding the line evicted again (with 16
  // rows x 8 groups x 8 waves in flight the L1 holds nothing for long).
  // Pairs are dealt round-robin to the 8 waves (wave w takes pairs w, w+8, ...): the waves advance in
  // step, so at any moment the workgroup reads 1 KiB contiguous from each of its rows, which keeps
  // DRAM pages open much longer than eight far-apart 128-byte streams per row would.
  const int64_t pairs = (K + 63) >> 6;
  const int64_t p0 = wave;
  const int64_t p1 = pairs;

  f32x4_t acc[R][NB];
#pragma unroll
  for (int r = 0; r < R; r++)
#pragma unroll
    for (int nb = 0; nb < NB; nb++) acc[r][nb] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  if (p0 < p1) {
    bf16x8_t a_cur[R][2], b_cur[NB][2];
    // GUARD: K is not a multiple of 64, the last pair is partly (or half) past the end of the rows
    auto load_pair = [&](int64_t pr, bf16x8_t (&a)[R][2], bf16x8_t (&b)[NB][2]) {
      const int64_t k = pr * 64;
#pragma unroll
      for (int r = 0; r < R; r++)
#pragma unroll
        for (int hf = 0; hf < 2; hf++) a[r][hf] = load_frag_nt(wp[r] + k + 32 * hf, !GUARD || (k + 32 * hf + 8 * lg < K));
#pragma unroll
      for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int hf = 0; hf < 2; hf++) b[nb][hf] = load_frag(xp[nb] + k + 32 * hf, !GUARD || (k + 32 * hf + 8 * lg < K));
    };
    auto multiply = [&]() {
#pragma unroll
      for (int hf = 0; hf < 2; hf++)
#pragma unroll
        for (int r = 0; r < R; r++)
#pragma unroll
          for (int nb = 0; nb < NB; nb++)
            acc[r][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_cur[r][hf], b_cur[nb][hf], acc[r][nb], 0, 0, 0);
    };
    load_pair(p0, a_cur, b_cur);
    // all but the last pair: fetch the next pair (unconditionally: it exists), multiply the current one
    int64_t pr = p0;
    for (; pr + GV_WAVES < p1; pr += GV_WAVES) {
      bf16x8_t a_nxt[R][2], b_nxt[NB][2];
      load_pair(pr + GV_WAVES, a_nxt, b_nxt);
      multiply();
#pragma unroll
      for (int r = 0; r < R; r++)
#pragma unroll
        for (int hf = 0; hf < 2; hf++) a_cur[r][hf] = a_nxt[r][hf];
#pragma unroll
      for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int hf = 0; hf < 2; hf++) b_cur[nb][hf] = b_nxt[nb][hf];
    }
    multiply();
  }

  // ---- sum the 8 k-slices through LDS, one row group at a time -------------
  // part_lds[w][nb][j][lane]; fin[b][local row]
  __shared__ float part_lds[GV_WAVES][NB][4][64];
  __shared__ float fin[16 * NB][16 * R + 1];
#pragma unroll
  for (int r = 0; r < R; r++) {
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
      for (int j = 0; j < 4; j++) part_lds[wave][nb][j][lane] = acc[r][nb][j];
    __syncthreads();
    for (int e = tid; e < NB * 256; e += GV_THREADS) {
      const int nb = e >> 8, j = (e >> 6) & 3, l = e & 63;
      float s = 0.f;
#pragma unroll
      for (int wv = 0; wv < GV_WAVES; wv++) s += part_lds[wv][nb][j][l];
      // D[i][b]: lane l, register j holds row i = 4*(l/16)+j, column b = l%16
      fin[(l & 15) + 16 * nb][16 * r + 4 * (l >> 4) + j] = s;
    }
    __syncthreads();
  }

  if (MODE == 0) {
    const int64_t n0 = (int64_t)blockIdx.x * (16 * R);
    for (int e = tid; e < B * 16 * R; e += GV_THREADS) {
      const int b = e / (16 * R), rl = e - b * (16 * R);
      const int64_t n = n0 + rl;
      if (n < N) {
        float v = fin[b][rl];
        if (bias) v += bf16_bits_to_f32(bias[n]);
        y[(int64_t)b * N + n] = f32_to_bf16_bits(v);
      }
    }
  } else if (MODE == 1) {
    const int64_t j0 = (int64_t)blockIdx.x * (8 * R);
    for (int e = tid; e < B * 8 * R; e += GV_THREADS) {
      const int b = e / (8 * R), rl = e - b * (8 * R);
      const int64_t jn = j0 + rl;
      if (jn < half) {
        float gate = fin[b][rl], up = fin[b][8 * R + rl];
        if (bias) {
          gate += bf16_bits_to_f32(bias[jn]);
          up += bf16_bits_to_f32(bias[half + jn]);
        }
        // round the pre-activations to bf16 first, as the unfused layer stack would
        gate = bf16_bits_to_f32(f32_to_bf16_bits(gate));
        up = bf16_bits_to_f32(f32_to_bf16_bits(up));
        y[(int64_t)b * half + jn] = f32_to_bf16_bits(silu_f(gate) * up);
      }
    }
  } else {
    const int64_t n0 = (int64_t)blockIdx.x * (16 * R);
    for (int b = wave; b < B; b += GV_WAVES) {
      float bv = 0.f;
      int64_t bi = INT64_MAX;
      bool have = false;
      for (int rl = lane; rl < 16 * R; rl += 64) {
        const int64_t n = n0 + rl;
        if (n < N) {
          const float v = fin[b][rl];
          if (!have || arg_better(v, n, bv, bi)) {
            bv = v;
            bi = n;
            have = true;
          }
        }
      }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, 64);
        const int64_t oi = __shfl_xor(bi, o, 64);
        const int oh = __shfl_xor((int)have, o, 64);
        if (oh && (!have || arg_better(ov, oi, bv, bi))) {
          bv = ov;
          bi = oi;
          have = true;
        }
      }
      if (lane == 0) part[(int64_t)blockIdx.x * B + b] = ArgPart{bv, (int32_t)bi};
    }
  }
}

__global__ __launch_bounds__(256) void argmax_finish_kernel(const ArgPart* __restrict__ part, int n_part, int B,
                                                            int64_t* __restrict__ idx, float* __restrict__ maxval) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int b = wave; b < B; b += 4) {
    float bv = 0.f;
    int64_t bi = INT64_MAX;
    bool have = false;
    for (int p = lane; p < n_part; p += 64) {
      const ArgPart a = part[(int64_t)p * B + b];
      if (!have || arg_better(a.v, a.i, bv, bi)) {
        bv = a.v;
        bi = a.i;
        have = true;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int64_t oi = __shfl_xor(bi, o, 64);
      const int oh = __shfl_xor((int)have, o, 64);
      if (oh && (!have || arg_better(ov, oi, bv, bi))) {
        bv = ov;
        bi = oi;
        have = true;
      }
    }
    if (lane == 0) {
      idx[b] = bi;
      if (maxval) maxval[b] = bv;
    }
  }
}

// Row-wise argmax over materialised logits: one workgroup per row.
template <typename T>
__global__ __launch_bounds__(256) void argmax_rows_kernel(const T* __restrict__ logits, int64_t* __restrict__ idx,
                                                          int64_t V) {
  const T* rp = logits + (int64_t)blockIdx.x * V;
  float bv = 0.f;
  int64_t bi = INT64_MAX;
  bool have = false;
  for (int64_t j = threadIdx.x; j < V; j += 256) {
    float v;
    if constexpr (sizeof(T) == 2)
      v = bf16_bits_to_f32(rp[j]);
    else
      v = rp[j];
    if (!have || arg_better(v, j, bv, bi)) {
      bv = v;
      bi = j;
      have = true;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, 64);
    const int64_t oi = __shfl_xor(bi, o, 64);
    const int oh = __shfl_xor((int)have, o, 64);
    if (oh && (!have || arg_better(ov, oi, bv, bi))) {
      bv = ov;
      bi = oi;
      have = true;
    }
  }
  __shared__ float sv[4];
  __shared__ int64_t si[4];
  __shared__ int sh[4];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) {
    sv[wave] = bv;
    si[wave] = bi;
    sh[wave] = have;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int wv = 1; wv < 4; wv++)
      if (sh[wv] && (!have || arg_better(sv[wv], si[wv], bv, bi))) {
        bv = sv[wv];
        bi = si[wv];
        have = true;
      }
    idx[blockIdx.x] = bi;
  }
}

int pick_rows_per_wg(int64_t B, int64_t N, int64_t K, int mode) {
  const char* e = getenv("MTP_GEMV_R");
  if (e) {
    const int r = atoi(e);
    if (r == 1 || r == 2 || r == 4 || r == 8) return (mode == 1 && r == 1) ? 2 : r;
  }
  // Aim for at least ~2 workgroups per CU (256 CUs); more rows per workgroup
  // means fewer re-reads of X from L2.
  const int64_t groups = (N + 15) / 16;
  // Measured on the 128256 x 4096 LM head: 4 groups for B <= 16 (2 workgroups per CU), 8 for larger
  // batches (fewer re-reads of X); small matrices want at least ~2 workgroups per CU.
  int r = B > 16 ? 8 : 4;
  while (r > 1 && groups / r < 512) r >>= 1;
  if (mode == 1 && r < 2) r = 2;
  (void)K;
  return r;
}

template <int MODE>
int launch_gemv(const void* x, const void* w, const void* bias, void* y, ArgPart* part, int64_t B, int64_t N,
                int64_t K, int R, hipStream_t s, unsigned* n_wg_out) {
  const int64_t rows_per_wg = (MODE == 1) ? 8 * R : 16 * R;
  const int64_t span = (MODE == 1) ? N / 2 : N;
  const unsigned n_wg = (unsigned)((span + rows_per_wg - 1) / rows_per_wg);
  if (n_wg_out) *n_wg_out = n_wg;
  const int NB = B > 16 ? 2 : 1;
#define GV_LAUNCH(RR, NNB)                                                                                      \
  do {                                                                                                          \
    if (K % 64 == 0)                                                                                            \
      hipLaunchKernelGGL((gemv_kernel<RR, NNB, MODE, false>), dim3(n_wg), dim3(GV_THREADS), 0, s,               \
                         (const uint16_t*)x, (const uint16_t*)w, (const uint16_t*)bias, (uint16_t*)y, part,     \
                         (int)B, N, K);                                                                         \
    else                                                                                                        \
      hipLaunchKernelGGL((gemv_kernel<RR, NNB, MODE, true>), dim3(n_wg), dim3(GV_THREADS), 0, s,                \
                         (const uint16_t*)x, (const uint16_t*)w, (const uint16_t*)bias, (uint16_t*)y, part,     \
                         (int)B, N, K);                                                                         \
  } while (0)
  if (NB == 1) {
    if (R == 8) GV_LAUNCH(8, 1);
    else if (R == 4) GV_LAUNCH(4, 1);
    else if (R == 2) GV_LAUNCH(2, 1);
    else if constexpr (MODE != 1) GV_LAUNCH(1, 1);
  } else {
    if (R == 8) GV_LAUNCH(8, 2);
    else if (R == 4) GV_LAUNCH(4, 2);
    else if (R == 2) GV_LAUNCH(2, 2);
    else if constexpr (MODE != 1) GV_LAUNCH(1, 2);
  }
#undef GV_LAUNCH
  MTP_CHECK_LAUNCH("gemv");
  return MTP_OK;
}

int check_gemv_args(const char* what, const void* x, const void* w, int64_t B, int64_t N, int64_t K) {
  MTP_REQUIRE(B >= 1 && B <= 32, MTP_EUNSUPPORTED, "%s: B=%lld outside [1,32]", what, (long long)B);
  MTP_REQUIRE(N >= 1 && K >= 1, MTP_EINVAL, "%s: N=%lld K=%lld", what, (long long)N, (long long)K);
  MTP_REQUIRE(N < (1ll << 31), MTP_EUNSUPPORTED, "%s: N=%lld exceeds 2^31-1", what, (long long)N);
  MTP_REQUIRE(K % 8 == 0, MTP_EUNSUPPORTED, "%s: K=%lld is not a multiple of 8", what, (long long)K);
  MTP_REQUIRE(x && w, MTP_EINVAL, "%s: null pointer", what);
  MTP_REQUIRE(((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15) == 0, MTP_EUNSUPPORTED,
              "%s: x and w must be 16-byte aligned", what);
  return MTP_OK;
}

}  // namespace

extern "C" int mtp_gemv(const void* x, const void* w, const void* bias, void* y, int64_t B, int64_t N, int64_t K,
                        int epilogue, void* stream) {
  int rc = check_gemv_args("gemv", x, w, B, N, K);
  if (rc) return rc;
  MTP_REQUIRE(y, MTP_EINVAL, "gemv: null output");
  MTP_REQUIRE(epilogue == MTP_EPI_NONE || epilogue == MTP_EPI_BIAS || epilogue == MTP_EPI_SWIGLU, MTP_EINVAL,
              "gemv: epilogue %d not supported", epilogue);
  MTP_REQUIRE(epilogue != MTP_EPI_BIAS || bias, MTP_EINVAL, "gemv: MTP_EPI_BIAS without bias");
  hipStream_t s = (hipStream_t)stream;
  if (epilogue == MTP_EPI_SWIGLU) {
    MTP_REQUIRE(N % 2 == 0, MTP_EINVAL, "gemv: SwiGLU needs an even N, got %lld", (long long)N);
    const int R = pick_rows_per_wg(B, N, K, 1);
    return launch_gemv<1>(x, w, bias, y, nullptr, B, N, K, R, s, nullptr);
  }
  const int R = pick_rows_per_wg(B, N, K, 0);
  return launch_gemv<0>(x, w, epilogue == MTP_EPI_NONE ? nullptr : bias, y, nullptr, B, N, K, R, s, nullptr);
}

extern "C" int64_t mtp_gemv_argmax_workspace_bytes(int64_t B, int64_t N, int64_t K) {
  (void)K;
  if (B < 1 || N < 1) return 0;
  // one partial per (workgroup, batch row); the smallest workgroup owns 16 rows
  return ((N + 15) / 16) * B * (int64_t)sizeof(ArgPart);
}

extern "C" int mtp_gemv_argmax(const void* x, const void* w, int64_t* idx, float* maxval, void* workspace,
                               int64_t workspace_bytes, int64_t B, int64_t N, int64_t K, void* stream) {
  int rc = check_gemv_args("gemv_argmax", x, w, B, N, K);
  if (rc) return rc;
  MTP_REQUIRE(idx && workspace, MTP_EINVAL, "gemv_argmax: null pointer");
  MTP_REQUIRE(workspace_bytes >= mtp_gemv_argmax_workspace_bytes(B, N, K), MTP_EWORKSPACE,
              "gemv_argmax: workspace %lld < %lld bytes", (long long)workspace_bytes,
              (long long)mtp_gemv_argmax_workspace_bytes(B, N, K));
  MTP_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 7) == 0, MTP_EINVAL, "gemv_argmax: workspace not 8-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const int R = pick_rows_per_wg(B, N, K, 2);
  unsigned n_wg = 0;
  rc = launch_gemv<2>(x, w, nullptr, nullptr, (ArgPart*)workspace, B, N, K, R, s, &n_wg);
  if (rc) return rc;
  hipLaunchKernelGGL(argmax_finish_kernel, dim3(1), dim3(256), 0, s, (const ArgPart*)workspace, (int)n_wg, (int)B,
                     idx, maxval);
  MTP_CHECK_LAUNCH("argmax_finish");
  return MTP_OK;
}

extern "C" int mtp_argmax_rows(const void* logits, int64_t* idx, int64_t B, int64_t V, int dtype, void* stream) {
  MTP_REQUIRE(B >= 0 && V >= 1, MTP_EINVAL, "argmax_rows: B=%lld V=%lld", (long long)B, (long long)V);
  MTP_REQUIRE(B < (1ll << 31), MTP_EUNSUPPORTED, "argmax_rows: B too large");
  if (B == 0) return MTP_OK;
  MTP_REQUIRE(logits && idx, MTP_EINVAL, "argmax_rows: null pointer");
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MTP_F32)
    hipLaunchKernelGGL(argmax_rows_kernel<float>, dim3((unsigned)B), dim3(256), 0, s, (const float*)logits, idx, V);
  else if (dtype == MTP_BF16)
    hipLaunchKernelGGL(argmax_rows_kernel<uint16_t>, dim3((unsigned)B), dim3(256), 0, s, (const uint16_t*)logits,
                       idx, V);
  else
    MTP_REQUIRE(false, MTP_EINVAL, "argmax_rows: unknown dtype %d", dtype);
  MTP_CHECK_LAUNCH("argmax_rows");
  return MTP_OK;
}
