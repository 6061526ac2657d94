// General GEMM on fp32 MFMA for gfx950: the fp32 path of the linear layers
// (GPT-2-small shaped config) and the catch-all for bf16 problems whose
// shape or alignment the bf16 MFMA kernel does not take (it converts bf16 to
// fp32 on the way into LDS, so it is exact in the products).
//
//   C[m,n] (+)= sum_k A(m,k) * B(n,k) (+ bias[n])
// with arbitrary element strides: A(m,k) = A[m*sam + k*sak], B(n,k) = B[n*sbn + k*sbk].
// forward: A = X (K,1), B = W (K,1); dgrad: A = dY (N,1), B = W (1,K) i.e. B(n=k_in, k=out);
// wgrad: A = dY (1,N), B = X (1,K).
//
// 128x128 tile, BK = 16, 4 waves each owning 64x64 as 2x2 blocks of
// v_mfma_f32_32x32x2_f32.  Both operands sit in LDS k-major ([k][m], m
// contiguous) so the one-float-per-lane fragment reads are conflict free.
// Global loads are staged through registers (next tile is fetched while the
// current one is multiplied).
#include "mtp_common.h"

namespace {

constexpr int GBM = 128, GBN = 128, GBK = 16;
constexpr int GPAD = 32;  // floats; puts the two k rows of one MFMA step on disjoint halves of the banks

struct GenArgs {
  const void* A;
  const void* B;
  void* C;
  const void* bias;
  int M, N, K;
  int64_t sam, sak, sbn, sbk, ldc;
  int accumulate;
};

template <typename T> __device__ __forceinline__ float ld_elem(const T* p);
template <> __device__ __forceinline__ float ld_elem<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ld_elem<uint16_t>(const uint16_t* p) { return bf16_bits_to_f32(*p); }
template <> __device__ __forceinline__ float ld_elem<f16s>(const f16s* p) { return X16<true>::from_bits(p->bits); }
template <typename T> __device__ __forceinline__ void st_elem(T* p, float v);
template <> __device__ __forceinline__ void st_elem<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void st_elem<uint16_t>(uint16_t* p, float v) { *p = f32_to_bf16_bits(v); }
template <> __device__ __forceinline__ void st_elem<f16s>(f16s* p, float v) { p->bits = X16<true>::to_bits(v); }

// Each thread stages 8 elements of the A tile and 8 of the B tile per k-tile:
// tile = 128 rows x 16 k = 2048 elements / 256 threads.
//   k-contiguous operand (stride_k == 1): thread -> (row = t/2, k = 8*(t%2) .. +7)
//   otherwise                            : thread -> (k = t/16, rows = 8*(t%16) .. +7)
template <typename T>
struct Stager {
  float v[8];
  __device__ __forceinline__ void load(const T* base, int64_t s_row, int64_t s_k, int row0, int rows, int k0, int K,
                                       int tid, bool kmajor_mem) {
    if (kmajor_mem) {
      const int r = row0 + (tid >> 1), kb = k0 + 8 * (tid & 1);
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const int k = kb + e;
        v[e] = (r < rows && k < K) ? ld_elem<T>(base + (int64_t)r * s_row + (int64_t)k * s_k) : 0.f;
      }
    } else {
      const int k = k0 + (tid >> 4), rb = row0 + 8 * (tid & 15);
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const int r = rb + e;
        v[e] = (r < rows && k < K) ? ld_elem<T>(base + (int64_t)r * s_row + (int64_t)k * s_k) : 0.f;
      }
    }
  }
  __device__ __forceinline__ void store(float (*tile)[GBM + GPAD], int tid, bool kmajor_mem) const {
    if (kmajor_mem) {
      const int r = tid >> 1, kb = 8 * (tid & 1);
#pragma unroll
      for (int e = 0; e < 8; e++) tile[kb + e][r] = v[e];
    } else {
      const int k = tid >> 4, rb = 8 * (tid & 15);
#pragma unroll
      for (int e = 0; e < 8; e++) tile[k][rb + e] = v[e];
    }
  }
};

template <typename T, typename TO>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const GenArgs p) {
  __shared__ float As[2][GBK][GBM + GPAD];
  __shared__ float Bs[2][GBK][GBN + GPAD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, lh = lane >> 5;
  const int tiles_n = (p.N + GBN - 1) / GBN;
  const int tm = blockIdx.x / tiles_n, tn = blockIdx.x - tm * tiles_n;
  const int m0 = tm * GBM, n0 = tn * GBN;
  const T* A = (const T*)p.A;
  const T* B = (const T*)p.B;
  const bool a_k = p.sak == 1, b_k = p.sbk == 1;

  f32x16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

  Stager<T> sa, sb;
  const int KT = (p.K + GBK - 1) / GBK;
  sa.load(A, p.sam, p.sak, m0, p.M, 0, p.K, tid, a_k);
  sb.load(B, p.sbn, p.sbk, n0, p.N, 0, p.K, tid, b_k);
  sa.store(As[0], tid, a_k);
  sb.store(Bs[0], tid, b_k);
  __syncthreads();
  for (int kt = 0; kt < KT; kt++) {
    const int buf = kt & 1;
    if (kt + 1 < KT) {
      sa.load(A, p.sam, p.sak, m0, p.M, (kt + 1) * GBK, p.K, tid, a_k);
      sb.load(B, p.sbn, p.sbk, n0, p.N, (kt + 1) * GBK, p.K, tid, b_k);
    }
#pragma unroll
    for (int s = 0; s < GBK / 2; s++) {
      float af[2], bf[2];
#pragma unroll
      for (int i = 0; i < 2; i++) af[i] = As[buf][2 * s + lh][wm * 64 + 32 * i + l32];
#pragma unroll
      for (int j = 0; j < 2; j++) bf[j] = Bs[buf][2 * s + lh][wn * 64 + 32 * j + l32];
#pragma unroll
      for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[j], af[i], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < KT) {
      sa.store(As[buf ^ 1], tid, a_k);
      sb.store(Bs[buf ^ 1], tid, b_k);
    }
    __syncthreads();
  }

  // D'[n_local][m_local]: lane (m = l32, h), register r -> n = 8*(r/4) + 4*h + r%4
  TO* C = (TO*)p.C;
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int row = m0 + wm * 64 + 32 * i + l32;
    if (row >= p.M) continue;
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int col = n0 + wn * 64 + 32 * j + 8 * (r >> 2) + 4 * lh + (r & 3);
        if (col < p.N) {
          float v = acc[i][j][r];
          if (p.bias) v += ld_elem<T>((const T*)p.bias + col);
          TO* q = C + (int64_t)row * p.ldc + col;
          if (p.accumulate) v += ld_elem<TO>(q);
          st_elem<TO>(q, v);
        }
      }
  }
}

// db[n] (+)= sum_m dY[m,n]; one workgroup per 64 columns, the 4 waves stride over rows.
template <typename T, typename TO>
__global__ __launch_bounds__(256) void colsum_kernel(const T* __restrict__ dy, TO* __restrict__ db, int M, int N,
                                                     int accumulate) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = blockIdx.x * 64 + lane;
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  if (col < N) {
    int m = wave;
    for (; m + 12 < M; m += 16) {
      s0 += ld_elem<T>(dy + (int64_t)m * N + col);
      s1 += ld_elem<T>(dy + (int64_t)(m + 4) * N + col);
      s2 += ld_elem<T>(dy + (int64_t)(m + 8) * N + col);
      s3 += ld_elem<T>(dy + (int64_t)(m + 12) * N + col);
    }
    for (; m < M; m += 4) s0 += ld_elem<T>(dy + (int64_t)m * N + col);
  }
  __shared__ float part[4][64];
  part[wave][lane] = (s0 + s1) + (s2 + s3);
  __syncthreads();
  if (wave == 0 && col < N) {
    float s = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
    if (accumulate) s += ld_elem<TO>(db + col);
    st_elem<TO>(db + col, s);
  }
}

// act = gelu_new(y) or silu(y[:, :H]) * y[:, H:]  (elementwise forward used behind the generic GEMM)
template <typename T>
__global__ __launch_bounds__(256) void act_fwd_kernel(const T* __restrict__ y, T* __restrict__ act, int64_t M,
                                                      int64_t N, int swiglu) {
  const int64_t W = swiglu ? N / 2 : N;
  const int64_t total = M * W;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int64_t m = i / W, c = i - m * W;
    float r;
    if (swiglu)
      r = silu_f(ld_elem<T>(y + m * N + c)) * ld_elem<T>(y + m * N + W + c);
    else
      r = gelu_new_f(ld_elem<T>(y + i));
    st_elem<T>(act + i, r);
  }
}

template <typename T, typename TO>
int launch_generic(const GenArgs& a, hipStream_t s) {
  const int64_t tiles = (int64_t)((a.M + GBM - 1) / GBM) * ((a.N + GBN - 1) / GBN);
  hipLaunchKernelGGL((gemm_generic_kernel<T, TO>), dim3((unsigned)tiles), dim3(256), 0, s, a);
  MTP_CHECK_LAUNCH("gemm_generic");
  return MTP_OK;
}

}  // namespace

// dtype: MTP_F32, MTP_BF16 or MTP_F16; out_dtype: the same or MTP_F32
int mtp_gemm_generic(const void* A, int64_t sam, int64_t sak, const void* B, int64_t sbn, int64_t sbk,
                     const void* bias, void* C, int64_t ldc, int64_t M, int64_t N, int64_t K, int dtype, int out_dtype,
                     int accumulate, hipStream_t s) {
  GenArgs a{};
  a.A = A; a.B = B; a.C = C; a.bias = bias;
  a.M = (int)M; a.N = (int)N; a.K = (int)K;
  a.sam = sam; a.sak = sak; a.sbn = sbn; a.sbk = sbk; a.ldc = ldc;
  a.accumulate = accumulate;
  if (dtype == MTP_F32 && out_dtype == MTP_F32) return launch_generic<float, float>(a, s);
  if (dtype == MTP_BF16 && out_dtype == MTP_BF16) return launch_generic<uint16_t, uint16_t>(a, s);
  if (dtype == MTP_BF16 && out_dtype == MTP_F32) return launch_generic<uint16_t, float>(a, s);
  if (dtype == MTP_F16 && out_dtype == MTP_F16) return launch_generic<f16s, f16s>(a, s);
  if (dtype == MTP_F16 && out_dtype == MTP_F32) return launch_generic<f16s, float>(a, s);
  mtp_set_error("gemm_generic: dtype %d -> %d not supported", dtype, out_dtype);
  return MTP_EUNSUPPORTED;
}

int mtp_colsum(const void* dy, void* db, int64_t M, int64_t N, int dtype, int out_dtype, int accumulate,
               hipStream_t s) {
  const unsigned blocks = (unsigned)((N + 63) / 64);
  if (dtype == MTP_F32 && out_dtype == MTP_F32)
    hipLaunchKernelGGL((colsum_kernel<float, float>), dim3(blocks), dim3(256), 0, s, (const float*)dy, (float*)db,
                       (int)M, (int)N, accumulate);
  else if (dtype == MTP_BF16 && out_dtype == MTP_BF16)
    hipLaunchKernelGGL((colsum_kernel<uint16_t, uint16_t>), dim3(blocks), dim3(256), 0, s, (const uint16_t*)dy,
                       (uint16_t*)db, (int)M, (int)N, accumulate);
  else if (dtype == MTP_F16 && out_dtype == MTP_F16)
    hipLaunchKernelGGL((colsum_kernel<f16s, f16s>), dim3(blocks), dim3(256), 0, s, (const f16s*)dy, (f16s*)db, (int)M,
                       (int)N, accumulate);
  else if (dtype == MTP_F16 && out_dtype == MTP_F32)
    hipLaunchKernelGGL((colsum_kernel<f16s, float>), dim3(blocks), dim3(256), 0, s, (const f16s*)dy, (float*)db, (int)M,
                       (int)N, accumulate);
  else if (dtype == MTP_BF16 && out_dtype == MTP_F32)
    hipLaunchKernelGGL((colsum_kernel<uint16_t, float>), dim3(blocks), dim3(256), 0, s, (const uint16_t*)dy,
                       (float*)db, (int)M, (int)N, accumulate);
  else {
    mtp_set_error("colsum: dtype %d -> %d not supported", dtype, out_dtype);
    return MTP_EUNSUPPORTED;
  }
  MTP_CHECK_LAUNCH("colsum");
  return MTP_OK;
}

int mtp_act_fwd(const void* y, void* act, int64_t M, int64_t N, int dtype, int swiglu, hipStream_t s) {
  const int64_t total = M * (swiglu ? N / 2 : N);
  int64_t blocks = (total + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  if (blocks < 1) blocks = 1;
  if (dtype == MTP_F32)
    hipLaunchKernelGGL(act_fwd_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, s, (const float*)y, (float*)act,
                       M, N, swiglu);
  else if (dtype == MTP_F16)
    hipLaunchKernelGGL(act_fwd_kernel<f16s>, dim3((unsigned)blocks), dim3(256), 0, s, (const f16s*)y, (f16s*)act, M, N,
                       swiglu);
  else
    hipLaunchKernelGGL(act_fwd_kernel<uint16_t>, dim3((unsigned)blocks), dim3(256), 0, s, (const uint16_t*)y,
                       (uint16_t*)act, M, N, swiglu);
  MTP_CHECK_LAUNCH("act_fwd");
  return MTP_OK;
}
