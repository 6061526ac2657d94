// Bandwidth-bound helpers around the GEMMs: backward of the fused
// activations, the bias gradient (column sum of dY), and two measurement
// kernels (streaming copy, register-resident MFMA loop).
#include "mtp_common.h"

namespace {

// ---- activation backward ---------------------------------------------------
// T = float, uint16_t (bf16 bits) or f16s (IEEE half bits); one thread handles one 16-byte vector.
template <typename T> struct Io;
template <> struct Io<float> {
  static constexpr int EPV = 4;
  __device__ static __forceinline__ void unpack(const u32x4_t& v, float* f) {
    f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y);
    f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
  }
  __device__ static __forceinline__ u32x4_t pack(const float* f) {
    return u32x4_t{__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3])};
  }
  __device__ static __forceinline__ float ld(const float* p) { return *p; }
  __device__ static __forceinline__ void st(float* p, float v) { *p = v; }
};
template <> struct Io<uint16_t> {
  static constexpr int EPV = 8;
  __device__ static __forceinline__ void unpack(const u32x4_t& v, float* f) {
    f[0] = bf16_lo(v.x); f[1] = bf16_hi(v.x); f[2] = bf16_lo(v.y); f[3] = bf16_hi(v.y);
    f[4] = bf16_lo(v.z); f[5] = bf16_hi(v.z); f[6] = bf16_lo(v.w); f[7] = bf16_hi(v.w);
  }
  __device__ static __forceinline__ u32x4_t pack(const float* f) {
    return u32x4_t{pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
                   pack_bf16x2(f[6], f[7])};
  }
  __device__ static __forceinline__ float ld(const uint16_t* p) { return bf16_bits_to_f32(*p); }
  __device__ static __forceinline__ void st(uint16_t* p, float v) { *p = f32_to_bf16_bits(v); }
};

template <> struct Io<f16s> {
  static constexpr int EPV = 8;
  using H = X16<true>;
  __device__ static __forceinline__ void unpack(const u32x4_t& v, float* f) {
    f[0] = H::lo(v.x); f[1] = H::hi(v.x); f[2] = H::lo(v.y); f[3] = H::hi(v.y);
    f[4] = H::lo(v.z); f[5] = H::hi(v.z); f[6] = H::lo(v.w); f[7] = H::hi(v.w);
  }
  __device__ static __forceinline__ u32x4_t pack(const float* f) {
    return u32x4_t{H::pack2(f[0], f[1]), H::pack2(f[2], f[3]), H::pack2(f[4], f[5]), H::pack2(f[6], f[7])};
  }
  __device__ static __forceinline__ float ld(const f16s* p) { return H::from_bits(p->bits); }
  __device__ static __forceinline__ void st(f16s* p, float v) { p->bits = H::to_bits(v); }
};

template <typename T>
__global__ __launch_bounds__(256) void gelu_bwd_kernel(const T* __restrict__ dact, const T* __restrict__ y,
                                                       T* __restrict__ dy, int64_t n) {
  constexpr int EPV = Io<T>::EPV;
  const int64_t nvec = n / EPV;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  const int64_t t0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (int64_t i = t0; i < nvec; i += stride) {
    u32x4_t a = reinterpret_cast<const u32x4_t*>(dact)[i];
    u32x4_t b = reinterpret_cast<const u32x4_t*>(y)[i];
    float fa[EPV], fb[EPV];
    Io<T>::unpack(a, fa);
    Io<T>::unpack(b, fb);
#pragma unroll
    for (int e = 0; e < EPV; e++) fa[e] *= gelu_new_grad_f(fb[e]);
    reinterpret_cast<u32x4_t*>(dy)[i] = Io<T>::pack(fa);
  }
  for (int64_t j = nvec * EPV + t0; j < n; j += stride) Io<T>::st(dy + j, Io<T>::ld(dact + j) * gelu_new_grad_f(Io<T>::ld(y + j)));
}

// y = [gate | up] of width N = 2H per row; dact has width H.
//   dgate = dact * up * silu'(gate),  dup = dact * silu(gate)
// VEC: rows are 16-byte aligned and H % EPV == 0.
// blockIdx.x picks 256 vectors of a row, blockIdx.y the rows (stride gridDim.y): no index arithmetic beyond
// additions, and two rows per step so that six loads per thread are on their way before the first is used.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const T* __restrict__ dact, const T* __restrict__ y,
                                                         T* __restrict__ dy, int64_t M, int64_t H) {
  constexpr int EPV = VEC ? Io<T>::EPV : 1;
  const int64_t c = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * EPV;   // first column of this thread
  if (c >= H) return;
  struct Row {
    float g[EPV], u[EPV], d[EPV];
  };
  auto load = [&](int64_t m, Row& r) {
    const T* pg = y + m * 2 * H + c;
    if constexpr (VEC) {
      // read once, by this kernel only: streaming loads
      const u32x4_t vg = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(pg));
      const u32x4_t vu = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(pg + H));
      const u32x4_t vd = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(dact + m * H + c));
      Io<T>::unpack(vg, r.g);
      Io<T>::unpack(vu, r.u);
      Io<T>::unpack(vd, r.d);
    } else {
      r.g[0] = Io<T>::ld(pg); r.u[0] = Io<T>::ld(pg + H); r.d[0] = Io<T>::ld(dact + m * H + c);
    }
  };
  auto finish = [&](int64_t m, const Row& r) {
    float rg[EPV], ru[EPV];
#pragma unroll
    for (int e = 0; e < EPV; e++) {
      const float s = sigmoid_f(r.g[e]);
      const float silu = r.g[e] * s;
      rg[e] = r.d[e] * r.u[e] * (s + silu * (1.0f - s));
      ru[e] = r.d[e] * silu;
    }
    T* og = dy + m * 2 * H + c;
    if constexpr (VEC) {
      *reinterpret_cast<u32x4_t*>(og) = Io<T>::pack(rg);
      *reinterpret_cast<u32x4_t*>(og + H) = Io<T>::pack(ru);
    } else {
      Io<T>::st(og, rg[0]); Io<T>::st(og + H, ru[0]);
    }
  };
  const int64_t step = gridDim.y;
  int64_t m = blockIdx.y;
  for (; m + step < M; m += 2 * step) {
    Row r0, r1;
    load(m, r0);
    load(m + step, r1);
    finish(m, r0);
    finish(m + step, r1);
  }
  if (m < M) {
    Row r0;
    load(m, r0);
    finish(m, r0);
  }
}

// ---- measurement -------------------------------------------------------------
__global__ __launch_bounds__(256) void stream_copy_kernel(const u32x4_t* __restrict__ src, u32x4_t* __restrict__ dst,
                                                          int64_t nvec) {
  // Workgroup b copies the 16 KiB pieces b, b + grid, ...: four vectors per lane, 4 KiB apart.  Contiguous
  // pieces per workgroup move 5.6-5.8 TB/s (read + write) on an MI355X; the same loop with the four vectors a
  // whole grid apart (every workgroup touching four far-apart 4 KiB pieces per step) moves 4.3-5.1 TB/s.
  constexpr int U = 4;
  const int64_t pieces = nvec / (256 * U);
  for (int64_t c = blockIdx.x; c < pieces; c += gridDim.x) {
    const int64_t i = c * (256 * U) + threadIdx.x;
    u32x4_t v[U];
#pragma unroll
    for (int u = 0; u < U; u++) v[u] = __builtin_nontemporal_load(src + i + u * 256);
#pragma unroll
    for (int u = 0; u < U; u++) __builtin_nontemporal_store(v[u], dst + i + u * 256);
  }
  // what is left of the last piece
  for (int64_t i = pieces * (256 * U) + (int64_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * 256)
    __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

// Register-resident MFMA loop.  What the matrix cores sustain depends on the operand bits, because the chip
// runs against a power limit: `random_data` fills the four A and four B fragments with pseudo-random
// mantissas and signs (exponents near 1.0, like N(0,1) activations); otherwise they hold small smooth
// values that toggle few wires.  Fragments rotate so that consecutive MFMAs see different operands.
__global__ __launch_bounds__(256) void mfma_peak_kernel(float* __restrict__ sink, int64_t iters, int random_data) {
  const int lane = threadIdx.x & 63;
  bf16x8_t a[4], b[4];
  uint32_t rng = 0x9e3779b9u * (uint32_t)(blockIdx.x * 256 + threadIdx.x + 1);
#pragma unroll
  for (int f = 0; f < 4; f++) {
    u32x4_t ra, rb;
    uint32_t* pa = reinterpret_cast<uint32_t*>(&ra);
    uint32_t* pb = reinterpret_cast<uint32_t*>(&rb);
#pragma unroll
    for (int q = 0; q < 4; q++) {
      if (random_data) {
        // two bf16 per word: sign and 7 mantissa bits random, exponent 0x7e..0x7f (values in +-[0.5, 2))
        rng ^= rng << 13; rng ^= rng >> 17; rng ^= rng << 5;
        pa[q] = (rng & 0x80ff80ffu) | 0x3f003f00u;
        rng ^= rng << 13; rng ^= rng >> 17; rng ^= rng << 5;
        pb[q] = (rng & 0x80ff80ffu) | 0x3f003f00u;
      } else {
        pa[q] = pack_bf16x2(0.001f * (lane + 2 * q + f), 0.001f * (lane + 2 * q + 1 + f));
        pb[q] = pack_bf16x2(0.002f * (lane - 2 * q - f), 0.002f * (lane - 2 * q - 1 - f));
      }
    }
    a[f] = __builtin_bit_cast(bf16x8_t, ra);
    b[f] = __builtin_bit_cast(bf16x8_t, rb);
  }
  f32x16_t c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
  for (int64_t it = 0; it < iters; it += 16) {
#pragma unroll
    for (int f = 0; f < 4; f++) {
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[f], b[f], c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[f], b[(f + 1) & 3], c1, 0, 0, 0);
      c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[f], b[(f + 2) & 3], c2, 0, 0, 0);
      c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[f], b[(f + 3) & 3], c3, 0, 0, 0);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; i++) s += c0[i] + c1[i] + c2[i] + c3[i];
  sink[(int64_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}

// The same measurement for the instruction stream of the 64-deep GEMM loop: v_mfma_f32_16x16x32_bf16 on 64
// accumulator quads (the whole accumulator file), operands from 32 register-resident fragments (two units of four
// 16-row blocks of A and of B, two k steps each) walked quadrant by quadrant as the GEMM walks a k-tile: 128 MFMAs
// per pass, no LDS reads, no memory traffic, no barriers.  One wave per SIMD, like the GEMM.  What this loop
// sustains is the ceiling of the GEMM's main loop on this board at its power limit.
__device__ __forceinline__ void mfma_gemm_loop_body(float* __restrict__ sink, int64_t iters, int random_data) {
  const int lane = threadIdx.x & 63;
  bf16x8_t ra[2][4][2], rb[2][4][2];
  uint32_t rng = 0x9e3779b9u * (uint32_t)(blockIdx.x * 256 + threadIdx.x + 1);
#pragma unroll
  for (int f = 0; f < 32; f++) {
    u32x4_t v;
    uint32_t* pv = reinterpret_cast<uint32_t*>(&v);
#pragma unroll
    for (int q = 0; q < 4; q++) {
      if (random_data) {
        rng ^= rng << 13; rng ^= rng >> 17; rng ^= rng << 5;
        pv[q] = (rng & 0x80ff80ffu) | 0x3f003f00u;      // sign and mantissa random, values in +-[0.5, 2)
      } else {
        pv[q] = pack_bf16x2(0.001f * (lane + 2 * q + f), 0.001f * (lane + 2 * q + 1 + f));
      }
    }
    if (f < 16) ra[f >> 3][(f >> 1) & 3][f & 1] = __builtin_bit_cast(bf16x8_t, v);
    else rb[(f >> 3) & 1][(f >> 1) & 3][f & 1] = __builtin_bit_cast(bf16x8_t, v);
  }
  f32x4_t acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j < 8; j++) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  for (int64_t it = 0; it < iters; it += 128) {
#pragma unroll
    for (int qd = 0; qd < 4; qd++) {          // Q00 Q01 Q11 Q10: consecutive quadrants share a unit
      const int MA = qd >> 1, MB = (qd & 1) ^ MA;
#pragma unroll
      for (int kk = 0; kk < 2; kk++)
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
          for (int jj = 0; jj < 4; jj++) {
            const int j = (i & 1) ? 3 - jj : jj;
            asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0"
                         : "+a"(acc[MA * 4 + i][MB * 4 + j])
                         : "v"(rb[MB][j][kk]), "v"(ra[MA][i][kk]));
          }
    }
  }
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");   // the last results reach the registers before they are read
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++)
#pragma unroll
    for (int j = 0; j < 8; j++) t += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
  sink[(int64_t)blockIdx.x * blockDim.x + threadIdx.x] = t;
}
__global__ __launch_bounds__(256) void mfma_gemm_loop_kernel(float* __restrict__ sink, int64_t iters, int random_data) {
  mfma_gemm_loop_body(sink, iters, random_data);
}

unsigned grid_for(int64_t work_items) {
  int64_t b = (work_items + 255) / 256;
  if (b > 256 * 32) b = 256 * 32;
  if (b < 1) b = 1;
  return (unsigned)b;
}

}  // namespace

extern "C" int mtp_activation_bwd(const void* dact, const void* y, void* dy, int64_t M, int64_t N, int dtype,
                                  int epilogue, void* stream) {
  MTP_REQUIRE(M >= 0 && N >= 1, MTP_EINVAL, "activation_bwd: M=%lld N=%lld", (long long)M, (long long)N);
  MTP_REQUIRE(dtype == MTP_F32 || dtype == MTP_BF16 || dtype == MTP_F16, MTP_EINVAL, "activation_bwd: unknown dtype %d",
              dtype);
  if (M == 0) return MTP_OK;
  MTP_REQUIRE(dact && y && dy, MTP_EINVAL, "activation_bwd: null pointer");
  hipStream_t s = (hipStream_t)stream;
  const uintptr_t al = reinterpret_cast<uintptr_t>(dact) | reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(dy);
  if (epilogue == MTP_EPI_BIAS_GELU || epilogue == MTP_EPI_GELU) {
    MTP_REQUIRE((al & 15) == 0, MTP_EUNSUPPORTED, "activation_bwd: buffers must be 16-byte aligned");
    const int64_t n = M * N;
    if (dtype == MTP_F32)
      hipLaunchKernelGGL(gelu_bwd_kernel<float>, dim3(grid_for(n / 4 + 1)), dim3(256), 0, s, (const float*)dact,
                         (const float*)y, (float*)dy, n);
    else if (dtype == MTP_F16)
      hipLaunchKernelGGL(gelu_bwd_kernel<f16s>, dim3(grid_for(n / 8 + 1)), dim3(256), 0, s, (const f16s*)dact,
                         (const f16s*)y, (f16s*)dy, n);
    else
      hipLaunchKernelGGL(gelu_bwd_kernel<uint16_t>, dim3(grid_for(n / 8 + 1)), dim3(256), 0, s,
                         (const uint16_t*)dact, (const uint16_t*)y, (uint16_t*)dy, n);
  } else if (epilogue == MTP_EPI_SWIGLU) {
    MTP_REQUIRE(N % 2 == 0, MTP_EINVAL, "activation_bwd: SwiGLU needs an even N, got %lld", (long long)N);
    MTP_REQUIRE(dy != dact, MTP_EINVAL, "activation_bwd: SwiGLU output may not alias dact");
    const int64_t H = N / 2;
    const int epv = dtype == MTP_F32 ? 4 : 8;
    const bool vec = (al & 15) == 0 && H % epv == 0;
    // columns in blocks of 256 threads; rows spread over about 16 workgroups per CU
    const int64_t col_blocks = ((vec ? H / epv : H) + 255) / 256;
    MTP_REQUIRE(col_blocks < (1ll << 31), MTP_EINVAL, "activation_bwd: rows too long");
    int64_t row_groups = (4096 + col_blocks - 1) / col_blocks;
    if (row_groups > M) row_groups = M;
    if (row_groups > 65535) row_groups = 65535;
    const dim3 grid((unsigned)col_blocks, (unsigned)row_groups);
#define MTP_SWIGLU_BWD(T)                                                                                          \
  do {                                                                                                             \
    if (vec)                                                                                                       \
      hipLaunchKernelGGL((swiglu_bwd_kernel<T, true>), grid, dim3(256), 0, s, (const T*)dact, (const T*)y, (T*)dy, \
                         M, H);                                                                                    \
    else                                                                                                           \
      hipLaunchKernelGGL((swiglu_bwd_kernel<T, false>), grid, dim3(256), 0, s, (const T*)dact, (const T*)y,        \
                         (T*)dy, M, H);                                                                            \
  } while (0)
    if (dtype == MTP_F32) MTP_SWIGLU_BWD(float);
    else if (dtype == MTP_F16) MTP_SWIGLU_BWD(f16s);
    else MTP_SWIGLU_BWD(uint16_t);
#undef MTP_SWIGLU_BWD
  } else {
    MTP_REQUIRE(false, MTP_EINVAL, "activation_bwd: epilogue %d has no activation", epilogue);
  }
  MTP_CHECK_LAUNCH("activation_bwd");
  return MTP_OK;
}

extern "C" int mtp_stream_copy(const void* src, void* dst, int64_t bytes, void* stream) {
  MTP_REQUIRE(bytes >= 0 && bytes % 16 == 0, MTP_EINVAL, "stream_copy: bytes=%lld not a multiple of 16", (long long)bytes);
  if (bytes == 0) return MTP_OK;
  MTP_REQUIRE(src && dst, MTP_EINVAL, "stream_copy: null pointer");
  MTP_REQUIRE(((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0, MTP_EINVAL,
              "stream_copy: buffers must be 16-byte aligned");
  const int64_t nvec = bytes / 16;
  int64_t blocks = (nvec + 256 * 4 - 1) / (256 * 4);
  if (blocks > 256 * 64) blocks = 256 * 64;
  hipLaunchKernelGGL(stream_copy_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const u32x4_t*)src, (u32x4_t*)dst, nvec);
  MTP_CHECK_LAUNCH("stream_copy");
  return MTP_OK;
}

extern "C" int mtp_mfma_peak(float* sink, int64_t n_waves, int64_t iters, int random_data, void* stream) {
  MTP_REQUIRE(sink && n_waves >= 4 && n_waves % 4 == 0 && iters >= 16 && iters % 16 == 0, MTP_EINVAL,
              "mfma_peak: n_waves must be a positive multiple of 4 and iters of 16");
  hipLaunchKernelGGL(mfma_peak_kernel, dim3((unsigned)(n_waves / 4)), dim3(256), 0, (hipStream_t)stream, sink, iters,
                     random_data);
  MTP_CHECK_LAUNCH("mfma_peak");
  return MTP_OK;
}

extern "C" int mtp_mfma_peak_gemm_loop(float* sink, int64_t n_waves, int64_t iters, int random_data, void* stream) {
  MTP_REQUIRE(sink && n_waves >= 4 && n_waves % 4 == 0 && iters >= 128 && iters % 128 == 0, MTP_EINVAL,
              "mfma_peak_gemm_loop: n_waves must be a positive multiple of 4 and iters of 128");
  hipLaunchKernelGGL(mfma_gemm_loop_kernel, dim3((unsigned)(n_waves / 4)), dim3(256), 0, (hipStream_t)stream, sink, iters,
                     random_data);
  MTP_CHECK_LAUNCH("mfma_peak_gemm_loop");
  return MTP_OK;
}
