// Shared device helpers for the gfx950 kernels: wave64 reductions, bf16
// conversion, 16-byte vector types, and the host-side error plumbing.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/merak_tp_gfx950.h"

#define MTP_WAVE 64

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;

#define LDS_PTR(p) ((void __attribute__((address_space(3)))*)(p))

// ---- bf16 <-> f32 --------------------------------------------------------
__device__ __forceinline__ float bf16_lo(uint32_t packed) {  // element 0 of a pair
  return __uint_as_float(packed << 16);
}
__device__ __forceinline__ float bf16_hi(uint32_t packed) {  // element 1 of a pair
  return __uint_as_float(packed & 0xffff0000u);
}
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}
// round-to-nearest-even through the hardware converter (v_cvt_pk_bf16_f32: one instruction per pair)
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) { return (uint16_t)(pack_bf16x2(f, 0.0f) & 0xffffu); }

// storage type of IEEE half tensors in templates (bf16 tensors travel as uint16_t)
struct f16s {
  uint16_t bits;
};

// ---- the two 16-bit element types of the MFMA kernels: bf16 (F16 = false) and IEEE half (F16 = true) ---------
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
template <bool F16> struct X16;
template <> struct X16<false> {
  static __device__ __forceinline__ float lo(uint32_t p) { return bf16_lo(p); }
  static __device__ __forceinline__ float hi(uint32_t p) { return bf16_hi(p); }
  static __device__ __forceinline__ uint32_t pack2(float a, float b) { return pack_bf16x2(a, b); }
  static __device__ __forceinline__ uint16_t to_bits(float f) { return f32_to_bf16_bits(f); }
  static __device__ __forceinline__ float from_bits(uint16_t b) { return bf16_bits_to_f32(b); }
  static __device__ __forceinline__ f32x16_t mfma32(bf16x8_t a, bf16x8_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4_t mfma16(bf16x8_t a, bf16x8_t b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  // r + the sum of the 8 elements of a (v_dot2 against ones)
  static __device__ __forceinline__ float sum8(bf16x8_t a, float r) {
    const bf16x2_t one = {(__bf16)1.0f, (__bf16)1.0f};
    r = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(a, a, 0, 1), one, r, false);
    r = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(a, a, 2, 3), one, r, false);
    r = __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(a, a, 4, 5), one, r, false);
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(a, a, 6, 7), one, r, false);
  }
};
template <> struct X16<true> {
  static __device__ __forceinline__ float lo(uint32_t p) { return (float)__builtin_bit_cast(f16x2_t, p)[0]; }
  static __device__ __forceinline__ float hi(uint32_t p) { return (float)__builtin_bit_cast(f16x2_t, p)[1]; }
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    const f32x2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));   // round to nearest even
  }
  static __device__ __forceinline__ uint16_t to_bits(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }
  static __device__ __forceinline__ float from_bits(uint16_t b) { return (float)__builtin_bit_cast(_Float16, b); }
  static __device__ __forceinline__ f32x16_t mfma32(bf16x8_t a, bf16x8_t b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0,
                                                  0);
  }
  static __device__ __forceinline__ f32x4_t mfma16(bf16x8_t a, bf16x8_t b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0,
                                                  0);
  }
  static __device__ __forceinline__ float sum8(bf16x8_t a, float r) {
    const f16x8_t h = __builtin_bit_cast(f16x8_t, a);
    const f16x2_t one = {(_Float16)1.0f, (_Float16)1.0f};
    r = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 0, 1), one, r, false);
    r = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 2, 3), one, r, false);
    r = __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 4, 5), one, r, false);
    return __builtin_amdgcn_fdot2(__builtin_shufflevector(h, h, 6, 7), one, r, false);
  }
};

// ---- wave64 reductions (butterfly over ds_bpermute-free shuffles) ---------
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// ---- activations -----------------------------------------------------------
// gelu_new(x) = 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))
// written as x * sigmoid(2u) with u the tanh argument (tanh(u) = 2 sigmoid(2u) - 1)
// 1 / (1 + exp(-t)) with the hardware reciprocal (1 ulp) in place of an IEEE division: the divisor is at least 1
// (or infinite, giving 0), never a denormal, and a division costs about ten instructions where this costs one
__device__ __forceinline__ float sigmoid_f(float t) { return __builtin_amdgcn_rcpf(1.0f + __expf(-t)); }
__device__ __forceinline__ float gelu_new_f(float x) {
  const float k0 = 0.7978845608028654f, k1 = 0.044715f;
  float u = k0 * (x + k1 * x * x * x);
  return x * sigmoid_f(2.0f * u);
}
__device__ __forceinline__ float gelu_new_grad_f(float x) {
  const float k0 = 0.7978845608028654f, k1 = 0.044715f;
  float u = k0 * (x + k1 * x * x * x);
  float s = sigmoid_f(2.0f * u);
  float du = k0 * (1.0f + 3.0f * k1 * x * x);
  return s + x * 2.0f * s * (1.0f - s) * du;
}
__device__ __forceinline__ float silu_f(float x) { return x * sigmoid_f(x); }

// ---- host side -------------------------------------------------------------
void mtp_set_error(const char* fmt, ...);

// Tuning variables (tile or slice choices that never change a result, only which correct kernel runs).  The
// environment is read once per variable, at its first use, and again only when mtp_reload_tuning() is called:
// a launch never calls getenv.
struct MtpTune {
  const char* name;
  int value;      // valid when state == 2
  int state;      // 0 = not read yet, 1 = unset in the environment, 2 = set
  MtpTune* next;
  explicit MtpTune(const char* n);
  // value of the variable, or dflt when it is not set
  int get(int dflt);
  bool is_set();
};

#define MTP_REQUIRE(cond, code, ...)        \
  do {                                      \
    if (!(cond)) {                          \
      mtp_set_error(__VA_ARGS__);           \
      return (code);                        \
    }                                       \
  } while (0)

#define MTP_CHECK_LAUNCH(what)                                              \
  do {                                                                      \
    hipError_t e_ = hipGetLastError();                                      \
    if (e_ != hipSuccess) {                                                 \
      mtp_set_error("%s: launch failed: %s", what, hipGetErrorString(e_));  \
      return MTP_EDEVICE;                                                   \
    }                                                                       \
  } while (0)
