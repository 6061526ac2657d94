// Vocab-parallel cross entropy for gfx950: one workgroup per logits row.
//
// Forward  : one pass over the row with an online (max, sum-exp) pair per
//            lane, combined across the wave by shuffles and across waves
//            through LDS.  Reads N*V elements, writes 4 floats per row.
// Backward : one pass that rewrites the row in place with
//            (softmax - onehot) * grad_out.  Reads N*V, writes N*V.
//
// Rows are streamed with 16-byte loads.  A row need not start on a 16-byte
// boundary (V=50257 fp32 rows do not): the few elements before the first
// aligned address and after the last full vector are handled by scalar code.
//
// Follows Merak/core/mpu/cross_entropy.py:29-106 (see the C header for the
// exact correspondence of outputs to reference lines).
#include "mtp_common.h"

namespace {

constexpr int CE_THREADS = 256;
constexpr int CE_WAVES = CE_THREADS / MTP_WAVE;
constexpr float LOG2E = 1.4426950408889634f;
constexpr float NEG_BIG = -1.0e30f;  // finite stand-in for -inf: NEG_BIG * log2(e) stays finite, exp2 of it is 0

template <typename T> struct Elem;
template <> struct Elem<float> {
  static constexpr int EPV = 4;  // elements per 16-byte vector
  __device__ static __forceinline__ float ld(const float* p) { return *p; }
  __device__ static __forceinline__ void st(float* p, float v) { *p = v; }
  __device__ static __forceinline__ void unpack(const u32x4_t& v, float* f) {
    f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y);
    f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
  }
  __device__ static __forceinline__ u32x4_t pack(const float* f) {
    u32x4_t v;
    v.x = __float_as_uint(f[0]); v.y = __float_as_uint(f[1]);
    v.z = __float_as_uint(f[2]); v.w = __float_as_uint(f[3]);
    return v;
  }
};
template <> struct Elem<uint16_t> {  // bf16 bits
  static constexpr int EPV = 8;
  __device__ static __forceinline__ float ld(const uint16_t* p) { return bf16_bits_to_f32(*p); }
  __device__ static __forceinline__ void st(uint16_t* p, float v) { *p = f32_to_bf16_bits(v); }
  __device__ static __forceinline__ void unpack(const u32x4_t& v, float* f) {
    f[0] = bf16_lo(v.x); f[1] = bf16_hi(v.x); f[2] = bf16_lo(v.y); f[3] = bf16_hi(v.y);
    f[4] = bf16_lo(v.z); f[5] = bf16_hi(v.z); f[6] = bf16_lo(v.w); f[7] = bf16_hi(v.w);
  }
  __device__ static __forceinline__ u32x4_t pack(const float* f) {
    u32x4_t v;
    v.x = pack_bf16x2(f[0], f[1]); v.y = pack_bf16x2(f[2], f[3]);
    v.z = pack_bf16x2(f[4], f[5]); v.w = pack_bf16x2(f[6], f[7]);
    return v;
  }
};

template <> struct Elem<f16s> {  // IEEE half bits
  static constexpr int EPV = 8;
  using H = X16<true>;
  __device__ static __forceinline__ float ld(const f16s* p) { return H::from_bits(p->bits); }
  __device__ static __forceinline__ void st(f16s* p, float v) { p->bits = H::to_bits(v); }
  __device__ static __forceinline__ void unpack(const u32x4_t& v, float* f) {
    f[0] = H::lo(v.x); f[1] = H::hi(v.x); f[2] = H::lo(v.y); f[3] = H::hi(v.y);
    f[4] = H::lo(v.z); f[5] = H::hi(v.z); f[6] = H::lo(v.w); f[7] = H::hi(v.w);
  }
  __device__ static __forceinline__ u32x4_t pack(const float* f) {
    u32x4_t v;
    v.x = H::pack2(f[0], f[1]); v.y = H::pack2(f[2], f[3]);
    v.z = H::pack2(f[4], f[5]); v.w = H::pack2(f[6], f[7]);
    return v;
  }
};

// Split a row of V elements starting at p into [0,head) scalar, nvec 16-byte vectors, and a scalar tail.  The
// vectors start at a 128-byte boundary, not merely a 16-byte one: a wave's 64 vectors then cover eight whole cache
// lines, where a body that starts inside a line makes every wave's stores end in a partial line that the next
// wave completes.  Rows whose length is not a multiple of 128 bytes start at every alignment in turn; measured on
// [8192, 50257] fp32 the in-place gradient pass went from 625 to 580 us with line-aligned bodies (the same rows
// padded to 50240 elements, which are line aligned by themselves: 578 us).  Reads do not care.
// head + tail stay below 2 * 128 / sizeof(T) elements: one element per lane of the smallest workgroup.
template <typename T>
__device__ __forceinline__ void row_split(const T* p, int64_t V, int& head, int64_t& nvec) {
  constexpr int EPV = Elem<T>::EPV;
  uintptr_t mis = reinterpret_cast<uintptr_t>(p) & 127u;
  int h = mis ? (int)((128u - mis) / sizeof(T)) : 0;
  if (h > V) h = (int)V;
  head = h;
  nvec = (V - h) / EPV;
}

// Products and differences that must be rounded on their own (the default -ffp-contract=fast would fuse
// a*b - c into an fma, whose result differs from fl(a*b) - c by the rounding residual of a*b; for the
// -1e30 "no data yet" sentinel that residual is astronomically large).
__device__ __forceinline__ float mul_rn(float a, float b) {
#pragma clang fp contract(off)
  return a * b;
}
__device__ __forceinline__ float sub_rn(float a, float b) {
#pragma clang fp contract(off)
  return a - b;
}

// Running (max, sum-exp) pair.  Exponentials are taken as exp2(fma(x, c, -fl(m*c))) with c = log2(e): one
// VALU op per element for the argument.  The rounding of m*c is the same for every term that shares
// an m, so s always means sum_j exp2(x_j*c - fl(m*c)) consistently; the residual fl(m*c) - m*c is
// exact in an fma and is folded back in once per row (ms_exact_sum).
struct MaxSum {
  float m, s;
};
__device__ __forceinline__ MaxSum ms_combine(MaxSum a, MaxSum b) {
  float m = fmaxf(a.m, b.m);
  const float mc = mul_rn(m, LOG2E);  // explicitly rounded products: no fma contraction here
  MaxSum r;
  r.m = m;
  r.s = a.s * __builtin_amdgcn_exp2f(sub_rn(mul_rn(a.m, LOG2E), mc)) +
        b.s * __builtin_amdgcn_exp2f(sub_rn(mul_rn(b.m, LOG2E), mc));
  return r;
}
// exp2(fl(m*c) - m*c): turns the consistent-but-shifted sum into sum_j exp((x_j - m))
__device__ __forceinline__ float ms_residual_scale(float m) {
  const float mc = mul_rn(m, LOG2E);
  return __builtin_amdgcn_exp2f(-__builtin_fmaf(m, LOG2E, -mc));
}

template <int N>
__device__ __forceinline__ void ms_accumulate(MaxSum& acc, const float* f) {
  float lm = f[0];
#pragma unroll
  for (int i = 1; i < N; i++) lm = fmaxf(lm, f[i]);
  float m = fmaxf(acc.m, lm);
  float mc = mul_rn(m, LOG2E);
  float s = acc.s * __builtin_amdgcn_exp2f(sub_rn(mul_rn(acc.m, LOG2E), mc));
#pragma unroll
  for (int i = 0; i < N; i++) s += __builtin_amdgcn_exp2f(__builtin_fmaf(f[i], LOG2E, -mc));
  acc.m = m;
  acc.s = s;
}

template <typename T, int NT>
__global__ __launch_bounds__(NT) void vocab_ce_fwd_kernel(
    const T* __restrict__ logits, const int64_t* __restrict__ target, float* __restrict__ loss,
    float* __restrict__ row_max, float* __restrict__ row_sumexp, float* __restrict__ pred, int64_t V,
    int64_t vocab_start) {
  constexpr int EPV = Elem<T>::EPV;
  constexpr int UNROLL = 4;
  const int64_t row = blockIdx.x;
  const T* rp = logits + row * V;
  const int tid = threadIdx.x;

  int head;
  int64_t nvec;
  row_split(rp, V, head, nvec);
  const u32x4_t* vp = reinterpret_cast<const u32x4_t*>(rp + head);

  MaxSum acc{NEG_BIG, 0.0f};

  int64_t i = tid;
  for (; i + (UNROLL - 1) * NT < nvec; i += UNROLL * NT) {
    u32x4_t v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) v[u] = __builtin_nontemporal_load(vp + i + u * NT);
    // the step's vectors as one block: one running-maximum update (and one rescaling exponential) per step
    float f[UNROLL * EPV];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) Elem<T>::unpack(v[u], f + u * EPV);
    ms_accumulate<UNROLL * EPV>(acc, f);
  }
  for (; i < nvec; i += NT) {
    u32x4_t v = __builtin_nontemporal_load(vp + i);
    float f[EPV];
    Elem<T>::unpack(v, f);
    ms_accumulate<EPV>(acc, f);
  }
  // scalar head and tail (fewer than 128 / sizeof(T) + EPV elements in total: one per lane)
  {
    const int64_t tail0 = head + nvec * EPV;
    const int n_edge = head + (int)(V - tail0);
    if (tid < n_edge) {
      int64_t j = tid < head ? tid : tail0 + (tid - head);
      float f = Elem<T>::ld(rp + j);
      ms_accumulate<1>(acc, &f);
    }
  }

  // wave butterfly, then across waves through LDS
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    MaxSum other;
    other.m = __shfl_xor(acc.m, o, 64);
    other.s = __shfl_xor(acc.s, o, 64);
    acc = ms_combine(acc, other);
  }
  __shared__ float sm[(NT / MTP_WAVE)], ss[(NT / MTP_WAVE)];
  if ((tid & 63) == 0) {
    sm[tid >> 6] = acc.m;
    ss[tid >> 6] = acc.s;
  }
  __syncthreads();
  if (tid == 0) {
    MaxSum t{sm[0], ss[0]};
#pragma unroll
    for (int w = 1; w < (NT / MTP_WAVE); w++) t = ms_combine(t, MaxSum{sm[w], ss[w]});
    t.s *= ms_residual_scale(t.m);
    const int64_t tl = target[row] - vocab_start;
    const bool in_range = tl >= 0 && tl < V;
    const float x_t = in_range ? Elem<T>::ld(rp + tl) : 0.0f;
    row_max[row] = t.m;
    row_sumexp[row] = t.s;
    pred[row] = x_t;
    loss[row] = logf(t.s) - (in_range ? (x_t - t.m) : 0.0f);
  }
}

template <typename T, int NT>
__global__ __launch_bounds__(NT) void vocab_ce_bwd_kernel(
    T* __restrict__ logits, const int64_t* __restrict__ target, const float* __restrict__ row_max,
    const float* __restrict__ row_sumexp, const float* __restrict__ grad_out, int64_t V, int64_t vocab_start) {
  constexpr int EPV = Elem<T>::EPV;
  constexpr int UNROLL = 4;
  const int64_t row = blockIdx.x;
  T* rp = logits + row * V;
  const int tid = threadIdx.x;

  int head;
  int64_t nvec;
  row_split(rp, V, head, nvec);
  u32x4_t* vp = reinterpret_cast<u32x4_t*>(rp + head);

  const float g = grad_out ? grad_out[row] : 1.0f;
  // row_max == nullptr: the buffer already holds the softmax, so the "exponential" is the value itself
  const bool from_softmax = row_max == nullptr;
  const float mc = from_softmax ? 0.0f : mul_rn(row_max[row], LOG2E);
  // softmax_j * g = exp2(x_j*c - fl(m*c)) * scale, the rounding residual of m*c folded into scale
  const float scale = from_softmax ? g : g * ms_residual_scale(row_max[row]) / row_sumexp[row];
  int64_t tl = target[row] - vocab_start;
  if (tl < 0 || tl >= V) tl = -1;
  // position of the target inside the vector body, in elements (or out of reach)
  const int64_t tv = (tl >= head) ? (tl - head) : -1;

  int64_t i = tid;
  for (; i + (UNROLL - 1) * NT < nvec; i += UNROLL * NT) {
    u32x4_t v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) v[u] = __builtin_nontemporal_load(vp + i + u * NT);
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
      float f[EPV];
      Elem<T>::unpack(v[u], f);
#pragma unroll
      for (int e = 0; e < EPV; e++) f[e] = (from_softmax ? f[e] : __builtin_amdgcn_exp2f(__builtin_fmaf(f[e], LOG2E, -mc))) * scale;
      const int64_t base = (i + u * NT) * EPV;
      if ((uint64_t)(tv - base) < (uint64_t)EPV) {
        const int e = (int)(tv - base);
#pragma unroll
        for (int q = 0; q < EPV; q++)
          if (q == e) f[q] -= g;
      }
      __builtin_nontemporal_store(Elem<T>::pack(f), vp + i + u * NT);
    }
  }
  for (; i < nvec; i += NT) {
    u32x4_t v = __builtin_nontemporal_load(vp + i);
    float f[EPV];
    Elem<T>::unpack(v, f);
#pragma unroll
    for (int e = 0; e < EPV; e++) f[e] = (from_softmax ? f[e] : __builtin_amdgcn_exp2f(__builtin_fmaf(f[e], LOG2E, -mc))) * scale;
    const int64_t base = i * EPV;
    if ((uint64_t)(tv - base) < (uint64_t)EPV) {
      const int e = (int)(tv - base);
#pragma unroll
      for (int q = 0; q < EPV; q++)
        if (q == e) f[q] -= g;
    }
    __builtin_nontemporal_store(Elem<T>::pack(f), vp + i);
  }
  {
    const int64_t tail0 = head + nvec * EPV;
    const int n_edge = head + (int)(V - tail0);
    if (tid < n_edge) {
      int64_t j = tid < head ? tid : tail0 + (tid - head);
      float f = Elem<T>::ld(rp + j);
      f = (from_softmax ? f : __builtin_amdgcn_exp2f(__builtin_fmaf(f, LOG2E, -mc))) * scale;
      if (j == tl) f -= g;
      Elem<T>::st(rp + j, f);
    }
  }
}

// ---- forward and backward in one pass ---------------------------------------
// One 1024-lane workgroup keeps a whole row in registers (NV 16-byte vectors per lane): loaded once, reduced to
// (max, sum-exp), then rewritten in place as (softmax - onehot) * g.  HBM sees one read and one write of the row
// instead of two reads and a write.
//
// A workgroup takes rows b, b + gridDim.x, ...: launched with fewer workgroups than rows it is persistent and asks
// for the next row's vectors right behind the stores of the current one, so that the next row is on its way while
// this one's stores drain; launched with gridDim.x = n_rows it is one workgroup per row (row_kernel_grid).
constexpr int FU_THREADS = 1024;
constexpr int FU_WAVES = FU_THREADS / MTP_WAVE;

// where a row's aligned 16-byte vectors and its scalar edges lie
template <typename T>
struct RowGeo {
  T* rp;
  u32x4_t* vp;
  int head, nvec, edge_j;
  bool has_edge;
  __device__ __forceinline__ void set(T* logits, int64_t row, int64_t V, int tid) {
    constexpr int EPV = Elem<T>::EPV;
    rp = logits + row * V;
    int64_t nvec64;
    row_split(rp, V, head, nvec64);
    nvec = (int)nvec64;  // the host checked nvec <= NV * FU_THREADS
    vp = reinterpret_cast<u32x4_t*>(rp + head);
    const int tail0 = head + nvec * EPV;
    const int n_edge = head + (int)(V - tail0);
    edge_j = tid < head ? tid : tail0 + (tid - head);
    has_edge = tid < n_edge;
  }
};

// WALK: the workgroup may have more than one row (gridDim.x < n_rows); without it the loop below runs once and
// nothing of the next row's bookkeeping takes registers.
template <typename T, int NV, bool WALK>
__global__ __launch_bounds__(FU_THREADS) void vocab_ce_fused_kernel(
    T* __restrict__ logits, const int64_t* __restrict__ target, const float* __restrict__ grad_rows,
    float grad_scale, float* __restrict__ loss, float* __restrict__ row_max, float* __restrict__ row_sumexp,
    float* __restrict__ pred, int64_t V, int64_t vocab_start, int64_t n_rows) {
  constexpr int EPV = Elem<T>::EPV;
  const int tid = threadIdx.x;
  int64_t row = blockIdx.x;
  if (row >= n_rows) return;

  RowGeo<T> geo;
  geo.set(logits, row, V, tid);
  u32x4_t v[NV] = {};
#pragma unroll
  for (int u = 0; u < NV; u++)
    if (tid + u * FU_THREADS < geo.nvec) v[u] = __builtin_nontemporal_load(geo.vp + tid + u * FU_THREADS);
  float fe = NEG_BIG;
  if (geo.has_edge) fe = Elem<T>::ld(geo.rp + geo.edge_j);

  // two sets of the cross-wave cells, used by alternate rows: a wave that is already reducing the next row must
  // not overwrite cells another wave still reads for this one (one barrier per row lies between a set's uses)
  __shared__ float red_m[2][FU_WAVES], red_s[2][FU_WAVES];
  int par = 0;

  for (;;) {
    int64_t tl = target[row] - vocab_start;
    if (tl < 0 || tl >= V) tl = -1;
    float x_t = 0.0f;
    if (tid == 0 && tl >= 0) x_t = Elem<T>::ld(geo.rp + tl);  // read before any lane stores to this row
    const float g = (grad_rows ? grad_rows[row] : 1.0f) * grad_scale;

    // Row maximum and sum of exponentials in one pass over the registers, two vectors at a time in the order they
    // arrive (the running maximum and the shifted sum of the forward kernel), so that this arithmetic runs while
    // the rest of the row is still on its way.
    MaxSum acc{NEG_BIG, 0.0f};
    if (geo.has_edge) ms_accumulate<1>(acc, &fe);
#pragma unroll
    for (int u = 0; u < NV; u += 2) {
      if (u + 1 < NV && tid + (u + 1) * FU_THREADS < geo.nvec) {
        float f[2 * EPV];
        Elem<T>::unpack(v[u], f);
        Elem<T>::unpack(v[u + 1], f + EPV);
        ms_accumulate<2 * EPV>(acc, f);
      } else if (tid + u * FU_THREADS < geo.nvec) {
        float f[EPV];
        Elem<T>::unpack(v[u], f);
        ms_accumulate<EPV>(acc, f);
      }
    }
    // keep the row as loaded: without this the compiler carries the unpacked floats into the gradient pass, which
    // doubles the registers a bf16 row needs
#pragma unroll
    for (int u = 0; u < NV; u++) asm volatile("" : "+v"(v[u]));
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      MaxSum other;
      other.m = __shfl_xor(acc.m, o, 64);
      other.s = __shfl_xor(acc.s, o, 64);
      acc = ms_combine(acc, other);
    }
    if ((tid & 63) == 0) {
      red_m[par][tid >> 6] = acc.m;
      red_s[par][tid >> 6] = acc.s;
    }
    __syncthreads();
    // every wave combines the 16 waves' pairs on its own lanes (16 lanes hold one copy) and takes lane 0's result
    static_assert(FU_WAVES == 16, "the cross-wave butterfly is written for 16 waves");
    MaxSum tot{red_m[par][tid & 15], red_s[par][tid & 15]};
    par ^= 1;
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) {
      MaxSum other;
      other.m = __shfl_xor(tot.m, o, 64);
      other.s = __shfl_xor(tot.s, o, 64);
      tot = ms_combine(tot, other);
    }
    const float m = __shfl(tot.m, 0, 64);
    const float s_raw = __shfl(tot.s, 0, 64);   // sum of exp2(x*c - fl(m*c)): the forward kernel's shifted sum
    const float mc = mul_rn(m, LOG2E);

    if (tid == 0) {
      const float s = s_raw * ms_residual_scale(m);
      row_max[row] = m;
      row_sumexp[row] = s;
      pred[row] = x_t;
      loss[row] = logf(s) - (tl >= 0 ? (x_t - m) : 0.0f);
    }

    // gradient, in place
    const int64_t next = row + gridDim.x;
    const bool more = WALK && next < n_rows;
    RowGeo<T> gn = geo;
    if (more) gn.set(logits, next, V, tid);
    const float scale = g / s_raw;  // exp2(x*c - fl(m*c)) / s_raw = softmax: the residual cancels
    const int tv = (tl >= geo.head) ? (int)(tl - geo.head) : -1;
#pragma unroll
    for (int u = 0; u < NV; u++) {
      if (tid + u * FU_THREADS < geo.nvec) {
        float f[EPV];
        Elem<T>::unpack(v[u], f);
#pragma unroll
        for (int e = 0; e < EPV; e++) f[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(f[e], LOG2E, -mc)) * scale;
        const int base = (tid + u * FU_THREADS) * EPV;
        if ((unsigned)(tv - base) < (unsigned)EPV) {
          const int e = tv - base;
#pragma unroll
          for (int q = 0; q < EPV; q++)
            if (q == e) f[q] -= g;
        }
        __builtin_nontemporal_store(Elem<T>::pack(f), geo.vp + tid + u * FU_THREADS);
      }
    }
    if (geo.has_edge) {
      float f = __builtin_amdgcn_exp2f(__builtin_fmaf(fe, LOG2E, -mc)) * scale;
      if (geo.edge_j == tl) f -= g;
      Elem<T>::st(geo.rp + geo.edge_j, f);
    }
    if (!more) break;
    // the next row is asked for behind the last store of this one, as one burst: reads mixed into the write burst
    // vector by vector cost 6 % (the memory then turns between reading and writing all the time)
#pragma unroll
    for (int u = 0; u < NV; u++)
      if (tid + u * FU_THREADS < gn.nvec) v[u] = __builtin_nontemporal_load(gn.vp + tid + u * FU_THREADS);
    fe = NEG_BIG;
    if (gn.has_edge) fe = Elem<T>::ld(gn.rp + gn.edge_j);
    geo = gn;
    row = next;
  }
}

// Backward with the row held in registers: every lane of a 1024-lane workgroup loads its NV vectors of the row,
// the workgroup meets at a barrier, then every lane rewrites them.  The memory sees the row as one burst of reads
// and one burst of writes (250 KiB each for a bf16 row of 128256) instead of 16 KiB steps that alternate
// between the two.  Walks rows b, b + gridDim.x, ... like the kernel above (one row per workgroup by default).
// Same arithmetic per element as vocab_ce_bwd_kernel, so the same bits.  (The row's maximum and sum are known
// before the row arrives, so the gradient could be computed in place under the read burst and the write burst be
// stores only: measured, that is slower — 580 -> 604 us on [8192, 50257] fp32, 588 -> 602 us on [8192, 100480]
// bf16, no change at 128256 — because the barrier then waits for the slowest wave's arithmetic as well.)
template <typename T, int NV, bool WALK>
__global__ __launch_bounds__(FU_THREADS) void vocab_ce_bwd_row_kernel(
    T* __restrict__ logits, const int64_t* __restrict__ target, const float* __restrict__ row_max,
    const float* __restrict__ row_sumexp, const float* __restrict__ grad_out, int64_t V, int64_t vocab_start,
    int64_t n_rows) {
  constexpr int EPV = Elem<T>::EPV;
  const int tid = threadIdx.x;
  int64_t row = blockIdx.x;
  if (row >= n_rows) return;

  RowGeo<T> geo;
  geo.set(logits, row, V, tid);
  u32x4_t v[NV] = {};
#pragma unroll
  for (int u = 0; u < NV; u++)
    if (tid + u * FU_THREADS < geo.nvec) v[u] = __builtin_nontemporal_load(geo.vp + tid + u * FU_THREADS);
  float fe = 0.0f;
  if (geo.has_edge) fe = Elem<T>::ld(geo.rp + geo.edge_j);
  const bool from_softmax = row_max == nullptr;

  for (;;) {
    const float g = grad_out ? grad_out[row] : 1.0f;
    const float mc = from_softmax ? 0.0f : mul_rn(row_max[row], LOG2E);
    const float scale = from_softmax ? g : g * ms_residual_scale(row_max[row]) / row_sumexp[row];
    int64_t tl = target[row] - vocab_start;
    if (tl < 0 || tl >= V) tl = -1;
    const int tv = (tl >= geo.head) ? (int)(tl - geo.head) : -1;
    const int64_t next = row + gridDim.x;
    const bool more = WALK && next < n_rows;
    RowGeo<T> gn = geo;
    if (more) gn.set(logits, next, V, tid);
#pragma unroll
    for (int u = 0; u < NV; u++) asm volatile("" : "+v"(v[u]));   // the whole row has arrived for this wave ...
    __syncthreads();                                              // ... and for every wave, before anyone writes

#pragma unroll
    for (int u = 0; u < NV; u++) {
      if (tid + u * FU_THREADS < geo.nvec) {
        float f[EPV];
        Elem<T>::unpack(v[u], f);
#pragma unroll
        for (int e = 0; e < EPV; e++) f[e] = (from_softmax ? f[e] : __builtin_amdgcn_exp2f(__builtin_fmaf(f[e], LOG2E, -mc))) * scale;
        const int base = (tid + u * FU_THREADS) * EPV;
        if ((unsigned)(tv - base) < (unsigned)EPV) {
          const int e = tv - base;
#pragma unroll
          for (int q = 0; q < EPV; q++)
            if (q == e) f[q] -= g;
        }
        __builtin_nontemporal_store(Elem<T>::pack(f), geo.vp + tid + u * FU_THREADS);
      }
    }
    if (geo.has_edge) {
      float f = (from_softmax ? fe : __builtin_amdgcn_exp2f(__builtin_fmaf(fe, LOG2E, -mc))) * scale;
      if (geo.edge_j == tl) f -= g;
      Elem<T>::st(geo.rp + geo.edge_j, f);
    }
    if (!more) break;
#pragma unroll
    for (int u = 0; u < NV; u++)
      if (tid + u * FU_THREADS < gn.nvec) v[u] = __builtin_nontemporal_load(gn.vp + tid + u * FU_THREADS);
    fe = 0.0f;
    if (gn.has_edge) fe = Elem<T>::ld(gn.rp + gn.edge_j);
    geo = gn;
    row = next;
  }
}

// Workgroups of the register-resident kernels: persistent (one per compute unit — each holds a row's worth of the
// register file — every one walking its share of the rows) or one per row.  Measured on [8192, 128256] bf16 and
// [8192, 50257] fp32: the one-launch kernel on 16-bit rows gains from walking (788 -> 759 us: the next row is on
// its way while the loss of this one is written, and a workgroup's start — target, target logit, row gradient,
// three dependent reads — happens once instead of per row); on fp32 rows it loses (634 -> 671 us) and the backward
// kernel, which has no such start, loses on both (741 -> 771, 630 -> 670 us): a workgroup that ends with its
// stores in flight hands the compute unit to the next row's loads sooner than a loop that, counting its memory
// operations in order, cannot look at the new row before those stores have landed.  Asking for the next row
// vector by vector between the stores of this one is worse still (+6 %: the memory then turns between reading
// and writing all the time).  MTP_CE_PERSIST = 0 / 1 forces one workgroup per row / walking for all of them.
inline unsigned row_kernel_grid(int64_t n_rows, bool walk_by_default) {
  static MtpTune tune_persist("MTP_CE_PERSIST");
  const int per = tune_persist.get(walk_by_default ? 1 : 0);
  if (per <= 0) return (unsigned)n_rows;
  const int64_t wgs = 256ll * per;
  return (unsigned)(n_rows < wgs ? n_rows : wgs);
}

// Rows of at least two unrolled steps of a 1024-lane workgroup are walked by 1024 lanes (64 KiB per step; bf16
// [8192, 128256] forward 312 -> 305 us, fp32 [8192, 50257] 254 -> 240 us: fewer, larger streams, and a last wave
// of workgroups that is a sixteenth of the launch instead of a quarter), shorter rows by 256 (a 1024-lane step
// would cover a 32000-element bf16 row only once, in its slower single-vector loop).
template <typename T>
bool long_row(int64_t vocab) { return vocab / Elem<T>::EPV >= 2 * 4 * 1024; }

template <typename T>
void launch_fwd(const void* logits, const int64_t* target, float* loss, float* row_max, float* row_sumexp, float* pred,
                int64_t n_rows, int64_t vocab, int64_t vocab_start, hipStream_t s) {
  if (long_row<T>(vocab))
    hipLaunchKernelGGL((vocab_ce_fwd_kernel<T, 1024>), dim3((unsigned)n_rows), dim3(1024), 0, s, (const T*)logits,
                       target, loss, row_max, row_sumexp, pred, vocab, vocab_start);
  else
    hipLaunchKernelGGL((vocab_ce_fwd_kernel<T, CE_THREADS>), dim3((unsigned)n_rows), dim3(CE_THREADS), 0, s,
                       (const T*)logits, target, loss, row_max, row_sumexp, pred, vocab, vocab_start);
}

template <typename T>
void launch_bwd(void* logits, const int64_t* target, const float* row_max, const float* row_sumexp,
                const float* grad_out, int64_t n_rows, int64_t vocab, int64_t vocab_start, hipStream_t s) {
  static MtpTune tune_row("MTP_CE_BWD_ROW");
  const int64_t need = (vocab / Elem<T>::EPV + FU_THREADS - 1) / FU_THREADS;
#define MTP_BWD_ROW_CASE(NV)                                                                                     \
  if (need <= NV) {                                                                                              \
    const unsigned grid = row_kernel_grid(n_rows, false);                                                        \
    if (grid < n_rows)                                                                                           \
      hipLaunchKernelGGL((vocab_ce_bwd_row_kernel<T, NV, true>), dim3(grid), dim3(FU_THREADS), 0, s, (T*)logits, \
                         target, row_max, row_sumexp, grad_out, vocab, vocab_start, n_rows);                     \
    else                                                                                                         \
      hipLaunchKernelGGL((vocab_ce_bwd_row_kernel<T, NV, false>), dim3(grid), dim3(FU_THREADS), 0, s, (T*)logits, \
                         target, row_max, row_sumexp, grad_out, vocab, vocab_start, n_rows);                     \
    return;                                                                                                      \
  }
  // rows of at least a quarter of what 1024 lanes hold; shorter rows are served as well by the stepping kernel
  if (tune_row.get(1) != 0 && need >= 4) {
    MTP_BWD_ROW_CASE(4)
    MTP_BWD_ROW_CASE(8)
    MTP_BWD_ROW_CASE(12)
    MTP_BWD_ROW_CASE(16)
    MTP_BWD_ROW_CASE(20)
  }
#undef MTP_BWD_ROW_CASE
  if (long_row<T>(vocab))
    hipLaunchKernelGGL((vocab_ce_bwd_kernel<T, 1024>), dim3((unsigned)n_rows), dim3(1024), 0, s, (T*)logits, target,
                       row_max, row_sumexp, grad_out, vocab, vocab_start);
  else
    hipLaunchKernelGGL((vocab_ce_bwd_kernel<T, CE_THREADS>), dim3((unsigned)n_rows), dim3(CE_THREADS), 0, s, (T*)logits,
                       target, row_max, row_sumexp, grad_out, vocab, vocab_start);
}

// grad[i,:] *= grad_rows[i] / assumed, skipped for rows where the two are equal
template <typename T>
__global__ __launch_bounds__(CE_THREADS) void vocab_ce_rescale_kernel(T* __restrict__ grad,
                                                                     const float* __restrict__ grad_rows,
                                                                     float assumed, int64_t V) {
  constexpr int EPV = Elem<T>::EPV;
  const int64_t row = blockIdx.x;
  const float gr = grad_rows[row];
  if (gr == assumed) return;
  const float ratio = gr / assumed;
  T* rp = grad + row * V;
  const int tid = threadIdx.x;
  int head;
  int64_t nvec;
  row_split(rp, V, head, nvec);
  u32x4_t* vp = reinterpret_cast<u32x4_t*>(rp + head);
  for (int64_t i = tid; i < nvec; i += CE_THREADS) {
    u32x4_t v = __builtin_nontemporal_load(vp + i);
    float f[EPV];
    Elem<T>::unpack(v, f);
#pragma unroll
    for (int e = 0; e < EPV; e++) f[e] *= ratio;
    __builtin_nontemporal_store(Elem<T>::pack(f), vp + i);
  }
  const int64_t tail0 = head + nvec * EPV;
  const int n_edge = head + (int)(V - tail0);
  if (tid < n_edge) {
    int64_t j = tid < head ? tid : tail0 + (tid - head);
    Elem<T>::st(rp + j, Elem<T>::ld(rp + j) * ratio);
  }
}

template <typename T, int NV>
void launch_fused(void* logits, const int64_t* target, const float* grad_rows, float grad_scale, float* loss,
                  float* row_max, float* row_sumexp, float* pred, int64_t n_rows, int64_t vocab,
                  int64_t vocab_start, hipStream_t s) {
  // (the 20-vector instantiation has no registers left for the next row's bookkeeping: it would spill)
  const unsigned grid = row_kernel_grid(n_rows, sizeof(T) == 2 && NV <= 16);
  if (grid < n_rows)
    hipLaunchKernelGGL((vocab_ce_fused_kernel<T, NV, true>), dim3(grid), dim3(FU_THREADS), 0, s, (T*)logits, target,
                       grad_rows, grad_scale, loss, row_max, row_sumexp, pred, vocab, vocab_start, n_rows);
  else
    hipLaunchKernelGGL((vocab_ce_fused_kernel<T, NV, false>), dim3(grid), dim3(FU_THREADS), 0, s, (T*)logits, target,
                       grad_rows, grad_scale, loss, row_max, row_sumexp, pred, vocab, vocab_start, n_rows);
}

template <typename T>
int dispatch_fused(void* logits, const int64_t* target, const float* grad_rows, float grad_scale, float* loss,
                   float* row_max, float* row_sumexp, float* pred, int64_t n_rows, int64_t vocab,
                   int64_t vocab_start, hipStream_t s) {
  // the row's aligned body has at most vocab / EPV vectors whatever its start address
  const int64_t nvec_max = vocab / Elem<T>::EPV;
  const int64_t need = (nvec_max + FU_THREADS - 1) / FU_THREADS;
#define MTP_FUSED_CASE(NV)                                                                                      \
  if (need <= NV) {                                                                                             \
    launch_fused<T, NV>(logits, target, grad_rows, grad_scale, loss, row_max, row_sumexp, pred, n_rows, vocab,  \
                        vocab_start, s);                                                                        \
    return MTP_OK;                                                                                              \
  }
  if (vocab <= 20ll * FU_THREADS * Elem<T>::EPV) {
    MTP_FUSED_CASE(4)
    MTP_FUSED_CASE(8)
    MTP_FUSED_CASE(12)
    MTP_FUSED_CASE(16)
    MTP_FUSED_CASE(20)
  }
#undef MTP_FUSED_CASE
  mtp_set_error("vocab_ce_fwd_bwd: a row of %lld elements does not fit the register-resident kernel (limit %lld)",
                (long long)vocab, (long long)(20ll * FU_THREADS * Elem<T>::EPV));
  return MTP_EUNSUPPORTED;
}

}  // namespace

extern "C" int mtp_vocab_ce_fwd(const void* logits, const int64_t* target, float* loss, float* row_max,
                                float* row_sumexp, float* pred, int64_t n_rows, int64_t vocab,
                                int64_t vocab_start, int dtype, void* stream) {
  MTP_REQUIRE(n_rows >= 0 && vocab >= 1, MTP_EINVAL, "vocab_ce_fwd: n_rows=%lld vocab=%lld", (long long)n_rows,
              (long long)vocab);
  MTP_REQUIRE(n_rows < (1ll << 31), MTP_EUNSUPPORTED, "vocab_ce_fwd: n_rows=%lld exceeds 2^31-1", (long long)n_rows);
  if (n_rows == 0) return MTP_OK;
  MTP_REQUIRE(logits && target && loss && row_max && row_sumexp && pred, MTP_EINVAL, "vocab_ce_fwd: null pointer");
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MTP_F32) {
    MTP_REQUIRE((reinterpret_cast<uintptr_t>(logits) & 3) == 0, MTP_EINVAL, "vocab_ce_fwd: fp32 logits not 4-byte aligned");
    launch_fwd<float>(logits, target, loss, row_max, row_sumexp, pred, n_rows, vocab, vocab_start, s);
  } else if (dtype == MTP_BF16) {
    MTP_REQUIRE((reinterpret_cast<uintptr_t>(logits) & 1) == 0, MTP_EINVAL, "vocab_ce_fwd: bf16 logits not 2-byte aligned");
    launch_fwd<uint16_t>(logits, target, loss, row_max, row_sumexp, pred, n_rows, vocab, vocab_start, s);
  } else if (dtype == MTP_F16) {
    MTP_REQUIRE((reinterpret_cast<uintptr_t>(logits) & 1) == 0, MTP_EINVAL, "vocab_ce_fwd: fp16 logits not 2-byte aligned");
    launch_fwd<f16s>(logits, target, loss, row_max, row_sumexp, pred, n_rows, vocab, vocab_start, s);
  } else {
    MTP_REQUIRE(false, MTP_EINVAL, "vocab_ce_fwd: unknown dtype %d", dtype);
  }
  MTP_CHECK_LAUNCH("vocab_ce_fwd");
  return MTP_OK;
}

extern "C" int mtp_vocab_ce_bwd(void* logits, const int64_t* target, const float* row_max, const float* row_sumexp,
                                const float* grad_out, int64_t n_rows, int64_t vocab, int64_t vocab_start, int dtype,
                                void* stream) {
  MTP_REQUIRE(n_rows >= 0 && vocab >= 1, MTP_EINVAL, "vocab_ce_bwd: n_rows=%lld vocab=%lld", (long long)n_rows,
              (long long)vocab);
  MTP_REQUIRE(n_rows < (1ll << 31), MTP_EUNSUPPORTED, "vocab_ce_bwd: n_rows=%lld exceeds 2^31-1", (long long)n_rows);
  if (n_rows == 0) return MTP_OK;
  MTP_REQUIRE(logits && target, MTP_EINVAL, "vocab_ce_bwd: null pointer");
  MTP_REQUIRE((row_max == nullptr) == (row_sumexp == nullptr), MTP_EINVAL,
              "vocab_ce_bwd: row_max and row_sumexp must both be given or both be null");
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MTP_F32) {
    MTP_REQUIRE((reinterpret_cast<uintptr_t>(logits) & 3) == 0, MTP_EINVAL, "vocab_ce_bwd: fp32 logits not 4-byte aligned");
    launch_bwd<float>(logits, target, row_max, row_sumexp, grad_out, n_rows, vocab, vocab_start, s);
  } else if (dtype == MTP_BF16) {
    MTP_REQUIRE((reinterpret_cast<uintptr_t>(logits) & 1) == 0, MTP_EINVAL, "vocab_ce_bwd: bf16 logits not 2-byte aligned");
    launch_bwd<uint16_t>(logits, target, row_max, row_sumexp, grad_out, n_rows, vocab, vocab_start, s);
  } else if (dtype == MTP_F16) {
    MTP_REQUIRE((reinterpret_cast<uintptr_t>(logits) & 1) == 0, MTP_EINVAL, "vocab_ce_bwd: fp16 logits not 2-byte aligned");
    launch_bwd<f16s>(logits, target, row_max, row_sumexp, grad_out, n_rows, vocab, vocab_start, s);
  } else {
    MTP_REQUIRE(false, MTP_EINVAL, "vocab_ce_bwd: unknown dtype %d", dtype);
  }
  MTP_CHECK_LAUNCH("vocab_ce_bwd");
  return MTP_OK;
}

extern "C" int64_t mtp_vocab_ce_fwd_bwd_max_vocab(int dtype) {
  if (dtype == MTP_F32) return 20ll * FU_THREADS * Elem<float>::EPV;
  if (dtype == MTP_BF16 || dtype == MTP_F16) return 20ll * FU_THREADS * Elem<uint16_t>::EPV;
  return 0;
}

extern "C" int mtp_vocab_ce_fwd_bwd(void* logits, const int64_t* target, const float* grad_rows, float grad_scale,
                                    float* loss, float* row_max, float* row_sumexp, float* pred, int64_t n_rows,
                                    int64_t vocab, int64_t vocab_start, int dtype, void* stream) {
  MTP_REQUIRE(n_rows >= 0 && vocab >= 1, MTP_EINVAL, "vocab_ce_fwd_bwd: n_rows=%lld vocab=%lld", (long long)n_rows,
              (long long)vocab);
  MTP_REQUIRE(n_rows < (1ll << 31), MTP_EUNSUPPORTED, "vocab_ce_fwd_bwd: n_rows=%lld exceeds 2^31-1",
              (long long)n_rows);
  if (n_rows == 0) return MTP_OK;
  MTP_REQUIRE(logits && target && loss && row_max && row_sumexp && pred, MTP_EINVAL, "vocab_ce_fwd_bwd: null pointer");
  hipStream_t s = (hipStream_t)stream;
  int rc;
  if (dtype == MTP_F32) {
    MTP_REQUIRE((reinterpret_cast<uintptr_t>(logits) & 3) == 0, MTP_EINVAL,
                "vocab_ce_fwd_bwd: fp32 logits not 4-byte aligned");
    rc = dispatch_fused<float>(logits, target, grad_rows, grad_scale, loss, row_max, row_sumexp, pred, n_rows, vocab,
                               vocab_start, s);
  } else if (dtype == MTP_BF16) {
    MTP_REQUIRE((reinterpret_cast<uintptr_t>(logits) & 1) == 0, MTP_EINVAL,
                "vocab_ce_fwd_bwd: bf16 logits not 2-byte aligned");
    rc = dispatch_fused<uint16_t>(logits, target, grad_rows, grad_scale, loss, row_max, row_sumexp, pred, n_rows,
                                  vocab, vocab_start, s);
  } else if (dtype == MTP_F16) {
    MTP_REQUIRE((reinterpret_cast<uintptr_t>(logits) & 1) == 0, MTP_EINVAL,
                "vocab_ce_fwd_bwd: fp16 logits not 2-byte aligned");
    rc = dispatch_fused<f16s>(logits, target, grad_rows, grad_scale, loss, row_max, row_sumexp, pred, n_rows, vocab,
                              vocab_start, s);
  } else {
    MTP_REQUIRE(false, MTP_EINVAL, "vocab_ce_fwd_bwd: unknown dtype %d", dtype);
  }
  if (rc != MTP_OK) return rc;
  MTP_CHECK_LAUNCH("vocab_ce_fwd_bwd");
  return MTP_OK;
}

extern "C" int mtp_vocab_ce_rescale(void* grad, const float* grad_rows, float assumed, int64_t n_rows, int64_t vocab,
                                    int dtype, void* stream) {
  MTP_REQUIRE(n_rows >= 0 && vocab >= 1, MTP_EINVAL, "vocab_ce_rescale: n_rows=%lld vocab=%lld", (long long)n_rows,
              (long long)vocab);
  MTP_REQUIRE(n_rows < (1ll << 31), MTP_EUNSUPPORTED, "vocab_ce_rescale: n_rows=%lld exceeds 2^31-1",
              (long long)n_rows);
  MTP_REQUIRE(assumed != 0.0f && assumed == assumed, MTP_EINVAL, "vocab_ce_rescale: assumed scale must be non-zero");
  if (n_rows == 0) return MTP_OK;
  MTP_REQUIRE(grad && grad_rows, MTP_EINVAL, "vocab_ce_rescale: null pointer");
  hipStream_t s = (hipStream_t)stream;
  dim3 grid((unsigned)n_rows), block(CE_THREADS);
  if (dtype == MTP_F32) {
    MTP_REQUIRE((reinterpret_cast<uintptr_t>(grad) & 3) == 0, MTP_EINVAL, "vocab_ce_rescale: fp32 buffer not 4-byte aligned");
    hipLaunchKernelGGL(vocab_ce_rescale_kernel<float>, grid, block, 0, s, (float*)grad, grad_rows, assumed, vocab);
  } else if (dtype == MTP_BF16) {
    MTP_REQUIRE((reinterpret_cast<uintptr_t>(grad) & 1) == 0, MTP_EINVAL, "vocab_ce_rescale: bf16 buffer not 2-byte aligned");
    hipLaunchKernelGGL(vocab_ce_rescale_kernel<uint16_t>, grid, block, 0, s, (uint16_t*)grad, grad_rows, assumed, vocab);
  } else if (dtype == MTP_F16) {
    MTP_REQUIRE((reinterpret_cast<uintptr_t>(grad) & 1) == 0, MTP_EINVAL, "vocab_ce_rescale: fp16 buffer not 2-byte aligned");
    hipLaunchKernelGGL(vocab_ce_rescale_kernel<f16s>, grid, block, 0, s, (f16s*)grad, grad_rows, assumed, vocab);
  } else {
    MTP_REQUIRE(false, MTP_EINVAL, "vocab_ce_rescale: unknown dtype %d", dtype);
  }
  MTP_CHECK_LAUNCH("vocab_ce_rescale");
  return MTP_OK;
}
