// Sampling tail of the decode loop for gfx950: temperature, top-k, top-p and
// one multinomial draw per batch row, in one kernel, one workgroup per row
// (Merak/inference/text_generation_inference.py:35-69 `top_k_logits`, :229-235).
//
//   z      = float(logits) / temperature                               (:230-231)
//   top-k  : drop z < (k-th largest z)            - ties with it stay  (:48-52)
//   top-p  : in descending order drop every token whose predecessors already
//            hold more than top_p of the (top-k filtered) softmax mass; the
//            first token always stays                                  (:54-68)
//   draw   : one token with probability softmax(z kept)                (:233-235)
//
// No sort.  Both thresholds are found by radix selection, 8 bits per pass, over
// an order preserving unsigned key: top-k counts elements per bin, top-p adds
// up probability mass per bin.  For bf16 logits the key is the 16-bit image of
// the logit itself (dividing by a positive temperature keeps order and, at
// bf16 spacing, never merges two values): 2 passes per threshold; for fp32 it
// is the 32-bit image of z: 4 passes.  Mass is held as 64-bit fixed point,
// q = round(exp(z - max) * 2^40), so that integer atomics give sums that do
// not depend on the order of addition: the kernel is reproducible bit for bit.
// The draw is the inverse CDF in index order on the same integers:
// token = first j with sum_{i<=j, kept} q_i > floor(u * Q).
//
// Every pass re-reads the row with 16-byte loads (L2 resident after the
// first): 1 (max) + 2 x 2 or 4 (thresholds) + 2 (draw) passes.  Where the
// reference keeps only some of several exactly equal logits at the top-p
// boundary (whichever its sort happened to put first), this kernel keeps all
// of them.
#include "mtp_common.h"

namespace {

constexpr int SP_THREADS = 1024;
constexpr int SP_WAVES = SP_THREADS / MTP_WAVE;
constexpr float SP_LOG2E = 1.4426950408889634f;
constexpr int SP_REP = 8;  // copies of the histogram: lanes of one instruction that hit the same bin are served one after another

// Element access: a row is cut into slots in index order: an unaligned head, 16-byte vectors, a tail.
template <typename T> struct Row;
template <> struct Row<float> {
  static constexpr int EPV = 4, KEY_BITS = 32;
  __device__ static __forceinline__ float ld(const float* p) { return *p; }
  __device__ static __forceinline__ void unpack(const u32x4_t& v, float* f) {
    f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y); f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
  }
  // ascending order preserving image of z (-0 and +0 coincide; NaN is not expected in logits)
  __device__ static __forceinline__ uint32_t key(float x, float z) {
    const uint32_t u = z == 0.0f ? 0u : __float_as_uint(z);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  }
};
template <> struct Row<uint16_t> {
  static constexpr int EPV = 8, KEY_BITS = 16;
  __device__ static __forceinline__ float ld(const uint16_t* p) { return bf16_bits_to_f32(*p); }
  __device__ static __forceinline__ void unpack(const u32x4_t& v, float* f) {
    f[0] = bf16_lo(v.x); f[1] = bf16_hi(v.x); f[2] = bf16_lo(v.y); f[3] = bf16_hi(v.y);
    f[4] = bf16_lo(v.z); f[5] = bf16_hi(v.z); f[6] = bf16_lo(v.w); f[7] = bf16_hi(v.w);
  }
  // 16-bit image of the bf16 logit itself: x -> x / T is strictly increasing on bf16 values
  __device__ static __forceinline__ uint32_t key(float x, float z) {
    const uint32_t u = x == 0.0f ? 0u : (__float_as_uint(x) >> 16);
    return (u & 0x8000u) ? (~u & 0xffffu) : (u | 0x8000u);
  }
};

template <typename T>
struct Slots {
  const T* row;
  int64_t V;
  int head;        // elements before the first 16-byte aligned address
  int64_t nvec;    // full vectors
  int64_t count;   // slots: head (may be empty), nvec vectors, tail (may be empty)
  __device__ __forceinline__ Slots(const T* r, int64_t v) : row(r), V(v) {
    constexpr int EPV = Row<T>::EPV;
    const uintptr_t mis = reinterpret_cast<uintptr_t>(r) & 15u;
    int h = mis ? (int)((16u - mis) / sizeof(T)) : 0;
    if (h > v) h = (int)v;
    head = h;
    nvec = (v - h) / EPV;
    count = nvec + 2;
  }
  // elements of slot s into x[], their first index into j0; returns how many
  __device__ __forceinline__ int load(int64_t s, float* x, int64_t& j0) const {
    constexpr int EPV = Row<T>::EPV;
    if (s >= 1 && s <= nvec) {
      j0 = head + (s - 1) * EPV;
      Row<T>::unpack(*reinterpret_cast<const u32x4_t*>(row + j0), x);
      return EPV;
    }
    int n;
    if (s == 0) {
      j0 = 0;
      n = head;
    } else {
      j0 = head + nvec * EPV;
      n = (int)(V - j0);
    }
#pragma unroll
    for (int e = 0; e < EPV; e++) x[e] = e < n ? Row<T>::ld(row + j0 + e) : 0.0f;
    return n;
  }
};

// f(x[EPV], n, j0) for every slot in [s_begin, s_end) taken `stride` apart starting at s_begin + first.  Four
// loads are issued before the first of them is used: with one load in flight per wave the passes run at
// the latency of L2, not its bandwidth.
template <typename T, typename F>
__device__ __forceinline__ void for_slots(const Slots<T>& sl, int64_t s_begin, int64_t s_end, int first, int stride,
                                          F&& f) {
  constexpr int EPV = Row<T>::EPV;
  int64_t s = s_begin + first;
  // slots 1..nvec are plain vectors; keep the unrolled part inside them
  for (; s >= 1 && s + 3 * (int64_t)stride <= sl.nvec && s + 3 * (int64_t)stride < s_end; s += 4 * (int64_t)stride) {
    u32x4_t v[4];
#pragma unroll
    for (int u = 0; u < 4; u++)
      v[u] = *reinterpret_cast<const u32x4_t*>(sl.row + sl.head + (s + u * (int64_t)stride - 1) * EPV);
#pragma unroll
    for (int u = 0; u < 4; u++) {
      float x[EPV];
      Row<T>::unpack(v[u], x);
      f(x, EPV, sl.head + (s + u * (int64_t)stride - 1) * EPV);
    }
  }
  for (; s < s_end; s += stride) {
    float x[EPV];
    int64_t j0;
    const int n = sl.load(s, x, j0);
    f(x, n, j0);
  }
}

// Probability mass relative to the row maximum, 40 fractional bits: round(exp(x/T - m) * 2^40) with the
// exponent argument formed as one fma, x * (log2(e)/T) - m*log2(e).  (The masses only have to be the same
// numbers in every pass; the filtered logits that leave the kernel are the true quotients x / T.)
struct Mass {
  float c1, mc;
  __device__ __forceinline__ Mass(float temperature, float m) : c1(SP_LOG2E / temperature), mc(m * SP_LOG2E) {}
  __device__ __forceinline__ uint64_t operator()(float x) const {
    const float f = __builtin_amdgcn_exp2f(__builtin_fmaf(x, c1, -mc)) * 1099511627776.0f;  // < 2^41
    const uint32_t hi = (uint32_t)(f * (1.0f / 65536.0f));
    const float rem = __builtin_fmaf(-(float)hi, 65536.0f, f);  // exact: f has 24 significant bits
    return ((uint64_t)hi << 16) + (uint32_t)(rem + 0.5f);
  }
};

__device__ __forceinline__ uint64_t wave_sum_u64(uint64_t v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += (uint64_t)__shfl_xor((long long)v, o, 64);
  return v;
}

// Histogram updates of one lane: logits of one row share their top key bits, so in the first pass nearly
// every element lands in the same two or three bins.  Each lane sums runs of equal bins privately and only
// touches LDS when the bin changes.
struct BinCache {
  int bin = -1;
  uint64_t acc = 0;
  __device__ __forceinline__ void add(uint64_t* bins, int b, uint64_t v) {
    if (b != bin) {
      flush(bins);
      bin = b;
    }
    acc += v;
  }
  __device__ __forceinline__ void flush(uint64_t* bins) {
    if (bin >= 0 && acc) atomicAdd((unsigned long long*)&bins[bin], (unsigned long long)acc);
    acc = 0;
  }
};

// Wave 0 scans 256 bins from the top: the first bin b with above(b) + bin(b) > limit.  Returns b (or -1)
// to every lane of wave 0 and the sum over the bins above it in `above` (the total when b = -1).
__device__ __forceinline__ int scan_bins_desc(const uint64_t* bins, uint64_t limit, int lane, uint64_t& above) {
  // lane l owns bins 255-4l .. 252-4l (descending order)
  uint64_t v[4], s = 0;
#pragma unroll
  for (int q = 0; q < 4; q++) {
    v[q] = bins[255 - 4 * lane - q];
    s += v[q];
  }
  uint64_t incl = s;  // inclusive prefix over lanes, in descending bin order
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const uint64_t t = (uint64_t)__shfl_up((long long)incl, o, 64);
    if (lane >= o) incl += t;
  }
  uint64_t run = incl - s;
  int found = -1;
  uint64_t found_above = 0;
#pragma unroll
  for (int q = 0; q < 4; q++) {
    if (found < 0 && run + v[q] > limit) {
      found = 255 - 4 * lane - q;
      found_above = run;
    }
    run += v[q];
  }
  const uint64_t has = __ballot(found >= 0);
  const uint64_t total = (uint64_t)__shfl((long long)incl, 63, 64);
  if (has == 0) {
    above = total;
    return -1;
  }
  const int src = __ffsll((long long)has) - 1;  // lowest lane = highest bins
  above = (uint64_t)__shfl((long long)found_above, src, 64);
  return __shfl(found, src, 64);
}

template <typename T>
__global__ __launch_bounds__(SP_THREADS) void sample_kernel(const T* __restrict__ logits, int64_t V,
                                                            float temperature, int top_k, float top_p,
                                                            const float* __restrict__ uniforms,
                                                            int64_t* __restrict__ tokens,
                                                            float* __restrict__ filtered) {
  constexpr int EPV = Row<T>::EPV, KEY_BITS = Row<T>::KEY_BITS;
  const Slots<T> sl(logits + (int64_t)blockIdx.x * V, V);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  __shared__ uint64_t bins_rep[SP_REP][256];
  uint64_t* const bins = bins_rep[lane & (SP_REP - 1)];  // this lane's copy; copy 0 holds the sum after fold
  __shared__ float red_f[SP_WAVES];
  __shared__ uint64_t red_u[SP_WAVES];
  __shared__ int sh_bin;
  __shared__ uint64_t sh_above;

  // ---- row maximum of z ---------------------------------------------------
  float m = -INFINITY;
  for_slots(sl, 0, sl.count, tid, SP_THREADS, [&](const float* x, int n, int64_t) {
#pragma unroll
    for (int e = 0; e < EPV; e++)
      if (e < n) m = fmaxf(m, x[e]);
  });
  m = wave_max(m);
  if (lane == 0) red_f[wave] = m;
  __syncthreads();
  m = red_f[0];
#pragma unroll
  for (int w = 1; w < SP_WAVES; w++) m = fmaxf(m, red_f[w]);
  m = m / temperature;  // x -> x / T is monotone: the maximum of the quotients is the quotient of the maximum
  const Mass mass(temperature, m);

  // ---- top-k: key of the k-th largest element -------------------------------
  uint32_t k_key = 0;  // elements with key < k_key are dropped
  if (top_k > 0 && top_k < V) {
    uint32_t prefix = 0;
    uint64_t want = (uint64_t)top_k;  // rank still to find inside the current prefix
    for (int shift = KEY_BITS - 8; shift >= 0; shift -= 8) {
      __syncthreads();
      for (int i = tid; i < SP_REP * 256; i += SP_THREADS) (&bins_rep[0][0])[i] = 0;
      __syncthreads();
      const uint32_t hi_mask = shift == KEY_BITS - 8 ? 0u : ~((1u << (shift + 8)) - 1u);
      BinCache cache;
      for_slots(sl, 0, sl.count, tid, SP_THREADS, [&](const float* x, int n, int64_t) {
#pragma unroll
        for (int e = 0; e < EPV; e++) {
          const uint32_t key = Row<T>::key(x[e], x[e] / temperature);
          if (e < n && (key & hi_mask) == prefix) cache.add(bins, (int)((key >> shift) & 0xff), 1ull);
        }
      });
      cache.flush(bins);
      __syncthreads();
      if (tid < 256) {
        uint64_t t = 0;
#pragma unroll
        for (int c = 0; c < SP_REP; c++) t += bins_rep[c][tid];
        bins_rep[0][tid] = t;
      }
      __syncthreads();
      if (wave == 0) {
        uint64_t above;
        const int b = scan_bins_desc(bins_rep[0], want - 1, lane, above);  // first bin with above + bin >= want
        if (lane == 0) {
          sh_bin = b;
          sh_above = above;
        }
      }
      __syncthreads();
      prefix |= (uint32_t)sh_bin << shift;
      want -= sh_above;
    }
    k_key = prefix;
  }

  // ---- top-p: key of the last token whose predecessors hold <= top_p of the mass ---
  uint32_t keep_key = k_key;
  if (top_p > 0.0f) {
    uint32_t prefix = 0;
    uint64_t limit = 0;
    bool all = false;
    for (int shift = KEY_BITS - 8; shift >= 0 && !all; shift -= 8) {
      __syncthreads();
      for (int i = tid; i < SP_REP * 256; i += SP_THREADS) (&bins_rep[0][0])[i] = 0;
      __syncthreads();
      const uint32_t hi_mask = shift == KEY_BITS - 8 ? 0u : ~((1u << (shift + 8)) - 1u);
      BinCache cache;
      for_slots(sl, 0, sl.count, tid, SP_THREADS, [&](const float* x, int n, int64_t) {
#pragma unroll
        for (int e = 0; e < EPV; e++) {
          const float z = x[e] / temperature;
          const uint32_t key = Row<T>::key(x[e], z);
          if (e < n && key >= k_key && (key & hi_mask) == prefix)
            cache.add(bins, (int)((key >> shift) & 0xff), mass(x[e]));
        }
      });
      cache.flush(bins);
      __syncthreads();
      if (tid < 256) {
        uint64_t t = 0;
#pragma unroll
        for (int c = 0; c < SP_REP; c++) t += bins_rep[c][tid];
        bins_rep[0][tid] = t;
      }
      __syncthreads();
      if (wave == 0) {
        if (shift == KEY_BITS - 8) {
          // total mass of the top-k survivors -> the limit in the same fixed point
          uint64_t t = 0;
#pragma unroll
          for (int q = 0; q < 4; q++) t += bins_rep[0][4 * lane + q];
          t = wave_sum_u64(t);
          const double lim = (double)top_p * (double)t;
          limit = lim >= 1.8e19 ? ~0ull : (uint64_t)lim;
        }
        uint64_t above;
        const int b = scan_bins_desc(bins_rep[0], limit, lane, above);
        if (lane == 0) {
          sh_bin = b;
          sh_above = above;
          red_u[0] = limit;
        }
      }
      __syncthreads();
      limit = red_u[0];
      if (sh_bin < 0) {
        all = true;  // the whole mass fits under top_p: nothing is dropped (top level only)
      } else {
        prefix |= (uint32_t)sh_bin << shift;
        limit -= sh_above;
      }
    }
    if (!all && prefix > keep_key) keep_key = prefix;
  }

  // ---- optional: the filtered logits the reference's top_k_logits returns -------
  if (filtered) {
    float* out = filtered + (int64_t)blockIdx.x * V;
    for_slots(sl, 0, sl.count, tid, SP_THREADS, [&](const float* x, int n, int64_t j0) {
#pragma unroll
      for (int e = 0; e < EPV; e++) {
        const float z = x[e] / temperature;
        if (e < n) out[j0 + e] = Row<T>::key(x[e], z) >= keep_key ? z : -INFINITY;
      }
    });
  }
  if (!tokens) return;

  // ---- draw: inverse CDF in index order.  Wave w owns a contiguous range of slots, a step is 64 slots,
  // lane l the l-th of them: slot order = index order.
  const int64_t per_wave = (sl.count + SP_WAVES - 1) / SP_WAVES;
  const int64_t s0 = (int64_t)wave * per_wave;
  const int64_t s1 = s0 + per_wave < sl.count ? s0 + per_wave : sl.count;
  auto slot_mass = [&](int64_t s, uint64_t* q, int64_t& j0) -> uint64_t {  // masses of the kept elements of slot s
    float x[EPV] = {};
    int n = 0;
    j0 = 0;
    if (s < s1) n = sl.load(s, x, j0);
    uint64_t t = 0;
#pragma unroll
    for (int e = 0; e < EPV; e++) {
      const float z = x[e] / temperature;
      q[e] = (e < n && Row<T>::key(x[e], z) >= keep_key) ? mass(x[e]) : 0;
      t += q[e];
    }
    return t;
  };
  uint64_t mine = 0;
  for_slots(sl, s0, s1, lane, 64, [&](const float* x, int n, int64_t) {
#pragma unroll
    for (int e = 0; e < EPV; e++) {
      const float z = x[e] / temperature;
      if (e < n && Row<T>::key(x[e], z) >= keep_key) mine += mass(x[e]);
    }
  });
  mine = wave_sum_u64(mine);
  __syncthreads();
  if (lane == 0) red_u[wave] = mine;
  __syncthreads();
  uint64_t total = 0;
#pragma unroll
  for (int w = 0; w < SP_WAVES; w++) total += red_u[w];
  // total >= 2^40 (the maximum itself is always kept)
  float u = uniforms[blockIdx.x];
  u = u < 0.0f ? 0.0f : u;
  uint64_t r = (uint64_t)((double)u * (double)total);
  if (r >= total) r = total - 1;
  uint64_t before = 0;
  int pick_wave = -1;
#pragma unroll
  for (int w = 0; w < SP_WAVES; w++) {
    if (pick_wave < 0) {
      if (before + red_u[w] > r)
        pick_wave = w;
      else
        before += red_u[w];
    }
  }
  if (wave != pick_wave) return;
  uint64_t run = before;
  for (int64_t base = s0; base < s1; base += 64) {
    uint64_t q[EPV];
    int64_t j0;
    const uint64_t t = slot_mass(base + lane, q, j0);
    uint64_t incl = t;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const uint64_t up = (uint64_t)__shfl_up((long long)incl, o, 64);
      if (lane >= o) incl += up;
    }
    const uint64_t hit = __ballot(run + incl > r);
    if (hit) {
      if (lane == __ffsll((long long)hit) - 1) {
        // the crossing lies inside this lane's slot: walk its elements
        uint64_t acc = run + incl - t;
        int64_t pick = -1;
#pragma unroll
        for (int e = 0; e < EPV; e++) {
          acc += q[e];
          if (pick < 0 && q[e] > 0 && acc > r) pick = j0 + e;
        }
        tokens[blockIdx.x] = pick;
      }
      return;
    }
    run += (uint64_t)__shfl((long long)incl, 63, 64);
  }
}

}  // namespace

extern "C" int mtp_sample_top_k_top_p(const void* logits, int dtype, int64_t B, int64_t V, float temperature,
                                      int top_k, float top_p, const float* uniforms, int64_t* tokens,
                                      float* filtered, void* stream) {
  MTP_REQUIRE(B >= 0 && V >= 1, MTP_EINVAL, "sample: B=%lld V=%lld", (long long)B, (long long)V);
  MTP_REQUIRE(B < (1ll << 31) && V < (1ll << 31), MTP_EUNSUPPORTED, "sample: a dimension exceeds 2^31-1");
  MTP_REQUIRE(dtype == MTP_F32 || dtype == MTP_BF16, MTP_EINVAL, "sample: unknown dtype %d", dtype);
  MTP_REQUIRE(temperature > 0.0f && temperature == temperature, MTP_EINVAL, "sample: temperature must be positive");
  MTP_REQUIRE(top_k >= 0 && top_p >= 0.0f, MTP_EINVAL, "sample: top_k=%d top_p=%g", top_k, (double)top_p);
  // torch.topk in the reference (:50) refuses k beyond the row length
  MTP_REQUIRE(top_k <= V, MTP_EINVAL, "sample: top_k=%d out of range for %lld logits per row", top_k, (long long)V);
  if (B == 0) return MTP_OK;
  MTP_REQUIRE(logits && (tokens || filtered), MTP_EINVAL, "sample: null pointer");
  MTP_REQUIRE(!tokens || uniforms, MTP_EINVAL, "sample: tokens requested without uniforms");
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MTP_F32)
    hipLaunchKernelGGL(sample_kernel<float>, dim3((unsigned)B), dim3(SP_THREADS), 0, s, (const float*)logits, V,
                       temperature, top_k, top_p, uniforms, tokens, filtered);
  else
    hipLaunchKernelGGL(sample_kernel<uint16_t>, dim3((unsigned)B), dim3(SP_THREADS), 0, s, (const uint16_t*)logits, V,
                       temperature, top_k, top_p, uniforms, tokens, filtered);
  MTP_CHECK_LAUNCH("sample");
  return MTP_OK;
}
