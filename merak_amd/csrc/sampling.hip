// Sampling tail of the decode loop for gfx950: temperature, top-k, top-p and
// one multinomial draw per batch row
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
// not depend on the order of addition: the result is reproducible bit for bit.
// The draw is the inverse CDF in index order on the same integers:
// token = first j with sum_{i<=j, kept} q_i > floor(u * Q).
//
// The work per element is a few dozen VALU instructions, and a decode batch
// has few rows, so every row is spread over SG workgroups and every pass is a
// launch of its own (B * SG workgroups): the per-pass histograms live in a
// caller-supplied workspace, each launch re-derives the state of the selection
// from the histograms of the passes before it (a 256-bin scan by one wave), and
// kernel boundaries are the only synchronisation.  Where the reference keeps
// only some of several exactly equal logits at the top-p boundary (whichever its
// sort happened to put first), these kernels keep all of them.
#include "mtp_common.h"

namespace {

constexpr int SP_THREADS = 256;
constexpr int SP_WAVES = SP_THREADS / MTP_WAVE;
constexpr int SG = 32;       // workgroups per row
constexpr int SP_MAXPASS = 8;
constexpr float SP_LOG2E = 1.4426950408889634f;
constexpr int SP_REP = 4;    // copies of the LDS histogram: lanes of one instruction that hit the same bin are served one after another

// Per batch row, in the workspace.
struct RowState {
  uint32_t max_key;              // order preserving image of the largest logit of the row
  uint32_t keep_key;             // elements with key >= keep_key survive both filters
  uint32_t pad[2];
  uint64_t part[SG];             // kept mass of each chunk of the row, chunks in index order
  uint64_t hist[SP_MAXPASS][256];  // one histogram per selection pass: top-k passes first, then top-p
};

__device__ __forceinline__ uint32_t f32_key(float v) {
  const uint32_t u = v == 0.0f ? 0u : __float_as_uint(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float f32_unkey(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k ^ 0x80000000u) : ~k);
}

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

template <> struct Row<f16s> {
  static constexpr int EPV = 8, KEY_BITS = 16;
  using H = X16<true>;
  __device__ static __forceinline__ float ld(const f16s* p) { return H::from_bits(p->bits); }
  __device__ static __forceinline__ void unpack(const u32x4_t& v, float* f) {
    f[0] = H::lo(v.x); f[1] = H::hi(v.x); f[2] = H::lo(v.y); f[3] = H::hi(v.y);
    f[4] = H::lo(v.z); f[5] = H::hi(v.z); f[6] = H::lo(v.w); f[7] = H::hi(v.w);
  }
  // 16-bit image of the half logit itself (the conversion back is exact): x -> x / T is increasing on it
  __device__ static __forceinline__ uint32_t key(float x, float z) {
    const uint32_t u = x == 0.0f ? 0u : (uint32_t)H::to_bits(x);
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


// State of the selection after the first `done` passes, replayed from their histograms by wave 0 and
// broadcast through LDS.  All threads of the workgroup must call it.
struct Selection {
  uint32_t k_key;     // valid once all top-k passes are done (0: no top-k)
  uint32_t prefix;    // key bits fixed so far in the phase that pass `done` belongs to
  uint64_t limit;     // top-p: mass that may lie above the threshold inside the current prefix
  uint64_t want;      // top-k: rank still to find inside the current prefix
  bool all;           // top-p: the whole mass fits under top_p, nothing is dropped
};

template <int KEY_BITS>
__device__ Selection replay(const RowState* st, int done, int top_k_passes, int top_p_passes, int top_k,
                            float top_p) {
  __shared__ Selection sh;
  const int lane = threadIdx.x & 63;
  if (threadIdx.x < 64) {
    Selection s{0u, 0u, 0ull, (uint64_t)top_k, false};
    int pass = 0;
    for (int lvl = 0; lvl < top_k_passes && pass < done; lvl++, pass++) {
      const int shift = KEY_BITS - 8 - 8 * lvl;
      uint64_t above;
      const int b = scan_bins_desc(st->hist[pass], s.want - 1, lane, above);  // first bin with above + bin >= want
      s.prefix |= (uint32_t)b << shift;
      s.want -= above;
      if (lvl == top_k_passes - 1) {
        s.k_key = s.prefix;
        s.prefix = 0;
      }
    }
    for (int lvl = 0; lvl < top_p_passes && pass < done && !s.all; lvl++, pass++) {
      const int shift = KEY_BITS - 8 - 8 * lvl;
      if (lvl == 0) {
        // total mass of the top-k survivors -> the limit in the same fixed point
        uint64_t t = 0;
#pragma unroll
        for (int q = 0; q < 4; q++) t += st->hist[pass][4 * lane + q];
        t = wave_sum_u64(t);
        const double lim = (double)top_p * (double)t;
        s.limit = lim >= 1.8e19 ? ~0ull : (uint64_t)lim;
      }
      uint64_t above;
      const int b = scan_bins_desc(st->hist[pass], s.limit, lane, above);
      if (b < 0) {
        s.all = true;
      } else {
        s.prefix |= (uint32_t)b << shift;
        s.limit -= above;
      }
    }
    if (lane == 0) sh = s;
  }
  __syncthreads();
  return sh;
}

__global__ __launch_bounds__(256) void sample_init_kernel(RowState* __restrict__ st, int64_t words) {
  uint64_t* p = reinterpret_cast<uint64_t*>(st);
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += stride) p[i] = 0;
}

// slots [s0, s1) of chunk g of a row
template <typename T>
__device__ __forceinline__ void chunk_range(const Slots<T>& sl, int g, int64_t& s0, int64_t& s1) {
  const int64_t per = (sl.count + SG - 1) / SG;
  s0 = (int64_t)g * per;
  s1 = s0 + per < sl.count ? s0 + per : sl.count;
  if (s0 > s1) s0 = s1;
}

template <typename T>
__global__ __launch_bounds__(SP_THREADS) void sample_max_kernel(const T* __restrict__ logits, int64_t V,
                                                                RowState* __restrict__ state) {
  constexpr int EPV = Row<T>::EPV;
  const int b = blockIdx.x / SG, g = blockIdx.x % SG;
  const Slots<T> sl(logits + (int64_t)b * V, V);
  int64_t s0, s1;
  chunk_range(sl, g, s0, s1);
  float m = -INFINITY;
  for_slots(sl, s0, s1, threadIdx.x, SP_THREADS, [&](const float* x, int n, int64_t) {
#pragma unroll
    for (int e = 0; e < EPV; e++)
      if (e < n) m = fmaxf(m, x[e]);
  });
  m = wave_max(m);
  if ((threadIdx.x & 63) == 0 && m > -INFINITY) atomicMax(&state[b].max_key, f32_key(m));
}

// One selection pass over one chunk: histogram of the digit at `pass` of the elements inside the current prefix
template <typename T>
__global__ __launch_bounds__(SP_THREADS) void sample_hist_kernel(const T* __restrict__ logits, int64_t V,
                                                                 float temperature, int top_k, float top_p,
                                                                 int top_k_passes, int top_p_passes, int pass,
                                                                 RowState* __restrict__ state) {
  constexpr int EPV = Row<T>::EPV, KEY_BITS = Row<T>::KEY_BITS;
  const int b = blockIdx.x / SG, g = blockIdx.x % SG;
  const int tid = threadIdx.x, lane = tid & 63;
  RowState* st = state + b;
  const Selection sel = replay<KEY_BITS>(st, pass, top_k_passes, top_p_passes, top_k, top_p);
  const bool mass_phase = pass >= top_k_passes;
  if (mass_phase && sel.all) return;  // nothing more to find
  const int lvl = mass_phase ? pass - top_k_passes : pass;
  const int shift = KEY_BITS - 8 - 8 * lvl;
  const uint32_t hi_mask = lvl == 0 ? 0u : ~((1u << (shift + 8)) - 1u);
  const uint32_t prefix = sel.prefix, k_key = sel.k_key;
  const Mass mass(temperature, f32_unkey(st->max_key) / temperature);

  __shared__ uint64_t bins_rep[SP_REP][256];
  for (int i = tid; i < SP_REP * 256; i += SP_THREADS) (&bins_rep[0][0])[i] = 0;
  __syncthreads();
  uint64_t* const bins = bins_rep[lane & (SP_REP - 1)];
  const Slots<T> sl(logits + (int64_t)b * V, V);
  int64_t s0, s1;
  chunk_range(sl, g, s0, s1);
  for_slots(sl, s0, s1, tid, SP_THREADS, [&](const float* x, int n, int64_t) {
#pragma unroll
    for (int e = 0; e < EPV; e++) {
      const float z = x[e] / temperature;
      const uint32_t key = Row<T>::key(x[e], z);
      if (e < n && (key & hi_mask) == prefix && (!mass_phase || key >= k_key))
        atomicAdd((unsigned long long*)&bins[(key >> shift) & 0xff], mass_phase ? (unsigned long long)mass(x[e]) : 1ull);
    }
  });
  __syncthreads();
  uint64_t t = 0;
#pragma unroll
  for (int c = 0; c < SP_REP; c++) t += bins_rep[c][tid];
  if (t) atomicAdd((unsigned long long*)&st->hist[pass][tid], (unsigned long long)t);
}

// Kept mass of every chunk (and the filtered logits, if asked for)
template <typename T>
__global__ __launch_bounds__(SP_THREADS) void sample_mass_kernel(const T* __restrict__ logits, int64_t V,
                                                                 float temperature, int top_k, float top_p,
                                                                 int top_k_passes, int top_p_passes,
                                                                 RowState* __restrict__ state,
                                                                 float* __restrict__ filtered) {
  constexpr int EPV = Row<T>::EPV, KEY_BITS = Row<T>::KEY_BITS;
  const int b = blockIdx.x / SG, g = blockIdx.x % SG;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  RowState* st = state + b;
  const Selection sel = replay<KEY_BITS>(st, top_k_passes + top_p_passes, top_k_passes, top_p_passes, top_k, top_p);
  uint32_t keep_key = sel.k_key;
  if (top_p_passes && !sel.all && sel.prefix > keep_key) keep_key = sel.prefix;
  const Mass mass(temperature, f32_unkey(st->max_key) / temperature);
  const Slots<T> sl(logits + (int64_t)b * V, V);
  int64_t s0, s1;
  chunk_range(sl, g, s0, s1);
  float* out = filtered ? filtered + (int64_t)b * V : nullptr;
  uint64_t mine = 0;
  for_slots(sl, s0, s1, tid, SP_THREADS, [&](const float* x, int n, int64_t j0) {
#pragma unroll
    for (int e = 0; e < EPV; e++) {
      const float z = x[e] / temperature;
      const bool keep = Row<T>::key(x[e], z) >= keep_key;
      if (e < n && keep) mine += mass(x[e]);
      if (out && e < n) out[j0 + e] = keep ? z : -INFINITY;
    }
  });
  mine = wave_sum_u64(mine);
  __shared__ uint64_t red[SP_WAVES];
  if (lane == 0) red[wave] = mine;
  __syncthreads();
  if (tid == 0) {
    uint64_t t = 0;
#pragma unroll
    for (int w = 0; w < SP_WAVES; w++) t += red[w];
    st->part[g] = t;
    if (g == 0) st->keep_key = keep_key;
  }
}

// The draw: one workgroup per row finds the chunk that holds the target mass; its 16 waves split that chunk's
// slots into contiguous ranges, sum them, and the wave whose range holds the target walks it 64 slots at a time.
constexpr int DR_WAVES = 16;
template <typename T>
__global__ __launch_bounds__(DR_WAVES * 64) void sample_draw_kernel(const T* __restrict__ logits, int64_t V,
                                                                    float temperature,
                                                                    const float* __restrict__ uniforms,
                                                                    const RowState* __restrict__ state,
                                                                    int64_t* __restrict__ tokens) {
  constexpr int EPV = Row<T>::EPV;
  const int b = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const RowState* st = state + b;
  uint64_t total = 0;
  for (int g = 0; g < SG; g++) total += st->part[g];
  // total >= 2^40 (the maximum itself is always kept)
  float u = uniforms[b];
  u = u < 0.0f ? 0.0f : u;
  uint64_t r = (uint64_t)((double)u * (double)total);
  if (r >= total) r = total - 1;
  uint64_t run = 0;
  int pick = 0;
  for (int g = 0; g < SG; g++) {
    if (run + st->part[g] > r) {
      pick = g;
      break;
    }
    run += st->part[g];
  }
  const uint32_t keep_key = st->keep_key;
  const Mass mass(temperature, f32_unkey(st->max_key) / temperature);
  const Slots<T> sl(logits + (int64_t)b * V, V);
  int64_t c0, c1;
  chunk_range(sl, pick, c0, c1);
  const int64_t per_wave = ((c1 - c0 + DR_WAVES * 64 - 1) / (DR_WAVES * 64)) * 64;  // whole steps of 64 slots
  int64_t s0 = c0 + (int64_t)wave * per_wave, s1 = s0 + per_wave;
  if (s0 > c1) s0 = c1;
  if (s1 > c1) s1 = c1;
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
  for (int64_t s = s0 + lane; s < s1; s += 64) {
    uint64_t q[EPV];
    int64_t j0;
    mine += slot_mass(s, q, j0);
  }
  mine = wave_sum_u64(mine);
  __shared__ uint64_t red[DR_WAVES];
  if (lane == 0) red[wave] = mine;
  __syncthreads();
  int pick_wave = -1;
#pragma unroll
  for (int w = 0; w < DR_WAVES; w++) {
    if (pick_wave < 0) {
      if (run + red[w] > r)
        pick_wave = w;
      else
        run += red[w];
    }
  }
  if (wave != pick_wave) return;
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
        int64_t tok = -1;
#pragma unroll
        for (int e = 0; e < EPV; e++) {
          acc += q[e];
          if (tok < 0 && q[e] > 0 && acc > r) tok = j0 + e;
        }
        tokens[b] = tok;
      }
      return;
    }
    run += (uint64_t)__shfl((long long)incl, 63, 64);
  }
}

template <typename T>
int launch_sample(const void* logits, int64_t B, int64_t V, float temperature, int top_k, float top_p,
                  const float* uniforms, int64_t* tokens, float* filtered, RowState* state, hipStream_t s) {
  const T* lg = (const T*)logits;
  const int per_threshold = Row<T>::KEY_BITS / 8;
  const int kp = (top_k > 0 && top_k < V) ? per_threshold : 0;
  const int pp = top_p > 0.0f ? per_threshold : 0;
  const dim3 grid((unsigned)(B * SG)), block(SP_THREADS);
  const int64_t words = B * (int64_t)(sizeof(RowState) / 8);
  hipLaunchKernelGGL(sample_init_kernel, dim3((unsigned)((words + 255) / 256 < 1024 ? (words + 255) / 256 : 1024)),
                     dim3(256), 0, s, state, words);
  hipLaunchKernelGGL(sample_max_kernel<T>, grid, block, 0, s, lg, V, state);
  for (int pass = 0; pass < kp + pp; pass++)
    hipLaunchKernelGGL(sample_hist_kernel<T>, grid, block, 0, s, lg, V, temperature, top_k, top_p, kp, pp, pass, state);
  hipLaunchKernelGGL(sample_mass_kernel<T>, grid, block, 0, s, lg, V, temperature, top_k, top_p, kp, pp, state,
                     filtered);
  if (tokens)
    hipLaunchKernelGGL(sample_draw_kernel<T>, dim3((unsigned)B), dim3(DR_WAVES * 64), 0, s, lg, V, temperature, uniforms, state,
                       tokens);
  MTP_CHECK_LAUNCH("sample");
  return MTP_OK;
}

}  // namespace

extern "C" int64_t mtp_sample_workspace_bytes(int64_t B) { return B > 0 ? B * (int64_t)sizeof(RowState) : 0; }

extern "C" int mtp_sample_top_k_top_p(const void* logits, int dtype, int64_t B, int64_t V, float temperature,
                                      int top_k, float top_p, const float* uniforms, int64_t* tokens,
                                      float* filtered, void* workspace, int64_t workspace_bytes, void* stream) {
  MTP_REQUIRE(B >= 0 && V >= 1, MTP_EINVAL, "sample: B=%lld V=%lld", (long long)B, (long long)V);
  MTP_REQUIRE(B < (1ll << 24) && V < (1ll << 31), MTP_EUNSUPPORTED, "sample: B=%lld or V=%lld too large", (long long)B,
              (long long)V);
  MTP_REQUIRE(dtype == MTP_F32 || dtype == MTP_BF16 || dtype == MTP_F16, MTP_EINVAL, "sample: unknown dtype %d", dtype);
  MTP_REQUIRE(temperature > 0.0f && temperature == temperature, MTP_EINVAL, "sample: temperature must be positive");
  MTP_REQUIRE(top_k >= 0 && top_p >= 0.0f, MTP_EINVAL, "sample: top_k=%d top_p=%g", top_k, (double)top_p);
  // torch.topk in the reference (:50) refuses k beyond the row length
  MTP_REQUIRE(top_k <= V, MTP_EINVAL, "sample: top_k=%d out of range for %lld logits per row", top_k, (long long)V);
  if (B == 0) return MTP_OK;
  MTP_REQUIRE(logits && (tokens || filtered), MTP_EINVAL, "sample: null pointer");
  MTP_REQUIRE(!tokens || uniforms, MTP_EINVAL, "sample: tokens requested without uniforms");
  MTP_REQUIRE(workspace && workspace_bytes >= mtp_sample_workspace_bytes(B), MTP_EWORKSPACE,
              "sample: workspace %lld < %lld bytes", (long long)workspace_bytes, (long long)mtp_sample_workspace_bytes(B));
  MTP_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 7) == 0, MTP_EINVAL, "sample: workspace not 8-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MTP_F32)
    return launch_sample<float>(logits, B, V, temperature, top_k, top_p, uniforms, tokens, filtered,
                                (RowState*)workspace, s);
  if (dtype == MTP_F16)
    return launch_sample<f16s>(logits, B, V, temperature, top_k, top_p, uniforms, tokens, filtered,
                               (RowState*)workspace, s);
  return launch_sample<uint16_t>(logits, B, V, temperature, top_k, top_p, uniforms, tokens, filtered,
                                 (RowState*)workspace, s);
}
