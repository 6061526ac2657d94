// Single-token decode step of a Llama-shaped block around the tensor-parallel linears, for gfx950:
// RMSNorm (with the residual add in front of it), rotary embedding of the new query/key with the append of
// the new key/value to a cache, and attention of the new query over the cached keys and values.
//
// The reference's generation loop re-runs the whole sequence for every token and keeps only position
// context_length-1 of the output (Merak/inference/text_generation_inference.py:199-203,223).  For a causal
// model that row depends on the earlier positions only through their keys and values, so keeping those in a
// cache and running one position gives the same row: that is what these kernels compute, for the HF Llama
// block the reference's examples wrap (LlamaRMSNorm, apply_rotary_pos_emb, grouped-query attention with the
// softmax in fp32).
//
// Cache layout: [batch, kv_head, max_len, 128] bf16, so the keys (values) of one (batch, kv_head) are one
// contiguous stream of 256-byte rows - what the attention kernel reads.
//
// attn_decode_kernel - bound: HBM (it streams len x 512 bytes per (batch, kv_head)):
//   * grid (splits, kv_heads, batch); a workgroup of 4 waves owns a range of 32-token tiles, its waves take
//     every fourth tile, each wave runs its own flash-style recurrence and the four are merged at the end;
//   * K and V tiles (8 KiB each) go global -> LDS by `buffer_load_dwordx4 ... lds` in 1 KiB contiguous
//     pieces into a per-wave ring of 4 slots: up to three of them are in flight while one is used.  A
//     wave only ever reads what it requested itself, so the main loop has no workgroup barrier, just
//     s_waitcnt vmcnt(n).  Rows past the sequence length read as zero through the buffer range check;
//   * the q heads that share a kv head (the group, up to 16) are the N dimension of
//     v_mfma_f32_16x16x32_bf16: S^T = K Q^T (tokens x heads), then O^T = V^T P^T (dims x heads).
//     In that orientation a lane owns one head, so the running maximum, the rescale factor and the
//     exponentials are per-lane scalars, and the S^T accumulators already sit where the second
//     product wants its B operand (no data movement for P).  K fragments are ds_read_b128,
//     V^T fragments ds_read_b64_tr_b16; 16-byte chunks of a row are stored at chunk ^ (token & 15),
//     which makes both conflict free;
//   * several splits: partial (O, max, sum) per split in a workspace and a small merge kernel.
#include "gemm_bf16_kernel.h"

namespace {

constexpr int AD_D = 128;                      // head dimension
constexpr int AD_TILE = 32;                    // tokens per tile
constexpr int AD_ITEM = AD_TILE * AD_D * 2;    // bytes of the K (or V) rows of one tile
constexpr int AD_RING = 4;                     // ring slots per wave
constexpr int AD_WAVES = 4;
constexpr int AD_PART = AD_D + 2;              // floats per partial result: O[128], max, sum
constexpr int AD_MAX_GROUP = 16;

struct AttnArgs {
  const uint16_t* q;      // [B, n_q_heads, 128]
  const uint16_t* k;      // [B, n_kv_heads, max_len, 128]
  const uint16_t* v;
  const int64_t* lens;    // [B] tokens to attend to (the new one included)
  uint16_t* out;          // [B, n_q_heads, 128]
  float* part;            // [B, n_q_heads, splits, AD_PART] when splits > 1
  int n_q_heads, n_kv_heads, group;
  int64_t max_len;
  int splits;
  float scale_log2e;      // softmax scale * log2(e)
};

__device__ __forceinline__ void wait_vm(int items_after) {
  // every item is 8 DMA instructions; "memory": LDS reads below must not move above the wait
  switch (items_after) {
    case 3: asm volatile("s_waitcnt vmcnt(24)" ::: "memory"); break;
    case 2: asm volatile("s_waitcnt vmcnt(16)" ::: "memory"); break;
    case 1: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
  }
}

__device__ __forceinline__ void attn_decode_body(const AttnArgs& p) {
  __shared__ __attribute__((aligned(1024))) char lds[AD_WAVES * AD_RING * AD_ITEM];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int G = p.group;
  const int h = lane & 15, q = lane >> 4;

  int64_t len = p.lens[b];
  len = len < 0 ? 0 : (len > p.max_len ? p.max_len : len);
  const int tiles = (int)((len + AD_TILE - 1) / AD_TILE);
  const int tps = (tiles + p.splits - 1) / p.splits;
  const int tile_lo = split * tps;
  const int tile_hi = tile_lo + tps < tiles ? tile_lo + tps : tiles;
  const int first = tile_lo + wave;
  const int n_my = tile_hi > first ? (tile_hi - first + AD_WAVES - 1) / AD_WAVES : 0;
  const int n_items = 2 * n_my;

  // this lane's share of Q^T as MFMA B operand: head h, dims 32c + 8q .. +7
  bf16x8_t qf[4];
  {
    const uint16_t* qrow = p.q + ((int64_t)b * p.n_q_heads + (int64_t)kvh * G + (h < G ? h : 0)) * AD_D;
#pragma unroll
    for (int c = 0; c < 4; c++) {
      u32x4_t raw = *reinterpret_cast<const u32x4_t*>(qrow + 32 * c + 8 * q);
      if (h >= G) raw = u32x4_t{0, 0, 0, 0};
      qf[c] = __builtin_bit_cast(bf16x8_t, raw);
    }
  }

  // DMA: instruction j of an item fills LDS rows (tokens) 4j .. 4j+3; lane -> token 4j + lane/16, LDS
  // chunk position lane%16, which holds the row's chunk position ^ (token & 15)
  uint32_t voff[4];
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int t = 4 * j + q;
    voff[j] = (uint32_t)(t * 256 + ((h ^ (t & 15)) << 4));
  }
  const uint32_t ring0 = __builtin_amdgcn_readfirstlane(lds_addr_of(lds)) + wave * (AD_RING * AD_ITEM);
  const char* ring = lds + wave * (AD_RING * AD_ITEM);
  const int64_t head_rows = ((int64_t)b * p.n_kv_heads + kvh) * p.max_len;

  auto issue = [&](int it) {
    // the slot's earlier contents have been read: keep those reads in front of the DMA, and wait for them
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const int64_t tok0 = (int64_t)(first + AD_WAVES * (it >> 1)) * AD_TILE;
    const char* base = reinterpret_cast<const char*>((it & 1) ? p.v : p.k) + (head_rows + tok0) * (AD_D * 2);
    const rsrc_t r = make_rsrc(base, (len - tok0) * (AD_D * 2));
    const uint32_t slot = ring0 + (it & (AD_RING - 1)) * AD_ITEM;
#pragma unroll
    for (int j = 0; j < 8; j++) dma16(r, slot + j * 1024, voff[j & 3] + (j >> 2) * 4096, 0);
  };

  // fragment addresses inside a slot
  //   K (A operand of S^T = K Q^T): lane (token m = lane%16, q) reads chunk 4c + q of rows m and 16 + m
  //   V^T (A operand of O^T = V^T P^T): in each group of 16 lanes, lane i addresses token 4q + i/4,
  //   dims 16dt + 4(i%4) .. +3 and receives dims 16dt + i of tokens 4q .. 4q+3 (second read: tokens + 16)
  const uint32_t krow = (uint32_t)(h * 256);
  const int vt = 4 * q + (h >> 2);
  const uint32_t vrow = (uint32_t)(vt * 256 + 8 * (h & 1));
  const int vc0 = (h & 3) >> 1;

  float m_run = -INFINITY, l_run = 0.0f;
  f32x4_t o[8];
#pragma unroll
  for (int dt = 0; dt < 8; dt++) o[dt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  if (n_items > 0) issue(0);
  if (n_items > 1) issue(1);
  if (n_items > 2) issue(2);

  for (int i = 0; i < n_my; i++) {
    // ---- K: scores of 32 tokens for the heads of the group ----
    {
      const int it = 2 * i;
      if (it + 3 < n_items) issue(it + 3);
      const int after = n_items - 1 - it;
      wait_vm(after < 3 ? after : 3);
    }
    const char* kslot = ring + ((2 * i) & (AD_RING - 1)) * AD_ITEM;
    f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 4; c++) {
      const uint32_t off = krow + (uint32_t)(((4 * c + q) ^ h) << 4);
      const bf16x8_t a0 = *reinterpret_cast<const bf16x8_t*>(kslot + off);
      const bf16x8_t a1 = *reinterpret_cast<const bf16x8_t*>(kslot + off + 16 * 256);
      s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, qf[c], s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, qf[c], s1, 0, 0, 0);
    }
    // this lane: head h, tokens 4q + j (s0) and 16 + 4q + j (s1) of the tile
    const int64_t valid = len - (int64_t)(first + AD_WAVES * i) * AD_TILE;
    float x0[4], x1[4];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      x0[j] = (4 * q + j) < valid ? s0[j] * p.scale_log2e : -INFINITY;
      x1[j] = (16 + 4 * q + j) < valid ? s1[j] * p.scale_log2e : -INFINITY;
      mx = fmaxf(mx, fmaxf(x0[j], x1[j]));
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m_run, mx);   // finite: the first token of a tile is always valid
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    m_run = m_new;
    float psum = 0.0f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      x0[j] = __builtin_amdgcn_exp2f(x0[j] - m_new);
      x1[j] = __builtin_amdgcn_exp2f(x1[j] - m_new);
      psum += x0[j] + x1[j];
    }
    l_run = l_run * alpha + psum;
    const u32x4_t praw = {pack_bf16x2(x0[0], x0[1]), pack_bf16x2(x0[2], x0[3]), pack_bf16x2(x1[0], x1[1]),
                          pack_bf16x2(x1[2], x1[3])};
    const bf16x8_t pf = __builtin_bit_cast(bf16x8_t, praw);
#pragma unroll
    for (int dt = 0; dt < 8; dt++) o[dt] *= alpha;

    // ---- V: O^T += V^T P^T ----
    {
      const int it = 2 * i + 1;
      if (it + 3 < n_items) issue(it + 3);
      const int after = n_items - 1 - it;
      wait_vm(after < 3 ? after : 3);
    }
    const char* vslot = ring + ((2 * i + 1) & (AD_RING - 1)) * AD_ITEM;
#pragma unroll
    for (int dt = 0; dt < 8; dt++) {
      const char* a = vslot + vrow + (uint32_t)(((2 * dt + vc0) ^ (vt & 15)) << 4);
      const bf16x4_t lo =
          __builtin_amdgcn_ds_read_tr16_b64_v4bf16((bf16x4_t __attribute__((address_space(3)))*)(a));
      const bf16x4_t hi =
          __builtin_amdgcn_ds_read_tr16_b64_v4bf16((bf16x4_t __attribute__((address_space(3)))*)(a + 16 * 256));
      const bf16x8_t vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, o[dt], 0, 0, 0);
    }
  }

  // ---- merge the four waves (each owns head h in lanes h, h+16, h+32, h+48) ----
  l_run += __shfl_xor(l_run, 16, 64);
  l_run += __shfl_xor(l_run, 32, 64);
  __syncthreads();   // every wave is done with its ring (all DMA waited for, all reads consumed)
  float* mine = reinterpret_cast<float*>(lds + wave * (AD_RING * AD_ITEM));
  if (h < G) {
#pragma unroll
    for (int dt = 0; dt < 8; dt++) *reinterpret_cast<f32x4_t*>(mine + h * AD_D + 16 * dt + 4 * q) = o[dt];
    if (q == 0) {
      mine[AD_MAX_GROUP * AD_D + 2 * h] = m_run;
      mine[AD_MAX_GROUP * AD_D + 2 * h + 1] = l_run;
    }
  }
  __syncthreads();
  for (int idx = tid; idx < G * AD_D; idx += AD_WAVES * 64) {
    const int hh = idx >> 7, d = idx & (AD_D - 1);
    float mw[AD_WAVES], mstar = -INFINITY;
#pragma unroll
    for (int w = 0; w < AD_WAVES; w++) {
      mw[w] = reinterpret_cast<const float*>(lds + w * (AD_RING * AD_ITEM))[AD_MAX_GROUP * AD_D + 2 * hh];
      mstar = fmaxf(mstar, mw[w]);
    }
    float acc = 0.0f, l = 0.0f;
#pragma unroll
    for (int w = 0; w < AD_WAVES; w++) {
      if (mw[w] == -INFINITY) continue;
      const float* src = reinterpret_cast<const float*>(lds + w * (AD_RING * AD_ITEM));
      const float f = __builtin_amdgcn_exp2f(mw[w] - mstar);
      acc += src[hh * AD_D + d] * f;
      l += src[AD_MAX_GROUP * AD_D + 2 * hh + 1] * f;
    }
    const int64_t hq = (int64_t)b * p.n_q_heads + (int64_t)kvh * G + hh;
    if (p.splits == 1) {
      p.out[hq * AD_D + d] = f32_to_bf16_bits(l > 0.0f ? acc / l : 0.0f);
    } else {
      float* dst = p.part + (hq * p.splits + split) * AD_PART;
      dst[d] = acc;
      if (d == 0) {
        dst[AD_D] = mstar;
        dst[AD_D + 1] = l;
      }
    }
  }
}

__global__ __launch_bounds__(AD_WAVES * 64) void attn_decode_kernel(const AttnArgs p) { attn_decode_body(p); }

// out[b, hq, :] from the per-split partials
__global__ __launch_bounds__(AD_D) void attn_merge_kernel(const float* __restrict__ part, uint16_t* __restrict__ out,
                                                          int splits) {
  const int64_t hq = (int64_t)blockIdx.y * gridDim.x + blockIdx.x;
  const int d = threadIdx.x;
  const float* src = part + hq * splits * AD_PART;
  float mstar = -INFINITY;
  for (int s = 0; s < splits; s++) mstar = fmaxf(mstar, src[s * AD_PART + AD_D]);
  float acc = 0.0f, l = 0.0f;
  for (int s = 0; s < splits; s++) {
    const float ms = src[s * AD_PART + AD_D];
    if (ms == -INFINITY) continue;
    const float f = __builtin_amdgcn_exp2f(ms - mstar);
    acc += src[s * AD_PART + d] * f;
    l += src[s * AD_PART + AD_D + 1] * f;
  }
  out[hq * AD_D + d] = f32_to_bf16_bits(l > 0.0f ? acc / l : 0.0f);
}

// ---- RMSNorm with the residual add in front of it ---------------------------------------------------
// h = x (+ residual), rounded to the tensor dtype as the model's own `residual + hidden_states` is;
// y = weight * dtype(h * rsqrt(mean(h^2) + eps)) - the rounding order of HF LlamaRMSNorm.forward
// (variance and the scaling in fp32, the product with the weight in the tensor dtype).
template <typename T> struct Elem;
template <> struct Elem<uint16_t> {
  static __device__ __forceinline__ float load(uint16_t v) { return bf16_bits_to_f32(v); }
  static __device__ __forceinline__ uint16_t store(float f) { return f32_to_bf16_bits(f); }
};
template <> struct Elem<float> {
  static __device__ __forceinline__ float load(float v) { return v; }
  static __device__ __forceinline__ float store(float f) { return f; }
};

template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const T* __restrict__ x, const T* __restrict__ residual,
                                                      const T* __restrict__ weight, T* __restrict__ y,
                                                      T* __restrict__ residual_out, int64_t dim, float eps) {
  const int64_t row = blockIdx.x;
  const T* xr = x + row * dim;
  const T* rr = residual ? residual + row * dim : nullptr;
  T* hr = residual_out ? residual_out + row * dim : nullptr;
  T* yr = y + row * dim;
  __shared__ float red[4];
  float ss = 0.0f;
  for (int64_t i = threadIdx.x; i < dim; i += 256) {
    float hval = Elem<T>::load(xr[i]);
    if (rr) hval = Elem<T>::load(Elem<T>::store(hval + Elem<T>::load(rr[i])));
    if (hr) hr[i] = Elem<T>::store(hval);
    ss += hval * hval;
  }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float inv = rsqrtf((red[0] + red[1] + red[2] + red[3]) / (float)dim + eps);
  for (int64_t i = threadIdx.x; i < dim; i += 256) {
    float hval = Elem<T>::load(xr[i]);
    if (rr) hval = Elem<T>::load(Elem<T>::store(hval + Elem<T>::load(rr[i])));
    const float n = Elem<T>::load(Elem<T>::store(hval * inv));
    yr[i] = Elem<T>::store(Elem<T>::load(weight[i]) * n);
  }
}

// ---- rotary embedding of the new q / k, append of the new k / v to the cache ---------------------------
// qkv [B, (n_q + 2 n_kv) * 128]: q heads, then k heads, then v heads (the fused QKV linear's output).
// HF apply_rotary_pos_emb: x * cos + rotate_half(x) * sin with rotate_half(x) = cat(-x[64:], x[:64]);
// cos / sin are tables [max_positions, 128] in the tensor dtype, indexed by the token's position.
__global__ __launch_bounds__(64) void rope_append_kernel(const uint16_t* __restrict__ qkv,
                                                         const uint16_t* __restrict__ cos_t,
                                                         const uint16_t* __restrict__ sin_t,
                                                         const int64_t* __restrict__ positions,
                                                         uint16_t* __restrict__ q_out, uint16_t* __restrict__ k_cache,
                                                         uint16_t* __restrict__ v_cache, int n_q, int n_kv,
                                                         int64_t max_len, int64_t max_positions) {
  const int head = blockIdx.x, b = blockIdx.y, j = threadIdx.x;
  const int64_t pos = positions[b];
  const uint16_t* src = qkv + ((int64_t)b * (n_q + 2 * n_kv) + head) * AD_D;
  if (head >= n_q + n_kv) {   // value head: plain copy into the cache
    if (pos < 0 || pos >= max_len) return;
    uint16_t* dst = v_cache + (((int64_t)b * n_kv + (head - n_q - n_kv)) * max_len + pos) * AD_D;
    dst[j] = src[j];
    dst[j + 64] = src[j + 64];
    return;
  }
  if (pos < 0 || pos >= max_positions) return;
  const float x1 = bf16_bits_to_f32(src[j]), x2 = bf16_bits_to_f32(src[j + 64]);
  const uint16_t* cr = cos_t + pos * AD_D;
  const uint16_t* sr = sin_t + pos * AD_D;
  const float c1 = bf16_bits_to_f32(cr[j]), c2 = bf16_bits_to_f32(cr[j + 64]);
  const float s1 = bf16_bits_to_f32(sr[j]), s2 = bf16_bits_to_f32(sr[j + 64]);
  // each product is rounded to bf16 before the sum, as the bf16 tensor expression does
  const float r1 = bf16_bits_to_f32(f32_to_bf16_bits(x1 * c1)) + bf16_bits_to_f32(f32_to_bf16_bits(-x2 * s1));
  const float r2 = bf16_bits_to_f32(f32_to_bf16_bits(x2 * c2)) + bf16_bits_to_f32(f32_to_bf16_bits(x1 * s2));
  uint16_t* dst;
  if (head < n_q) {
    dst = q_out + ((int64_t)b * n_q + head) * AD_D;
  } else {
    if (pos >= max_len) return;
    dst = k_cache + (((int64_t)b * n_kv + (head - n_q)) * max_len + pos) * AD_D;
  }
  dst[j] = f32_to_bf16_bits(r1);
  dst[j + 64] = f32_to_bf16_bits(r2);
}

int pick_splits(int64_t B, int n_kv, int64_t len_bound) {
  if (const char* e = getenv("MTP_ATTN_SPLITS")) {
    const int v = atoi(e);
    if (v >= 1) return v;
  }
  const int64_t tiles = (len_bound + AD_TILE - 1) / AD_TILE;
  const int64_t by_len = (tiles + 2 * AD_WAVES - 1) / (2 * AD_WAVES);   // at least two tiles per wave
  const int64_t by_grid = (1024 + B * n_kv - 1) / (B * n_kv);           // about four workgroups per CU slot
  int64_t s = by_len < by_grid ? by_len : by_grid;
  if (s < 1) s = 1;
  if (s > 256) s = 256;
  return (int)s;
}

}  // namespace

extern "C" int64_t mtp_attn_decode_workspace_bytes(int64_t B, int n_q_heads, int n_kv_heads, int64_t len_bound) {
  if (B <= 0 || n_q_heads <= 0 || n_kv_heads <= 0 || len_bound <= 0) return 0;
  return B * n_q_heads * (int64_t)pick_splits(B, n_kv_heads, len_bound) * AD_PART * (int64_t)sizeof(float);
}

extern "C" int mtp_attn_decode(const void* q, const void* k_cache, const void* v_cache, const int64_t* lens, void* out,
                               void* workspace, int64_t workspace_bytes, int64_t B, int n_q_heads, int n_kv_heads,
                               int head_dim, int64_t max_len, int64_t len_bound, float scale, int dtype,
                               void* stream) {
  MTP_REQUIRE(dtype == MTP_BF16, MTP_EUNSUPPORTED, "attn_decode: bf16 only");
  MTP_REQUIRE(head_dim == AD_D, MTP_EUNSUPPORTED, "attn_decode: head_dim %d (128 supported)", head_dim);
  MTP_REQUIRE(B >= 0 && n_q_heads > 0 && n_kv_heads > 0 && n_q_heads % n_kv_heads == 0, MTP_EINVAL,
              "attn_decode: B=%lld heads %d/%d", (long long)B, n_q_heads, n_kv_heads);
  const int group = n_q_heads / n_kv_heads;
  MTP_REQUIRE(group <= AD_MAX_GROUP, MTP_EUNSUPPORTED, "attn_decode: %d q heads per kv head (at most %d)", group,
              AD_MAX_GROUP);
  MTP_REQUIRE(max_len > 0 && len_bound > 0 && len_bound <= max_len, MTP_EINVAL,
              "attn_decode: max_len=%lld len_bound=%lld", (long long)max_len, (long long)len_bound);
  MTP_REQUIRE(B <= 65535 && n_kv_heads <= 65535, MTP_EINVAL, "attn_decode: grid too large");
  if (B == 0) return MTP_OK;
  MTP_REQUIRE(q && k_cache && v_cache && lens && out, MTP_EINVAL, "attn_decode: null pointer");
  MTP_REQUIRE(((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)v_cache) % 16 == 0, MTP_EINVAL,
              "attn_decode: q and the caches must be 16-byte aligned");
  const int splits = pick_splits(B, n_kv_heads, len_bound);
  if (splits > 1) {
    const int64_t need = B * n_q_heads * (int64_t)splits * AD_PART * (int64_t)sizeof(float);
    MTP_REQUIRE(workspace && workspace_bytes >= need, MTP_EINVAL, "attn_decode: workspace %lld bytes, need %lld",
                (long long)workspace_bytes, (long long)need);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  AttnArgs a;
  a.q = static_cast<const uint16_t*>(q);
  a.k = static_cast<const uint16_t*>(k_cache);
  a.v = static_cast<const uint16_t*>(v_cache);
  a.lens = lens;
  a.out = static_cast<uint16_t*>(out);
  a.part = static_cast<float*>(workspace);
  a.n_q_heads = n_q_heads;
  a.n_kv_heads = n_kv_heads;
  a.group = group;
  a.max_len = max_len;
  a.splits = splits;
  a.scale_log2e = scale * 1.4426950408889634f;
  hipLaunchKernelGGL(attn_decode_kernel, dim3(splits, n_kv_heads, (unsigned)B), dim3(AD_WAVES * 64), 0, s, a);
  MTP_CHECK_LAUNCH("attn_decode");
  if (splits > 1) {
    hipLaunchKernelGGL(attn_merge_kernel, dim3(n_q_heads, (unsigned)B), dim3(AD_D), 0, s, a.part, a.out, splits);
    MTP_CHECK_LAUNCH("attn_merge");
  }
  return MTP_OK;
}

extern "C" int mtp_rmsnorm(const void* x, const void* residual, const void* weight, void* y, void* residual_out,
                           int64_t rows, int64_t dim, float eps, int dtype, void* stream) {
  MTP_REQUIRE(dtype == MTP_BF16 || dtype == MTP_F32, MTP_EINVAL, "rmsnorm: dtype %d", dtype);
  MTP_REQUIRE(rows >= 0 && dim > 0 && rows <= 0x7fffffffll, MTP_EINVAL, "rmsnorm: rows=%lld dim=%lld", (long long)rows,
              (long long)dim);
  if (rows == 0) return MTP_OK;
  MTP_REQUIRE(x && weight && y, MTP_EINVAL, "rmsnorm: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == MTP_BF16)
    hipLaunchKernelGGL(rmsnorm_kernel<uint16_t>, dim3((unsigned)rows), dim3(256), 0, s,
                       static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(residual),
                       static_cast<const uint16_t*>(weight), static_cast<uint16_t*>(y),
                       static_cast<uint16_t*>(residual_out), dim, eps);
  else
    hipLaunchKernelGGL(rmsnorm_kernel<float>, dim3((unsigned)rows), dim3(256), 0, s, static_cast<const float*>(x),
                       static_cast<const float*>(residual), static_cast<const float*>(weight), static_cast<float*>(y),
                       static_cast<float*>(residual_out), dim, eps);
  MTP_CHECK_LAUNCH("rmsnorm");
  return MTP_OK;
}

extern "C" int mtp_rope_kv_append(const void* qkv, const void* cos_table, const void* sin_table,
                                  const int64_t* positions, void* q_out, void* k_cache, void* v_cache, int64_t B,
                                  int n_q_heads, int n_kv_heads, int head_dim, int64_t max_len, int64_t max_positions,
                                  int dtype, void* stream) {
  MTP_REQUIRE(dtype == MTP_BF16, MTP_EUNSUPPORTED, "rope_kv_append: bf16 only");
  MTP_REQUIRE(head_dim == AD_D, MTP_EUNSUPPORTED, "rope_kv_append: head_dim %d (128 supported)", head_dim);
  MTP_REQUIRE(B >= 0 && B <= 65535 && n_q_heads > 0 && n_kv_heads > 0 && max_len > 0 && max_positions > 0, MTP_EINVAL,
              "rope_kv_append: B=%lld heads %d/%d max_len=%lld", (long long)B, n_q_heads, n_kv_heads,
              (long long)max_len);
  if (B == 0) return MTP_OK;
  MTP_REQUIRE(qkv && cos_table && sin_table && positions && q_out && k_cache && v_cache, MTP_EINVAL,
              "rope_kv_append: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(rope_append_kernel, dim3(n_q_heads + 2 * n_kv_heads, (unsigned)B), dim3(64), 0, s,
                     static_cast<const uint16_t*>(qkv), static_cast<const uint16_t*>(cos_table),
                     static_cast<const uint16_t*>(sin_table), positions, static_cast<uint16_t*>(q_out),
                     static_cast<uint16_t*>(k_cache), static_cast<uint16_t*>(v_cache), n_q_heads, n_kv_heads, max_len,
                     max_positions);
  MTP_CHECK_LAUNCH("rope_kv_append");
  return MTP_OK;
}
