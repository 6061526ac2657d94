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
constexpr int AD_MAX_WAVES = 8;
constexpr int AD_PART = AD_D + 2;              // floats per partial result: O[128], max, sum
constexpr int AD_MAX_GROUP = 16;

struct AttnArgs {
  const uint16_t* q;      // [B, n_q_heads, 128]                       (plain form)
  uint16_t* k;            // [B, n_kv_heads, max_len, 128]
  uint16_t* v;
  const int64_t* lens;    // [B] tokens to attend to                   (plain form)
  uint16_t* out;          // [B, n_q_heads, 128]
  float* part;            // [B, n_q_heads, splits, AD_PART] when splits > 1
  int32_t* arrived;       // [B, n_kv_heads] zero between launches: splits that have delivered their partial
  int n_q_heads, n_kv_heads, group;
  int64_t max_len;
  int splits;
  int rot_mul;            // tile rotation per workgroup index
  float scale_log2e;      // softmax scale * log2(e)
  // appending form: the new position comes straight from the QKV projection
  const uint16_t* qkv;        // [B, (n_q_heads + 2 n_kv_heads) * 128]
  const uint16_t* cos_t;      // [max_positions, 128]
  const uint16_t* sin_t;
  const int64_t* positions;   // [B] position of the new token = number of tokens already cached
  int64_t max_positions;
};

// x * cos + rotate_half(x) * sin for 8 elements of one head: `own` holds dims d .. d+7, `other` the dims
// 64 away, sign = -1 for d < 64 (rotate_half = cat(-x[64:], x[:64])).  Every product is rounded to bf16
// before the sum, and the sum again, as the bf16 tensor expression rounds.
template <bool F16>
__device__ __forceinline__ u32x4_t rope8(u32x4_t own, u32x4_t other, u32x4_t c, u32x4_t s, float sign) {
  using X = X16<F16>;
  u32x4_t r;
#pragma unroll
  for (int e = 0; e < 4; e++) {
    float a0 = X::lo(own[e]) * X::lo(c[e]), a1 = X::hi(own[e]) * X::hi(c[e]);
    float b0 = sign * X::lo(other[e]) * X::lo(s[e]), b1 = sign * X::hi(other[e]) * X::hi(s[e]);
    // the products exist as fp32 values here: with half tensors the compiler otherwise narrows the whole
    // expression to packed half arithmetic and folds one rounded product into a fused multiply-add
    asm volatile("" : "+v"(a0), "+v"(a1), "+v"(b0), "+v"(b1));
    const uint32_t pa = X::pack2(a0, a1), pb = X::pack2(b0, b1);
    r[e] = X::pack2(X::lo(pa) + X::lo(pb), X::hi(pa) + X::hi(pb));
  }
  return r;
}

// dma16 with the streaming (non-temporal) hint: the cache rows are read once per launch
__device__ __forceinline__ void dma16_nt(rsrc_t rsrc, uint32_t lds_addr, uint32_t voff, uint32_t soff) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen nt lds"
               :
               : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff));
}

// device-scope accesses: served at the level all XCDs share
__device__ __forceinline__ void coherent_store(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float coherent_load(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void wait_vm(int items_after) {
  // every item is 8 DMA instructions; "memory": LDS reads below must not move above the wait
  switch (items_after) {
    case 5: asm volatile("s_waitcnt vmcnt(40)" ::: "memory"); break;
    case 4: asm volatile("s_waitcnt vmcnt(32)" ::: "memory"); break;
    case 3: asm volatile("s_waitcnt vmcnt(24)" ::: "memory"); break;
    case 2: asm volatile("s_waitcnt vmcnt(16)" ::: "memory"); break;
    case 1: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
    default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
  }
}

// AD_WAVES waves with AD_RING ring slots each: 32 KiB of LDS per wave with 4 slots, 48 KiB with 6
template <bool APPEND, int AD_WAVES, int AD_RING, bool NT, bool F16>
__device__ __forceinline__ void attn_decode_body(const AttnArgs& p) {
  using X = X16<F16>;   // bf16 or IEEE half
  __shared__ __attribute__((aligned(1024))) char lds[AD_WAVES * AD_RING * AD_ITEM];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int G = p.group;
  const int h = lane & 15, q = lane >> 4;

  // tokens to read from the cache; the appending form adds the new one from registers
  int64_t len;
  bool fresh = false;     // this row has a new token to rotate, append and attend to
  int64_t pos = 0;
  if (APPEND) {
    pos = p.positions[b];
    fresh = pos >= 0 && pos < p.max_len && pos < p.max_positions;
    len = fresh ? pos : 0;
  } else {
    len = p.lens[b];
    len = len < 0 ? 0 : (len > p.max_len ? p.max_len : len);
  }
  const int tiles = (int)((len + AD_TILE - 1) / AD_TILE);
  const int tps = (tiles + p.splits - 1) / p.splits;
  const int tile_lo = split * tps;
  const int tile_hi = tile_lo + tps < tiles ? tile_lo + tps : tiles;
  // The workgroup's tiles are taken in rotated order, by an amount that differs between workgroups: the
  // sequences start a multiple of the cache's row stride apart, and workgroups walking them in step would
  // all be on the same memory channels at the same time.  (The recurrence does not care about the order.)
  const int n_wg = tile_hi > tile_lo ? tile_hi - tile_lo : 0;
  const int wg_lin = ((int)b * p.n_kv_heads + kvh) * p.splits + split;
  const int rot = n_wg > 0 ? (int)(((int64_t)wg_lin * p.rot_mul) % n_wg) : 0;
  const int n_my = n_wg > wave ? (n_wg - wave + AD_WAVES - 1) / AD_WAVES : 0;
  auto tile_of = [&](int i) {      // i-th tile of this wave
    int j = wave + AD_WAVES * i + rot;
    if (j >= n_wg) j -= n_wg;
    return tile_lo + j;
  };
  const int n_items = 2 * n_my;

  // this lane's share of Q^T as MFMA B operand: head h, dims 32c + 8q .. +7
  bf16x8_t qf[4];
  u32x4_t cs[4], sn[4];   // appending form: cos / sin of this lane's dims at the new position
  {
    const int64_t heads_row = APPEND ? (int64_t)b * (p.n_q_heads + 2 * p.n_kv_heads) : (int64_t)b * p.n_q_heads;
    const uint16_t* qrow = (APPEND ? p.qkv : p.q) + (heads_row + (int64_t)kvh * G + (h < G ? h : 0)) * AD_D;
    u32x4_t raw[4];
#pragma unroll
    for (int c = 0; c < 4; c++) raw[c] = *reinterpret_cast<const u32x4_t*>(qrow + 32 * c + 8 * q);
    if (APPEND) {
      const int64_t trow = (fresh ? pos : 0) * AD_D;
#pragma unroll
      for (int c = 0; c < 4; c++) {
        cs[c] = *reinterpret_cast<const u32x4_t*>(p.cos_t + trow + 32 * c + 8 * q);
        sn[c] = *reinterpret_cast<const u32x4_t*>(p.sin_t + trow + 32 * c + 8 * q);
      }
      u32x4_t rot[4];
#pragma unroll
      for (int c = 0; c < 4; c++) rot[c] = rope8<F16>(raw[c], raw[c ^ 2], cs[c], sn[c], c < 2 ? -1.0f : 1.0f);
#pragma unroll
      for (int c = 0; c < 4; c++) raw[c] = rot[c];
    }
#pragma unroll
    for (int c = 0; c < 4; c++) {
      if (h >= G) raw[c] = u32x4_t{0, 0, 0, 0};
      qf[c] = __builtin_bit_cast(bf16x8_t, raw[c]);
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
    const int64_t tok0 = (int64_t)tile_of(it >> 1) * AD_TILE;
    const char* base = reinterpret_cast<const char*>((it & 1) ? p.v : p.k) + (head_rows + tok0) * (AD_D * 2);
    const rsrc_t r = make_rsrc(base, (len - tok0) * (AD_D * 2));
    const uint32_t slot = ring0 + (it % AD_RING) * AD_ITEM;
#pragma unroll
    for (int j = 0; j < 8; j++) {
      if (NT)
        dma16_nt(r, slot + j * 1024, voff[j & 3] + (j >> 2) * 4096, 0);
      else
        dma16(r, slot + j * 1024, voff[j & 3] + (j >> 2) * 4096, 0);
    }
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

  constexpr int AHEAD = AD_RING - 1;     // items in flight while one is used
#pragma unroll
  for (int it = 0; it < AHEAD; it++)
    if (it < n_items) issue(it);

  if (APPEND && fresh && split == 0 && wave == 0) {
    // The new token: rotate its key, append key and value to the cache, and start the recurrence from it
    // (score s, probability 1, O = v).  No workgroup reads row `pos` of the cache in this launch.
    const uint16_t* krow = p.qkv + ((int64_t)b * (p.n_q_heads + 2 * p.n_kv_heads) + p.n_q_heads + kvh) * AD_D;
    const uint16_t* vrow_new = krow + (int64_t)p.n_kv_heads * AD_D;
    u32x4_t kraw[4], krot[4];
#pragma unroll
    for (int c = 0; c < 4; c++) kraw[c] = *reinterpret_cast<const u32x4_t*>(krow + 32 * c + 8 * q);
#pragma unroll
    for (int c = 0; c < 4; c++) krot[c] = rope8<F16>(kraw[c], kraw[c ^ 2], cs[c], sn[c], c < 2 ? -1.0f : 1.0f);
    float dot = 0.0f;
#pragma unroll
    for (int c = 0; c < 4; c++) {
      const u32x4_t qq = __builtin_bit_cast(u32x4_t, qf[c]);
#pragma unroll
      for (int e = 0; e < 4; e++)
        dot += X::lo(qq[e]) * X::lo(krot[c][e]) + X::hi(qq[e]) * X::hi(krot[c][e]);
    }
    dot += __shfl_xor(dot, 16, 64);
    dot += __shfl_xor(dot, 32, 64);
    m_run = dot * p.scale_log2e;
    l_run = q == 0 ? 1.0f : 0.0f;          // summed over the four lanes of a head at the end
    uint16_t* kdst = p.k + (head_rows + pos) * AD_D;
    uint16_t* vdst = p.v + (head_rows + pos) * AD_D;
#pragma unroll
    for (int dt = 0; dt < 8; dt++) {
      const u32x2_t vv = *reinterpret_cast<const u32x2_t*>(vrow_new + 16 * dt + 4 * q);
      o[dt] = f32x4_t{X::lo(vv[0]), X::hi(vv[0]), X::lo(vv[1]), X::hi(vv[1])};
    }
    if (h == 0) {
#pragma unroll
      for (int c = 0; c < 4; c++) {
        *reinterpret_cast<u32x4_t*>(kdst + 32 * c + 8 * q) = krot[c];
        *reinterpret_cast<u32x4_t*>(vdst + 32 * c + 8 * q) = *reinterpret_cast<const u32x4_t*>(vrow_new + 32 * c + 8 * q);
      }
    }
  }

  for (int i = 0; i < n_my; i++) {
    // ---- K: scores of 32 tokens for the heads of the group ----
    {
      const int it = 2 * i;
      if (it + AHEAD < n_items) issue(it + AHEAD);
      const int after = n_items - 1 - it;
      wait_vm(after < AHEAD ? after : AHEAD);
    }
    const char* kslot = ring + ((2 * i) % AD_RING) * AD_ITEM;
    f32x4_t s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 4; c++) {
      const uint32_t off = krow + (uint32_t)(((4 * c + q) ^ h) << 4);
      const bf16x8_t a0 = *reinterpret_cast<const bf16x8_t*>(kslot + off);
      const bf16x8_t a1 = *reinterpret_cast<const bf16x8_t*>(kslot + off + 16 * 256);
      s0 = X::mfma16(a0, qf[c], s0);
      s1 = X::mfma16(a1, qf[c], s1);
    }
    // this lane: head h, tokens 4q + j (s0) and 16 + 4q + j (s1) of the tile
    const int64_t valid = len - (int64_t)tile_of(i) * AD_TILE;
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
    const u32x4_t praw = {X::pack2(x0[0], x0[1]), X::pack2(x0[2], x0[3]), X::pack2(x1[0], x1[1]),
                          X::pack2(x1[2], x1[3])};
    const bf16x8_t pf = __builtin_bit_cast(bf16x8_t, praw);
#pragma unroll
    for (int dt = 0; dt < 8; dt++) o[dt] *= alpha;

    // ---- V: O^T += V^T P^T ----
    {
      const int it = 2 * i + 1;
      if (it + AHEAD < n_items) issue(it + AHEAD);
      const int after = n_items - 1 - it;
      wait_vm(after < AHEAD ? after : AHEAD);
    }
    const char* vslot = ring + ((2 * i + 1) % AD_RING) * AD_ITEM;
#pragma unroll
    for (int dt = 0; dt < 8; dt++) {
      const char* a = vslot + vrow + (uint32_t)(((2 * dt + vc0) ^ (vt & 15)) << 4);
      const bf16x4_t lo =
          __builtin_amdgcn_ds_read_tr16_b64_v4bf16((bf16x4_t __attribute__((address_space(3)))*)(a));
      const bf16x4_t hi =
          __builtin_amdgcn_ds_read_tr16_b64_v4bf16((bf16x4_t __attribute__((address_space(3)))*)(a + 16 * 256));
      const bf16x8_t vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      o[dt] = X::mfma16(vf, pf, o[dt]);
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
      p.out[hq * AD_D + d] = X::to_bits(l > 0.0f ? acc / l : 0.0f);
    } else {
      float* dst = p.part + (hq * p.splits + split) * AD_PART;
      coherent_store(dst + d, acc);
      if (d == 0) {
        coherent_store(dst + AD_D, mstar);
        coherent_store(dst + AD_D + 1, l);
      }
    }
  }
  if (p.splits == 1) return;

  // The split that delivers last merges all of them.  Partials travel through device-coherent stores and
  // loads (they bypass the per-XCD L2), so no cache write-back or invalidate is needed: a workgroup waits for
  // its stores to be acknowledged, then bumps the counter; whoever sees the counter full reads afterwards.
  __shared__ int last_one;
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (tid == 0) {
    int32_t* cnt = p.arrived + (int64_t)b * p.n_kv_heads + kvh;
    const int seen = __hip_atomic_fetch_add(cnt, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last_one = seen == p.splits - 1;
    if (last_one) __hip_atomic_store(cnt, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // for the next launch
  }
  __syncthreads();
  if (!last_one) return;
  for (int idx = tid; idx < G * AD_D; idx += AD_WAVES * 64) {
    const int hh = idx >> 7, d = idx & (AD_D - 1);
    const int64_t hq = (int64_t)b * p.n_q_heads + (int64_t)kvh * G + hh;
    const float* src = p.part + hq * p.splits * AD_PART;
    // 16 splits at a time, all their loads in flight together; running (max, sum, O) across the chunks
    float mstar = -INFINITY, acc = 0.0f, l = 0.0f;
    for (int s0 = 0; s0 < p.splits; s0 += 16) {
      float ms[16], av[16], lv[16];
#pragma unroll
      for (int u = 0; u < 16; u++) {
        const bool ok = s0 + u < p.splits;
        const float* one = src + (ok ? s0 + u : s0) * AD_PART;
        ms[u] = coherent_load(one + AD_D);
        av[u] = coherent_load(one + d);
        lv[u] = coherent_load(one + AD_D + 1);
        if (!ok) ms[u] = -INFINITY;
      }
      float mnew = mstar;
#pragma unroll
      for (int u = 0; u < 16; u++) mnew = fmaxf(mnew, ms[u]);
      if (mnew == -INFINITY) continue;
      const float keep = __builtin_amdgcn_exp2f(mstar - mnew);
      acc *= keep;
      l *= keep;
#pragma unroll
      for (int u = 0; u < 16; u++) {
        const float f = ms[u] == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f(ms[u] - mnew);
        acc += (ms[u] == -INFINITY ? 0.0f : av[u]) * f;
        l += (ms[u] == -INFINITY ? 0.0f : lv[u]) * f;
      }
      mstar = mnew;
    }
    p.out[hq * AD_D + d] = X::to_bits(l > 0.0f ? acc / l : 0.0f);
  }
}

template <bool APPEND, int AD_WAVES, int AD_RING, bool NT, bool F16>
__global__ __launch_bounds__(AD_WAVES * 64) void attn_decode_kernel(const AttnArgs p) {
  attn_decode_body<APPEND, AD_WAVES, AD_RING, NT, F16>(p);
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
template <> struct Elem<f16s> {
  static __device__ __forceinline__ float load(f16s v) { return X16<true>::from_bits(v.bits); }
  static __device__ __forceinline__ f16s store(float f) { return f16s{X16<true>::to_bits(f)}; }
};
template <> struct Elem<float> {
  static __device__ __forceinline__ float load(float v) { return v; }
  static __device__ __forceinline__ float store(float f) { return f; }
};

// General form: any dim, two passes over the row (the second re-reads it), element at a time.
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const T* x, const T* residual, const T* weight, T* y,
                                                      T* residual_out, int64_t dim, float eps) {
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
    ss += hval * hval;
  }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float inv = rsqrtf((red[0] + red[1] + red[2] + red[3]) / (float)dim + eps);
  // a thread reads and writes the same elements in both passes, so y may alias x and residual_out residual
  for (int64_t i = threadIdx.x; i < dim; i += 256) {
    float hval = Elem<T>::load(xr[i]);
    if (rr) hval = Elem<T>::load(Elem<T>::store(hval + Elem<T>::load(rr[i])));
    const float n = Elem<T>::load(Elem<T>::store(hval * inv));
    if (hr) hr[i] = Elem<T>::store(hval);
    yr[i] = Elem<T>::store(Elem<T>::load(weight[i]) * n);
  }
}

// Fast form: the row sits in registers between the two passes, 16 bytes per access, up to NV accesses per
// thread (dim <= 256 * NV * elements per 16 bytes).  All loads of a thread come before its stores.
template <typename T> struct Vec16;
template <> struct Vec16<uint16_t> {
  static constexpr int N = 8;
  static __device__ __forceinline__ void unpack(u32x4_t v, float* f) {
#pragma unroll
    for (int e = 0; e < 4; e++) {
      f[2 * e] = bf16_lo(v[e]);
      f[2 * e + 1] = bf16_hi(v[e]);
    }
  }
  static __device__ __forceinline__ u32x4_t pack(const float* f) {
    return u32x4_t{pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]), pack_bf16x2(f[6], f[7])};
  }
  static __device__ __forceinline__ float round(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }
};
template <> struct Vec16<f16s> {
  static constexpr int N = 8;
  using H = X16<true>;
  static __device__ __forceinline__ void unpack(u32x4_t v, float* f) {
#pragma unroll
    for (int e = 0; e < 4; e++) {
      f[2 * e] = H::lo(v[e]);
      f[2 * e + 1] = H::hi(v[e]);
    }
  }
  static __device__ __forceinline__ u32x4_t pack(const float* f) {
    return u32x4_t{H::pack2(f[0], f[1]), H::pack2(f[2], f[3]), H::pack2(f[4], f[5]), H::pack2(f[6], f[7])};
  }
  static __device__ __forceinline__ float round(float f) { return H::from_bits(H::to_bits(f)); }
};
template <> struct Vec16<float> {
  static constexpr int N = 4;
  static __device__ __forceinline__ void unpack(u32x4_t v, float* f) {
#pragma unroll
    for (int e = 0; e < 4; e++) f[e] = __uint_as_float(v[e]);
  }
  static __device__ __forceinline__ u32x4_t pack(const float* f) {
    return u32x4_t{__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]), __float_as_uint(f[3])};
  }
  static __device__ __forceinline__ float round(float f) { return f; }
};

template <typename T, int NV>
__global__ __launch_bounds__(256) void rmsnorm_vec_kernel(const T* x, const T* residual, const T* weight, T* y,
                                                          T* residual_out, int64_t dim, float eps) {
  using V = Vec16<T>;
  constexpr int N = V::N;
  const int64_t row = blockIdx.x;
  const int nvec = (int)(dim / N);
  const u32x4_t* xv = reinterpret_cast<const u32x4_t*>(x + row * dim);
  const u32x4_t* rv = residual ? reinterpret_cast<const u32x4_t*>(residual + row * dim) : nullptr;
  const u32x4_t* wv = reinterpret_cast<const u32x4_t*>(weight);
  u32x4_t* hv = residual_out ? reinterpret_cast<u32x4_t*>(residual_out + row * dim) : nullptr;
  u32x4_t* yv = reinterpret_cast<u32x4_t*>(y + row * dim);
  __shared__ float red[4];
  u32x4_t xin[NV], rin[NV], win[NV];
#pragma unroll
  for (int j = 0; j < NV; j++) {
    const int i = threadIdx.x + 256 * j;
    xin[j] = rin[j] = win[j] = u32x4_t{0u, 0u, 0u, 0u};
    if (i < nvec) {
      xin[j] = xv[i];
      if (rv) rin[j] = rv[i];
      win[j] = wv[i];
    }
  }
  float hval[NV][N];
  float ss = 0.0f;
#pragma unroll
  for (int j = 0; j < NV; j++) {
    float r[N];
    V::unpack(xin[j], hval[j]);
    V::unpack(rin[j], r);
#pragma unroll
    for (int e = 0; e < N; e++) {
      if (rv) hval[j][e] = V::round(hval[j][e] + r[e]);
      ss += hval[j][e] * hval[j][e];
    }
  }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float inv = rsqrtf((red[0] + red[1] + red[2] + red[3]) / (float)dim + eps);
#pragma unroll
  for (int j = 0; j < NV; j++) {
    const int i = threadIdx.x + 256 * j;
    if (i >= nvec) continue;
    float g[N], out[N];
    V::unpack(win[j], g);
#pragma unroll
    for (int e = 0; e < N; e++) out[e] = g[e] * V::round(hval[j][e] * inv);
    if (hv) hv[i] = V::pack(hval[j]);
    yv[i] = V::pack(out);
  }
}

// ---- rotary embedding of the new q / k, append of the new k / v to the cache ---------------------------
// qkv [B, (n_q + 2 n_kv) * 128]: q heads, then k heads, then v heads (the fused QKV linear's output).
// HF apply_rotary_pos_emb: x * cos + rotate_half(x) * sin with rotate_half(x) = cat(-x[64:], x[:64]);
// cos / sin are tables [max_positions, 128] in the tensor dtype, indexed by the token's position.
template <bool F16>
__global__ __launch_bounds__(64) void rope_append_kernel(const uint16_t* __restrict__ qkv,
                                                         const uint16_t* __restrict__ cos_t,
                                                         const uint16_t* __restrict__ sin_t,
                                                         const int64_t* __restrict__ positions,
                                                         uint16_t* __restrict__ q_out, uint16_t* __restrict__ k_cache,
                                                         uint16_t* __restrict__ v_cache, int n_q, int n_kv,
                                                         int64_t max_len, int64_t max_positions) {
  using X = X16<F16>;
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
  const float x1 = X::from_bits(src[j]), x2 = X::from_bits(src[j + 64]);
  const uint16_t* cr = cos_t + pos * AD_D;
  const uint16_t* sr = sin_t + pos * AD_D;
  const float c1 = X::from_bits(cr[j]), c2 = X::from_bits(cr[j + 64]);
  const float s1 = X::from_bits(sr[j]), s2 = X::from_bits(sr[j + 64]);
  // each product is rounded to the tensor dtype before the sum, as the tensor expression does.  The products are
  // pinned as fp32 values: with half tensors the compiler otherwise narrows the arithmetic to half and folds one
  // of the rounded products into a fused multiply-add.
  float a1 = x1 * c1, a2 = x2 * c2, b1 = -x2 * s1, b2 = x1 * s2;
  asm volatile("" : "+v"(a1), "+v"(a2), "+v"(b1), "+v"(b2));
  const uint32_t pa = X::pack2(a1, a2), pb = X::pack2(b1, b2);
  const uint32_t pr = X::pack2(X::lo(pa) + X::lo(pb), X::hi(pa) + X::hi(pb));
  uint16_t* dst;
  if (head < n_q) {
    dst = q_out + ((int64_t)b * n_q + head) * AD_D;
  } else {
    if (pos >= max_len) return;
    dst = k_cache + (((int64_t)b * n_kv + (head - n_q)) * max_len + pos) * AD_D;
  }
  dst[j] = (uint16_t)(pr & 0xffffu);
  dst[j + 64] = (uint16_t)(pr >> 16);
}

int pick_splits(int64_t B, int n_kv, int64_t len_bound) {
  static MtpTune tune_splits("MTP_ATTN_SPLITS");
  if (tune_splits.get(0) >= 1) return tune_splits.get(0);
  const int64_t tiles = (len_bound + AD_TILE - 1) / AD_TILE;
  const int64_t by_len = (tiles + 2 * AD_MAX_WAVES - 1) / (2 * AD_MAX_WAVES);   // at least two tiles per wave
  // about one workgroup per CU: a workgroup's start-up and its merge are paid once per split
  const int64_t by_grid = (256 + B * n_kv / 2) / (B * n_kv);
  int64_t s = by_len < by_grid ? by_len : by_grid;
  // Few sequences and a short context leave that rule with a handful of workgroups; up to 16 splits (one pass of
  // the final merge) pay even when they leave waves without a tile: B = 1, 2048 tokens 13.3 -> 10.2 us.
  int64_t s_small = by_grid < 16 ? by_grid : 16;
  if (s_small > tiles) s_small = tiles;
  if (s < s_small) s = s_small;
  if (s < 1) s = 1;
  if (s > 256) s = 256;
  return (int)s;
}

}  // namespace

namespace {
int64_t counter_bytes(int64_t B, int n_kv) { return (B * n_kv * (int64_t)sizeof(int32_t) + 255) / 256 * 256; }

int64_t workspace_need(int64_t B, int n_q, int n_kv, int splits) {
  if (splits <= 1) return 0;
  return counter_bytes(B, n_kv) + B * n_q * (int64_t)splits * AD_PART * (int64_t)sizeof(float);
}

// checks shared by the two forms; fills what they have in common and launches
int launch_attn(bool append, AttnArgs a, const char* what, void* workspace, int64_t workspace_bytes, int64_t B,
                int n_q_heads, int n_kv_heads, int head_dim, int64_t max_len, int64_t len_bound, float scale, int dtype,
                void* stream) {
  MTP_REQUIRE(dtype == MTP_BF16 || dtype == MTP_F16, MTP_EUNSUPPORTED, "%s: dtype %d (bf16 or f16)", what, dtype);
  MTP_REQUIRE(head_dim == AD_D, MTP_EUNSUPPORTED, "%s: head_dim %d (128 supported)", what, head_dim);
  MTP_REQUIRE(B >= 0 && n_q_heads > 0 && n_kv_heads > 0 && n_q_heads % n_kv_heads == 0, MTP_EINVAL,
              "%s: B=%lld heads %d/%d", what, (long long)B, n_q_heads, n_kv_heads);
  const int group = n_q_heads / n_kv_heads;
  MTP_REQUIRE(group <= AD_MAX_GROUP, MTP_EUNSUPPORTED, "%s: %d q heads per kv head (at most %d)", what, group,
              AD_MAX_GROUP);
  MTP_REQUIRE(max_len > 0 && len_bound > 0 && len_bound <= max_len, MTP_EINVAL, "%s: max_len=%lld len_bound=%lld", what,
              (long long)max_len, (long long)len_bound);
  MTP_REQUIRE(B <= 65535 && n_kv_heads <= 65535, MTP_EINVAL, "%s: grid too large", what);
  if (B == 0) return MTP_OK;
  MTP_REQUIRE(a.k && a.v && a.out, MTP_EINVAL, "%s: null pointer", what);
  MTP_REQUIRE(((uintptr_t)a.k | (uintptr_t)a.v | (uintptr_t)a.q | (uintptr_t)a.qkv | (uintptr_t)a.cos_t |
               (uintptr_t)a.sin_t) % 16 == 0,
              MTP_EINVAL, "%s: tensors must be 16-byte aligned", what);
  const int splits = pick_splits(B, n_kv_heads, len_bound);
  const int64_t need = workspace_need(B, n_q_heads, n_kv_heads, splits);
  MTP_REQUIRE(need == 0 || (workspace && workspace_bytes >= need && (uintptr_t)workspace % 16 == 0), MTP_EINVAL,
              "%s: workspace %lld bytes, need %lld (16-byte aligned)", what, (long long)workspace_bytes,
              (long long)need);
  a.arrived = static_cast<int32_t*>(workspace);
  a.part = need ? reinterpret_cast<float*>(static_cast<char*>(workspace) + counter_bytes(B, n_kv_heads)) : nullptr;
  a.n_q_heads = n_q_heads;
  a.n_kv_heads = n_kv_heads;
  a.group = group;
  a.max_len = max_len;
  a.splits = splits;
  static MtpTune tune_rot("MTP_ATTN_ROT"), tune_cfg("MTP_ATTN_CFG");
  a.rot_mul = tune_rot.get(1);
  if (a.rot_mul < 0) a.rot_mul = 0;   // taken modulo the tile count: must not go negative
  a.scale_log2e = scale * 1.4426950408889634f;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(splits, n_kv_heads, (unsigned)B);
  const int cfg = tune_cfg.get(0);
  const bool f16 = dtype == MTP_F16;
#define MTP_ATTN_LAUNCH(W, R, NT)                                                                        \
  do {                                                                                                   \
    if (append && f16)                                                                                   \
      hipLaunchKernelGGL((attn_decode_kernel<true, W, R, NT, true>), grid, dim3(W * 64), 0, s, a);       \
    else if (append)                                                                                     \
      hipLaunchKernelGGL((attn_decode_kernel<true, W, R, NT, false>), grid, dim3(W * 64), 0, s, a);      \
    else if (f16)                                                                                        \
      hipLaunchKernelGGL((attn_decode_kernel<false, W, R, NT, true>), grid, dim3(W * 64), 0, s, a);      \
    else                                                                                                 \
      hipLaunchKernelGGL((attn_decode_kernel<false, W, R, NT, false>), grid, dim3(W * 64), 0, s, a);     \
  } while (0)
  if (cfg == 1)
    MTP_ATTN_LAUNCH(8, 2, false);
  else if (cfg == 2)
    MTP_ATTN_LAUNCH(4, 4, true);
  else
    MTP_ATTN_LAUNCH(8, 2, true);
#undef MTP_ATTN_LAUNCH
  MTP_CHECK_LAUNCH(what);
  return MTP_OK;
}
}  // namespace

extern "C" int64_t mtp_attn_decode_workspace_bytes(int64_t B, int n_q_heads, int n_kv_heads, int64_t len_bound) {
  if (B <= 0 || n_q_heads <= 0 || n_kv_heads <= 0 || len_bound <= 0) return 0;
  return workspace_need(B, n_q_heads, n_kv_heads, pick_splits(B, n_kv_heads, len_bound));
}

extern "C" int mtp_attn_decode(const void* q, const void* k_cache, const void* v_cache, const int64_t* lens, void* out,
                               void* workspace, int64_t workspace_bytes, int64_t B, int n_q_heads, int n_kv_heads,
                               int head_dim, int64_t max_len, int64_t len_bound, float scale, int dtype,
                               void* stream) {
  MTP_REQUIRE(B == 0 || (q && lens), MTP_EINVAL, "attn_decode: null pointer");
  AttnArgs a = {};
  a.q = static_cast<const uint16_t*>(q);
  a.k = static_cast<uint16_t*>(const_cast<void*>(k_cache));     // only read in this form
  a.v = static_cast<uint16_t*>(const_cast<void*>(v_cache));
  a.lens = lens;
  a.out = static_cast<uint16_t*>(out);
  return launch_attn(false, a, "attn_decode", workspace, workspace_bytes, B, n_q_heads, n_kv_heads, head_dim, max_len,
                     len_bound, scale, dtype, stream);
}

extern "C" int mtp_attn_decode_append(const void* qkv, const void* cos_table, const void* sin_table,
                                      const int64_t* positions, void* k_cache, void* v_cache, void* out,
                                      void* workspace, int64_t workspace_bytes, int64_t B, int n_q_heads,
                                      int n_kv_heads, int head_dim, int64_t max_len, int64_t max_positions,
                                      int64_t len_bound, float scale, int dtype, void* stream) {
  MTP_REQUIRE(B == 0 || (qkv && cos_table && sin_table && positions), MTP_EINVAL, "attn_decode_append: null pointer");
  MTP_REQUIRE(max_positions > 0, MTP_EINVAL, "attn_decode_append: max_positions=%lld", (long long)max_positions);
  AttnArgs a = {};
  a.qkv = static_cast<const uint16_t*>(qkv);
  a.cos_t = static_cast<const uint16_t*>(cos_table);
  a.sin_t = static_cast<const uint16_t*>(sin_table);
  a.positions = positions;
  a.max_positions = max_positions;
  a.k = static_cast<uint16_t*>(k_cache);
  a.v = static_cast<uint16_t*>(v_cache);
  a.out = static_cast<uint16_t*>(out);
  return launch_attn(true, a, "attn_decode_append", workspace, workspace_bytes, B, n_q_heads, n_kv_heads, head_dim,
                     max_len, len_bound, scale, dtype, stream);
}

extern "C" int mtp_rmsnorm(const void* x, const void* residual, const void* weight, void* y, void* residual_out,
                           int64_t rows, int64_t dim, float eps, int dtype, void* stream) {
  MTP_REQUIRE(dtype == MTP_BF16 || dtype == MTP_F32 || dtype == MTP_F16, MTP_EINVAL, "rmsnorm: dtype %d", dtype);
  MTP_REQUIRE(rows >= 0 && dim > 0 && rows <= 0x7fffffffll, MTP_EINVAL, "rmsnorm: rows=%lld dim=%lld", (long long)rows,
              (long long)dim);
  if (rows == 0) return MTP_OK;
  MTP_REQUIRE(x && weight && y, MTP_EINVAL, "rmsnorm: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int epv = dtype == MTP_F32 ? 4 : 8;
  const bool aligned = ((uintptr_t)x | (uintptr_t)residual | (uintptr_t)weight | (uintptr_t)y |
                        (uintptr_t)residual_out) % 16 == 0;
  const int64_t nvec = dim / epv;
  const bool fast = aligned && dim % epv == 0 && nvec <= 256 * 8;
  const dim3 grid((unsigned)rows), block(256);
#define MTP_RMS_LAUNCH(T, KERNEL)                                                                            \
  hipLaunchKernelGGL(KERNEL, grid, block, 0, s, static_cast<const T*>(x), static_cast<const T*>(residual), \
                     static_cast<const T*>(weight), static_cast<T*>(y), static_cast<T*>(residual_out), dim, eps)
#define MTP_RMS_PICK(T)                                                \
  do {                                                                 \
    if (!fast) MTP_RMS_LAUNCH(T, rmsnorm_kernel<T>);                   \
    else if (nvec <= 256 * 2) MTP_RMS_LAUNCH(T, (rmsnorm_vec_kernel<T, 2>)); \
    else if (nvec <= 256 * 4) MTP_RMS_LAUNCH(T, (rmsnorm_vec_kernel<T, 4>)); \
    else MTP_RMS_LAUNCH(T, (rmsnorm_vec_kernel<T, 8>));                \
  } while (0)
  if (dtype == MTP_BF16)
    MTP_RMS_PICK(uint16_t);
  else if (dtype == MTP_F16)
    MTP_RMS_PICK(f16s);
  else
    MTP_RMS_PICK(float);
#undef MTP_RMS_PICK
#undef MTP_RMS_LAUNCH
  MTP_CHECK_LAUNCH("rmsnorm");
  return MTP_OK;
}

extern "C" int mtp_rope_kv_append(const void* qkv, const void* cos_table, const void* sin_table,
                                  const int64_t* positions, void* q_out, void* k_cache, void* v_cache, int64_t B,
                                  int n_q_heads, int n_kv_heads, int head_dim, int64_t max_len, int64_t max_positions,
                                  int dtype, void* stream) {
  MTP_REQUIRE(dtype == MTP_BF16 || dtype == MTP_F16, MTP_EUNSUPPORTED, "rope_kv_append: dtype %d (bf16 or f16)", dtype);
  MTP_REQUIRE(head_dim == AD_D, MTP_EUNSUPPORTED, "rope_kv_append: head_dim %d (128 supported)", head_dim);
  MTP_REQUIRE(B >= 0 && B <= 65535 && n_q_heads > 0 && n_kv_heads > 0 && max_len > 0 && max_positions > 0, MTP_EINVAL,
              "rope_kv_append: B=%lld heads %d/%d max_len=%lld", (long long)B, n_q_heads, n_kv_heads,
              (long long)max_len);
  if (B == 0) return MTP_OK;
  MTP_REQUIRE(qkv && cos_table && sin_table && positions && q_out && k_cache && v_cache, MTP_EINVAL,
              "rope_kv_append: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(n_q_heads + 2 * n_kv_heads, (unsigned)B), block(64);
#define MTP_ROPE_ARGS                                                                                       \
  static_cast<const uint16_t*>(qkv), static_cast<const uint16_t*>(cos_table),                               \
      static_cast<const uint16_t*>(sin_table), positions, static_cast<uint16_t*>(q_out),                    \
      static_cast<uint16_t*>(k_cache), static_cast<uint16_t*>(v_cache), n_q_heads, n_kv_heads, max_len,     \
      max_positions
  if (dtype == MTP_F16)
    hipLaunchKernelGGL(rope_append_kernel<true>, grid, block, 0, s, MTP_ROPE_ARGS);
  else
    hipLaunchKernelGGL(rope_append_kernel<false>, grid, block, 0, s, MTP_ROPE_ARGS);
#undef MTP_ROPE_ARGS
  MTP_CHECK_LAUNCH("rope_kv_append");
  return MTP_OK;
}
