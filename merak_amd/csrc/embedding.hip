// Vocab-parallel embedding lookup (and its dense gradient) for gfx950.
//
// Forward is a pure row copy: out[i,:] = table[ids[i]-vocab_start,:], or a
// row of zeros when the id lies outside this rank's [vocab_start, vocab_end)
// (Merak/core/mpu/layers.py:148-152,162).  One thread moves one 16-byte
// piece, consecutive threads move consecutive pieces of a row, so a wave
// reads and writes 1 KiB contiguous runs.  Narrower pieces (8/4/2/1 bytes)
// serve rows whose size or base address is not 16-byte aligned.
#include "mtp_common.h"

namespace {

template <typename V>
__global__ __launch_bounds__(256) void embedding_gather_kernel(const int64_t* __restrict__ ids,
                                                               const V* __restrict__ table, V* __restrict__ out,
                                                               int64_t n_ids, int64_t vec_per_row,
                                                               int64_t vocab_start, int64_t vocab_end,
                                                               int32_t* __restrict__ oob_count) {
  const int64_t total = n_ids * vec_per_row;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int64_t r = i / vec_per_row;
    const int64_t c = i - r * vec_per_row;
    const int64_t id = ids[r];
    const bool ok = id >= vocab_start && id < vocab_end;
    V v = V{};
    if (ok) v = table[(id - vocab_start) * vec_per_row + c];
    out[i] = v;
    if (!ok && c == 0 && oob_count) atomicAdd(oob_count, 1);
  }
}

// Rows of at least 256 pieces: one workgroup per row (grid-stride over rows), the id read once per row, up to four
// pieces per lane requested before the first is stored; no division per piece.
template <typename V>
__global__ __launch_bounds__(256) void embedding_gather_rows_kernel(const int64_t* __restrict__ ids,
                                                                    const V* __restrict__ table, V* __restrict__ out,
                                                                    int64_t n_ids, int vec_per_row, int64_t vocab_start,
                                                                    int64_t vocab_end, int32_t* __restrict__ oob_count) {
  for (int64_t r = blockIdx.x; r < n_ids; r += gridDim.x) {
    const int64_t id = ids[r];
    const bool ok = id >= vocab_start && id < vocab_end;
    const V* src = table + (ok ? id - vocab_start : 0) * (int64_t)vec_per_row;
    V* dst = out + r * (int64_t)vec_per_row;
    for (int c0 = threadIdx.x; c0 < vec_per_row; c0 += 4 * 256) {
      V v[4];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int c = c0 + 256 * u;
        v[u] = V{};
        if (ok && c < vec_per_row) v[u] = src[c];
      }
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int c = c0 + 256 * u;
        if (c < vec_per_row) dst[c] = v[u];
      }
    }
    if (!ok && threadIdx.x == 0 && oob_count) atomicAdd(oob_count, 1);
  }
}

// ---- dense gradient of the lookup ---------------------------------------------
// dtable[id - start, :] += sum of dout[i, :] over the tokens i with ids[i] == id, with fp32 accumulation in an
// order that depends on the ids alone: the result does not depend on scheduling (no atomics on the gradient).
// The order: ascending token index; for an id carried by more than EMB_SEG tokens, ascending token index inside
// blocks of EMB_SEG of its tokens, the block sums added in ascending order inside blocks of EMB_SEG blocks, and
// those added in ascending order.
//
// Pass 1 (one workgroup per token) chains the tokens of equal id: rank[i] = how many earlier tokens have this
// id, next[i] = the next later token with it (or -1).  Pass 2 (one workgroup per token and column chunk): the
// first token of a "light" id walks its chain (at most EMB_SEG tokens) and adds the sum to its table row; every
// EMB_SEG-th token of a "heavy" id walks EMB_SEG tokens and leaves the sum in a slot of the workspace.  Pass 3:
// every EMB_SEG^2-th token of a heavy id adds EMB_SEG block sums up into a second slot.  Pass 4: the first token
// of a heavy id adds those up and adds the result to the table row.  The longest dependent walk is
// 2 EMB_SEG + count / EMB_SEG^2 steps (a batch of 8192 equal ids: 72 instead of 8192).
// Pass 1 compares every pair of tokens of shared buckets (at most n^2 / 2 id loads from L2, a few tens of
// microseconds at 8192 tokens).
constexpr int EMB_SEG = 32;
struct TokenLink {
  int32_t next;   // next token with the same id, -1 at the end of the chain
  int32_t rank;   // number of earlier tokens with the same id; -1: id out of range
  int32_t slot;   // heavy ids, rank % EMB_SEG == 0: where this block's sum goes; -1 otherwise
  int32_t next_head;   // heavy ids, rank % EMB_SEG == 0: first token of the next block (written by pass 2), or -1
  int32_t next_head2;  // heavy ids, rank % EMB_SEG^2 == 0: first token of the next block of blocks (pass 3), or -1
};

// Most ids of a batch occur once.  A table of counters, several per token and indexed by the id modulo its size,
// tells which tokens may have company: a token alone in its bucket is a first token without a chain and skips
// the comparison with all the others.  (Sharing a bucket with another id only costs the comparison.)
__global__ __launch_bounds__(256) void embedding_bucket_zero_kernel(int32_t* __restrict__ bucket, int n_bucket) {
  const int b = blockIdx.x * 256 + threadIdx.x;
  if (b < n_bucket) bucket[b] = 0;   // bucket[n_bucket - 1 + 1 ..] does not exist: the slot counter sits at [-1]
  if (b == 0) bucket[-1] = 0;
}
__global__ __launch_bounds__(256) void embedding_bucket_count_kernel(const int64_t* __restrict__ ids,
                                                                     int32_t* __restrict__ bucket, int n_bucket,
                                                                     int n_ids, int64_t vocab_start, int64_t vocab_end) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n_ids) return;
  const int64_t id = ids[i];
  if (id >= vocab_start && id < vocab_end) atomicAdd(bucket + (int)((id - vocab_start) & (n_bucket - 1)), 1);
}

__global__ __launch_bounds__(256) void embedding_link_kernel(const int64_t* __restrict__ ids,
                                                             TokenLink* __restrict__ link, int n_ids,
                                                             int64_t vocab_start, int64_t vocab_end,
                                                             int32_t* __restrict__ bucket, int n_bucket,
                                                             int32_t* __restrict__ head_of_slot) {
  const int i = blockIdx.x;
  const int tid = threadIdx.x;
  const int64_t id = ids[i];
  if (id < vocab_start || id >= vocab_end) {
    if (tid == 0) link[i] = TokenLink{-1, -1, -1, -1, -1};
    return;
  }
  const int in_bucket = bucket[(int)((id - vocab_start) & (n_bucket - 1))];
  if (in_bucket == 1) {   // the only token of its bucket
    if (tid == 0) link[i] = TokenLink{-1, 0, -1, -1, -1};
    return;
  }
  // every thread looks at its share of the other tokens, four loads in flight, and the workgroup adds up once:
  // earlier tokens with this id (the rank), later ones, and the first of those
  int before = 0, later = 0, first = INT32_MAX;
  for (int base = 0; base < n_ids; base += 1024) {
    int64_t v[4];
#pragma unroll
    for (int u = 0; u < 4; u++) {
      const int j = base + 256 * u + tid;
      v[u] = j < n_ids ? ids[j] : vocab_start - 1;
    }
#pragma unroll
    for (int u = 0; u < 4; u++) {
      const int j = base + 256 * u + tid;
      if (v[u] == id && j != i) {
        if (j < i) {
          before++;
        } else {
          later++;
          first = j < first ? j : first;
        }
      }
    }
  }
  __shared__ int s_before, s_later, first_after;
  if (tid == 0) {
    s_before = 0;
    s_later = 0;
    first_after = INT32_MAX;
  }
  __syncthreads();
  if (before) atomicAdd(&s_before, before);
  if (later) {
    atomicAdd(&s_later, later);
    atomicMin(&first_after, first);
  }
  __syncthreads();
  const int rank = s_before;
  later = s_later;
  if (tid == 0) {
    int slot = -1;
    // An id is heavy when more than EMB_SEG tokens carry it (rank + 1 + later of them): every EMB_SEG-th of its
    // tokens heads a block with a slot of its own.  Which slot does not matter for the result.  At most
    // n / EMB_SEG + n / (EMB_SEG + 1) blocks exist: count / EMB_SEG + 1 per heavy id, at most n / (EMB_SEG + 1) ids.
    if (rank + 1 + later > EMB_SEG && rank % EMB_SEG == 0) {
      slot = atomicAdd(bucket - 1, 1);
      head_of_slot[slot] = i;   // passes 3 and 4 run one workgroup column per slot, not per token
    }
    link[i] = TokenLink{first_after == INT32_MAX ? -1 : first_after, rank, slot, -1, -1};
  }
}

// element <-> float for float, uint16_t (bf16 bits) and f16s (IEEE half bits)
__device__ __forceinline__ float elem_f32(float v) { return v; }
__device__ __forceinline__ float elem_f32(uint16_t v) { return bf16_bits_to_f32(v); }
__device__ __forceinline__ float elem_f32(f16s v) { return X16<true>::from_bits(v.bits); }
__device__ __forceinline__ void elem_set(float* p, float v) { *p = v; }
__device__ __forceinline__ void elem_set(uint16_t* p, float v) { *p = f32_to_bf16_bits(v); }
__device__ __forceinline__ void elem_set(f16s* p, float v) { p->bits = X16<true>::to_bits(v); }

template <typename T, int N> struct alignas(sizeof(T) * N) Pack {
  T v[N];
};

// Pass 2.  W columns per lane: 8 (16-byte loads of 16-bit gradients; dim % 8 == 0 and 32-byte aligned tensors) or
// 4 with a ragged end.  partial: [slots, dim] fp32.
template <typename T, typename TO, int W>
__global__ __launch_bounds__(256) void embedding_bwd_kernel(const int64_t* __restrict__ ids,
                                                            const T* __restrict__ dout, TO* __restrict__ dtable,
                                                            TokenLink* __restrict__ link, float* __restrict__ partial,
                                                            int64_t dim, int64_t vocab_start) {
  const int i = blockIdx.x;
  const TokenLink me = link[i];
  const bool heavy_head = me.slot >= 0;
  if (!(heavy_head || (me.rank == 0 && me.slot < 0))) return;
  // the first token of a heavy id has a slot; a first token without one is light: its chain is at most EMB_SEG long
  const int64_t c0 = ((int64_t)blockIdx.y * 256 + threadIdx.x) * W;
  if (c0 >= dim) return;
  const int nc = dim - c0 < W ? (int)(dim - c0) : W;
  float acc[W];
#pragma unroll
  for (int e = 0; e < W; e++) acc[e] = 0.f;
  int j = i;
  for (int step = 0; j >= 0 && (!heavy_head || step < EMB_SEG); step++) {
    if constexpr (W == 8) {
      const Pack<T, 8> p = *reinterpret_cast<const Pack<T, 8>*>(dout + (int64_t)j * dim + c0);
#pragma unroll
      for (int e = 0; e < 8; e++) acc[e] += elem_f32(p.v[e]);
    } else {
      const T* src = dout + (int64_t)j * dim + c0;
      for (int e = 0; e < nc; e++) acc[e] += elem_f32(src[e]);
    }
    j = link[j].next;
  }
  if (heavy_head) {
    float* dst = partial + (int64_t)me.slot * dim + c0;
    for (int e = 0; e < nc; e++) dst[e] = acc[e];
    if (blockIdx.y == 0 && threadIdx.x == 0) link[i].next_head = j;
    return;
  }
  TO* dst = dtable + (ids[i] - vocab_start) * dim + c0;
  if constexpr (W == 8) {
    Pack<TO, 8> t = *reinterpret_cast<Pack<TO, 8>*>(dst);
#pragma unroll
    for (int e = 0; e < 8; e++) elem_set(&t.v[e], elem_f32(t.v[e]) + acc[e]);
    *reinterpret_cast<Pack<TO, 8>*>(dst) = t;
  } else {
    for (int e = 0; e < nc; e++) elem_set(dst + e, elem_f32(dst[e]) + acc[e]);
  }
}

// Pass 3: every EMB_SEG^2-th token of a heavy id adds EMB_SEG block sums up, in ascending order, into partial2
__global__ __launch_bounds__(256) void embedding_bwd_level2_kernel(TokenLink* __restrict__ link,
                                                                   const float* __restrict__ partial,
                                                                   float* __restrict__ partial2, int64_t dim,
                                                                   const int32_t* __restrict__ n_slots,
                                                                   const int32_t* __restrict__ head_of_slot) {
  if ((int)blockIdx.x >= *n_slots) return;
  const int i = head_of_slot[blockIdx.x];
  const TokenLink me = link[i];
  if (me.slot < 0 || me.rank % (EMB_SEG * EMB_SEG) != 0) return;
  const int64_t c0 = ((int64_t)blockIdx.y * 256 + threadIdx.x) * 4;
  if (c0 >= dim) return;
  const int nc = dim - c0 < 4 ? (int)(dim - c0) : 4;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  int h = i;
  for (int step = 0; h >= 0 && step < EMB_SEG; step++) {
    const TokenLink t = link[h];
    const float* src = partial + (int64_t)t.slot * dim + c0;
    for (int e = 0; e < nc; e++) acc[e] += src[e];
    h = t.next_head;
  }
  float* dst = partial2 + (int64_t)me.slot * dim + c0;
  for (int e = 0; e < nc; e++) dst[e] = acc[e];
  if (blockIdx.y == 0 && threadIdx.x == 0) link[i].next_head2 = h;
}

// Pass 4: the first token of a heavy id adds the sums of pass 3 up in ascending order
template <typename TO>
__global__ __launch_bounds__(256) void embedding_bwd_heavy_kernel(const int64_t* __restrict__ ids, TO* __restrict__ dtable,
                                                                  const TokenLink* __restrict__ link,
                                                                  const float* __restrict__ partial2, int64_t dim,
                                                                  int64_t vocab_start, const int32_t* __restrict__ n_slots,
                                                                  const int32_t* __restrict__ head_of_slot) {
  if ((int)blockIdx.x >= *n_slots) return;
  const int i = head_of_slot[blockIdx.x];
  const TokenLink me = link[i];
  if (me.rank != 0 || me.slot < 0) return;
  const int64_t c0 = ((int64_t)blockIdx.y * 256 + threadIdx.x) * 4;
  if (c0 >= dim) return;
  const int nc = dim - c0 < 4 ? (int)(dim - c0) : 4;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int h = i; h >= 0;) {
    const TokenLink t = link[h];
    const float* src = partial2 + (int64_t)t.slot * dim + c0;
    for (int e = 0; e < nc; e++) acc[e] += src[e];
    h = t.next_head2;
  }
  TO* dst = dtable + (ids[i] - vocab_start) * dim + c0;
  for (int e = 0; e < nc; e++) elem_set(dst + e, elem_f32(dst[e]) + acc[e]);
}

template <typename V>
int launch_gather(const int64_t* ids, const void* table, void* out, int64_t n_ids, int64_t row_bytes,
                  int64_t vocab_start, int64_t vocab_end, int32_t* oob, hipStream_t s) {
  const int64_t vpr = row_bytes / (int64_t)sizeof(V);
  if (vpr >= 256 && vpr < (1ll << 30)) {
    const int64_t rows = n_ids < 256 * 256 ? n_ids : 256 * 256;
    hipLaunchKernelGGL(embedding_gather_rows_kernel<V>, dim3((unsigned)rows), dim3(256), 0, s, ids, (const V*)table,
                       (V*)out, n_ids, (int)vpr, vocab_start, vocab_end, oob);
    MTP_CHECK_LAUNCH("embedding_gather");
    return MTP_OK;
  }
  const int64_t total = n_ids * vpr;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 256 * 64) blocks = 256 * 64;
  hipLaunchKernelGGL(embedding_gather_kernel<V>, dim3((unsigned)blocks), dim3(256), 0, s, ids, (const V*)table,
                     (V*)out, n_ids, vpr, vocab_start, vocab_end, oob);
  MTP_CHECK_LAUNCH("embedding_gather");
  return MTP_OK;
}

}  // namespace

extern "C" int mtp_embedding_gather(const int64_t* ids, const void* table, void* out, int64_t n_ids,
                                    int64_t row_bytes, int64_t vocab_start, int64_t vocab_end, int32_t* oob_count,
                                    void* stream) {
  MTP_REQUIRE(n_ids >= 0 && row_bytes >= 1, MTP_EINVAL, "embedding_gather: n_ids=%lld row_bytes=%lld",
              (long long)n_ids, (long long)row_bytes);
  MTP_REQUIRE(vocab_end >= vocab_start, MTP_EINVAL, "embedding_gather: empty vocab range [%lld,%lld)",
              (long long)vocab_start, (long long)vocab_end);
  if (n_ids == 0) return MTP_OK;
  MTP_REQUIRE(ids && out && (table || vocab_end == vocab_start), MTP_EINVAL, "embedding_gather: null pointer");
  hipStream_t s = (hipStream_t)stream;
  const uintptr_t a = reinterpret_cast<uintptr_t>(table) | reinterpret_cast<uintptr_t>(out) | (uintptr_t)row_bytes;
  if ((a & 15) == 0) return launch_gather<u32x4_t>(ids, table, out, n_ids, row_bytes, vocab_start, vocab_end, oob_count, s);
  if ((a & 7) == 0) return launch_gather<u32x2_t>(ids, table, out, n_ids, row_bytes, vocab_start, vocab_end, oob_count, s);
  if ((a & 3) == 0) return launch_gather<uint32_t>(ids, table, out, n_ids, row_bytes, vocab_start, vocab_end, oob_count, s);
  if ((a & 1) == 0) return launch_gather<uint16_t>(ids, table, out, n_ids, row_bytes, vocab_start, vocab_end, oob_count, s);
  return launch_gather<uint8_t>(ids, table, out, n_ids, row_bytes, vocab_start, vocab_end, oob_count, s);
}

namespace {
// counters per batch: the power of two at or above 8 per token, between 1024 and 2^24
int64_t embedding_buckets(int64_t n_ids) {
  int64_t nb = 1024;
  while (nb < 8 * n_ids && nb < (1ll << 24)) nb <<= 1;
  return nb;
}
}  // namespace

// workspace: links [n], slot counter + bucket counters, head token of every slot, block sums of pass 2 and of pass 3
// ([emb_slots(n), dim] fp32 each)
namespace {
int64_t emb_slots(int64_t n_ids) { return n_ids / EMB_SEG + n_ids / (EMB_SEG + 1) + 1; }
int64_t emb_ws_links(int64_t n_ids) { return (n_ids * (int64_t)sizeof(TokenLink) + 255) / 256 * 256; }
int64_t emb_ws_buckets(int64_t n_ids) { return ((embedding_buckets(n_ids) + 1) * (int64_t)sizeof(int32_t) + 255) / 256 * 256; }
int64_t emb_ws_heads(int64_t n_ids) { return (emb_slots(n_ids) * (int64_t)sizeof(int32_t) + 255) / 256 * 256; }
}  // namespace

extern "C" int64_t mtp_embedding_bwd_workspace_bytes(int64_t n_ids, int64_t dim) {
  if (n_ids <= 0 || dim <= 0) return 0;
  return emb_ws_links(n_ids) + emb_ws_buckets(n_ids) + emb_ws_heads(n_ids) + 2 * emb_slots(n_ids) * dim * (int64_t)sizeof(float);
}

extern "C" int mtp_embedding_bwd(const int64_t* ids, const void* dout, void* dtable, void* workspace,
                                 int64_t workspace_bytes, int64_t n_ids, int64_t dim, int dtype, int dtable_dtype,
                                 int64_t vocab_start, int64_t vocab_end, void* stream) {
  MTP_REQUIRE(n_ids >= 0 && dim >= 1, MTP_EINVAL, "embedding_bwd: n_ids=%lld dim=%lld", (long long)n_ids,
              (long long)dim);
  MTP_REQUIRE(n_ids < (1ll << 31), MTP_EUNSUPPORTED, "embedding_bwd: n_ids=%lld exceeds 2^31-1", (long long)n_ids);
  MTP_REQUIRE(dtype == MTP_F32 || dtype == MTP_BF16 || dtype == MTP_F16, MTP_EINVAL, "embedding_bwd: unknown dtype %d",
              dtype);
  MTP_REQUIRE(dtable_dtype == MTP_F32 || dtable_dtype == MTP_BF16 || dtable_dtype == MTP_F16, MTP_EINVAL,
              "embedding_bwd: unknown dtable_dtype %d", dtable_dtype);
  if (n_ids == 0) return MTP_OK;
  MTP_REQUIRE(ids && dout && dtable && workspace, MTP_EINVAL, "embedding_bwd: null pointer");
  MTP_REQUIRE(workspace_bytes >= mtp_embedding_bwd_workspace_bytes(n_ids, dim), MTP_EWORKSPACE,
              "embedding_bwd: workspace %lld < %lld bytes", (long long)workspace_bytes,
              (long long)mtp_embedding_bwd_workspace_bytes(n_ids, dim));
  MTP_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 15) == 0, MTP_EINVAL, "embedding_bwd: workspace not 16-byte aligned");
  const int64_t chunks = (dim + 1023) / 1024;
  MTP_REQUIRE(chunks <= 65535, MTP_EUNSUPPORTED, "embedding_bwd: dim=%lld too large", (long long)dim);
  hipStream_t s = (hipStream_t)stream;
  TokenLink* link = (TokenLink*)workspace;
  // the slot counter sits in front of the bucket counters
  int32_t* bucket = reinterpret_cast<int32_t*>(static_cast<char*>(workspace) + emb_ws_links(n_ids)) + 1;
  int32_t* head_of_slot = reinterpret_cast<int32_t*>(static_cast<char*>(workspace) + emb_ws_links(n_ids) + emb_ws_buckets(n_ids));
  float* partial = reinterpret_cast<float*>(static_cast<char*>(workspace) + emb_ws_links(n_ids) + emb_ws_buckets(n_ids) +
                                            emb_ws_heads(n_ids));
  float* partial2 = partial + emb_slots(n_ids) * dim;
  const int n_bucket = (int)embedding_buckets(n_ids);
  hipLaunchKernelGGL(embedding_bucket_zero_kernel, dim3((unsigned)((n_bucket + 255) / 256)), dim3(256), 0, s, bucket,
                     n_bucket);
  hipLaunchKernelGGL(embedding_bucket_count_kernel, dim3((unsigned)((n_ids + 255) / 256)), dim3(256), 0, s, ids, bucket,
                     n_bucket, (int)n_ids, vocab_start, vocab_end);
  hipLaunchKernelGGL(embedding_link_kernel, dim3((unsigned)n_ids), dim3(256), 0, s, ids, link, (int)n_ids,
                     vocab_start, vocab_end, bucket, n_bucket, head_of_slot);
  MTP_CHECK_LAUNCH("embedding_link");
  const dim3 block(256);
  const bool vec = dim % 8 == 0 &&
                   ((reinterpret_cast<uintptr_t>(dout) | reinterpret_cast<uintptr_t>(dtable)) & 31) == 0;
  const dim3 grid((unsigned)n_ids, (unsigned)(vec ? (dim + 2047) / 2048 : chunks));
  const dim3 grid3((unsigned)emb_slots(n_ids), (unsigned)chunks);
#define MTP_EMB_BWD(T, TO)                                                                                           \
  do {                                                                                                               \
    if (vec)                                                                                                         \
      hipLaunchKernelGGL((embedding_bwd_kernel<T, TO, 8>), grid, block, 0, s, ids, (const T*)dout, (TO*)dtable, link, \
                         partial, dim, vocab_start);                                                                 \
    else                                                                                                             \
      hipLaunchKernelGGL((embedding_bwd_kernel<T, TO, 4>), grid, block, 0, s, ids, (const T*)dout, (TO*)dtable, link, \
                         partial, dim, vocab_start);                                                                 \
    hipLaunchKernelGGL(embedding_bwd_level2_kernel, grid3, block, 0, s, link, partial, partial2, dim, bucket - 1,    \
                       head_of_slot);                                                                                \
    hipLaunchKernelGGL((embedding_bwd_heavy_kernel<TO>), grid3, block, 0, s, ids, (TO*)dtable, link, partial2, dim,  \
                       vocab_start, bucket - 1, head_of_slot);                                                       \
  } while (0)
  if (dtype == MTP_F32 && dtable_dtype == MTP_F32)
    MTP_EMB_BWD(float, float);
  else if (dtype == MTP_BF16 && dtable_dtype == MTP_F32)
    MTP_EMB_BWD(uint16_t, float);
  else if (dtype == MTP_BF16 && dtable_dtype == MTP_BF16)
    MTP_EMB_BWD(uint16_t, uint16_t);
  else if (dtype == MTP_F16 && dtable_dtype == MTP_F32)
    MTP_EMB_BWD(f16s, float);
  else if (dtype == MTP_F16 && dtable_dtype == MTP_F16)
    MTP_EMB_BWD(f16s, f16s);
  else
    MTP_REQUIRE(false, MTP_EUNSUPPORTED, "embedding_bwd: the table gradient is fp32 or of the dtype of dout (%d -> %d)",
                dtype, dtable_dtype);
#undef MTP_EMB_BWD
  MTP_CHECK_LAUNCH("embedding_bwd");
  return MTP_OK;
}

