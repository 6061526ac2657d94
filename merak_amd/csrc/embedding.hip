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

// dtable[id - start, :] += dout[i, :]  (fp32 atomics; one thread per element pair)
template <typename T>
__global__ __launch_bounds__(256) void embedding_bwd_kernel(const int64_t* __restrict__ ids,
                                                            const T* __restrict__ dout, float* __restrict__ dtable,
                                                            int64_t n_ids, int64_t dim, int64_t vocab_start,
                                                            int64_t vocab_end) {
  const int64_t total = n_ids * dim;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    const int64_t r = i / dim;
    const int64_t c = i - r * dim;
    const int64_t id = ids[r];
    if (id < vocab_start || id >= vocab_end) continue;
    float g;
    if constexpr (sizeof(T) == 2)
      g = bf16_bits_to_f32(dout[i]);
    else
      g = dout[i];
    unsafeAtomicAdd(dtable + (id - vocab_start) * dim + c, g);
  }
}

template <typename V>
int launch_gather(const int64_t* ids, const void* table, void* out, int64_t n_ids, int64_t row_bytes,
                  int64_t vocab_start, int64_t vocab_end, int32_t* oob, hipStream_t s) {
  const int64_t vpr = row_bytes / (int64_t)sizeof(V);
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

extern "C" int mtp_embedding_bwd(const int64_t* ids, const void* dout, float* dtable, int64_t n_ids, int64_t dim,
                                 int dtype, int64_t vocab_start, int64_t vocab_end, void* stream) {
  MTP_REQUIRE(n_ids >= 0 && dim >= 1, MTP_EINVAL, "embedding_bwd: n_ids=%lld dim=%lld", (long long)n_ids,
              (long long)dim);
  MTP_REQUIRE(dtype == MTP_F32 || dtype == MTP_BF16, MTP_EINVAL, "embedding_bwd: unknown dtype %d", dtype);
  if (n_ids == 0) return MTP_OK;
  MTP_REQUIRE(ids && dout && dtable, MTP_EINVAL, "embedding_bwd: null pointer");
  hipStream_t s = (hipStream_t)stream;
  const int64_t total = n_ids * dim;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 256 * 64) blocks = 256 * 64;
  if (dtype == MTP_F32)
    hipLaunchKernelGGL(embedding_bwd_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, s, ids, (const float*)dout,
                       dtable, n_ids, dim, vocab_start, vocab_end);
  else
    hipLaunchKernelGGL(embedding_bwd_kernel<uint16_t>, dim3((unsigned)blocks), dim3(256), 0, s, ids,
                       (const uint16_t*)dout, dtable, n_ids, dim, vocab_start, vocab_end);
  MTP_CHECK_LAUNCH("embedding_bwd");
  return MTP_OK;
}
