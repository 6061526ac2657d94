// Decode-step GEMV for gfx950: Y[B,N] = X[B,K] W[N,K]^T with B <= 32 rows of
// single-token activations, bf16 in / fp32 accumulate, and a variant that
// reduces the LM-head row straight to (max, argmax) without ever writing the
// logits (Merak/inference/text_generation_inference.py:223,226-227).
//
// The weight matrix is streamed from HBM exactly once, straight into the A
// operand of v_mfma_f32_16x16x32_bf16 (lane (i = l%16, g = l/16) supplies row
// i, k-group g).  What one load instruction touches decides the bandwidth: 16
// rows x 64 bytes (the natural operand layout) uses half of every 128-byte
// line per instruction and stalls near 5.7 TB/s; 8 rows x 128 bytes reaches
// 6.9 TB/s.  So the two loads of a 64-element k-pair are arranged as
//   load A: lane (i,g) <- row i%8,     bytes 64*(i/8)     + 16 g of the pair
//   load B: lane (i,g) <- row 8 + i%8, bytes 64*(1 - i/8) + 16 g
// and the two MFMA operands are picked per lane: first half of the pair =
// (i < 8 ? A : B), which holds row i at position i; second half = (i < 8 ? B : A),
// which holds row i^8 at position i and is rotated 8 lanes inside its group of
// 16 (one DPP move per register) to put row i at position i as well.
// The B operand is X^T (lane (b = l%16, g) loads X[b][k0+8g..]); X is tiny
// and stays in L2/L1.  The result tile D[i][b] needs no cross-lane reduction.
//
// A workgroup of 8 waves owns 16*R weight rows; the 128-byte k-pairs of those
// rows are dealt round-robin to the waves (split-K inside the workgroup), the 8
// partial tiles are summed through LDS in a fixed order, so results are
// bit-reproducible run to run.
#include "mtp_common.h"
#include <stdlib.h>
#include <mutex>
#include <type_traits>

namespace {

constexpr int GV_MAX_WAVES = 8;  // waves per workgroup: 8, or 4 for the register-heavy configurations
constexpr int GV_MAX_SLICES = 8; // slices along k, one workgroup each

// a workgroup's best (value, index) of one batch row, packed: see arg_key
typedef uint64_t ArgPart;

// torch.argmax ordering: NaN beats everything, ties go to the lower index
__device__ __forceinline__ bool arg_better(float va, int64_t ia, float vb, int64_t ib) {
  const bool na = va != va, nb = vb != vb;
  if (na != nb) return na;
  if (na) return ia < ib;
  return va > vb || (va == vb && ia < ib);
}

// The same order as one unsigned 64-bit key (row indices are below 2^31): larger key = better candidate,
// 0 = no candidate.  High word: the float mapped monotonically to unsigned, every NaN to the top; low word:
// the complement of the index, so that equal values prefer the lower index.
__device__ __forceinline__ uint64_t arg_key(float v, int64_t n) {
  const uint32_t u = v == 0.0f ? 0u : __float_as_uint(v);  // -0 and +0 compare equal
  uint32_t o = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  if (v != v) o = 0xffffffffu;
  return ((uint64_t)o << 32) | (uint32_t)(0xffffffffu - (uint32_t)n);
}
__device__ __forceinline__ float arg_key_value(uint64_t key) {
  const uint32_t o = (uint32_t)(key >> 32);
  if (o == 0xffffffffu) return __uint_as_float(0x7fc00000u);
  return __uint_as_float((o & 0x80000000u) ? (o ^ 0x80000000u) : ~o);
}
__device__ __forceinline__ int32_t arg_key_index(uint64_t key) { return (int32_t)(0xffffffffu - (uint32_t)key); }

// `ok` is a compile-time true on the unguarded path, which then has no branches at all
__device__ __forceinline__ bf16x8_t load_frag(const uint16_t* p, bool ok) {
  u32x4_t v = {0u, 0u, 0u, 0u};
  if (ok) v = *reinterpret_cast<const u32x4_t*>(p);
  return __builtin_bit_cast(bf16x8_t, v);
}

// weights are read exactly once: streaming (non-temporal) loads keep them from displacing X in the caches
__device__ __forceinline__ bf16x8_t load_frag_nt(const uint16_t* p, bool ok) {
  u32x4_t v = {0u, 0u, 0u, 0u};
  if (ok) v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
  return __builtin_bit_cast(bf16x8_t, v);
}

// value of the lane 8 places around inside each group of 16 lanes (DPP row_ror:8), i.e. of lane ^ 8
__device__ __forceinline__ uint32_t rot8_in_row(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x128, 0xf, 0xf, false);
}

// What a decoder block fuses around its linears.  NORM (template flag): X is the residual stream and the kernel
// multiplies by RMSNorm(X) instead: y = W (g * dtype(x * rstd_b)), rstd_b = rsqrt(mean_k x[b,k]^2 + eps), with the
// sum of squares handed over as partial sums per 16 elements (the producer below writes exactly those).  Every
// workgroup builds RMSNorm(X) in its LDS while its first weights are on their way (up to 8 rows of 4096 elements,
// see gemv_norm_fits) and takes its X fragments from there; the normalised rows never go to memory.
// `residual` (plain stores only): y = dtype(dtype(W x + bias) + residual), the model's `residual + hidden_states`;
// `sumsq_out`: per batch row and per 16 output rows, the sum of the squares of what was stored.
struct GemvFuse {
  const uint16_t* norm_w;    // NORM: RMSNorm weight [K]
  const float* sumsq_in;     // NORM: [B, K / 16]
  float eps;
  const uint16_t* residual;  // [B, N] or null
  float* sumsq_out;          // [B, ceil(N / 16)] or null
};

// MODE 0: store Y (+bias); MODE 1: SwiGLU store; MODE 2: argmax partials;
// MODE 3: SwiGLU with mixed row groups: rows 0-7 of a 16-row MFMA tile are gate rows, rows 8-15 the matching up
// rows, so a workgroup may own any number R of groups (8 R gate rows and their up rows) and the workgroup count can
// be made a multiple of the CU count (R = 7 gives exactly 256 workgroups for 14336 gate rows; with R = 4 the 448
// workgroups leave a quarter of the CUs with half the bytes in flight: 5.4 instead of 6.4 TB/s).  Load A fetches the
// gate rows of a k-pair, load B the up rows of the same pair: one product and one accumulator per tile, and two
// operand sets in the registers.  (A first form had the up rows walk half a row ahead of the gate rows, as the
// paired groups of MODE 1 do against the DRAM page conflicts of two streams a large power of two apart: a tile
// then holds two k positions and is multiplied with X at both, into two accumulators.  Measured, walking in step
// costs nothing here, and the registers it frees pay for the second operand set: 28672 x 4096 at 8 rows 39.8 ->
// 37.4 us, at 16 rows 39.6 -> 37.5 us.)
// W waves split K.  Configurations whose registers allow only 8 waves per CU run as two independent workgroups of
// 4 waves rather than one of 8: while one sums its partial tiles and writes its outputs the other keeps streaming.
// Everything a launch hands to a workgroup.
struct GemvArgs {
  const uint16_t* x;
  const uint16_t* w;
  const uint16_t* bias;
  uint16_t* y;
  ArgPart* part;
  int B;
  int64_t N, K;
  int rot_mul;
  int64_t ld;
  float* kpart;
  int32_t* karrived;
  int flags;
  GemvFuse fz;
  int n_part;     // MODE 2: row blocks of the launch = keys per batch row in `part` ([B][n_part])
};

// LDS of one workgroup, carved out of one buffer (so that a launch that holds two kinds of workgroups needs the
// larger of the two, not their sum): the partial tiles of the waves, the finished tile, the "I am last" cell, and
// with NORM the normalised rows of X and their scales.
template <int R, int NB, int W, bool NORM>
struct GemvLds {
  static constexpr int GP = (R * NB <= 8) ? R : 8 / NB;            // row groups per reduction phase
  static constexpr int XL_PAD = 32, XL_ELEMS = 8 * (4096 + XL_PAD);
  static constexpr int PART = 0;                                    // float [W][GP][NB][4][64]
  static constexpr int PART_BYTES = W * GP * NB * 4 * 64 * 4;
  static constexpr int FIN = PART + PART_BYTES;                     // float [16 NB][16 R + 1]
  static constexpr int FIN_BYTES = 16 * NB * (16 * R + 1) * 4;
  static constexpr int LAST = (FIN + FIN_BYTES + 15) / 16 * 16;     // int
  static constexpr int RSTD = LAST + 16;                            // float [32]
  static constexpr int XL = RSTD + 128;                             // uint16_t [XL_ELEMS]
  static constexpr int BYTES = NORM ? XL + XL_ELEMS * 2 : RSTD;
};

// bx, by, gy: the workgroup's place (row block, k slice) and the number of k slices; smem: GemvLds<...>::BYTES of LDS
// E > 0 (mixed SwiGLU groups, gate and up rows in step): the workgroup also owns E plain 16-row groups of a second
// matrix over the same X (xa: its weights, bias, output and row count; ebx: which block of 16 E rows), streamed in
// the same loop as E more row groups and stored without an activation.
template <int R, int NB, int MODE, bool GUARD, int D, int W, bool F16, bool NORM, bool PP, int E = 0>
__device__ __forceinline__ void gemv_body(const GemvArgs& ga, const int bx, const int by, const int gy, char* smem,
                                          const GemvArgs* xa = nullptr, const int ebx = 0) {
  constexpr int RT = R + E;   // row groups in the loop
  static_assert(E == 0 || (MODE == 3 && !NORM && !GUARD), "extra plain groups ride on mixed SwiGLU groups");
  const uint16_t* __restrict__ x = ga.x;
  const uint16_t* __restrict__ w = ga.w;
  const uint16_t* __restrict__ bias = ga.bias;
  uint16_t* __restrict__ y = ga.y;
  ArgPart* __restrict__ part = ga.part;
  const int B = ga.B;
  const int64_t N = ga.N, K = ga.K, ld = ga.ld;
  const int rot_mul = ga.rot_mul, flags = ga.flags;
  float* __restrict__ kpart = ga.kpart;
  int32_t* __restrict__ karrived = ga.karrived;
  const GemvFuse& fz = ga.fz;
  using L = GemvLds<RT, NB, W, NORM>;
  static_assert(!NORM || (!GUARD && MODE != 2), "the norm prologue needs K % 64 == 0 and a stored output");
  // K is the extent along k that this workgroup covers and ld the row stride of X and W: with gy > 1
  // the k range is cut into gy slices of K elements, one workgroup per (row block, slice); the
  // slices' partial sums meet in `kpart` and the slice that delivers last adds them up in slice order.
  const int64_t koff = (int64_t)by * K;
  using X = X16<F16>;   // bf16 or IEEE half: the MFMA and the conversions of the epilogue
  constexpr int GV_WAVES = W, GV_THREADS = W * MTP_WAVE;
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int li = lane & 15;  // weight row inside a 16-row group / batch column
  const int lg = lane >> 4;  // 8-element k group

  // rows of the R groups owned by this workgroup
  const int64_t half = N >> 1;  // SwiGLU: W = [gate rows | up rows]
  // Per row group: a wave-uniform base (first row of the group) and 32-bit per-lane element offsets for
  // the two loads.  GUARD (K not a multiple of 64) keeps the plain layout: load A = first 64 bytes of the
  // pair at row li, load B = the next 64.  Rows past the end are clamped to the last row (never stored).
  const uint16_t* wbase[RT];
  uint32_t offa[RT], offb[RT];
#pragma unroll
  for (int r = 0; r < RT; r++) {
    int64_t row0, lim;
    const bool extra = E > 0 && r >= R;
    if (extra) {
      row0 = (int64_t)ebx * (16 * E) + 16 * (r - R);
      lim = xa->N;
    } else if (MODE == 3) {
      row0 = (int64_t)bx * (8 * R) + 8 * r;
      lim = half;
    } else if (MODE == 1) {
      const int64_t j0 = (int64_t)bx * (8 * R);
      row0 = (r < R / 2) ? j0 + 16 * r : half + j0 + 16 * (r - R / 2);
      lim = (r < R / 2) ? half : N;
    } else {
      row0 = (int64_t)bx * (16 * R) + 16 * r;
      lim = N;
    }
    if (row0 >= lim) row0 = lim - 1;                 // a group entirely past the end reads the last row
    const int last = (int)(lim - 1 - row0);          // >= 0: largest valid row offset inside this group
    wbase[r] = (extra ? xa->w : w) + row0 * ld + koff;
    if (GUARD) {
      const int ra = li < last ? li : last;
      offa[r] = (uint32_t)(ra * ld + 8 * lg);
      offb[r] = offa[r] + 32;
    } else if (MODE == 3 && !extra) {
      // load A: gate row row0 + li%8; load B: the up row of the same index, `half` rows further down (the host
      // checks that this offset fits 32 bits)
      const int ra = (li & 7) < last ? (li & 7) : last;
      offa[r] = (uint32_t)(ra * ld + 32 * (li >> 3) + 8 * lg);
      offb[r] = (uint32_t)((half + ra) * ld + 32 * (1 - (li >> 3)) + 8 * lg);
    } else {
      const int ra = (li & 7) < last ? (li & 7) : last, rb = 8 + (li & 7) < last ? 8 + (li & 7) : last;
      offa[r] = (uint32_t)(ra * ld + 32 * (li >> 3) + 8 * lg);
      offb[r] = (uint32_t)(rb * ld + 32 * (1 - (li >> 3)) + 8 * lg);
    }
  }
  const uint16_t* xp[NB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    int b = li + 16 * nb;
    if (b >= B) b = B - 1;
    xp[nb] = x + (int64_t)b * ld + koff + 8 * lg;
  }

  // This wave's k range, in pairs of 32-element steps: a pair covers 64 elements = one 128-byte line of
  // every weight row, and the two 64-byte halves of a line are requested by adjacent instructions, so the
  // second request merges with the first one's miss instead of finding the line evicted again (with 16
  // rows x 8 groups x 8 waves in flight the L1 holds nothing for long).
  // Pairs are dealt round-robin to the 8 waves (wave w takes pairs w, w+8, ...): the waves advance in
  // step, so at any moment the workgroup reads 1 KiB contiguous from each of its rows, which keeps
  // DRAM pages open much longer than eight far-apart 128-byte streams per row would.
  const int64_t pairs = (K + 63) >> 6;
  const int64_t p0 = wave;
  // Every workgroup starts its walk along k at a different pair and wraps around: if all of them began at
  // k = 0 the whole chip would, at any moment, ask for the same few hundred bytes of every row, which
  // (rows being a power-of-two apart) live in the same few memory channels.
  // (Summation order along k therefore differs between workgroups: equal weight rows that live in different
  // workgroups give logits that are equal to rounding, not necessarily bit for bit.)
  const int64_t rot = GUARD || (pairs % GV_MAX_WAVES) ? 0 : ((int64_t)(bx + by) * rot_mul) % pairs;

  static_assert(MODE != 3 || (!GUARD && D == 1), "mixed SwiGLU groups: K % 64 == 0, depth 1");
  constexpr bool MIX = MODE == 3;
  f32x4_t acc[RT][NB];
#pragma unroll
  for (int r = 0; r < RT; r++)
#pragma unroll
    for (int nb = 0; nb < NB; nb++) acc[r][nb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const bool low = li < 8;

  // D pairs (8 apart) per step: with few rows per workgroup this is what keeps enough bytes in flight.
  // The host only picks D > 1 when every wave's share of the pairs is a multiple of D.
  const int64_t n_it = ((pairs - p0 + GV_WAVES - 1) / GV_WAVES) / D;
  // SwiGLU: the "up" rows sit exactly N/2 rows below the "gate" rows of the same workgroup, for the usual
  // shapes a large power of two apart, i.e. in the same memory channel and bank but another DRAM page.
  // Walking both at the same k makes the two streams evict each other's open page, so the up rows walk
  // half a row ahead (XS = 2 sets of X fragments, one per k position).
  // (paired groups with one batch tile only; the mixed groups walk in step)
  constexpr int XS = ((MODE == 1) && NB == 1 && !GUARD && E == 0) ? 2 : 1;
  const int64_t up_shift = (XS == 2 && pairs % GV_WAVES == 0 && !(flags & 1)) ? ((pairs / 2) & ~(int64_t)(GV_WAVES - 1)) : 0;
  // Operand registers of one step.  PP: two such sets used in turn, the next step's requests go out before the
  // current step's operands are waited for.  Otherwise one set is rotated by copying, which the compiler folds
  // into the requests themselves: each goes out right behind the last MFMA that read its register.
  bf16x8_t a_s0[D][RT][2], b_s0[D][XS][NB][2];
  bf16x8_t a_s1[D][RT][2], b_s1[D][XS][NB][2];
  // NORM: RMSNorm(X) is built once per workgroup in LDS, rows padded so that the 16-byte fragment reads of four
  // batch rows fall into different banks
  constexpr int XL_PAD = L::XL_PAD;
  [[maybe_unused]] const int xl_ld = (int)K + XL_PAD;
  [[maybe_unused]] uint16_t* x_lds = reinterpret_cast<uint16_t*>(smem + L::XL);
  const int b_row = li < B ? li : B - 1;
  // GUARD: K is not a multiple of 64, the last pair is partly (or half) past the end of the rows
  auto pair_k = [&](int64_t pq0, int d, int64_t (&ks)[2]) {
    int64_t pr = pq0 + d * GV_WAVES;
    if (pr >= pairs) pr -= pairs;
    int64_t pu = pr + up_shift;
    if (pu >= pairs) pu -= pairs;
    ks[0] = pr * 64;
    ks[1] = pu * 64;
  };
  auto load_w = [&](int64_t pq0, bf16x8_t (&a)[D][RT][2]) {
#pragma unroll
    for (int d = 0; d < D; d++) {
      int64_t ks[2];
      pair_k(pq0, d, ks);
#pragma unroll
      for (int r = 0; r < RT; r++) {
        if (MIX && r < R) {   // gate rows and up rows of the same pair
          a[d][r][0] = load_frag_nt(wbase[r] + ks[0] + offa[r], true);
          a[d][r][1] = load_frag_nt(wbase[r] + ks[1] + offb[r], true);
          continue;
        }
        const int64_t k = ks[(XS == 2 && r >= R / 2) ? 1 : 0];
        a[d][r][0] = load_frag_nt(wbase[r] + k + offa[r], !GUARD || (k + 8 * lg < K));
        a[d][r][1] = load_frag_nt(wbase[r] + k + offb[r], !GUARD || (k + 32 + 8 * lg < K));
      }
    }
  };
  auto load_x = [&](int64_t pq0, bf16x8_t (&b)[D][XS][NB][2]) {
#pragma unroll
    for (int d = 0; d < D; d++) {
      int64_t ks[2];
      pair_k(pq0, d, ks);
#pragma unroll
      for (int xs = 0; xs < XS; xs++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
          for (int hf = 0; hf < 2; hf++) {
            if constexpr (NORM)
              b[d][xs][nb][hf] = *reinterpret_cast<const bf16x8_t*>(&x_lds[b_row * xl_ld + (int)ks[xs] + 32 * hf + 8 * lg]);
            else
              b[d][xs][nb][hf] = load_frag(xp[nb] + ks[xs] + 32 * hf, !GUARD || (ks[xs] + 32 * hf + 8 * lg < K));
          }
    }
  };
  auto load_set = [&](int64_t pq0, bf16x8_t (&a)[D][RT][2], bf16x8_t (&b)[D][XS][NB][2]) {
    load_w(pq0, a);
    load_x(pq0, b);
  };
  // The two halves of group r's k-pair as MFMA operands.  GUARD: a0 / a1 are the halves themselves.  Otherwise pick
  // them per lane out of loads A and B; the second half then sits 8 lanes away inside its group of 16 (row i^8 at
  // position i): one DPP rotation per register puts it in place.
  auto halves = [&](const bf16x8_t& a0, const bf16x8_t& a1, bf16x8_t& h0, bf16x8_t& h1) {
    h0 = a0;
    h1 = a1;
    if (!GUARD) {
      h0 = low ? a0 : a1;
      const u32x4_t t = __builtin_bit_cast(u32x4_t, low ? a1 : a0);
      u32x4_t rt;
      rt.x = rot8_in_row(t.x); rt.y = rot8_in_row(t.y); rt.z = rot8_in_row(t.z); rt.w = rot8_in_row(t.w);
      h1 = __builtin_bit_cast(bf16x8_t, rt);
    }
  };
  // (the single-set loop takes the first halves of all batch tiles before the second ones: two dependent
  // products never stand next to each other inside its pinned sections)
  auto multiply_group = [&](int r, const bf16x8_t& h0, const bf16x8_t& h1, bf16x8_t (&bx)[XS][NB][2]) {
    if constexpr (PP) {
      const int xs = (XS == 2 && r >= R / 2) ? 1 : 0;
#pragma unroll
      for (int nb = 0; nb < NB; nb++) {
        acc[r][nb] = X::mfma16(h0, bx[xs][nb][0], acc[r][nb]);
        acc[r][nb] = X::mfma16(h1, bx[xs][nb][1], acc[r][nb]);
      }
    } else {
      const int xs = (XS == 2 && r >= R / 2) ? 1 : 0;
#pragma unroll
      for (int nb = 0; nb < NB; nb++) acc[r][nb] = X::mfma16(h0, bx[xs][nb][0], acc[r][nb]);
#pragma unroll
      for (int nb = 0; nb < NB; nb++) acc[r][nb] = X::mfma16(h1, bx[xs][nb][1], acc[r][nb]);
    }
  };
  auto multiply = [&](bf16x8_t (&a_cur)[D][RT][2], bf16x8_t (&b_cur)[D][XS][NB][2]) {
#pragma unroll
    for (int d = 0; d < D; d++)
#pragma unroll
      for (int r = 0; r < RT; r++) {
        bf16x8_t h0, h1;
        halves(a_cur[d][r][0], a_cur[d][r][1], h0, h1);
        multiply_group(r, h0, h1, b_cur[d]);
      }
  };
  // One step with a single set of weight registers: group after group, the two registers of a group are taken,
  // asked for again at once for the next step (pair pq_next), and only then multiplied; the order is pinned, so the
  // wait in front of a group covers that group's two loads alone and fifteen of sixteen requests stay in flight
  // while the step is multiplied.  (Left to itself the compiler gathers the selects of all groups at the top of
  // the loop behind one wait for every load: nothing in flight during the products.)  The X fragments of the
  // next step are asked for first, into the second set.
  auto roll_step = [&](int64_t pq_next, bf16x8_t (&a)[D][RT][2], bf16x8_t (&b_cur)[D][XS][NB][2],
                       bf16x8_t (&b_nxt)[D][XS][NB][2]) {
    load_x(pq_next, b_nxt);
#pragma unroll
    for (int d = 0; d < D; d++) {
      int64_t ks[2];
      pair_k(pq_next, d, ks);
#pragma unroll
      for (int r = 0; r < RT; r++) {
        bf16x8_t h0, h1;
        halves(a[d][r][0], a[d][r][1], h0, h1);
        __builtin_amdgcn_sched_barrier(0);   // the two registers are free from here on: the requests reuse them
        if (MIX && r < R) {
          a[d][r][0] = load_frag_nt(wbase[r] + ks[0] + offa[r], true);
          a[d][r][1] = load_frag_nt(wbase[r] + ks[1] + offb[r], true);
        } else {
          const int64_t k = ks[(XS == 2 && r >= R / 2) ? 1 : 0];
          a[d][r][0] = load_frag_nt(wbase[r] + k + offa[r], !GUARD || (k + 8 * lg < K));
          a[d][r][1] = load_frag_nt(wbase[r] + k + offb[r], !GUARD || (k + 32 + 8 * lg < K));
        }
        multiply_group(r, h0, h1, b_cur[d]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // NORM prologue, part 1: everything it reads is asked for before the first weights, folded after them, so
  // that the reduction, the normalisation and their two barriers sit inside the latency of that first request.
  //  * the row statistics: 16 lanes per batch row add up its partial sums of squares (16 bytes per load);
  //  * the rows themselves: thread t owns the 16-byte pieces t, t + 512, ... of every row and the matching
  //    pieces of the norm weight (B K <= 8 x 4096 elements: at most 8 pieces of X per thread).
  static_assert(!NORM || (NB == 1 && W == 8 && !GUARD && MODE != 2), "norm prologue: up to 8 rows, 512 threads, K % 64 == 0");
  constexpr int SQ_LOADS = 8, XV = 8;
  [[maybe_unused]] f32x4_t sv[SQ_LOADS];
  [[maybe_unused]] u32x4_t xv[XV], gv[XV];
  [[maybe_unused]] const int sq_nq = (int)(K >> 6);   // 16-byte groups of partial sums per row: (K / 16) / 4
  [[maybe_unused]] const int sq_b = tid >> 4, sq_sub = tid & 15;
  [[maybe_unused]] const int kvecs = (int)(K >> 3), kv_per = (kvecs + GV_THREADS - 1) / GV_THREADS;   // pieces per row / thread
  if constexpr (NORM) {
    const f32x4_t* sp = reinterpret_cast<const f32x4_t*>(fz.sumsq_in + (int64_t)(sq_b < B ? sq_b : 0) * (K >> 4));
#pragma unroll
    for (int u = 0; u < SQ_LOADS; u++) {   // no branches: out-of-range lanes read element 0 and drop it later
      const int q = sq_sub + 16 * u;
      sv[u] = sp[q < sq_nq ? q : 0];
    }
#pragma unroll
    for (int u = 0; u < XV; u++) {         // piece u: k-vector u % kv_per of batch row u / kv_per
      const int j = u % kv_per, b = u / kv_per;
      const int kv = tid + GV_THREADS * j;
      const bool ok = b < B && kv < kvecs;
      xv[u] = reinterpret_cast<const u32x4_t*>(x + (int64_t)(ok ? b : 0) * ld)[ok ? kv : 0];
      gv[u] = reinterpret_cast<const u32x4_t*>(fz.norm_w)[ok ? kv : 0];
    }
  }

  int64_t pq = p0 + rot;  // first pair of the step in flight; pairs % 8 == 0 whenever rot != 0, so wrapping keeps the wave's residue
  if (pq >= pairs) pq -= pairs;
  // (NORM: the host only launches with an equal, non-zero share of pairs for every wave; leaving the condition
  // out keeps the wait for the prologue's loads from covering these younger requests as well)
  if (NORM || n_it > 0) load_w(pq, a_s0);
  if constexpr (NORM) __builtin_amdgcn_sched_barrier(0);   // nothing of the prologue is waited for before this point
  if constexpr (!NORM) {
    if (n_it > 0) load_x(pq, b_s0);
  } else {
    // part 2: scale of every row, then the normalised rows into LDS
    float* rstd_lds = reinterpret_cast<float*>(smem + L::RSTD);
    {
      float s = 0.f;
#pragma unroll
      for (int u = 0; u < SQ_LOADS; u++)
        if (sq_b < B && sq_sub + 16 * u < sq_nq) s += (sv[u][0] + sv[u][1]) + (sv[u][2] + sv[u][3]);
      // the same order in all 16 lanes of a row: every lane ends with the same bits
      s += __shfl_xor(s, 8, 64);
      s += __shfl_xor(s, 4, 64);
      s += __shfl_xor(s, 2, 64);
      s += __shfl_xor(s, 1, 64);
      if (sq_sub == 0) rstd_lds[sq_b] = sq_b < B ? rsqrtf(s / (float)K + fz.eps) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < XV; u++) {
      const int j = u % kv_per, b = u / kv_per;
      const int kv = tid + GV_THREADS * j;
      if (b < B && kv < kvecs) {
        const float rs = rstd_lds[b];
        u32x4_t o;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          // g * dtype(x * rstd): the scaling in fp32, rounded to the tensor dtype, the product with the weight in
          // the tensor dtype (HF LlamaRMSNorm.forward)
          const uint32_t n = X::pack2(X::lo(xv[u][e]) * rs, X::hi(xv[u][e]) * rs);
          o[e] = X::pack2(X::lo(gv[u][e]) * X::lo(n), X::hi(gv[u][e]) * X::hi(n));
        }
        *reinterpret_cast<u32x4_t*>(&x_lds[b * xl_ld + 8 * kv]) = o;
      }
    }
    __syncthreads();
    load_x(pq, b_s0);
  }

  if (n_it > 0) {
    auto advance = [&]() {
      pq += GV_WAVES * D;
      if (pq >= pairs) pq -= pairs;
    };
    if constexpr (PP) {
      // set 0 holds the oldest step that has not been multiplied yet
      int64_t it = 1;
      for (; it + 1 < n_it; it += 2) {
        advance();
        load_set(pq, a_s1, b_s1);
        __builtin_amdgcn_sched_barrier(0);   // requests first, then the wait for the older set
        multiply(a_s0, b_s0);
        advance();
        load_set(pq, a_s0, b_s0);
        __builtin_amdgcn_sched_barrier(0);
        multiply(a_s1, b_s1);
      }
      if (it < n_it) {
        advance();
        load_set(pq, a_s1, b_s1);
        __builtin_amdgcn_sched_barrier(0);
        multiply(a_s0, b_s0);
        multiply(a_s1, b_s1);
      } else {
        multiply(a_s0, b_s0);
      }
    } else {
      // one set of weight registers (a_s0), two of X fragments used in turn
      int64_t it = 1;
      for (; it + 1 < n_it; it += 2) {
        advance();
        roll_step(pq, a_s0, b_s0, b_s1);
        advance();
        roll_step(pq, a_s0, b_s1, b_s0);
      }
      if (it < n_it) {
        advance();
        roll_step(pq, a_s0, b_s0, b_s1);
        multiply(a_s0, b_s1);
      } else {
        multiply(a_s0, b_s0);
      }
    }
  }

  // MODE 0 stores B x 16 R values, EPT per thread at most.  The residual values they are added to are asked for
  // here, ahead of the reduction below, and all of a thread's loads come before its stores (y may be the
  // residual tensor itself: a thread reads and writes the same elements).
  constexpr int EPT = (16 * NB * 16 * R + GV_THREADS - 1) / GV_THREADS;
  [[maybe_unused]] uint16_t rres[EPT];
  if constexpr (MODE == 0) {
    if (fz.residual) {
#pragma unroll
      for (int i = 0; i < EPT; i++) {
        const int e = i * GV_THREADS + tid;
        const int b = e / (16 * R), rl = e - b * (16 * R);
        const int64_t n = (int64_t)bx * (16 * R) + rl;
        rres[i] = (e < B * 16 * R && n < N) ? fz.residual[(int64_t)b * N + n] : (uint16_t)0;
      }
    }
  }

  // ---- sum the 8 k-slices through LDS: up to 8 tiles (row group x batch tile) per wave at a time, i.e. one
  // phase (two barriers) for all but the largest configuration ---------------------------------------------
  // part_lds[w][group][nb][j][lane]; fin[b][local row]
  constexpr int GP = L::GP;  // row groups per phase
  float (*part_lds)[GP][NB][4][64] = reinterpret_cast<float (*)[GP][NB][4][64]>(smem + L::PART);
  float (*fin)[16 * RT + 1] = reinterpret_cast<float (*)[16 * RT + 1]>(smem + L::FIN);
#pragma unroll
  for (int r0 = 0; r0 < RT; r0 += GP) {
#pragma unroll
    for (int rr = 0; rr < GP; rr++)
      if (r0 + rr < RT) {   // (the last phase of an odd number of groups is part empty)
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
          for (int j = 0; j < 4; j++) part_lds[wave][rr][nb][j][lane] = acc[r0 + rr][nb][j];
      }
    __syncthreads();
    const int live = (RT - r0 < GP ? RT - r0 : GP) * NB * 256;
    for (int e = tid; e < live; e += GV_THREADS) {
      const int rr = e / (NB * 256), nb = (e >> 8) % NB, j = (e >> 6) & 3, l = e & 63;
      float s = 0.f;
#pragma unroll
      for (int wv = 0; wv < GV_WAVES; wv++) s += part_lds[wv][rr][nb][j][l];
      // D[i][b]: lane l, register j holds row i = 4*(l/16)+j, column b = l%16
      fin[(l & 15) + 16 * nb][16 * (r0 + rr) + 4 * (l >> 4) + j] = s;
    }
    __syncthreads();
  }

  if (MODE != 2 && gy > 1) {
    // k slices: hand the partial over with device-scope stores, count arrivals; the last slice to arrive sums
    // all of them in slice order (its own included, read back), so the result does not depend on who is last.
    // Two values per access, and a thread asks for all it will sum before it looks at the first: the sum is a
    // single round trip to the memory-side cache whatever the batch and the number of row groups.
    constexpr int FIN = 16 * R;
    constexpr int PER = (16 * NB * FIN / 2 + GV_THREADS - 1) / GV_THREADS;   // pairs of values per thread
    const int S = gy, cnt = B * FIN;
    uint64_t* mine = reinterpret_cast<uint64_t*>(kpart + ((int64_t)bx * S + by) * cnt);
#pragma unroll
    for (int i = 0; i < PER; i++) {
      const int e = 2 * (i * GV_THREADS + tid);
      if (e < cnt) {
        const float lo = fin[e / FIN][e % FIN], hi = fin[(e + 1) / FIN][(e + 1) % FIN];
        __hip_atomic_store(mine + (e >> 1), ((uint64_t)__float_as_uint(hi) << 32) | __float_as_uint(lo), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    int* last_one = reinterpret_cast<int*>(smem + L::LAST);
    if (tid == 0) {
      const int seen = __hip_atomic_fetch_add(karrived + bx, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      *last_one = seen == S - 1;
      if (*last_one) __hip_atomic_store(karrived + bx, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!*last_one) return;
    const uint64_t* all = reinterpret_cast<const uint64_t*>(kpart + (int64_t)bx * S * cnt);
    const int64_t slice_stride = cnt >> 1;
    uint64_t v[PER][GV_MAX_SLICES];
#pragma unroll
    for (int i = 0; i < PER; i++) {
      const int e = 2 * (i * GV_THREADS + tid);
#pragma unroll
      for (int sl = 0; sl < GV_MAX_SLICES; sl++)
        v[i][sl] = (e < cnt && sl < S)
                       ? __hip_atomic_load(all + sl * slice_stride + (e >> 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                       : 0ull;
    }
#pragma unroll
    for (int i = 0; i < PER; i++) {
      const int e = 2 * (i * GV_THREADS + tid);
      if (e < cnt) {
        float lo = __uint_as_float((uint32_t)v[i][0]), hi = __uint_as_float((uint32_t)(v[i][0] >> 32));
#pragma unroll
        for (int sl = 1; sl < GV_MAX_SLICES; sl++) {   // slices beyond S hold +0: adding them changes nothing
          lo += __uint_as_float((uint32_t)v[i][sl]);
          hi += __uint_as_float((uint32_t)(v[i][sl] >> 32));
        }
        fin[e / FIN][e % FIN] = lo;
        fin[(e + 1) / FIN][(e + 1) % FIN] = hi;
      }
    }
    __syncthreads();
  }

  if (MODE == 3) {
    // fin[b][16 r + i]: i < 8 gate row j0 + 8 r + i, i >= 8 the up row of gate row j0 + 8 r + i - 8
    const int64_t j0 = (int64_t)bx * (8 * R);
    for (int e = tid; e < B * 8 * R; e += GV_THREADS) {
      const int b = e / (8 * R), rl = e - b * (8 * R);
      const int64_t jn = j0 + rl;
      if (jn < half) {
        const int col = 16 * (rl >> 3) + (rl & 7);
        float gate = fin[b][col], up = fin[b][col + 8];
        if (bias) {
          gate += X::from_bits(bias[jn]);
          up += X::from_bits(bias[half + jn]);
        }
        gate = X::from_bits(X::to_bits(gate));
        up = X::from_bits(X::to_bits(up));
        y[(int64_t)b * half + jn] = X::to_bits(silu_f(gate) * up);
      }
    }
    if constexpr (E > 0) {
      // the plain groups: fin[b][16 R + i] is row ebx * 16 E + i of the second matrix
      const int64_t n0 = (int64_t)ebx * (16 * E), n_x = xa->N;
      for (int e = tid; e < B * 16 * E; e += GV_THREADS) {
        const int b = e / (16 * E), rl = e - b * (16 * E);
        const int64_t n = n0 + rl;
        if (n < n_x) {
          float v = fin[b][16 * R + rl];
          if (xa->bias) v += X::from_bits(xa->bias[n]);
          xa->y[(int64_t)b * n_x + n] = X::to_bits(v);
        }
      }
    }
  } else if (MODE == 0) {
    // 16 consecutive lanes hold 16 consecutive output rows of one batch row: their squares meet in one
    // partial sum (fixed butterfly order), which is what the norm prologue of the next linear adds up
    const int64_t n0 = (int64_t)bx * (16 * R);
    const int total = B * 16 * R;
    const int64_t parts_out = (N + 15) >> 4;
#pragma unroll
    for (int i = 0; i < EPT; i++) {
      const int e = i * GV_THREADS + tid;
      const bool on = e < total;
      const int b = on ? e / (16 * R) : 0, rl = on ? e - b * (16 * R) : 0;
      const int64_t n = n0 + rl;
      float sq = 0.f;
      if (on && n < N) {
        float v = fin[b][rl];
        if (bias) v += X::from_bits(bias[n]);
        uint16_t out = X::to_bits(v);
        if (fz.residual) out = X::to_bits(X::from_bits(out) + X::from_bits(rres[i]));
        y[(int64_t)b * N + n] = out;
        const float f = X::from_bits(out);
        sq = f * f;
      }
      if (fz.sumsq_out && i * GV_THREADS < total) {   // (uniform over the workgroup)
        sq += __shfl_xor(sq, 8, 64);
        sq += __shfl_xor(sq, 4, 64);
        sq += __shfl_xor(sq, 2, 64);
        sq += __shfl_xor(sq, 1, 64);
        if (on && (rl & 15) == 0 && n < N) fz.sumsq_out[(int64_t)b * parts_out + (n >> 4)] = sq;
      }
    }
  } else if (MODE == 1) {
    const int64_t j0 = (int64_t)bx * (8 * R);
    for (int e = tid; e < B * 8 * R; e += GV_THREADS) {
      const int b = e / (8 * R), rl = e - b * (8 * R);
      const int64_t jn = j0 + rl;
      if (jn < half) {
        float gate = fin[b][rl], up = fin[b][8 * R + rl];
        if (bias) {
          gate += X::from_bits(bias[jn]);
          up += X::from_bits(bias[half + jn]);
        }
        // round the pre-activations to bf16 first, as the unfused layer stack would
        gate = X::from_bits(X::to_bits(gate));
        up = X::from_bits(X::to_bits(up));
        y[(int64_t)b * half + jn] = X::to_bits(silu_f(gate) * up);
      }
    }
  } else {
    // 512 / (16 NB) lanes per batch row: each folds its share of the 16 R rows, then a butterfly inside the
    // lane group.  (value, index) travel as one 64-bit key whose unsigned maximum is torch.argmax's choice.
    const int64_t n0 = (int64_t)bx * (16 * R);
    constexpr int TPB = GV_THREADS / (16 * NB);
    const int b = tid / TPB, sub = tid % TPB;
    uint64_t key = 0;
    if (b < B)
      for (int rl = sub; rl < 16 * R; rl += TPB) {
        const int64_t n = n0 + rl;
        if (n < N) {
          const uint64_t kk = arg_key(fin[b][rl], n);
          key = kk > key ? kk : key;
        }
      }
#pragma unroll
    for (int o = TPB / 2; o > 0; o >>= 1) {
      const uint64_t ok = (uint64_t)__shfl_xor((long long)key, o, 64);
      key = ok > key ? ok : key;
    }
    // (Finishing the pick inside this launch — every workgroup counts itself in at a counter, the last one of a
    // group folds the group's keys, the last group the groups — was built and measured: the counter's round trip
    // at the end of every one of 1000-2000 workgroups costs more than the second kernel it saves, 157 -> 175-183 us
    // at 1-8 batch rows, no change at 32.)
    // [batch row][row block]: the finishing kernel's lanes then read neighbouring keys
    if (sub == 0 && b < B) part[(int64_t)b * ga.n_part + bx] = key;
  }
}

template <int R, int NB, int MODE, bool GUARD, int D, int W, bool F16, bool NORM, bool PP>
__global__ __launch_bounds__(W * MTP_WAVE) void gemv_kernel(const GemvArgs ga) {
  __shared__ __attribute__((aligned(16))) char smem[GemvLds<R, NB, W, NORM>::BYTES];
  gemv_body<R, NB, MODE, GUARD, D, W, F16, NORM, PP>(ga, (int)blockIdx.x, (int)blockIdx.y, (int)gridDim.y, smem);
}

// Two products over the same X in one grid.  The grid is the second product's (SwiGLU: one workgroup per row block,
// as when it runs alone); the first n1 workgroups multiply a row block of the first product (plain store) before
// their own.  A product with few rows (QKV beside gate/up) then neither starts nor drains the chip in a launch of
// its own, and the grid stays at the second product's size (these configurations hold one workgroup per compute
// unit: a grid with more workgroups than compute units would run its last few alone).
// Tried and dropped: the first product's row blocks as workgroups of their own in front of the second's (272
// workgroups: 82 us against 63 us for the two launches, with one or two workgroups per compute unit alike).
constexpr int gemv_pair_depth(int r1) { return r1 == 1 ? 4 : r1 == 2 ? 2 : 1; }
// INLOOP (mixed groups only): the first n1 workgroups stream a block of 16 R1 rows of the first product in the same
// loop as their own rows, as R1 more row groups, instead of in a pass of their own.
template <int R1, int R2, int MODE2, int NB, int W, bool F16, bool INLOOP = false>
__global__ __launch_bounds__(W * MTP_WAVE) void gemv_pair_kernel(const GemvArgs g1, const GemvArgs g2, const int n1) {
  using L1 = GemvLds<R1, NB, W, false>;
  using L2 = GemvLds<INLOOP ? R1 + R2 : R2, NB, W, false>;
  __shared__ __attribute__((aligned(16))) char smem[L1::BYTES > L2::BYTES ? L1::BYTES : L2::BYTES];
  const int bid = (int)blockIdx.x;
  if constexpr (INLOOP) {
    if (bid < n1) gemv_body<R2, NB, MODE2, false, 1, W, F16, false, true, R1>(g2, bid, 0, 1, smem, &g1, bid);
    else gemv_body<R2, NB, MODE2, false, 1, W, F16, false, true>(g2, bid, 0, 1, smem);
    return;
  }
  if (bid < n1) {
    // a block of few rows lives on latency: it walks several k-pairs per step instead (the host checks that every
    // wave's share of the pairs divides)
    gemv_body<R1, NB, 0, false, gemv_pair_depth(R1), W, F16, false, true>(g1, bid, 0, 1, smem);
    __syncthreads();   // the second product reuses the LDS
  }
  gemv_body<R2, NB, MODE2, false, 1, W, F16, false, true>(g2, bid, 0, 1, smem);
}

// One workgroup per batch row folds that row's per-workgroup partials.  The kernel is a chain of memory
// latencies (its input was written a moment ago by other CUs), so every thread asks for eight partials
// before it looks at the first: 256 threads cover 2048 partials per round trip.
constexpr int AF_THREADS = 256, AF_WAVES = AF_THREADS / MTP_WAVE, AF_DEPTH = 8;
__global__ __launch_bounds__(AF_THREADS) void argmax_finish_kernel(const uint64_t* __restrict__ part, int n_part, int B,
                                                                   int64_t* __restrict__ idx, float* __restrict__ maxval) {
  const int b = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  uint64_t best = 0;
  for (int p0 = threadIdx.x; p0 < n_part; p0 += AF_THREADS * AF_DEPTH) {
    uint64_t a[AF_DEPTH];
#pragma unroll
    for (int u = 0; u < AF_DEPTH; u++) {
      const int p = p0 + u * AF_THREADS;
      a[u] = part[(int64_t)b * n_part + (p < n_part ? p : p0)];   // past the end: the first one again (changes nothing)
    }
#pragma unroll
    for (int u = 0; u < AF_DEPTH; u++) best = a[u] > best ? a[u] : best;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const uint64_t ok = (uint64_t)__shfl_xor((long long)best, o, 64);
    best = ok > best ? ok : best;
  }
  __shared__ uint64_t sk[AF_WAVES];
  if (lane == 0) sk[wave] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int wv = 1; wv < AF_WAVES; wv++) best = sk[wv] > best ? sk[wv] : best;
    idx[b] = arg_key_index(best);
    if (maxval) maxval[b] = arg_key_value(best);
  }
}

// Row-wise argmax over materialised logits: one workgroup per row.
template <typename T>
__global__ __launch_bounds__(256) void argmax_rows_kernel(const T* __restrict__ logits, int64_t* __restrict__ idx,
                                                          int64_t V) {
  const T* rp = logits + (int64_t)blockIdx.x * V;
  float bv = 0.f;
  int64_t bi = INT64_MAX;
  bool have = false;
  for (int64_t j = threadIdx.x; j < V; j += 256) {
    float v;
    if constexpr (std::is_same<T, f16s>::value)
      v = X16<true>::from_bits(rp[j].bits);
    else if constexpr (sizeof(T) == 2)
      v = bf16_bits_to_f32(rp[j]);
    else
      v = rp[j];
    if (!have || arg_better(v, j, bv, bi)) {
      bv = v;
      bi = j;
      have = true;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, 64);
    const int64_t oi = __shfl_xor(bi, o, 64);
    const int oh = __shfl_xor((int)have, o, 64);
    if (oh && (!have || arg_better(ov, oi, bv, bi))) {
      bv = ov;
      bi = oi;
      have = true;
    }
  }
  __shared__ float sv[4];
  __shared__ int64_t si[4];
  __shared__ int sh[4];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) {
    sv[wave] = bv;
    si[wave] = bi;
    sh[wave] = have;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int wv = 1; wv < 4; wv++)
      if (sh[wv] && (!have || arg_better(sv[wv], si[wv], bv, bi))) {
        bv = sv[wv];
        bi = si[wv];
        have = true;
      }
    idx[blockIdx.x] = bi;
  }
}

struct GemvCfg {
  int R;  // 16-row groups per workgroup
  int D;  // k-pairs in flight per wave and step
  int S;  // slices along k, one workgroup each (needs a workspace); 1 = the workgroup walks all of k
};

bool depth_ok(int64_t K, int d) { return d == 1 || (K % 64 == 0 && ((K / 64) % (GV_MAX_WAVES * d)) == 0); }

// The counters take the same 8 KiB whatever the shape, so that one zeroed workspace serves launches of different
// shapes in turn: with a size that followed N, the partial sums of a matrix with few rows would land where a
// larger one keeps its counters.  2048 counters cover every shape that is cut (fewer than 190 row blocks).
constexpr int64_t GV_COUNTER_BYTES = 8192;
GemvCfg pick_gemv_cfg(int64_t B, int64_t N, int64_t K, int mode, bool may_split = false) {
  const int64_t groups = ((mode == 1 ? N / 2 : N) + 15) / 16 * (mode == 1 ? 2 : 1);
  // Bytes in flight are what a bandwidth-bound kernel lives on: R*D k-pairs (2 KiB each) per wave.  Large
  // matrices take them as rows (X is re-read from L2 once per 16*R rows, which is what batches above 16
  // care about); matrices with few row groups keep every CU busy by going deeper along k instead.
  // Measured on 128256x4096, 28672x4096, 6144x4096, 4096x14336, 8192x3584 and 1280x8192 at B = 1, 8, 32.
  GemvCfg c{B > 16 ? 8 : 4, 1, 1};
  // The argmax form takes 8 row groups (4-wave workgroups) at every batch: 128256 x 4096 with its finishing kernel
  // 154.5 against 155.5 us at 1 row, 154 against 157 us at 8, 152 against 159 us at 16 (half as many keys to fold,
  // half as many reads of X).
  if (mode == 2) c.R = 8;
  // Above 16 batch rows X is read twice per 16 R weight rows: halving R until there are enough workgroups
  // makes the L2 -> CU traffic of X a multiple of the weight stream.  With a workspace the rows stay and k is
  // cut instead (each slice reads only its part of X); every wave of a slice gets the same number of pairs.
  // Measured (B = 16 and 32): 4096x14336 gains 17-23 %, matrices with K = 4096 lose (too little k per slice to
  // pay for the hand-over), batches up to 8 gain nothing.
  // Above 16 rows the cut is tried with 4 row groups (8 waves) first: 4096x14336 at 32 rows as 64 row blocks x 4
  // slices takes 26.7 us, as 32 x 8 (8 groups, 4 waves) 29.6 us.  MTP_GEMV_R forces the row groups here too.
  if (may_split && mode != 2 && K % 64 == 0 && groups * (int64_t)sizeof(int32_t) <= GV_COUNTER_BYTES) {
    int want = (B > 8 && K >= 8192) ? 0 : -1;
    static MtpTune tune_s("MTP_GEMV_S"), tune_r0("MTP_GEMV_R");
    want = tune_s.get(want);
    const int forced_r = tune_r0.get(0);
    const int cand[2] = {B > 16 ? 4 : c.R, c.R};
    GemvCfg best = c;
    int64_t best_wgs = 0;
    for (int ci = 0; ci < 2 && want >= 0; ci++) {
      GemvCfg t = c;
      t.R = (forced_r == 2 || forced_r == 4 || forced_r == 8) ? forced_r : cand[ci];
      if (groups / t.R >= 190) continue;
      const int waves = t.R >= 8 ? 4 : GV_MAX_WAVES;
      for (int sl = 2; sl <= GV_MAX_SLICES; sl *= 2) {
        if ((K / 64) % (sl * waves) != 0 || (want == 0 && K / 64 / (sl * waves) < 6)) break;
        t.S = sl;
        if (want ? sl >= want : groups / t.R * sl >= 190) break;
      }
      const int64_t wgs = groups / t.R * t.S;
      if (t.S > 1 && wgs > best_wgs) {
        best = t;
        best_wgs = wgs;
      }
      if (best_wgs >= 190) break;
    }
    if (best.S > 1) return best;
  }
  while (c.R > 1 && groups / c.R < 190) c.R >>= 1;
  if (mode == 1 && c.R < 2) c.R = 2;
  c.D = (B > 16 || c.R >= 4) ? 1 : 2;
  while (!depth_ok(K, c.D)) c.D >>= 1;
  static MtpTune tune_r("MTP_GEMV_R"), tune_d("MTP_GEMV_D");
  if (tune_r.is_set()) {
    const int r = tune_r.get(0);
    if (r == 1 || r == 2 || r == 4 || r == 8) c.R = (mode == 1 && r == 1) ? 2 : r;
    if (c.R * c.D > 4) c.D = c.R >= 4 ? 1 : 4 / c.R;
  }
  if (tune_d.is_set()) {
    const int d = tune_d.get(0);
    if ((d == 1 || d == 2 || d == 4) && c.R * d <= 4 && depth_ok(K, d)) c.D = d;
  }
  if (c.R >= 4) c.D = 1;
  return c;
}

// bytes of the arrival counters in front of the partial sums: one per 16 rows covers every configuration
int64_t gemv_counter_bytes(int64_t N) {
  (void)N;
  return GV_COUNTER_BYTES;
}

template <int MODE, bool NORM = false>
int launch_gemv(const void* x, const void* w, const void* bias, void* y, ArgPart* part, int64_t B, int64_t N,
                int64_t K, GemvCfg cfg, hipStream_t s, unsigned* n_wg_out, bool f16, void* workspace = nullptr,
                GemvFuse fz = GemvFuse{nullptr, nullptr, 0.f, nullptr, nullptr}) {
  const int R = cfg.R;
  const int64_t rows_per_wg = (MODE == 1) ? 8 * R : 16 * R;
  const int64_t span = (MODE == 1) ? N / 2 : N;
  const unsigned n_wg = (unsigned)((span + rows_per_wg - 1) / rows_per_wg);
  if (n_wg_out) *n_wg_out = n_wg;
  const int NB = B > 16 ? 2 : 1;
  static MtpTune tune_rot("MTP_GEMV_ROT"), tune_noshift("MTP_GEMV_NOSHIFT");
  int rot_mul = tune_rot.get(1);
  if (rot_mul < 0) rot_mul = 0;   // the rotation is taken modulo the number of pairs: it must not go negative
  int flags = 0;                  // bit 0: SwiGLU up rows walk in step with the gate rows (slower, same result)
  flags |= tune_noshift.get(0) ? 1 : 0;
  // k slices: counters first (one per row block, zero between launches), then the partial sums
  const int S = workspace ? cfg.S : 1;
  int32_t* karrived = static_cast<int32_t*>(workspace);
  float* kpart = workspace ? reinterpret_cast<float*>(static_cast<char*>(workspace) + gemv_counter_bytes(N)) : nullptr;
  const int64_t k_slice = K / S;
// two operand sets wherever the registers hold them (8 waves: 256 per lane)
#define GV_PP(RR, NNB) (MODE != 2)
  const GemvArgs ga{(const uint16_t*)x, (const uint16_t*)w, (const uint16_t*)bias, (uint16_t*)y, part, (int)B, N, k_slice,
                    rot_mul, K, kpart, karrived, flags, fz, (int)n_wg};
#define GV_LAUNCH_T(RR, NNB, GG, DD, FF)                                                                        \
  hipLaunchKernelGGL((gemv_kernel<RR, NNB, MODE, GG, DD, (RR >= 8 ? 4 : 8), FF, NORM, GV_PP(RR, NNB)>), dim3(n_wg, S), \
                     dim3((RR >= 8 ? 4 : 8) * MTP_WAVE), 0, s, ga)
#define GV_LAUNCH(RR, NNB, GG, DD)                 \
  do {                                             \
    if (f16) GV_LAUNCH_T(RR, NNB, GG, DD, true);   \
    else GV_LAUNCH_T(RR, NNB, GG, DD, false);      \
  } while (0)
#define GV_BY_DEPTH(RR, NNB)                                                   \
  do {                                                                         \
    if (K % 64 != 0) {                                                         \
      if constexpr (!NORM) GV_LAUNCH(RR, NNB, true, 1);                        \
    } else if (S > 1) GV_LAUNCH(RR, NNB, false, 1);                            \
    else if (RR * 4 <= 4 && cfg.D == 4) GV_LAUNCH(RR, NNB, false, (RR * 4 <= 4 ? 4 : 1)); \
    else if (RR * 2 <= 4 && cfg.D == 2) GV_LAUNCH(RR, NNB, false, (RR * 2 <= 4 ? 2 : 1)); \
    else GV_LAUNCH(RR, NNB, false, 1);                                         \
  } while (0)
  if (NB == 1) {
    if (R == 8) {
      if constexpr (!NORM) GV_BY_DEPTH(8, 1);   // 4 waves: batches above 16 only
    } else if (R == 4) GV_BY_DEPTH(4, 1);
    else if (R == 2) GV_BY_DEPTH(2, 1);
    else if constexpr (MODE != 1) GV_BY_DEPTH(1, 1);
  } else if constexpr (!NORM) {
    if (R == 8) GV_BY_DEPTH(8, 2);
    else if (R == 4) GV_BY_DEPTH(4, 2);
    else if (R == 2) GV_BY_DEPTH(2, 2);
    else if constexpr (MODE != 1) GV_BY_DEPTH(1, 2);
  }
#undef GV_BY_DEPTH
#undef GV_LAUNCH
#undef GV_LAUNCH_T
#undef GV_PP
  MTP_CHECK_LAUNCH("gemv");
  return MTP_OK;
}

// SwiGLU with mixed row groups (MODE 3): how many groups per workgroup.  0 = this shape keeps MODE 1.
// Every CU should hold the same number of bytes in flight: prefer the R whose workgroup count fills whole
// layers of 256 workgroups best, then the larger R (fewer reductions); too few workgroups are not an option.
// (28672 x 4096 at 17-32 batch rows: seven groups on 256 workgroups 41-42 us, eight paired groups on 224
// workgroups 44.5-46 us.  The first form built for two batch tiles kept the up rows half a row ahead, i.e. twice
// the accumulators and one operand set, and took 46 us; with 8 waves instead of 4 the present form spills and
// takes 50 us.)
int pick_mixed_groups(int64_t B, int64_t N, int64_t K) {
  const int64_t half = N / 2;
  if (K % 64 != 0 || (K / 64) % GV_MAX_WAVES != 0 || (half + 64) * K >= (1ll << 32)) return 0;
  static MtpTune tune_mix("MTP_GEMV_MIX");
  if (tune_mix.is_set()) {
    const int r = tune_mix.get(0);
    return r >= 1 && r <= 7 ? r : 0;
  }
  (void)B;   // one or two batch tiles: the same choice
  const int64_t groups = (half + 7) / 8;
  int best = 0;
  double best_eff = 0.0;
  for (int r = 1; r <= 7; r++) {
    const int64_t wgs = (groups + r - 1) / r;
    if (wgs < 200) continue;
    const double eff = (double)wgs / (double)((wgs + 255) / 256 * 256);
    if (eff >= best_eff - 1e-9) {
      best_eff = eff;
      best = r;
    }
  }
  return best_eff >= 0.9 ? best : 0;   // MODE 1 with R = 4 reaches 0.875 on the usual shapes
}

template <bool NORM = false>
int launch_gemv_mixed(const void* x, const void* w, const void* bias, void* y, int64_t B, int64_t N, int64_t K, int R,
                      hipStream_t s, bool f16, GemvFuse fz = GemvFuse{nullptr, nullptr, 0.f, nullptr, nullptr}) {
  const int64_t half = N / 2;
  const unsigned n_wg = (unsigned)((half + 8 * R - 1) / (8 * R));
  static MtpTune tune_rot("MTP_GEMV_ROT");
  int rot_mul = tune_rot.get(1);
  if (rot_mul < 0) rot_mul = 0;
  const GemvArgs ga{(const uint16_t*)x, (const uint16_t*)w, (const uint16_t*)bias, (uint16_t*)y, nullptr, (int)B, N, K,
                    rot_mul, K, nullptr, nullptr, 0, fz, 0};
#define GVM_T(RR, FF)                                                                                              \
  hipLaunchKernelGGL((gemv_kernel<RR, 1, 3, false, 1, GV_MAX_WAVES, FF, NORM, true>), dim3(n_wg),                      \
                     dim3(GV_MAX_WAVES * MTP_WAVE), 0, s, ga)
#define GVM(RR)                  \
  case RR:                       \
    if (f16) GVM_T(RR, true);    \
    else GVM_T(RR, false);       \
    break
  if (B > 16) {
    // two batch tiles: one k position per tile, two operand sets; four waves from five groups on (above 256 registers)
    if constexpr (!NORM) {
#define GVM2_T(RR, FF)                                                                                            \
  hipLaunchKernelGGL((gemv_kernel<RR, 2, 3, false, 1, (RR >= 5 ? 4 : GV_MAX_WAVES), FF, false, true>), dim3(n_wg), \
                     dim3((RR >= 5 ? 4 : GV_MAX_WAVES) * MTP_WAVE), 0, s, ga)
#define GVM2(RR)                  \
  case RR:                        \
    if (f16) GVM2_T(RR, true);    \
    else GVM2_T(RR, false);       \
    break
      switch (R) {
        GVM2(1);
        GVM2(2);
        GVM2(3);
        GVM2(4);
        GVM2(5);
        GVM2(6);
        GVM2(7);
        default: mtp_set_error("gemv: %d mixed row groups", R); return MTP_EINVAL;
      }
#undef GVM2
#undef GVM2_T
    }
    MTP_CHECK_LAUNCH("gemv");
    return MTP_OK;
  }
  switch (R) {
    GVM(1);
    GVM(2);
    GVM(3);
    GVM(4);
    GVM(5);
    GVM(6);
    GVM(7);
    default: mtp_set_error("gemv: %d mixed row groups", R); return MTP_EINVAL;
  }
#undef GVM
#undef GVM_T
  MTP_CHECK_LAUNCH("gemv");
  return MTP_OK;
}

// the norm prologue keeps RMSNorm(X) in LDS (8 rows of 4096 + 32 elements) and every thread of the 512 holds
// at most 8 sixteen-byte pieces of X on the way there
bool gemv_norm_fits(int64_t B, int64_t K) {
  if (B < 1 || K < 512 || K % 512 != 0 || K > 8192) return false;   // 8192 / 16 partial sums: 8 loads of 16 lanes
  const int64_t per_thread = (K / 8 + 511) / 512;
  return per_thread * B <= 8 && B * (K + 32) <= 8 * (4096 + 32);
}

int check_gemv_args(const char* what, const void* x, const void* w, int64_t B, int64_t N, int64_t K, int dtype) {
  MTP_REQUIRE(dtype == MTP_BF16 || dtype == MTP_F16, MTP_EUNSUPPORTED, "%s: dtype %d (bf16 or f16)", what, dtype);
  MTP_REQUIRE(B >= 1 && B <= 32, MTP_EUNSUPPORTED, "%s: B=%lld outside [1,32]", what, (long long)B);
  MTP_REQUIRE(N >= 1 && K >= 1, MTP_EINVAL, "%s: N=%lld K=%lld", what, (long long)N, (long long)K);
  MTP_REQUIRE(N < (1ll << 31), MTP_EUNSUPPORTED, "%s: N=%lld exceeds 2^31-1", what, (long long)N);
  MTP_REQUIRE(K % 8 == 0, MTP_EUNSUPPORTED, "%s: K=%lld is not a multiple of 8", what, (long long)K);
  MTP_REQUIRE(x && w, MTP_EINVAL, "%s: null pointer", what);
  MTP_REQUIRE(((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15) == 0, MTP_EUNSUPPORTED,
              "%s: x and w must be 16-byte aligned", what);
  return MTP_OK;
}

}  // namespace

extern "C" int64_t mtp_gemv_workspace_bytes(int64_t B, int64_t N, int64_t K, int epilogue) {
  if (B < 1 || B > 32 || N < 1 || K < 1) return 0;
  const GemvCfg c = pick_gemv_cfg(B, N, K, epilogue == MTP_EPI_SWIGLU ? 1 : 0, true);
  if (c.S <= 1) return 0;
  // every row block leaves B x (its rows) partial sums per slice; row blocks may overhang N by one block
  const int64_t rows = (N + 16 * c.R - 1) / (16 * c.R) * (16 * c.R) + (epilogue == MTP_EPI_SWIGLU ? 16 * c.R : 0);
  return gemv_counter_bytes(N) + (int64_t)c.S * B * rows * (int64_t)sizeof(float);
}

namespace {
int gemv_dispatch(const void* x, const void* w, const void* bias, void* y, void* workspace, int64_t workspace_bytes,
                  int64_t B, int64_t N, int64_t K, int epilogue, int dtype, void* stream, GemvFuse fz) {
  int rc = check_gemv_args("gemv", x, w, B, N, K, dtype);
  const bool f16 = dtype == MTP_F16;
  if (rc) return rc;
  MTP_REQUIRE(y, MTP_EINVAL, "gemv: null output");
  MTP_REQUIRE(y != x, MTP_EINVAL, "gemv: the output must not be the input (every workgroup reads all of X)");
  MTP_REQUIRE(epilogue == MTP_EPI_NONE || epilogue == MTP_EPI_BIAS || epilogue == MTP_EPI_SWIGLU, MTP_EINVAL,
              "gemv: epilogue %d not supported", epilogue);
  MTP_REQUIRE(epilogue != MTP_EPI_BIAS || bias, MTP_EINVAL, "gemv: MTP_EPI_BIAS without bias");
  hipStream_t s = (hipStream_t)stream;
  const int mode = epilogue == MTP_EPI_SWIGLU ? 1 : 0;
  const bool norm = fz.norm_w != nullptr;
  // without a workspace (or with one too small for the slices) every workgroup walks all of k; so does the
  // norm prologue, whose row statistics cover all of k
  const int64_t need = workspace && !norm ? mtp_gemv_workspace_bytes(B, N, K, epilogue) : 0;
  const bool split = need > 0 && workspace_bytes >= need && (reinterpret_cast<uintptr_t>(workspace) & 15) == 0;
  const GemvCfg cfg = pick_gemv_cfg(B, N, K, mode, split);
  if (mode == 1) {
    MTP_REQUIRE(N % 2 == 0, MTP_EINVAL, "gemv: SwiGLU needs an even N, got %lld", (long long)N);
    if (const int mixed = pick_mixed_groups(B, N, K))
      return norm ? launch_gemv_mixed<true>(x, w, bias, y, B, N, K, mixed, s, f16, fz)
                  : launch_gemv_mixed<false>(x, w, bias, y, B, N, K, mixed, s, f16, fz);
    if (norm) return launch_gemv<1, true>(x, w, bias, y, nullptr, B, N, K, cfg, s, nullptr, f16, nullptr, fz);
    return launch_gemv<1>(x, w, bias, y, nullptr, B, N, K, cfg, s, nullptr, f16, split ? workspace : nullptr, fz);
  }
  const void* b0 = epilogue == MTP_EPI_NONE ? nullptr : bias;
  if (norm) return launch_gemv<0, true>(x, w, b0, y, nullptr, B, N, K, cfg, s, nullptr, f16, nullptr, fz);
  return launch_gemv<0>(x, w, b0, y, nullptr, B, N, K, cfg, s, nullptr, f16, split ? workspace : nullptr, fz);
}
}  // namespace

extern "C" int mtp_gemv_ws(const void* x, const void* w, const void* bias, void* y, void* workspace,
                           int64_t workspace_bytes, int64_t B, int64_t N, int64_t K, int epilogue, int dtype,
                           void* stream) {
  return gemv_dispatch(x, w, bias, y, workspace, workspace_bytes, B, N, K, epilogue, dtype, stream,
                       GemvFuse{nullptr, nullptr, 0.f, nullptr, nullptr});
}

extern "C" int mtp_gemv_norm_fits(int64_t B, int64_t K) { return gemv_norm_fits(B, K) ? 1 : 0; }

// Two products over the same activations: y1 = x W1^T (+ bias1), act2 = SwiGLU(x W2^T (+ bias2)).  Above 16 batch
// rows (two batch tiles: the shape whose launches pay most for starting and draining on their own) and for the
// usual sizes both go out as one grid of 4-wave workgroups, the first product's row blocks in front; everything
// else runs as the two launches mtp_gemv_ws would make.  MTP_GEMV_PAIR = 0 keeps the two launches.
extern "C" int mtp_gemv_pair(const void* x, const void* w1, const void* bias1, void* y1, int64_t N1, const void* w2,
                             const void* bias2, void* act2, int64_t N2, void* workspace, int64_t workspace_bytes,
                             int64_t B, int64_t K, int dtype, void* stream) {
  int rc = check_gemv_args("gemv_pair", x, w1, B, N1, K, dtype);
  if (rc) return rc;
  rc = check_gemv_args("gemv_pair", x, w2, B, N2, K, dtype);
  if (rc) return rc;
  MTP_REQUIRE(y1 && act2, MTP_EINVAL, "gemv_pair: null output");
  MTP_REQUIRE(y1 != x && act2 != x, MTP_EINVAL, "gemv_pair: an output must not be the input");
  MTP_REQUIRE(N2 % 2 == 0, MTP_EINVAL, "gemv_pair: SwiGLU needs an even N2, got %lld", (long long)N2);
  static MtpTune tune_pair("MTP_GEMV_PAIR");
  hipStream_t s = (hipStream_t)stream;
  const bool f16 = dtype == MTP_F16;
  const int64_t half2 = N2 / 2;
  // one grid: two batch tiles, whole 64-element pairs, a second product that fills the chip by itself with one
  // workgroup per compute unit (seven mixed groups, or eight paired ones), 32-bit row offsets inside a workgroup's rows
  const int mixed = pick_mixed_groups(B, N2, K);
  const bool grid_ok = tune_pair.get(1) != 0 && K % 64 == 0 && 128 * K < (1ll << 31);
  const bool mix_grid = grid_ok && mixed == 7 && (B > 16 || tune_pair.get(1) != 2);
  const bool one_grid = mix_grid || (grid_ok && B > 16 && mixed == 0 && pick_gemv_cfg(B, N2, K, 1).R == 8 &&
                                     pick_gemv_cfg(B, N2, K, 1).S == 1);
  if (!one_grid) {
    rc = mtp_gemv_ws(x, w1, bias1, y1, workspace, workspace_bytes, B, N1, K, bias1 ? MTP_EPI_BIAS : MTP_EPI_NONE, dtype, stream);
    if (rc) return rc;
    return mtp_gemv_ws(x, w2, bias2, act2, workspace, workspace_bytes, B, N2, K, MTP_EPI_SWIGLU, dtype, stream);
  }
  static MtpTune tune_rot("MTP_GEMV_ROT"), tune_noshift("MTP_GEMV_NOSHIFT");
  int rot_mul = tune_rot.get(1);
  if (rot_mul < 0) rot_mul = 0;
  const int flags = tune_noshift.get(0) ? 1 : 0;
  const GemvFuse none{nullptr, nullptr, 0.f, nullptr, nullptr};
  const GemvArgs g1{(const uint16_t*)x, (const uint16_t*)w1, (const uint16_t*)bias1, (uint16_t*)y1, nullptr, (int)B, N1, K,
                    rot_mul, K, nullptr, nullptr, flags, none, 0};
  const GemvArgs g2{(const uint16_t*)x, (const uint16_t*)w2, (const uint16_t*)bias2, (uint16_t*)act2, nullptr, (int)B, N2, K,
                    rot_mul, K, nullptr, nullptr, flags, none, 0};
  // the first product's rows in blocks of 16 R1 rows, as few rows per block as still leaves no more blocks than
  // the second product has workgroups
  const unsigned n2 = mix_grid ? (unsigned)((half2 + 55) / 56) : (unsigned)((half2 + 63) / 64);
  // mixed groups: the first product's rows as one or two more row groups in the loop of the first workgroups
  // (MTP_GEMV_PAIR = 2 keeps the block in front of the loop)
  if (mix_grid && tune_pair.get(1) != 2) {
    const int e = (N1 + 15) / 16 <= (int64_t)n2 ? 1 : 2;
    const unsigned n1e = (unsigned)((N1 + 16 * e - 1) / (16 * e));
    if (n1e <= n2) {
#define GVE(EE, FF)                                                                                                    \
  do {                                                                                                                 \
    if (B > 16)                                                                                                        \
      hipLaunchKernelGGL((gemv_pair_kernel<EE, 7, 3, 2, 4, FF, true>), dim3(n2), dim3(4 * MTP_WAVE), 0, s, g1, g2, (int)n1e); \
    else                                                                                                               \
      hipLaunchKernelGGL((gemv_pair_kernel<EE, 7, 3, 1, 4, FF, true>), dim3(n2), dim3(4 * MTP_WAVE), 0, s, g1, g2, (int)n1e); \
  } while (0)
      if (e == 1) {
        if (f16) GVE(1, true);
        else GVE(1, false);
      } else {
        if (f16) GVE(2, true);
        else GVE(2, false);
      }
#undef GVE
      MTP_CHECK_LAUNCH("gemv_pair");
      return MTP_OK;
    }
  }
  int r1 = 1;
  while (r1 < 8 && (N1 + 16 * r1 - 1) / (16 * r1) > (int64_t)n2) r1 *= 2;
  if (B <= 16) r1 = 0;   // one batch tile: the in-loop form or two launches
  const unsigned n1 = (unsigned)((N1 + 16 * r1 - 1) / (16 * r1));
  if (r1 == 0 || n1 > n2 || (K / 64) % (4 * gemv_pair_depth(r1)) != 0) {
    rc = mtp_gemv_ws(x, w1, bias1, y1, workspace, workspace_bytes, B, N1, K, bias1 ? MTP_EPI_BIAS : MTP_EPI_NONE, dtype, stream);
    if (rc) return rc;
    return mtp_gemv_ws(x, w2, bias2, act2, workspace, workspace_bytes, B, N2, K, MTP_EPI_SWIGLU, dtype, stream);
  }
#define GVP_T(RR, FF)                                                                                               \
  do {                                                                                                              \
    if (mix_grid)                                                                                                   \
      hipLaunchKernelGGL((gemv_pair_kernel<RR, 7, 3, 2, 4, FF>), dim3(n2), dim3(4 * MTP_WAVE), 0, s, g1, g2, (int)n1); \
    else                                                                                                            \
      hipLaunchKernelGGL((gemv_pair_kernel<RR, 8, 1, 2, 4, FF>), dim3(n2), dim3(4 * MTP_WAVE), 0, s, g1, g2, (int)n1); \
  } while (0)
#define GVP(RR)                \
  case RR:                     \
    if (f16) GVP_T(RR, true);  \
    else GVP_T(RR, false);     \
    break
  switch (r1) {
    GVP(1);
    GVP(2);
    GVP(4);
    GVP(8);
  }
#undef GVP
#undef GVP_T
  MTP_CHECK_LAUNCH("gemv_pair");
  return MTP_OK;
}

extern "C" int mtp_gemv_fused(const void* x, const void* w, const void* bias, void* y, const void* norm_weight,
                              const float* sumsq_in, float eps, const void* residual, float* sumsq_out,
                              void* workspace, int64_t workspace_bytes, int64_t B, int64_t N, int64_t K, int epilogue,
                              int dtype, void* stream) {
  if (norm_weight || sumsq_in) {
    MTP_REQUIRE(norm_weight && sumsq_in, MTP_EINVAL, "gemv_fused: the norm prologue needs its weight and the sums of squares");
    // every wave of a workgroup walks the same number of 64-element pairs, and a row's partial sums (one per 16
    // elements) are read 16 bytes at a time
    MTP_REQUIRE(K % 512 == 0, MTP_EUNSUPPORTED, "gemv_fused: the norm prologue needs K %% 512 == 0, got %lld", (long long)K);
    MTP_REQUIRE(gemv_norm_fits(B, K), MTP_EUNSUPPORTED,
                "gemv_fused: the norm prologue holds B K <= 8 x 4096 elements, K <= 8192, got B=%lld K=%lld (mtp_gemv_norm_fits)",
                (long long)B, (long long)K);
    MTP_REQUIRE(((reinterpret_cast<uintptr_t>(norm_weight) | reinterpret_cast<uintptr_t>(sumsq_in)) & 15) == 0,
                MTP_EUNSUPPORTED, "gemv_fused: norm_weight and sumsq_in must be 16-byte aligned");
    MTP_REQUIRE(eps >= 0.f, MTP_EINVAL, "gemv_fused: eps %g", (double)eps);
  }
  if (residual || sumsq_out) {
    MTP_REQUIRE(epilogue == MTP_EPI_NONE || epilogue == MTP_EPI_BIAS, MTP_EINVAL,
                "gemv_fused: residual / sumsq_out go with plain stores, not epilogue %d", epilogue);
    MTP_REQUIRE((reinterpret_cast<uintptr_t>(sumsq_out) & 3) == 0, MTP_EINVAL, "gemv_fused: sumsq_out not 4-byte aligned");
  }
  return gemv_dispatch(x, w, bias, y, workspace, workspace_bytes, B, N, K, epilogue, dtype, stream,
                       GemvFuse{(const uint16_t*)norm_weight, sumsq_in, eps, (const uint16_t*)residual, sumsq_out});
}

extern "C" int mtp_gemv(const void* x, const void* w, const void* bias, void* y, int64_t B, int64_t N, int64_t K,
                        int epilogue, int dtype, void* stream) {
  return mtp_gemv_ws(x, w, bias, y, nullptr, 0, B, N, K, epilogue, dtype, stream);
}

extern "C" int64_t mtp_gemv_argmax_workspace_bytes(int64_t B, int64_t N, int64_t K) {
  (void)K;
  if (B < 1 || N < 1) return 0;
  // one key per (workgroup, batch row); the smallest workgroup owns 16 rows
  return ((N + 15) / 16) * B * (int64_t)sizeof(ArgPart);
}

extern "C" int mtp_gemv_argmax(const void* x, const void* w, int64_t* idx, float* maxval, void* workspace,
                               int64_t workspace_bytes, int64_t B, int64_t N, int64_t K, int dtype, void* stream) {
  int rc = check_gemv_args("gemv_argmax", x, w, B, N, K, dtype);
  if (rc) return rc;
  MTP_REQUIRE(idx && workspace, MTP_EINVAL, "gemv_argmax: null pointer");
  MTP_REQUIRE(workspace_bytes >= mtp_gemv_argmax_workspace_bytes(B, N, K), MTP_EWORKSPACE,
              "gemv_argmax: workspace %lld < %lld bytes", (long long)workspace_bytes,
              (long long)mtp_gemv_argmax_workspace_bytes(B, N, K));
  MTP_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 7) == 0, MTP_EINVAL, "gemv_argmax: workspace not 8-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  unsigned n_wg = 0;
  rc = launch_gemv<2>(x, w, nullptr, nullptr, (ArgPart*)workspace, B, N, K, pick_gemv_cfg(B, N, K, 2), s, &n_wg,
                      dtype == MTP_F16);
  if (rc) return rc;
  hipLaunchKernelGGL(argmax_finish_kernel, dim3((unsigned)B), dim3(AF_THREADS), 0, s, (const ArgPart*)workspace, (int)n_wg,
                     (int)B, idx, maxval);
  MTP_CHECK_LAUNCH("argmax_finish");
  return MTP_OK;
}

// ---- the greedy pick for callers that cannot allocate --------------------------------------------------------
// Same kernels as mtp_gemv_argmax; the per-workgroup partial maxima live in a device array of this library
// instead of a caller's workspace.  Every GPU holds its own copy of the array at its own address: the address is
// asked for once per device (hipGetSymbolAddress, with that device current) and kept.
#define MTP_ARGMAX_STATIC_BYTES (4ll << 20)
static __device__ __align__(256) unsigned char g_argmax_scratch[MTP_ARGMAX_STATIC_BYTES];
namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};
// device address of g_argmax_scratch on the current device, or null (error set)
void* argmax_scratch_ptr() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    mtp_set_error("gemv_argmax_noalloc: hipGetDevice: %s (device %d)", hipGetErrorString(e), dev);
    return nullptr;
  }
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* q = nullptr;
    e = hipGetSymbolAddress(&q, HIP_SYMBOL(g_argmax_scratch));
    if (e != hipSuccess || !q) {
      mtp_set_error("gemv_argmax_noalloc: hipGetSymbolAddress: %s", hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = q;
  }
  return g_scratch_ptr[dev];
}
}  // namespace

extern "C" int64_t mtp_gemv_argmax_noalloc_max_bytes(void) { return MTP_ARGMAX_STATIC_BYTES; }

extern "C" int mtp_gemv_argmax_noalloc(const void* x, const void* w, int64_t* idx, float* maxval, int64_t B, int64_t N,
                                       int64_t K, int dtype, void* stream) {
  int rc = check_gemv_args("gemv_argmax_noalloc", x, w, B, N, K, dtype);
  if (rc) return rc;
  MTP_REQUIRE(idx, MTP_EINVAL, "gemv_argmax_noalloc: null pointer");
  const int64_t need = mtp_gemv_argmax_workspace_bytes(B, N, K);
  MTP_REQUIRE(need <= MTP_ARGMAX_STATIC_BYTES, MTP_EWORKSPACE,
              "gemv_argmax_noalloc: B=%lld N=%lld needs %lld bytes of scratch, the library holds %lld (use mtp_gemv_argmax "
              "with a workspace)", (long long)B, (long long)N, (long long)need, (long long)MTP_ARGMAX_STATIC_BYTES);
  void* scratch = argmax_scratch_ptr();
  if (!scratch) return MTP_EDEVICE;
  return mtp_gemv_argmax(x, w, idx, maxval, scratch, MTP_ARGMAX_STATIC_BYTES, B, N, K, dtype, stream);
}

extern "C" int mtp_argmax_rows(const void* logits, int64_t* idx, int64_t B, int64_t V, int dtype, void* stream) {
  MTP_REQUIRE(B >= 0 && V >= 1, MTP_EINVAL, "argmax_rows: B=%lld V=%lld", (long long)B, (long long)V);
  MTP_REQUIRE(B < (1ll << 31), MTP_EUNSUPPORTED, "argmax_rows: B too large");
  if (B == 0) return MTP_OK;
  MTP_REQUIRE(logits && idx, MTP_EINVAL, "argmax_rows: null pointer");
  hipStream_t s = (hipStream_t)stream;
  if (dtype == MTP_F32)
    hipLaunchKernelGGL(argmax_rows_kernel<float>, dim3((unsigned)B), dim3(256), 0, s, (const float*)logits, idx, V);
  else if (dtype == MTP_BF16)
    hipLaunchKernelGGL(argmax_rows_kernel<uint16_t>, dim3((unsigned)B), dim3(256), 0, s, (const uint16_t*)logits,
                       idx, V);
  else if (dtype == MTP_F16)
    hipLaunchKernelGGL(argmax_rows_kernel<f16s>, dim3((unsigned)B), dim3(256), 0, s, (const f16s*)logits, idx, V);
  else
    MTP_REQUIRE(false, MTP_EINVAL, "argmax_rows: unknown dtype %d", dtype);
  MTP_CHECK_LAUNCH("argmax_rows");
  return MTP_OK;
}
