// Backward of the key-length-masked attention for gfx950 (head dims up to 64, bf16 / fp16 storage, fp32 arithmetic).
//
// With S = Q K^T / sqrt(d), P = exp(S - lse) (lse saved by the training forward), D_i = sum_d O[i, d] dO[i, d]:
//   dV = P^T dO,   dP = dO V^T,   dS = P * (dP - D) / sqrt(d),   dQ = dS K,   dK = dS^T Q
// (the recipe of the reference's backward kernels, accelerators/attention/kernels/tilelang.py:405-435, 598-699).
// Two kernels, both recomputing S and dP from the inputs, so that every output element has exactly one writer and a
// fixed summation order (the reference accumulates dQ with floating-point atomics):
//   attn_bwd_dq_kernel   one workgroup per (batch, head, 128 queries): a lane owns one query, the keys stream through
//                        LDS in chunks of 64; also writes D for the second kernel.
//   attn_bwd_dkv_kernel  one workgroup per (batch, head, 128 keys): a lane owns one key, the queries stream through LDS.
// All products are formed transposed, as in the forward kernel: the streamed operand is the MFMA A operand (rows from
// LDS), the lane-owned operand the B operand (registers), so the accumulator holds one owned column per lane and the
// 16 registers run over the streamed rows (register r <-> row (r / 4) * 8 + hh * 4 + r % 4 of a 32-row tile). The
// second product of each pair consumes those values as a B operand; its streamed A operand is the same chunk read
// column-wise with ds_read_b64_tr_b16, at row offsets that follow that register order, so every chunk is staged once,
// row-major, and nothing is transposed on the way into LDS.
#include <math.h>

#include "ts_common.h"

namespace taac {
namespace {

constexpr int kThreads = 256;
constexpr int kOwn = 128;    // owned rows (queries or keys) per workgroup: 32 per wavefront
constexpr int kChunk = 64;   // streamed rows per LDS chunk

struct AttnBwdParams {
  const void* q;
  const void* k;
  const void* v;
  const void* o;
  const void* dout;
  const float* lse;       // [B, H, Tq]
  float* delta;           // [B, H, Tq] workspace: written by the dQ kernel, read by the dK / dV kernel
  void* dq;
  void* dk;
  void* dv;
  const int32_t* key_lengths;
  const uint8_t* drop_mask;  // byte mask with rows [Tq][Tk] at batch / head strides mask_bs / mask_hs, or null:
                             // training dropout (keep mask, non-zero = keep) or pair visibility (non-zero = visible)
  int64_t mask_bs, mask_hs;  // elements between the mask matrices of consecutive samples / heads (0: shared)
  const uint8_t* key_valid;  // visibility mode: [B, Tk] bytes, non-zero = the key can be seen at all; or null
                             // (bit modes: [B, ceil(Tk / 32)] words)
  const uint32_t* bit_words; // bit modes: rows of ceil(Tk / 32) words per query, bits_bs words between the samples' matrices
  int64_t bits_bs;
  float drop_scale;          // 1 / (1 - p)
  int32_t B, H, Tq, Tk, d;
  int64_t qs[4], ks[4], vs[4], os[4], dos[4], dqs[4], dks[4], dvs[4];
  float scale;            // 1 / sqrt(d)
  int32_t zero_pad;       // query rows at or beyond key_lengths[b] carry no gradient
  int32_t causal;
  uint32_t nblk;          // owned-row blocks per (batch, head)
  uint32_t total;
};

template <typename T>
struct Mfma32;
template <>
struct Mfma32<bf16_t> {
  static __device__ __forceinline__ f32x16 run(bf16x8 a, bf16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mfma32<f16_t> {
  static __device__ __forceinline__ f32x16 run(f16x8 a, f16x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

__device__ __forceinline__ float pair_sum(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, static_cast<uint32_t>(r[0])) + __builtin_bit_cast(float, static_cast<uint32_t>(r[1]));
}

template <typename T>
__device__ __forceinline__ uint32_t pack2(T lo, T hi) {
  return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, lo)) |
         (static_cast<uint32_t>(__builtin_bit_cast(uint16_t, hi)) << 16);
}

// A streamed chunk (kChunk rows of DP features) lies row-major and unpadded in LDS, the 16-byte pieces of row r stored
// at piece ^ row_swizzle(r), and serves two kinds of reads without bank conflicts:
//   rows as MFMA A operands (lane l32 reads one piece of row l32: 16 consecutive rows of one piece cover all banks);
//   columns as MFMA A operands through ds_read_b64_tr_b16: a 16-lane group reads 32 contiguous bytes of four
//   consecutive rows and every lane receives four rows of one feature (see streamed_column_offset below).
// +32 rows leave the swizzle unchanged, +16 rows too, +8 rows flip kSwizzleBit8 of it.
template <int DP>
__device__ __forceinline__ int row_swizzle(int r) {
  static_assert(DP == 32 || DP == 64, "row swizzles are written for 64- and 128-byte rows");
  return DP == 32 ? (r >> 2) & 3 : ((r >> 1) & 7) ^ (((r >> 1) & 1) << 2);
}
template <int DP>
struct SwizzleStep {
  static constexpr uint32_t kRows8 = (DP == 32 ? 2 : 4) * 16;  // address bits that +8 rows flip
};

// Staging of one streamed operand. DMA: the chunk goes from global memory straight into LDS (one 1 KB transfer per
// wavefront and piece slot, no staging registers); rows at or beyond row_end repeat the last valid row, whose products
// the callers cancel (finite values times a zero probability); needs d == DP and 32-bit source offsets. Otherwise the
// chunk travels through registers (fetch, then commit after the barrier), with zeros for rows at or beyond row_end and
// features at or beyond d. The lane's slot i * 256 + tid is (row slot / C8, stored piece slot % C8).
template <typename T, int DP, bool DMA>
struct Streamed {
  typedef typename Vec8<T>::type vec_t;
  static constexpr int C8 = DP / 8, ROWB = DP * 2, TILE_BYTES = kChunk * ROWB;
  static constexpr int PPT = kChunk * C8 / kThreads;
  static_assert(kChunk * C8 % kThreads == 0, "whole transfers per wavefront");
  const T* base;
  int64_t stride;
  int srow, piece;          // the lane's row inside a chunk (slot 0) and the logical piece stored at its slot
  uint32_t row_bytes;
  vec_t reg[DMA ? 1 : PPT];
  __device__ __forceinline__ void init(const T* b, int64_t st, int tid) {
    base = b;
    stride = st;
    srow = tid / C8;
    piece = (tid % C8) ^ row_swizzle<DP>(srow);
    row_bytes = static_cast<uint32_t>(st) * 2u;
  }
  __device__ __forceinline__ void fetch(int row0, int row_end, int d, uint8_t* tile, int tid) {
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      int row = row0 + srow + i * (kThreads / C8);
      if (DMA) {
        row = row < row_end ? row : row_end - 1;  // row_end >= 1 here
        lds_dma16_offset(base, __umul24(static_cast<uint32_t>(row), row_bytes) + static_cast<uint32_t>(piece * 16),
                         tile + i * (kThreads * 16) + (tid / kWave) * (kWave * 16));
      } else if (row < row_end && piece * 8 < d) {
        reg[DMA ? 0 : i] = *reinterpret_cast<const vec_t*>(base + row * stride + piece * 8);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) reg[DMA ? 0 : i][e] = static_cast<T>(0.f);
      }
    }
  }
  __device__ __forceinline__ void commit(uint8_t* tile, int tid) const {
    if (DMA) return;
#pragma unroll
    for (int i = 0; i < PPT; ++i) *reinterpret_cast<vec_t*>(tile + i * (kThreads * 16) + tid * 16) = reg[DMA ? 0 : i];
  }
};

// Byte offset (inside a chunk tile) of the lane's row fragment of k-step 0 of a 32-row tile: row l32, piece hh; k-step s
// is this offset with s * 32 XORed in, the next 32-row tile 32 * ROWB further.
template <int DP>
__device__ __forceinline__ uint32_t streamed_row_offset(int l32, int hh) {
  return static_cast<uint32_t>(l32 * (DP * 2) + ((hh ^ row_swizzle<DP>(l32)) * 16));
}

// Byte offset of the lane's address for the transposed reads. Accumulator register j of a 32-row tile belongs to row
// (j / 4) * 8 + hh * 4 + j % 4, so the B operand of the second product (registers 8 s2 .. 8 s2 + 7) runs over rows
// 16 s2 + hh * 4 + 0..3 and 16 s2 + 8 + hh * 4 + 0..3. The matching A operand holds, for feature l32 (of row block mb),
// those eight rows: two transposed reads, at row offsets 16 s2 and 16 s2 + 8, in each of which lane r of 16-lane group
// g points at row hh * 4 + r / 4, features 16 (g % 2) + 4 (r % 4) .. + 3. Row block mb XORs 64 mb into the offset and
// the read 8 rows further SwizzleStep<DP>::kRows8.
template <int DP>
__device__ __forceinline__ uint32_t streamed_column_offset(int lane) {
  const int row = 4 * (lane / 32) + (lane % 16) / 4;
  const int piece = 2 * ((lane / 16) % 2) + (lane % 4) / 2;
  return static_cast<uint32_t>(row * (DP * 2) + ((piece ^ row_swizzle<DP>(row)) * 16) + (lane % 2) * 8);
}

// A operand of the second product for (32-row tile at byte offset tile_off, k-step s2) from a tile base address.
template <typename T, int DP, int TILE_OFF>
__device__ __forceinline__ void read_columns(u32x2 (&frag)[2], uint32_t addr) {
  lds_read_tr16<TILE_OFF>(frag[0], addr);
  lds_read_tr16<TILE_OFF + 8 * DP * 2>(frag[1], addr ^ SwizzleStep<DP>::kRows8);
}

// Owned rows as B-operand fragments: lane (l32, hh) holds features 16 s + 8 hh .. + 7 of row `row` (zeros when !ok).
template <typename T, int DP>
__device__ __forceinline__ void load_owned(const T* __restrict__ base, int64_t stride, int row, bool ok, int d, int hh,
                                           typename Vec8<T>::type (&frag)[DP / 16]) {
  typedef typename Vec8<T>::type vec_t;
#pragma unroll
  for (int s = 0; s < DP / 16; ++s) {
    const int col = 16 * s + 8 * hh;
    if (ok && col < d) {
      frag[s] = *reinterpret_cast<const vec_t*>(base + row * stride + col);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) frag[s][e] = static_cast<T>(0.f);
    }
  }
}

// Writes MB accumulators (transposed tile: rows = features, column = owned row of the lane) as rows of `out`.
template <typename T, int DP>
__device__ __forceinline__ void store_owned(const f32x16 (&acc)[DP / 32], uint8_t* tile, T* __restrict__ out,
                                            int64_t stride, int row0, int row_limit, int d, int lane) {
  typedef typename Vec8<T>::type vec_t;
  typedef typename Vec8<T>::half_type vec4_t;
  constexpr int C8 = DP / 8, OROW = DP * 2 + 16;
  const int l32 = lane % 32, hh = lane / 32;
#pragma unroll
  for (int mb = 0; mb < DP / 32; ++mb)
#pragma unroll
    for (int jq = 0; jq < 4; ++jq) {
      vec4_t ov;
#pragma unroll
      for (int e = 0; e < 4; ++e) ov[e] = static_cast<T>(acc[mb][jq * 4 + e]);
      *reinterpret_cast<vec4_t*>(tile + l32 * OROW + (mb * 32 + jq * 8 + hh * 4) * 2) = ov;
    }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  constexpr int RPP = kWave / C8;
  const int c8 = lane % C8;
#pragma unroll
  for (int pass = 0; pass < 32 / RPP; ++pass) {
    const int r = pass * RPP + lane / C8;
    const vec_t val = *reinterpret_cast<const vec_t*>(tile + r * OROW + c8 * 16);
    if (row0 + r < row_limit && c8 * 8 < d) *reinterpret_cast<vec_t*>(out + (row0 + r) * stride + c8 * 8) = val;
  }
}

// The second product of a 32-row tile: acc[mb] += columns(tile)^T-fragments x b[s2], the column fragments read
// transposed from the chunk tile at `addr` (tile base + streamed_column_offset), one row block at a time.
template <typename T, int DP, int TILE_OFF>
__device__ __forceinline__ void accumulate_columns(f32x16 (&acc)[DP / 32], const typename Vec8<T>::type (&b)[2], uint32_t addr) {
  typedef typename Vec8<T>::type vec_t;
  static_for<DP / 32>([&](auto mb_tag) {
    constexpr int mb = decltype(mb_tag)::value;
    u32x2 f[2][2];
    read_columns<T, DP, TILE_OFF>(f[0], addr ^ (mb * 64));
    read_columns<T, DP, TILE_OFF + 16 * DP * 2>(f[1], addr ^ (mb * 64));
    // hand-issued reads are awaited by hand; the fragments are tied to the wait so that no consumer moves above it
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(f[0][0]), "+v"(f[0][1]), "+v"(f[1][0]), "+v"(f[1][1]) : : "memory");
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      const u32x4 bits = {f[s2][0][0], f[s2][0][1], f[s2][1][0], f[s2][1][1]};
      acc[mb] = Mfma32<T>::run(__builtin_bit_cast(vec_t, bits), b[s2], acc[mb]);
    }
  });
}

// Same for two accumulators that share the tile position (dV from dO and P, dK from Q and dS).
template <typename T, int DP, int TILE_OFF>
__device__ __forceinline__ void accumulate_columns2(f32x16 (&acc_a)[DP / 32], const typename Vec8<T>::type (&b_a)[2],
                                                    uint32_t addr_a, f32x16 (&acc_b)[DP / 32],
                                                    const typename Vec8<T>::type (&b_b)[2], uint32_t addr_b) {
  typedef typename Vec8<T>::type vec_t;
  static_for<DP / 32>([&](auto mb_tag) {
    constexpr int mb = decltype(mb_tag)::value;
    u32x2 fa[2][2], fb[2][2];
    read_columns<T, DP, TILE_OFF>(fa[0], addr_a ^ (mb * 64));
    read_columns<T, DP, TILE_OFF + 16 * DP * 2>(fa[1], addr_a ^ (mb * 64));
    read_columns<T, DP, TILE_OFF>(fb[0], addr_b ^ (mb * 64));
    read_columns<T, DP, TILE_OFF + 16 * DP * 2>(fb[1], addr_b ^ (mb * 64));
    asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(fa[0][0]), "+v"(fa[0][1]), "+v"(fa[1][0]), "+v"(fa[1][1]) : : "memory");
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      const u32x4 bits = {fa[s2][0][0], fa[s2][0][1], fa[s2][1][0], fa[s2][1][1]};
      acc_a[mb] = Mfma32<T>::run(__builtin_bit_cast(vec_t, bits), b_a[s2], acc_a[mb]);
    }
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fb[0][0]), "+v"(fb[0][1]), "+v"(fb[1][0]), "+v"(fb[1][1]) : : "memory");
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      const u32x4 bits = {fb[s2][0][0], fb[s2][0][1], fb[s2][1][0], fb[s2][1][1]};
      acc_b[mb] = Mfma32<T>::run(__builtin_bit_cast(vec_t, bits), b_b[s2], acc_b[mb]);
    }
  });
}

// Keep bytes of four consecutive keys of one mask row as one word (byte e = key key0 + e); keys at or beyond Tk read as 0.
__device__ __forceinline__ uint32_t keep_bytes4(const uint8_t* row, int key0, int Tk, bool aligned) {
  if (aligned && key0 + 3 < Tk) return *reinterpret_cast<const uint32_t*>(row + key0);
  uint32_t w = 0u;
#pragma unroll
  for (int e = 0; e < 4; ++e)
    if (key0 + e < Tk) w |= static_cast<uint32_t>(row[key0 + e]) << (8 * e);
  return w;
}

// MODE (both kernels) says what the byte mask is. kMaskDropout: the caller's keep mask of the training forward; dV takes
// keep ? P / (1 - p) : 0 and the score gradient P * ((keep ? dP / (1 - p) : 0) - D) / sqrt(d), as the reference's backward
// kernel does (tilelang.py:535-570). kMaskVisible: the pairs the forward's mask let through (any bool mask, e.g. a
// structured one written out); an invisible pair has probability 0 - the log-sum-exp was taken over the visible ones.
// kMaskBits: the same as bits, in the layout of the structured forward: drop_mask holds 32-bit words, row i of a sample's
// matrix at word (b * mask_bs + i * wpr), wpr = ceil(Tk / 32), bit j % 32 of word j / 32 = pair (i, j); key_valid holds
// [B, wpr] words. One word per 32-key tile instead of 32 bytes.
// kMaskBitsDropout: the bit form for the pairs AND the byte keep mask of dropout (both pointers).
constexpr int kMaskNone = 0, kMaskDropout = 1, kMaskVisible = 2, kMaskBits = 3, kMaskBitsDropout = 4;

template <typename T, int DP, bool DMA, int MODE = kMaskNone>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(DP == 32 ? 4 : 3))) void attn_bwd_dq_kernel(const AttnBwdParams p) {
  constexpr bool DROPOUT = MODE == kMaskDropout || MODE == kMaskBitsDropout;
  constexpr bool BITS = MODE == kMaskBits || MODE == kMaskBitsDropout;
  typedef typename Vec8<T>::type vec_t;
  constexpr int KSTEPS = DP / 16, MB = DP / 32;
  constexpr int ROWB = DP * 2, TILE_BYTES = kChunk * ROWB, BUF_BYTES = 2 * TILE_BYTES;  // a chunk of K, then of V
  constexpr int NBUF = DMA ? 2 : 1;  // direct transfers land in the other buffer while this one is consumed
  constexpr int OROW = DP * 2 + 16;
  constexpr int OUT_BYTES = (kThreads / kWave) * 32 * OROW;
  __shared__ __attribute__((aligned(1024))) uint8_t smem[NBUF * BUF_BYTES > OUT_BYTES ? NBUF * BUF_BYTES : OUT_BYTES];

  const uint32_t logical = xcd_remap(blockIdx.x, p.total);
  const int blk = static_cast<int>(logical % p.nblk);
  const int bh = static_cast<int>(logical / p.nblk);
  const int h = bh % p.H, b = bh / p.H;
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave, l32 = lane % 32, hh = lane / 32;
  const T* qb = static_cast<const T*>(p.q) + b * p.qs[0] + h * p.qs[1];
  const T* kb = static_cast<const T*>(p.k) + b * p.ks[0] + h * p.ks[1];
  const T* vb = static_cast<const T*>(p.v) + b * p.vs[0] + h * p.vs[1];
  const T* ob = static_cast<const T*>(p.o) + b * p.os[0] + h * p.os[1];
  const T* dob = static_cast<const T*>(p.dout) + b * p.dos[0] + h * p.dos[1];
  T* dqb = static_cast<T*>(p.dq) + b * p.dqs[0] + h * p.dqs[1];

  int len = p.Tk;
  if (p.key_lengths != nullptr) {
    len = p.key_lengths[b];
    len = len < 0 ? 0 : (len > p.Tk ? p.Tk : len);
  }
  const int q_valid = p.zero_pad ? (len < p.Tq ? len : p.Tq) : p.Tq;
  const int q_begin = blk * kOwn;
  const int qi = q_begin + wave * 32 + l32;
  const bool q_ok = qi < q_valid;
  int kv_end = len;
  if (p.causal) kv_end = kv_end < q_begin + kOwn ? kv_end : q_begin + kOwn;
  if (q_begin >= q_valid) kv_end = 0;  // a block of padded queries: zero gradient, no key is staged
  // A wavefront whose 32 queries all lie in the padding only helps staging.
  const bool wave_active = q_begin + wave * 32 < q_valid;

  vec_t qf[KSTEPS], dof[KSTEPS], of[KSTEPS];
  load_owned<T, DP>(qb, p.qs[2], qi, q_ok, p.d, hh, qf);
  load_owned<T, DP>(dob, p.dos[2], qi, q_ok, p.d, hh, dof);
  load_owned<T, DP>(ob, p.os[2], qi, q_ok, p.d, hh, of);
  float delta = 0.f;
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
    for (int e = 0; e < 8; ++e) delta = fmaf(static_cast<float>(of[s][e]), static_cast<float>(dof[s][e]), delta);
  delta = pair_sum(delta);
  const int64_t stat = (static_cast<int64_t>(b) * p.H + h) * p.Tq + qi;
  if (hh == 0 && qi < p.Tq) p.delta[stat] = delta;
  const float lse = q_ok ? p.lse[stat] : -INFINITY;
  const float c = p.scale * 1.4426950408889634f;  // scores -> base-2 exponent
  // a row without a visible key (or in the padding) gets +inf: exp2(x - inf) = 0 switches it off without a select
  const float lse2 = lse > -INFINITY ? lse * 1.4426950408889634f : INFINITY;
  const float delta_scaled = delta * p.scale;

  f32x16 dqacc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int j = 0; j < 16; ++j) dqacc[mb][j] = 0.f;

  Streamed<T, DP, DMA> k_rows, v_rows;
  k_rows.init(kb, p.ks[2], tid);
  v_rows.init(vb, p.vs[2], tid);
  auto fetch = [&](int kc0, int buffer) {
    k_rows.fetch(kc0, kv_end, p.d, smem + buffer * BUF_BYTES, tid);
    v_rows.fetch(kc0, kv_end, p.d, smem + buffer * BUF_BYTES + TILE_BYTES, tid);
  };
  const uint32_t row_off = streamed_row_offset<DP>(l32, hh);
  const uint32_t col_off = streamed_column_offset<DP>(lane);
  // bit mode: the lane's query row of the mask, two words (64 keys) per chunk, requested one chunk ahead of their use
  [[maybe_unused]] uint32_t chunk_words[kChunk / 32] = {}, next_words[kChunk / 32] = {};
  auto fetch_words = [&](int kc0, uint32_t (&dst)[kChunk / 32]) {
    const int wpr = (p.Tk + 31) / 32;
    const uint32_t* row = p.bit_words + b * p.bits_bs + static_cast<int64_t>(qi < p.Tq ? qi : 0) * wpr;
    const uint32_t* valid = p.key_valid != nullptr ? reinterpret_cast<const uint32_t*>(p.key_valid) + static_cast<int64_t>(b) * wpr : nullptr;
#pragma unroll
    for (int t = 0; t < kChunk / 32; ++t) {
      const int w = kc0 / 32 + t;
      const bool inside = qi < p.Tq && w < wpr;  // a tile at or beyond Tk has no word
      dst[t] = inside ? row[w] : 0u;
      if (inside && valid != nullptr) dst[t] &= valid[w];
    }
  };
  if (BITS && kv_end > 0) fetch_words(0, chunk_words);
  if (kv_end > 0) fetch(0, 0);
  int buf = 0;
  for (int kc0 = 0; kc0 < kv_end; kc0 += kChunk) {
    if (BITS && kc0 + kChunk < kv_end) fetch_words(kc0 + kChunk, next_words);
    if (DMA) {
      vm_wait<0>();     // this wavefront's pieces of the chunk have landed ...
      __syncthreads();  // ... everyone's have, and everyone is done reading the other buffer
      if (kc0 + kChunk < kv_end) fetch(kc0 + kChunk, buf ^ 1);
    } else {
      if (kc0 > 0) __syncthreads();  // every wavefront is done reading the previous chunk
      k_rows.commit(smem, tid);
      v_rows.commit(smem + TILE_BYTES, tid);
      __syncthreads();
      if (kc0 + kChunk < kv_end) fetch(kc0 + kChunk, 0);
    }
    const uint8_t* kt_rows = smem + buf * BUF_BYTES;
    const uint32_t col_addr = lds_offset(kt_rows) + col_off;
    if (DMA) buf ^= 1;
    static_for<kChunk / 32>([&](auto kt_tag) {
      constexpr int kt = decltype(kt_tag)::value;
      if (kc0 + kt * 32 >= kv_end || !wave_active) return;  // wavefront-uniform
      if (p.causal && kc0 + kt * 32 > q_begin + wave * 32 + 31) return;  // every key of the tile lies after the queries
      f32x16 sacc, dpacc;
#pragma unroll
      for (int j = 0; j < 16; ++j) sacc[j] = dpacc[j] = 0.f;
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s) {
        const uint32_t off = kt * 32 * ROWB + (row_off ^ (s * 32));
        const vec_t ka = *reinterpret_cast<const vec_t*>(kt_rows + off);
        const vec_t va = *reinterpret_cast<const vec_t*>(kt_rows + TILE_BYTES + off);
        sacc = Mfma32<T>::run(ka, qf[s], sacc);
        dpacc = Mfma32<T>::run(va, dof[s], dpacc);
      }
      // only a tile that crosses the end of the keys or the causal diagonal needs per-element tests
      const int k_tile = kc0 + kt * 32;
      const bool tail = k_tile + 32 > kv_end || (p.causal && k_tile + 31 > q_begin + wave * 32);
      if (tail) {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const int key = k_tile + (j / 4) * 8 + hh * 4 + (j % 4);
          if (key >= kv_end || (p.causal && key > qi)) sacc[j] = -INFINITY;
        }
      }
      vec_t dsb[2];
      if (MODE == kMaskBits) {
        const uint32_t word = chunk_words[kt];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const bool on = ((word >> ((j / 4) * 8 + hh * 4 + (j % 4))) & 1u) != 0u;
          const float prob = on ? __builtin_amdgcn_exp2f(fmaf(sacc[j], c, -lse2)) : 0.f;
          dsb[j / 8][j % 8] = static_cast<T>(prob * fmaf(dpacc[j], p.scale, -delta_scaled));
        }
      } else if (MODE == kMaskBitsDropout) {
        const uint32_t word = chunk_words[kt];
        const bool aligned = (p.Tk % 4 == 0) && (reinterpret_cast<uintptr_t>(p.drop_mask) % 4 == 0) &&
                             p.mask_bs % 4 == 0 && p.mask_hs % 4 == 0;
        const uint8_t* row = p.drop_mask + b * p.mask_bs + h * p.mask_hs + static_cast<int64_t>(qi < p.Tq ? qi : 0) * p.Tk;
#pragma unroll
        for (int jq = 0; jq < 4; ++jq) {
          const uint32_t keep = qi < p.Tq ? keep_bytes4(row, k_tile + jq * 8 + hh * 4, p.Tk, aligned) : 0u;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int j = jq * 4 + e;
            const bool visible = ((word >> (jq * 8 + hh * 4 + e)) & 1u) != 0u;
            const float prob = visible ? __builtin_amdgcn_exp2f(fmaf(sacc[j], c, -lse2)) : 0.f;
            const float dp = ((keep >> (8 * e)) & 0xffu) != 0u ? dpacc[j] * p.drop_scale : 0.f;
            dsb[j / 8][j % 8] = static_cast<T>(prob * fmaf(dp, p.scale, -delta_scaled));
          }
        }
      } else if (MODE != kMaskNone) {
        const bool aligned = (p.Tk % 4 == 0) && (reinterpret_cast<uintptr_t>(p.drop_mask) % 4 == 0) &&
                             p.mask_bs % 4 == 0 && p.mask_hs % 4 == 0;
        const uint8_t* row = p.drop_mask + b * p.mask_bs + h * p.mask_hs + static_cast<int64_t>(qi < p.Tq ? qi : 0) * p.Tk;
        const bool with_valid = MODE == kMaskVisible && p.key_valid != nullptr;  // uniform
        const uint8_t* valid_row = with_valid ? p.key_valid + static_cast<int64_t>(b) * p.Tk : nullptr;
        const bool valid_aligned = with_valid && (p.Tk % 4 == 0) && (reinterpret_cast<uintptr_t>(p.key_valid) % 4 == 0);
#pragma unroll
        for (int jq = 0; jq < 4; ++jq) {
          const uint32_t keep = qi < p.Tq ? keep_bytes4(row, k_tile + jq * 8 + hh * 4, p.Tk, aligned) : 0u;
          const uint32_t kval = with_valid ? keep_bytes4(valid_row, k_tile + jq * 8 + hh * 4, p.Tk, valid_aligned) : ~0u;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int j = jq * 4 + e;
            const bool on = ((keep >> (8 * e)) & 0xffu) != 0u && ((kval >> (8 * e)) & 0xffu) != 0u;
            float prob = __builtin_amdgcn_exp2f(fmaf(sacc[j], c, -lse2));
            if (DROPOUT) {
              const float dp = on ? dpacc[j] * p.drop_scale : 0.f;
              dsb[j / 8][j % 8] = static_cast<T>(prob * fmaf(dp, p.scale, -delta_scaled));
            } else {
              prob = on ? prob : 0.f;
              dsb[j / 8][j % 8] = static_cast<T>(prob * fmaf(dpacc[j], p.scale, -delta_scaled));
            }
          }
        }
      } else {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const float prob = __builtin_amdgcn_exp2f(fmaf(sacc[j], c, -lse2));
          dsb[j / 8][j % 8] = static_cast<T>(prob * fmaf(dpacc[j], p.scale, -delta_scaled));
        }
      }
      accumulate_columns<T, DP, kt * 32 * ROWB>(dqacc, dsb, col_addr);
    });
    if (BITS) {
#pragma unroll
      for (int t = 0; t < kChunk / 32; ++t) chunk_words[t] = next_words[t];
    }
  }
  __syncthreads();  // the staging buffers now hold the output tiles
  store_owned<T, DP>(dqacc, smem + wave * (32 * OROW), dqb, p.dqs[2], q_begin + wave * 32, p.Tq, p.d, lane);
}

template <typename T, int DP, bool DMA, int MODE = kMaskNone>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu((DP == 32 ? 4 : 3) - (DMA ? 0 : 1)))) void attn_bwd_dkv_kernel(const AttnBwdParams p) {
  constexpr bool DROPOUT = MODE == kMaskDropout || MODE == kMaskBitsDropout;
  constexpr bool BITS = MODE == kMaskBits || MODE == kMaskBitsDropout;
  typedef typename Vec8<T>::type vec_t;
  constexpr int KSTEPS = DP / 16, MB = DP / 32;
  constexpr int ROWB = DP * 2, TILE_BYTES = kChunk * ROWB;
  // a chunk of Q, of dO, then its row statistics; bit mode: then the mask words of the chunk's rows for the 32 keys of
  // each wavefront, [wavefront][row]
  constexpr int kWaves = kThreads / kWave;
  static_assert(kThreads == kWaves * kChunk, "one mask word per thread and chunk");
  constexpr int BUF_BYTES = 2 * TILE_BYTES + 2 * kChunk * 4 + (BITS ? kWaves * kChunk * 4 : 0);
  constexpr int NBUF = DMA ? 2 : 1;
  constexpr int OROW = DP * 2 + 16;
  constexpr int OUT_BYTES = (kThreads / kWave) * 32 * OROW;
  __shared__ __attribute__((aligned(1024))) uint8_t smem[NBUF * BUF_BYTES > OUT_BYTES ? NBUF * BUF_BYTES : OUT_BYTES];

  const uint32_t logical = xcd_remap(blockIdx.x, p.total);
  const int blk = static_cast<int>(logical % p.nblk);
  const int bh = static_cast<int>(logical / p.nblk);
  const int h = bh % p.H, b = bh / p.H;
  const int tid = threadIdx.x, wave = tid / kWave, lane = tid % kWave, l32 = lane % 32, hh = lane / 32;
  const T* qb = static_cast<const T*>(p.q) + b * p.qs[0] + h * p.qs[1];
  const T* kb = static_cast<const T*>(p.k) + b * p.ks[0] + h * p.ks[1];
  const T* vb = static_cast<const T*>(p.v) + b * p.vs[0] + h * p.vs[1];
  const T* dob = static_cast<const T*>(p.dout) + b * p.dos[0] + h * p.dos[1];
  T* dkb = static_cast<T*>(p.dk) + b * p.dks[0] + h * p.dks[1];
  T* dvb = static_cast<T*>(p.dv) + b * p.dvs[0] + h * p.dvs[1];

  int len = p.Tk;
  if (p.key_lengths != nullptr) {
    len = p.key_lengths[b];
    len = len < 0 ? 0 : (len > p.Tk ? p.Tk : len);
  }
  const int q_valid = p.zero_pad ? (len < p.Tq ? len : p.Tq) : p.Tq;
  const int k_begin = blk * kOwn;
  const int kj = k_begin + wave * 32 + l32;
  // visibility mode: whether the lane's key can be seen at all (its own byte of the key validity, if one was given)
  // bit mode: column (kj / 32) of the sample's word matrix; (k_begin + wave * 32) is a multiple of 32, so the wavefront's
  // keys share the word and key kj is bit l32
  [[maybe_unused]] const int bit_wpr = (p.Tk + 31) / 32;
  [[maybe_unused]] bool key_seen = kj < p.Tk;
  if (MODE == kMaskVisible && key_seen && p.key_valid != nullptr) key_seen = p.key_valid[static_cast<int64_t>(b) * p.Tk + kj] != 0;
  if (BITS && key_seen && p.key_valid != nullptr)
    key_seen = ((reinterpret_cast<const uint32_t*>(p.key_valid)[static_cast<int64_t>(b) * ((p.Tk + 31) / 32) + kj / 32] >> (kj % 32)) & 1u) != 0u;
  const bool k_ok = kj < len;
  // queries that can see a key of this block: all valid ones, or (causal) those at or after the block's first key
  const int q_start = p.causal ? (k_begin / kChunk) * kChunk : 0;

  vec_t kf[KSTEPS], vf[KSTEPS];
  load_owned<T, DP>(kb, p.ks[2], kj, k_ok, p.d, hh, kf);
  load_owned<T, DP>(vb, p.vs[2], kj, k_ok, p.d, hh, vf);
  f32x16 dkacc[MB], dvacc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int j = 0; j < 16; ++j) dkacc[mb][j] = dvacc[mb][j] = 0.f;
  const float c = p.scale * 1.4426950408889634f;
  const int64_t stat0 = (static_cast<int64_t>(b) * p.H + h) * p.Tq;

  if (k_begin < len) {  // workgroup-uniform: a block of padding keys gets zero gradients without any work
    Streamed<T, DP, DMA> q_rows, do_rows;
    q_rows.init(qb, p.qs[2], tid);
    do_rows.init(dob, p.dos[2], tid);
    float lse_next = -INFINITY, delta_next = 0.f;
    [[maybe_unused]] uint32_t word_next = 0u;
    auto fetch = [&](int qc0, int buffer) {
      q_rows.fetch(qc0, q_valid, p.d, smem + buffer * BUF_BYTES, tid);
      do_rows.fetch(qc0, q_valid, p.d, smem + buffer * BUF_BYTES + TILE_BYTES, tid);
      if (tid < kChunk) {
        const int qi = qc0 + tid;
        lse_next = qi < q_valid ? p.lse[stat0 + qi] : -INFINITY;
        delta_next = qi < q_valid ? p.delta[stat0 + qi] : 0.f;
      }
      if (BITS) {  // thread (w, r): the word of query row qc0 + r that covers the keys of wavefront w
        const int qi = qc0 + tid % kChunk, key0 = k_begin + (tid / kChunk) * 32;
        word_next = (qi < q_valid && key0 < p.Tk) ? p.bit_words[b * p.bits_bs + static_cast<int64_t>(qi) * bit_wpr + key0 / 32] : 0u;
      }
    };
    // the row statistics travel through registers: base-2 log-sum-exp (+inf: the row carries nothing, exp2(x - inf) = 0)
    // and D_i / sqrt(d)
    auto commit_stats = [&](int buffer) {
      if (tid < kChunk) {
        float* stats = reinterpret_cast<float*>(smem + buffer * BUF_BYTES + 2 * TILE_BYTES);
        stats[tid] = lse_next > -INFINITY ? lse_next * 1.4426950408889634f : INFINITY;
        stats[kChunk + tid] = delta_next * p.scale;
      }
      if (BITS)
        reinterpret_cast<uint32_t*>(smem + buffer * BUF_BYTES + 2 * TILE_BYTES + 2 * kChunk * 4)[tid] = word_next;
    };
    const uint32_t row_off = streamed_row_offset<DP>(l32, hh);
    const uint32_t col_off = streamed_column_offset<DP>(lane);
    if (q_start < q_valid) {
      fetch(q_start, 0);
      if (DMA) commit_stats(0);
    }
    int buf = 0;
    for (int qc0 = q_start; qc0 < q_valid; qc0 += kChunk) {
      const bool more = qc0 + kChunk < q_valid;
      if (DMA) {
        vm_wait<0>();     // this wavefront's pieces of the chunk have landed ...
        __syncthreads();  // ... everyone's have (and the statistics), and everyone is done reading the other buffer
        if (more) fetch(qc0 + kChunk, buf ^ 1);
      } else {
        if (qc0 > q_start) __syncthreads();  // every wavefront is done reading the previous chunk
        q_rows.commit(smem, tid);
        do_rows.commit(smem + TILE_BYTES, tid);
        commit_stats(0);
        __syncthreads();
        if (more) fetch(qc0 + kChunk, 0);
      }
      const uint8_t* q_tile = smem + buf * BUF_BYTES;
      const float* sLse = reinterpret_cast<const float*>(q_tile + 2 * TILE_BYTES);
      const float* sDelta = sLse + kChunk;
      [[maybe_unused]] const uint32_t* sWords = reinterpret_cast<const uint32_t*>(sDelta + kChunk) + wave * kChunk;
      const uint32_t q_col_addr = lds_offset(q_tile) + col_off;
      if (DMA) buf ^= 1;
      static_for<kChunk / 32>([&](auto qt_tag) {
        constexpr int qt = decltype(qt_tag)::value;
        if (qc0 + qt * 32 >= q_valid || k_begin + wave * 32 >= len) return;  // wavefront-uniform
        if (p.causal && qc0 + qt * 32 + 31 < k_begin + wave * 32) return;     // every query of the tile lies before the keys
        f32x16 sacc, dpacc;
#pragma unroll
        for (int j = 0; j < 16; ++j) sacc[j] = dpacc[j] = 0.f;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
          const uint32_t off = qt * 32 * ROWB + (row_off ^ (s * 32));
          const vec_t qa = *reinterpret_cast<const vec_t*>(q_tile + off);
          const vec_t da = *reinterpret_cast<const vec_t*>(q_tile + TILE_BYTES + off);
          sacc = Mfma32<T>::run(qa, kf[s], sacc);
          dpacc = Mfma32<T>::run(da, vf[s], dpacc);
        }
        // (causal) a query before the key: the score becomes -inf, the probability 0; only a tile that crosses the
        // causal diagonal needs per-element tests. A padded key of the lane (zeros in kf and vf) collects finite
        // values in its own accumulator column only, which is cleared after the loop.
        const bool diagonal = p.causal && qc0 + qt * 32 < k_begin + wave * 32 + 31;
        if (diagonal) {  // wavefront-uniform: the other tiles pay nothing for the triangle
#pragma unroll
          for (int j = 0; j < 16; ++j)
            if (kj > qc0 + qt * 32 + (j / 4) * 8 + hh * 4 + (j % 4)) sacc[j] = -INFINITY;
        }
        vec_t pb[2], dsb[2];
#pragma unroll
        for (int jq = 0; jq < 4; ++jq) {
          const int r0 = qt * 32 + jq * 8 + hh * 4;  // four consecutive queries of the chunk
          const f32x4 l4 = *reinterpret_cast<const f32x4*>(&sLse[r0]);
          const f32x4 d4 = *reinterpret_cast<const f32x4*>(&sDelta[r0]);  // already times 1 / sqrt(d)
          [[maybe_unused]] u32x4 w4 = {0u, 0u, 0u, 0u};
          if (BITS) w4 = *reinterpret_cast<const u32x4*>(&sWords[r0]);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int j = jq * 4 + e;
            float prob = __builtin_amdgcn_exp2f(fmaf(sacc[j], c, -l4[e]));
            if (MODE == kMaskBits) {
              // the lane owns key kj; register j is query qc0 + r0 + e: bit l32 of that row's word for the wavefront's keys
              prob = (key_seen && ((w4[e] >> l32) & 1u) != 0u) ? prob : 0.f;
              pb[j / 8][j % 8] = static_cast<T>(prob);
              dsb[j / 8][j % 8] = static_cast<T>(prob * fmaf(dpacc[j], p.scale, -d4[e]));
            } else if (MODE == kMaskBitsDropout) {
              const int qrow = qc0 + r0 + e;
              prob = (key_seen && ((w4[e] >> l32) & 1u) != 0u) ? prob : 0.f;
              const bool keep = qrow < p.Tq && kj < p.Tk &&
                                p.drop_mask[b * p.mask_bs + h * p.mask_hs + static_cast<int64_t>(qrow) * p.Tk + kj] != 0;
              pb[j / 8][j % 8] = static_cast<T>(keep ? prob * p.drop_scale : 0.f);
              dsb[j / 8][j % 8] = static_cast<T>(prob * fmaf(keep ? dpacc[j] * p.drop_scale : 0.f, p.scale, -d4[e]));
            } else if (MODE != kMaskNone) {
              // the lane owns key kj; register j is query qc0 + r0 + e: one mask byte per register
              const int qrow = qc0 + r0 + e;
              const bool keep = qrow < p.Tq && key_seen &&
                                p.drop_mask[b * p.mask_bs + h * p.mask_hs + static_cast<int64_t>(qrow) * p.Tk + kj] != 0;
              if (DROPOUT) {
                pb[j / 8][j % 8] = static_cast<T>(keep ? prob * p.drop_scale : 0.f);
                dsb[j / 8][j % 8] = static_cast<T>(prob * fmaf(keep ? dpacc[j] * p.drop_scale : 0.f, p.scale, -d4[e]));
              } else {
                prob = keep ? prob : 0.f;
                pb[j / 8][j % 8] = static_cast<T>(prob);
                dsb[j / 8][j % 8] = static_cast<T>(prob * fmaf(dpacc[j], p.scale, -d4[e]));
              }
            } else {
              pb[j / 8][j % 8] = static_cast<T>(prob);
              dsb[j / 8][j % 8] = static_cast<T>(prob * fmaf(dpacc[j], p.scale, -d4[e]));
            }
          }
        }
        accumulate_columns2<T, DP, qt * 32 * ROWB>(dvacc, pb, q_col_addr + TILE_BYTES, dkacc, dsb, q_col_addr);
      });
      if (DMA && more) commit_stats(buf);  // the next chunk's statistics: the barrier above publishes them
    }
  }
  if (!k_ok) {  // a key in the padding receives no gradient
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int j = 0; j < 16; ++j) dkacc[mb][j] = dvacc[mb][j] = 0.f;
  }
  __syncthreads();
  uint8_t* tile = smem + wave * (32 * OROW);
  store_owned<T, DP>(dkacc, tile, dkb, p.dks[2], k_begin + wave * 32, p.Tk, p.d, lane);
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  store_owned<T, DP>(dvacc, tile, dvb, p.dvs[2], k_begin + wave * 32, p.Tk, p.d, lane);
}

bool strides_ok(const int64_t* st) {
  if (!st || st[3] != 1) return false;
  for (int i = 0; i < 3; ++i)
    if (st[i] % 8 != 0 || st[i] < 0) return false;
  return true;
}

// 32-bit source offsets with a 24-bit row multiply: row strides below 4 M elements, sequences below 2^31 bytes.
bool small_offsets(int64_t rows, int64_t stride) {
  return stride < (1 << 22) && rows < (1 << 22) && rows * stride * 2 < (1ll << 31);
}

template <typename T, int DP, int MODE>
void launch_bwd_mode(AttnBwdParams p, bool register_staging, hipStream_t s) {
  // TAAC_ATTN_REGISTER_STAGING keeps the register-staged kernels for full head dims too (comparison route of the caller).
  const bool direct = p.d == DP && !register_staging;
  p.nblk = static_cast<uint32_t>((p.Tq + kOwn - 1) / kOwn);
  p.total = p.nblk * p.B * p.H;
  if (direct && small_offsets(p.Tk, p.ks[2]) && small_offsets(p.Tk, p.vs[2]))
    hipLaunchKernelGGL((attn_bwd_dq_kernel<T, DP, true, MODE>), dim3(p.total), dim3(kThreads), 0, s, p);
  else
    hipLaunchKernelGGL((attn_bwd_dq_kernel<T, DP, false, MODE>), dim3(p.total), dim3(kThreads), 0, s, p);
  p.nblk = static_cast<uint32_t>((p.Tk + kOwn - 1) / kOwn);
  p.total = p.nblk * p.B * p.H;
  if (direct && small_offsets(p.Tq, p.qs[2]) && small_offsets(p.Tq, p.dos[2]))
    hipLaunchKernelGGL((attn_bwd_dkv_kernel<T, DP, true, MODE>), dim3(p.total), dim3(kThreads), 0, s, p);
  else
    hipLaunchKernelGGL((attn_bwd_dkv_kernel<T, DP, false, MODE>), dim3(p.total), dim3(kThreads), 0, s, p);
}

template <typename T, int DP>
void launch_bwd_dp(const AttnBwdParams& p, int mode, bool register_staging, hipStream_t s) {
  if (mode == kMaskDropout)
    launch_bwd_mode<T, DP, kMaskDropout>(p, register_staging, s);
  else if (mode == kMaskVisible)
    launch_bwd_mode<T, DP, kMaskVisible>(p, register_staging, s);
  else if (mode == kMaskBits)
    launch_bwd_mode<T, DP, kMaskBits>(p, register_staging, s);
  else if (mode == kMaskBitsDropout)
    launch_bwd_mode<T, DP, kMaskBitsDropout>(p, register_staging, s);
  else
    launch_bwd_mode<T, DP, kMaskNone>(p, register_staging, s);
}

template <typename T>
void launch_bwd(const AttnBwdParams& p, int mode, bool register_staging, hipStream_t s) {
  if (p.d <= 32)
    launch_bwd_dp<T, 32>(p, mode, register_staging, s);
  else
    launch_bwd_dp<T, 64>(p, mode, register_staging, s);
}

}  // namespace
}  // namespace taac

namespace taac {
namespace {
int attention_bwd_entry(const char* name, const void* q, const void* k, const void* v, const void* o, const void* dout,
                        const float* lse, const int32_t* key_lengths, const uint8_t* drop_mask, float drop_scale, void* dq,
                        void* dk, void* dv, float* delta, int32_t B, int32_t H, int32_t Tq, int32_t Tk, int32_t d,
                        const int64_t q_strides[4], const int64_t k_strides[4], const int64_t v_strides[4],
                        const int64_t o_strides[4], const int64_t do_strides[4], const int64_t dq_strides[4],
                        const int64_t dk_strides[4], const int64_t dv_strides[4], int is_causal, int zero_padded_queries,
                        int dtype, void* stream, int mask_mode = -1, int64_t mask_bs = 0, int64_t mask_hs = 0,
                        const uint8_t* key_valid = nullptr, const uint32_t* bit_words = nullptr, int64_t bits_bs = 0) {
  // mask_mode -1: dropout when a mask is given (its matrices follow the (B, H) order), nothing otherwise
  if (mask_mode < 0 || mask_mode == kMaskBitsDropout) {
    if (mask_mode < 0) mask_mode = drop_mask != nullptr ? kMaskDropout : kMaskNone;
    mask_hs = static_cast<int64_t>(Tq) * Tk;
    mask_bs = mask_hs * H;
  }
  if (mask_bs < 0 || mask_hs < 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: negative mask stride", name);
  if (drop_mask != nullptr && !(drop_scale >= 1.f))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: dropout_scale = 1 / (1 - p) must be >= 1", name);
  if (B < 0 || H < 0 || Tq < 0 || Tk < 0 || d <= 0)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: negative dimension or non-positive head_dim", name);
  if (is_causal & ~(TAAC_ATTN_CAUSAL | TAAC_ATTN_REGISTER_STAGING))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: unknown bits in is_causal (%d)", name, is_causal);
  const bool register_staging = (is_causal & TAAC_ATTN_REGISTER_STAGING) != 0;
  if (dtype != TAAC_BF16 && dtype != TAAC_F16)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: dtype must be bf16 or fp16 (got %d)", name, dtype);
  if (d % 8 != 0 || d > 64)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: head_dim %d unsupported (multiple of 8, at most 64)", name, d);
  if (B == 0 || H == 0 || (Tq == 0 && Tk == 0)) return TAAC_OK;
  if (Tq == 0 || Tk == 0)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: empty query or key sequences are not supported", name);
  if (!q || !k || !v || !o || !dout || !lse || !dq || !dk || !dv || !delta)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  const int64_t* all[8] = {q_strides, k_strides, v_strides, o_strides, do_strides, dq_strides, dk_strides, dv_strides};
  for (const int64_t* st : all)
    if (!strides_ok(st))
      return set_error(TAAC_ERR_UNSUPPORTED,
                       "%s: strides must be non-negative multiples of 8 elements with a unit last stride", name);
  const void* ptrs[8] = {q, k, v, o, dout, dq, dk, dv};
  for (const void* ptr : ptrs)
    if (!aligned16(ptr)) return set_error(TAAC_ERR_UNSUPPORTED, "%s: tensor base pointers must be 16-byte aligned", name);
  if (zero_padded_queries && Tq != Tk)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: zero_padded_queries requires Tq == Tk", name);
  const int64_t blocks = (static_cast<int64_t>(Tq > Tk ? Tq : Tk) + kOwn - 1) / kOwn * B * H;
  if (blocks > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: too many workgroups", name);
  AttnBwdParams p{};
  p.q = q;
  p.k = k;
  p.v = v;
  p.o = o;
  p.dout = dout;
  p.lse = lse;
  p.delta = delta;
  p.dq = dq;
  p.dk = dk;
  p.dv = dv;
  p.key_lengths = key_lengths;
  p.drop_mask = drop_mask;
  p.mask_bs = mask_bs;
  p.mask_hs = mask_hs;
  p.key_valid = key_valid;
  p.bit_words = bit_words;
  p.bits_bs = bits_bs;
  p.drop_scale = drop_scale;
  p.B = B;
  p.H = H;
  p.Tq = Tq;
  p.Tk = Tk;
  p.d = d;
  for (int i = 0; i < 4; ++i) {
    p.qs[i] = q_strides[i];
    p.ks[i] = k_strides[i];
    p.vs[i] = v_strides[i];
    p.os[i] = o_strides[i];
    p.dos[i] = do_strides[i];
    p.dqs[i] = dq_strides[i];
    p.dks[i] = dk_strides[i];
    p.dvs[i] = dv_strides[i];
  }
  p.scale = 1.0f / sqrtf(static_cast<float>(d));
  p.zero_pad = zero_padded_queries ? 1 : 0;
  p.causal = (is_causal & TAAC_ATTN_CAUSAL) ? 1 : 0;
  hipStream_t s = as_stream(stream);
  if (dtype == TAAC_BF16)
    launch_bwd<bf16_t>(p, mask_mode, register_staging, s);
  else
    launch_bwd<f16_t>(p, mask_mode, register_staging, s);
  return check_launch(name);
}
}  // namespace
}  // namespace taac

extern "C" int taac_flash_attn_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout,
                                   const float* lse, const int32_t* key_lengths, void* dq, void* dk, void* dv,
                                   float* delta, int32_t B, int32_t H, int32_t Tq, int32_t Tk, int32_t d,
                                   const int64_t q_strides[4], const int64_t k_strides[4], const int64_t v_strides[4],
                                   const int64_t o_strides[4], const int64_t do_strides[4], const int64_t dq_strides[4],
                                   const int64_t dk_strides[4], const int64_t dv_strides[4], int is_causal,
                                   int zero_padded_queries, int dtype, void* stream) {
  return taac::attention_bwd_entry("taac_flash_attn_bwd", q, k, v, o, dout, lse, key_lengths, nullptr, 1.f, dq, dk, dv, delta,
                                   B, H, Tq, Tk, d, q_strides, k_strides, v_strides, o_strides, do_strides, dq_strides,
                                   dk_strides, dv_strides, is_causal, zero_padded_queries, dtype, stream);
}

extern "C" int taac_flash_attn_dropout_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout,
                                           const float* lse, const int32_t* key_lengths, const uint8_t* dropout_mask,
                                           float dropout_scale, void* dq, void* dk, void* dv, float* delta, int32_t B,
                                           int32_t H, int32_t Tq, int32_t Tk, int32_t d, const int64_t q_strides[4],
                                           const int64_t k_strides[4], const int64_t v_strides[4],
                                           const int64_t o_strides[4], const int64_t do_strides[4],
                                           const int64_t dq_strides[4], const int64_t dk_strides[4],
                                           const int64_t dv_strides[4], int is_causal, int zero_padded_queries, int dtype,
                                           void* stream) {
  const char* name = "taac_flash_attn_dropout_bwd";
  if (!dropout_mask) return taac::set_error(TAAC_ERR_INVALID_VALUE, "%s: dropout_mask must be given", name);
  return taac::attention_bwd_entry(name, q, k, v, o, dout, lse, key_lengths, dropout_mask, dropout_scale, dq, dk, dv, delta,
                                   B, H, Tq, Tk, d, q_strides, k_strides, v_strides, o_strides, do_strides, dq_strides,
                                   dk_strides, dv_strides, is_causal, zero_padded_queries, dtype, stream);
}

extern "C" int taac_flash_attn_mask_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout,
                                        const float* lse, const int32_t* key_lengths, const uint8_t* visible,
                                        int64_t visible_batch_stride, int64_t visible_head_stride,
                                        const uint8_t* key_valid, void* dq, void* dk,
                                        void* dv, float* delta, int32_t B, int32_t H, int32_t Tq, int32_t Tk, int32_t d,
                                        const int64_t q_strides[4], const int64_t k_strides[4], const int64_t v_strides[4],
                                        const int64_t o_strides[4], const int64_t do_strides[4],
                                        const int64_t dq_strides[4], const int64_t dk_strides[4],
                                        const int64_t dv_strides[4], int zero_padded_queries, int dtype, void* stream) {
  const char* name = "taac_flash_attn_mask_bwd";
  if (!visible) return taac::set_error(TAAC_ERR_INVALID_VALUE, "%s: the visibility mask must be given", name);
  return taac::attention_bwd_entry(name, q, k, v, o, dout, lse, key_lengths, visible, 1.f, dq, dk, dv, delta, B, H, Tq, Tk, d,
                                   q_strides, k_strides, v_strides, o_strides, do_strides, dq_strides, dk_strides,
                                   dv_strides, 0, zero_padded_queries, dtype, stream, taac::kMaskVisible,
                                   visible_batch_stride, visible_head_stride, key_valid);
}

extern "C" int taac_flash_attn_bits_bwd(const void* q, const void* k, const void* v, const void* o, const void* dout,
                                        const float* lse, const int32_t* key_lengths, const uint32_t* struct_bits,
                                        int64_t struct_sample_stride, const uint32_t* valid_bits,
                                        const uint8_t* dropout_mask, float dropout_scale, void* dq, void* dk, void* dv,
                                        float* delta, int32_t B, int32_t H, int32_t Tq, int32_t Tk, int32_t d,
                                        const int64_t q_strides[4], const int64_t k_strides[4], const int64_t v_strides[4],
                                        const int64_t o_strides[4], const int64_t do_strides[4],
                                        const int64_t dq_strides[4], const int64_t dk_strides[4],
                                        const int64_t dv_strides[4], int zero_padded_queries, int dtype, void* stream) {
  const char* name = "taac_flash_attn_bits_bwd";
  if (!struct_bits) return taac::set_error(TAAC_ERR_INVALID_VALUE, "%s: struct_bits must be given", name);
  if (struct_sample_stride < 0) return taac::set_error(TAAC_ERR_INVALID_VALUE, "%s: negative sample stride", name);
  return taac::attention_bwd_entry(name, q, k, v, o, dout, lse, key_lengths, dropout_mask,
                                   dropout_mask != nullptr ? dropout_scale : 1.f, dq, dk, dv, delta, B, H, Tq, Tk, d,
                                   q_strides, k_strides, v_strides, o_strides, do_strides, dq_strides, dk_strides,
                                   dv_strides, 0, zero_padded_queries, dtype, stream,
                                   dropout_mask != nullptr ? taac::kMaskBitsDropout : taac::kMaskBits, 0, 0,
                                   reinterpret_cast<const uint8_t*>(valid_bits), struct_bits, struct_sample_stride);
}
