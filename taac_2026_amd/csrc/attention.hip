// Key-padding-masked attention forward for gfx950.
//
// Work decomposition
//   One workgroup (4 wavefronts) owns 128 query rows of one (batch, head); each wavefront owns 32 of them for the
//   whole kernel, with its Q fragment, running max / sum and output accumulator in registers. Keys and values
//   are streamed through LDS in chunks of 64 keys shared by the four wavefronts. Only key chunks below the
//   sample's valid length are visited; query blocks entirely in the padding are either zero-filled or skipped.
//   Sibling workgroups of the same (batch, head) get adjacent logical ids on the same accelerator die so that their
//   K/V re-reads hit that die's L2.
//
// MFMA formulation (v_mfma_f32_32x32x16, 64-wide wavefront)
//   Scores are computed transposed, S^T[key, query] = K Q^T, so that in the accumulator layout every lane owns ONE
//   query column (lane % 32) and 16 of the tile's 32 keys: the softmax row reductions are in-register plus one
//   exchange with lane ^ 32. The probabilities are then already in the B-operand layout of the second product
//   O^T[d, query] = V^T P^T, so P never leaves registers. V stays row-major in LDS: its fragments (8 keys of one
//   feature per lane) are read column-wise with ds_read_b64_tr_b16, at key offsets that follow the accumulator's key
//   order (4-key runs interleaved between the two lane halves).
//
// Semantics follow the reference's inference kernel (accelerators/attention/kernels/tilelang.py:36-138): base-2
// online softmax with scale log2(e)/sqrt(d), key j visible iff j < key_lengths[b] (and j <= i when causal),
// P rounded to the storage dtype before the second product, rows with an empty visible set produce 0.
#include <math.h>
#include <stdlib.h>

#include <type_traits>

#include "common.h"
#include "ts_common.h"

namespace taac {
namespace {

constexpr int kThreads = 256;
constexpr int kQB = 128;  // query rows per workgroup
constexpr int kKC = 64;   // keys per LDS chunk

struct AttnParams {
  const void* q;
  const void* k;
  const void* v;
  void* o;
  const int32_t* key_lengths;
  const float* q_row_scale;  // [B, Tq] / [B, Tk] factors of the query / key rows (shared by the heads), or null
  const float* k_row_scale;
  const float* q_col_scale;  // [H, d] factors of the query features, or null
  float* amax_out;           // receives max |o| over everything written (atomic max), or null
  const uint8_t* drop_mask;  // training dropout: [B, H, Tq, Tk] keep mask (non-zero = keep), or null
  float drop_scale;          // 1 / (1 - p)
  // Structured mask: key j is visible to query i of sample b iff bit j of struct_bits[i] and of valid_bits[b] is set.
  const uint32_t* struct_bits;  // [Tq][wpr] words, bit j % 32 of word j / 32; null: no structured mask
  int64_t struct_stride;        // words between the matrices of consecutive samples; 0: one matrix for the batch
  const uint32_t* valid_bits;   // [B][wpr] or null (every key valid)
  const uint32_t* self_bits;    // [B][ceil(Tq / 32)] or null: flagged query rows return their own value row
  const uint8_t* block_any;     // [nqc][nkc]: some query of the 128-row block sees some key of the 64-key chunk;
                                // null (per-sample structure only): every chunk is visited
  // Per-tile kernel (compact form of the structure, taac_mask_compact): for every 32-query tile the key columns some
  // query of the tile can see, in ascending order, cut into compact tiles of 32; struct_bits then holds, per query row,
  // one word per compact tile (bit j = the row sees key compact_keys[32 c + j]).
  const int32_t* compact_keys;   // [samples][nqt][32 wpr], -1 beyond the tile's keys
  const uint64_t* compact_tiles; // [samples][nqt][64]: the 32-key words of Tk that hold keys of compact tile c (0: no such tile)
  float* lse;                   // [B, H, Tq] log-sum-exp of the scaled scores (natural log) for the backward, or null
  int32_t wpr;                  // words per row of struct_bits / valid_bits = ceil(Tk / 32)
  int32_t nkc;                  // key chunks = ceil(Tk / 64)
  int32_t B, H, Tq, Tk, d;
  int64_t qs[4], ks[4], vs[4], os[4];
  float scale_log2;  // log2(e) / sqrt(d)
  int32_t zero_pad;
  uint32_t nqc;    // query chunks per (batch, head)
  uint32_t total;  // workgroups
  uint32_t nqc_magic, h_magic;  // floor(2^32 / nqc), floor(2^32 / H) (0 for a divisor of 1): divisions without a divide
  uint32_t nqt_magic;           // the same for the number of 32-query tiles
  // direct-transfer kernel: whether a workgroup takes a pair of query blocks, workgroups per (batch, head), their grid
  int32_t pair_blocks;
  uint32_t nqg, nqg_magic, total_g;
};

// x / d and x % d for a divisor known to the host: q = mulhi(x, floor(2^32 / d)) is at most two short of the quotient.
__device__ __forceinline__ void magic_divmod(uint32_t x, uint32_t d, uint32_t magic, uint32_t& q, uint32_t& r) {
  q = magic == 0u ? x : __umulhi(x, magic);
  r = x - q * d;
#pragma unroll
  for (int i = 0; i < 2; ++i)
    if (r >= d) {
      ++q;
      r -= d;
    }
}
inline uint32_t magic_of(uint32_t d) { return d <= 1u ? 0u : static_cast<uint32_t>((1ull << 32) / d); }

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

// Combine a value with the one held by lane ^ 32 (both lanes of a pair own the same query column).
__device__ __forceinline__ float pair_max(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);  // r[0] = lower half's, r[1] = upper half's
  return fmaxf(__builtin_bit_cast(float, static_cast<uint32_t>(r[0])), __builtin_bit_cast(float, static_cast<uint32_t>(r[1])));
}
__device__ __forceinline__ float pair_sum(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, static_cast<uint32_t>(r[0])) + __builtin_bit_cast(float, static_cast<uint32_t>(r[1]));
}

// acc + the sum of the eight rounded values of a fragment: four two-element dot products with (1, 1).
__device__ __forceinline__ float frag_sum(const bf16x8& v, float acc) {
  typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
  const bf16x2 ones = {static_cast<__bf16>(1.0f), static_cast<__bf16>(1.0f)};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const bf16x2 pair = {v[2 * i], v[2 * i + 1]};
    acc = __builtin_amdgcn_fdot2_f32_bf16(pair, ones, acc, false);
  }
  return acc;
}
__device__ __forceinline__ float frag_sum(const f16x8& v, float acc) {
  typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2;
  const f16x2 ones = {static_cast<_Float16>(1.0f), static_cast<_Float16>(1.0f)};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const f16x2 pair = {v[2 * i], v[2 * i + 1]};
    acc = __builtin_amdgcn_fdot2(pair, ones, acc, false);
  }
  return acc;
}

// Keep bytes of four consecutive keys of one mask row as one word (byte e = key key0 + e); keys at or beyond Tk read as 0.
// `aligned`: Tk is a multiple of 4 and the mask is 4-byte aligned, so a word never straddles rows.
__device__ __forceinline__ uint32_t keep_bytes4(const uint8_t* row, int key0, int Tk, bool aligned) {
  if (aligned && key0 + 3 < Tk) return *reinterpret_cast<const uint32_t*>(row + key0);
  uint32_t w = 0u;
#pragma unroll
  for (int e = 0; e < 4; ++e)
    if (key0 + e < Tk) w |= static_cast<uint32_t>(row[key0 + e]) << (8 * e);
  return w;
}

// The lane's feature factors of the query (q_col_scale, fp32, 16-byte aligned rows): features 16 * s + 0..7 of k-step s,
// counted from `offset`; fetched with two 16-byte loads per k-step, all requested before the first is used. Without
// factors (or in kernels without them) the product is the scale alone.
template <bool SCALED, int KSTEPS>
struct QueryFeatureFactors {
  f32x4 v[SCALED ? KSTEPS : 1][2];
  bool present = false;
  __device__ __forceinline__ void load(const float* q_col_scale, int offset) {
    if constexpr (SCALED) {
      present = q_col_scale != nullptr;  // uniform over the launch
      if (present) {
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
          v[s][0] = *reinterpret_cast<const f32x4*>(q_col_scale + offset + 16 * s);
          v[s][1] = *reinterpret_cast<const f32x4*>(q_col_scale + offset + 16 * s + 4);
        }
      }
    }
  }
  __device__ __forceinline__ float times(int s, int e, float c) const {
    if constexpr (SCALED) {
      if (present) return v[s][e / 4][e % 4] * c;
    }
    return c;
  }
};

template <typename T, int DP, bool CAUSAL, bool SCALED, bool MASKED, bool DROPOUT = false>
__global__ __launch_bounds__(kThreads) void flash_attn_fwd_kernel(const AttnParams p) {
  static_assert(!(DROPOUT && SCALED && !MASKED), "dropout comes with the masks of the training path, not with row factors");
  static_assert(!(MASKED && CAUSAL), "a structured mask carries its own causal triangle");
  typedef typename Vec8<T>::type vec_t;
  typedef typename Vec8<T>::half_type vec4_t;
  constexpr int KSTEPS = DP / 16;  // MFMA k-steps of the score product
  constexpr int MB = DP / 32;      // 32-row blocks of O^T
  constexpr int C8 = DP / 8;       // 128-bit column chunks per row
  constexpr int KSTR = DP + 8;     // K row stride in elements (+16 bytes: 16 lanes reading one piece of 16 rows hit all banks)
  // V stays row-major as well; its fragments are read column-wise with ds_read_b64_tr_b16, where 32 lanes touch 64
  // contiguous bytes of four consecutive rows: a row stride of 16 or 48 dwords (mod 64) spreads those over all banks.
  constexpr int VSTR = DP == 32 ? DP : DP + 32;
  constexpr int OROW = DP * 2 + 16;                 // bytes per row of a wavefront's output tile
  constexpr int KV_BYTES = (kKC * KSTR + kKC * VSTR) * 2;
  constexpr int OT_BYTES = (kThreads / kWave) * 32 * OROW;
  __shared__ __attribute__((aligned(16))) uint8_t smem[KV_BYTES > OT_BYTES ? KV_BYTES : OT_BYTES];
  T* sK = reinterpret_cast<T*>(smem);               // [kKC][KSTR]
  T* sV = sK + kKC * KSTR;                          // [kKC][VSTR]

  const uint32_t logical = xcd_remap(blockIdx.x, p.total);
  const int qc = static_cast<int>(logical % p.nqc);
  const int bh = static_cast<int>(logical / p.nqc);
  const int h = bh % p.H;
  const int b = bh / p.H;

  const int tid = threadIdx.x;
  const int wave = tid / kWave;
  const int lane = tid % kWave;
  const int l32 = lane % 32;
  const int hh = lane / 32;

  const T* qb = static_cast<const T*>(p.q) + b * p.qs[0] + h * p.qs[1];
  const T* kb = static_cast<const T*>(p.k) + b * p.ks[0] + h * p.ks[1];
  const T* vb = static_cast<const T*>(p.v) + b * p.vs[0] + h * p.vs[1];
  T* ob = static_cast<T*>(p.o) + b * p.os[0] + h * p.os[1];

  int len = p.Tk;
  if (p.key_lengths != nullptr) {
    len = p.key_lengths[b];
    len = len < 0 ? 0 : (len > p.Tk ? p.Tk : len);
  }
  const int q_begin = qc * kQB;
  const int q_valid = p.zero_pad ? (len < p.Tq ? len : p.Tq) : p.Tq;  // rows at or beyond are written as zeros

  vec_t zero_vec;
#pragma unroll
  for (int e = 0; e < 8; ++e) zero_vec[e] = static_cast<T>(0.f);

  if (q_begin >= q_valid) {
    // Whole block lies in the padding: zero-fill its rows, or leave them alone.
    if (p.lse != nullptr) {
      for (int idx = tid; idx < kQB; idx += kThreads)
        if (q_begin + idx < p.Tq) p.lse[(static_cast<int64_t>(b) * p.H + h) * p.Tq + q_begin + idx] = -INFINITY;
    }
    if (p.zero_pad == 2) return;
    const int c8n = p.d / 8;
    for (int idx = tid; idx < kQB * c8n; idx += kThreads) {
      const int row = q_begin + idx / c8n;
      const int c8 = idx % c8n;
      if (row < p.Tq) *reinterpret_cast<vec_t*>(ob + row * p.os[2] + c8 * 8) = zero_vec;
    }
    return;
  }

  int kv_end = len;
  if (CAUSAL) kv_end = kv_end < q_begin + kQB ? kv_end : q_begin + kQB;

  // Q fragments: B operand of S^T = K Q^T; lane holds query row l32, features 16*s + 8*hh .. +7.
  const int qi = q_begin + wave * 32 + l32;
  vec_t qf[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    const int col = 16 * s + 8 * hh;
    // Query rows in the padding are not read (they may be uninitialised memory): a zero query keeps the arithmetic finite.
    qf[s] = (qi < q_valid && col < p.d) ? *reinterpret_cast<const vec_t*>(qb + qi * p.qs[2] + col) : zero_vec;
    if (SCALED && p.q_col_scale != nullptr && col < p.d) {
      const float* cf = p.q_col_scale + h * p.d + col;
#pragma unroll
      for (int e = 0; e < 8; ++e) qf[s][e] = static_cast<T>(static_cast<float>(qf[s][e]) * cf[e]);
    }
  }

  f32x16 oacc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int j = 0; j < 16; ++j) oacc[mb][j] = 0.f;
  float m_run = -INFINITY;
  float l_run = 0.f;
  // Row factors: the query's multiplies every score of its column, so it joins the softmax scale of the lane (it is
  // positive, the running max keeps its meaning); the key's is applied to the key row on its way into LDS.
  float c = p.scale_log2;
  if (SCALED && p.q_row_scale != nullptr && qi < q_valid) c *= p.q_row_scale[static_cast<int64_t>(b) * p.Tq + qi];

  int wave_kv_end = kv_end;
  if (CAUSAL) {
    const int wlim = q_begin + wave * 32 + 32;
    wave_kv_end = wave_kv_end < wlim ? wave_kv_end : wlim;
  }
  // A wavefront whose 32 query rows all lie in the padding (or beyond Tq) only helps staging; its output is zeros.
  if (q_begin + wave * 32 >= q_valid) wave_kv_end = 0;

  // K / V staging is split into a register fetch and an LDS commit so that the global loads of chunk c + 1 are in
  // flight while chunk c is being consumed. Piece idx of a chunk, of K and of V: (key idx / C8, 8 features idx % C8).
  constexpr int KLD = (kKC * C8 + kThreads - 1) / kThreads;
  vec_t kreg[KLD], vreg[KLD];
  float kfac[SCALED ? KLD : 1];
  const bool scale_keys = SCALED && p.k_row_scale != nullptr;
  // MASKED: the two 32-key words of the lane's query for the chunk being fetched / being consumed (structure only),
  // and the sample's key-validity words of the same keys (all ones without valid_bits).
  uint32_t mw_next[2] = {0u, 0u}, mw[2] = {0u, 0u};
  uint32_t vw_next[2] = {~0u, ~0u}, vw[2] = {~0u, ~0u};
  // Key validity enters the scores through the matrix unit instead of per-element selects: one more k-step per tile
  // whose key operand is -BIG at k = 0 for an invalid key (0 for a valid one) and whose query operand is the inverse of
  // the query's row factor at k = 0 (1 without one), so that after the lane's scale the score of an invalid key is about
  // -BIG * log2(e) / sqrt(d) (BIG = 2^30, 2^15 for fp16), whatever the factor, and its probability underflows to exactly 0, while valid keys get
  // 0 added, exactly. Tiles whose structure is all ones then stay on the fast path however the padding is scattered.
  // (A query with no valid key at all still ends at 0: the value rows of invalid keys are staged as zeros.)
  vec_t qbias;
  if (MASKED) {
    const float factor = c / p.scale_log2;  // the query's row factor, 1 without one
    const T inv = static_cast<T>(1.0f / factor);
    u32x4 bits = {hh == 0 ? static_cast<uint32_t>(__builtin_bit_cast(uint16_t, inv)) : 0u, 0u, 0u, 0u};
    qbias = __builtin_bit_cast(vec_t, bits);
  }
  constexpr uint32_t kNegBigBits = std::is_same<T, bf16_t>::value ? 0xCE80u : 0xF800u;  // -2^30 (bf16) / -32768 (fp16)
  // MASKED with per-sample key validity: a key outside it reaches LDS as zeros whatever its rows hold - they may be
  // uninitialised memory (a caller that skips the padded positions never writes them), and a masked probability of
  // zero times a NaN would still poison the output. The rows are loaded like any other and cleared on their way into
  // LDS (commit), against the chunk's two validity words, so that the loads do not wait for those words.
  auto key_is_valid = [&](int key_in_chunk) -> bool {
    if (!MASKED) return true;
    return ((vw_next[key_in_chunk / 32] >> (key_in_chunk % 32)) & 1u) != 0u;
  };
  auto fetch = [&](int kc0) {
    if (MASKED) {
      const int w0 = kc0 / 32;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        uint32_t bits = 0u;
        if (qi < q_valid && w0 + kt < p.wpr) {  // a query row in the padding sees nothing (and has no row of bits)
          bits = p.struct_bits[b * p.struct_stride + static_cast<int64_t>(qi) * p.wpr + w0 + kt];
        }
        mw_next[kt] = bits;
        vw_next[kt] = (p.valid_bits != nullptr && w0 + kt < p.wpr) ? p.valid_bits[static_cast<int64_t>(b) * p.wpr + w0 + kt] : ~0u;
      }
    }
#pragma unroll
    for (int i = 0; i < KLD; ++i) {
      const int idx = tid + i * kThreads;
      const int kidx = kc0 + idx / C8;
      const int c8 = idx % C8;
      const bool ok = idx < kKC * C8 && kidx < kv_end && c8 * 8 < p.d;
      kreg[i] = ok ? *reinterpret_cast<const vec_t*>(kb + kidx * p.ks[2] + c8 * 8) : zero_vec;
      vreg[i] = ok ? *reinterpret_cast<const vec_t*>(vb + kidx * p.vs[2] + c8 * 8) : zero_vec;
      if (SCALED) kfac[SCALED ? i : 0] = (ok && scale_keys) ? p.k_row_scale[static_cast<int64_t>(b) * p.Tk + kidx] : 1.0f;
    }
  };
  auto commit = [&]() {
#pragma unroll
    for (int i = 0; i < KLD; ++i) {
      const int idx = tid + i * kThreads;
      if (SCALED && scale_keys) {
#pragma unroll
        for (int e = 0; e < 8; ++e) kreg[i][e] = static_cast<T>(static_cast<float>(kreg[i][e]) * kfac[SCALED ? i : 0]);
      }
      if (idx < kKC * C8) {
        const bool valid = key_is_valid(idx / C8);
        *reinterpret_cast<vec_t*>(&sK[(idx / C8) * KSTR + (idx % C8) * 8]) = valid ? kreg[i] : zero_vec;
        *reinterpret_cast<vec_t*>(&sV[(idx / C8) * VSTR + (idx % C8) * 8]) = valid ? vreg[i] : zero_vec;
      }
    }
  };
  // Address of the lane's transposed reads of V (see lds_read_tr16): lane r of 16-lane group g points at key
  // 4 * hh + r / 4 of an 8-key group, features 16 (g % 2) + 4 (r % 4) .. + 3 of a 32-feature row block. With the read at
  // key offset 16 s2 (+ 8) of a tile, lane (l32, hh) receives the keys 16 s2 (+ 8) + 4 hh + 0..3 of feature l32: the
  // key order of the probabilities in its accumulator registers 8 s2 .. 8 s2 + 7.
  const uint32_t v_addr = lds_offset(sV) + static_cast<uint32_t>((4 * hh + (lane % 16) / 4) * (VSTR * 2) +
                                                                  (16 * ((lane / 16) % 2) + 4 * (lane % 4)) * 2);

  // Chunks are walked in order; with a structured mask the chunks in which no query of this workgroup's block sees
  // any key (block_any, shared by the batch) are skipped altogether: not staged, not synchronised on.
  // The block's row of block_any is read once, as one bit per chunk (at most 64 chunks: Tk <= 4096 with a mask).
  uint64_t chunk_bits = ~0ull;
  if (MASKED && p.block_any != nullptr)
    chunk_bits = __builtin_amdgcn_ballot_w64(lane < p.nkc && p.block_any[qc * p.nkc + (lane < p.nkc ? lane : 0)] != 0);
  auto next_chunk = [&](int kc) -> int {
    if (MASKED) {
      const uint64_t rest = kc < 64 ? chunk_bits >> kc : 0ull;
      if (rest == 0ull) return -1;
      kc += __builtin_ctzll(rest);
    }
    return kc * kKC < kv_end ? kc : -1;
  };
  int kc = next_chunk(0);
  if (kc >= 0) fetch(kc * kKC);
  bool first_chunk = true;
  while (kc >= 0) {
    const int kc0 = kc * kKC;
    if (!first_chunk) __syncthreads();  // every wavefront is done reading the previous chunk
    first_chunk = false;
    commit();
    if (MASKED) {
      mw[0] = mw_next[0];
      mw[1] = mw_next[1];
      vw[0] = vw_next[0];
      vw[1] = vw_next[1];
    }
    __syncthreads();
    kc = next_chunk(kc + 1);
    if (kc >= 0) fetch(kc * kKC);

    // One softmax update per chunk: both 32-key tiles when the second one has a visible key for this wavefront
    // (NT = 2), one tile alone otherwise (NT = 1, tile T0). Per update: scores S^T (NT tiles of 32 keys x 32 queries),
    // running max / sum of one query per lane pair, P rounded to the storage type, one rescale of O^T, O^T += V^T P^T.
    if (kc0 >= wave_kv_end) continue;  // wavefront-uniform: nothing visible in this chunk (padding / causal bound)
    auto update = [&](auto nt_tag, auto t0_tag) {
      constexpr int NT = decltype(nt_tag)::value;
      constexpr int T0 = decltype(t0_tag)::value;  // first 32-key tile of the chunk taken by this update
      f32x16 sacc[NT];
#pragma unroll
      for (int kt = 0; kt < NT; ++kt) {
#pragma unroll
        for (int j = 0; j < 16; ++j) sacc[kt][j] = 0.f;
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
          const vec_t a = *reinterpret_cast<const vec_t*>(&sK[((T0 + kt) * 32 + l32) * KSTR + 16 * s + 8 * hh]);
          sacc[kt] = Mfma32<T>::run(a, qf[s], sacc[kt]);
        }
        if (MASKED) {  // + (invalid key ? -BIG : 0) / (row factor of the query); the lane's key is key l32 of the tile
          const uint32_t word = __builtin_amdgcn_readfirstlane(vw[T0 + kt]);  // the same for every lane: one sample
          if (word != ~0u) {
            const bool invalid = ((word >> l32) & 1u) == 0u;
            const u32x4 kbits = {(hh == 0 && invalid) ? kNegBigBits : 0u, 0u, 0u, 0u};
            sacc[kt] = Mfma32<T>::run(__builtin_bit_cast(vec_t, kbits), qbias, sacc[kt]);
          }
        }
      }
      const int k_last = kc0 + (T0 + NT) * 32;  // one past the last key of this update
      const bool tail = (k_last > kv_end) || (CAUSAL && (k_last - 1 > q_begin + wave * 32));
      if (tail) {
#pragma unroll
        for (int kt = 0; kt < NT; ++kt)
#pragma unroll
          for (int j = 0; j < 16; ++j) {
            const int key = kc0 + (T0 + kt) * 32 + (j / 4) * 8 + hh * 4 + (j % 4);
            const bool masked = key >= kv_end || (CAUSAL && key > qi);
            if (masked) sacc[kt][j] = -INFINITY;
          }
      }
      if (MASKED) {
        // Accumulator register j of the lane is key (j / 4) * 8 + hh * 4 + j % 4 of the tile: bit of the lane's word.
        bool all_visible = true;
#pragma unroll
        for (int kt = 0; kt < NT; ++kt) all_visible = all_visible && mw[T0 + kt] == 0xffffffffu;
        if (__builtin_amdgcn_ballot_w64(!all_visible) != 0) {  // wavefront-uniform
#pragma unroll
          for (int kt = 0; kt < NT; ++kt) {
            const uint32_t bits = mw[T0 + kt] >> (hh * 4);
#pragma unroll
            for (int j = 0; j < 16; ++j)
              if (((bits >> ((j / 4) * 8 + (j % 4))) & 1u) == 0u) sacc[kt][j] = -INFINITY;
          }
        }
      }
      // ---- online softmax, one query per lane (pair of lanes l, l ^ 32) ------------------------------------
      float mx = sacc[0][0];
#pragma unroll
      for (int kt = 0; kt < NT; ++kt)
#pragma unroll
        for (int j = 0; j < 16; ++j) mx = fmaxf(mx, sacc[kt][j]);
      mx = pair_max(mx);
      const float m_new = fmaxf(m_run, mx);
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * c);
      const float mc = -m_use * c;
      float rs = 0.f;
      vec_t pb[NT][2];
#pragma unroll
      for (int kt = 0; kt < NT; ++kt) {
        float pr[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) pr[j] = __builtin_amdgcn_exp2f(fmaf(sacc[kt][j], c, mc));
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          pb[kt][0][e] = static_cast<T>(pr[e]);
          pb[kt][1][e] = static_cast<T>(pr[8 + e]);
        }
        if (DROPOUT) {
          // Training dropout with the caller's keep mask (tilelang.py:224-247 of the reference kernel): the normaliser
          // sums the probabilities before the mask, the second product takes keep ? P / (1 - p) : 0.
          const bool aligned = (p.Tk % 4 == 0) && (reinterpret_cast<uintptr_t>(p.drop_mask) % 4 == 0);
          const uint8_t* row = p.drop_mask + ((static_cast<int64_t>(b) * p.H + h) * p.Tq + (qi < p.Tq ? qi : 0)) * p.Tk;
#pragma unroll
          for (int jq = 0; jq < 4; ++jq) {
            const uint32_t keep = qi < p.Tq ? keep_bytes4(row, kc0 + (T0 + kt) * 32 + jq * 8 + hh * 4, p.Tk, aligned) : 0u;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              rs += pr[jq * 4 + e];
              pr[jq * 4 + e] = ((keep >> (8 * e)) & 0xffu) != 0u ? pr[jq * 4 + e] * p.drop_scale : 0.f;
            }
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            pb[kt][0][e] = static_cast<T>(pr[e]);
            pb[kt][1][e] = static_cast<T>(pr[8 + e]);
          }
        } else {
          // the normaliser sums the rounded probabilities, the values the second product uses: two per instruction
          rs = frag_sum(pb[kt][0], rs);
          rs = frag_sum(pb[kt][1], rs);
        }
      }
      rs = pair_sum(rs);
      l_run = l_run * alpha + rs;
      m_run = m_new;
      // ---- O^T += V^T P^T --------------------------------------------------------------------------------
      // The rescale is unconditional on purpose: a wavefront-uniform branch around it placed the accumulator read-back
      // of the preceding MFMA on a path without the required wait states (wrong values in the last accumulator register).
      static_for<MB>([&](auto mb_tag) {
        constexpr int mb = decltype(mb_tag)::value;
#pragma unroll
        for (int j = 0; j < 16; ++j) oacc[mb][j] *= alpha;
        static_for<NT>([&](auto kt_tag) {
          constexpr int kt = decltype(kt_tag)::value;
          constexpr int key0 = (T0 + kt) * 32;
          u32x2 vt[2][2];
          lds_read_tr16<key0 * VSTR * 2 + mb * 64>(vt[0][0], v_addr);
          lds_read_tr16<(key0 + 8) * VSTR * 2 + mb * 64>(vt[0][1], v_addr);
          lds_read_tr16<(key0 + 16) * VSTR * 2 + mb * 64>(vt[1][0], v_addr);
          lds_read_tr16<(key0 + 24) * VSTR * 2 + mb * 64>(vt[1][1], v_addr);
          // the transposed reads were issued by hand: wait for them by hand (everything of this wavefront's LDS queue);
          // the fragments are tied to the wait so that their consumers cannot be scheduled above it
          asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(vt[0][0]), "+v"(vt[0][1]), "+v"(vt[1][0]), "+v"(vt[1][1]) : : "memory");
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) {
            const u32x4 bits = {vt[s2][0][0], vt[s2][0][1], vt[s2][1][0], vt[s2][1][1]};
            oacc[mb] = Mfma32<T>::run(__builtin_bit_cast(vec_t, bits), pb[kt][s2], oacc[mb]);
          }
        });
      });
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, 1> I1;
    typedef std::integral_constant<int, 2> I2;
    if (MASKED) {
      // tiles in which no query of this wavefront sees a key are not computed
      const bool any0 = __builtin_amdgcn_ballot_w64((mw[0] & vw[0]) != 0u) != 0;
      const bool any1 = __builtin_amdgcn_ballot_w64((mw[1] & vw[1]) != 0u) != 0 && kc0 + 32 < wave_kv_end;
      if (any0 && any1)
        update(I2{}, I0{});
      else if (any0)
        update(I1{}, I0{});
      else if (any1)
        update(I1{}, I1{});
    } else if (kc0 + 32 < wave_kv_end) {
      update(I2{}, I0{});
    } else {
      update(I1{}, I0{});
    }
  }

  // ---- finalise: O / l (0 for rows in the padding), transpose through a wavefront-private LDS tile, 16-byte stores --
  const float inv = l_run > 0.f ? __builtin_amdgcn_rcpf(l_run) : 0.f;  // 1 ulp; the products are rounded to 16 bits
  const float fin = (qi < q_valid) ? inv : 0.f;
  if (p.lse != nullptr && hh == 0 && qi < p.Tq)
    p.lse[(static_cast<int64_t>(b) * p.H + h) * p.Tq + qi] =
        (qi < q_valid && l_run > 0.f) ? (m_run * c + __builtin_amdgcn_logf(l_run)) * 0.6931471805599453f : -INFINITY;
  __syncthreads();  // every wavefront is done with sK / sV: the buffer now holds the output tiles
  uint8_t* tile = smem + wave * (32 * OROW);
  float omax = 0.f;
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
    for (int jq = 0; jq < 4; ++jq) {
      vec4_t ov;
#pragma unroll
      for (int e = 0; e < 4; ++e) ov[e] = static_cast<T>(oacc[mb][jq * 4 + e] * fin);
      *reinterpret_cast<vec4_t*>(tile + l32 * OROW + (mb * 32 + jq * 8 + hh * 4) * 2) = ov;
      if (p.amax_out != nullptr) {
#pragma unroll
        for (int e = 0; e < 4; ++e) omax = fmaxf(omax, fabsf(static_cast<float>(ov[e])));
      }
    }
  }
  if (p.amax_out != nullptr) {
    // per-tensor scale of the layer that consumes the output (FP8 dense layers): one atomic per wavefront on the float's
    // bit pattern, skipped when the published value already covers it
    omax = group_max<kWave>(omax);
    if (lane == 0 && omax > __builtin_nontemporal_load(p.amax_out))
      atomicMax(reinterpret_cast<unsigned int*>(p.amax_out), __float_as_uint(omax));
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  constexpr int RPP = kWave / C8;  // rows per pass: C8 lanes cover one row
  const int c8 = lane % C8;
#pragma unroll
  for (int pass = 0; pass < 32 / RPP; ++pass) {
    const int row = pass * RPP + lane / C8;
    const int q_row = q_begin + wave * 32 + row;
    vec_t v = *reinterpret_cast<const vec_t*>(tile + row * OROW + c8 * 16);
    if (MASKED && p.self_bits != nullptr && q_row < p.Tq && c8 * 8 < p.d) {
      // a flagged query attends to itself only: its output is its own value row
      const uint32_t word = p.self_bits[static_cast<int64_t>(b) * ((p.Tq + 31) / 32) + q_row / 32];
      if ((word >> (q_row % 32)) & 1u) v = *reinterpret_cast<const vec_t*>(vb + q_row * p.vs[2] + c8 * 8);
    }
    const int q_store_end = p.zero_pad == 2 ? q_valid : p.Tq;  // mode 2: rows in the padding are left untouched
    if (q_row < q_store_end && c8 * 8 < p.d) *reinterpret_cast<vec_t*>(ob + q_row * p.os[2] + c8 * 8) = v;
  }
}

// ------------------------------------------------------------------------------------------------------------------
// The plain case at head dims 32 and 64 (key-length / causal masking only, no row factors, no structured mask): K and V
// chunks go from global memory straight into LDS (one 1 KB transfer per wavefront and operand, no staging registers,
// no transposition arithmetic), into two buffers, so that chunk c + 1 is in flight while chunk c is consumed and one
// barrier per chunk is enough.
//   K: row-major [64 keys][32 features]; a transfer cannot pad rows, so the four 16-byte pieces of row r are stored
//      at piece ^ ((r / 4) % 4): the 16 lanes that read the same piece of 16 consecutive rows hit 64 distinct banks.
//   V: row-major as well. The A operand of O^T += V^T P^T needs, per lane, 8 keys of ONE feature: it is read with
//      ds_read_b64_tr_b16, which hands element e of lane j of a 16-lane group element j % 4 of the 8-byte row supplied
//      by lane 4 * e + j / 4 of that group. With lane 4 * e + q pointing at V[k0 + e][f0 + 4 * q ..] lane j receives
//      V[k0 .. k0 + 3][f0 + j]: four keys of its feature; two such reads make a fragment, in the key order of P.
// Rows at or beyond the valid length are never requested: the transfer repeats the last valid row (finite values; the
// scores of those keys are masked), since uninitialised memory could hold NaNs that a zero probability would not cancel.
// ------------------------------------------------------------------------------------------------------------------
// MASKED: per-sample structure bits on top (struct_bits with a sample stride, every listed key valid, no chunk map): the
// form in which samples with their valid tokens moved to the front arrive. The lane's two words of a chunk are fetched
// with the chunk's transfers; tiles that are fully visible to the wavefront skip the bit tests.
template <typename T, int DP, bool CAUSAL, bool SCALED, bool MASKED>
__global__ __launch_bounds__(kThreads) void flash_attn_fwd_dma_kernel(const AttnParams p) {
  static_assert(!(MASKED && CAUSAL), "a structured mask carries its own causal triangle");
  typedef typename Vec8<T>::type vec_t;
  typedef typename Vec8<T>::half_type vec4_t;
  static_assert(DP == 32 || DP == 64, "row swizzles are written for 64- and 128-byte rows");
  constexpr int KSTEPS = DP / 16;
  constexpr int MB = DP / 32;
  constexpr int C8 = DP / 8;
  constexpr int ROWB = DP * 2;                      // bytes per staged row
  constexpr int TILE_BYTES = kKC * ROWB;            // one operand of one chunk
  constexpr int BUF_BYTES = 2 * TILE_BYTES;         // K then V
  constexpr int PPT = kKC * C8 / kThreads;          // 16-byte pieces per lane, operand and chunk
  constexpr int OROW = DP * 2 + 16;
  constexpr int OT_BYTES = (kThreads / kWave) * 32 * OROW;
  static_assert(kKC * C8 % kThreads == 0, "whole transfers per wavefront");
  // Head dim 32: three chunk buffers, chunk c is consumed while c + 1 and c + 2 are in flight. Head dim 64: two (a chunk is
  // 16 KB: with three a compute unit holds three workgroups, with two it holds as many as the registers allow), chunk c + 1
  // is requested once every wavefront has left chunk c - 1.
  constexpr int NBUF = DP == 64 ? 2 : 3;
  __shared__ __attribute__((aligned(1024))) uint8_t smem[NBUF * BUF_BYTES > OT_BYTES ? NBUF * BUF_BYTES : OT_BYTES];

  // A workgroup takes two query blocks of one (sample, head), g and nqc - 1 - g (one, for the middle block of an odd
  // count): under key lengths the first is the one more likely to hold valid queries, so few workgroups find nothing to
  // do (a workgroup that only learns from the sample's length that it is idle has held its registers and LDS for two
  // memory latencies), and under a causal mask the pair's work is the same for every g.
  const uint32_t logical = xcd_remap(blockIdx.x, p.total_g);
  uint32_t bh_u, qg_u, b_u, h_u;
  magic_divmod(logical, p.nqg, p.nqg_magic, bh_u, qg_u);
  magic_divmod(bh_u, static_cast<uint32_t>(p.H), p.h_magic, b_u, h_u);
  const int h = static_cast<int>(h_u), b = static_cast<int>(b_u);
  const int qc_a = static_cast<int>(qg_u);
  const int qc_b = p.pair_blocks ? static_cast<int>(p.nqc) - 1 - qc_a : qc_a;

  const T* qb = static_cast<const T*>(p.q) + b * p.qs[0] + h * p.qs[1];
  const T* kb = static_cast<const T*>(p.k) + b * p.ks[0] + h * p.ks[1];
  const T* vb = static_cast<const T*>(p.v) + b * p.vs[0] + h * p.vs[1];
  T* ob = static_cast<T*>(p.o) + b * p.os[0] + h * p.os[1];

  int len = p.Tk;
  if (p.key_lengths != nullptr) {
    len = p.key_lengths[b];
    len = len < 0 ? 0 : (len > p.Tk ? p.Tk : len);
  }
  const int q_valid = p.zero_pad ? (len < p.Tq ? len : p.Tq) : p.Tq;
  // One query block. The body is instantiated once per block of the pair (no loop around it: a loop's preheader
  // collects constants and lane offsets in registers for the whole kernel), and everything a block derives from the lane
  // index is derived from an opaque copy of it, so that the second instance shares no vector register with the first
  // (the kernel lives on its 96 registers: five wavefronts per SIMD).
  auto block = [&](const int qc, auto second_tag) __attribute__((always_inline)) {
  uint32_t opaque_tid = threadIdx.x;
  if constexpr (decltype(second_tag)::value) asm volatile("" : "+v"(opaque_tid));
  const int tid = static_cast<int>(opaque_tid & (kThreads - 1));
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int lane = tid % kWave;
  const int l32 = lane % 32;
  const int hh = lane / 32;
  const int q_begin = qc * kQB;
  vec_t zero_vec;
#pragma unroll
  for (int e = 0; e < 8; ++e) zero_vec[e] = static_cast<T>(0.f);
  if (q_begin >= q_valid) {  // whole block in the padding: zero-fill its rows, or leave them alone
    if (p.lse != nullptr) {
      for (int idx = tid; idx < kQB; idx += kThreads)
        if (q_begin + idx < p.Tq) p.lse[(static_cast<int64_t>(b) * p.H + h) * p.Tq + q_begin + idx] = -INFINITY;
    }
    if (p.zero_pad == 2) return;  // the blocks behind this one lie in the padding as well
    for (int idx = tid; idx < kQB * C8; idx += kThreads) {
      const int row = q_begin + idx / C8;
      if (row < p.Tq) *reinterpret_cast<vec_t*>(ob + row * p.os[2] + (idx % C8) * 8) = zero_vec;
    }
    return;
  }
  int kv_end = len;
  if (CAUSAL) kv_end = kv_end < q_begin + kQB ? kv_end : q_begin + kQB;

  const int qi = q_begin + wave * 32 + l32;
  // The query enters the products already multiplied by the softmax scale (and log2 e), rounded once more to the storage
  // type: the score tiles then come out of the matrix unit in the exponent's units. SCALED: the query's row factor joins
  // the lane's softmax scale, the feature factors multiply it per feature. Every load is requested before the first
  // value is used (one memory latency for the row factor, the query rows and the feature factors together).
  float q_row_factor = 1.0f;
  if (SCALED && p.q_row_scale != nullptr && qi < q_valid) q_row_factor = p.q_row_scale[static_cast<int64_t>(b) * p.Tq + qi];
  // A lane whose query lies in the padding reads the block's first row instead (valid here: the block holds a valid query):
  // finite values whose results are never used (the lane's output factor is zero and its row is not stored) - and a load
  // without a branch around it, so that its wait can sink below the requests for the first K / V chunks.
  const int q_row_read = qi < q_valid ? qi : q_begin;
  // (rows of q and of the output are addressed like the K / V sources: a 24-bit multiply into a 32-bit byte offset)
  const uint8_t* q_row_ptr = reinterpret_cast<const uint8_t*>(qb) +
                             (__umul24(static_cast<uint32_t>(q_row_read), static_cast<uint32_t>(p.qs[2]) * 2u) + 16u * hh);
  vec_t qf[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) qf[s] = *reinterpret_cast<const vec_t*>(q_row_ptr + 32 * s);
  QueryFeatureFactors<SCALED, KSTEPS> feature_factors;
  feature_factors.load(p.q_col_scale, h * p.d + 8 * hh);
  const float c = (SCALED && p.q_row_scale != nullptr) ? p.scale_log2 * q_row_factor : p.scale_log2;
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
    for (int e = 0; e < 8; ++e) qf[s][e] = static_cast<T>(static_cast<float>(qf[s][e]) * feature_factors.times(s, e, c));

  f32x16 oacc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int j = 0; j < 16; ++j) oacc[mb][j] = 0.f;
  // Softmax with a lazily moved reference: the exponent's offset -m is the C operand of the first score product (sixteen
  // equal registers), so a tile arrives as s - m and goes straight into exp2; m is moved (and the accumulators rescaled)
  // only when a score exceeds it by more than kLazyBits, which keeps every probability below 2^kLazyBits - exact in the
  // float32 accumulators and neutral for the relative rounding of the 16-bit probabilities. Each lane sums the rounded
  // probabilities of its own keys; the two lanes of a query are added once, at the end.
  constexpr float kLazyBits = 8.f;
  f32x16 negm;
#pragma unroll
  for (int j = 0; j < 16; ++j) negm[j] = 0.f;
  float l_lane = 0.f;
  bool m_set = false;                 // the query has seen a visible key (its reference is meaningful)
  float thr = -3.0e38f;               // the lane's tile maximum above this moves the reference: any finite score at first
  int wave_kv_end = kv_end;
  if (CAUSAL) {
    const int wlim = q_begin + wave * 32 + 32;
    wave_kv_end = wave_kv_end < wlim ? wave_kv_end : wlim;
  }
  if (q_begin + wave * 32 >= q_valid) wave_kv_end = 0;

  // Row swizzles (a transfer cannot pad rows): the 16-byte piece `piece` of row r is stored at piece ^ swizzle(r).
  //   K: (r / 4) % 4 for 64-byte rows, (r / 2) % 8 for 128-byte rows: the 16 lanes that read the same piece of 16
  //      consecutive rows hit 64 distinct banks.
  //   V: none for 64-byte rows; 4 * ((r / 2) % 2) for 128-byte rows, which keeps the four rows a 16-lane group of a
  //      transposed read touches (and the neighbouring group's) on distinct banks.
  auto k_swizzle = [](int r) -> int { return DP == 32 ? (r / 4) % 4 : (r / 2) % 8; };
  auto v_swizzle = [](int r) -> int { return DP == 32 ? 0 : 4 * ((r / 2) % 2); };
  // The lane's pieces of a chunk: slot i * 256 + 64 * wave + lane = (row, stored piece), i < PPT; rows of successive i
  // are 256 / C8 apart, which leaves the swizzles unchanged. Sources are addressed as a wavefront-uniform base + a
  // 32-bit per-lane byte offset (the host checks that the offsets fit): row * stride with a 24-bit multiply + the piece.
  const int slot = wave * kWave + lane;
  const int srow = slot / C8;
  const uint32_t k_piece_off = static_cast<uint32_t>(((slot % C8) ^ k_swizzle(srow)) * 16);
  const uint32_t v_piece_off = static_cast<uint32_t>(((slot % C8) ^ v_swizzle(srow)) * 16);
  const uint32_t k_row_bytes = static_cast<uint32_t>(p.ks[2]) * 2u, v_row_bytes = static_cast<uint32_t>(p.vs[2]) * 2u;
  // SCALED with a key factor: the K rows are multiplied by it on their way into LDS, so they go through registers (into
  // the same swizzled slots) while V still takes the direct route.
  const bool scale_keys = SCALED && p.k_row_scale != nullptr;
  vec_t kreg[SCALED ? PPT : 1];
  float kfac[SCALED ? PPT : 1];
  // mask words of the two chunks in flight (even / odd chunk) and of the chunk being consumed
  uint32_t mw_even[2] = {0u, 0u}, mw_odd[2] = {0u, 0u}, mw[2] = {0u, 0u};
  auto issue = [&](int chunk, int buffer) {
    if (MASKED) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        const int w = chunk * 2 + kt;
        const uint32_t word = (qi < q_valid && w < p.wpr)
                                  ? p.struct_bits[b * p.struct_stride + static_cast<int64_t>(qi) * p.wpr + w] : 0u;
        if (chunk & 1)
          mw_odd[kt] = word;
        else
          mw_even[kt] = word;
      }
    }
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      int row = chunk * kKC + srow + i * (kThreads / C8);
      row = row < kv_end ? row : kv_end - 1;  // kv_end >= 1 here
      uint8_t* dst = smem + buffer * BUF_BYTES + i * (kThreads * 16) + wave * (kWave * 16);
      if (scale_keys) {
        kreg[SCALED ? i : 0] = *reinterpret_cast<const vec_t*>(reinterpret_cast<const uint8_t*>(kb) +
                                                              __umul24(static_cast<uint32_t>(row), k_row_bytes) + k_piece_off);
        kfac[SCALED ? i : 0] = p.k_row_scale[static_cast<int64_t>(b) * p.Tk + row];
      } else {
        lds_dma16_offset(kb, __umul24(static_cast<uint32_t>(row), k_row_bytes) + k_piece_off, dst);
      }
      lds_dma16_offset(vb, __umul24(static_cast<uint32_t>(row), v_row_bytes) + v_piece_off, dst + TILE_BYTES);
    }
  };
  // The K pieces fetched by issue() for `buffer`, scaled and stored at this lane's slots.
  auto commit_keys = [&](int buffer) {
    if (!scale_keys) return;
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      vec_t v = kreg[SCALED ? i : 0];
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = static_cast<T>(static_cast<float>(v[e]) * kfac[SCALED ? i : 0]);
      *reinterpret_cast<vec_t*>(smem + buffer * BUF_BYTES + i * (kThreads * 16) + wave * (kWave * 16) + lane * 16) = v;
    }
  };
  // Per-lane LDS offsets of the fragment reads (relative to the chunk buffer).
  const uint32_t smem_off = lds_offset(smem);
  //   K fragment (tile, k-step s): row tile * 32 + l32 (tile * 32 leaves the swizzle alone), piece (2 * s + hh) ^ swizzle:
  //   the offset of k-step s is that of k-step 0 with s * 32 XORed in
  const uint32_t k_off0 = static_cast<uint32_t>(l32 * ROWB + ((hh ^ k_swizzle(l32)) * 16));
  //   V transposed read: group g = lane / 16 covers features 16 * (g % 2) .. + 15 (of row block mb) and keys
  //   4 * (g / 2) .. + 3 of a 16-key group; lane r = lane % 16 of the group points at key r / 4, features
  //   4 * (r % 4) .. + 3 = half of piece 2 * (g % 2) + (r % 4) / 2 (+ 4 * mb: XORs 64 * mb into the address)
  const int v_key = 4 * (lane / 32) + (lane % 16) / 4;
  const uint32_t v_off = static_cast<uint32_t>(
      TILE_BYTES + v_key * ROWB + ((2 * ((lane / 16) % 2) + (lane % 4) / 2) ^ v_swizzle(v_key)) * 16 + (lane % 2) * 8);

  // Operands of the key-length tail product (see step): the lower half-wavefront holds the k = 0..7 slots of a fragment.
  constexpr uint32_t kMaskedKeyPair = std::is_same<T, bf16_t>::value ? 0xce80ce80u : 0xf800f800u;  // 2 x -2^30 / 2 x -32768
  constexpr uint32_t kOnePair = std::is_same<T, bf16_t>::value ? 0x3f803f80u : 0x3c003c00u;

  const int nchunks = (kv_end + kKC - 1) / kKC;
  if (nchunks > 0) {
    issue(0, 0);
    commit_keys(0);
  }
  if (nchunks > 1) {
    issue(1, 1);
    commit_keys(1);
  }
  int buf = 0;
  // transfers (and mask words) of one chunk per wavefront: what may stay in flight while the chunk before it is awaited.
  // With key factors the keys pass through registers and are waited for when they are committed: wait for everything.
  constexpr int kInFlight = 2 * PPT + (MASKED ? 2 : 0);
  // One chunk: wait for its transfers, publish them, start the next chunk's, then (NT > 0) take the chunk's first NT key
  // tiles into the running softmax. NT is a compile-time property of the call site: a wavefront sees whole chunks first,
  // then at most one chunk of which only the first tile holds visible keys, then chunks that only the other wavefronts of
  // the workgroup still need - three straight-line loops instead of one loop whose paths merge the accumulators.
  auto step = [&](int chunk, auto nt_tag) {
    constexpr int NT = decltype(nt_tag)::value;
    // this wavefront's pieces of the chunk have landed (the next chunk's, issued after them, may still be in flight) ...
    // (two buffers: only chunk 1, requested with chunk 0 in front of the loop, can be in flight behind the awaited one)
    if (chunk + 1 < nchunks && !scale_keys && (NBUF == 3 || chunk == 0))
      vm_wait<kInFlight>();
    else
      vm_wait<0>();
    __syncthreads();  // ... everyone's have, and everyone is done reading the buffer of the chunk before
    if (MASKED) {
      mw[0] = (chunk & 1) ? mw_odd[0] : mw_even[0];
      mw[1] = (chunk & 1) ? mw_odd[1] : mw_even[1];
    }
    // the chunk requested now: two ahead into the buffer (buf + 2) % 3, or the next one into the buffer left last
    const bool more = NBUF == 3 ? chunk + 2 < nchunks : (chunk >= 1 && chunk + 1 < nchunks);
    const int ahead = NBUF == 3 ? (buf == 0 ? 2 : buf - 1) : 1 - buf;
    if (more) issue(NBUF == 3 ? chunk + 2 : chunk + 1, ahead);
    const int kc0 = chunk * kKC;
    const uint32_t base = smem_off + buf * BUF_BYTES;
    buf = buf == NBUF - 1 ? 0 : buf + 1;
    if constexpr (NT > 0) {
      f32x16 sacc[NT];
#pragma unroll
      for (int kt = 0; kt < NT; ++kt) {
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s) {
          const vec_t a = *reinterpret_cast<const vec_t*>(smem + (base - smem_off) + kt * 32 * ROWB + (k_off0 ^ (s * 32)));
          sacc[kt] = Mfma32<T>::run(a, qf[s], s == 0 ? negm : sacc[kt]);
        }
      }
      const int k_last = kc0 + NT * 32;
      if (!CAUSAL && k_last > kv_end) {
        // Keys at or beyond the valid length (their staged rows repeat the last valid one): one more product per tile adds
        // 8 * kMaskedKey to every score of such a key - A holds kMaskedKey in the k = 0..7 slots of the key's row, B ones in
        // the same slots of every query - so the masked scores leave the matrix unit at about -2^33 (16-bit floats: -2^18)
        // and their probabilities are exact zeros. Two vector instructions per tile instead of two per score register.
        // (the operands are formed here, from the thread index, so that nothing of them is live across the chunk loop)
        // (the two constants sit in scalar registers: as vector-register literals they would be hoisted out of the loop)
        uint32_t t = static_cast<uint32_t>(tid);
        asm volatile("" : "+v"(t));
        uint32_t masked_pair = kMaskedKeyPair, one_pair = kOnePair;
        asm volatile("" : "+s"(masked_pair), "+s"(one_pair));
        const bool lower = (t & 32u) == 0u;
        const uint32_t one = lower ? one_pair : 0u;
        const u32x4 b_bits = {one, one, one, one};
        const int key0 = kc0 + static_cast<int>(t & 31u);
#pragma unroll
        for (int kt = 0; kt < NT; ++kt) {
          if (kc0 + kt * 32 + 32 > kv_end) {  // wavefront-uniform
            const uint32_t bits = (lower && key0 + kt * 32 >= kv_end) ? masked_pair : 0u;
            const u32x4 a_bits = {bits, bits, bits, bits};
            sacc[kt] = Mfma32<T>::run(__builtin_bit_cast(vec_t, a_bits), __builtin_bit_cast(vec_t, b_bits), sacc[kt]);
          }
        }
      }
      const bool tail = CAUSAL && ((k_last > kv_end) || (k_last - 1 > q_begin + wave * 32));
      if (tail) {
        // register j of tile kt is key kc0 + hh * 4 + (kt * 32 + (j / 4) * 8 + j % 4): one lane-dependent limit, then a
        // compare against a constant per register
        int lim = kv_end - kc0 - hh * 4;
        if (CAUSAL) lim = min(lim, qi + 1 - kc0 - hh * 4);
#pragma unroll
        for (int kt = 0; kt < NT; ++kt)
#pragma unroll
          for (int j = 0; j < 16; ++j)
            sacc[kt][j] = (kt * 32 + (j / 4) * 8 + (j % 4)) < lim ? sacc[kt][j] : -INFINITY;
      }
      if (MASKED) {
        // Accumulator register j of the lane is key (j / 4) * 8 + hh * 4 + j % 4 of the tile: bit of the lane's word.
        bool all_visible = true;
#pragma unroll
        for (int kt = 0; kt < NT; ++kt) all_visible = all_visible && mw[kt] == 0xffffffffu;
        if (__builtin_amdgcn_ballot_w64(!all_visible) != 0) {  // wavefront-uniform
#pragma unroll
          for (int kt = 0; kt < NT; ++kt) {
            const uint32_t bits = mw[kt] >> (hh * 4);
#pragma unroll
            for (int j = 0; j < 16; ++j)
              if (((bits >> ((j / 4) * 8 + (j % 4))) & 1u) == 0u) sacc[kt][j] = -INFINITY;
          }
        }
      }
      float mx = sacc[0][0];
#pragma unroll
      for (int kt = 0; kt < NT; ++kt)
#pragma unroll
        for (int j = 0; j < 16; ++j) mx = fmaxf(mx, sacc[kt][j]);
      if (__builtin_amdgcn_ballot_w64(mx > thr) != 0) {  // wavefront-uniform, rare after a query's first tile
        // Both lanes of a query decide on the pair's maximum, so they keep one reference between them.
        const float mxp = pair_max(mx);
        const bool move = mxp > thr;
        const float shift = move ? mxp : 0.f;
#pragma unroll
        for (int kt = 0; kt < NT; ++kt)
#pragma unroll
          for (int j = 0; j < 16; ++j) sacc[kt][j] -= shift;
#pragma unroll
        for (int j = 0; j < 16; ++j) negm[j] -= shift;
        // what a query has accumulated is rescaled only if some query of the wavefront has accumulated anything: not at
        // a query block's first visible tile, which is where the reference almost always moves
        if (__builtin_amdgcn_ballot_w64(move && m_set) != 0) {
          const float alpha = (move && m_set) ? __builtin_amdgcn_exp2f(-mxp) : 1.f;
          l_lane *= alpha;
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int j = 0; j < 16; ++j) oacc[mb][j] *= alpha;
        }
        if (move) {
          m_set = true;
          thr = kLazyBits;
        }
      }
      vec_t pb[NT][2];
#pragma unroll
      for (int kt = 0; kt < NT; ++kt) {
        float pr[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) pr[j] = __builtin_amdgcn_exp2f(sacc[kt][j]);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          pb[kt][0][e] = static_cast<T>(pr[e]);
          pb[kt][1][e] = static_cast<T>(pr[8 + e]);
        }
        l_lane = frag_sum(pb[kt][0], l_lane);
        l_lane = frag_sum(pb[kt][1], l_lane);
      }
      // V fragments of one row block at a time: requested once the scores are dead (registers), in flight during the
      // bookkeeping below
      const uint32_t v_addr = base + v_off;
      static_for<MB>([&](auto mc_tag) {
        constexpr int mb = decltype(mc_tag)::value;
        const uint32_t v_addr_mb = v_addr ^ (mb * 64);
        u32x2 vt[NT][2][2];
        static_for<NT * 2>([&](auto ic) {
          constexpr int kt = decltype(ic)::value / 2, s2 = decltype(ic)::value % 2;
          lds_read_tr16<(kt * 32 + s2 * 16) * ROWB>(vt[kt][s2][0], v_addr_mb);
          lds_read_tr16<(kt * 32 + s2 * 16 + 8) * ROWB>(vt[kt][s2][1], v_addr_mb);
        });
        // the transposed reads were issued by hand: wait for them by hand (everything of this wavefront's LDS queue);
        // the fragments are tied to the wait so that their consumers cannot be scheduled above it
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(vt[0][0][0]) : : "memory");
#pragma unroll
        for (int kt = 0; kt < NT; ++kt)
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) {
            asm volatile("" : "+v"(vt[kt][s2][0]));
            asm volatile("" : "+v"(vt[kt][s2][1]));
          }
#pragma unroll
        for (int kt = 0; kt < NT; ++kt)
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) {
            const u32x4 bits = {vt[kt][s2][0][0], vt[kt][s2][0][1], vt[kt][s2][1][0], vt[kt][s2][1][1]};
            oacc[mb] = Mfma32<T>::run(__builtin_bit_cast(vec_t, bits), pb[kt][s2], oacc[mb]);
          }
      });
    }
    if (more) commit_keys(ahead);  // that chunk's K, fetched before the update: the next barrier publishes it
  };
  // chunks of which both tiles hold keys visible to this wavefront: 64 * chunk + 32 < wave_kv_end
  const int whole = wave_kv_end >= 33 ? (wave_kv_end - 33) / kKC + 1 : 0;
  int chunk = 0;
  for (; chunk < whole; ++chunk) step(chunk, std::integral_constant<int, 2>{});
  if (chunk < nchunks && chunk * kKC < wave_kv_end) {
    step(chunk, std::integral_constant<int, 1>{});
    ++chunk;
  }
  for (; chunk < nchunks; ++chunk) step(chunk, std::integral_constant<int, 0>{});

  const float l_run = pair_sum(l_lane);
  const float inv = l_run > 0.f ? __builtin_amdgcn_rcpf(l_run) : 0.f;  // 1 ulp; the products are rounded to 16 bits
  const float fin = (qi < q_valid) ? inv : 0.f;
  if (p.lse != nullptr && hh == 0 && qi < p.Tq)
    p.lse[(static_cast<int64_t>(b) * p.H + h) * p.Tq + qi] =
        (qi < q_valid && l_run > 0.f) ? (__builtin_amdgcn_logf(l_run) - negm[0]) * 0.6931471805599453f : -INFINITY;
  __syncthreads();  // every wavefront is done with the chunk buffers: they now hold the output tiles
  uint8_t* tile = smem + wave * (32 * OROW);
  float omax = 0.f;
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
    for (int jq = 0; jq < 4; ++jq) {
      vec4_t ov;
#pragma unroll
      for (int e = 0; e < 4; ++e) ov[e] = static_cast<T>(oacc[mb][jq * 4 + e] * fin);
      *reinterpret_cast<vec4_t*>(tile + l32 * OROW + (mb * 32 + jq * 8 + hh * 4) * 2) = ov;
      if (p.amax_out != nullptr) {
#pragma unroll
        for (int e = 0; e < 4; ++e) omax = fmaxf(omax, fabsf(static_cast<float>(ov[e])));
      }
    }
  }
  if (p.amax_out != nullptr) {
    // per-tensor scale of the layer that consumes the output (FP8 dense layers): one atomic per wavefront on the float's
    // bit pattern, skipped when the published value already covers it
    omax = group_max<kWave>(omax);
    if (lane == 0 && omax > __builtin_nontemporal_load(p.amax_out))
      atomicMax(reinterpret_cast<unsigned int*>(p.amax_out), __float_as_uint(omax));
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  constexpr int RPP = kWave / C8;
  const int c8 = lane % C8;
  const int q_store_end = p.zero_pad == 2 ? q_valid : p.Tq;
#pragma unroll
  for (int pass = 0; pass < 32 / RPP; ++pass) {
    const int row = pass * RPP + lane / C8;
    const int q_row = q_begin + wave * 32 + row;
    const vec_t v = *reinterpret_cast<const vec_t*>(tile + row * OROW + c8 * 16);
    if (q_row < q_store_end)
      *reinterpret_cast<vec_t*>(reinterpret_cast<uint8_t*>(ob) +
                                (__umul24(static_cast<uint32_t>(q_row), static_cast<uint32_t>(p.os[2]) * 2u) + c8 * 16u)) = v;
  }
  };
  block(qc_a, std::false_type{});
  if (qc_b != qc_a) {
    __syncthreads();  // the second block's first chunks land in the buffers the output tiles were read from
    block(qc_b, std::true_type{});
  }
}


// ------------------------------------------------------------------------------------------------------------------
// Structured masks whose visible part is a small fraction of the score matrix (sliding windows plus a few always-visible
// columns and rows): one wavefront per 32-query tile, on its own - no workgroup, no barrier, no shared chunk list.
//   * The lane's row of structure bits (ANDed with the sample's key validity and the valid length) is read once, 16
//     words at a time; a ballot per word gives the 32-key tiles in which some query of the wavefront sees some key, and
//     only those tiles are visited. Query rows in the padding and self-only rows contribute nothing to that set.
//   * K fragments (the A operand of S^T = K Q^T: key l32, 8 features) come straight from global memory - a tile's rows
//     are read completely by the 64 lanes - and the V tile's pieces are requested one tile ahead of their use. V passes
//     through a wavefront-private LDS tile (row-major, rows of 128 bytes swizzled like the chunked kernel's) and is read
//     column-wise with transposed LDS reads. Rows of invalid keys may be uninitialised memory: their scores are replaced
//     by selects, their V rows stored as zeros.
// Same arithmetic per tile as the general kernel taken one tile at a time.
// ------------------------------------------------------------------------------------------------------------------
constexpr int kSparseWaves = 4;  // independent wavefronts per workgroup: the same query tile of consecutive (batch, head)s

template <typename T, int DP, bool SCALED>
__global__ __launch_bounds__(kSparseWaves * kWave) void flash_attn_fwd_sparse_kernel(const AttnParams p) {
  typedef typename Vec8<T>::type vec_t;
  typedef typename Vec8<T>::half_type vec4_t;
  static_assert(DP == 32 || DP == 64, "row swizzles are written for 64- and 128-byte rows");
  constexpr int KSTEPS = DP / 16;
  constexpr int MB = DP / 32;
  constexpr int C8 = DP / 8;
  constexpr int ROWB = DP * 2;
  constexpr int VT_BYTES = 32 * ROWB;       // the V tile
  constexpr int PPT = 32 * C8 / kWave;      // 16-byte pieces per lane and tile
  constexpr int OROW = DP * 2 + 16;
  constexpr int OT_BYTES = 32 * OROW;
  constexpr int WAVE_LDS = ((VT_BYTES > OT_BYTES ? VT_BYTES : OT_BYTES) + 1023) / 1024 * 1024;
  __shared__ __attribute__((aligned(1024))) uint8_t smem_all[kSparseWaves * WAVE_LDS];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  uint8_t* smem = smem_all + wave * WAVE_LDS;

  // Workgroup g takes query tile g % nqt of the (batch, head)s 4 (g / nqt) .. + 3, one per wavefront: wavefronts of a
  // workgroup have like amounts of work, the tiles of one (batch, head) sit in neighbouring workgroups (one die's L2).
  const uint32_t nqt = static_cast<uint32_t>((p.Tq + 31) / 32);
  const uint32_t logical = xcd_remap(blockIdx.x, gridDim.x);
  uint32_t group_u, qt_u, b_u, h_u;
  magic_divmod(logical, nqt, p.nqt_magic, group_u, qt_u);
  const uint32_t bh_u = group_u * kSparseWaves + static_cast<uint32_t>(wave);
  if (bh_u >= static_cast<uint32_t>(p.B) * static_cast<uint32_t>(p.H)) return;
  magic_divmod(bh_u, static_cast<uint32_t>(p.H), p.h_magic, b_u, h_u);
  const int qt = static_cast<int>(qt_u), h = static_cast<int>(h_u), b = static_cast<int>(b_u);
  const int lane = threadIdx.x % kWave;
  const int l32 = lane % 32;
  const int hh = lane / 32;

  const T* qb = static_cast<const T*>(p.q) + b * p.qs[0] + h * p.qs[1];
  const T* kb = static_cast<const T*>(p.k) + b * p.ks[0] + h * p.ks[1];
  const T* vb = static_cast<const T*>(p.v) + b * p.vs[0] + h * p.vs[1];
  T* ob = static_cast<T*>(p.o) + b * p.os[0] + h * p.os[1];

  int len = p.Tk;
  if (p.key_lengths != nullptr) {
    len = p.key_lengths[b];
    len = len < 0 ? 0 : (len > p.Tk ? p.Tk : len);
  }
  const int q_begin = qt * 32;
  const int q_valid = p.zero_pad ? (len < p.Tq ? len : p.Tq) : p.Tq;
  vec_t zero_vec;
#pragma unroll
  for (int e = 0; e < 8; ++e) zero_vec[e] = static_cast<T>(0.f);
  const int c8 = lane % C8;
  constexpr int RPP = kWave / C8;
  if (q_begin >= q_valid) {  // whole tile in the padding: zero-fill its rows, or leave them alone
    if (p.zero_pad == 2) return;
#pragma unroll
    for (int pass = 0; pass < 32 / RPP; ++pass) {
      const int row = q_begin + pass * RPP + lane / C8;
      if (row < p.Tq) *reinterpret_cast<vec_t*>(ob + row * p.os[2] + c8 * 8) = zero_vec;
    }
    return;
  }

  const int qi = q_begin + l32;
  // self-only rows return their value row (epilogue) and take no part in the products
  uint32_t self_word = 0u;
  if (p.self_bits != nullptr) self_word = p.self_bits[static_cast<int64_t>(b) * ((p.Tq + 31) / 32) + qt];
  const bool row_active = qi < q_valid && ((self_word >> l32) & 1u) == 0u;
  const uint32_t* bits_row = p.struct_bits + b * p.struct_stride + static_cast<int64_t>(qi < p.Tq ? qi : 0) * p.wpr;
  // Lane w holds word w of the sample's key validity, cut at the valid length (at most 64 words: Tk <= 2048); lane c the
  // set of key words that compact tile c of this query tile draws its keys from: one ballot names the compact tiles
  // that can hold a valid key (a tile none of whose words has a valid key is never visited).
  const int64_t compact_base = (p.struct_stride != 0 ? static_cast<int64_t>(b) * nqt : 0) + qt;
  const int32_t* keys_tile = p.compact_keys + compact_base * (32 * p.wpr);
  uint32_t valid_lane = 0u;
  if (lane < p.wpr) valid_lane = p.valid_bits != nullptr ? p.valid_bits[static_cast<int64_t>(b) * p.wpr + lane] : ~0u;
  const uint64_t words_of_tile = p.compact_tiles[compact_base * 64 + lane];
  // The keys of the first two compact tiles are requested now, with everything else the prologue loads: they are
  // almost always the first tiles visited, and their K / V rows can then be requested as soon as the tile set is known.
  const int key_first = keys_tile[l32];
  const int key_second = p.wpr > 1 ? keys_tile[32 + l32] : -1;
  {
    const int rest = len - lane * 32;
    if (rest < 32) valid_lane &= rest <= 0 ? 0u : ((1u << rest) - 1u);
  }
  // validity of key `key` (per lane): the bit of the word held by lane key / 32
  auto key_is_valid = [&](int key) -> bool {
    const uint32_t word = static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute((key >> 5) << 2, static_cast<int>(valid_lane)));
    return key >= 0 && ((word >> (key & 31)) & 1u) != 0u;
  };

  // The query enters the products already multiplied by the softmax scale, log2 e and its row / feature factors, rounded
  // once more to the storage type: the score tiles come out of the matrix unit in the exponent's units.
  float q_row_factor = 1.0f;
  if (SCALED && p.q_row_scale != nullptr && qi < q_valid) q_row_factor = p.q_row_scale[static_cast<int64_t>(b) * p.Tq + qi];
  vec_t qf[KSTEPS];
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s)
    qf[s] = qi < q_valid ? *reinterpret_cast<const vec_t*>(qb + qi * p.qs[2] + 16 * s + 8 * hh) : zero_vec;
  QueryFeatureFactors<SCALED, KSTEPS> feature_factors;
  feature_factors.load(p.q_col_scale, h * p.d + 8 * hh);
  const float c = (SCALED && p.q_row_scale != nullptr) ? p.scale_log2 * q_row_factor : p.scale_log2;
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
    for (int e = 0; e < 8; ++e) qf[s][e] = static_cast<T>(static_cast<float>(qf[s][e]) * feature_factors.times(s, e, c));
  // ---- the tiles this wavefront visits: bit kt of `tiles` (none when every row is in the padding or self-only) -------
  const uint64_t words_with_valid_keys = __builtin_amdgcn_ballot_w64(valid_lane != 0u);
  uint64_t tiles = __builtin_amdgcn_ballot_w64((words_of_tile & words_with_valid_keys) != 0ull);
  if (__builtin_amdgcn_ballot_w64(row_active) == 0ull) tiles = 0ull;

  f32x16 oacc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int j = 0; j < 16; ++j) oacc[mb][j] = 0.f;
  // Softmax with a lazily moved reference, as in the chunked direct-transfer kernel: -m is the C operand of the first
  // score product, m moves (and the accumulators are rescaled) only when a score exceeds it by more than kLazyBits.
  constexpr float kLazyBits = 8.f;
  f32x16 negm;
#pragma unroll
  for (int j = 0; j < 16; ++j) negm[j] = 0.f;
  float l_lane = 0.f;
  bool m_set = false;
  float thr = -3.0e38f;

  auto v_swizzle = [](int r) -> int { return DP == 32 ? 0 : 4 * ((r / 2) % 2); };
  const uint32_t k_row_bytes = static_cast<uint32_t>(p.ks[2]) * 2u, v_row_bytes = static_cast<uint32_t>(p.vs[2]) * 2u;
  const bool scale_keys = SCALED && p.k_row_scale != nullptr;
  // Operands of a tile: the lane's pieces of the V tile (piece i * 64 + lane = row / C8, 16 bytes / C8), its K fragments,
  // its word of the mask and its key's factor. Two sets: a tile is consumed while the one after it is in flight.
  struct TileOperands {
    vec_t v[PPT], kf[KSTEPS];
    uint32_t word;
    uint32_t valid;  // the lane's key (key l32 of the compact tile) is valid
    float kfac;
  };
  // `key` = the lane's key of compact tile kt (compact_keys[32 kt + l32], fetched a tile earlier still), -1: none.
  auto issue = [&](int kt, int key, TileOperands& t) {
    const int krow = key < 0 ? 0 : key;
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      const int slot = i * kWave + lane;
      const int row = __builtin_amdgcn_ds_bpermute((slot / C8) << 2, krow);  // the key of row slot / C8 of the tile
      t.v[i] = *reinterpret_cast<const vec_t*>(reinterpret_cast<const uint8_t*>(vb) +
                                               __umul24(static_cast<uint32_t>(row), v_row_bytes) + (slot % C8) * 16);
    }
    const uint8_t* ksrc = reinterpret_cast<const uint8_t*>(kb) + __umul24(static_cast<uint32_t>(krow), k_row_bytes) + hh * 16;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) t.kf[s] = *reinterpret_cast<const vec_t*>(ksrc + s * 32);
    t.word = row_active ? bits_row[kt] : 0u;
    t.valid = key_is_valid(key) ? 1u : 0u;
    t.kfac = 1.f;
    if (SCALED && scale_keys) t.kfac = p.k_row_scale[static_cast<int64_t>(b) * p.Tk + krow];
  };

  const uint32_t smem_off = lds_offset(smem);
  const int v_key = 4 * (lane / 32) + (lane % 16) / 4;
  const uint32_t v_addr = smem_off + static_cast<uint32_t>(
      v_key * ROWB + ((2 * ((lane / 16) % 2) + (lane % 4) / 2) ^ v_swizzle(v_key)) * 16 + (lane % 2) * 8);

  auto consume = [&](int kt, TileOperands& t) {
    const uint32_t vword = static_cast<uint32_t>(__builtin_amdgcn_ballot_w64(t.valid != 0u));  // lanes 0 .. 31: key l32
    const uint32_t word = t.word & vword;
    // The V tile goes into the wavefront's LDS tile (the transposed reads of the tile before it have been waited for);
    // rows of invalid keys are stored as zeros.
#pragma unroll
    for (int i = 0; i < PPT; ++i) {
      const int slot = i * kWave + lane;
      const int r = slot / C8;
      const bool ok = ((vword >> r) & 1u) != 0u;
      *reinterpret_cast<vec_t*>(smem + r * ROWB + ((slot % C8) ^ v_swizzle(r)) * 16) = ok ? t.v[i] : zero_vec;
    }
    if (SCALED && scale_keys) {
#pragma unroll
      for (int s = 0; s < KSTEPS; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) t.kf[s][e] = static_cast<T>(static_cast<float>(t.kf[s][e]) * t.kfac);
    }
    f32x16 sacc;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) sacc = Mfma32<T>::run(t.kf[s], qf[s], s == 0 ? negm : sacc);
    if (__builtin_amdgcn_ballot_w64(word != 0xffffffffu) != 0ull) {  // wavefront-uniform
      const uint32_t bits = word >> (hh * 4);
#pragma unroll
      for (int j = 0; j < 16; ++j)
        if (((bits >> ((j / 4) * 8 + (j % 4))) & 1u) == 0u) sacc[j] = -INFINITY;
    }
    float mx = sacc[0];
#pragma unroll
    for (int j = 1; j < 16; ++j) mx = fmaxf(mx, sacc[j]);
    if (__builtin_amdgcn_ballot_w64(mx > thr) != 0ull) {  // wavefront-uniform, rare after a query's first visible tile
      const float mxp = pair_max(mx);  // both lanes of a query keep one reference between them
      const bool move = mxp > thr;
      const float shift = move ? mxp : 0.f;
      const float alpha = (move && m_set) ? __builtin_amdgcn_exp2f(-mxp) : 1.f;
#pragma unroll
      for (int j = 0; j < 16; ++j) sacc[j] -= shift;
#pragma unroll
      for (int j = 0; j < 16; ++j) negm[j] -= shift;
      l_lane *= alpha;
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int j = 0; j < 16; ++j) oacc[mb][j] *= alpha;
      if (move) {
        m_set = true;
        thr = kLazyBits;
      }
    }
    float pr[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) pr[j] = __builtin_amdgcn_exp2f(sacc[j]);
    vec_t pb[2];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      pb[0][e] = static_cast<T>(pr[e]);
      pb[1][e] = static_cast<T>(pr[8 + e]);
    }
    l_lane = frag_sum(pb[0], l_lane);
    l_lane = frag_sum(pb[1], l_lane);
    static_for<MB>([&](auto mb_tag) {
      constexpr int mb = decltype(mb_tag)::value;
      const uint32_t v_addr_mb = v_addr ^ (mb * 64);
      u32x2 vt[2][2];
      lds_read_tr16<0>(vt[0][0], v_addr_mb);
      lds_read_tr16<8 * ROWB>(vt[0][1], v_addr_mb);
      lds_read_tr16<16 * ROWB>(vt[1][0], v_addr_mb);
      lds_read_tr16<24 * ROWB>(vt[1][1], v_addr_mb);
      asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(vt[0][0]), "+v"(vt[0][1]), "+v"(vt[1][0]), "+v"(vt[1][1]) : : "memory");
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) {
        const u32x4 bits = {vt[s2][0][0], vt[s2][0][1], vt[s2][1][0], vt[s2][1][1]};
        oacc[mb] = Mfma32<T>::run(__builtin_bit_cast(vec_t, bits), pb[s2], oacc[mb]);
      }
    });
  };

  auto pop_tile = [&]() -> int {
    if (tiles == 0ull) return -1;
    const int kt = __builtin_ctzll(tiles);
    tiles &= tiles - 1ull;
    return kt;
  };
  // Pipeline: the keys of a compact tile are fetched two tiles ahead, its K / V rows and mask word one tile ahead.
  auto load_key = [&](int kt) -> int {
    if (kt < 0) return -1;
    if (kt == 0) return key_first;
    if (kt == 1) return key_second;
    return keys_tile[kt * 32 + l32];
  };
  TileOperands next;
  int kt = pop_tile();
  int kt_next = pop_tile();
  int key_next = load_key(kt_next);
  if (kt >= 0) issue(kt, load_key(kt), next);
  while (kt >= 0) {
    TileOperands cur = next;
    const int kt_after = pop_tile();
    const int key_after = load_key(kt_after);
    if (kt_next >= 0) issue(kt_next, key_next, next);
    consume(kt, cur);
    kt = kt_next;
    kt_next = kt_after;
    key_next = key_after;
  }

  // ---- finalise: O / l, transpose through the wavefront's LDS tile, self rows, 16-byte stores -------------------------
  const float l_run = pair_sum(l_lane);
  const float inv = l_run > 0.f ? __builtin_amdgcn_rcpf(l_run) : 0.f;  // 1 ulp; the products are rounded to 16 bits
  const float fin = (qi < q_valid) ? inv : 0.f;
  uint8_t* tile = smem;
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
    for (int jq = 0; jq < 4; ++jq) {
      vec4_t ov;
#pragma unroll
      for (int e = 0; e < 4; ++e) ov[e] = static_cast<T>(oacc[mb][jq * 4 + e] * fin);
      *reinterpret_cast<vec4_t*>(tile + l32 * OROW + (mb * 32 + jq * 8 + hh * 4) * 2) = ov;
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  const int q_store_end = p.zero_pad == 2 ? q_valid : p.Tq;
#pragma unroll
  for (int pass = 0; pass < 32 / RPP; ++pass) {
    const int row = pass * RPP + lane / C8;
    const int q_row = q_begin + row;
    vec_t v = *reinterpret_cast<const vec_t*>(tile + row * OROW + c8 * 16);
    if (((self_word >> row) & 1u) != 0u && q_row < p.Tq) v = *reinterpret_cast<const vec_t*>(vb + q_row * p.vs[2] + c8 * 8);
    if (q_row < q_store_end) *reinterpret_cast<vec_t*>(ob + q_row * p.os[2] + c8 * 8) = v;
  }
}

template <typename T, int DP>
void launch(const AttnParams& p, bool causal, bool register_staging, hipStream_t s) {
  const bool scaled = p.q_row_scale != nullptr || p.k_row_scale != nullptr || p.q_col_scale != nullptr;
  // TAAC_ATTN_REGISTER_STAGING keeps the general kernel for full head dims too (comparison route of the caller).
  const bool dma_staging = !register_staging;
  // 32-bit source offsets with a 24-bit row multiply: row strides below 8 M elements, sequences below 2^31 bytes
  // (the same for the query and output rows)
  const bool small_offsets = p.ks[2] < (1 << 22) && p.vs[2] < (1 << 22) && p.Tk < (1 << 22) &&
                             static_cast<int64_t>(p.Tk) * p.ks[2] * 2 < (1ll << 31) &&
                             static_cast<int64_t>(p.Tk) * p.vs[2] * 2 < (1ll << 31) &&
                             p.qs[2] >= 0 && p.os[2] >= 0 && p.qs[2] < (1 << 22) && p.os[2] < (1 << 22) && p.Tq < (1 << 22) &&
                             static_cast<int64_t>(p.Tq) * p.qs[2] * 2 < (1ll << 31) &&
                             static_cast<int64_t>(p.Tq) * p.os[2] * 2 < (1ll << 31);
  if constexpr (DP == 32 || DP == 64) {
    if (p.compact_keys != nullptr) {  // the entry point has checked the shape
      const int64_t groups = static_cast<int64_t>((p.Tq + 31) / 32) * ((static_cast<int64_t>(p.B) * p.H + kSparseWaves - 1) / kSparseWaves);
      if (scaled)
        hipLaunchKernelGGL((flash_attn_fwd_sparse_kernel<T, DP, true>), dim3(static_cast<uint32_t>(groups)),
                           dim3(kSparseWaves * kWave), 0, s, p);
      else
        hipLaunchKernelGGL((flash_attn_fwd_sparse_kernel<T, DP, false>), dim3(static_cast<uint32_t>(groups)),
                           dim3(kSparseWaves * kWave), 0, s, p);
      return;
    }
    // structure bits ride along when they are all there is to the mask: per sample, no validity or self rows, no chunk map
    const bool structure_only = p.struct_bits != nullptr && p.valid_bits == nullptr && p.self_bits == nullptr &&
                                p.block_any == nullptr;
    if (p.d == DP && (p.struct_bits == nullptr || structure_only) && dma_staging && small_offsets && p.drop_mask == nullptr) {
      if (structure_only && scaled)
        hipLaunchKernelGGL((flash_attn_fwd_dma_kernel<T, DP, false, true, true>), dim3(p.total_g), dim3(kThreads), 0, s, p);
      else if (structure_only)
        hipLaunchKernelGGL((flash_attn_fwd_dma_kernel<T, DP, false, false, true>), dim3(p.total_g), dim3(kThreads), 0, s, p);
      else if (causal && scaled)
        hipLaunchKernelGGL((flash_attn_fwd_dma_kernel<T, DP, true, true, false>), dim3(p.total_g), dim3(kThreads), 0, s, p);
      else if (causal)
        hipLaunchKernelGGL((flash_attn_fwd_dma_kernel<T, DP, true, false, false>), dim3(p.total_g), dim3(kThreads), 0, s, p);
      else if (scaled)
        hipLaunchKernelGGL((flash_attn_fwd_dma_kernel<T, DP, false, true, false>), dim3(p.total_g), dim3(kThreads), 0, s, p);
      else
        hipLaunchKernelGGL((flash_attn_fwd_dma_kernel<T, DP, false, false, false>), dim3(p.total_g), dim3(kThreads), 0, s, p);
      return;
    }
  }
  if (p.drop_mask != nullptr && p.struct_bits != nullptr)
    hipLaunchKernelGGL((flash_attn_fwd_kernel<T, DP, false, true, true, true>), dim3(p.total), dim3(kThreads), 0, s, p);
  else if (p.drop_mask != nullptr && causal)
    hipLaunchKernelGGL((flash_attn_fwd_kernel<T, DP, true, false, false, true>), dim3(p.total), dim3(kThreads), 0, s, p);
  else if (p.drop_mask != nullptr)
    hipLaunchKernelGGL((flash_attn_fwd_kernel<T, DP, false, false, false, true>), dim3(p.total), dim3(kThreads), 0, s, p);
  else if (p.struct_bits != nullptr)
    hipLaunchKernelGGL((flash_attn_fwd_kernel<T, DP, false, true, true>), dim3(p.total), dim3(kThreads), 0, s, p);
  else if (causal && scaled)
    hipLaunchKernelGGL((flash_attn_fwd_kernel<T, DP, true, true, false>), dim3(p.total), dim3(kThreads), 0, s, p);
  else if (causal)
    hipLaunchKernelGGL((flash_attn_fwd_kernel<T, DP, true, false, false>), dim3(p.total), dim3(kThreads), 0, s, p);
  else if (scaled)
    hipLaunchKernelGGL((flash_attn_fwd_kernel<T, DP, false, true, false>), dim3(p.total), dim3(kThreads), 0, s, p);
  else
    hipLaunchKernelGGL((flash_attn_fwd_kernel<T, DP, false, false, false>), dim3(p.total), dim3(kThreads), 0, s, p);
}

template <typename T>
void launch_dp(const AttnParams& p, bool causal, bool register_staging, hipStream_t s) {
  if (p.d <= 32)
    launch<T, 32>(p, causal, register_staging, s);
  else if (p.d <= 64)
    launch<T, 64>(p, causal, register_staging, s);
  else
    launch<T, 128>(p, causal, register_staging, s);
}

bool strides_ok(const int64_t* st) {
  if (st[3] != 1) return false;
  for (int i = 0; i < 3; ++i)
    if (st[i] % 8 != 0 || st[i] < 0) return false;
  return true;
}

// One word per thread: bit c % 32 of word c / 32 of a row is set iff mask[row][c] != 0; bits beyond cols are zero.
__global__ __launch_bounds__(256) void pack_bits_kernel(const uint8_t* __restrict__ mask, int64_t rows, int cols,
                                                        int wpr, uint32_t* __restrict__ bits) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= rows * wpr) return;
  const int64_t row = idx / wpr;
  const int w = static_cast<int>(idx % wpr);
  const uint8_t* src = mask + row * cols + w * 32;
  const int n = cols - w * 32 < 32 ? cols - w * 32 : 32;
  uint32_t word = 0u;
  for (int c = 0; c < n; ++c) word |= (src[c] != 0 ? 1u : 0u) << c;
  bits[idx] = word;
}

// block_any[qc][kc] = some query of rows [128 qc, 128 qc + 127] sees some key of [64 kc, 64 kc + 63]. One wavefront
// per (qc, kc): each lane ORs the two words of two rows.
__global__ __launch_bounds__(kWave) void block_any_kernel(const uint32_t* __restrict__ bits, int Tq, int wpr, int nkc,
                                                          uint8_t* __restrict__ block_any) {
  const int qc = blockIdx.x / nkc, kc = blockIdx.x % nkc;
  uint32_t acc = 0u;
  for (int r = qc * kQB + static_cast<int>(threadIdx.x); r < (qc + 1) * kQB && r < Tq; r += kWave) {
    acc |= bits[static_cast<int64_t>(r) * wpr + 2 * kc];
    if (2 * kc + 1 < wpr) acc |= bits[static_cast<int64_t>(r) * wpr + 2 * kc + 1];
  }
  const bool any = __builtin_amdgcn_ballot_w64(acc != 0u) != 0;
  if (threadIdx.x == 0) block_any[blockIdx.x] = any ? 1 : 0;
}

struct MaskArgs {
  const uint32_t* struct_bits = nullptr;
  int64_t struct_stride = 0;
  const uint8_t* block_any = nullptr;
  const uint32_t* valid_bits = nullptr;
  const uint32_t* self_bits = nullptr;
  const int32_t* compact_keys = nullptr;    // given (with compact_tiles): the one-wavefront-per-query-tile kernel
  const uint64_t* compact_tiles = nullptr;
};

int attention_entry(const char* name, const void* q, const void* k, const void* v, const int32_t* key_lengths,
                    const MaskArgs& mask, const float* q_row_scale, const float* k_row_scale, const float* q_col_scale,
                    float* lse, float* amax_out, void* o, int32_t B, int32_t H, int32_t Tq, int32_t Tk, int32_t d, const int64_t q_strides[4],
                    const int64_t k_strides[4], const int64_t v_strides[4], const int64_t o_strides[4], int mask_flags,
                    int zero_padded_queries, int dtype, void* stream, const uint8_t* drop_mask = nullptr,
                    float drop_scale = 1.f) {
  if (drop_mask != nullptr && (mask.self_bits != nullptr || mask.compact_keys != nullptr || q_row_scale != nullptr ||
                               k_row_scale != nullptr || q_col_scale != nullptr))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: dropout does not come with self-only query rows or row factors", name);
  if (drop_mask != nullptr && !(drop_scale >= 1.f))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: dropout_scale = 1 / (1 - p) must be >= 1", name);
  if (mask_flags & ~(TAAC_ATTN_CAUSAL | TAAC_ATTN_REGISTER_STAGING))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: unknown bits in is_causal (%d)", name, mask_flags);
  const int is_causal = mask_flags & TAAC_ATTN_CAUSAL;
  const bool register_staging = (mask_flags & TAAC_ATTN_REGISTER_STAGING) != 0;
  if (mask.struct_bits != nullptr) {
    if (mask.block_any == nullptr && mask.struct_stride == 0 && mask.compact_keys == nullptr)
      return set_error(TAAC_ERR_INVALID_VALUE, "%s: struct_bits shared by the batch needs block_any", name);
    if (mask.struct_stride < 0 || (mask.struct_stride != 0 && mask.struct_stride < static_cast<int64_t>(Tq) * ((Tk + 31) / 32)))
      return set_error(TAAC_ERR_INVALID_VALUE, "%s: struct_sample_stride must be 0 or cover a sample's matrix", name);
    if (Tk > 64 * kKC) return set_error(TAAC_ERR_UNSUPPORTED, "%s: structured masks cover at most %d keys", name, 64 * kKC);
    if (is_causal)
      return set_error(TAAC_ERR_INVALID_VALUE, "%s: a structured mask carries its own causal triangle", name);
    if (mask.self_bits != nullptr && Tq != Tk)
      return set_error(TAAC_ERR_INVALID_VALUE, "%s: self rows require Tq == Tk", name);
  } else if (mask.valid_bits != nullptr || mask.self_bits != nullptr || mask.block_any != nullptr) {
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: valid_bits / self_bits / block_any need struct_bits", name);
  }
  if (B < 0 || H < 0 || Tq < 0 || Tk < 0 || d <= 0)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: negative dimension or non-positive head_dim", name);
  if (dtype != TAAC_BF16 && dtype != TAAC_F16)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: dtype must be bf16 or fp16 (got %d)", name, dtype);
  if (d % 8 != 0 || d > 128)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: head_dim %d unsupported (multiple of 8, at most 128)", name, d);
  if (!q_strides || !k_strides || !v_strides || !o_strides)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: null stride array", name);
  if (B == 0 || H == 0 || Tq == 0) return TAAC_OK;
  if (!q || !o || (Tk > 0 && (!k || !v))) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  if (!strides_ok(q_strides) || !strides_ok(k_strides) || !strides_ok(v_strides) || !strides_ok(o_strides))
    return set_error(TAAC_ERR_UNSUPPORTED,
                     "%s: strides must be non-negative multiples of 8 elements with a unit last stride", name);
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o) || !aligned16(q_col_scale))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: tensor base pointers (and q_col_scale) must be 16-byte aligned", name);
  if (zero_padded_queries && Tq != Tk)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: zero_padded_queries requires Tq == Tk", name);

  AttnParams p;
  p.q = q;
  p.k = k;
  p.v = v;
  p.o = o;
  p.key_lengths = key_lengths;
  p.q_row_scale = q_row_scale;
  p.k_row_scale = k_row_scale;
  p.q_col_scale = q_col_scale;
  p.amax_out = amax_out;
  p.drop_mask = drop_mask;
  p.drop_scale = drop_scale;
  p.lse = lse;
  p.struct_bits = mask.struct_bits;
  p.struct_stride = mask.struct_stride;
  p.valid_bits = mask.valid_bits;
  p.self_bits = mask.self_bits;
  p.block_any = mask.block_any;
  p.compact_keys = mask.compact_keys;
  p.compact_tiles = mask.compact_tiles;
  p.wpr = (Tk + 31) / 32;
  p.nkc = (Tk + kKC - 1) / kKC;
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
  }
  p.scale_log2 = 1.4426950408889634f / sqrtf(static_cast<float>(d));
  p.zero_pad = zero_padded_queries == 2 ? 2 : (zero_padded_queries ? 1 : 0);
  p.nqc = static_cast<uint32_t>((Tq + kQB - 1) / kQB);
  const int64_t total = static_cast<int64_t>(p.nqc) * B * H;
  if (total > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: too many workgroups (%lld)", name, (long long)total);
  p.total = static_cast<uint32_t>(total);
  p.nqc_magic = magic_of(p.nqc);
  p.h_magic = magic_of(static_cast<uint32_t>(H));
  p.nqt_magic = magic_of(static_cast<uint32_t>((Tq + 31) / 32));
  // Pairs of query blocks per workgroup where blocks differ in work or may be empty (key lengths, a causal triangle);
  // with neither, every block is the same and single blocks fill the last round of the launch better.
  p.pair_blocks = (p.nqc > 1 && (key_lengths != nullptr || is_causal != 0)) ? 1 : 0;
  p.nqg = p.pair_blocks ? (p.nqc + 1) / 2 : p.nqc;
  p.nqg_magic = magic_of(p.nqg);
  p.total_g = p.nqg * static_cast<uint32_t>(B) * static_cast<uint32_t>(H);

  hipStream_t s = as_stream(stream);
  if (dtype == TAAC_BF16)
    launch_dp<bf16_t>(p, is_causal != 0, register_staging, s);
  else
    launch_dp<f16_t>(p, is_causal != 0, register_staging, s);
  return check_launch(name);
}

}  // namespace
}  // namespace taac

extern "C" int taac_flash_attn_fwd(const void* q, const void* k, const void* v, const int32_t* key_lengths, void* o,
                                   int32_t B, int32_t H, int32_t Tq, int32_t Tk, int32_t d,
                                   const int64_t q_strides[4], const int64_t k_strides[4], const int64_t v_strides[4],
                                   const int64_t o_strides[4], int is_causal, int zero_padded_queries, int dtype,
                                   void* stream) {
  return taac::attention_entry("taac_flash_attn_fwd", q, k, v, key_lengths, taac::MaskArgs{}, nullptr, nullptr, nullptr,
                               nullptr, nullptr, o, B, H, Tq, Tk, d,
                               q_strides, k_strides, v_strides, o_strides, is_causal, zero_padded_queries, dtype, stream);
}

extern "C" int taac_flash_attn_scaled_fwd(const void* q, const void* k, const void* v, const int32_t* key_lengths,
                                          const float* q_row_scale, const float* k_row_scale,
                                          const float* q_col_scale, void* o, int32_t B, int32_t H, int32_t Tq,
                                          int32_t Tk, int32_t d, const int64_t q_strides[4],
                                          const int64_t k_strides[4], const int64_t v_strides[4],
                                          const int64_t o_strides[4], int is_causal, int zero_padded_queries, int dtype,
                                          void* stream) {
  return taac::attention_entry("taac_flash_attn_scaled_fwd", q, k, v, key_lengths, taac::MaskArgs{}, q_row_scale,
                               k_row_scale, q_col_scale, nullptr, nullptr, o, B, H, Tq, Tk, d, q_strides, k_strides, v_strides,
                               o_strides, is_causal, zero_padded_queries, dtype, stream);
}

namespace taac {
namespace {
__global__ void attn_clear_kernel(float* a) {
  if (threadIdx.x == 0 && blockIdx.x == 0) *a = 0.f;
}
}  // namespace
}  // namespace taac

extern "C" int taac_flash_attn_amax_fwd(const void* q, const void* k, const void* v, const int32_t* key_lengths,
                                        const float* q_row_scale, const float* k_row_scale, const float* q_col_scale,
                                        void* o, float* amax_out, int32_t B, int32_t H, int32_t Tq, int32_t Tk, int32_t d,
                                        const int64_t q_strides[4], const int64_t k_strides[4],
                                        const int64_t v_strides[4], const int64_t o_strides[4], int is_causal,
                                        int zero_padded_queries, int dtype, void* stream) {
  if (!amax_out) return taac::set_error(TAAC_ERR_INVALID_VALUE, "taac_flash_attn_amax_fwd: amax_out must be given");
  if (!taac::maxima_precleared) {
    hipLaunchKernelGGL(taac::attn_clear_kernel, dim3(1), dim3(taac::kWave), 0, taac::as_stream(stream), amax_out);
    const int rc = taac::check_launch("taac_flash_attn_amax_fwd");
    if (rc != TAAC_OK) return rc;
  }
  return taac::attention_entry("taac_flash_attn_amax_fwd", q, k, v, key_lengths, taac::MaskArgs{}, q_row_scale,
                               k_row_scale, q_col_scale, nullptr, amax_out, o, B, H, Tq, Tk, d, q_strides, k_strides,
                               v_strides, o_strides, is_causal, zero_padded_queries, dtype, stream);
}

extern "C" int taac_flash_attn_masked_fwd(const void* q, const void* k, const void* v, const int32_t* key_lengths,
                                          const uint32_t* struct_bits, int64_t struct_sample_stride,
                                          const uint8_t* block_any,
                                          const uint32_t* valid_bits, const uint32_t* self_bits,
                                          const float* q_row_scale, const float* k_row_scale, const float* q_col_scale,
                                          void* o, int32_t B, int32_t H, int32_t Tq, int32_t Tk, int32_t d,
                                          const int64_t q_strides[4], const int64_t k_strides[4],
                                          const int64_t v_strides[4], const int64_t o_strides[4],
                                          int zero_padded_queries, int dtype, void* stream) {
  if (!struct_bits)
    return taac::set_error(TAAC_ERR_INVALID_VALUE, "taac_flash_attn_masked_fwd: struct_bits must be given");
  taac::MaskArgs mask;
  mask.struct_bits = struct_bits;
  mask.struct_stride = struct_sample_stride;
  mask.block_any = block_any;
  mask.valid_bits = valid_bits;
  mask.self_bits = self_bits;
  return taac::attention_entry("taac_flash_attn_masked_fwd", q, k, v, key_lengths, mask, q_row_scale, k_row_scale,
                               q_col_scale, nullptr, nullptr, o, B, H, Tq, Tk, d, q_strides, k_strides, v_strides, o_strides,
                               0, zero_padded_queries, dtype, stream);
}

extern "C" int taac_flash_attn_masked_train_fwd(const void* q, const void* k, const void* v, const int32_t* key_lengths,
                                                const uint32_t* struct_bits, int64_t struct_sample_stride,
                                                const uint8_t* block_any, const uint32_t* valid_bits,
                                                const uint32_t* self_bits, const uint8_t* dropout_mask,
                                                float dropout_scale, void* o, float* lse, int32_t B, int32_t H,
                                                int32_t Tq, int32_t Tk, int32_t d, const int64_t q_strides[4],
                                                const int64_t k_strides[4], const int64_t v_strides[4],
                                                const int64_t o_strides[4], int zero_padded_queries, int dtype,
                                                void* stream) {
  const char* name = "taac_flash_attn_masked_train_fwd";
  if (!struct_bits) return taac::set_error(TAAC_ERR_INVALID_VALUE, "%s: struct_bits must be given", name);
  if (!lse && B > 0 && H > 0 && Tq > 0) return taac::set_error(TAAC_ERR_INVALID_VALUE, "%s: lse must be given", name);
  taac::MaskArgs mask;
  mask.struct_bits = struct_bits;
  mask.struct_stride = struct_sample_stride;
  mask.block_any = block_any;
  mask.valid_bits = valid_bits;
  mask.self_bits = self_bits;
  return taac::attention_entry(name, q, k, v, key_lengths, mask, nullptr, nullptr, nullptr, lse, nullptr, o, B, H, Tq, Tk, d,
                               q_strides, k_strides, v_strides, o_strides, 0, zero_padded_queries, dtype, stream,
                               dropout_mask, dropout_mask != nullptr ? dropout_scale : 1.f);
}

extern "C" int taac_flash_attn_sparse_fwd(const void* q, const void* k, const void* v, const int32_t* key_lengths,
                                          const uint32_t* compact_bits, int64_t compact_sample_stride,
                                          const int32_t* compact_keys, const uint64_t* compact_tiles,
                                          const uint32_t* valid_bits, const uint32_t* self_bits,
                                          const float* q_row_scale, const float* k_row_scale, const float* q_col_scale,
                                          void* o, int32_t B, int32_t H, int32_t Tq, int32_t Tk, int32_t d,
                                          const int64_t q_strides[4], const int64_t k_strides[4],
                                          const int64_t v_strides[4], const int64_t o_strides[4],
                                          int zero_padded_queries, int dtype, void* stream) {
  using namespace taac;
  const char* name = "taac_flash_attn_sparse_fwd";
  if (!compact_bits || !compact_keys || !compact_tiles)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: compact_bits, compact_keys and compact_tiles must be given", name);
  if (d != 32 && d != 64) return set_error(TAAC_ERR_UNSUPPORTED, "%s: head_dim must be 32 or 64 (got %d)", name, d);
  if (Tk < 1 || Tk > 2048) return set_error(TAAC_ERR_UNSUPPORTED, "%s: 1 <= Tk <= 2048 required (got %d)", name, Tk);
  if (!k_strides || !v_strides) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null stride array", name);
  if (k_strides[2] >= (1 << 22) || v_strides[2] >= (1 << 22) || static_cast<int64_t>(Tk) * k_strides[2] * 2 >= (1ll << 31) ||
      static_cast<int64_t>(Tk) * v_strides[2] * 2 >= (1ll << 31))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: key / value row strides must fit 32-bit byte offsets", name);
  if (static_cast<int64_t>((Tq + 31) / 32) * B * H > 0x7fffffffLL)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: too many query tiles", name);
  MaskArgs mask;
  mask.struct_bits = compact_bits;
  mask.struct_stride = compact_sample_stride;
  mask.valid_bits = valid_bits;
  mask.self_bits = self_bits;
  mask.compact_keys = compact_keys;
  mask.compact_tiles = compact_tiles;
  return attention_entry(name, q, k, v, key_lengths, mask, q_row_scale, k_row_scale, q_col_scale, nullptr, nullptr, o, B, H,
                         Tq, Tk, d, q_strides, k_strides, v_strides, o_strides, 0, zero_padded_queries, dtype, stream);
}

namespace taac {
namespace {
// One wavefront per (sample, 32-query tile): the key columns some row of the tile can see, in ascending order
// (compact_keys, -1 behind them), per compact tile of 32 such keys the set of 32-key words of Tk it draws from
// (compact_tiles), and per query row one word per compact tile (compact_bits: bit j = the row sees key 32 c + j of the list).
__global__ __launch_bounds__(kWave) void mask_compact_kernel(const uint32_t* __restrict__ bits, int Tq, int wpr, int64_t stride,
                                                            uint32_t* __restrict__ compact_bits,
                                                            int32_t* __restrict__ compact_keys,
                                                            uint64_t* __restrict__ compact_tiles) {
  __shared__ int32_t keys[2048];
  const int nqt = (Tq + 31) / 32;
  const int t = blockIdx.x % nqt;
  const int64_t smp = blockIdx.x / nqt;
  const int lane = threadIdx.x;
  const uint32_t* src = bits + smp * stride;
  // union of the tile's rows, word `lane`
  uint32_t seen = 0u;
  if (lane < wpr)
    for (int r = t * 32; r < t * 32 + 32 && r < Tq; ++r) seen |= src[static_cast<int64_t>(r) * wpr + lane];
  // exclusive prefix sum of the words' population counts over the lanes
  const int count = __builtin_popcount(seen);
  int before = count;
#pragma unroll
  for (int d = 1; d < kWave; d *= 2) {
    const int up = __shfl_up(before, d, kWave);
    if (lane >= d) before += up;
  }
  const int total = __shfl(before, kWave - 1, kWave);
  before -= count;
  for (int j = lane; j < 32 * wpr; j += kWave) keys[j] = -1;
  __syncthreads();
  uint32_t rest = seen;
  for (int i = 0; rest != 0u; ++i) {
    const int bit = __builtin_ctz(rest);
    rest &= rest - 1u;
    keys[before + i] = lane * 32 + bit;
  }
  __syncthreads();
  const int ntiles = (total + 31) / 32;
  int32_t* keys_out = compact_keys + (smp * nqt + t) * (32 * static_cast<int64_t>(wpr));
  for (int j = lane; j < 32 * wpr; j += kWave) keys_out[j] = keys[j];
  uint64_t words = 0ull;
  if (lane < ntiles)
    for (int j = 0; j < 32; ++j) {
      const int key = keys[lane * 32 + j];
      if (key >= 0) words |= 1ull << (key >> 5);
    }
  compact_tiles[(smp * nqt + t) * 64 + lane] = words;
  // two rows per pass: lanes 0 .. 31 the even row of the pair, lanes 32 .. 63 the odd one
  for (int r2 = 0; r2 < 32; r2 += 2) {
    const int row = t * 32 + r2 + lane / 32;
    for (int c = 0; c < wpr; ++c) {
      bool bit = false;
      if (row < Tq && c < ntiles) {
        const int key = keys[c * 32 + lane % 32];
        bit = key >= 0 && ((src[static_cast<int64_t>(row) * wpr + (key >> 5)] >> (key & 31)) & 1u) != 0u;
      }
      const uint64_t both = __builtin_amdgcn_ballot_w64(bit);
      if (row < Tq && lane % 32 == 0)
        compact_bits[(smp * Tq + row) * static_cast<int64_t>(wpr) + c] = static_cast<uint32_t>(lane == 0 ? both : both >> 32);
    }
  }
}
}  // namespace
}  // namespace taac

extern "C" int taac_mask_compact(const uint32_t* struct_bits, int32_t samples, int32_t Tq, int32_t Tk,
                                 int64_t struct_sample_stride, uint32_t* compact_bits, int32_t* compact_keys,
                                 uint64_t* compact_tiles, void* stream) {
  using namespace taac;
  const char* name = "taac_mask_compact";
  if (samples <= 0 || Tq <= 0 || Tk <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: samples, Tq and Tk must be positive", name);
  if (Tk > 2048) return set_error(TAAC_ERR_UNSUPPORTED, "%s: Tk <= 2048 required (got %d)", name, Tk);
  if (!struct_bits || !compact_bits || !compact_keys || !compact_tiles)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  const int wpr = (Tk + 31) / 32;
  if (samples > 1 && struct_sample_stride < static_cast<int64_t>(Tq) * wpr)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: struct_sample_stride must cover a sample's matrix", name);
  const int64_t groups = static_cast<int64_t>(samples) * ((Tq + 31) / 32);
  if (groups > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: mask too large", name);
  hipLaunchKernelGGL(mask_compact_kernel, dim3(static_cast<uint32_t>(groups)), dim3(kWave), 0, as_stream(stream), struct_bits,
                     Tq, wpr, struct_sample_stride, compact_bits, compact_keys, compact_tiles);
  return check_launch(name);
}

extern "C" int taac_mask_pack_bits(const void* mask, int64_t rows, int32_t cols, uint32_t* bits, void* stream) {
  using namespace taac;
  const char* name = "taac_mask_pack_bits";
  if (rows < 0 || cols <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: rows >= 0 and cols > 0 required", name);
  if (rows == 0) return TAAC_OK;
  if (!mask || !bits) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  const int wpr = (cols + 31) / 32;
  const int64_t words = rows * wpr;
  if (words > 0x7fffffffLL * 256) return set_error(TAAC_ERR_UNSUPPORTED, "%s: mask too large", name);
  hipLaunchKernelGGL(pack_bits_kernel, dim3(static_cast<uint32_t>((words + 255) / 256)), dim3(256), 0, as_stream(stream),
                     static_cast<const uint8_t*>(mask), rows, cols, wpr, bits);
  return check_launch(name);
}

extern "C" int taac_mask_block_any(const uint32_t* struct_bits, int32_t Tq, int32_t Tk, uint8_t* block_any,
                                   void* stream) {
  using namespace taac;
  const char* name = "taac_mask_block_any";
  if (Tq <= 0 || Tk <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: Tq and Tk must be positive", name);
  if (!struct_bits || !block_any) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  const int nqc = (Tq + kQB - 1) / kQB, nkc = (Tk + kKC - 1) / kKC;
  hipLaunchKernelGGL(block_any_kernel, dim3(nqc * nkc), dim3(kWave), 0, as_stream(stream), struct_bits, Tq,
                     (Tk + 31) / 32, nkc, block_any);
  return check_launch(name);
}

extern "C" int taac_flash_attn_train_dropout_fwd(const void* q, const void* k, const void* v, const int32_t* key_lengths,
                                                 const uint8_t* dropout_mask, float dropout_scale, void* o, float* lse,
                                                 int32_t B, int32_t H, int32_t Tq, int32_t Tk, int32_t d,
                                                 const int64_t q_strides[4], const int64_t k_strides[4],
                                                 const int64_t v_strides[4], const int64_t o_strides[4], int is_causal,
                                                 int zero_padded_queries, int dtype, void* stream) {
  const char* name = "taac_flash_attn_train_dropout_fwd";
  if (!lse) return taac::set_error(TAAC_ERR_INVALID_VALUE, "%s: lse must be given", name);
  if (!dropout_mask) return taac::set_error(TAAC_ERR_INVALID_VALUE, "%s: dropout_mask must be given", name);
  return taac::attention_entry(name, q, k, v, key_lengths, taac::MaskArgs{}, nullptr, nullptr, nullptr, lse, nullptr, o, B,
                               H, Tq, Tk, d, q_strides, k_strides, v_strides, o_strides, is_causal, zero_padded_queries,
                               dtype, stream, dropout_mask, dropout_scale);
}

extern "C" int taac_flash_attn_train_fwd(const void* q, const void* k, const void* v, const int32_t* key_lengths,
                                         void* o, float* lse, int32_t B, int32_t H, int32_t Tq, int32_t Tk, int32_t d,
                                         const int64_t q_strides[4], const int64_t k_strides[4],
                                         const int64_t v_strides[4], const int64_t o_strides[4], int is_causal,
                                         int zero_padded_queries, int dtype, void* stream) {
  if (!lse) return taac::set_error(TAAC_ERR_INVALID_VALUE, "taac_flash_attn_train_fwd: lse must be given");
  return taac::attention_entry("taac_flash_attn_train_fwd", q, k, v, key_lengths, taac::MaskArgs{}, nullptr, nullptr,
                               nullptr, lse, nullptr, o, B, H, Tq, Tk, d, q_strides, k_strides, v_strides, o_strides,
                               is_causal, zero_padded_queries, dtype, stream);
}
