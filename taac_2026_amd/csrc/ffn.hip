// Token-stationary fused dense kernels for gfx950 (model width D = 256 or 128):
//   taac_swiglu_ffn_fwd : out = residual + down( silu(gate) * value ),  gate, value = up( rmsnorm(x) ).chunk(2)
//   taac_norm_linear_fwd: out = [residual +] linear( [rmsnorm](x) )
//
// Why token-stationary. With D <= 256 the whole reduction axis of a token fits in registers: a wavefront keeps the
// (optionally RMS-normalised) rows of its tokens as MFMA B-operand fragments for the entire kernel and only the
// WEIGHTS stream past it. The weights are staged through LDS in fragment order by direct global->LDS loads (no
// register staging, one 1 KB fragment per wavefront-wide instruction), double-buffered, with one workgroup barrier
// per step. The token matrix is read from HBM exactly once and nothing is written back between the fused stages.
// Weights can be handed over pre-packed in fragment order (taac_ffn_pack_weights / taac_linear_pack_weights): every
// staging instruction then reads 1 KB of contiguous memory instead of gathering 16-byte pieces from 32 rows.
//
// Fused SwiGLU FFN. The products are formed transposed: H^T[hidden, token] = W_up X^T, so a lane owns one token and
// eight hidden units of a 16-unit chunk; silu(g) * u is formed in registers and is already the B operand of the
// second product O^T[feature, token] += W_down[:, chunk] H^T. The row order in which a chunk's W_up rows are loaded
// is chosen so that the accumulator's register order of hidden units equals the natural k order of W_down's
// fragments. The [M, 2F] projection and the [M, F] gated hidden state never exist in memory.
// Replaces SwiGLUFeedForward.forward + the ffn_norm and residual of UnifiedInteractionBlock.forward
// (experiments/symbiosis/backbone.py:19-21, 66-67).
//
// Epilogue. Accumulators are in the MFMA layout (a lane holds 4-feature runs of one token). They are rounded to
// bf16, transposed through a wavefront-private LDS tile and written as 16-byte pieces, eight lanes per 128-byte row
// segment; the residual is read the same way and added after the rounding of the layer output, which is the order
// of roundings of the reference's bf16 evaluation (linear output rounded, then the residual add rounded).
#include "common.h"
#include "ts_common.h"

namespace taac {
namespace {

constexpr int kFrag = 1024;  // bytes of one 32 x 16 bf16 MFMA operand fragment
constexpr int kNC = 64;      // output features per chunk of the plain linear kernel
constexpr int kHU = 16;      // hidden units per FFN chunk
constexpr int kCPB = 2;      // FFN chunks per barrier step
constexpr int kStageRow = kNC * 2 + 16;       // bytes per token row of the epilogue tile (64 features + pad)
constexpr int kStageWave = 32 * kStageRow;    // epilogue tile of one wavefront: 32 tokens x 64 features

struct TsParams {
  const bf16_t* x;          // [M, D] row stride ldx
  const bf16_t* norm_w;     // [D] or null (no normalisation)
  const bf16_t* w1;         // FFN: w_up [2F, D] or the packed blob; linear: w [N, D] or the packed blob
  const bf16_t* b1;         // FFN: b_up [2F] or null; linear: bias [N] or null
  const bf16_t* w2;         // FFN: w_down [D, F] (unused when packed)
  const bf16_t* b2;         // FFN: b_down [D] or null
  const bf16_t* residual;   // [M, D or N] row stride ldr, or null
  bf16_t* out;              // [M, D or N] row stride ldo
  int64_t M, ldx, ldr, ldo;
  int32_t F;                // FFN hidden size
  int32_t N;                // linear output features
  float eps;
  int32_t gate_first;
  int32_t packed;           // weights are in fragment order
  const int32_t* rows;      // optional row index: token i lives in row rows[i] of x / residual / out
  const int32_t* n_rows;    // with rows: device pointer to the number of tokens (at most M)
  const int32_t* x_rows;    // optional, with rows: token i's row of x when it differs from rows[i] (x and residual / out
                            // laid out differently: samples with their valid tokens moved to the front on one side)
  int32_t units;            // FFN: compute units the last, partial round of workgroups is spread over
  // Query / key mode of the linear kernel (the packed q | k | v projection of an attention layer):
  const bf16_t* qk_w;       // [qk_chunks * 64] norm weights of the query and key features (q | k), or null (ones)
  const bf16_t* cos_sin;    // rotary table [tokens_per_sample][head_dim] of (cos, sin) pairs, or null
  float* qk_sumsq;          // [qk_chunks][M] sum of squares of a token's 64 features of one chunk
  int32_t qk_chunks;        // leading 64-feature chunks that belong to the query and key projections
  int32_t head_dim, tokens_per_sample;
  // Attention output projection in front of the FFN (x is then the attention output, residual the block input):
  const bf16_t* w0;         // packed [D, D] projection (linear blob)
  const bf16_t* b0;         // its bias [D] or null
  int32_t norm_folded;      // linear kernel: norm_w is already part of the packed weights (taac_linear_pack_weights_norm):
                            // the rows enter the products as they are and only the factor rsqrt(mean + eps) is applied, to the
                            // accumulators
  const bf16_t* gate;       // GATE: [M, D] pre-activation of the update's gate (rows like residual), row stride ldg
  int64_t ldg;
  // Feature planes (the backbone's private q | k | v and attention-output buffers): with a shift s > 0 the tensor is a
  // stack of planes of 2^s features, [cols / 2^s][M][2^s] - element (row, col) at ((col >> s) * M + row) * 2^s + col % 2^s -
  // instead of [M][cols] rows; a head's rows are then contiguous for the attention kernel.
  int32_t x_plane_shift;    // layout of x (0: rows of ldx elements)
  int32_t out_plane_shift;  // layout of out (linear kernel without residual or query / key epilogue; 0: rows of ldo elements)
  // Readout riding on the feed-forward epilogue: token_dots[row] = sum over the features of out[row] * head_w (fp32, from
  // the rounded output), so that a mean-pooling linear head behind the layer need not read the rows again.
  const bf16_t* head_w;     // [D] or null
  float* token_dots;        // [M] (rows like out), written for the tokens the kernel stores
};

__device__ __forceinline__ float silu_f(float v) {
  return v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * v));
}

// Hidden unit (0..15) loaded into row slot m16 of the gate (or value) half of an up fragment: chosen so that
// accumulator register j < 8 of lane half hh holds hidden unit 8*hh + j, the k order of a W_down fragment.
__host__ __device__ __forceinline__ int up_unit_of_slot(int m16) {
  return 8 * ((m16 >> 2) & 1) + 4 * (m16 >> 3) + (m16 & 3);
}

// ---- fragment-order packing ------------------------------------------------------------------------------------------
// FFN blob: step s (32 hidden units) holds, for chunk q = 0, 1: KS up fragments (k-step r) then MB down fragments
// (row block r - KS); exactly the image one barrier step needs in LDS. A fragment is 64 lanes x 16 bytes.
// col_scale (optional, [D]): weight of the RMSNorm in front of the up projection, folded into its fragments (see
// linear_pack_piece).
// fold_act: the constants of the gate's activation join the same rounding - the gated half is multiplied by -log2(e), the
// other half by -ln 2, so that silu(g) * u = g' * u' / (1 + 2^g') with g' and u' as they leave the matrix unit (the
// kernel's FOLD form: one multiplication less per hidden unit and token; the first-layer bias is scaled when it is staged).
constexpr float kFoldGate = -1.4426950408889634f, kFoldValue = -0.6931471805599453f;
__device__ __forceinline__ void ffn_pack_piece(const bf16_t* __restrict__ w_up, const bf16_t* __restrict__ w_down,
                                               bf16x8* __restrict__ packed, int D, int F, int gate_first, int64_t gid,
                                               const bf16_t* __restrict__ col_scale = nullptr, bool fold_act = false) {
  const int KS = D / 16, MB = D / 32, CFRAG = KS + MB, NFRAG = kCPB * CFRAG;
  const int lane = static_cast<int>(gid % 64);
  const int f = static_cast<int>((gid / 64) % NFRAG);
  const int64_t step = gid / 64 / NFRAG;
  const int q = f / CFRAG, r = f % CFRAG;
  const int64_t unit0 = (step * kCPB + q) * kHU;
  const int l32 = lane % 32, hh = lane / 32;
  const bf16_t* src;
  if (r < KS)
    src = w_up + (((l32 < 16) == (gate_first != 0) ? 0 : F) + unit0 + up_unit_of_slot(l32 & 15)) * D + r * 16 + hh * 8;
  else
    src = w_down + static_cast<int64_t>((r - KS) * 32 + l32) * F + unit0 + hh * 8;
  bf16x8 v = *reinterpret_cast<const bf16x8*>(src);
  if ((col_scale != nullptr || fold_act) && r < KS) {
    bf16x8 g;
    if (col_scale != nullptr) {
      g = *reinterpret_cast<const bf16x8*>(col_scale + r * 16 + hh * 8);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) g[e] = static_cast<bf16_t>(1.0f);
    }
    const float c = fold_act ? (l32 < 16 ? kFoldGate : kFoldValue) : 1.0f;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = static_cast<bf16_t>(static_cast<float>(v[e]) * static_cast<float>(g[e]) * c);
  }
  packed[gid] = v;
}

__global__ void ffn_pack_kernel(const bf16_t* __restrict__ w_up, const bf16_t* __restrict__ w_down,
                                bf16x8* __restrict__ packed, int D, int F, int gate_first,
                                const bf16_t* __restrict__ col_scale, bool fold_act) {
  const int64_t total = static_cast<int64_t>(3) * D * F / 8;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (gid < total) ffn_pack_piece(w_up, w_down, packed, D, F, gate_first, gid, col_scale, fold_act);
}

// Plain SiLU MLP blob (fc1 [F, D], fc2 [D, F]): chunk c (32 hidden units) holds KS fc1 fragments (k-step r; row slots
// 0..15 the chunk's first 16 units, 16..31 its second 16, each in the slot order of up_unit_of_slot) and then 2 * MB fc2
// fragments (k-step (r - KS) / MB of the chunk, row block (r - KS) % MB).
__global__ void mlp_pack_kernel(const bf16_t* __restrict__ w1, const bf16_t* __restrict__ w2, bf16x8* __restrict__ packed,
                                int D, int F) {
  const int64_t total = static_cast<int64_t>(2) * D * F / 8;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (gid >= total) return;
  const int KS = D / 16, MB = D / 32, CFRAG = KS + 2 * MB;
  const int lane = static_cast<int>(gid % 64);
  const int r = static_cast<int>((gid / 64) % CFRAG);
  const int64_t unit0 = gid / 64 / CFRAG * 32;
  const int l32 = lane % 32, hh = lane / 32;
  const bf16_t* src;
  if (r < KS)
    src = w1 + (unit0 + 16 * (l32 / 16) + up_unit_of_slot(l32 & 15)) * D + r * 16 + hh * 8;
  else
    src = w2 + static_cast<int64_t>(((r - KS) % MB) * 32 + l32) * F + unit0 + ((r - KS) / MB) * 16 + hh * 8;
  packed[gid] = *reinterpret_cast<const bf16x8*>(src);
}

// Linear blob: chunk c (64 output features) holds fragments (row block rb, k-step ks) at index rb * KS + ks.
// col_scale (optional, [K]): every weight is multiplied by the factor of its input feature and rounded once - the weight
// of an RMSNorm in front of the layer, folded into the layer (linear(x * r * g) = r * linear_g(x) with linear_g's weights
// w[n, k] * g[k]; the kernel then applies the per-token factor r to its accumulators).
__device__ __forceinline__ void linear_pack_piece(const bf16_t* __restrict__ w, bf16x8* __restrict__ packed, int K,
                                                  int64_t gid, const bf16_t* __restrict__ col_scale = nullptr) {
  const int KS = K / 16, NFRAG = 2 * KS;
  const int lane = static_cast<int>(gid % 64);
  const int f = static_cast<int>((gid / 64) % NFRAG);
  const int64_t chunk = gid / 64 / NFRAG;
  const int l32 = lane % 32, hh = lane / 32;
  const int col = (f % KS) * 16 + hh * 8;
  bf16x8 v = *reinterpret_cast<const bf16x8*>(w + (chunk * kNC + (f / KS) * 32 + l32) * K + col);
  if (col_scale != nullptr) {
    const bf16x8 g = *reinterpret_cast<const bf16x8*>(col_scale + col);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = static_cast<bf16_t>(static_cast<float>(v[e]) * static_cast<float>(g[e]));
  }
  packed[gid] = v;
}

__global__ void linear_pack_kernel(const bf16_t* __restrict__ w, bf16x8* __restrict__ packed, int N, int K,
                                   const bf16_t* __restrict__ col_scale) {
  const int64_t total = static_cast<int64_t>(N) * K / 8;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (gid < total) linear_pack_piece(w, packed, K, gid, col_scale);
}

// All weights of up to kPackBatch backbone blocks in one launch: blockIdx.y = block, blockIdx.x walks the 16-byte
// pieces of its qkv, out and feed-forward blobs in that order.
constexpr int kPackBatch = 16;
struct PackBatch {
  const bf16_t* qkv[kPackBatch];
  const bf16_t* qkv_norm[kPackBatch];  // weight of the RMSNorm in front of the projection (folded into its blob), or null
  const bf16_t* out[kPackBatch];
  const bf16_t* up[kPackBatch];
  const bf16_t* ffn_norm[kPackBatch];  // weight of the RMSNorm in front of the up projection (folded into its blob), or null
  const bf16_t* down[kPackBatch];
  bf16x8* packed_qkv[kPackBatch];
  bf16x8* packed_out[kPackBatch];
  bf16x8* packed_ffn[kPackBatch];
};
__global__ void pack_blocks_kernel(const PackBatch batch, int D, int F, bool fold_act) {
  const int blk = blockIdx.y;
  const int64_t n_qkv = static_cast<int64_t>(3) * D * D / 8, n_out = static_cast<int64_t>(D) * D / 8;
  const int64_t n_ffn = static_cast<int64_t>(3) * D * F / 8;
  int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (gid < n_qkv) return linear_pack_piece(batch.qkv[blk], batch.packed_qkv[blk], D, gid, batch.qkv_norm[blk]);
  gid -= n_qkv;
  if (gid < n_out) return linear_pack_piece(batch.out[blk], batch.packed_out[blk], D, gid);
  gid -= n_out;
  if (gid < n_ffn)
    ffn_pack_piece(batch.up[blk], batch.down[blk], batch.packed_ffn[blk], D, F, 1, gid, batch.ffn_norm[blk], fold_act);
}

// ---- shared pieces ---------------------------------------------------------------------------------------------------

// Number of tokens to process: M, or *n_rows (clamped to M) when a row index is given.
__device__ __forceinline__ int64_t token_count(const TsParams& p) {
  if (p.rows == nullptr) return p.M;
  const int64_t n = *p.n_rows;
  return n < p.M ? n : p.M;
}

// Row of x / residual / out that holds token `tok`. Tokens at or beyond the count are mapped to the last token: they
// compute bit-identical values, so loading and storing them again is benign and every wavefront issues the same
// number of memory operations.
__device__ __forceinline__ int64_t token_row(const TsParams& p, int64_t count, int64_t tok) {
  tok = tok < count ? tok : count - 1;
  return p.rows != nullptr ? static_cast<int64_t>(p.rows[tok]) : tok;
}

// Row of x that holds token `tok`: its own index when one is given, the common one otherwise.
__device__ __forceinline__ int64_t input_row(const TsParams& p, int64_t count, int64_t tok) {
  if (p.x_rows == nullptr) return token_row(p, count, tok);
  tok = tok < count ? tok : count - 1;
  return static_cast<int64_t>(p.x_rows[tok]);
}

// Rows of N tokens at once (token i = tok_of(i)), in two phases: request() issues the N index loads inside ONE test of
// the index pointer and touches none of the loaded values, row() turns entry i into a row number. Whatever the caller
// requests between the two is in flight together with the index (token_row() per token puts every load behind its own
// test of the pointer and a wait behind every load).
template <int N>
struct TokenRows {
  int64_t tok[N];
  int32_t loaded[N];
  bool indexed;
  template <typename F>
  __device__ __forceinline__ void request(const int32_t* index, int64_t count, F tok_of) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const int64_t t = tok_of(i);
      tok[i] = t < count ? t : count - 1;
      loaded[i] = 0;
    }
    indexed = index != nullptr;
    if (indexed) {
#pragma unroll
      for (int i = 0; i < N; ++i) loaded[i] = index[tok[i]];
    }
  }
  // Marks the point up to which the loaded entries stay untouched (the compiler would otherwise widen them right behind
  // their loads, with a wait in front).
  __device__ __forceinline__ void arrive() {
#pragma unroll
    for (int i = 0; i < N; ++i) asm volatile("" : "+v"(loaded[i]));
  }
  __device__ __forceinline__ int64_t row(int i) const { return indexed ? static_cast<int64_t>(loaded[i]) : tok[i]; }
};
template <int N, typename F>
__device__ __forceinline__ void token_rows_batch(const int32_t* index, int64_t count, F tok_of, int64_t (&row)[N]) {
  TokenRows<N> rows;
  rows.request(index, count, tok_of);
  // the entries are awaited here, on this path: left pending, the compiler protects their registers with waits for ALL
  // vector-memory operations wherever the paths of the caller meet again (in front of the MFMAs of every step)
  rows.arrive();
#pragma unroll
  for (int i = 0; i < N; ++i) row[i] = rows.row(i);
}

// Loads the wavefront's token rows as B-operand fragments: lane (l32, hh) holds features 16*ks + 8*hh .. +7 of token
// l32 of each 32-token tile.
// The same from row numbers the caller already holds (r[t]: memory row of token l32 of tile t).
template <int D, int TT>
__device__ __forceinline__ void load_token_rows_at(const TsParams& p, const int64_t (&r)[TT], int hh, bf16x8 (&xf)[TT][D / 16]) {
  constexpr int KS = D / 16;
  if (p.x_plane_shift > 0) {  // feature planes: k-step ks lies in plane (16 * ks) >> shift
    const int sh = p.x_plane_shift;
    const int64_t plane_elems = p.M << sh;
#pragma unroll
    for (int t = 0; t < TT; ++t) {
      const bf16_t* row = p.x + (r[t] << sh) + hh * 8;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        xf[t][ks] = *reinterpret_cast<const bf16x8*>(row + ((ks * 16) >> sh) * plane_elems + ((ks * 16) & ((1 << sh) - 1)));
    }
    return;
  }
#pragma unroll
  for (int t = 0; t < TT; ++t) {
    const bf16_t* row = p.x + r[t] * p.ldx + hh * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) xf[t][ks] = *reinterpret_cast<const bf16x8*>(row + ks * 16);
  }
}

template <int D, int TT>
__device__ __forceinline__ void load_token_rows(const TsParams& p, int64_t count, int64_t tok0, int l32, int hh,
                                                bf16x8 (&xf)[TT][D / 16]) {
  // the row numbers of all tiles first: one memory latency in front of the row loads, not one per tile
  int64_t r[TT];
  token_rows_batch<TT>(p.x_rows != nullptr ? p.x_rows : p.rows, count, [&](int t) { return tok0 + t * 32 + l32; }, r);
  load_token_rows_at<D, TT>(p, r, hh, xf);
}

// RMS-normalises the loaded rows in place: y = bf16( x * rsqrt(mean(x^2) + eps) * w ), w read from its LDS copy.
// folded: the norm's weight is part of the layer that consumes the rows; only the per-token factor is applied.
template <int D, int TT>
__device__ __forceinline__ void normalize_tokens(float eps, const bf16_t* norm_w_lds, int hh, bf16x8 (&xf)[TT][D / 16],
                                                 bool folded = false) {
  constexpr int KS = D / 16;
  float scale[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) {
    float ss = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float v = static_cast<float>(xf[t][ks][e]);
        ss += v * v;
      }
    ss += __shfl_xor(ss, 32, kWave);
    scale[t] = rsqrtf(ss * (1.0f / D) + eps);
  }
  // Make the packed rows opaque here: otherwise the compiler keeps all D fp32 copies from the first sweep alive for
  // the second one, which does not fit the register file next to the accumulators.
#pragma unroll
  for (int t = 0; t < TT; ++t)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(xf[t][ks]));
  if (folded) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
#pragma unroll
      for (int t = 0; t < TT; ++t) {
#pragma unroll
        for (int e = 0; e < 8; ++e) xf[t][ks][e] = static_cast<bf16_t>(static_cast<float>(xf[t][ks][e]) * scale[t]);
        asm volatile("" : "+v"(xf[t][ks]));
      }
    return;
  }
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const bf16x8 wv = *reinterpret_cast<const bf16x8*>(norm_w_lds + ks * 16 + hh * 8);
#pragma unroll
    for (int t = 0; t < TT; ++t) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        xf[t][ks][e] = static_cast<bf16_t>(static_cast<float>(xf[t][ks][e]) * scale[t] * static_cast<float>(wv[e]));
      asm volatile("" : "+v"(xf[t][ks]));
    }
  }
}

// rsqrt(mean(x^2) + eps) of the loaded rows, per lane for its token of each tile; the rows themselves stay as they are
// (the norm's weight is part of the packed layer, the factor goes to the accumulators). The squares are summed two
// elements per instruction (v_dot2_f32_bf16).
template <int D, int TT>
__device__ __forceinline__ void token_rstd(float eps, const bf16x8 (&xf)[TT][D / 16], float (&rstd)[TT]) {
  typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
#pragma unroll
  for (int t = 0; t < TT; ++t) {
    float ss = 0.f;
#pragma unroll
    for (int ks = 0; ks < D / 16; ++ks)
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        const bf16x2 pair = {xf[t][ks][e], xf[t][ks][e + 1]};
        ss = __builtin_amdgcn_fdot2_f32_bf16(pair, pair, ss, false);
      }
    ss += __shfl_xor(ss, 32, kWave);
    rstd[t] = rsqrtf(ss * (1.0f / D) + eps);
  }
}

// Bias values of a 64-feature chunk in accumulator order: piece rb*4 + jq holds features rb*32 + jq*8 + hh*4 .. +3.
__device__ __forceinline__ void read_chunk_bias(const bf16_t* bias_lds, int hh, bf16x4 (&bv)[8]) {
#pragma unroll
  for (int q = 0; q < 8; ++q) bv[q] = *reinterpret_cast<const bf16x4*>(bias_lds + (q / 4) * 32 + (q % 4) * 8 + hh * 4);
}

// The same from a float32 copy of the bias (no widening per value in the epilogue).
__device__ __forceinline__ void read_chunk_bias(const float* bias_lds, int hh, f32x4 (&bv)[8]) {
#pragma unroll
  for (int q = 0; q < 8; ++q) bv[q] = *reinterpret_cast<const f32x4*>(bias_lds + (q / 4) * 32 + (q % 4) * 8 + hh * 4);
}

// Writes two 32-feature accumulator blocks (64 features) of one 32-token tile into the wavefront's epilogue tile,
// adding the bias and rounding to bf16. Accumulator register jq*4 + e of lane (l32, hh) is feature jq*8 + hh*4 + e.
template <typename BiasVec>  // bf16x4 or f32x4 pieces
__device__ __forceinline__ void tile_to_lds(uint8_t* tile, const f32x16& a0, const f32x16& a1, const BiasVec (&bv)[8],
                                            int l32, int hh, float scale = 1.0f) {
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) {
#pragma unroll
    for (int jq = 0; jq < 4; ++jq) {
      const int col = rb * 32 + jq * 8 + hh * 4;
      bf16x4 ov;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        ov[e] = static_cast<bf16_t>(fmaf(rb == 0 ? a0[jq * 4 + e] : a1[jq * 4 + e], scale, static_cast<float>(bv[rb * 4 + jq][e])));
      *reinterpret_cast<bf16x4*>(tile + l32 * kStageRow + col * 2) = ov;
    }
  }
}

// tile_to_lds that also returns the sum of squares of the lane's 32 rounded values (half of its token's 64 features).
__device__ __forceinline__ float tile_to_lds_sumsq(uint8_t* tile, const f32x16& a0, const f32x16& a1,
                                                   const bf16x4 (&bv)[8], int l32, int hh, float scale = 1.0f) {
  float ss = 0.f;
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) {
#pragma unroll
    for (int jq = 0; jq < 4; ++jq) {
      const int col = rb * 32 + jq * 8 + hh * 4;
      bf16x4 ov;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        ov[e] = static_cast<bf16_t>(fmaf(rb == 0 ? a0[jq * 4 + e] : a1[jq * 4 + e], scale, static_cast<float>(bv[rb * 4 + jq][e])));
        const float r = static_cast<float>(ov[e]);
        ss = fmaf(r, r, ss);
      }
      *reinterpret_cast<bf16x4*>(tile + l32 * kStageRow + col * 2) = ov;
    }
  }
  return ss;
}

// Sum of a value and the one held by lane ^ 32.
__device__ __forceinline__ float half_wave_pair_sum(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, static_cast<uint32_t>(r[0])) + __builtin_bit_cast(float, static_cast<uint32_t>(r[1]));
}

// Reads the epilogue tile back row-wise (lane -> token 8*i + lane/8, features 8*(lane%8) .. +7), adds the residual
// pieces loaded earlier and stores 16 bytes per lane: every 128-byte row segment is written by 8 consecutive lanes.
// prow[i] is the memory row of token 8*i + lane/8 of the tile, live[i] whether that token exists.
// head_w (optional): the lane's share of the dot product of each stored row with head_w is added to hdot[i].
template <bool RES>
__device__ __forceinline__ void tile_to_global(const uint8_t* tile, bf16_t* out, int64_t ldo, const int64_t (&prow)[4],
                                               const bool (&live)[4], int col0, const bf16x8 (&res)[4], int lane,
                                               const bf16_t* head_w, float (&hdot)[4]) {
  bf16x8 hw;
  if (head_w != nullptr) {
    hw = *reinterpret_cast<const bf16x8*>(head_w + col0 + (lane % 8) * 8);
    // awaited here, on the path that loads it: otherwise the wait (for every vector-memory operation, the stores of the
    // tile included) lands where the paths meet again, in front of the next piece of every launch
    asm volatile("" : "+v"(hw));
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = i * 8 + lane / 8;
    bf16x8 v = *reinterpret_cast<const bf16x8*>(tile + row * kStageRow + (lane % 8) * 16);
    if (RES) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        v[e] = static_cast<bf16_t>(static_cast<float>(v[e]) + static_cast<float>(res[i][e]));
    }
    if (live[i]) *reinterpret_cast<bf16x8*>(out + prow[i] * ldo + col0 + (lane % 8) * 8) = v;
    if (head_w != nullptr) {
#pragma unroll
      for (int e = 0; e < 8; ++e) hdot[i] = fmaf(static_cast<float>(v[e]), static_cast<float>(hw[e]), hdot[i]);
    }
  }
}

__device__ __forceinline__ void load_residual(const bf16_t* residual, int64_t ldr, const int64_t (&prow)[4], int col0,
                                              bf16x8 (&res)[4], int lane) {
#pragma unroll
  for (int i = 0; i < 4; ++i)
    res[i] = *reinterpret_cast<const bf16x8*>(residual + prow[i] * ldr + col0 + (lane % 8) * 8);
}

// ------------------------------------------------------------------------------------------------------------------
// Fused RMSNorm -> up -> SiLU-gate -> down -> + residual
//
// A chunk is 16 hidden units. Its up-projection fragment has 32 rows: 16 gate rows on top of the 16 matching value
// rows, so ONE accumulator (16 registers per lane) holds g in registers 0..7 and u in registers 8..15 for the same
// eight hidden units of the lane's token. silu(g) * u of those eight is exactly one B-operand fragment (k = 16) of
// the down projection. Two chunks are staged and consumed per barrier.
// LDS: [2 or 3 weight buffers][b_up (2F) | b_down (D) | norm weight (D) | OUTP: projection bias (D)]; after the main
// loop the weight buffers hold the epilogue tiles.
//
// OUTP: the attention output projection and its residual run in front, in the same registers. p.x is then the
// attention output A, p.residual the block input h, and the kernel evaluates
//   x1 = bf16( bf16(A W0^T + b0) + h ),   out = bf16( x1 + down(silu(gate) * value) + b_down ),  gate, value = up(rmsnorm(x1))
// The projection is formed transposed like the down projection, X1^T[feature, token] = W0 A^T, into the accumulators of
// the final result; the packed W0 streams through weight buffers 1 and 2 one 64-feature chunk at a time. Bias and h
// are added per chunk in accumulator order, the rounded x1 stays in the accumulators as the start value of the down
// projection (so x1 never exists in memory and the final sum is rounded once), and its normalised copy is turned into
// B-operand fragments with one half-wavefront exchange per register pair: the accumulator holds 4-feature runs of a
// token per lane, a fragment needs 8-feature runs, and lanes l and l ^ 32 own the two halves of each run.
// Replaces the out projection + residual and the feed-forward half of UnifiedInteractionBlock.forward
// (experiments/symbiosis/backbone.py:60-67) in one pass over the tokens.
//
// GATE (with OUTP): the projected update is multiplied by a sigmoid gate before it joins the residual stream,
//   x1 = bf16( h + bf16( bf16(sigmoid(g)) * bf16(A W0^T + b0) ) ),
// g = p.gate, the gate layer's output in 16 bits (TokenFormerBlock.forward, experiments/tokenformer/model.py:209-214:
// the gate layer reads the normalised block input, which only the projection kernel in front of attention holds, so
// it arrives as a tensor). Its pieces of a chunk are requested behind the chunk's MFMAs, into the registers the weight
// fragments have left, so the variant takes no registers of its own.
// ------------------------------------------------------------------------------------------------------------------
template <int D, int TT, int NWAVES, int CPB, bool DEFER, bool OUTP, bool GATE = false, bool GLU = true, bool FOLD = false>
__global__ __launch_bounds__(NWAVES * kWave, TT == 1 ? 2 : 1) void swiglu_ffn_kernel(const TsParams p) {
  static_assert(!GATE || OUTP, "the gate belongs to the projection in front");
  static_assert(!FOLD || GLU, "the folded constants belong to the gated form");
  constexpr int kTokPerWg = NWAVES * 32 * TT;  // TT token tiles of 32 per wavefront
  constexpr int KS = D / 16;             // k-steps of the up projection = up fragments per chunk
  constexpr int MB = D / 32;             // 32-feature row blocks of the down projection
  // GLU: a chunk is 16 hidden units (16 gated rows + 16 partner rows) and one k-step of the down projection. Plain MLP
  // (!GLU: down(silu(up(x)))): all 32 rows of a chunk's fragment are hidden units, whose activations fill two k-steps.
  constexpr int DK = GLU ? 1 : 2;        // k-steps of the down projection per chunk
  constexpr int NDOWN = DK * MB;         // down fragments per chunk
  constexpr int CFRAG = KS + NDOWN;      // fragments per chunk
  constexpr int NFRAG = CPB * CFRAG;     // fragments per barrier step
  constexpr int FPW = NFRAG / NWAVES;    // fragments staged per wavefront
  static_assert(NFRAG % NWAVES == 0, "fragments must divide over the wavefronts");
  constexpr int NBUF = DEFER ? 3 : 2;    // weight buffers in LDS
  static_assert(MB == 4 || MB == 8, "the activation pairs are spread over the down-projection MFMAs");
  static_assert(NBUF * NFRAG * kFrag >= NWAVES * kStageWave, "epilogue tiles must fit in the weight buffers");
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  bf16_t* bias_lds = reinterpret_cast<bf16_t*>(smem + NBUF * NFRAG * kFrag);

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);  // wavefront-uniform, kept in a scalar register
  const int lane = tid % kWave;
  const int l32 = lane % 32;
  const int hh = lane / 32;
  // Work split: workgroups [0, base) take one full tile of kTokPerWg tokens each, base = the largest multiple of
  // p.units not above the number of complete tiles; the tokens that remain (fewer than p.units tiles) are spread
  // evenly over the next p.units workgroups in slices of whole 32-token wavefront tiles, so that the last round keeps
  // every compute unit busy for a fraction of a tile instead of some of them for a whole one.
  const int64_t count = token_count(p);
  const int64_t base = count / kTokPerWg / p.units * p.units;
  int64_t wg_tok0;
  int wg_ntok;
  if (static_cast<int64_t>(blockIdx.x) < base) {
    wg_tok0 = static_cast<int64_t>(blockIdx.x) * kTokPerWg;
    wg_ntok = kTokPerWg;
  } else {
    const int64_t rest = count - base * kTokPerWg;  // < p.units * kTokPerWg
    const int64_t per = ((rest + p.units - 1) / p.units + 32 * TT - 1) / (32 * TT) * (32 * TT);
    const int64_t j = static_cast<int64_t>(blockIdx.x) - base;
    wg_tok0 = base * kTokPerWg + j * per;
    const int64_t left = count - wg_tok0;
    wg_ntok = static_cast<int>(left < per ? left : per);
    if (j >= p.units || wg_ntok <= 0) return;  // whole workgroup: no tokens left for it
  }
  // A wavefront whose tile lies beyond the workgroup's slice only helps staging the weights.
  const bool active = wave * (32 * TT) < wg_ntok;
  const int64_t tok0 = wg_tok0 + wave * (32 * TT);
  const int F = p.F;
  const int UPB = GLU ? 2 * F : F;  // entries of the staged first-layer bias
  const int nsteps = F / (kHU * DK * CPB);

  // Source address of a staged fragment = wavefront-uniform base (scalar registers) + a 32-bit per-lane byte offset.
  //   packed:   blob + (step * NFRAG + f) KB + 16 * lane
  //   unpacked: up fragment (chunk q, k-step r): row slot l32 -> W_up row [value ? F : 0] + unit0 + unit(l32 % 16),
  //             cols r*16 + hh*8; down fragment (chunk q, block mb): W_down row mb*32 + l32, cols unit0 + hh*8
  const char* w_up_bytes = reinterpret_cast<const char*>(p.w1);
  const char* w_down_bytes = reinterpret_cast<const char*>(p.w2);
  auto stage = [&](int step, int buf) {
    // The lane offsets are recomputed from an opaque copy of the lane id on every call: as loop invariants they
    // would be kept live (and spilled) across the whole main loop.
    int ln = lane;
    asm volatile("" : "+v"(ln));
    uint8_t* base = smem + buf * (NFRAG * kFrag) + wave * (FPW * kFrag);
    if (p.packed) {
      const char* src = w_up_bytes + (static_cast<int64_t>(step) * NFRAG + wave * FPW) * kFrag;  // scalar registers
      const uint32_t lane_off = static_cast<uint32_t>(ln * 16);
#pragma unroll
      for (int i = 0; i < FPW; ++i) lds_dma16_offset(src + i * kFrag, lane_off, base + i * kFrag);
      return;
    }
    if constexpr (!GLU) return;  // the plain MLP takes packed weights only (checked on the host)
    const int s32 = ln & 31, shh = ln >> 5;
    const uint32_t up_lane_off =
        static_cast<uint32_t>(((((s32 < 16) == (p.gate_first != 0) ? 0 : F) + up_unit_of_slot(s32 & 15)) * D + shh * 8) * 2);
    const uint32_t down_lane_off = static_cast<uint32_t>((s32 * F + shh * 8) * 2);
#pragma unroll
    for (int i = 0; i < FPW; ++i) {
      const int f = wave * FPW + i;  // wavefront-uniform
      const int q = f / CFRAG;       // chunk inside the step
      const int r = f % CFRAG;
      const int64_t unit0 = static_cast<int64_t>(step * CPB + q) * kHU;
      if (r < KS)
        lds_dma16(w_up_bytes + (unit0 * D + r * 16) * 2 + up_lane_off, base + i * kFrag);
      else
        lds_dma16(w_down_bytes + (static_cast<int64_t>(r - KS) * 32 * F + unit0) * 2 + down_lane_off, base + i * kFrag);
    }
  };

  // OUTP: chunk c of the packed projection (2 * KS fragments) goes to weight buffer 1 + (c & 1).
  [[maybe_unused]] auto stage_proj = [&](int c, int buf) {
    constexpr int CF = 2 * KS, CFW = CF / NWAVES;
    static_assert(CF % NWAVES == 0 && CF <= NFRAG, "a projection chunk is staged by all wavefronts into one buffer");
    int ln = lane;
    asm volatile("" : "+v"(ln));
    uint8_t* base = smem + buf * (NFRAG * kFrag) + wave * (CFW * kFrag);
    const char* src = reinterpret_cast<const char*>(p.w0) + (static_cast<int64_t>(c) * CF + wave * CFW) * kFrag;
    const uint32_t lane_off = static_cast<uint32_t>(ln * 16);
#pragma unroll
    for (int i = 0; i < CFW; ++i) lds_dma16_offset(src + i * kFrag, lane_off, base + i * kFrag);
  };

  stage(0, 0);
  if constexpr (OUTP) stage_proj(0, 1);
  // The token rows (a row-index load, then the rows) are requested before the bias vectors are staged, so that the two
  // chains of memory latencies run side by side; OUTP: so is the row number of the block input read by the projection.
  // The workgroup's start is a chain of memory latencies with nothing to hide them behind (it owns the compute unit), so
  // everything that does not depend on something else is requested at once: the row numbers of the wavefront's tokens and
  // the bias vectors first (their values stay in registers), then - one latency later - the token rows, and only then
  // are the bias vectors written to LDS. Two latencies instead of one per vector.
  TokenRows<TT> out_rows, x_rows;  // rows of the wavefront's tokens in residual / out, and in x when x has an index of its own
  out_rows.request(p.rows, count, [&](int t) { return tok0 + t * 32 + l32; });
  x_rows.request(p.x_rows, count, [&](int t) { return tok0 + t * 32 + l32; });
  constexpr int kThreadsWg = NWAVES * kWave;
  constexpr int UB = 4;  // first-layer bias entries per thread held in registers (F <= UB * threads / 2 needs no second round)
  // First-layer bias in fragment row order: entry chunk * 32 + m belongs to row slot m of the chunk's up fragment (GLU: slots
  // 0..15 the gated half, 16..31 the other half; plain MLP: slots 0..15 the chunk's first 16 units, 16..31 the others), so
  // lane l32 of a wavefront finds the bias of its fragment row at chunk * 32 + l32. Zeros when there is no bias.
  auto up_bias_src = [&](int i) -> int {  // index into b1 of staged entry i
    const int m = i % 32;
    if constexpr (GLU)
      return ((m < 16) == (p.gate_first != 0) ? 0 : F) + (i / 32) * kHU + up_unit_of_slot(m % 16);
    else
      return (i / 32) * 32 + 16 * (m / 16) + up_unit_of_slot(m % 16);
  };
  bf16_t up_bias_regs[UB];
#pragma unroll
  for (int u = 0; u < UB; ++u) up_bias_regs[u] = static_cast<bf16_t>(0.f);
  if (p.b1 != nullptr) {
#pragma unroll
    for (int u = 0; u < UB; ++u) {
      const int i = tid + u * kThreadsWg;
      up_bias_regs[u] = p.b1[up_bias_src(i < UPB ? i : UPB - 1)];
      if constexpr (FOLD)  // the packed layer's constants (see ffn_pack_piece), one more rounding of the bias
        up_bias_regs[u] = static_cast<bf16_t>(static_cast<float>(up_bias_regs[u]) * (i % 32 < 16 ? kFoldGate : kFoldValue));
    }
  }
  const int vec_at = tid * 8 < D ? tid * 8 : D - 8;  // the D-wide vectors: 16 bytes per thread, the first D / 8 threads store
  bf16x8 b2_regs, normw_regs, b0_regs;
#pragma unroll
  for (int e = 0; e < 8; ++e) b2_regs[e] = normw_regs[e] = b0_regs[e] = static_cast<bf16_t>(0.f);
  if (p.b2 != nullptr) b2_regs = *reinterpret_cast<const bf16x8*>(p.b2 + vec_at);
  if (p.norm_w != nullptr) normw_regs = *reinterpret_cast<const bf16x8*>(p.norm_w + vec_at);
  if constexpr (OUTP) {
    if (p.b0 != nullptr) b0_regs = *reinterpret_cast<const bf16x8*>(p.b0 + vec_at);
  }
  out_rows.arrive();
  x_rows.arrive();
  int64_t hrow_index[TT];  // OUTP: where the projection reads the block input
  int64_t xrow_index[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) {
    hrow_index[t] = out_rows.row(t);
    xrow_index[t] = p.x_rows != nullptr ? x_rows.row(t) : hrow_index[t];
  }
  // (wavefronts without tokens load as well - their row numbers are clamped to the last token: a load behind a branch leaves
  // its registers pending where the paths meet, and the compiler then waits for them again in every later block of code)
  bf16x8 xf[TT][KS];
  load_token_rows_at<D, TT>(p, xrow_index, hh, xf);
#pragma unroll
  for (int u = 0; u < UB; ++u) {
    const int i = tid + u * kThreadsWg;
    if (i < UPB) bias_lds[i] = up_bias_regs[u];
  }
  for (int i = tid + UB * kThreadsWg; i < UPB; i += kThreadsWg) {  // wider hidden layers: the rest, one entry at a time
    bf16_t b = p.b1 != nullptr ? p.b1[up_bias_src(i)] : static_cast<bf16_t>(0.f);
    if constexpr (FOLD) b = static_cast<bf16_t>(static_cast<float>(b) * (i % 32 < 16 ? kFoldGate : kFoldValue));
    bias_lds[i] = b;
  }
  if (tid * 8 < D) {
    *reinterpret_cast<bf16x8*>(bias_lds + UPB + vec_at) = b2_regs;
    if (p.norm_w != nullptr) *reinterpret_cast<bf16x8*>(bias_lds + UPB + D + vec_at) = normw_regs;
    if constexpr (OUTP) *reinterpret_cast<bf16x8*>(bias_lds + UPB + 2 * D + vec_at) = b0_regs;
  }

  f32x16 oacc[TT][MB];
#pragma unroll
  for (int t = 0; t < TT; ++t)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int j = 0; j < 16; ++j) oacc[t][mb][j] = 0.f;

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  // The token rows have landed; the compiler is told so here, on the one path every wavefront takes: used for the first
  // time inside the `if (active)` blocks below, they would count as pending again wherever such a block ends, and every
  // later block would wait for them anew (with counts that also cover the transfers and loads issued by hand).
#pragma unroll
  for (int t = 0; t < TT; ++t)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(xf[t][ks]));
  __syncthreads();
  if (!OUTP && active && p.norm_w != nullptr) normalize_tokens<D, TT>(p.eps, bias_lds + UPB + D, hh, xf, p.norm_folded != 0);

  // One barrier step = CPB chunks = NFRAG fragments, consumed in their LDS order: per chunk KS up fragments, then MB
  // down fragments. Fragment reads run P fragments ahead of their MFMAs through a ring of P registers sets; the two
  // bias vectors of a chunk are read just before the chunk's first fragment, so they have landed (operations
  // complete in order) whenever a later fragment has.
  constexpr int P = 4;
  const uint32_t smem_off = lds_offset(smem) + lane * 16;
  const uint32_t bias_off = lds_offset(bias_lds) + l32 * 2;
  // The up-projection bias enters through the matrix unit: one extra MFMA per chunk whose A operand carries the bias of
  // fragment row l32 at k = 0 and whose B operand is 1 at k = 0 and 0 elsewhere (k = 0..7 live in lanes 0..31).
  u32x4 ones_bits = {hh == 0 ? 0x3f80u : 0u, 0u, 0u, 0u};
  asm volatile("" : "+v"(ones_bits));
  const bf16x8 ones = __builtin_bit_cast(bf16x8, ones_bits);

  if constexpr (OUTP) {
    static_assert(DEFER, "the projection chunks use weight buffers 1 and 2");
    constexpr int NCH = D / kNC;  // 64-feature chunks of the projection
    constexpr int CF = 2 * KS;    // fragments of a chunk: (row block rb, k-step ks) at rb * KS + ks
    const bf16_t* b0_lds = bias_lds + UPB + 2 * D;
    float ss[TT];
    const bf16_t* hrow[TT];
    [[maybe_unused]] const bf16_t* grow[TT];
#pragma unroll
    for (int t = 0; t < TT; ++t) {
      ss[t] = 0.f;
      // GATE: block input in accumulator order (4-feature runs); otherwise as B-operand fragments (8-feature runs)
      hrow[t] = p.residual + hrow_index[t] * p.ldr + (GATE ? hh * 4 : hh * 8);
      if constexpr (GATE) grow[t] = p.gate + hrow_index[t] * p.ldg + hh * 4;
    }
    // Without a gate the bias and the block input join the projection inside the matrix unit: per 32-feature row block
    // one more product multiplies a bias fragment with the ones fragment of the feed-forward's bias trick, and - after
    // the rounding of the layer output - two more multiply an identity fragment (row l32 of the block = k index l32 of a
    // 32-feature slice) with the block input held as B-operand fragments, which adds h exactly in fp32. The roundings stay
    // those of the 16-bit evaluation layer by layer, x1 = bf16(bf16(A W0^T + b0) + h); what is left for the vector unit
    // per element is the two roundings with their widening back to fp32 and half a dot-product instruction for the
    // norm's sum of squares (3.5 instead of 8 instructions per element).
    [[maybe_unused]] bf16x8 ident[2];
    if constexpr (!GATE) {
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const int e0 = l32 - 16 * k - 8 * hh;  // element of this lane's eight k slots that is the row's own feature
        u32x4 bits = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int d = 0; d < 4; ++d)
          bits[d] = (e0 >> 1) == d && e0 >= 0 && e0 < 8 ? ((e0 & 1) ? 0x3f800000u : 0x00003f80u) : 0u;
        ident[k] = __builtin_bit_cast(bf16x8, bits);
      }
    }
    static_for<NCH>([&](auto cc) {
      constexpr int c = decltype(cc)::value;
      // GATE: block input of this chunk's 64 features in accumulator order: piece rb*4 + jq = features rb*32 + jq*8 + hh*4 .. +3
      [[maybe_unused]] bf16x4 hv[TT][GATE ? 8 : 1];
      // !GATE: the same 64 features as four B-operand fragments (k-steps 4c .. 4c+3 of the model width)
      [[maybe_unused]] bf16x8 hf[TT][GATE ? 1 : 4];
      [[maybe_unused]] uint32_t b0row[2] = {0u, 0u};  // !GATE: bias of this lane's feature row of the chunk's two row blocks
      if (active) {
#pragma unroll
        for (int t = 0; t < TT; ++t) {
          if constexpr (GATE) {
#pragma unroll
            for (int q = 0; q < 8; ++q)
              hv[t][q] = *reinterpret_cast<const bf16x4*>(hrow[t] + c * kNC + (q / 4) * 32 + (q % 4) * 8);
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)  // requested by hand: the wait behind the chunk's MFMAs is counted by hand as well
              asm volatile("global_load_dwordx4 %0, %1, off offset:%2"
                           : "=v"(hf[t][j])
                           : "v"(hrow[t]), "n"((c * kNC + j * 16) * 2)
                           : "memory");
          }
        }
        if constexpr (!GATE) {
#pragma unroll
          for (int rb = 0; rb < 2; ++rb)
            b0row[rb] = static_cast<uint32_t>(reinterpret_cast<const uint16_t*>(b0_lds)[c * kNC + rb * 32 + l32]);
        }
      }
      if constexpr (c + 1 < NCH) stage_proj(c + 1, 1 + ((c + 1) & 1));
      if (active) {
        const uint32_t wb0 = smem_off + (1 + (c & 1)) * (NFRAG * kFrag);
        bf16x8 pring[P];
        static_for<P>([&](auto ic) { lds_read_frag<decltype(ic)::value * kFrag>(pring[decltype(ic)::value], wb0); });
        static_for<CF>([&](auto ic) {
          constexpr int i = decltype(ic)::value;
          constexpr int after = P - 1 < CF - 1 - i ? P - 1 : CF - 1 - i;
          lds_wait_frag<after>(pring[i % P]);
#pragma unroll
          for (int t = 0; t < TT; ++t)
            oacc[t][2 * c + i / KS] =
                __builtin_amdgcn_mfma_f32_32x32x16_bf16(pring[i % P], xf[t][i % KS], oacc[t][2 * c + i / KS], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
          if constexpr (i + P < CF) lds_read_frag<(i + P) * kFrag>(pring[i % P], wb0);
        });
        if constexpr (!GATE) {
          // The block input of this chunk, requested in front of the next chunk's weight transfers: awaited by hand, with
          // those transfers left in flight. (The compiler's own count does not know the transfers, so its wait for these
          // registers - placed at their first use - would be a wait for the transfers as well, with the epilogue
          // arithmetic of this chunk still to come.)
          constexpr int kNewer = c + 1 < NCH ? CF / NWAVES : 0;  // transfers of stage_proj(c + 1) per wavefront
#pragma unroll
          for (int t = 0; t < TT; ++t)  // the pieces are tied to the wait so that their consumers cannot move above it
            asm volatile("s_waitcnt vmcnt(%4)"
                         : "+v"(hf[t][0]), "+v"(hf[t][1]), "+v"(hf[t][2]), "+v"(hf[t][3])
                         : "n"(kNewer)
                         : "memory");
        }
        if constexpr (GATE) {
          // x1 = bf16( bf16(sigmoid(g)) * bf16(projection + b0) + h ), kept in the accumulators; sum of squares for the
          // norm that follows
          bf16x4 bv[8];
          read_chunk_bias(b0_lds + c * kNC, hh, bv);
          bf16x4 gv[TT][8];
#pragma unroll
          for (int t = 0; t < TT; ++t)
#pragma unroll
            for (int q = 0; q < 8; ++q)
              gv[t][q] = *reinterpret_cast<const bf16x4*>(grow[t] + c * kNC + (q / 4) * 32 + (q % 4) * 8);
#pragma unroll
          for (int t = 0; t < TT; ++t)
#pragma unroll
            for (int q = 0; q < 8; ++q)
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const float a = oacc[t][2 * c + q / 4][(q % 4) * 4 + e];
                float lin = static_cast<float>(static_cast<bf16_t>(a + static_cast<float>(bv[q][e])));
                const float g = static_cast<float>(gv[t][q][e]);
                const float sg = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g));
                lin = static_cast<float>(static_cast<bf16_t>(static_cast<float>(static_cast<bf16_t>(sg)) * lin));
                const float x1 = static_cast<float>(static_cast<bf16_t>(lin + static_cast<float>(hv[t][q][e])));
                oacc[t][2 * c + q / 4][(q % 4) * 4 + e] = x1;
                ss[t] = fmaf(x1, x1, ss[t]);
              }
        } else {
          // + b0 through the matrix unit, lin = bf16(accumulator); + h through the matrix unit (exact in fp32),
          // x1 = bf16(accumulator), kept in the accumulators as fp32
          typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
#pragma unroll
          for (int t = 0; t < TT; ++t)
#pragma unroll
            for (int rb = 0; rb < 2; ++rb) {
              f32x16& acc = oacc[t][2 * c + rb];
              const u32x4 bias_bits = {b0row[rb], 0u, 0u, 0u};
              acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, bias_bits), ones, acc, 0, 0, 0);
#pragma unroll
              for (int j = 0; j < 16; j += 2) {  // one packed conversion per pair, widened back from the packed word
                const bf16x2 pair = {static_cast<bf16_t>(acc[j]), static_cast<bf16_t>(acc[j + 1])};
                uint32_t bits = __builtin_bit_cast(uint32_t, pair);
                asm("" : "+v"(bits));  // opaque: the optimiser otherwise splits the pair into two conversions again
                acc[j] = __builtin_bit_cast(float, bits << 16);
                acc[j + 1] = __builtin_bit_cast(float, bits & 0xffff0000u);
              }
              acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ident[0], hf[t][2 * rb], acc, 0, 0, 0);
              acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ident[1], hf[t][2 * rb + 1], acc, 0, 0, 0);
#pragma unroll
              for (int j = 0; j < 16; j += 2) {
                const bf16x2 pair = {static_cast<bf16_t>(acc[j]), static_cast<bf16_t>(acc[j + 1])};
                uint32_t bits = __builtin_bit_cast(uint32_t, pair);
                asm("" : "+v"(bits));  // opaque: the optimiser otherwise splits the pair into two conversions again
                acc[j] = __builtin_bit_cast(float, bits << 16);
                acc[j + 1] = __builtin_bit_cast(float, bits & 0xffff0000u);
                const bf16x2 rounded = __builtin_bit_cast(bf16x2, bits);
                ss[t] = __builtin_amdgcn_fdot2_f32_bf16(rounded, rounded, ss[t], false);
              }
            }
        }
      }
      // the next chunk has landed (and, with the first wait, the first step of the feed-forward weights)
      vm_wait<0>();
      __syncthreads();
    });
    if (active) {
      // rmsnorm(x1) as B-operand fragments. k-step ks covers features 16*ks .. +15 = the 8-feature groups jq = 2*(ks%2)
      // and jq + 1 of row block ks / 2; the lower half-wavefront needs all of the first group, the upper half all of
      // the second, and each half holds 4 features of both.
      const bf16_t* nw_lds = bias_lds + UPB + D;
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        const float scale = p.norm_w != nullptr ? rsqrtf(half_wave_pair_sum(ss[t]) * (1.0f / D) + p.eps) : 1.0f;
        static_for<KS>([&](auto kc) {
          constexpr int ks = decltype(kc)::value;
          constexpr int mb = ks / 2, jq = 2 * (ks % 2);
          bf16x4 lo, hi;
          if (p.norm_w != nullptr && p.norm_folded) {  // the norm's weight is part of the packed up projection
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              lo[e] = static_cast<bf16_t>(oacc[t][mb][jq * 4 + e] * scale);
              hi[e] = static_cast<bf16_t>(oacc[t][mb][(jq + 1) * 4 + e] * scale);
            }
          } else if (p.norm_w != nullptr) {
            const bf16x4 wl = *reinterpret_cast<const bf16x4*>(nw_lds + mb * 32 + jq * 8 + hh * 4);
            const bf16x4 wh = *reinterpret_cast<const bf16x4*>(nw_lds + mb * 32 + (jq + 1) * 8 + hh * 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              lo[e] = static_cast<bf16_t>(oacc[t][mb][jq * 4 + e] * scale * static_cast<float>(wl[e]));
              hi[e] = static_cast<bf16_t>(oacc[t][mb][(jq + 1) * 4 + e] * scale * static_cast<float>(wh[e]));
            }
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              lo[e] = static_cast<bf16_t>(oacc[t][mb][jq * 4 + e]);
              hi[e] = static_cast<bf16_t>(oacc[t][mb][(jq + 1) * 4 + e]);
            }
          }
          const u32x2 ul = __builtin_bit_cast(u32x2, lo), uh = __builtin_bit_cast(u32x2, hi);
          // swap: result 0 = (lower lanes of the first, lower lanes of the second), result 1 = the upper lanes
          const auto r0 = __builtin_amdgcn_permlane32_swap(ul[0], uh[0], false, false);
          const auto r1 = __builtin_amdgcn_permlane32_swap(ul[1], uh[1], false, false);
          const u32x4 frag = {static_cast<uint32_t>(r0[0]), static_cast<uint32_t>(r1[0]), static_cast<uint32_t>(r0[1]),
                              static_cast<uint32_t>(r1[1])};
          xf[t][ks] = __builtin_bit_cast(bf16x8, frag);
        });
      }
    }
  }

  // DEFER: the down projection of a chunk is issued one chunk late, interleaved with the SiLU arithmetic of the next
  // chunk (MFMA j of the old chunk, then two gated values of the new one), so the matrix unit has work while the
  // wavefront evaluates the activation. hb is the gated hidden state whose down projection is pending; before the
  // first chunk it is zero and the (finite) fragments it is multiplied with do not matter.
  bf16x8 hb[TT][DK];
#pragma unroll
  for (int t = 0; t < TT; ++t)
#pragma unroll
    for (int k = 0; k < DK; ++k)
#pragma unroll
      for (int e = 0; e < 8; ++e) hb[t][k][e] = static_cast<bf16_t>(0.f);
  // Activation of accumulator register e of a chunk (e < 8 * DK): the B-operand element it becomes.
  auto activate = [](const f32x16& gu, int e) -> bf16_t {
    if constexpr (FOLD)  // gu[e] = -log2(e) g, gu[8 + e] = -ln(2) u: their product is g u
      return static_cast<bf16_t>(gu[e] * gu[8 + e] * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(gu[e])));
    return static_cast<bf16_t>(GLU ? silu_f(gu[e]) * gu[8 + e] : silu_f(gu[e]));
  };
  int buf = 0;
  uint32_t wb_prev = smem_off;
  for (int step = 0; step < nsteps; ++step) {
    // The target buffer was last read before the barrier that ended the previous step (with DEFER: its down
    // fragments at the start of the previous step, hence three buffers).
    if (step + 1 < nsteps) stage(step + 1, buf == NBUF - 1 ? 0 : buf + 1);
    const uint32_t wb = smem_off + buf * (NFRAG * kFrag);
    const uint32_t bias_step = bias_off + step * (CPB * 32 * 2);
    if (active) {
    bf16x8 ring[P];
    uint32_t brow[CPB];  // bias of this lane's fragment row, one per chunk, zero-extended bf16
    f32x16 gu[TT];
    bf16x8 hb_new[TT][DK];
    // Fragment i of the step's stream: chunk q = i / CFRAG; r < KS is up fragment r of chunk q, r >= KS is down
    // fragment r - KS of chunk q (of the chunk before q with DEFER, which for q = 0 lives in the previous buffer).
    auto read_stream = [&](auto ic, bf16x8& dst) {
      constexpr int i = decltype(ic)::value;
      constexpr int q = i / CFRAG, r = i % CFRAG;
      if constexpr (!DEFER || r < KS)
        lds_read_frag<i * kFrag>(dst, wb);
      else if constexpr (q == 0)
        lds_read_frag<((CPB - 1) * CFRAG + r) * kFrag>(dst, wb_prev);
      else
        lds_read_frag<((q - 1) * CFRAG + r) * kFrag>(dst, wb);
    };
    lds_read_u16<0>(brow[0], bias_step);
    static_for<P>([&](auto ic) { read_stream(ic, ring[decltype(ic)::value]); });
    static_for<NFRAG>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      constexpr int q = i / CFRAG;  // chunk inside the step
      constexpr int r = i % CFRAG;  // fragment inside the chunk
      // Operations issued after the read of fragment i: the next P - 1 fragments (fewer at the end of the step) and
      // the bias read of the following chunk if it was issued among them.
      constexpr int after = (P - 1 < NFRAG - 1 - i ? P - 1 : NFRAG - 1 - i) +
                            ((i / CFRAG != (i + P - 1) / CFRAG && (i + P - 1) < NFRAG) ? 1 : 0);
      if constexpr (r == 0)
        lds_wait_frag<after>(ring[i % P], brow[q]);  // the bias read is older than the chunk's first fragment
      else
        lds_wait_frag<after>(ring[i % P]);
      if constexpr (r < KS) {
        // ---- up projection: rows 0..15 gated half, rows 16..31 the other half ------------------------------------------
        if constexpr (r == 0) {
          const u32x4 bias_bits = {brow[q], 0u, 0u, 0u};
          const bf16x8 bias_frag = __builtin_bit_cast(bf16x8, bias_bits);
          const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          f32x16 binit = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bias_frag, ones, zero, 0, 0, 0);
#pragma unroll
          for (int t = 0; t < TT; ++t)
            gu[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[i % P], xf[t][r], binit, 0, 0, 0);
        } else {
#pragma unroll
          for (int t = 0; t < TT; ++t)
            gu[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[i % P], xf[t][r], gu[t], 0, 0, 0);
        }
      } else {
        // ---- down projection: O^T[feature, token] += W_down[feature, chunk] H^T --------------------------------------
        constexpr int jd = r - KS;  // k-step jd / MB of the chunk, row block jd % MB
#pragma unroll
        for (int t = 0; t < TT; ++t)
          oacc[t][jd % MB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ring[i % P], hb[t][jd / MB], oacc[t][jd % MB], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (i + P < NFRAG) {
        if constexpr ((i + P) % CFRAG == 0) lds_read_u16<((i + P) / CFRAG) * 64>(brow[(i + P) / CFRAG], bias_step);
        read_stream(std::integral_constant<int, i + P>{}, ring[i % P]);
      }
      // ---- SiLU gate: register e < 8 is the gated value, register 8 + e its partner, hidden unit unit0 + 8*hh + e -----
      if constexpr (!DEFER && r == KS - 1) {
#pragma unroll
        for (int t = 0; t < TT; ++t)
#pragma unroll
          for (int e = 0; e < 8 * DK; ++e) hb[t][e / 8][e % 8] = activate(gu[t], e);
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (DEFER && r >= KS) {
        constexpr int j = r - KS;  // down MFMA just issued; the 4 * DK pairs of activations are spread over the NDOWN MFMAs
#pragma unroll
        for (int t = 0; t < TT; ++t)
#pragma unroll
          for (int g = (j * 4 * DK) / NDOWN; g < ((j + 1) * 4 * DK) / NDOWN; ++g)
#pragma unroll
            for (int e = 2 * g; e < 2 * g + 2; ++e) hb_new[t][e / 8][e % 8] = activate(gu[t], e);
        if constexpr (r == CFRAG - 1) {
#pragma unroll
          for (int t = 0; t < TT; ++t)
#pragma unroll
            for (int k = 0; k < DK; ++k) hb[t][k] = hb_new[t][k];
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    });
    }  // active
    // The next step's weights must have landed (the only vector-memory operations of this loop).
    vm_wait<0>();
    __syncthreads();
    wb_prev = wb;
    buf = buf == NBUF - 1 ? 0 : buf + 1;
  }
  if constexpr (DEFER) {
    // The down projection of the last chunk is still pending; its fragments are in the last step's buffer.
    if (active) {
    bf16x8 tail[NDOWN];
    static_for<NDOWN>([&](auto ic) {
      constexpr int j = decltype(ic)::value;
      lds_read_frag<((CPB - 1) * CFRAG + KS + j) * kFrag>(tail[j], wb_prev);
    });
    static_for<NDOWN>([&](auto ic) {
      constexpr int j = decltype(ic)::value;
      lds_wait_frag<NDOWN - 1 - j>(tail[j]);
#pragma unroll
      for (int t = 0; t < TT; ++t)
        oacc[t][j % MB] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(tail[j], hb[t][j / MB], oacc[t][j % MB], 0, 0, 0);
    });
    }
    __syncthreads();  // the epilogue tiles below overwrite the weight buffers
  }

  // ---- epilogue: + b_down, round, transpose through the wavefront's LDS tile, + residual, coalesced bf16 stores ----
  if (!active) return;  // no barrier below
  uint8_t* tile = smem + wave * kStageWave;  // the weight buffers are free after the last barrier
  const bf16_t* bdown_lds = bias_lds + UPB;
#pragma unroll
  for (int t = 0; t < TT; ++t) {
    const int64_t tok_base = tok0 + t * 32;
    int64_t prow[4];
    bool live[4];
    token_rows_batch<4>(p.rows, count, [&](int i) { return tok_base + i * 8 + lane / 8; }, prow);  // one memory latency, not four
#pragma unroll
    for (int i = 0; i < 4; ++i) live[i] = tok_base + i * 8 + lane / 8 < wg_tok0 + wg_ntok;
    float hdot[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int pr = 0; pr < MB / 2; ++pr) {  // 64 features at a time
      bf16x8 res[4];
      const bool add_residual = !OUTP && p.residual != nullptr;  // OUTP: the accumulators started from x1
      if (add_residual) load_residual(p.residual, p.ldr, prow, pr * 64, res, lane);
      bf16x4 bv[8];
      read_chunk_bias(bdown_lds + pr * 64, hh, bv);
      tile_to_lds(tile, oacc[t][2 * pr], oacc[t][2 * pr + 1], bv, l32, hh);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      if (add_residual)
        tile_to_global<true>(tile, p.out, p.ldo, prow, live, pr * 64, res, lane, p.head_w, hdot);
      else
        tile_to_global<false>(tile, p.out, p.ldo, prow, live, pr * 64, res, lane, p.head_w, hdot);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
    }
    if (p.head_w != nullptr) {
      // the eight lanes of a row hold its eight 8-feature shares: add them in a fixed order, lane % 8 == 0 stores
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float d = hdot[i];
        d += __shfl_xor(d, 1);
        d += __shfl_xor(d, 2);
        d += __shfl_xor(d, 4);
        if (lane % 8 == 0 && live[i]) p.token_dots[prow[i]] = d;
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------------------------
// [RMSNorm ->] linear [-> + residual], K = D, N a multiple of 64
//
// Persistent: a workgroup (8 wavefronts x TT tiles of 32 tokens) walks token tiles blockIdx.x, blockIdx.x + gridDim.x, ...; for
// each tile it walks the N / 64 output chunks (the tiles of the last, partial round are split by chunks over several
// workgroups). The weight chunks form one endless stream over the workgroup's step number, staged by DMA into a ring of three LDS buffers two steps ahead of their use, so
// the stream never drains at a tile boundary.
//
// Memory-counter discipline. The weight transfers are issued by hand (lds_dma16) and are invisible to the compiler,
// so their completion is awaited by hand; everything else (token rows, residual pieces, output stores) is ordinary
// code whose waits the compiler inserts with its own - hence conservative - counts.
//   * weight fragments are read from LDS with ds_read_b128 four (row block 0, row block 1) pairs ahead of their MFMAs;
//   * per step and wavefront the vector-memory operations are issued in this order:
//       [RES: NST residual loads of step s+1] [FPW weight DMAs of step s+2] ... [NST output stores of step s]
//     (NST = 4 per 32-token tile) and the step ends with vmcnt(FPW + NST) (vmcnt(NST) when no DMA was issued): the
//     weights of step s+1 have landed, the weights of step s+2 and the stores of step s may stay in flight.
//   Every wavefront issues at least these counts after the transfer it waits for: tokens beyond the count are mapped
//   to the last token for loads AND stores (they compute bit-identical values, so the duplicate stores are benign),
//   and the "memory" clobbers of the hand-written statements keep loads and stores on their side of them.
// LDS: [3 weight buffers of 2*KS fragments][8 epilogue tiles][bias (N) | norm weight (D)]
// ------------------------------------------------------------------------------------------------------------------
template <int D, int TT, bool RES, int QK>
__global__ __launch_bounds__(8 * kWave, 2) void norm_linear_kernel(const TsParams p) {
  static_assert(!(QK != 0 && RES), "the query / key epilogue has no residual");
  constexpr int NWAVES = 8;
  constexpr int kTokPerWg = NWAVES * 32 * TT;  // TT token tiles of 32 per wavefront
  constexpr int KS = D / 16;
  constexpr int NFRAG = 2 * KS;  // two 32-feature row blocks per chunk
  constexpr int FPW = NFRAG / NWAVES;
  constexpr int kBuf = NFRAG * kFrag;
  constexpr int PRE = 4;  // fragment pairs in flight
  constexpr int NST = 4 * TT;  // output stores (and residual pieces) per wavefront and step
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  uint8_t* tiles = smem + 3 * kBuf;
  bf16_t* bias_lds = reinterpret_cast<bf16_t*>(tiles + NWAVES * kStageWave);

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int lane = tid % kWave;
  const int l32 = lane % 32;
  const int hh = lane / 32;
  // QK: (memory row, position in the sample) of the wavefront's tokens, kept in LDS behind the bias and norm weights
  // (written and read by the same wavefront only), instead of in registers.
  int2* rowinfo = reinterpret_cast<int2*>(reinterpret_cast<uint8_t*>(bias_lds) + ((p.N + D) * 2 + 15) / 16 * 16) + wave * kWave;
  // QK == 0: a float32 copy of the bias in the same place (the epilogue adds it in float32: read as it is needed, the
  // widening of 64 values per step and wavefront is done once per workgroup instead)
  float* bias_f32 = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(bias_lds) + ((p.N + D) * 2 + 15) / 16 * 16);
  const int nchunks = p.N / kNC;
  const int64_t count = token_count(p);
  const int num_tiles = static_cast<int>((count + kTokPerWg - 1) / kTokPerWg);
  // Work split. The first full_rounds * gridDim.x tiles go round-robin to the workgroups, every one with all of its
  // output chunks. The R = num_tiles % gridDim.x tiles that remain would keep R workgroups busy for a whole tile
  // while the others idle, so each of them is split by output chunks (they are independent) into S = gridDim.x / R
  // segments handled by different workgroups, which all load the tile's rows.
  const int G = static_cast<int>(gridDim.x);
  const int wg = static_cast<int>(blockIdx.x);
  const int full_rounds = num_tiles / G;
  const int R = num_tiles % G;
  int S = R > 0 ? G / R : 1;
  S = S < nchunks ? S : nchunks;
  const bool has_tail = R > 0 && wg < R * S;
  const int tail_tile = full_rounds * G + wg / S;
  const int tail_begin = has_tail ? ((wg % S) * nchunks) / S : 0;
  const int tail_len = has_tail ? (((wg % S) + 1) * nchunks) / S - tail_begin : 0;
  const int full_total = full_rounds * nchunks;
  const int total = full_total + tail_len;
  if (total == 0) return;  // whole workgroup: nothing assigned to it
  // Step s of this workgroup works on chunk_of(s) of tile tile_of(s); first_of_tile(s) opens a new tile.
  auto chunk_of = [&](int step) -> int { return step < full_total ? step % nchunks : tail_begin + (step - full_total); };
  auto tile_of = [&](int step) -> int { return step < full_total ? wg + (step / nchunks) * G : tail_tile; };
  auto first_of_tile = [&](int step) -> bool { return step < full_total ? step % nchunks == 0 : step == full_total; };

  // fragment f of a chunk = (row block f / KS, k-step f % KS); source = uniform base + 32-bit per-lane byte offset
  const char* w_bytes = reinterpret_cast<const char*>(p.w1);
  auto stage = [&](int chunk, int buf) {
    int ln = lane;
    asm volatile("" : "+v"(ln));
    uint8_t* base = smem + buf * kBuf + wave * (FPW * kFrag);
    if (p.packed) {
      const char* src = w_bytes + (static_cast<int64_t>(chunk) * NFRAG + wave * FPW) * kFrag;  // scalar registers
      const uint32_t lane_off = static_cast<uint32_t>(ln * 16);
#pragma unroll
      for (int i = 0; i < FPW; ++i) lds_dma16_offset(src + i * kFrag, lane_off, base + i * kFrag);
      return;
    }
    const uint32_t lane_off = static_cast<uint32_t>(((ln & 31) * D + (ln >> 5) * 8) * 2);
#pragma unroll
    for (int i = 0; i < FPW; ++i) {
      const int f = wave * FPW + i;  // wavefront-uniform
      const int64_t row0 = static_cast<int64_t>(chunk) * kNC + (f / KS) * 32;
      lds_dma16(w_bytes + (row0 * D + (f % KS) * 16) * 2 + lane_off, base + i * kFrag);
    }
  };
  // First token of this wavefront in token tile `tile`.
  auto tokens_of_tile = [&](int tile) -> int64_t { return static_cast<int64_t>(tile) * kTokPerWg + wave * (32 * TT); };
  // Memory rows of a tile in the layout of the epilogue stores: piece i = token (i / 4) * 32 + 8 * (i % 4) + lane / 8.
  // Without a residual the row numbers are only needed for the stores, so the lane's store offset is kept instead, in
  // units of 16 bytes (row * ldo / 8 + lane % 8; the host checks that it fits 32 bits): a store then needs one
  // multiply-add for its address instead of a 64-bit row * stride product per piece and step.
  const uint32_t ld16 = static_cast<uint32_t>(p.ldo >> 3);
  auto rows_of_tile = [&](int64_t tok_base, int32_t (&prow)[NST]) {
    // all row numbers are requested before the first is used (one memory latency for the tile, not one per piece): the
    // layout branch below must not sit between the loads
    int64_t row64[NST];
    token_rows_batch<NST>(p.rows, count, [&](int i) { return tok_base + (i / 4) * 32 + (i % 4) * 8 + lane / 8; }, row64);
#pragma unroll
    for (int i = 0; i < NST; ++i) prow[i] = static_cast<int32_t>(row64[i]);
    if (RES) return;
    if (p.out_plane_shift > 0) {
      // feature planes: the lane's piece j = lane % 8 of a 64-feature chunk lies in plane (8 * j) >> shift of the chunk's
      // planes, at 16-byte piece j % (plane width / 8) of the row
      const int psh = p.out_plane_shift - 3;  // log2 of the 16-byte pieces per plane row
      const uint32_t j = static_cast<uint32_t>(lane % 8);
      const uint32_t plane_base = (j >> psh) * static_cast<uint32_t>(p.M);
      const uint32_t piece = j & ((1u << psh) - 1u);
#pragma unroll
      for (int i = 0; i < NST; ++i)
        prow[i] = static_cast<int32_t>(((plane_base + static_cast<uint32_t>(prow[i])) << psh) + piece);
      return;
    }
#pragma unroll
    for (int i = 0; i < NST; ++i)
      prow[i] = static_cast<int32_t>(static_cast<uint32_t>(prow[i]) * ld16 + static_cast<uint32_t>(lane % 8));
  };
  // bytes between the 64-feature chunks of the output: 128 in a row, 64 features of M rows in the plane layout
  const int64_t chunk_bytes = (!RES && p.out_plane_shift > 0) ? static_cast<int64_t>(kNC) * 2 * p.M : kNC * 2;
  // Address of the lane's 16-byte piece of output chunk `chunk` for piece slot value v (a row with RES, an offset without).
  auto out_piece = [&](int32_t v, int chunk) -> bf16x8* {
    const uint32_t off16 = RES ? static_cast<uint32_t>(v) * ld16 + static_cast<uint32_t>(lane % 8) : static_cast<uint32_t>(v);
    return reinterpret_cast<bf16x8*>(reinterpret_cast<char*>(p.out) + chunk * chunk_bytes + (static_cast<uint64_t>(off16) << 4));
  };
  auto request_residual = [&](const int32_t (&prow)[NST], int chunk, bf16x8 (&res)[NST]) {
#pragma unroll
    for (int i = 0; i < NST; ++i)
      res[i] = *reinterpret_cast<const bf16x8*>(p.residual + static_cast<int64_t>(prow[i]) * p.ldr + chunk * kNC +
                                                (lane % 8) * 8);
  };
  bf16x8 xf[TT][KS];
  int32_t prow[NST], prow_next[NST];  // piece slots (see rows_of_tile) of the current tile / of the tile the next step belongs to
  auto load_tile = [&](int64_t tok_base) {
    load_token_rows<D, TT>(p, count, tok_base, l32, hh, xf);
    // Consume the rows right here: otherwise the compiler's wait for them lands in front of the first MFMA of EVERY
    // step, where it also waits for the weights and stores that are meant to stay in flight.
#pragma unroll
    for (int t = 0; t < TT; ++t)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(xf[t][ks]));
    if constexpr (QK == 0 && !RES) {
      // the same for the store offsets (their row numbers were loaded just before the rows): otherwise the compiler
      // waits for them in front of the first store of every step, with a count that also covers the weight transfers
      // and the stores that are meant to stay in flight
#pragma unroll
      for (int i = 0; i < NST; ++i) asm volatile("" : "+v"(prow[i]));
    }
    if (QK != 0) {  // lane <-> token `lane` of the wavefront's 32 * TT tokens
      // the token's position inside its sample is that of its row of x (the side that keeps the caller's layout)
      const int64_t tok = tok_base + (lane < 32 * TT ? lane : 0);
      rowinfo[lane] = make_int2(static_cast<int>(token_row(p, count, tok)),
                                static_cast<int>(input_row(p, count, tok) % p.tokens_per_sample));
    }
  };

  bf16x8 res_cur[NST], res_next[NST];
  int64_t tok_wave = tokens_of_tile(tile_of(0));
  if constexpr (QK == 0) rows_of_tile(tok_wave, prow);
  stage(chunk_of(0), 0);
  if (total > 1) stage(chunk_of(1), 1);
  if (RES) request_residual(prow, chunk_of(0), res_cur);
  if constexpr (QK == 0) {
    for (int i = tid * 8; i < p.N; i += NWAVES * kWave * 8) {
      f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
      if (p.b1 != nullptr) {
        const bf16x8 v = *reinterpret_cast<const bf16x8*>(p.b1 + i);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          lo[e] = static_cast<float>(v[e]);
          hi[e] = static_cast<float>(v[4 + e]);
        }
      }
      *reinterpret_cast<f32x4*>(bias_f32 + i) = lo;
      *reinterpret_cast<f32x4*>(bias_f32 + i + 4) = hi;
    }
  } else {
    stage_bias(p.b1, bias_lds, p.N, tid, NWAVES * kWave);
  }
  if (p.norm_w != nullptr) stage_bias(p.norm_w, bias_lds + p.N, D, tid, NWAVES * kWave);
  load_tile(tok_wave);
  vm_wait<0>();
  __syncthreads();
  // The norm in front of the layer: either its weight is part of the packed layer and only the per-token factor is formed
  // here (it multiplies the accumulators in the epilogue), or the rows are normalised in place.
  float rstd[TT];
#pragma unroll
  for (int t = 0; t < TT; ++t) rstd[t] = 1.0f;
  auto apply_norm = [&]() {
    if (p.norm_w == nullptr) return;
    if (p.norm_folded)
      token_rstd<D, TT>(p.eps, xf, rstd);
    else
      normalize_tokens<D, TT>(p.eps, bias_lds + p.N, hh, xf);
  };
  apply_norm();

  uint8_t* tile_lds = tiles + wave * kStageWave;
  int buf = 0;                                        // ring slot of step s
  for (int s = 0; s < total; ++s) {
    const int chunk = chunk_of(s);
    // ---- requests for later steps ------------------------------------------------------------------------------------
    const bool has_next = s + 1 < total;
    const bool stage_ahead = s + 2 < total;
    const bool new_tile = s > 0 && first_of_tile(s);  // the workgroup moves to its next token tile in this step
    if (new_tile) {
      tok_wave = tokens_of_tile(tile_of(s));
      if (RES) {
#pragma unroll
        for (int i = 0; i < NST; ++i) prow[i] = prow_next[i];
      } else if constexpr (QK == 0) {
        rows_of_tile(tok_wave, prow);
      }
    }
    if (RES && has_next) {
      if (first_of_tile(s + 1)) {  // the next step opens the next tile
        rows_of_tile(tokens_of_tile(tile_of(s + 1)), prow_next);
        request_residual(prow_next, chunk_of(s + 1), res_next);
      } else {
        request_residual(prow, chunk_of(s + 1), res_next);
      }
    }
    if (stage_ahead) stage(chunk_of(s + 2), buf == 0 ? 2 : buf - 1);  // slot (s + 2) % 3, last read in step s - 1
    if (new_tile) {
      // The rows are requested after the weights and residual pieces of the later steps, so that those are not held
      // back by the wait for the rows.
      load_tile(tok_wave);
      apply_norm();
    }

    // ---- the products of this chunk ------------------------------------------------------------------------------------
    const uint32_t wb = lds_offset(smem) + buf * kBuf + lane * 16;
    f32x16 acc0[TT], acc1[TT];
#pragma unroll
    for (int t = 0; t < TT; ++t)
#pragma unroll
      for (int j = 0; j < 16; ++j) acc0[t][j] = acc1[t][j] = 0.f;
    bf16x8 fa[PRE], fb[PRE];
#define TAAC_READ_PAIR(K_)                                  \
  lds_read_frag<(K_) * kFrag>(fa[(K_) % PRE], wb);          \
  lds_read_frag<(KS + (K_)) * kFrag>(fb[(K_) % PRE], wb)
    static_assert(PRE == 4 && KS % 4 == 0, "the read schedule below is written for four pairs in flight");
    TAAC_READ_PAIR(0);
    TAAC_READ_PAIR(1);
    TAAC_READ_PAIR(2);
    TAAC_READ_PAIR(3);
    // (compile-time k-steps: the fragment offsets of the reads go into the instructions' offset fields instead of a vector
    // add per read)
    static_for<KS / 4>([&](auto kc) {
      constexpr int k4 = 4 * decltype(kc)::value;
      constexpr bool last = k4 + 4 >= KS;
      // pair k4 + i: pairs up to k4 + i + 3 (or KS - 1) have been requested after it
#define TAAC_STEP(I_)                                                                                   \
  if constexpr (last)                                                                                   \
    lds_wait_pair<2 * (3 - (I_))>(fa[I_], fb[I_]);                                                       \
  else                                                                                                  \
    lds_wait_pair<6>(fa[I_], fb[I_]);                                                                    \
  _Pragma("unroll") for (int t = 0; t < TT; ++t) {                                                      \
    acc0[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[I_], xf[t][k4 + (I_)], acc0[t], 0, 0, 0);      \
    acc1[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[I_], xf[t][k4 + (I_)], acc1[t], 0, 0, 0);      \
  }                                                                                                     \
  __builtin_amdgcn_sched_barrier(0)
#define TAAC_NEXT_PAIR(I_)                                           \
  if constexpr (!last) {                                             \
    lds_read_frag<(k4 + 4 + (I_)) * kFrag>(fa[I_], wb);              \
    lds_read_frag<(KS + k4 + 4 + (I_)) * kFrag>(fb[I_], wb);         \
  }
      // The read of pair k4 + 4 + i reuses the registers of pair k4 + i right after its two MFMAs were issued.
      TAAC_STEP(0);
      TAAC_NEXT_PAIR(0)
      TAAC_STEP(1);
      TAAC_NEXT_PAIR(1)
      TAAC_STEP(2);
      TAAC_NEXT_PAIR(2)
      TAAC_STEP(3);
      TAAC_NEXT_PAIR(3)
#undef TAAC_NEXT_PAIR
#undef TAAC_STEP
    });
#undef TAAC_READ_PAIR

    // ---- epilogue of this chunk: bias, rounding, transpose through LDS, residual, 4 stores ---------------------------
    [[maybe_unused]] bf16x4 bv[8];
    [[maybe_unused]] f32x4 bvf[8];
    if constexpr (QK == 0) read_chunk_bias(bias_f32 + chunk * kNC, hh, bvf);
    if constexpr (QK != 0) {
      // Query and key chunks: the sum of squares of the rounded projection goes to qk_sumsq (one value per token and
      // chunk; the statistic of the norm over the model width is their sum). QK == 2 also multiplies the features by
      // the norm weight and rotates them. The per-token factor rsqrt(mean + eps) commutes with both and is applied by
      // the attention kernel. Value chunks are stored as they are.
      constexpr bool XF = QK == 2;
      const bool qk_chunk = chunk < p.qk_chunks;  // wavefront-uniform
      const int col8 = chunk * kNC + (lane % 8) * 8;
      const bool rotate = XF && qk_chunk && p.cos_sin != nullptr;
      const bool transform = XF && qk_chunk;
      bf16x8 wn;
      if (XF) {
#pragma unroll
        for (int e = 0; e < 8; ++e) wn[e] = static_cast<bf16_t>(1.0f);
        if (qk_chunk && p.qk_w != nullptr) wn = *reinterpret_cast<const bf16x8*>(p.qk_w + col8);
      }
      const int d0 = rotate ? col8 % p.head_dim : 0;
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        read_chunk_bias(bias_lds + chunk * kNC, hh, bv);  // per tile: not held while the pieces are processed
        if (qk_chunk && p.qk_sumsq != nullptr) {
          float ss = tile_to_lds_sumsq(tile_lds, acc0[t], acc1[t], bv, l32, hh, rstd[t]);
          ss = half_wave_pair_sum(ss);
          const int row = rowinfo[t * 32 + l32].x;
          if (hh == 0) p.qk_sumsq[static_cast<int64_t>(chunk) * p.M + row] = ss;
        } else {
          tile_to_lds(tile_lds, acc0[t], acc1[t], bv, l32, hh, rstd[t]);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        // two pieces at a time: rows (and table pieces) first, then the arithmetic and the stores
#pragma unroll
        for (int i2 = 0; i2 < 4; i2 += 2) {
          int2 info[2];
          bf16x8 cs[2];
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            info[j] = rowinfo[t * 32 + (i2 + j) * 8 + lane / 8];
            if (XF && rotate)
              cs[j] = *reinterpret_cast<const bf16x8*>(p.cos_sin + static_cast<int64_t>(info[j].y) * p.head_dim + d0);
          }
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const int row = (i2 + j) * 8 + lane / 8;
            bf16x8 v = *reinterpret_cast<const bf16x8*>(tile_lds + row * kStageRow + (lane % 8) * 16);
            if (XF && transform) {
              float f[8];
#pragma unroll
              for (int e = 0; e < 8; ++e) f[e] = static_cast<float>(v[e]) * static_cast<float>(wn[e]);
              if (rotate) {
#pragma unroll
                for (int e = 0; e < 8; e += 2) {
                  const float even = f[e], odd = f[e + 1];
                  const float cv = static_cast<float>(cs[j][e]), sv = static_cast<float>(cs[j][e + 1]);
                  f[e] = even * cv - odd * sv;
                  f[e + 1] = even * sv + odd * cv;
                }
              }
#pragma unroll
              for (int e = 0; e < 8; ++e) v[e] = static_cast<bf16_t>(f[e]);
            }
            // feature planes: column col8 lies in plane col8 >> shift, at col8 % 2^shift of the row
            const int64_t at = p.out_plane_shift > 0
                                   ? (((static_cast<int64_t>(col8 >> p.out_plane_shift) * p.M + info[j].x) << p.out_plane_shift) +
                                      (col8 & ((1 << p.out_plane_shift) - 1)))
                                   : static_cast<int64_t>(info[j].x) * p.ldo + col8;
            __builtin_nontemporal_store(v, reinterpret_cast<bf16x8*>(p.out + at));
          }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      }
    }
#pragma unroll
    for (int t = 0; t < (QK != 0 ? 0 : TT); ++t) {
      tile_to_lds(tile_lds, acc0[t], acc1[t], bvf, l32, hh, rstd[t]);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int row = i * 8 + lane / 8;
        bf16x8 v = *reinterpret_cast<const bf16x8*>(tile_lds + row * kStageRow + (lane % 8) * 16);
        if (RES) {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            v[e] = static_cast<bf16_t>(static_cast<float>(v[e]) + static_cast<float>(res_cur[t * 4 + i][e]));
        }
        // non-temporal: the 64 KB a workgroup stores per step are not read again by this kernel; as ordinary stores they
        // wait for the cache lines they displace (stand-alone 0.166 against 0.176 ms for q | k | v, 0.093 against 0.112 ms
        // for the out projection; inside the step the kernel behind reads the rows from memory either way)
        __builtin_nontemporal_store(v, out_piece(prow[t * 4 + i], chunk));
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    // ---- close the step ------------------------------------------------------------------------------------------------
    if (has_next) {
      if (stage_ahead) {
        // The transfer that must have landed (step s + 1) was issued one step ago: behind it are the NST stores of step
        // s - 1, the FPW transfers of step s + 2 and the NST stores of this step, whatever else was issued. The query /
        // key epilogue issues more (statistic stores, table loads), so it uses the full count; the plain epilogue keeps
        // the tighter one (it makes no difference there).
        vm_wait<QK != 0 ? FPW + 2 * NST : FPW + NST>();
      } else {
        vm_wait<NST>();
      }
      __syncthreads();
      if (RES) {
#pragma unroll
        for (int i = 0; i < NST; ++i) res_cur[i] = res_next[i];
      }
    }
    buf = buf == 2 ? 0 : buf + 1;
  }
}

// The kernels use more than the default 64 KB of dynamic LDS; the opt-in is idempotent and cheap, so it is simply
// repeated before every launch (no cached per-process state to go stale across devices).
template <typename K>
int launch_ts(K kernel, const TsParams& p, int threads, int tokens_per_wg, size_t lds_bytes, hipStream_t s,
              const char* name) {
  if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                          static_cast<int>(lds_bytes)) != hipSuccess)
    return set_error(TAAC_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS", name, lds_bytes);
  // upper bound of the kernel's own split: one workgroup per complete tile plus one per unit for the rest
  const int64_t grid = p.M / tokens_per_wg + p.units;
  if (grid > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: too many workgroups", name);
  hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(grid)), dim3(threads), lds_bytes, s, p);
  return check_launch(name);
}

bool ptr_ok(const void* p, uintptr_t mask) { return (reinterpret_cast<uintptr_t>(p) & mask) == 0; }

constexpr int kMaxLdsBytes = 160 * 1024;

}  // namespace
}  // namespace taac

namespace taac {
// Packs the qkv / out / feed-forward weights (gate first) of n backbone blocks with as few launches as possible.
int pack_backbone_blocks(const taac_block_weights* blocks, int n, int32_t D, int32_t F, void* const* packed_qkv,
                         void* const* packed_out, void* const* packed_ffn, bool fold_act, hipStream_t s, const char* name) {
  for (int base = 0; base < n; base += kPackBatch) {
    PackBatch batch{};
    const int m = n - base < kPackBatch ? n - base : kPackBatch;
    for (int i = 0; i < m; ++i) {
      const taac_block_weights& w = blocks[base + i];
      if (!ptr_ok(w.qkv_weight, 15) || !ptr_ok(w.out_weight, 15) || !ptr_ok(w.up_weight, 15) ||
          !ptr_ok(w.down_weight, 15) || !ptr_ok(w.attn_norm_weight, 15) || !ptr_ok(w.ffn_norm_weight, 15))
        return set_error(TAAC_ERR_UNSUPPORTED, "%s: weights must be 16-byte aligned", name);
      batch.qkv[i] = static_cast<const bf16_t*>(w.qkv_weight);
      batch.qkv_norm[i] = static_cast<const bf16_t*>(w.attn_norm_weight);
      batch.out[i] = static_cast<const bf16_t*>(w.out_weight);
      batch.up[i] = static_cast<const bf16_t*>(w.up_weight);
      batch.ffn_norm[i] = static_cast<const bf16_t*>(w.ffn_norm_weight);
      batch.down[i] = static_cast<const bf16_t*>(w.down_weight);
      batch.packed_qkv[i] = static_cast<bf16x8*>(packed_qkv[base + i]);
      batch.packed_out[i] = static_cast<bf16x8*>(packed_out[base + i]);
      batch.packed_ffn[i] = static_cast<bf16x8*>(packed_ffn[base + i]);
    }
    const int64_t pieces = (static_cast<int64_t>(4) * D * D + static_cast<int64_t>(3) * D * F) / 8;
    hipLaunchKernelGGL(pack_blocks_kernel, dim3(static_cast<uint32_t>((pieces + 255) / 256), m), dim3(256), 0, s, batch,
                       D, F, fold_act);
    const int rc = check_launch(name);
    if (rc != TAAC_OK) return rc;
  }
  return TAAC_OK;
}
}  // namespace taac

extern "C" int64_t taac_ffn_packed_bytes(int32_t D, int32_t F) {
  if ((D != 128 && D != 256) || F <= 0 || F % (taac::kHU * taac::kCPB) != 0) return -1;
  return static_cast<int64_t>(3) * D * F * 2;
}

namespace taac {
namespace {
int ffn_pack(const char* name, const void* w_up, const void* w_down, const void* norm_weight, void* packed, int32_t D,
             int32_t F, int gate_first, void* stream, bool fold_act = false);
}
}  // namespace taac

extern "C" int taac_ffn_activation_fold_supported(int32_t D, int32_t F) { return taac::ffn_act_fold_supported(D, F) ? 1 : 0; }

extern "C" int taac_ffn_pack_weights_folded(const void* w_up, const void* w_down, const void* norm_weight, void* packed,
                                            int32_t D, int32_t F, int gate_first, int fold_activation, void* stream) {
  const char* name = "taac_ffn_pack_weights_folded";
  if (fold_activation && !taac::ffn_act_fold_supported(D, F))
    return taac::set_error(TAAC_ERR_UNSUPPORTED, "%s: the kernels do not take the activation's constants from the blob at D=%d, F=%d",
                           name, D, F);
  return taac::ffn_pack(name, w_up, w_down, norm_weight, packed, D, F, gate_first, stream, fold_activation != 0);
}

extern "C" int taac_ffn_pack_weights(const void* w_up, const void* w_down, void* packed, int32_t D, int32_t F,
                                     int gate_first, void* stream) {
  return taac::ffn_pack("taac_ffn_pack_weights", w_up, w_down, nullptr, packed, D, F, gate_first, stream);
}

extern "C" int taac_ffn_pack_weights_norm(const void* w_up, const void* w_down, const void* norm_weight, void* packed,
                                          int32_t D, int32_t F, int gate_first, void* stream) {
  const char* name = "taac_ffn_pack_weights_norm";
  if (!norm_weight) return taac::set_error(TAAC_ERR_INVALID_VALUE, "%s: null norm weight", name);
  return taac::ffn_pack(name, w_up, w_down, norm_weight, packed, D, F, gate_first, stream);
}

namespace taac {
namespace {
int ffn_pack(const char* name, const void* w_up, const void* w_down, const void* norm_weight, void* packed, int32_t D,
             int32_t F, int gate_first, void* stream, bool fold_act) {
  if (taac_ffn_packed_bytes(D, F) < 0)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: D must be 128 or 256 and F a positive multiple of 32", name);
  if (!w_up || !w_down || !packed) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  if (!ptr_ok(w_up, 15) || !ptr_ok(w_down, 15) || !ptr_ok(packed, 15) || !ptr_ok(norm_weight, 15))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: pointers must be 16-byte aligned", name);
  const int64_t pieces = static_cast<int64_t>(3) * D * F / 8;
  hipLaunchKernelGGL(ffn_pack_kernel, dim3(static_cast<uint32_t>((pieces + 255) / 256)), dim3(256), 0,
                     as_stream(stream), static_cast<const bf16_t*>(w_up), static_cast<const bf16_t*>(w_down),
                     static_cast<bf16x8*>(packed), D, F, gate_first ? 1 : 0, static_cast<const bf16_t*>(norm_weight), fold_act);
  return check_launch(name);
}
}  // namespace
}  // namespace taac


extern "C" int64_t taac_linear_packed_bytes(int32_t N, int32_t K) {
  if ((K != 128 && K != 256) || N <= 0 || N % taac::kNC != 0) return -1;
  return static_cast<int64_t>(N) * K * 2;
}

namespace taac {
namespace {
int linear_pack(const char* name, const void* w, const void* norm_weight, void* packed, int32_t N, int32_t K, void* stream) {
  if (taac_linear_packed_bytes(N, K) < 0)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: K must be 128 or 256 and N a positive multiple of 64", name);
  if (!w || !packed) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  if (!ptr_ok(w, 15) || !ptr_ok(packed, 15) || !ptr_ok(norm_weight, 15))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: pointers must be 16-byte aligned", name);
  const int64_t pieces = static_cast<int64_t>(N) * K / 8;
  hipLaunchKernelGGL(linear_pack_kernel, dim3(static_cast<uint32_t>((pieces + 255) / 256)), dim3(256), 0,
                     as_stream(stream), static_cast<const bf16_t*>(w), static_cast<bf16x8*>(packed), N, K,
                     static_cast<const bf16_t*>(norm_weight));
  return check_launch(name);
}
}  // namespace
}  // namespace taac

extern "C" int taac_linear_pack_weights(const void* w, void* packed, int32_t N, int32_t K, void* stream) {
  return taac::linear_pack("taac_linear_pack_weights", w, nullptr, packed, N, K, stream);
}

extern "C" int taac_linear_pack_weights_norm(const void* w, const void* norm_weight, void* packed, int32_t N, int32_t K,
                                             void* stream) {
  const char* name = "taac_linear_pack_weights_norm";
  if (!norm_weight) return taac::set_error(TAAC_ERR_INVALID_VALUE, "%s: null norm weight", name);
  return taac::linear_pack(name, w, norm_weight, packed, N, K, stream);
}

namespace taac {
namespace {

// Shared body of taac_swiglu_ffn_fwd and taac_attn_out_ffn_fwd (out_packed != null: the attention output projection
// runs in front; x is then the attention output and residual the block input).
int ffn_entry(const char* name, const void* x, int64_t ldx, const void* out_bias, const void* out_packed,
              const void* norm_weight, float eps, const void* w_up, const void* b_up, const void* w_down,
              const void* b_down, const void* packed_weights, const void* residual, int64_t ldr, void* out, int64_t ldo,
              int64_t M, int32_t D, int32_t F, int gate_first, const int32_t* rows, const int32_t* n_rows,
              const int32_t* x_rows, int norm_folded, void* stream, const void* update_gate = nullptr, int64_t ldg = 0,
              bool glu = true, int x_plane = 0, const void* head_w = nullptr, float* token_dots = nullptr) {
  const bool with_proj = out_packed != nullptr;
  if (norm_folded < 0 || norm_folded > (TAAC_FOLDED_NORM | TAAC_FOLDED_ACTIVATION))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: norm_folded holds TAAC_FOLDED_NORM and / or TAAC_FOLDED_ACTIVATION", name);
  const bool act_folded = (norm_folded & TAAC_FOLDED_ACTIVATION) != 0;
  norm_folded &= TAAC_FOLDED_NORM;
  if (act_folded && (!glu || update_gate != nullptr || packed_weights == nullptr || !ffn_act_fold_supported(D, F)))
    return set_error(TAAC_ERR_INVALID_VALUE,
                     "%s: TAAC_FOLDED_ACTIVATION needs the blob of taac_ffn_pack_weights_folded (gated form without an update "
                     "gate, a shape taac_ffn_activation_fold_supported accepts)", name);
  if ((head_w == nullptr) != (token_dots == nullptr) || !ptr_ok(head_w, 15))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: the readout needs a 16-byte aligned head weight and a buffer of token dots", name);
  if (x_plane != 0 && ((x_plane != 32 && x_plane != 64) || D % x_plane != 0))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: input planes are 32 or 64 features wide", name);
  if (norm_folded && (!norm_weight || !packed_weights))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: norm_folded needs the norm weight and the packed weights it was folded into", name);
  if (!glu && (with_proj || !packed_weights))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: the plain MLP takes packed weights and no projection in front", name);
  if (update_gate && !with_proj)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: an update gate needs the projection in front", name);
  if (update_gate && (ldg < D || ldg % 8 || !ptr_ok(update_gate, 15)))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: the gate's row stride must cover a row and be a multiple of 8, its base 16-byte aligned", name);
  if (M < 0 || D <= 0 || F <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: M must be >= 0, D and F > 0", name);
  if (D != 256 && D != 128)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: fused kernel is built for D = 128 or 256 (got %d)", name, D);
  if (F % (kHU * kCPB) != 0)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: F=%d must be a multiple of %d", name, F, kHU * kCPB);
  if (ldx < D || ldo < D || (residual && ldr < D) || ldx % 8 || ldo % 8 || (residual && ldr % 8))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: row strides must cover a row and be multiples of 8", name);
  if (M == 0) return TAAC_OK;
  if (!x || !out || (!packed_weights && (!w_up || !w_down)))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  if (with_proj && (!residual || !packed_weights))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: the projection needs the block input and packed feed-forward weights", name);
  if ((rows == nullptr) != (n_rows == nullptr))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: rows and n_rows must be given together", name);
  if (x_rows && !rows) return set_error(TAAC_ERR_INVALID_VALUE, "%s: x_rows needs rows and n_rows", name);
  if (rows && M > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: a row index covers at most 2^31 rows", name);
  if (!ptr_ok(x, 15) || !ptr_ok(w_up, 15) || !ptr_ok(w_down, 15) || !ptr_ok(out, 15) || !ptr_ok(residual, 15) ||
      !ptr_ok(norm_weight, 15) || !ptr_ok(b_up, 15) || !ptr_ok(b_down, 15) || !ptr_ok(packed_weights, 15) ||
      !ptr_ok(out_packed, 15) || !ptr_ok(out_bias, 15))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: tensor base pointers must be 16-byte aligned", name);
  const int KS = D / 16, MB = D / 32;
  const size_t bias_bytes = static_cast<size_t>((glu ? 2 : 1) * F + (with_proj ? 3 : 2) * D) * 2;
  const size_t buffer_bytes = glu ? static_cast<size_t>(kCPB * (KS + MB)) * kFrag : static_cast<size_t>(KS + 2 * MB) * kFrag;
  if ((with_proj || !glu ? 3 : 2) * buffer_bytes + bias_bytes > kMaxLdsBytes)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: F=%d does not fit the LDS (limit %d bytes)", name, F, kMaxLdsBytes);
  TsParams p{};
  p.x = static_cast<const bf16_t*>(x);
  p.norm_w = static_cast<const bf16_t*>(norm_weight);
  p.w1 = static_cast<const bf16_t*>(packed_weights ? packed_weights : w_up);
  p.b1 = static_cast<const bf16_t*>(b_up);
  p.w2 = static_cast<const bf16_t*>(w_down);
  p.b2 = static_cast<const bf16_t*>(b_down);
  p.residual = static_cast<const bf16_t*>(residual);
  p.out = static_cast<bf16_t*>(out);
  p.M = M;
  p.ldx = ldx;
  p.ldr = ldr;
  p.ldo = ldo;
  p.F = F;
  p.eps = eps;
  p.gate_first = gate_first ? 1 : 0;
  p.packed = packed_weights ? 1 : 0;
  p.rows = rows;
  p.n_rows = n_rows;
  p.x_rows = x_rows;
  p.w0 = static_cast<const bf16_t*>(out_packed);
  p.b0 = static_cast<const bf16_t*>(out_bias);
  p.gate = static_cast<const bf16_t*>(update_gate);
  p.ldg = ldg;
  p.norm_folded = norm_folded ? 1 : 0;
  p.x_plane_shift = x_plane == 32 ? 5 : (x_plane == 64 ? 6 : 0);
  p.head_w = static_cast<const bf16_t*>(head_w);
  p.token_dots = token_dots;
  p.units = compute_units();
  if (p.units <= 0) return set_error(TAAC_ERR_LAUNCH, "%s: cannot query the device", name);
  if (const int limit = test_max_workgroups(); limit > 0 && limit < p.units) p.units = limit;  // taac_test_hooks
  hipStream_t s = as_stream(stream);
#define TAAC_FFN_LAUNCH(DD, TT, NW, CPB, DEFER, ...)                                                         \
  return launch_ts(swiglu_ffn_kernel<DD, TT, NW, CPB, DEFER, __VA_ARGS__>, p, NW * kWave, NW * 32 * TT,      \
                   static_cast<size_t>((DEFER ? 3 : 2) * CPB * (KS + MB)) * kFrag + bias_bytes, s, name)
  if (!glu) {  // one 32-unit chunk per barrier step, deferred down projection: three buffers of KS + 2 * MB fragments
#define TAAC_MLP_LAUNCH(DD)                                                                              \
  return launch_ts(swiglu_ffn_kernel<DD, 1, 8, 1, true, false, false, false>, p, 8 * kWave, 8 * 32,      \
                   3 * buffer_bytes + bias_bytes, s, name)
    if (D == 256) TAAC_MLP_LAUNCH(256);
    TAAC_MLP_LAUNCH(128);
#undef TAAC_MLP_LAUNCH
  }
  if (with_proj && update_gate) {
    if (D == 256) TAAC_FFN_LAUNCH(256, 1, 8, 2, true, true, true);
    TAAC_FFN_LAUNCH(128, 1, 8, 2, true, true, true);
  }
  if (with_proj && act_folded) {
    if (D == 256) TAAC_FFN_LAUNCH(256, 1, 8, 2, true, true, false, true, true);
    TAAC_FFN_LAUNCH(128, 1, 8, 2, true, true, false, true, true);
  }
  if (with_proj) {
    if (D == 256) TAAC_FFN_LAUNCH(256, 1, 8, 2, true, true);
    TAAC_FFN_LAUNCH(128, 1, 8, 2, true, true);
  }
  if (act_folded) {  // three buffers fit (ffn_act_fold_supported)
    if (D == 256) TAAC_FFN_LAUNCH(256, 1, 8, 2, true, false, false, true, true);
    TAAC_FFN_LAUNCH(128, 1, 8, 2, true, false, false, true, true);
  }
  // Schedule: the down projection of a chunk is deferred by one chunk and interleaved with the next activation (three
  // weight buffers); when a large F leaves no room for the third buffer next to the biases it follows its activation
  // directly (two buffers).
  const int cfg = 3 * buffer_bytes + bias_bytes > kMaxLdsBytes ? 0 : 1;
  if (D == 256) {
    if (cfg == 1) TAAC_FFN_LAUNCH(256, 1, 8, 2, true, false);
    TAAC_FFN_LAUNCH(256, 1, 8, 2, false, false);
  }
  if (cfg == 1) TAAC_FFN_LAUNCH(128, 1, 8, 2, true, false);
  TAAC_FFN_LAUNCH(128, 1, 8, 2, false, false);
#undef TAAC_FFN_LAUNCH
}

}  // namespace
}  // namespace taac

extern "C" int taac_swiglu_ffn_fwd(const void* x, int64_t ldx, const void* norm_weight, float eps, const void* w_up,
                                   const void* b_up, const void* w_down, const void* b_down, const void* packed_weights,
                                   const void* residual, int64_t ldr, void* out, int64_t ldo, int64_t M, int32_t D,
                                   int32_t F, int gate_first, const int32_t* rows, const int32_t* n_rows,
                                   int norm_folded, void* stream) {
  return taac::ffn_entry("taac_swiglu_ffn_fwd", x, ldx, nullptr, nullptr, norm_weight, eps, w_up, b_up, w_down, b_down,
                         packed_weights, residual, ldr, out, ldo, M, D, F, gate_first, rows, n_rows, nullptr, norm_folded,
                         stream);
}

extern "C" int taac_attn_out_ffn_fwd(const void* attn, int64_t ld_attn, const void* out_bias,
                                     const void* packed_out_weights, const void* residual, int64_t ldr,
                                     const void* norm_weight, float eps, const void* b_up, const void* b_down,
                                     const void* packed_ffn_weights, void* out, int64_t ldo, int64_t M, int32_t D,
                                     int32_t F, const int32_t* rows, const int32_t* n_rows,
                                     const int32_t* attn_rows, int norm_folded, void* stream) {
  const char* name = "taac_attn_out_ffn_fwd";
  if (!packed_out_weights || !packed_ffn_weights)
    return taac::set_error(TAAC_ERR_INVALID_VALUE, "%s: both weight sets must be packed", name);
  return taac::ffn_entry(name, attn, ld_attn, out_bias, packed_out_weights, norm_weight, eps, nullptr, b_up, nullptr,
                         b_down, packed_ffn_weights, residual, ldr, out, ldo, M, D, F, 1, rows, n_rows, attn_rows,
                         norm_folded, stream);
}

extern "C" int64_t taac_silu_mlp_packed_bytes(int32_t D, int32_t F) {
  if ((D != 128 && D != 256) || F <= 0 || F % 32 != 0) return -1;
  return static_cast<int64_t>(2) * D * F * 2;
}

extern "C" int taac_silu_mlp_pack_weights(const void* w1, const void* w2, void* packed, int32_t D, int32_t F,
                                          void* stream) {
  using namespace taac;
  const char* name = "taac_silu_mlp_pack_weights";
  if (taac_silu_mlp_packed_bytes(D, F) < 0)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: D must be 128 or 256 and F a positive multiple of 32", name);
  if (!w1 || !w2 || !packed) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  if (!ptr_ok(w1, 15) || !ptr_ok(w2, 15) || !ptr_ok(packed, 15))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: pointers must be 16-byte aligned", name);
  const int64_t pieces = static_cast<int64_t>(2) * D * F / 8;
  hipLaunchKernelGGL(mlp_pack_kernel, dim3(static_cast<uint32_t>((pieces + 255) / 256)), dim3(256), 0, as_stream(stream),
                     static_cast<const bf16_t*>(w1), static_cast<const bf16_t*>(w2), static_cast<bf16x8*>(packed), D, F);
  return check_launch(name);
}

extern "C" int taac_silu_mlp_fwd(const void* x, int64_t ldx, const void* norm_weight, float eps, const void* b1,
                                 const void* b2, const void* packed_weights, const void* residual, int64_t ldr, void* out,
                                 int64_t ldo, int64_t M, int32_t D, int32_t F, const int32_t* rows, const int32_t* n_rows,
                                 void* stream) {
  const char* name = "taac_silu_mlp_fwd";
  if (!packed_weights) return taac::set_error(TAAC_ERR_INVALID_VALUE, "%s: the weights must be packed", name);
  return taac::ffn_entry(name, x, ldx, nullptr, nullptr, norm_weight, eps, nullptr, b1, nullptr, b2, packed_weights,
                         residual, ldr, out, ldo, M, D, F, 1, rows, n_rows, nullptr, 0, stream, nullptr, 0, false);
}

extern "C" int taac_attn_out_gate_ffn_fwd(const void* attn, int64_t ld_attn, const void* out_bias,
                                          const void* packed_out_weights, const void* update_gate, int64_t ld_gate,
                                          const void* residual, int64_t ldr, const void* norm_weight, float eps,
                                          const void* b_up, const void* b_down, const void* packed_ffn_weights,
                                          void* out, int64_t ldo, int64_t M, int32_t D, int32_t F,
                                          const int32_t* rows, const int32_t* n_rows, const int32_t* attn_rows,
                                          int norm_folded, void* stream) {
  const char* name = "taac_attn_out_gate_ffn_fwd";
  if (!packed_out_weights || !packed_ffn_weights)
    return taac::set_error(TAAC_ERR_INVALID_VALUE, "%s: both weight sets must be packed", name);
  if (!update_gate) return taac::set_error(TAAC_ERR_INVALID_VALUE, "%s: null gate pointer", name);
  return taac::ffn_entry(name, attn, ld_attn, out_bias, packed_out_weights, norm_weight, eps, nullptr, b_up, nullptr,
                         b_down, packed_ffn_weights, residual, ldr, out, ldo, M, D, F, 1, rows, n_rows, attn_rows,
                         norm_folded, stream, update_gate, ld_gate);
}

namespace taac {
namespace {

// Query / key extras of the linear kernel; all null / zero for a plain layer.
struct QkExtras {
  const void* qk_weight = nullptr;
  const void* cos_sin = nullptr;
  float* qk_sumsq = nullptr;
  int32_t qk_chunks = 0, head_dim = 0, tokens_per_sample = 0;
  bool enabled = false;
};

int norm_linear_launch(const char* name, const void* x, int64_t ldx, const void* norm_weight, float eps, const void* w,
                       const void* bias, const void* packed_weights, const void* residual, int64_t ldr, void* out,
                       int64_t ldo, int64_t M, int32_t N, int32_t K, const int32_t* rows, const int32_t* n_rows,
                       const int32_t* x_rows, const QkExtras& qk, int norm_folded, void* stream, int out_plane = 0) {
  if (out_plane != 0 && (residual || (out_plane != 32 && out_plane != 64) || static_cast<int64_t>(8) * M + 8 > 0xffffffffLL ||
                         (qk.enabled && qk.head_dim != out_plane)))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: output planes are 32 or 64 features wide (the head width under a query / key epilogue), without residual", name);
  if (norm_folded != 0 && norm_folded != TAAC_FOLDED_NORM)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: norm_folded is 0 or TAAC_FOLDED_NORM for a linear layer", name);
  if (norm_folded && (!norm_weight || !packed_weights))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: norm_folded needs the norm weight and the packed weights it was folded into", name);
  if (M < 0 || N <= 0 || K <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: M must be >= 0, N and K > 0", name);
  if (K != 256 && K != 128)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: token-stationary kernel is built for K = 128 or 256 (got %d)", name, K);
  if (N % kNC != 0) return set_error(TAAC_ERR_UNSUPPORTED, "%s: N=%d must be a multiple of %d", name, N, kNC);
  if (ldx < K || ldo < N || (residual && ldr < N) || ldx % 8 || ldo % 8 || (residual && ldr % 8))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: row strides must cover a row and be multiples of 8", name);
  if (M == 0) return TAAC_OK;
  if (!x || !out || (!packed_weights && !w)) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  if ((rows == nullptr) != (n_rows == nullptr))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: rows and n_rows must be given together", name);
  if (x_rows && !rows) return set_error(TAAC_ERR_INVALID_VALUE, "%s: x_rows needs rows and n_rows", name);
  if (M > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: at most 2^31 rows", name);
  if (M * (ldo / 8) + 8 > 0xffffffffLL)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: the output spans more than 2^32 16-byte pieces", name);
  if (!ptr_ok(x, 15) || !ptr_ok(w, 15) || !ptr_ok(out, 15) || !ptr_ok(residual, 15) || !ptr_ok(norm_weight, 15) ||
      !ptr_ok(bias, 15) || !ptr_ok(packed_weights, 15) || !ptr_ok(qk.qk_weight, 15) || !ptr_ok(qk.cos_sin, 15) ||
      !ptr_ok(qk.qk_sumsq, 3))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: tensor base pointers must be 16-byte aligned", name);
  // behind the 16-bit bias and norm weight: the query / key epilogue's row table, or the float32 copy of the bias
  const size_t rowinfo_bytes = qk.enabled ? 16 + 8 * static_cast<size_t>(kWave) * sizeof(int2) : 16 + static_cast<size_t>(N) * 4;
  const size_t lds_bytes = static_cast<size_t>(3 * 2 * (K / 16)) * kFrag + 8 * static_cast<size_t>(kStageWave) +
                           static_cast<size_t>(N + K) * 2 + rowinfo_bytes;
  if (lds_bytes > kMaxLdsBytes)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: N=%d does not fit the LDS (limit %d bytes)", name, N, kMaxLdsBytes);
  TsParams p{};
  p.x = static_cast<const bf16_t*>(x);
  p.norm_w = static_cast<const bf16_t*>(norm_weight);
  p.w1 = static_cast<const bf16_t*>(packed_weights ? packed_weights : w);
  p.b1 = static_cast<const bf16_t*>(bias);
  p.residual = static_cast<const bf16_t*>(residual);
  p.out = static_cast<bf16_t*>(out);
  p.M = M;
  p.ldx = ldx;
  p.ldr = ldr;
  p.ldo = ldo;
  p.N = N;
  p.eps = eps;
  p.packed = packed_weights ? 1 : 0;
  p.norm_folded = norm_folded ? 1 : 0;
  p.rows = rows;
  p.n_rows = n_rows;
  p.x_rows = x_rows;
  p.out_plane_shift = out_plane == 32 ? 5 : (out_plane == 64 ? 6 : 0);
  p.qk_w = static_cast<const bf16_t*>(qk.qk_weight);
  p.cos_sin = static_cast<const bf16_t*>(qk.cos_sin);
  p.qk_sumsq = qk.qk_sumsq;
  p.qk_chunks = qk.qk_chunks;
  p.head_dim = qk.head_dim;
  p.tokens_per_sample = qk.tokens_per_sample;
  hipStream_t s = as_stream(stream);
  // Without a residual two token tiles per wavefront fit the register file: every weight fragment read from LDS then
  // feeds two MFMAs, which halves the LDS reads (and their share of the power budget) per token.
  const int tt = residual ? 1 : 2;
  const int64_t tiles64 = (M + 256 * tt - 1) / (256 * tt);
  if (tiles64 > 0x3fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: too many token tiles", name);
  const int num_tiles = static_cast<int>(tiles64);  // upper bound: with a row index the kernel derives its own
  const int cus = compute_units();
  if (cus <= 0) return set_error(TAAC_ERR_LAUNCH, "%s: cannot query the device", name);
  int grid = num_tiles < cus ? num_tiles : cus;
  // taac_test_hooks: cap the number of persistent workgroups so that small inputs exercise the multi-tile path.
  if (const int limit = test_max_workgroups(); limit > 0 && limit < grid) grid = limit;
#define TAAC_LIN_LAUNCH(KK, TT, RR, QQ)                                                                           \
  do {                                                                                                            \
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(norm_linear_kernel<KK, TT, RR, QQ>),                    \
                            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)) != hipSuccess) \
      return set_error(TAAC_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS", name, lds_bytes);                  \
    hipLaunchKernelGGL((norm_linear_kernel<KK, TT, RR, QQ>), dim3(grid), dim3(8 * kWave), lds_bytes, s, p);       \
    return check_launch(name);                                                                                    \
  } while (0)
  const bool qk_transform = qk.enabled && (qk.qk_weight != nullptr || qk.cos_sin != nullptr);
  if (K == 256) {
    if (qk_transform) TAAC_LIN_LAUNCH(256, 2, false, 2);
    if (qk.enabled) TAAC_LIN_LAUNCH(256, 2, false, 1);
    if (residual) TAAC_LIN_LAUNCH(256, 1, true, 0);
    TAAC_LIN_LAUNCH(256, 2, false, 0);
  }
  if (qk_transform) TAAC_LIN_LAUNCH(128, 2, false, 2);
  if (qk.enabled) TAAC_LIN_LAUNCH(128, 2, false, 1);
  if (residual) TAAC_LIN_LAUNCH(128, 1, true, 0);
  TAAC_LIN_LAUNCH(128, 2, false, 0);
#undef TAAC_LIN_LAUNCH
}

// rstd[which][row] = rsqrt(sum over the `parts` chunks of the query (which = 0) / key (1) projection / d_model + eps).
__global__ __launch_bounds__(256) void row_rstd_kernel(const float* __restrict__ sumsq, float* __restrict__ rstd,
                                                       int64_t M, int parts, float inv_cols, float eps,
                                                       const int32_t* __restrict__ rows,
                                                       const int32_t* __restrict__ n_rows) {
  const int64_t count = rows ? static_cast<int64_t>(*n_rows) : M;
  const int64_t unit = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t slot = unit >> 1;
  const int which = static_cast<int>(unit & 1);
  if (slot >= count) return;
  const int64_t row = rows ? static_cast<int64_t>(rows[slot]) : slot;
  float ss = 0.f;
  for (int c = 0; c < parts; ++c) ss += sumsq[(static_cast<int64_t>(which) * parts + c) * M + row];
  rstd[which * M + row] = rsqrtf(ss * inv_cols + eps);
}

}  // namespace
}  // namespace taac

extern "C" int taac_norm_linear_heads_fwd(const void* x, int64_t ldx, const void* norm_weight, float eps, const void* bias,
                                          const void* packed_weights, void* out, int32_t head_dim, int64_t M, int32_t N,
                                          int32_t K, const int32_t* rows, const int32_t* n_rows, int norm_folded,
                                          void* stream) {
  const char* name = "taac_norm_linear_heads_fwd";
  if (!packed_weights) return taac::set_error(TAAC_ERR_INVALID_VALUE, "%s: the weights must be packed", name);
  if (head_dim != 32 && head_dim != 64)
    return taac::set_error(TAAC_ERR_UNSUPPORTED, "%s: head_dim must be 32 or 64 (got %d)", name, head_dim);
  return taac::norm_linear_launch(name, x, ldx, norm_weight, eps, nullptr, bias, packed_weights, nullptr, 0, out, N, M, N,
                                  K, rows, n_rows, nullptr, taac::QkExtras{}, norm_folded, stream, head_dim);
}

extern "C" int taac_attn_out_ffn_heads_fwd(const void* attn, int32_t head_dim, const void* out_bias,
                                           const void* packed_out_weights, const void* residual, int64_t ldr,
                                           const void* norm_weight, float eps, const void* b_up, const void* b_down,
                                           const void* packed_ffn_weights, void* out, int64_t ldo, int64_t M, int32_t D,
                                           int32_t F, const int32_t* rows, const int32_t* n_rows, int norm_folded,
                                           void* stream) {
  const char* name = "taac_attn_out_ffn_heads_fwd";
  if (!packed_out_weights || !packed_ffn_weights)
    return taac::set_error(TAAC_ERR_INVALID_VALUE, "%s: both weight sets must be packed", name);
  if (head_dim != 32 && head_dim != 64)
    return taac::set_error(TAAC_ERR_UNSUPPORTED, "%s: head_dim must be 32 or 64 (got %d)", name, head_dim);
  return taac::ffn_entry(name, attn, D, out_bias, packed_out_weights, norm_weight, eps, nullptr, b_up, nullptr, b_down,
                         packed_ffn_weights, residual, ldr, out, ldo, M, D, F, 1, rows, n_rows, nullptr, norm_folded,
                         stream, nullptr, 0, true, head_dim);
}

namespace taac {
// taac_norm_linear_qk_fwd (packed weights) writing q | k | v as per-head planes like taac_norm_linear_heads_fwd.
int norm_linear_qk_heads(const void* x, int64_t ldx, const void* norm_weight, float eps, const void* bias,
                         const void* packed_weights, void* out, int64_t M, int32_t d_model, int32_t num_heads,
                         int32_t tokens_per_sample, const void* qk_weight, const void* cos_sin, float* qk_sumsq,
                         const int32_t* rows, const int32_t* n_rows, int norm_folded, void* stream) {
  QkExtras qk;
  qk.enabled = true;
  qk.qk_weight = qk_weight;
  qk.cos_sin = cos_sin;
  qk.qk_sumsq = qk_sumsq;
  qk.qk_chunks = 2 * d_model / kNC;
  qk.head_dim = d_model / num_heads;
  qk.tokens_per_sample = tokens_per_sample;
  return norm_linear_launch("taac_backbone_fwd", x, ldx, norm_weight, eps, nullptr, bias, packed_weights, nullptr, 0, out,
                            3 * d_model, M, 3 * d_model, d_model, rows, n_rows, nullptr, qk, norm_folded, stream,
                            d_model / num_heads);
}

// taac_attn_out_ffn_fwd (attn_plane = 0) / taac_attn_out_ffn_heads_fwd (attn_plane = head_dim) that also leaves, for every
// token it stores, the dot product of the output row with head_w in token_dots[row] (see TsParams::head_w).
int attn_out_ffn_readout(const void* attn, int64_t ld_attn, int attn_plane, const void* out_bias,
                         const void* packed_out_weights, const void* residual, int64_t ldr, const void* norm_weight,
                         float eps, const void* b_up, const void* b_down, const void* packed_ffn_weights, void* out,
                         int64_t ldo, int64_t M, int32_t D, int32_t F, const int32_t* rows, const int32_t* n_rows,
                         int norm_folded, const void* head_w, float* token_dots, void* stream) {
  return ffn_entry("taac_backbone_fwd", attn, ld_attn, out_bias, packed_out_weights, norm_weight, eps, nullptr, b_up, nullptr,
                   b_down, packed_ffn_weights, residual, ldr, out, ldo, M, D, F, 1, rows, n_rows, nullptr, norm_folded,
                   stream, nullptr, 0, true, attn_plane, head_w, token_dots);
}

// Whether the kernels take the activation's constants from the packed weights at this shape: the gated form with the
// deferred down projection (three weight buffers next to the biases; the out projection's bias counted in).
bool ffn_act_fold_supported(int32_t D, int32_t F) {
  if ((D != 128 && D != 256) || F <= 0 || F % (kHU * kCPB) != 0) return false;
  const size_t buffer_bytes = static_cast<size_t>(kCPB * (D / 16 + D / 32)) * kFrag;
  return 3 * buffer_bytes + static_cast<size_t>(2 * F + 3 * D) * 2 <= static_cast<size_t>(kMaxLdsBytes);
}
}  // namespace taac

extern "C" int taac_norm_linear_fwd(const void* x, int64_t ldx, const void* norm_weight, float eps, const void* w,
                                    const void* bias, const void* packed_weights, const void* residual, int64_t ldr,
                                    void* out, int64_t ldo, int64_t M, int32_t N, int32_t K, const int32_t* rows,
                                    const int32_t* n_rows, const int32_t* x_rows, int norm_folded, void* stream) {
  return taac::norm_linear_launch("taac_norm_linear_fwd", x, ldx, norm_weight, eps, w, bias, packed_weights, residual,
                                  ldr, out, ldo, M, N, K, rows, n_rows, x_rows, taac::QkExtras{}, norm_folded, stream);
}

extern "C" int taac_norm_linear_qk_fwd(const void* x, int64_t ldx, const void* norm_weight, float eps, const void* w,
                                       const void* bias, const void* packed_weights, void* out, int64_t ldo, int64_t M,
                                       int32_t d_model, int32_t num_heads, int32_t tokens_per_sample,
                                       const void* qk_weight, const void* cos_sin, float* qk_sumsq,
                                       const int32_t* rows, const int32_t* n_rows, const int32_t* x_rows,
                                       int norm_folded, void* stream) {
  using namespace taac;
  const char* name = "taac_norm_linear_qk_fwd";
  if (d_model <= 0 || num_heads <= 0 || tokens_per_sample <= 0 || d_model % num_heads != 0)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: d_model, num_heads, tokens_per_sample > 0 and d_model divisible by num_heads", name);
  if (d_model % kNC != 0) return set_error(TAAC_ERR_UNSUPPORTED, "%s: d_model must be a multiple of %d", name, kNC);
  if (cos_sin && (d_model / num_heads) % 8 != 0)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: with a rotary table head_dim must be a multiple of 8", name);
  if (!qk_sumsq && !qk_weight && !cos_sin)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: nothing to do for the query and key features", name);
  QkExtras qk;
  qk.enabled = true;
  qk.qk_weight = qk_weight;
  qk.cos_sin = cos_sin;
  qk.qk_sumsq = qk_sumsq;
  qk.qk_chunks = 2 * d_model / kNC;
  qk.head_dim = d_model / num_heads;
  qk.tokens_per_sample = tokens_per_sample;
  return norm_linear_launch(name, x, ldx, norm_weight, eps, w, bias, packed_weights, nullptr, 0, out, ldo, M,
                            3 * d_model, d_model, rows, n_rows, x_rows, qk, norm_folded, stream);
}

extern "C" int taac_row_rstd(const float* qk_sumsq, int64_t M, int32_t d_model, float eps, float* rstd,
                             const int32_t* rows, const int32_t* n_rows, void* stream) {
  using namespace taac;
  const char* name = "taac_row_rstd";
  if (M < 0 || d_model <= 0 || d_model % kNC != 0)
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: M >= 0 and d_model a positive multiple of %d required", name, kNC);
  if (M == 0) return TAAC_OK;
  if (!qk_sumsq || !rstd) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  if ((rows == nullptr) != (n_rows == nullptr))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: rows and n_rows must be given together", name);
  if (M > 0x3fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: at most 2^30 rows", name);
  const int64_t blocks = (2 * M + 255) / 256;
  hipLaunchKernelGGL(row_rstd_kernel, dim3(static_cast<uint32_t>(blocks)), dim3(256), 0, as_stream(stream), qk_sumsq,
                     rstd, M, d_model / kNC, 1.0f / static_cast<float>(d_model), eps, rows, n_rows);
  return check_launch(name);
}
