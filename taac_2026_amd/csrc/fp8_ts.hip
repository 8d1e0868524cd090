// Token-stationary FP8 (OCP e4m3fn, per-tensor scales) dense layer for K = 256 on gfx950:
//   out = epilogue( (q(a) q(w)^T) * (amax_a / 448) * (amax_w / 448) + bias )
// with q(a) formed while the token rows are loaded (bf16 activations) or taken as given (e4m3 activations), and the
// epilogues of taac_linear_fp8 (none / + residual / SiLU-gate).
//
// Same scheme as the bf16 token-stationary linear kernel: a persistent workgroup of 8 wavefronts owns 512 tokens at a
// time (two 32-token tiles per wavefront; one with the residual epilogue); each wavefront quantises its rows once into MFMA B-operand fragments
// (v_mfma_scale_f32_32x32x64_f8f6f4: lane (l32, hh) holds the 32 bytes k = 64*ks + 32*hh .. +31 of token l32) and keeps
// them in 64 registers; the e4m3 weights stream L2 -> LDS by DMA, 64 weight rows per step, through a ring of three
// buffers two steps ahead of their use. A fragment (32 rows x 64 k) is 2 KB in LDS: two 1 KB halves, each written by
// one DMA instruction (lane l -> row l % 32, bytes 64*ks + 32*(l / 32) + 16*half .. +15) and read back with one
// ds_read_b128 per half. The weights stay in their [N, K] row-major layout.
//
// Epilogue: dequantisation, bias and SiLU-gate in fp32 on the accumulators, which then cross a wavefront-private fp32
// LDS tile so that every lane ends up with 8 consecutive features of one token; the residual is added there in fp32
// and the sum is rounded to bf16 once, like the tiled kernel of linear.hip does.
//
// Vector-memory discipline as in the bf16 kernel (operations complete in issue order; counts per wavefront and step):
//   [RES: NST residual loads of step s+1] [2 weight DMAs of step s+2] ... [NST stores of step s]; the step ends with
//   a hand-written vmcnt(2 + NST) (vmcnt(NST) when no DMA was issued) for the weights of step s+1. Rows beyond M are
//   clamped to row M-1 for loads and stores, so every wavefront issues the same number of operations.
#include <cstdlib>

#include "common.h"
#include "ts_common.h"

namespace taac {
namespace {

constexpr int kFrag8 = 2048;             // bytes of one 32 x 64 e4m3 fragment
constexpr int kWaves = 8;
// Per reduction length K: 32-row weight blocks per step (two for K = 256, one for K = 1024, whose fragments are four
// times as many), and the epilogue tile of a wavefront (fp32, 32 tokens x 32 features per row block + 16 bytes pad).
constexpr int row_blocks(int K) { return K <= 256 ? 2 : 1; }
constexpr int tile_row_bytes(int K) { return row_blocks(K) * 32 * 4 + 16; }
constexpr int step_bytes(int K) { return row_blocks(K) * (K / 64) * kFrag8; }
constexpr int kScaleOne = 127;           // E8M0 exponent of 1.0 for the block-scale operands of the f8f6f4 MFMA

// 32-token tiles per wavefront: two (every weight fragment read from LDS feeds two MFMAs) for K = 256 without a
// residual; one with the residual epilogue, whose double-buffered residual pieces would not fit the register file next
// to two tiles, and for K = 1024, where one tile's fragments already take 128 registers.
constexpr int tiles_per_wave(int K, int epilogue) { return (epilogue == TAAC_EPI_RESIDUAL || K > 256) ? 1 : 2; }

struct Fp8TsParams {
  const void* a;            // [M, K] bf16 or e4m3, row stride lda (elements)
  const uint8_t* w;         // [N, K] e4m3
  const bf16_t* bias;       // [N] or null
  const bf16_t* residual;   // [M, N] row stride ldo, or null
  bf16_t* out;              // [M, N] (SwiGLU: [M, N / 2]) row stride ldo
  const float* amax_a;
  const float* amax_w;
  int64_t M, lda, ldo, ldr;
  int32_t N;                // weight rows
  int32_t gate_first;
  // taac_norm_linear_fp8_fwd only:
  const bf16_t* norm_w;     // [K] RMSNorm weight applied to the rows before quantisation, or null
  float eps;
  const int32_t* rows;      // optional row index: token i lives in row rows[i] of a / residual / out
  const int32_t* n_rows;    // with rows: device pointer to the number of tokens
  float* amax_out;          // STATS: receives max |bf16(rmsnorm(out, out_norm_w))| (max |out| without a weight)
  const bf16_t* out_norm_w; // [N] or null
  float out_eps;
};

__device__ __forceinline__ float clamp448(float x) { return __builtin_fminf(__builtin_fmaxf(x, -448.f), 448.f); }

// 8 bf16 -> 8 e4m3 bytes (two dwords), value * inv_scale, saturating, round to nearest even.
__device__ __forceinline__ void quant8(const bf16x8& v, float inv_scale, int& lo, int& hi) {
  float f[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) f[e] = clamp448(static_cast<float>(v[e]) * inv_scale);
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], 0, false);
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], lo, true);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], 0, false);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], hi, true);
}

__device__ __forceinline__ float silu_f(float v) {
  return v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * v));
}

template <int OFFSET>
__device__ __forceinline__ void lds_read16(u32x4& dst, uint32_t addr) {
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFFSET) : "memory");
}
template <int N>
__device__ __forceinline__ void lds_wait_halves(u32x4& a, u32x4& b) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N) : "memory");
}

// STATS (taac_norm_linear_fp8_fwd): the epilogue also reduces, per token, the sum of squares and max |out * weight| of
// the rounded output over the steps of a tile, and from them the maximum over all tokens of |rmsnorm(out) * weight| - the
// per-tensor scale of the layer that consumes the output - without a pass of its own over it.
// NORM: the rows are RMS-normalised (weight p.norm_w) before they are quantised.
template <int kK, int EPI, bool A_FP8, bool STATS, bool NORM = false>
__global__ __launch_bounds__(kWaves * kWave, 2) void linear_fp8_ts_kernel(const Fp8TsParams p, const int /*max_tiles*/) {
  static_assert(!NORM || (kK == 256 && !A_FP8), "the normalisation is built for bf16 rows of 256 features");
  constexpr bool RES = EPI == TAAC_EPI_RESIDUAL;
  constexpr int kTT = tiles_per_wave(kK, EPI);
  constexpr int kTokPerWg = kWaves * 32 * kTT;
  constexpr bool GLU = EPI == TAAC_EPI_SWIGLU;
  constexpr int kKS = kK / 64;                    // k-steps of the fp8 MFMA
  constexpr int RB = row_blocks(kK);              // 32-row weight blocks per step
  constexpr int kRows = RB * 32;                  // weight rows per step
  constexpr int kNFrag = RB * kKS;                // fragments per step
  constexpr int kBuf8 = step_bytes(kK);
  constexpr int FPW = kNFrag * 2 / kWaves;        // DMA instructions per wavefront and step
  constexpr int kTileRow = tile_row_bytes(kK);
  constexpr int kTileWave = 32 * kTileRow;
  static_assert(!GLU || RB == 2, "the SiLU-gate epilogue pairs two row blocks");
  static_assert(kNFrag * 2 % kWaves == 0, "the DMA instructions of a step divide over the wavefronts");
  constexpr int OUTC = GLU ? 32 : kRows;          // output features per step
  constexpr int PIECES = OUTC / 8;                // 16-byte output pieces per token row
  constexpr int ROWS_PER_STORE = kWave / PIECES;  // token rows covered by one store instruction
  constexpr int NSTT = 32 / ROWS_PER_STORE;       // stores per 32-token tile
  constexpr int NST = NSTT * kTT;                 // stores (and residual pieces) per wavefront and step
  constexpr int P = 4;             // fragments in flight
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  uint8_t* tiles = smem + 3 * kBuf8;
  bf16_t* bias_lds = reinterpret_cast<bf16_t*>(tiles + kWaves * kTileWave);

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int lane = tid % kWave;
  const int l32 = lane % 32;
  const int hh = lane / 32;
  const int F = p.N / 2;
  const int nsteps_tile = GLU ? F / 32 : p.N / kRows;
  // tokens: M, or the device-side count of a row index
  int64_t count = p.M;
  if (p.rows != nullptr) {
    const int64_t n = *p.n_rows;
    count = n < p.M ? n : p.M;
  }
  const int num_tiles = static_cast<int>((count + kTokPerWg - 1) / kTokPerWg);
  const int my_tiles = (num_tiles - static_cast<int>(blockIdx.x) + static_cast<int>(gridDim.x) - 1) /
                       static_cast<int>(gridDim.x);
  if (my_tiles <= 0) return;  // whole workgroup: no tile for it (fewer tokens than the grid was sized for)
  const int total = my_tiles * nsteps_tile;
  // memory row of token `tok`; tokens at or beyond the count repeat the last one (same values, benign duplicate stores)
  auto row_of = [&](int64_t tok) -> int64_t {
    tok = tok < count ? tok : count - 1;
    return p.rows != nullptr ? static_cast<int64_t>(p.rows[tok]) : tok;
  };
  bf16_t* normw_lds = bias_lds + p.N;           // [K] (taac_norm_linear_fp8_fwd)
  bf16_t* outw_lds = normw_lds + kK;            // [N]
  float* red = reinterpret_cast<float*>(outw_lds + p.N);

  const float amax_a = fmaxf(*p.amax_a, 1e-12f);
  const float amax_w = fmaxf(*p.amax_w, 1e-12f);
  const float inv_scale_a = 448.0f / amax_a;
  const float dq = (amax_a / 448.0f) * (amax_w / 448.0f);

  // First weight row of row block rb in step `chunk`: plain layers walk the rows 64 at a time; the SiLU-gate layer pairs
  // 32 rows of the gated half (block 0) with the matching 32 rows of the other half (block 1).
  auto block_row0 = [&](int chunk, int rb) -> int {
    if (GLU) return ((rb == 0) == (p.gate_first != 0) ? 0 : F) + chunk * 32;
    return chunk * kRows + rb * 32;
  };
  // DMA instruction d of a step (two per fragment) moves half d % 2 of fragment d / 2 = (row block f / KS, k-step
  // f % KS); wavefront w issues instructions w * FPW .. + FPW - 1.
  auto stage = [&](int chunk, int buf) {
    int ln = lane;
    asm volatile("" : "+v"(ln));
    const uint32_t lane_off = static_cast<uint32_t>((ln & 31) * kK + (ln >> 5) * 32);
#pragma unroll
    for (int i = 0; i < FPW; ++i) {
      const int d = wave * FPW + i;  // wavefront-uniform
      const int f = d / 2, half = d % 2;
      const uint8_t* src = p.w + static_cast<int64_t>(block_row0(chunk, f / kKS)) * kK + (f % kKS) * 64 + half * 16 + lane_off;
      lds_dma16(src, smem + buf * kBuf8 + f * kFrag8 + half * 1024);
    }
  };
  auto rows_of_tile = [&](int idx) -> int64_t {
    return (static_cast<int64_t>(blockIdx.x) + static_cast<int64_t>(idx) * gridDim.x) * kTokPerWg + wave * (32 * kTT);
  };
  // Residual pieces in the layout of the epilogue stores: piece t*NSTT + i = token 32*t + ROWS_PER_STORE*i +
  // lane / PIECES, features 8 * (lane % PIECES) .. +7 of the step's OUTC features.
  auto request_residual = [&](int64_t tok_base, int chunk, bf16x8 (&res)[NST]) {
#pragma unroll
    for (int i = 0; i < NST; ++i) {
      const int64_t row = row_of(tok_base + (i / NSTT) * 32 + (i % NSTT) * ROWS_PER_STORE + lane / PIECES);
      res[i] = *reinterpret_cast<const bf16x8*>(p.residual + row * p.ldr + chunk * OUTC + (lane % PIECES) * 8);
    }
  };
  // Token rows -> e4m3 B-operand fragments.
  i32x8 xq[kTT][kKS];
  auto load_tile = [&](int64_t tok_base) {
#pragma unroll
    for (int t = 0; t < kTT; ++t) {
      const int64_t tok = row_of(tok_base + t * 32 + l32);
      if (A_FP8) {
        const uint8_t* row = static_cast<const uint8_t*>(p.a) + tok * p.lda + hh * 32;
#pragma unroll
        for (int ks = 0; ks < kKS; ++ks) {
          const u32x4 lo = *reinterpret_cast<const u32x4*>(row + ks * 64);
          const u32x4 hi = *reinterpret_cast<const u32x4*>(row + ks * 64 + 16);
          xq[t][ks] = i32x8{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
        }
      } else {
        const bf16_t* row = static_cast<const bf16_t*>(p.a) + tok * p.lda + hh * 32;
        // Four k-steps (16 loads, 64 registers) at a time: load, then quantise.
#pragma unroll
        for (int k4 = 0; k4 < kKS; k4 += 4) {
          bf16x8 raw[4][4];
#pragma unroll
          for (int ks = 0; ks < 4; ++ks)
#pragma unroll
            for (int c = 0; c < 4; ++c) raw[ks][c] = *reinterpret_cast<const bf16x8*>(row + (k4 + ks) * 64 + c * 8);
          if constexpr (NORM) {
            // RMSNorm of the row (a lane and its partner lane ^ 32 hold its two halves), rounded to bf16 as the
            // stand-alone norm rounds its output, then quantised
            float ss = 0.f;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
#pragma unroll
              for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                  const float v = static_cast<float>(raw[ks][c][e]);
                  ss = fmaf(v, v, ss);
                }
            const uint32_t ssb = __builtin_bit_cast(uint32_t, ss);
            const auto sw = __builtin_amdgcn_permlane32_swap(ssb, ssb, false, false);
            ss = __builtin_bit_cast(float, static_cast<uint32_t>(sw[0])) + __builtin_bit_cast(float, static_cast<uint32_t>(sw[1]));
            const float scale = rsqrtf(ss * (1.0f / kK) + p.eps);
            // opaque here: otherwise the fp32 copies of the first sweep are kept alive for the second one
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
#pragma unroll
              for (int c = 0; c < 4; ++c) asm volatile("" : "+v"(raw[ks][c]));
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
#pragma unroll
              for (int c = 0; c < 4; ++c) {
                const bf16x8 wv = *reinterpret_cast<const bf16x8*>(normw_lds + ks * 64 + hh * 32 + c * 8);
#pragma unroll
                for (int e = 0; e < 8; ++e)
                  raw[ks][c][e] = static_cast<bf16_t>(static_cast<float>(raw[ks][c][e]) * scale * static_cast<float>(wv[e]));
              }
          }
#pragma unroll
          for (int ks = 0; ks < 4; ++ks) {
            int q[8];
#pragma unroll
            for (int c = 0; c < 4; ++c) quant8(raw[ks][c], inv_scale_a, q[2 * c], q[2 * c + 1]);
            xq[t][k4 + ks] = i32x8{q[0], q[1], q[2], q[3], q[4], q[5], q[6], q[7]};
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    // Consume the fragments here, so that the compiler's wait for the loads sits in this (once per tile) path and
    // not in front of the first MFMA of every step.
#pragma unroll
    for (int t = 0; t < kTT; ++t)
#pragma unroll
      for (int ks = 0; ks < kKS; ++ks) asm volatile("" : "+v"(xq[t][ks]));
  };

  bf16x8 res_cur[NST], res_next[NST];
  int tile_idx = 0;
  int64_t tok_wave = rows_of_tile(0);
  stage(0, 0);
  if (total > 1) stage(nsteps_tile > 1 ? 1 : 0, 1);
  if (RES) request_residual(tok_wave, 0, res_cur);
  stage_bias(p.bias, bias_lds, p.N, tid, kWaves * kWave);
  if constexpr (NORM) {
    stage_bias(p.norm_w, normw_lds, kK, tid, kWaves * kWave);
    __syncthreads();  // the first tile is normalised before the common barrier below
  }
  if (STATS) stage_bias(p.out_norm_w, outw_lds, p.N, tid, kWaves * kWave);
  load_tile(tok_wave);
  vm_wait<0>();
  __syncthreads();
  // STATS: per piece slot (token of the epilogue layout) the sum of squares and max |value * weight| over the tile's steps
  [[maybe_unused]] float st_ss[NST], st_mw[NST];
  [[maybe_unused]] float st_max = 0.f;
#pragma unroll
  for (int i = 0; i < NST; ++i) st_ss[i] = st_mw[i] = 0.f;

  uint8_t* tile_lds = tiles + wave * kTileWave;
  int chunk = 0;                    // step inside the tile
  int buf = 0;                      // ring slot of step s
  int chunk2 = 2 % nsteps_tile;     // step s + 2 inside its tile
  for (int s = 0; s < total; ++s) {
    const bool has_next = s + 1 < total;
    const bool stage_ahead = s + 2 < total;
    const bool new_tile = s > 0 && chunk == 0;
    if (new_tile) tok_wave = rows_of_tile(++tile_idx);
    if (RES && has_next) {
      const int next_chunk = chunk + 1 == nsteps_tile ? 0 : chunk + 1;
      request_residual(next_chunk == 0 ? rows_of_tile(tile_idx + 1) : tok_wave, next_chunk, res_next);
    }
    if (stage_ahead) stage(chunk2, buf == 0 ? 2 : buf - 1);  // slot (s + 2) % 3, last read in step s - 1
    if (new_tile) load_tile(tok_wave);

    // ---- the products of this step: fragment stream (ks, rb) = (i / RB, i % RB), LDS fragment index rb * KS + ks -----
    const uint32_t wb = lds_offset(smem) + buf * kBuf8 + lane * 16;
    f32x16 acc[RB][kTT];
    u32x4 rlo[P], rhi[P];
    auto read_frag = [&](auto ic, int slot) {
      constexpr int i = decltype(ic)::value;
      constexpr int f = (i % RB) * kKS + i / RB;
      lds_read16<f * kFrag8>(rlo[slot], wb);
      lds_read16<f * kFrag8 + 1024>(rhi[slot], wb);
    };
    static_for<P>([&](auto ic) { read_frag(ic, decltype(ic)::value); });
    static_for<kNFrag>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      constexpr int ks = i / RB, rb = i % RB;
      constexpr int after = 2 * (P - 1 < kNFrag - 1 - i ? P - 1 : kNFrag - 1 - i);
      lds_wait_halves<after>(rlo[i % P], rhi[i % P]);
      const u32x4 lo = rlo[i % P], hi = rhi[i % P];
      const i32x8 wf = {(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
#pragma unroll
      for (int t = 0; t < kTT; ++t) {
        if constexpr (ks == 0) {
          const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
          acc[rb][t] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf, xq[t][ks], zero, 0, 0, 0, kScaleOne, 0, kScaleOne);
        } else {
          acc[rb][t] =
              __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf, xq[t][ks], acc[rb][t], 0, 0, 0, kScaleOne, 0, kScaleOne);
        }
        // The product has no side effect, so instruction selection may sink a whole accumulation chain below the LDS reads
        // that follow it and keep every fragment of the step live at once; this empty statement keeps it in place.
        asm volatile("" : "+v"(acc[rb][t]));
      }
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (i + P < kNFrag) read_frag(std::integral_constant<int, i + P>{}, i % P);
    });

    // ---- epilogue: dequantise, bias, gate; fp32 tile transpose; residual; one rounding; NST stores -------------------
    // Accumulator register jq*4 + e of lane (l32, hh) is row jq*8 + hh*4 + e of its 32-row block, token l32.
    bf16x4 bv[4 * RB];
#pragma unroll
    for (int q = 0; q < 4 * RB; ++q)
      bv[q] = *reinterpret_cast<const bf16x4*>(bias_lds + block_row0(chunk, q / 4) + (q % 4) * 8 + hh * 4);
#pragma unroll
    for (int t = 0; t < kTT; ++t) {
#pragma unroll
      for (int jq = 0; jq < 4; ++jq) {
        f32x4 v[RB];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
          for (int e = 0; e < 4; ++e) v[rb][e] = acc[rb][t][jq * 4 + e] * dq + static_cast<float>(bv[rb * 4 + jq][e]);
        if constexpr (GLU) {
#pragma unroll
          for (int e = 0; e < 4; ++e) v[0][e] = silu_f(v[0][e]) * v[1][e];
          *reinterpret_cast<f32x4*>(tile_lds + l32 * kTileRow + (jq * 8 + hh * 4) * 4) = v[0];
        } else {
#pragma unroll
          for (int rb = 0; rb < RB; ++rb)
            *reinterpret_cast<f32x4*>(tile_lds + l32 * kTileRow + (rb * 32 + jq * 8 + hh * 4) * 4) = v[rb];
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
      for (int i = 0; i < NSTT; ++i) {
        const int row = i * ROWS_PER_STORE + lane / PIECES;
        const int64_t tok = row_of(tok_wave + t * 32 + row);
        const f32x4 a0 = *reinterpret_cast<const f32x4*>(tile_lds + row * kTileRow + (lane % PIECES) * 32);
        const f32x4 a1 = *reinterpret_cast<const f32x4*>(tile_lds + row * kTileRow + (lane % PIECES) * 32 + 16);
        bf16x8 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float x0 = a0[e], x1 = a1[e];
          if (RES) {
            x0 += static_cast<float>(res_cur[t * NSTT + i][e]);
            x1 += static_cast<float>(res_cur[t * NSTT + i][4 + e]);
          }
          o[e] = static_cast<bf16_t>(x0);
          o[4 + e] = static_cast<bf16_t>(x1);
        }
        __builtin_nontemporal_store(o, reinterpret_cast<bf16x8*>(p.out + tok * p.ldo + chunk * OUTC + (lane % PIECES) * 8));
        if constexpr (STATS) {
          const bf16x8 wv = *reinterpret_cast<const bf16x8*>(outw_lds + chunk * OUTC + (lane % PIECES) * 8);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float r = static_cast<float>(o[e]);
            st_ss[t * NSTT + i] = fmaf(r, r, st_ss[t * NSTT + i]);
            const float rw = p.out_norm_w != nullptr ? r * static_cast<float>(wv[e]) : r;
            st_mw[t * NSTT + i] = fmaxf(st_mw[t * NSTT + i], fabsf(rw));
          }
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    if constexpr (STATS) {
      if (chunk == nsteps_tile - 1) {  // the tile is complete: a token's statistics are spread over PIECES lanes
#pragma unroll
        for (int i = 0; i < NST; ++i) {
          float ss = st_ss[i], mw = st_mw[i];
#pragma unroll
          for (int off = 1; off < PIECES; off <<= 1) {
            ss += __shfl_xor(ss, off, kWave);
            mw = fmaxf(mw, __shfl_xor(mw, off, kWave));
          }
          const int64_t tok = tok_wave + (i / NSTT) * 32 + (i % NSTT) * ROWS_PER_STORE + lane / PIECES;
          float v = mw;
          if (p.out_norm_w != nullptr)
            v = static_cast<float>(static_cast<bf16_t>(mw * rsqrtf(ss * (1.0f / static_cast<float>(p.N)) + p.out_eps)));
          if (tok < count) st_max = fmaxf(st_max, v);
          st_ss[i] = st_mw[i] = 0.f;
        }
      }
    }
    // ---- close the step ------------------------------------------------------------------------------------------------
    if (has_next) {
      if (stage_ahead) {
        vm_wait<FPW + NST>();
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
    if (++chunk == nsteps_tile) chunk = 0;
    if (++chunk2 == nsteps_tile) chunk2 = 0;
  }
  if constexpr (STATS) {
    // maximum over the workgroup, one atomic on the float's bit pattern (non-negative floats order like their bits)
    st_max = group_max<kWave>(st_max);
    if (lane == 0) red[wave] = st_max;
    __syncthreads();
    if (tid == 0) {
      for (int w = 1; w < kWaves; ++w) st_max = fmaxf(st_max, red[w]);
      if (st_max > __builtin_nontemporal_load(p.amax_out))
        atomicMax(reinterpret_cast<unsigned int*>(p.amax_out), __float_as_uint(st_max));
    }
  }
}

// Launches the token-stationary kernel when the shape fits it: K = 256 (any epilogue, weight rows a multiple of 64) or
// K = 1024 (no SiLU-gate, weight rows a multiple of 32), 16-byte aligned rows. Returns TAAC_OK after a launch, a negative
// status on a launch error and 1 when the shape is not covered (the caller then uses the tiled kernel).
template <int K>
int launch_fp8_ts_for_k(const Fp8TsParams& p, int a_is_fp8, int epilogue, hipStream_t s, const char* name) {
  const size_t lds_bytes = static_cast<size_t>(3 * step_bytes(K)) + static_cast<size_t>(kWaves) * 32 * tile_row_bytes(K) +
                           static_cast<size_t>(p.N) * 2;
  if (lds_bytes > 160 * 1024) return 1;
  const int tok_per_wg = kWaves * 32 * tiles_per_wave(K, epilogue);
  const int64_t tiles64 = (p.M + tok_per_wg - 1) / tok_per_wg;
  if (tiles64 > 0x3fffffffLL) return 1;
  const int num_tiles = static_cast<int>(tiles64);
  const int cus = compute_units();
  if (cus <= 0) return set_error(TAAC_ERR_LAUNCH, "%s: cannot query the device", name);
  int grid = num_tiles < cus ? num_tiles : cus;
  if (const int limit = test_max_workgroups(); limit > 0 && limit < grid) grid = limit;  // taac_test_hooks
#define TAAC_FP8_TS_LAUNCH(EPI, AF8)                                                                                \
  do {                                                                                                              \
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(linear_fp8_ts_kernel<K, EPI, AF8, false>),                       \
                            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)) != hipSuccess) \
      return set_error(TAAC_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS", name, lds_bytes);                    \
    hipLaunchKernelGGL((linear_fp8_ts_kernel<K, EPI, AF8, false>), dim3(grid), dim3(kWaves * kWave), lds_bytes, s, p,      \
                       num_tiles);                                                                                  \
    return check_launch(name);                                                                                      \
  } while (0)
  if (epilogue == TAAC_EPI_NONE) {
    if (a_is_fp8) TAAC_FP8_TS_LAUNCH(TAAC_EPI_NONE, true);
    TAAC_FP8_TS_LAUNCH(TAAC_EPI_NONE, false);
  }
  if (epilogue == TAAC_EPI_RESIDUAL) {
    if (a_is_fp8) TAAC_FP8_TS_LAUNCH(TAAC_EPI_RESIDUAL, true);
    TAAC_FP8_TS_LAUNCH(TAAC_EPI_RESIDUAL, false);
  }
  if constexpr (row_blocks(K) == 2) {
    if (a_is_fp8) TAAC_FP8_TS_LAUNCH(TAAC_EPI_SWIGLU, true);
    TAAC_FP8_TS_LAUNCH(TAAC_EPI_SWIGLU, false);
  }
  return 1;
#undef TAAC_FP8_TS_LAUNCH
}

}  // namespace

int launch_linear_fp8_ts(const void* a, int a_is_fp8, int64_t lda, const void* w, const float* amax_a,
                         const float* amax_w, const void* bias, const void* residual, void* out, int64_t ldo,
                         int64_t M, int32_t N, int32_t K, int epilogue, int gate_first, hipStream_t s,
                         const char* name) {
  if ((K != 256 && K != 1024) || M <= 0) return 1;
  if (N % (row_blocks(K) * 32) != 0) return 1;
  if (K == 1024 && epilogue == TAAC_EPI_SWIGLU) return 1;
  if (lda % (a_is_fp8 ? 16 : 8) != 0 || ldo % 8 != 0 || (reinterpret_cast<uintptr_t>(bias) & 15u)) return 1;
  if (test_fp8_tiled()) return 1;  // taac_test_hooks: force the tiled kernel
  Fp8TsParams p{};
  p.a = a;
  p.w = static_cast<const uint8_t*>(w);
  p.bias = static_cast<const bf16_t*>(bias);
  p.residual = static_cast<const bf16_t*>(residual);
  p.out = static_cast<bf16_t*>(out);
  p.amax_a = amax_a;
  p.amax_w = amax_w;
  p.M = M;
  p.lda = lda;
  p.ldo = ldo;
  p.ldr = ldo;
  p.N = N;
  p.gate_first = gate_first ? 1 : 0;
  if (K == 256) return launch_fp8_ts_for_k<256>(p, a_is_fp8, epilogue, s, name);
  return launch_fp8_ts_for_k<1024>(p, a_is_fp8, epilogue, s, name);
}

}  // namespace taac

namespace taac {
namespace {
__global__ void fp8_ts_clear_kernel(float* a) {
  if (threadIdx.x == 0 && blockIdx.x == 0) *a = 0.f;
}
}  // namespace
}  // namespace taac

extern "C" int taac_norm_linear_fp8_fwd(const void* x, int64_t ldx, const void* norm_weight, float eps, const void* w_fp8,
                                        const void* bias, const float* amax_x, const float* amax_w, const void* residual,
                                        int64_t ldr, void* out, int64_t ldo, int64_t M, int32_t N, int32_t K,
                                        const int32_t* rows, const int32_t* n_rows, const void* out_norm_weight,
                                        float out_eps, float* amax_out, void* stream) {
  using namespace taac;
  const char* name = "taac_norm_linear_fp8_fwd";
  if (M < 0 || N <= 0 || K <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: M must be >= 0, N and K > 0", name);
  if (K != 256) return set_error(TAAC_ERR_UNSUPPORTED, "%s: built for K = 256 (got %d)", name, K);
  if (N % 64 != 0) return set_error(TAAC_ERR_UNSUPPORTED, "%s: N=%d must be a multiple of 64", name, N);
  if (ldx < K || ldo < N || (residual && ldr < N) || ldx % 8 || ldo % 8 || (residual && ldr % 8))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: row strides must cover a row and be multiples of 8", name);
  if (!amax_x || !amax_w) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null scale pointer", name);
  if ((rows == nullptr) != (n_rows == nullptr))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: rows and n_rows must be given together", name);
  if (out_norm_weight && !amax_out) return set_error(TAAC_ERR_INVALID_VALUE, "%s: out_norm_weight without amax_out", name);
  hipStream_t s = as_stream(stream);
  if (amax_out != nullptr && !maxima_precleared) {
    hipLaunchKernelGGL(fp8_ts_clear_kernel, dim3(1), dim3(kWave), 0, s, amax_out);
    const int rc = check_launch(name);
    if (rc != TAAC_OK) return rc;
  }
  if (M == 0) return TAAC_OK;
  if (!x || !w_fp8 || !out) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  if (M > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: at most 2^31 rows", name);
  const void* ptrs[7] = {x, w_fp8, out, residual, bias, norm_weight, out_norm_weight};
  for (const void* ptr : ptrs)
    if (reinterpret_cast<uintptr_t>(ptr) & 15u)
      return set_error(TAAC_ERR_UNSUPPORTED, "%s: tensor base pointers must be 16-byte aligned", name);
  Fp8TsParams p{};
  p.a = x;
  p.w = static_cast<const uint8_t*>(w_fp8);
  p.bias = static_cast<const bf16_t*>(bias);
  p.residual = static_cast<const bf16_t*>(residual);
  p.out = static_cast<bf16_t*>(out);
  p.amax_a = amax_x;
  p.amax_w = amax_w;
  p.M = M;
  p.lda = ldx;
  p.ldo = ldo;
  p.ldr = ldr;
  p.N = N;
  p.norm_w = static_cast<const bf16_t*>(norm_weight);
  p.eps = eps;
  p.rows = rows;
  p.n_rows = n_rows;
  p.amax_out = amax_out;
  p.out_norm_w = static_cast<const bf16_t*>(out_norm_weight);
  p.out_eps = out_eps;
  const int epilogue = residual ? TAAC_EPI_RESIDUAL : TAAC_EPI_NONE;
  const size_t lds_bytes = static_cast<size_t>(3 * step_bytes(256)) + static_cast<size_t>(kWaves) * 32 * tile_row_bytes(256) +
                           static_cast<size_t>(2 * N + 256) * 2 + 64;
  if (lds_bytes > 160 * 1024) return set_error(TAAC_ERR_UNSUPPORTED, "%s: N=%d does not fit the LDS", name, N);
  const int tok_per_wg = kWaves * 32 * tiles_per_wave(256, epilogue);
  const int64_t tiles64 = (M + tok_per_wg - 1) / tok_per_wg;
  const int num_tiles = static_cast<int>(tiles64);
  const int cus = compute_units();
  if (cus <= 0) return set_error(TAAC_ERR_LAUNCH, "%s: cannot query the device", name);
  int grid = num_tiles < cus ? num_tiles : cus;
  if (const int limit = test_max_workgroups(); limit > 0 && limit < grid) grid = limit;  // taac_test_hooks
#define TAAC_NL_FP8(EPI, ST, NM)                                                                                          \
  do {                                                                                                                    \
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(linear_fp8_ts_kernel<256, EPI, false, ST, NM>),                 \
                            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)) != hipSuccess)       \
      return set_error(TAAC_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS", name, lds_bytes);                          \
    hipLaunchKernelGGL((linear_fp8_ts_kernel<256, EPI, false, ST, NM>), dim3(grid), dim3(kWaves * kWave), lds_bytes, s, p, \
                       num_tiles);                                                                                        \
    return check_launch(name);                                                                                            \
  } while (0)
#define TAAC_NL_FP8_EPI(EPI)                              \
  do {                                                    \
    if (amax_out && norm_weight) TAAC_NL_FP8(EPI, true, true);   \
    if (amax_out) TAAC_NL_FP8(EPI, true, false);          \
    if (norm_weight) TAAC_NL_FP8(EPI, false, true);       \
    TAAC_NL_FP8(EPI, false, false);                       \
  } while (0)
  if (residual) TAAC_NL_FP8_EPI(TAAC_EPI_RESIDUAL);
  TAAC_NL_FP8_EPI(TAAC_EPI_NONE);
#undef TAAC_NL_FP8_EPI
#undef TAAC_NL_FP8
}
