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
  int64_t M, lda, ldo;
  int32_t N;                // weight rows
  int32_t gate_first;
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

template <int kK, int EPI, bool A_FP8>
__global__ __launch_bounds__(kWaves * kWave, 2) void linear_fp8_ts_kernel(const Fp8TsParams p, const int num_tiles) {
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
  const int my_tiles = (num_tiles - static_cast<int>(blockIdx.x) + static_cast<int>(gridDim.x) - 1) /
                       static_cast<int>(gridDim.x);
  const int total = my_tiles * nsteps_tile;

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
      int64_t tok = tok_base + (i / NSTT) * 32 + (i % NSTT) * ROWS_PER_STORE + lane / PIECES;
      tok = tok < p.M ? tok : p.M - 1;
      res[i] = *reinterpret_cast<const bf16x8*>(p.residual + tok * p.ldo + chunk * OUTC + (lane % PIECES) * 8);
    }
  };
  // Token rows -> e4m3 B-operand fragments.
  i32x8 xq[kTT][kKS];
  auto load_tile = [&](int64_t tok_base) {
#pragma unroll
    for (int t = 0; t < kTT; ++t) {
      int64_t tok = tok_base + t * 32 + l32;
      tok = tok < p.M ? tok : p.M - 1;
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
  load_tile(tok_wave);
  vm_wait<0>();
  __syncthreads();

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
        int64_t tok = tok_wave + t * 32 + row;
        tok = tok < p.M ? tok : p.M - 1;
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
        *reinterpret_cast<bf16x8*>(p.out + tok * p.ldo + chunk * OUTC + (lane % PIECES) * 8) = o;
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
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
  if (const char* cap = getenv("TAAC_TS_MAX_WORKGROUPS")) {  // test hook, as in the bf16 kernel
    const int limit = atoi(cap);
    if (limit > 0 && limit < grid) grid = limit;
  }
#define TAAC_FP8_TS_LAUNCH(EPI, AF8)                                                                                \
  do {                                                                                                              \
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(linear_fp8_ts_kernel<K, EPI, AF8>),                       \
                            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)) != hipSuccess) \
      return set_error(TAAC_ERR_LAUNCH, "%s: cannot reserve %zu bytes of LDS", name, lds_bytes);                    \
    hipLaunchKernelGGL((linear_fp8_ts_kernel<K, EPI, AF8>), dim3(grid), dim3(kWaves * kWave), lds_bytes, s, p,      \
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
  if (getenv("TAAC_FP8_TILED") != nullptr) return 1;  // tuning / test hook: force the tiled kernel
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
  p.N = N;
  p.gate_first = gate_first ? 1 : 0;
  if (K == 256) return launch_fp8_ts_for_k<256>(p, a_is_fp8, epilogue, s, name);
  return launch_fp8_ts_for_k<1024>(p, a_is_fp8, epilogue, s, name);
}

}  // namespace taac
