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
#include <cstdlib>

#include "common.h"

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
};

__device__ __forceinline__ float silu_f(float v) {
  return v * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * v));
}

// 16 bytes per lane from global memory straight into LDS; lane l lands at lds_wave_base + 16 * l.
__device__ __forceinline__ void lds_dma16(const void* gsrc, void* lds_wave_base) {
  __builtin_amdgcn_global_load_lds(gsrc, lds_wave_base, 16, 0, 0);
}

// Hidden unit (0..15) loaded into row slot m16 of the gate (or value) half of an up fragment: chosen so that
// accumulator register j < 8 of lane half hh holds hidden unit 8*hh + j, the k order of a W_down fragment.
__host__ __device__ __forceinline__ int up_unit_of_slot(int m16) {
  return 8 * ((m16 >> 2) & 1) + 4 * (m16 >> 3) + (m16 & 3);
}

// ---- fragment-order packing ------------------------------------------------------------------------------------------
// FFN blob: step s (32 hidden units) holds, for chunk q = 0, 1: KS up fragments (k-step r) then MB down fragments
// (row block r - KS); exactly the image one barrier step needs in LDS. A fragment is 64 lanes x 16 bytes.
__global__ void ffn_pack_kernel(const bf16_t* __restrict__ w_up, const bf16_t* __restrict__ w_down,
                                bf16x8* __restrict__ packed, int D, int F) {
  const int KS = D / 16, MB = D / 32, CFRAG = KS + MB, NFRAG = kCPB * CFRAG;
  const int64_t total = static_cast<int64_t>(F / (kHU * kCPB)) * NFRAG * 64;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (gid >= total) return;
  const int lane = static_cast<int>(gid % 64);
  const int f = static_cast<int>((gid / 64) % NFRAG);
  const int64_t step = gid / 64 / NFRAG;
  const int q = f / CFRAG, r = f % CFRAG;
  const int64_t unit0 = (step * kCPB + q) * kHU;
  const int l32 = lane % 32, hh = lane / 32;
  const bf16_t* src;
  if (r < KS)
    src = w_up + ((l32 >= 16 ? F : 0) + unit0 + up_unit_of_slot(l32 & 15)) * D + r * 16 + hh * 8;
  else
    src = w_down + static_cast<int64_t>((r - KS) * 32 + l32) * F + unit0 + hh * 8;
  packed[gid] = *reinterpret_cast<const bf16x8*>(src);
}

// Linear blob: chunk c (64 output features) holds fragments (row block rb, k-step ks) at index rb * KS + ks.
__global__ void linear_pack_kernel(const bf16_t* __restrict__ w, bf16x8* __restrict__ packed, int N, int K) {
  const int KS = K / 16, NFRAG = 2 * KS;
  const int64_t total = static_cast<int64_t>(N / kNC) * NFRAG * 64;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (gid >= total) return;
  const int lane = static_cast<int>(gid % 64);
  const int f = static_cast<int>((gid / 64) % NFRAG);
  const int64_t chunk = gid / 64 / NFRAG;
  const int l32 = lane % 32, hh = lane / 32;
  const bf16_t* src = w + (chunk * kNC + (f / KS) * 32 + l32) * K + (f % KS) * 16 + hh * 8;
  packed[gid] = *reinterpret_cast<const bf16x8*>(src);
}

// ---- shared pieces ---------------------------------------------------------------------------------------------------

// Loads the wavefront's token rows as B-operand fragments and, if norm_w is given, RMS-normalises them in place:
// y = bf16( x * rsqrt(mean(x^2) + eps) * w ). Lane (l32, hh) holds features 16*ks + 8*hh .. +7 of token l32.
template <int D, int TT>
__device__ __forceinline__ void load_tokens(const TsParams& p, int64_t tok0, int l32, int hh,
                                            bf16x8 (&xf)[TT][D / 16]) {
  constexpr int KS = D / 16;
#pragma unroll
  for (int t = 0; t < TT; ++t) {
    // Rows beyond M are clamped to the last row: their results are computed but never stored.
    int64_t tok = tok0 + t * 32 + l32;
    tok = tok < p.M ? tok : p.M - 1;
    const bf16_t* row = p.x + tok * p.ldx + hh * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) xf[t][ks] = *reinterpret_cast<const bf16x8*>(row + ks * 16);
  }
  if (p.norm_w == nullptr) return;
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
    scale[t] = rsqrtf(ss * (1.0f / D) + p.eps);
  }
  // Make the packed rows opaque here: otherwise the compiler keeps all D fp32 copies from the first sweep alive for
  // the second one, which does not fit the register file next to the accumulators.
#pragma unroll
  for (int t = 0; t < TT; ++t)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" : "+v"(xf[t][ks]));
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const bf16x8 wv = *reinterpret_cast<const bf16x8*>(p.norm_w + ks * 16 + hh * 8);
#pragma unroll
    for (int t = 0; t < TT; ++t) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        xf[t][ks][e] = static_cast<bf16_t>(static_cast<float>(xf[t][ks][e]) * scale[t] * static_cast<float>(wv[e]));
      asm volatile("" : "+v"(xf[t][ks]));
    }
  }
}

// Copies n bf16 values (or zeros when src is null) into LDS with the whole workgroup; n is a multiple of 8.
__device__ __forceinline__ void stage_bias(const bf16_t* src, bf16_t* dst, int n, int tid, int nthreads) {
  for (int i = tid * 8; i < n; i += nthreads * 8) {
    bf16x8 v;
    if (src != nullptr) {
      v = *reinterpret_cast<const bf16x8*>(src + i);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = static_cast<bf16_t>(0.f);
    }
    *reinterpret_cast<bf16x8*>(dst + i) = v;
  }
}

// Writes two 32-feature accumulator blocks (64 features) of one 32-token tile into the wavefront's epilogue tile,
// adding the bias and rounding to bf16. Accumulator register jq*4 + e of lane (l32, hh) is feature jq*8 + hh*4 + e.
__device__ __forceinline__ void tile_to_lds(uint8_t* tile, const f32x16& a0, const f32x16& a1, const bf16_t* bias_lds,
                                            int l32, int hh) {
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) {
#pragma unroll
    for (int jq = 0; jq < 4; ++jq) {
      const int col = rb * 32 + jq * 8 + hh * 4;
      const bf16x4 bv = *reinterpret_cast<const bf16x4*>(bias_lds + col);
      bf16x4 ov;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        ov[e] = static_cast<bf16_t>((rb == 0 ? a0[jq * 4 + e] : a1[jq * 4 + e]) + static_cast<float>(bv[e]));
      *reinterpret_cast<bf16x4*>(tile + l32 * kStageRow + col * 2) = ov;
    }
  }
}

// Reads the epilogue tile back row-wise (lane -> token 8*i + lane/8, features 8*(lane%8) .. +7), adds the residual
// pieces loaded earlier and stores 16 bytes per lane: every 128-byte row segment is written by 8 consecutive lanes.
template <bool RES>
__device__ __forceinline__ void tile_to_global(const uint8_t* tile, bf16_t* out, int64_t ldo, int64_t tok_base,
                                               int64_t M, int col0, const bf16x8 (&res)[4], int lane) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = i * 8 + lane / 8;
    const int64_t tok = tok_base + row;
    bf16x8 v = *reinterpret_cast<const bf16x8*>(tile + row * kStageRow + (lane % 8) * 16);
    if (RES) {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        v[e] = static_cast<bf16_t>(static_cast<float>(v[e]) + static_cast<float>(res[i][e]));
    }
    if (tok < M) *reinterpret_cast<bf16x8*>(out + tok * ldo + col0 + (lane % 8) * 8) = v;
  }
}

__device__ __forceinline__ void load_residual(const bf16_t* residual, int64_t ldr, int64_t tok_base, int64_t M,
                                              int col0, bf16x8 (&res)[4], int lane) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    int64_t tok = tok_base + i * 8 + lane / 8;
    tok = tok < M ? tok : M - 1;
    res[i] = *reinterpret_cast<const bf16x8*>(residual + tok * ldr + col0 + (lane % 8) * 8);
  }
}

// ------------------------------------------------------------------------------------------------------------------
// Fused RMSNorm -> up -> SiLU-gate -> down -> + residual
//
// A chunk is 16 hidden units. Its up-projection fragment has 32 rows: 16 gate rows on top of the 16 matching value
// rows, so ONE accumulator (16 registers per lane) holds g in registers 0..7 and u in registers 8..15 for the same
// eight hidden units of the lane's token. silu(g) * u of those eight is exactly one B-operand fragment (k = 16) of
// the down projection. Two chunks are staged and consumed per barrier.
// LDS: [2 weight buffers][b_up (2F) | b_down (D)]; after the main loop the weight buffers hold the epilogue tiles.
// ------------------------------------------------------------------------------------------------------------------
template <int D, int TT, int NWAVES, int CPB>
__global__ __launch_bounds__(NWAVES * kWave, TT == 1 ? 2 : 1) void swiglu_ffn_kernel(const TsParams p) {
  constexpr int kTokPerWg = NWAVES * 32 * TT;  // TT token tiles of 32 per wavefront
  constexpr int KS = D / 16;             // k-steps of the up projection = up fragments per chunk
  constexpr int MB = D / 32;             // 32-feature row blocks of the down projection = down fragments per chunk
  constexpr int CFRAG = KS + MB;         // fragments per chunk
  constexpr int NFRAG = CPB * CFRAG;     // fragments per barrier step
  constexpr int FPW = NFRAG / NWAVES;    // fragments staged per wavefront
  static_assert(NFRAG % NWAVES == 0, "fragments must divide over the wavefronts");
  static_assert(2 * NFRAG * kFrag >= NWAVES * kStageWave, "epilogue tiles must fit in the weight buffers");
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  bf16_t* bias_lds = reinterpret_cast<bf16_t*>(smem + 2 * NFRAG * kFrag);

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);  // wavefront-uniform, kept in a scalar register
  const int lane = tid % kWave;
  const int l32 = lane % 32;
  const int hh = lane / 32;
  const int64_t tok0 = static_cast<int64_t>(blockIdx.x) * kTokPerWg + wave * (32 * TT);
  const int F = p.F;
  const int nsteps = F / (kHU * CPB);

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
      const char* src = w_up_bytes + (static_cast<int64_t>(step) * NFRAG + wave * FPW) * kFrag + ln * 16;
#pragma unroll
      for (int i = 0; i < FPW; ++i) lds_dma16(src + i * kFrag, base + i * kFrag);
      return;
    }
    const int s32 = ln & 31, shh = ln >> 5;
    const uint32_t up_lane_off =
        static_cast<uint32_t>((((s32 >= 16 ? F : 0) + up_unit_of_slot(s32 & 15)) * D + shh * 8) * 2);
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

  stage(0, 0);
  stage_bias(p.b1, bias_lds, 2 * F, tid, NWAVES * kWave);
  stage_bias(p.b2, bias_lds + 2 * F, D, tid, NWAVES * kWave);

  bf16x8 xf[TT][KS];
  load_tokens<D, TT>(p, tok0, l32, hh, xf);

  f32x16 oacc[TT][MB];
#pragma unroll
  for (int t = 0; t < TT; ++t)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int j = 0; j < 16; ++j) oacc[t][mb][j] = 0.f;

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  for (int step = 0; step < nsteps; ++step) {
    const int buf = step & 1;
    if (step + 1 < nsteps) stage(step + 1, buf ^ 1);
#pragma unroll
    for (int q = 0; q < CPB; ++q) {
      const uint8_t* wb = smem + buf * (NFRAG * kFrag) + q * (CFRAG * kFrag) + lane * 16;
      const int unit0 = (step * CPB + q) * kHU;
      // ---- up projection: rows 0..15 gate, rows 16..31 value, every token tile -------------------------------------
      f32x16 gu[TT];
#pragma unroll
      for (int t = 0; t < TT; ++t)
#pragma unroll
        for (int j = 0; j < 16; ++j) gu[t][j] = 0.f;
      // Fragment reads run kPre fragments ahead of their MFMAs; the scheduling fences keep the compiler from hoisting
      // every read of the chunk to the top (which would not fit the register file).
      constexpr int kPre = 3;
      bf16x8 apipe[kPre + 1];
#pragma unroll
      for (int i = 0; i < kPre; ++i) apipe[i] = *reinterpret_cast<const bf16x8*>(wb + i * kFrag);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (ks + kPre < KS + MB)
          apipe[(ks + kPre) % (kPre + 1)] = *reinterpret_cast<const bf16x8*>(wb + (ks + kPre) * kFrag);
        const bf16x8 a = apipe[ks % (kPre + 1)];
#pragma unroll
        for (int t = 0; t < TT; ++t) gu[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, xf[t][ks], gu[t], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      // ---- bias + SiLU gate: register j < 8 is g, register 8 + j is u of hidden unit unit0 + 8*hh + j --------------
      const bf16x8 vg = *reinterpret_cast<const bf16x8*>(bias_lds + unit0 + 8 * hh);
      const bf16x8 vu = *reinterpret_cast<const bf16x8*>(bias_lds + F + unit0 + 8 * hh);
      bf16x8 hb[TT];
#pragma unroll
      for (int t = 0; t < TT; ++t)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float g = gu[t][e] + static_cast<float>(vg[e]);
          const float u = gu[t][8 + e] + static_cast<float>(vu[e]);
          hb[t][e] = static_cast<bf16_t>(p.gate_first ? silu_f(g) * u : g * silu_f(u));
        }
      // ---- down projection: O^T[feature, token] += W_down[feature, chunk] H^T --------------------------------------
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int f = KS + mb;  // fragment index inside the chunk; the first kPre down fragments are already in flight
        if (f + kPre < KS + MB)
          apipe[(f + kPre) % (kPre + 1)] = *reinterpret_cast<const bf16x8*>(wb + (f + kPre) * kFrag);
        const bf16x8 ad = apipe[f % (kPre + 1)];
#pragma unroll
        for (int t = 0; t < TT; ++t)
          oacc[t][mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ad, hb[t], oacc[t][mb], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  }

  // ---- epilogue: + b_down, round, transpose through the wavefront's LDS tile, + residual, coalesced bf16 stores ----
  uint8_t* tile = smem + wave * kStageWave;  // the weight buffers are free after the last barrier
  const bf16_t* bdown_lds = bias_lds + 2 * F;
#pragma unroll
  for (int t = 0; t < TT; ++t) {
    const int64_t tok_base = tok0 + t * 32;
#pragma unroll
    for (int pr = 0; pr < MB / 2; ++pr) {  // 64 features at a time
      bf16x8 res[4];
      if (p.residual != nullptr) load_residual(p.residual, p.ldr, tok_base, p.M, pr * 64, res, lane);
      tile_to_lds(tile, oacc[t][2 * pr], oacc[t][2 * pr + 1], bdown_lds + pr * 64, l32, hh);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      if (p.residual != nullptr)
        tile_to_global<true>(tile, p.out, p.ldo, tok_base, p.M, pr * 64, res, lane);
      else
        tile_to_global<false>(tile, p.out, p.ldo, tok_base, p.M, pr * 64, res, lane);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
    }
  }
}

// ------------------------------------------------------------------------------------------------------------------
// [RMSNorm ->] linear [-> + residual], K = D, N a multiple of 64
// LDS: [2 weight buffers of 2*KS fragments][NWAVES epilogue tiles][bias (N)]
// ------------------------------------------------------------------------------------------------------------------
template <int D, int TT, int NWAVES>
__global__ __launch_bounds__(NWAVES * kWave, TT == 1 ? 2 : 1) void norm_linear_kernel(const TsParams p) {
  constexpr int kTokPerWg = NWAVES * 32 * TT;
  constexpr int KS = D / 16;
  constexpr int NFRAG = 2 * KS;    // two 32-feature row blocks per chunk
  constexpr int FPW = NFRAG / NWAVES;
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  uint8_t* tiles = smem + 2 * NFRAG * kFrag;
  bf16_t* bias_lds = reinterpret_cast<bf16_t*>(tiles + NWAVES * kStageWave);

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int lane = tid % kWave;
  const int l32 = lane % 32;
  const int hh = lane / 32;
  const int64_t tok0 = static_cast<int64_t>(blockIdx.x) * kTokPerWg + wave * (32 * TT);
  const int nchunks = p.N / kNC;

  // fragment f of a chunk = (row block f / KS, k-step f % KS); source = uniform base + 32-bit per-lane byte offset
  const char* w_bytes = reinterpret_cast<const char*>(p.w1);
  auto stage = [&](int chunk, int buf) {
    int ln = lane;
    asm volatile("" : "+v"(ln));
    uint8_t* base = smem + buf * (NFRAG * kFrag) + wave * (FPW * kFrag);
    if (p.packed) {
      const char* src = w_bytes + (static_cast<int64_t>(chunk) * NFRAG + wave * FPW) * kFrag + ln * 16;
#pragma unroll
      for (int i = 0; i < FPW; ++i) lds_dma16(src + i * kFrag, base + i * kFrag);
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

  stage(0, 0);
  stage_bias(p.b1, bias_lds, p.N, tid, NWAVES * kWave);
  bf16x8 xf[TT][KS];
  load_tokens<D, TT>(p, tok0, l32, hh, xf);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  uint8_t* tile = tiles + wave * kStageWave;
  for (int c = 0; c < nchunks; ++c) {
    const int buf = c & 1;
    // Residual pieces of this chunk are requested BEFORE the next chunk's weights, so that waiting for them does not
    // also wait for the weight transfer (memory operations complete in issue order).
    bf16x8 res[TT][4];
    if (p.residual != nullptr) {
#pragma unroll
      for (int t = 0; t < TT; ++t) load_residual(p.residual, p.ldr, tok0 + t * 32, p.M, c * kNC, res[t], lane);
    }
    if (c + 1 < nchunks) stage(c + 1, buf ^ 1);
    const uint8_t* wb = smem + buf * (NFRAG * kFrag) + lane * 16;
    f32x16 acc[2][TT];  // [row block][token tile]
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int t = 0; t < TT; ++t)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[rb][t][j] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const bf16x8 a0 = *reinterpret_cast<const bf16x8*>(wb + ks * kFrag);
      const bf16x8 a1 = *reinterpret_cast<const bf16x8*>(wb + (KS + ks) * kFrag);
#pragma unroll
      for (int t = 0; t < TT; ++t) {
        acc[0][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, xf[t][ks], acc[0][t], 0, 0, 0);
        acc[1][t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, xf[t][ks], acc[1][t], 0, 0, 0);
      }
    }
    // Wait for the next chunk's weights (and this chunk's residual pieces) BEFORE the output stores are issued: the
    // memory counter also counts stores, and waiting on it after them would expose the full write latency per chunk.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int t = 0; t < TT; ++t) {
      tile_to_lds(tile, acc[0][t], acc[1][t], bias_lds + c * kNC, l32, hh);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      if (p.residual != nullptr)
        tile_to_global<true>(tile, p.out, p.ldo, tok0 + t * 32, p.M, c * kNC, res[t], lane);
      else
        tile_to_global<false>(tile, p.out, p.ldo, tok0 + t * 32, p.M, c * kNC, res[t], lane);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    __syncthreads();
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
  const int64_t grid = (p.M + tokens_per_wg - 1) / tokens_per_wg;
  if (grid > 0x7fffffffLL) return set_error(TAAC_ERR_UNSUPPORTED, "%s: too many workgroups", name);
  hipLaunchKernelGGL(kernel, dim3(static_cast<uint32_t>(grid)), dim3(threads), lds_bytes, s, p);
  return check_launch(name);
}

// Workgroup shape of the token-stationary kernels (tuning knob, read once from TAAC_TS_CONFIG; default 1, the
// fastest of the three on MI355X at D = 256):
//   0 = 4 wavefronts x 32 tokens, one FFN chunk per barrier  -> two workgroups per CU run independently
//   1 = 8 wavefronts x 32 tokens, two FFN chunks per barrier -> one workgroup per CU, two wavefronts per SIMD
//   2 = 4 wavefronts x 64 tokens, two FFN chunks per barrier -> one workgroup per CU, one wavefront per SIMD
int ts_config() {
  static const int config = [] {
    const char* env = getenv("TAAC_TS_CONFIG");
    return (env != nullptr && env[0] >= '0' && env[0] <= '2') ? env[0] - '0' : 1;
  }();
  return config;
}

bool ptr_ok(const void* p, uintptr_t mask) { return (reinterpret_cast<uintptr_t>(p) & mask) == 0; }

constexpr int kMaxLdsBytes = 160 * 1024;

}  // namespace
}  // namespace taac

extern "C" int64_t taac_ffn_packed_bytes(int32_t D, int32_t F) {
  if ((D != 128 && D != 256) || F <= 0 || F % (taac::kHU * taac::kCPB) != 0) return -1;
  return static_cast<int64_t>(3) * D * F * 2;
}

extern "C" int taac_ffn_pack_weights(const void* w_up, const void* w_down, void* packed, int32_t D, int32_t F,
                                     void* stream) {
  using namespace taac;
  const char* name = "taac_ffn_pack_weights";
  if (taac_ffn_packed_bytes(D, F) < 0)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: D must be 128 or 256 and F a positive multiple of 32", name);
  if (!w_up || !w_down || !packed) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  if (!ptr_ok(w_up, 15) || !ptr_ok(w_down, 15) || !ptr_ok(packed, 15))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: pointers must be 16-byte aligned", name);
  const int64_t pieces = static_cast<int64_t>(3) * D * F / 8;
  hipLaunchKernelGGL(ffn_pack_kernel, dim3(static_cast<uint32_t>((pieces + 255) / 256)), dim3(256), 0,
                     as_stream(stream), static_cast<const bf16_t*>(w_up), static_cast<const bf16_t*>(w_down),
                     static_cast<bf16x8*>(packed), D, F);
  return check_launch(name);
}

extern "C" int64_t taac_linear_packed_bytes(int32_t N, int32_t K) {
  if ((K != 128 && K != 256) || N <= 0 || N % taac::kNC != 0) return -1;
  return static_cast<int64_t>(N) * K * 2;
}

extern "C" int taac_linear_pack_weights(const void* w, void* packed, int32_t N, int32_t K, void* stream) {
  using namespace taac;
  const char* name = "taac_linear_pack_weights";
  if (taac_linear_packed_bytes(N, K) < 0)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: K must be 128 or 256 and N a positive multiple of 64", name);
  if (!w || !packed) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null pointer", name);
  if (!ptr_ok(w, 15) || !ptr_ok(packed, 15))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: pointers must be 16-byte aligned", name);
  const int64_t pieces = static_cast<int64_t>(N) * K / 8;
  hipLaunchKernelGGL(linear_pack_kernel, dim3(static_cast<uint32_t>((pieces + 255) / 256)), dim3(256), 0,
                     as_stream(stream), static_cast<const bf16_t*>(w), static_cast<bf16x8*>(packed), N, K);
  return check_launch(name);
}

extern "C" int taac_swiglu_ffn_fwd(const void* x, int64_t ldx, const void* norm_weight, float eps, const void* w_up,
                                   const void* b_up, const void* w_down, const void* b_down, const void* packed_weights,
                                   const void* residual, int64_t ldr, void* out, int64_t ldo, int64_t M, int32_t D,
                                   int32_t F, int gate_first, void* stream) {
  using namespace taac;
  const char* name = "taac_swiglu_ffn_fwd";
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
  if (!ptr_ok(x, 15) || !ptr_ok(w_up, 15) || !ptr_ok(w_down, 15) || !ptr_ok(out, 15) || !ptr_ok(residual, 15) ||
      !ptr_ok(norm_weight, 15) || !ptr_ok(b_up, 15) || !ptr_ok(b_down, 15) || !ptr_ok(packed_weights, 15))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: tensor base pointers must be 16-byte aligned", name);
  if (static_cast<size_t>(2 * kCPB * (D / 16 + D / 32)) * kFrag + static_cast<size_t>(2 * F + D) * 2 > kMaxLdsBytes)
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
  hipStream_t s = as_stream(stream);
  const int KS = D / 16, MB = D / 32;
  const size_t bias_bytes = static_cast<size_t>(2 * F + D) * 2;
#define TAAC_FFN_LAUNCH(DD, TT, NW, CPB)                                                                      \
  return launch_ts(swiglu_ffn_kernel<DD, TT, NW, CPB>, p, NW * kWave, NW * 32 * TT,                          \
                   static_cast<size_t>(2 * CPB * (KS + MB)) * kFrag + bias_bytes, s, name)
  const int cfg = ts_config();
  if (D == 256) {
    if (cfg == 0) TAAC_FFN_LAUNCH(256, 1, 4, 1);
    if (cfg == 1) TAAC_FFN_LAUNCH(256, 1, 8, 2);
    TAAC_FFN_LAUNCH(256, 2, 4, 2);
  }
  if (cfg == 0) TAAC_FFN_LAUNCH(128, 1, 4, 1);
  if (cfg == 1) TAAC_FFN_LAUNCH(128, 1, 8, 2);
  TAAC_FFN_LAUNCH(128, 2, 4, 2);
#undef TAAC_FFN_LAUNCH
}

extern "C" int taac_norm_linear_fwd(const void* x, int64_t ldx, const void* norm_weight, float eps, const void* w,
                                    const void* bias, const void* packed_weights, const void* residual, int64_t ldr,
                                    void* out, int64_t ldo, int64_t M, int32_t N, int32_t K, void* stream) {
  using namespace taac;
  const char* name = "taac_norm_linear_fwd";
  if (M < 0 || N <= 0 || K <= 0) return set_error(TAAC_ERR_INVALID_VALUE, "%s: M must be >= 0, N and K > 0", name);
  if (K != 256 && K != 128)
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: token-stationary kernel is built for K = 128 or 256 (got %d)", name, K);
  if (N % kNC != 0) return set_error(TAAC_ERR_UNSUPPORTED, "%s: N=%d must be a multiple of %d", name, N, kNC);
  if (ldx < K || ldo < N || (residual && ldr < N) || ldx % 8 || ldo % 8 || (residual && ldr % 8))
    return set_error(TAAC_ERR_INVALID_VALUE, "%s: row strides must cover a row and be multiples of 8", name);
  if (M == 0) return TAAC_OK;
  if (!x || !out || (!packed_weights && !w)) return set_error(TAAC_ERR_INVALID_VALUE, "%s: null tensor pointer", name);
  if (!ptr_ok(x, 15) || !ptr_ok(w, 15) || !ptr_ok(out, 15) || !ptr_ok(residual, 15) || !ptr_ok(norm_weight, 15) ||
      !ptr_ok(bias, 15) || !ptr_ok(packed_weights, 15))
    return set_error(TAAC_ERR_UNSUPPORTED, "%s: tensor base pointers must be 16-byte aligned", name);
  if (static_cast<size_t>(2 * 2 * (K / 16)) * kFrag + 8 * static_cast<size_t>(kStageWave) + static_cast<size_t>(N) * 2 >
      kMaxLdsBytes)
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
  hipStream_t s = as_stream(stream);
#define TAAC_LIN_LAUNCH(KK, TT, NW)                                                                            \
  return launch_ts(norm_linear_kernel<KK, TT, NW>, p, NW * kWave, NW * 32 * TT,                               \
                   static_cast<size_t>(2 * 2 * (KK / 16)) * kFrag + static_cast<size_t>(NW) * kStageWave +    \
                       static_cast<size_t>(N) * 2,                                                             \
                   s, name)
  const int cfg = ts_config();
  if (K == 256) {
    if (cfg == 0) TAAC_LIN_LAUNCH(256, 1, 4);
    if (cfg == 1) TAAC_LIN_LAUNCH(256, 1, 8);
    TAAC_LIN_LAUNCH(256, 2, 4);
  }
  if (cfg == 0) TAAC_LIN_LAUNCH(128, 1, 4);
  if (cfg == 1) TAAC_LIN_LAUNCH(128, 1, 8);
  TAAC_LIN_LAUNCH(128, 2, 4);
#undef TAAC_LIN_LAUNCH
}
